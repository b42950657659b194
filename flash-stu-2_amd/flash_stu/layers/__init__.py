from .attention_layer import AttentionLayer
from .stu_layer import STULayer

__all__ = ["STULayer", "AttentionLayer"]
