from .attention import Attention
from .norm import RMSNorm
from .stu import STU
from .swiglu import MLP

__all__ = ["STU", "Attention", "MLP", "RMSNorm"]
