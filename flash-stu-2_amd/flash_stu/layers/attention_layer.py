"""RMSNorm -> Attention -> (+) -> RMSNorm -> MLP -> (+)
(reference: flash_stu/layers/attention_layer.py:29-87)."""
import torch
import torch.nn as nn

from .. import _hip
from ..modules.attention import Attention
from ..modules.norm import RMSNorm
from ..modules.swiglu import MLP


class AttentionLayer(nn.Module):
    def __init__(self, config) -> None:
        super().__init__()
        self.config = config
        self.attn_norm = RMSNorm(config.n_embd, config.rms_norm_eps, dtype=config.torch_dtype)
        self.attn = Attention(config)
        self.mlp_norm = RMSNorm(config.n_embd, config.rms_norm_eps, dtype=config.torch_dtype)
        self.mlp = MLP(config, dtype=config.torch_dtype)

    @torch.no_grad()
    def forward(self, x: torch.Tensor, past_key_value=None, use_cache: bool = True):
        a = self.attn_norm(x)
        if use_cache or past_key_value is not None:
            y, present = self.attn(a, past_key_value=past_key_value, use_cache=True)
        else:
            y, present = self.attn(a, past_key_value=None, use_cache=False), None
        h2 = self.mlp_norm.add_then_norm(x, y)
        m = self.mlp(h2, residual=x)
        if m is not None:
            _hip.add_rmsnorm(x, m.contiguous(), None, 0.0, want_norm=False)
        return (x, present) if use_cache else x
