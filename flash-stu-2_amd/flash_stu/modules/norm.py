"""RMSNorm with the reference's parameter name (`weight`) evaluated by the
fused HIP kernel (reference: torch.nn.RMSNorm fallback at
flash_stu/layers/stu_layer.py:32-36)."""
import torch
import torch.nn as nn

from .. import _hip


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim, dtype=dtype))

    @torch.no_grad()
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return _hip.add_rmsnorm(x.contiguous(), None, self.weight, self.eps)

    @torch.no_grad()
    def add_then_norm(self, x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        """x += delta in place, returns norm(x)."""
        return _hip.add_rmsnorm(x, delta.contiguous(), self.weight, self.eps)
