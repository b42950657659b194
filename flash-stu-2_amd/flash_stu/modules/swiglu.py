"""Gated MLP of Flash STU: down(gelu_tanh(gate(x)) * up(x))
(reference: flash_stu/modules/swiglu.py:4-29; the gate is tanh-GELU despite the
file name)."""
import torch
import torch.nn as nn

from .. import _hip


class MLP(nn.Module):
    def __init__(self, config, dtype=None):
        super().__init__()
        dtype = dtype if dtype is not None else config.torch_dtype
        self.hidden_size = config.n_embd
        self.intermediate_size = config.n_embd * config.mlp_scale
        self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=config.bias, dtype=dtype)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=config.bias, dtype=dtype)
        self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=config.bias, dtype=dtype)

    @torch.no_grad()
    def forward(self, x: torch.Tensor, residual: torch.Tensor = None):
        """x (..., d).  Up to 16 rows take the skinny MFMA kernels with the gate fused; more rows in bf16 take the
        matrix-core GEMM kernel with the gate as the epilogue of the gate/up pair.  With `residual` (same shape as x,
        contiguous rows) the sum residual + mlp(x) is written into `residual` where the down projection can carry the add
        as its epilogue, and None is returned; otherwise the MLP output is returned and the caller adds it."""
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        rows = x2.shape[0]
        if self.gate_proj.bias is not None:
            g = _hip.linear(x2, self.gate_proj.weight, self.gate_proj.bias)
            u = _hip.linear(x2, self.up_proj.weight, self.up_proj.bias)
            act = _hip.gelu_mul(g.contiguous(), u.contiguous(), out=g)
            out = _hip.linear(act, self.down_proj.weight, self.down_proj.bias)
        elif rows <= _hip.MAX_DECODE_ROWS:
            act = _hip.glu_decode(x2, self.gate_proj.weight, self.up_proj.weight)
            out = _hip.linear_decode(act, self.down_proj.weight)
        elif (_hip.gemm_supported(x2, self.gate_proj.weight) and self.up_proj.weight.is_contiguous()
              and self.intermediate_size % 32 == 0 and self.down_proj.weight.is_contiguous()
              and self.down_proj.weight.data_ptr() % 16 == 0):
            act = _hip.gemm(x2, self.gate_proj.weight, up_weight=self.up_proj.weight)
            if residual is not None and residual.is_contiguous():
                r2 = residual.view(-1, shape[-1])
                _hip.gemm(act, self.down_proj.weight, residual=r2, out=r2)
                return None
            out = _hip.gemm(act, self.down_proj.weight)
        else:
            # fp32 (the parity configuration) and shapes the bf16 matrix-core kernel does not take: the general kernel
            g = _hip.gemm_any(x2, self.gate_proj.weight)
            u = _hip.gemm_any(x2, self.up_proj.weight)
            act = _hip.gelu_mul(g, u, out=g)
            out = _hip.gemm_any(act, self.down_proj.weight)
        return out.reshape(shape)
