"""RMSNorm -> STU -> (+) -> RMSNorm -> MLP -> (+)
(reference: flash_stu/layers/stu_layer.py:28-120).  The residual stream is
updated in place, as the reference's x.add_() does; each add is fused with the
following RMSNorm in one kernel."""
import torch
import torch.nn as nn

from .. import _hip
from ..modules.norm import RMSNorm
from ..modules.stu import STU
from ..modules.swiglu import MLP


class STULayer(nn.Module):
    def __init__(self, config, phi, n):
        super().__init__()
        self.config = config
        self.stu_norm = RMSNorm(config.n_embd, config.rms_norm_eps, dtype=config.torch_dtype)
        # optional sandwich (stu_layer.py:38-63): up-project -> SiLU -> STU on the hidden width -> down-project
        self.stu_mlp_enabled = bool(config.stu_enable_mlp_sandwich)
        if self.stu_mlp_enabled:
            self.stu_mlp_hidden_size = (config.stu_mlp_hidden_size if config.stu_mlp_hidden_size is not None
                                        else config.intermediate_size)
            self.stu_mlp_in_proj = nn.Linear(config.n_embd, self.stu_mlp_hidden_size, bias=config.bias,
                                             dtype=config.torch_dtype)
            self.stu = STU(config, phi, n, feature_dim=self.stu_mlp_hidden_size)
            self.stu_mlp_out_proj = nn.Linear(self.stu_mlp_hidden_size, config.n_embd, bias=config.bias,
                                              dtype=config.torch_dtype)
        else:
            self.stu = STU(config, phi, n)
        self.mlp_norm = RMSNorm(config.n_embd, config.rms_norm_eps, dtype=config.torch_dtype)
        self.mlp = MLP(config, dtype=config.torch_dtype)

    @torch.no_grad()
    def forward(self, x: torch.Tensor, past_key_value=None, use_cache: bool = False):
        """Returns x, or (x, state) when use_cache.  Unlike the reference, whose
        STU layers return None as their cache entry (stu_layer.py:118-119), the
        entry returned here is the decode state of the STU."""
        h = self.stu_norm(x)
        if self.stu_mlp_enabled:
            h = _hip.linear(h, self.stu_mlp_in_proj.weight, None).contiguous()
            _hip.bias_act(h, self.stu_mlp_in_proj.bias, silu=True)
        if use_cache or past_key_value is not None:
            y, state = self.stu(h, past_state=past_key_value, use_cache=True)
        else:
            y, state = self.stu(h), None
        if self.stu_mlp_enabled:
            y = _hip.linear(y.contiguous(), self.stu_mlp_out_proj.weight, self.stu_mlp_out_proj.bias).contiguous()
        h2 = self.mlp_norm.add_then_norm(x, y)
        m = self.mlp(h2, residual=x)
        if m is not None:
            _hip.add_rmsnorm(x, m.contiguous(), None, 0.0, want_norm=False)
        return (x, state) if use_cache else x
