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
        if config.stu_enable_mlp_sandwich:
            raise NotImplementedError("stu_enable_mlp_sandwich is not implemented on the HIP path")
        self.stu_norm = RMSNorm(config.n_embd, config.rms_norm_eps, dtype=config.torch_dtype)
        self.stu = STU(config, phi, n)
        self.mlp_norm = RMSNorm(config.n_embd, config.rms_norm_eps, dtype=config.torch_dtype)
        self.mlp = MLP(config, dtype=config.torch_dtype)

    @torch.no_grad()
    def forward(self, x: torch.Tensor, past_key_value=None, use_cache: bool = False):
        """Returns x, or (x, state) when use_cache.  Unlike the reference, whose
        STU layers return None as their cache entry (stu_layer.py:118-119), the
        entry returned here is the decode state of the STU."""
        h = self.stu_norm(x)
        if use_cache or past_key_value is not None:
            y, state = self.stu(h, past_state=past_key_value, use_cache=True)
        else:
            y, state = self.stu(h), None
        h2 = self.mlp_norm.add_then_norm(x, y)
        m = self.mlp(h2)
        _hip.add_rmsnorm(x, m.contiguous(), None, 0.0, want_norm=False)
        return (x, state) if use_cache else x
