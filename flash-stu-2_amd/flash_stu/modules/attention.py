"""Sliding-window attention with ALiBi and tanh soft-capping
(reference: flash_stu/modules/attention.py:16-105, whose only backend is the
flash-attn CUDA wheel).  K/V are cached in a ring of window+1 positions laid
out (B,H,cap,hd); a reference-style growing cache (k,v) of shape (B,t,H,hd) is
accepted and converted."""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import _hip
from ..utils.numerics import nearest_power_of_two


def alibi_slopes(n_heads: int, interpolation_factor: float = 0.25) -> torch.Tensor:
    """fp32 slopes (attention.py:38-57)."""
    def gen(n):
        start = 2 ** (-(2 ** -(math.log2(n) - 3)))
        return [start * (start ** i) for i in range(n)]
    if math.log2(n_heads).is_integer():
        s = gen(n_heads)
    else:
        n = nearest_power_of_two(n_heads, round_up=False)
        s = gen(n) + gen(2 * n)[0::2][: n_heads - n]
    return torch.tensor(s, dtype=torch.float32) * interpolation_factor


class Attention(nn.Module):
    def __init__(self, config):
        super().__init__()
        assert config.n_embd % config.n_heads == 0
        self.n_heads = config.n_heads
        self.head_dim = config.n_embd // config.n_heads
        self.c_attn = nn.Linear(config.n_embd, 3 * config.n_embd, bias=config.bias, dtype=config.torch_dtype)
        self.c_proj = nn.Linear(config.n_embd, config.n_embd, bias=config.bias, dtype=config.torch_dtype)
        self.c_proj.SCALE_INIT = 1
        self.register_buffer("alibi_slopes", alibi_slopes(self.n_heads), persistent=False)
        w = config.window_size
        if isinstance(w, (tuple, list)):
            if len(w) != 2 or int(w[1]) != 0:
                raise NotImplementedError("only causal windows (left, 0) are supported")
            w = w[0]
        self.window_size = int(w)
        self.softcap = float(config.softcap or 0.0)

    def _ring_from_reference_cache(self, k: torch.Tensor, v: torch.Tensor):
        B, t, H, hd = k.shape
        cap = self.window_size + 1
        kr = k.new_zeros(B, H, cap, hd)
        vr = v.new_zeros(B, H, cap, hd)
        keep = min(t, cap)
        pos = torch.arange(t - keep, t, device=k.device)
        kr[:, :, pos % cap] = k[:, t - keep:].transpose(1, 2)
        vr[:, :, pos % cap] = v[:, t - keep:].transpose(1, 2)
        return kr, vr, torch.full((B,), t, dtype=torch.int64)

    @torch.no_grad()
    def forward(self, x: torch.Tensor, past_key_value=None, use_cache: bool = True):
        x = x.contiguous()
        B, T, d = x.shape
        H, hd, W = self.n_heads, self.head_dim, self.window_size
        slopes = self.alibi_slopes
        if past_key_value is None:
            qkv = _hip.linear(x, self.c_attn.weight, self.c_attn.bias).contiguous()
            o = _hip.swa_prefill(qkv, slopes, H, W, self.softcap)
            y = _hip.linear(o, self.c_proj.weight, self.c_proj.bias)
            if not use_cache:
                return y
            cap = W + 1
            # slots the prompt does not fill are written by the decode step that reaches their position before any
            # step reads them (a step reads positions below its own only): no zero fill
            kr = x.new_empty(B, H, cap, hd)
            vr = x.new_empty(B, H, cap, hd)
            _hip.kv_fill(qkv, kr, vr, 0)
            return y, (kr, vr, torch.full((B,), T, dtype=torch.int64))
        if T != 1:
            raise ValueError("a decode call with past_key_value takes exactly one new position")
        if len(past_key_value) == 2:
            past_key_value = self._ring_from_reference_cache(*past_key_value)
        kr, vr, pos_t = past_key_value
        pos = int(pos_t[0])
        qkv = _hip.linear(x.reshape(B, d), self.c_attn.weight, self.c_attn.bias)
        o = _hip.swa_decode(qkv, kr, vr, slopes, pos, W, self.softcap, append=True)
        y = _hip.linear(o, self.c_proj.weight, self.c_proj.bias).reshape(B, 1, d)
        return (y, (kr, vr, pos_t + 1)) if use_cache else y
