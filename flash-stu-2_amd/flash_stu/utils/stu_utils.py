"""Spectral filters of the STU: top eigenvectors of a fixed Hankel matrix.

Host-side, float64, run once per model (reference:
flash_stu/utils/stu_utils.py:18-31,33-143,146-193).  Unlike the reference this
needs no GPU: the eigen-decomposition runs in numpy on the host either way.
"""
from __future__ import annotations

import os
from typing import Optional

import numpy as np
import torch


def get_hankel(seq_len: int, use_hankel_L: bool = False) -> np.ndarray:
    idx = np.arange(1, seq_len + 1, dtype=np.float64)
    s = idx[:, None] + idx[None, :]
    if use_hankel_L:
        return ((-1.0) ** (s - 2.0) + 1.0) * (8.0 / ((s + 3.0) * (s - 1.0) * (s + 1.0)))
    return 2.0 / (s ** 3 - s)


def save_spectral_filters(phi: torch.Tensor, path: str, seq_len: Optional[int] = None, K: Optional[int] = None,
                          use_hankel_L: bool = False, **metadata) -> None:
    """Stores filters with the metadata keys the reference writes
    (stu_utils.py:33-82) so files are interchangeable."""
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    L, k = phi.shape
    torch.save({"phi": phi.detach().cpu(), "seq_len": seq_len or L, "K": K or k, "use_hankel_L": use_hankel_L,
                "dtype": str(phi.dtype), **metadata}, path)


def load_spectral_filters(path: str, device=None, dtype: Optional[torch.dtype] = None,
                          verify_shape: Optional[tuple] = None) -> torch.Tensor:
    """Loads a filter file (tensor-only payload; nothing in it is executed)."""
    if not os.path.exists(path):
        raise FileNotFoundError(f"Filter file not found: {path}")
    blob = torch.load(path, map_location="cpu", weights_only=True)
    phi = blob["phi"] if isinstance(blob, dict) else blob
    if verify_shape is not None and tuple(phi.shape) != tuple(verify_shape):
        raise ValueError(f"Filter shape mismatch: expected {tuple(verify_shape)}, got {tuple(phi.shape)}")
    if dtype is not None:
        phi = phi.to(dtype)
    if device is None:
        device = torch.device("cuda" if torch.cuda.is_available() else "cpu")
    return phi.to(device)


def get_spectral_filters(seq_len: int, K: int, use_hankel_L: bool = False, device=None,
                         dtype: torch.dtype = torch.bfloat16, load_from: Optional[str] = None) -> torch.Tensor:
    """(seq_len, K) filters: eigenvectors of the K largest eigenvalues (ascending
    order) scaled by eigenvalue**0.25, cast to `dtype`."""
    if load_from is not None:
        return load_spectral_filters(load_from, device=device, dtype=dtype, verify_shape=(seq_len, K))
    if device is None:
        device = torch.device("cuda" if torch.cuda.is_available() else "cpu")
    sigma, vecs = np.linalg.eigh(get_hankel(seq_len, use_hankel_L))
    sigma, vecs = sigma[-K:], vecs[:, -K:]
    return torch.tensor(vecs * sigma ** 0.25, device=device, dtype=dtype)


# ---------------------------------------------------------------- the spectral convolution as an operator
def nearest_power_of_two(x: int, round_up: bool = False) -> int:
    """flash_stu/utils/numerics.py:3-6."""
    return 1 << (int(x) - 1).bit_length() if round_up else 1 << (int(x).bit_length() - 1)


def _alt_sign(L: int, like: torch.Tensor) -> torch.Tensor:
    s = torch.ones(L, 1, dtype=like.dtype, device=like.device)
    s[1::2] = -1
    return s


def _causal_conv(u: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """u (B,T,d) with the per-channel filter v (L,d): out[b,t,c] = T(sum_{s<=t} v[s,c] u[b,t-s,c]), one branch.
    FFT kernel from 32 positions on (as far as the in-LDS transform reaches), time-domain kernel otherwise."""
    from .. import _hip
    T = u.shape[1]
    n = _hip.fft_length(T) if T >= 32 else 0
    if n == 0:
        return _hip.stu_conv_direct(u.contiguous(), v.contiguous(), single_branch=True)
    return _hip.stu_conv_fft(u.contiguous(), _hip.stu_fft_filter(v.contiguous(), n, single_branch=True), single_branch=True)


class _ApproxConvolve(torch.autograd.Function):
    """Both sign branches of the approx-mode convolution with their gradients.  The minus branch
    sgn * conv(sgn * u, v) equals conv(u, v * (-1)^s), so every piece of forward and backward is the one causal
    convolution kernel:
      d/du: correlation with the filter     = time-reversed convolution of the time-reversed gradient
      d/dv: correlation of gradient and u   = per batch row, convolution of the time-reversed gradient with that
            row's input as the filter, read backwards; summed over the batch in fp32
    The backward runs in fp32 whatever the input dtype (the reference differentiates through an fp32 FFT,
    stu_utils.py:226-228) and rounds the two gradients once at the end."""

    @staticmethod
    def forward(ctx, u, v, both):
        ctx.save_for_backward(u, v)
        ctx.both = both
        up = _causal_conv(u, v)
        if not both:
            return up, torch.zeros(0, dtype=u.dtype, device=u.device)
        return up, _causal_conv(u, v * _alt_sign(v.shape[0], v))

    @staticmethod
    def backward(ctx, gp, gm):
        u, v = ctx.saved_tensors
        B, T, d = u.shape
        L = v.shape[0]
        uf, vf = u.float(), v.float()
        gpf = gp.float().flip(1).contiguous()
        gmf = gm.float().flip(1).contiguous() if ctx.both else None
        gu = gv = None
        if ctx.needs_input_grad[0]:
            gu = _causal_conv(gpf, vf)
            if ctx.both:
                gu = gu + _causal_conv(gmf, vf * _alt_sign(L, vf))
            gu = gu.flip(1).to(u.dtype)
        if ctx.needs_input_grad[1]:
            taps = min(L, T)
            acc_p = torch.zeros(T, d, dtype=torch.float32, device=u.device)
            acc_m = torch.zeros_like(acc_p) if ctx.both else None
            for b in range(B):
                ub = uf[b].contiguous()                              # (T,d): this row's input as the filter
                acc_p += _causal_conv(gpf[b:b + 1], ub)[0]
                if ctx.both:
                    acc_m += _causal_conv(gmf[b:b + 1], ub)[0]
            gv = torch.zeros(L, d, dtype=torch.float32, device=u.device)
            gv[:taps] = acc_p.flip(0)[:taps]                         # lag s sits at position T-1-s
            if ctx.both:
                gv[:taps] += acc_m.flip(0)[:taps] * _alt_sign(taps, acc_m)
            gv = gv.to(v.dtype)
        return gu, gv, None


def convolve(u: torch.Tensor, v: torch.Tensor, n: int, use_approx: bool = True, return_both: bool = True,
             sgn: Optional[torch.Tensor] = None, v_fft: Optional[torch.Tensor] = None):
    """The reference's causal convolution (flash_stu/utils/stu_utils.py:195-246), same arguments and results:
    u (B,T,d); approx mode v (L,d) per-channel filters -> (U_plus, U_minus) of shape (B,T,d); exact mode v (L,K) filter
    bank -> (B,T,K,d) each; U_minus is None with return_both=False.  Results are rounded to u's dtype.  `n` must cover
    the linear convolution (n >= 2T-1, as the reference chooses it); the kernels pick their own transform length, and
    `sgn` / `v_fft` (the reference's cached operands) are accepted and not needed.  Approx mode is differentiable in
    u and v (training-side use: flash_stu/modules/stu.py:89-98 under autograd); exact mode is forward only."""
    from .. import _hip
    if u.dim() != 3 or v.dim() != 2:
        raise ValueError("convolve: u must be (B,T,d) and v (L,d) or (L,K)")
    B, T, d = u.shape
    if n < 2 * T - 1:
        raise ValueError(f"convolve: n={n} is shorter than the linear convolution of {T} positions")
    if not u.is_cuda:
        raise _hip.FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    v = v.to(u.dtype)
    if use_approx:
        if v.shape[1] != d:
            raise ValueError(f"convolve: approx mode needs one filter per channel, got v {tuple(v.shape)} for d={d}")
        up, um = _ApproxConvolve.apply(u, v, bool(return_both))
        return up, (um if return_both else None)
    if u.requires_grad or v.requires_grad:
        raise NotImplementedError("convolve: exact mode (use_approx=False) is forward only")
    K = v.shape[1]
    up = torch.empty(B, T, K, d, dtype=u.dtype, device=u.device)
    um = torch.empty_like(up) if return_both else None
    nn_ = _hip.fft_length(T) if T >= 32 else 0
    if nn_ == 0:
        _hip.stu_conv_bank(u.contiguous(), v.contiguous(), up, um)
    else:
        spec = _hip.stu_fft_filter(v.contiguous(), nn_, single_branch=not return_both)
        ut = u.transpose(1, 2).contiguous().transpose(1, 2)        # time-major copy: coalesced column loads
        _hip.stu_conv_bank_fft(ut, spec, up, um)
    return up, um
