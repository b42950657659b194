"""Distillation of the STU's effective convolution filter into a diagonal
linear recurrence, done on the host in float64 when a model is prepared for
decoding.

In approx mode the two sign branches of the spectral convolution add up to a
causal filter that is 2*f[s] on even lags and zero on odd lags, f = phi @
M_filters (flash_stu/modules/stu.py:87-98,120 of the reference).  The even-lag
samples f[2m] are fitted by S real exponentials a_j^m on a fixed log-spaced
pole grid, so that one token step is  h_j <- a_j*h_j + x ; y = 2*sum_j ce_j*h_j
on the bank of the token's parity (cf. the shipped distillation used by
mini_stu/stu_lds.py:213-338, which is tied to one sequence length).
"""
from __future__ import annotations

import numpy as np
import torch

DEFAULT_STATE_DIM = 64


def pole_grid(n_lags: int, S: int) -> np.ndarray:
    """S poles in [0,1): 1-a log-spaced from 1/(8*n_lags) to 1, rounded to fp32
    so the kernel steps with exactly the fitted values."""
    om = np.exp(np.linspace(np.log(1.0 / (8.0 * max(n_lags, 2))), 0.0, S))
    return (1.0 - om).astype(np.float32)


def fit_even_lag_lds(filt_even, S: int = DEFAULT_STATE_DIM, ridge: float = 1e-14, per_channel: bool = False):
    """filt_even: (M,d) even-lag samples f[2m,c] (tensor or array, any float).
    Returns (a (S,) fp32 tensor, ce (S,d) fp32 tensor, max abs fit error); with per_channel the error is the
    (d,) array of per-channel maxima."""
    f = filt_even.detach().cpu().double().numpy() if isinstance(filt_even, torch.Tensor) else np.asarray(filt_even, np.float64)
    M = f.shape[0]
    a = pole_grid(M, S)
    V = a.astype(np.float64)[None, :] ** np.arange(M, dtype=np.float64)[:, None]     # (M,S)
    sc = np.sqrt((V * V).sum(0))
    Vs = V / sc
    G = Vs.T @ Vs + ridge * np.eye(S)
    C = np.linalg.solve(G, Vs.T @ f) / sc[:, None]
    C32 = C.astype(np.float32)
    err_c = np.abs(V @ C32.astype(np.float64) - f).max(0)
    return torch.from_numpy(a.copy()), torch.from_numpy(C32), (err_c if per_channel else float(err_c.max()))


def check_lds_fit(err_c, filt) -> None:
    """Raises when the distilled recurrence does not reproduce the filter it was fitted to.  err_c: per-channel
    largest fit error (d,) or one number, filt: the fitted taps (M,d).  The STU output of every channel is added to one
    residual stream, so the errors count against a common scale: every channel must be reproduced to one bf16 step
    (2^-8) of the root-mean-square over the channels of their largest taps, twice the rounding the reference itself
    applies to phi_proj.  Mixtures of Hankel filters (random-init and trained M_filters, 128...8192 taps) fit 2-50
    times better; a filter that is no sum of decaying exponentials does not, and such a model has to decode in
    history mode."""
    f = filt.detach().cpu().double().numpy() if isinstance(filt, torch.Tensor) else np.asarray(filt, np.float64)
    peak = np.abs(f).max(0)
    tol = 2.0 ** -8 * max(float(np.sqrt((peak * peak).mean())), 1e-30)
    err_c = np.atleast_1d(np.asarray(err_c, np.float64))
    bad = np.nonzero(~(err_c <= tol))[0]
    if bad.size:
        c = int(bad[np.argmax(err_c[bad])])
        raise ValueError(f"the recurrence fits {bad.size} of {err_c.size} STU filter channels worse than one bf16 step of the "
                         f"filters' largest taps (channel {c}: error {err_c[c]:.3e}, limit {tol:.3e}): decode with "
                         "stu_decode_mode='history'")
