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


def fit_even_lag_lds(filt_even, S: int = DEFAULT_STATE_DIM, ridge: float = 1e-14):
    """filt_even: (M,d) even-lag samples f[2m,c] (tensor or array, any float).
    Returns (a (S,) fp32 tensor, ce (S,d) fp32 tensor, max abs fit error)."""
    f = filt_even.detach().cpu().double().numpy() if isinstance(filt_even, torch.Tensor) else np.asarray(filt_even, np.float64)
    M = f.shape[0]
    a = pole_grid(M, S)
    V = a.astype(np.float64)[None, :] ** np.arange(M, dtype=np.float64)[:, None]     # (M,S)
    sc = np.sqrt((V * V).sum(0))
    Vs = V / sc
    G = Vs.T @ Vs + ridge * np.eye(S)
    C = np.linalg.solve(G, Vs.T @ f) / sc[:, None]
    C32 = C.astype(np.float32)
    err = float(np.abs(V @ C32.astype(np.float64) - f).max())
    return torch.from_numpy(a.copy()), torch.from_numpy(C32), err
