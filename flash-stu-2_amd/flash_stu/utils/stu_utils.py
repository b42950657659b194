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
