"""ctypes binding of libflashstu_hip.so (the C ABI declared in include/flashstu_hip.h).

Every wrapper takes torch tensors that already live on the GPU, checks what the
kernels assume (device, dtype, contiguity, shapes) and launches on torch's
current HIP stream.  There is no CPU or eager fallback: if the shared library
is missing or a tensor is not on the GPU the call raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "csrc", "libflashstu_hip.so")

FSTU_F32, FSTU_BF16 = 0, 1
MAX_DECODE_ROWS = 16

_lib = None

_vp, _i, _i64, _f, _u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_uint64

# name -> argtypes; the complete export list of the library
SIGNATURES = {
    "fstu_embed": [_vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "fstu_add_rmsnorm": [_vp, _vp, _i, _i, _i, _vp, _vp, _i, _i, _f, _i, _vp],
    "fstu_add_slices": [_vp, _vp, _i, _i, _i, _i, _vp],
    "fstu_linear_decode": [_vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "fstu_glu_decode": [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "fstu_linear_decode_splitk": [_vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "fstu_gelu_mul": [_vp, _vp, _vp, _i64, _i, _vp],
    "fstu_bias_act": [_vp, _vp, _i64, _i, _i, _i, _vp],
    "fstu_stu_step_hist": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_step_lds": [_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_step_lds_pair": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_step_lds_pair_add": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_step_lds_pair_cached": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_step_lds_prime": [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_step_lds_single": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_bank_step_lds": [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_inproj_step": [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_res_inproj_step": [_vp, _vp, _i, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_scan_lds": [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_lds_state_from_hist": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_lds_state_ring_from_hist": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_conv_direct": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_conv_bank": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_fft_length": [_i],
    "fstu_fft_twiddles": [_vp, _i, _vp],
    "fstu_stu_fft_filter": [_vp, _i64, _i64, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_conv_fft": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_stu_conv_fft_strided": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_transpose": [_vp, _vp, _i, _i, _i, _i, _vp],
    "fstu_stu_conv_bank_fft": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_kv_append": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_kv_fill": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "fstu_swa_decode": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _vp],
    "fstu_swa_append_decode": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _vp],
    "fstu_swa_prefill": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _vp],
    "fstu_swa_prefill_ws_elems": [_i, _i, _i, _i],
    "fstu_swa_prefill_mfma": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _vp],
    "fstu_sample": [_vp, _vp, _i64, _i, _i, _f, _i, _f, _i, _u64, _i, _i, _vp],
    "fstu_sample_ws_bytes": [],
    "fstu_head_maxima": [_vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _vp, _i, _vp],
    "fstu_head_maxima_packed": [_vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _vp, _vp],
    "fstu_sample_topk": [_vp, _i64, _vp, _vp, _vp, _i64, _i, _i, _f, _i, _f, _u64, _i, _vp],
    "fstu_head_argmax": [_vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _vp, _vp, _i64, _i, _vp],
    "fstu_head_argmax_static": [_vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _vp, _i64, _i, _vp],
    "fstu_pack_rows": [_vp, _vp, _i, _i, _vp],
    "fstu_packed_elems": [_i, _i],
    "fstu_glu_packed_supported": [_i, _i, _i],
    "fstu_mlp_packed_rows32_supported": [_i, _i, _i],
    "fstu_glu_packed": [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "fstu_glu_packed_norm": [_vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "fstu_linear_packed": [_vp, _i, _vp, _f, _vp, _vp, _i, _i, _i, _i, _vp],
    "fstu_linear_packed_add": [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _vp],
    "fstu_linear_packed_res": [_vp, _vp, _i, _vp, _vp, _f, _vp, _vp, _i, _i, _i, _i, _vp],
    "fstu_down_packed_splitk": [_vp, _i, _vp, _vp, _i, _i, _i, _vp, _vp],
    "fstu_decode_step": [_vp, _vp, _vp, _i64, _i, _f, _i, _f, _i, _u64, _i, _vp],
    "fstu_decode_graph_create": [_vp, _vp, _i64, _vp, _i, _i, _f, _i, _f, _i, _u64, _vp, _vp],
    "fstu_decode_graph_launch": [_vp, _vp],
    "fstu_decode_graph_seek": [_vp, ctypes.c_longlong],
    "fstu_decode_graph_destroy": [_vp],
    "fstu_prof_begin": [_i, _i],
    "fstu_prof_end": [_vp, _vp],
    "fstu_prof_copy": [_vp, _vp, ctypes.c_size_t, _vp],
    "fstu_prof_glu_loop": [_vp, _i, _vp, _vp, _vp],
    "fstu_gemm_bf16": [_vp, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _i, _i, _i, _i, _vp],
    "fstu_gemm_bf16_splitk": [_vp, _i64, _vp, _vp, _i, _i, _i, _i, _vp],
    "fstu_gemm_any": [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i, _i, _i, _i, _vp],
    "fstu_gemm_bf16_ta": [_vp, _i64, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _i, _i, _i, _i, _i, _vp],
    "fstu_lds_sequence_ws_floats": [_i, _i, _i],
    "fstu_lds_sequence_status": [_vp, _vp],
    "fstu_lds_sequence": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "fstu_lds_steps": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
}


class FlashSTUHipError(RuntimeError):
    pass


def load(path: Optional[str] = None):
    """Loads the shared library (once) and declares every entry point."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise FlashSTUHipError(
            f"{p} not found: build it with `python flash-stu-2_amd/csrc/build.py` "
            "(hipcc --offload-arch=gfx950). There is no fallback path.")
    lib = ctypes.CDLL(p)
    lib.fstu_version.restype = ctypes.c_int
    lib.fstu_last_error.restype = ctypes.c_char_p
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = ctypes.c_int
    lib.fstu_packed_elems.restype = ctypes.c_int64
    lib.fstu_sample_ws_bytes.restype = ctypes.c_int64
    lib.fstu_swa_prefill_ws_elems.restype = ctypes.c_int64
    lib.fstu_lds_sequence_ws_floats.restype = ctypes.c_size_t
    if path is None:
        _lib = lib
    return lib


def is_available() -> bool:
    return os.path.exists(LIB_PATH) and torch.cuda.is_available()


def _check(rc: int, name: str):
    if rc != 0:
        msg = load().fstu_last_error().decode("utf-8", "replace")
        raise FlashSTUHipError(f"{name} failed (code {rc}): {msg}")


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return FSTU_F32
    if t.dtype == torch.bfloat16:
        return FSTU_BF16
    raise FlashSTUHipError(f"unsupported dtype {t.dtype}: the HIP kernels take float32 or bfloat16")


def _dev(*ts: Optional[torch.Tensor]):
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
        if not t.is_contiguous():
            raise FlashSTUHipError(f"tensor of shape {tuple(t.shape)} must be contiguous")


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _rows_view(t: torch.Tensor):
    """(rows, row stride in elements) of a 2-D tensor whose rows are dense."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise FlashSTUHipError(f"expected a 2-D tensor with dense rows, got shape {tuple(t.shape)} stride {t.stride()}")
    if not t.is_cuda:
        raise FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    return t.shape[0], t.stride(0)


# ---------------------------------------------------------------- wrappers
def embed(ids: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    ids = ids.contiguous()
    _dev(ids, table, out)
    assert ids.dtype == torch.int64
    rows = ids.numel()
    V, d = table.shape
    if out is None:
        out = torch.empty(*ids.shape, d, dtype=table.dtype, device=table.device)
    _check(load().fstu_embed(_p(ids), _p(table), _p(out), rows, d, V, _dt(table), _stream()), "fstu_embed")
    return out


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], w: Optional[torch.Tensor], eps: float,
                y: Optional[torch.Tensor] = None, delta_mode: int = 0, nslices: int = 1,
                single_branch: bool = False, want_norm: bool = True) -> Optional[torch.Tensor]:
    """x (rows..., d) is updated in place by delta (if given); returns rmsnorm(x)*w if want_norm."""
    _dev(x, delta, w, y)
    d = x.shape[-1]
    rows = x.numel() // d
    if want_norm and y is None:
        y = torch.empty_like(x)
    if delta is not None:
        if delta_mode == 0:
            assert delta.dtype == x.dtype and delta.numel() == x.numel()
        else:
            assert delta.dtype == torch.float32
            assert delta.numel() == nslices * (2 if delta_mode == 2 else 1) * rows * d, "partial-sum buffer has the wrong size"
    _check(load().fstu_add_rmsnorm(_p(x), _p(delta), delta_mode, nslices, int(single_branch),
                                   _p(w) if want_norm else None, _p(y) if want_norm else None,
                                   rows, d, float(eps), _dt(x), _stream()), "fstu_add_rmsnorm")
    return y if want_norm else None


def add_slices(x: torch.Tensor, slices: torch.Tensor) -> torch.Tensor:
    """x (rows,d) bf16 += T(sum of the fp32 slices (n,rows,d)) in place, over the whole chip; returns x."""
    _dev(x, slices)
    rows, d = x.shape
    assert x.is_contiguous() and slices.dtype == torch.float32 and slices.is_contiguous() and slices.shape[1:] == (rows, d)
    _check(load().fstu_add_slices(_p(x), _p(slices), slices.shape[0], rows, d, _dt(x), _stream()), "fstu_add_slices")
    return x


def linear_decode(x: torch.Tensor, W: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x (rows<=16, K) @ W(N,K)^T -> (rows, N); x and out may be row-strided views."""
    rows, ldx = _rows_view(x)
    _dev(W)
    N, K = W.shape
    assert x.shape[1] == K and x.dtype == W.dtype
    if out is None:
        out = torch.empty(rows, N, dtype=x.dtype, device=x.device)
    orow, ldy = _rows_view(out)
    assert orow == rows and out.shape[1] == N
    _check(load().fstu_linear_decode(_p(x), ldx, _p(W), _p(out), ldy, rows, N, K, _dt(x), _stream()), "fstu_linear_decode")
    return out


def glu_decode(x: torch.Tensor, Wg: torch.Tensor, Wu: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    rows, ldx = _rows_view(x)
    _dev(Wg, Wu)
    I, K = Wg.shape
    assert Wu.shape == Wg.shape and x.shape[1] == K and x.dtype == Wg.dtype == Wu.dtype
    if out is None:
        out = torch.empty(rows, I, dtype=x.dtype, device=x.device)
    orow, ldo = _rows_view(out)
    assert orow == rows and out.shape[1] == I
    _check(load().fstu_glu_decode(_p(x), ldx, _p(Wg), _p(Wu), _p(out), ldo, rows, I, K, _dt(x), _stream()), "fstu_glu_decode")
    return out


def linear_decode_splitk(x: torch.Tensor, W: torch.Tensor, ksplit: int, partial: Optional[torch.Tensor] = None) -> torch.Tensor:
    rows, ldx = _rows_view(x)
    _dev(W, partial)
    N, K = W.shape
    assert x.shape[1] == K and x.dtype == W.dtype
    if partial is None:
        partial = torch.empty(ksplit, rows, N, dtype=torch.float32, device=x.device)
    assert partial.dtype == torch.float32 and partial.numel() >= ksplit * rows * N
    _check(load().fstu_linear_decode_splitk(_p(x), ldx, _p(W), _p(partial), rows, N, K, ksplit, _dt(x), _stream()),
           "fstu_linear_decode_splitk")
    return partial


def gelu_mul(g: torch.Tensor, u: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(g, u, out)
    assert g.shape == u.shape and g.dtype == u.dtype
    if out is None:
        out = torch.empty_like(g)
    _check(load().fstu_gelu_mul(_p(g), _p(u), _p(out), g.numel(), _dt(g), _stream()), "fstu_gelu_mul")
    return out


def bias_act(y: torch.Tensor, bias: Optional[torch.Tensor], silu: bool = False) -> torch.Tensor:
    """In place y = act(y + bias) over the last dimension; bias may be None."""
    _dev(y, bias)
    n = y.shape[-1]
    if bias is not None and (bias.shape != (n,) or bias.dtype != y.dtype):
        raise FlashSTUHipError(f"bias must be ({n},) {y.dtype}")
    _check(load().fstu_bias_act(_p(y), _p(bias), y.numel() // n, n, int(silu), _dt(y), _stream()), "fstu_bias_act")
    return y


def gemm_supported(x2: torch.Tensor, weight: torch.Tensor) -> bool:
    """Shapes the matrix-core prompt GEMM takes: bf16, K a multiple of 32, N a multiple of 4, rows 16-byte aligned."""
    K = x2.shape[-1]
    return (x2.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x2.dim() == 2 and K % 32 == 0 and
            weight.shape[0] % 4 == 0 and weight.is_contiguous() and x2.stride(1) == 1 and x2.stride(0) % 8 == 0 and
            x2.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def gemm(x2: torch.Tensor, weight: torch.Tensor, up_weight: Optional[torch.Tensor] = None,
         residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x2 (M,K) @ weight (N,K)^T on the matrix cores (bf16).  up_weight: the gated pair
    T(T(gelu_tanh(T(x2 @ weight^T))) * T(x2 @ up_weight^T)); residual (M,N): T(residual + T(x2 @ weight^T))."""
    _dev(weight, up_weight)
    for t in (x2, residual, out):          # rows may be strided
        if t is not None and not t.is_cuda:
            raise FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    if not gemm_supported(x2, weight):
        raise FlashSTUHipError(f"gemm: unsupported operands {tuple(x2.shape)} {x2.dtype} x {tuple(weight.shape)} {weight.dtype}")
    if up_weight is not None and residual is not None:
        raise FlashSTUHipError("gemm: the gated pair and the residual epilogue do not combine")
    M, K = x2.shape
    N = weight.shape[0]
    if weight.shape[1] != K or (up_weight is not None and (up_weight.shape != weight.shape or not up_weight.is_contiguous()
                                                            or up_weight.dtype != weight.dtype)):
        raise FlashSTUHipError("gemm: weight shapes")
    if out is None:
        out = torch.empty(M, N, dtype=x2.dtype, device=x2.device)
    if out.shape != (M, N) or out.stride(1) != 1 or out.dtype != x2.dtype:
        raise FlashSTUHipError("gemm: out must be (M,N) with contiguous rows")
    mode, ldr = 0, 0
    if up_weight is not None:
        mode = 1
    elif residual is not None:
        if residual.shape != (M, N) or residual.stride(1) != 1 or residual.dtype != x2.dtype:
            raise FlashSTUHipError("gemm: residual must be (M,N) with contiguous rows")
        mode, ldr = 2, residual.stride(0)
    _check(load().fstu_gemm_bf16(_p(x2), x2.stride(0), _p(weight), _p(up_weight), _p(residual), ldr, _p(out), out.stride(0),
                                 M, N, K, mode, _stream()), "fstu_gemm_bf16")
    return out


def gemm_any(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out (M,N) = T(a @ w^T) for ANY strided 2-D views a (M,K) and w (N,K) of one dtype (fp32 or bf16): the general
    kernel behind everything the bf16 matrix-core GEMM does not take.  fp32 accumulation, one rounding."""
    for t in (a, w, out):
        if t is not None and not t.is_cuda:
            raise FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    if a.dim() != 2 or w.dim() != 2 or a.shape[1] != w.shape[1] or a.dtype != w.dtype:
        raise FlashSTUHipError(f"gemm_any: operands {tuple(a.shape)} {a.dtype} x {tuple(w.shape)} {w.dtype}")
    M, K = a.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty(M, N, dtype=a.dtype, device=a.device)
    if out.shape != (M, N) or out.stride(1) != 1 or out.dtype != a.dtype:
        raise FlashSTUHipError("gemm_any: out must be (M,N) with contiguous rows")
    # a size-1 dimension may carry any stride: give it a positive one
    sam, sak = max(a.stride(0), 1), max(a.stride(1), 1)
    swn, swk = max(w.stride(0), 1), max(w.stride(1), 1)
    _check(load().fstu_gemm_any(_p(a), sam, sak, _p(w), swn, swk, _p(out), out.stride(0), M, N, K, _dt(a), _stream()),
           "fstu_gemm_any")
    return out


def gemm_ta(slabs: torch.Tensor, weight: torch.Tensor, residual: Optional[torch.Tensor] = None,
            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[b] = T(slabs[b]^T @ weight^T) (+ residual[b], rounded again) for slabs (nb, K, M) whose last index is
    contiguous (the reduction index is the slow one: the time-major U of the exact-mode STU operator), weight (N, K).
    M must be a multiple of 128; slab rows may be strided (a view of a wider buffer)."""
    _dev(weight)
    for t in (slabs, residual, out):
        if t is not None and not t.is_cuda:
            raise FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    if slabs.dim() != 3 or slabs.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or slabs.stride(2) != 1:
        raise FlashSTUHipError("gemm_ta: slabs must be (nb, K, M) bf16 with M contiguous")
    nb, K, M = slabs.shape
    N = weight.shape[0]
    if weight.shape != (N, K) or not weight.is_contiguous():
        raise FlashSTUHipError("gemm_ta: weight must be (N, K) contiguous")
    if out is None:
        out = torch.empty(nb, M, N, dtype=slabs.dtype, device=slabs.device)
    for t, name in ((out, "out"), (residual, "residual")):
        if t is not None and (t.shape != (nb, M, N) or t.stride(2) != 1 or t.dtype != slabs.dtype):
            raise FlashSTUHipError(f"gemm_ta: {name} must be (nb, M, N) with contiguous rows")
    mode = 2 if residual is not None else 0
    _check(load().fstu_gemm_bf16_ta(_p(slabs), slabs.stride(1), slabs.stride(0) if nb > 1 else 0, _p(weight), _p(residual),
                                    residual.stride(1) if residual is not None else 0,
                                    residual.stride(0) if residual is not None and nb > 1 else 0, _p(out), out.stride(1),
                                    out.stride(0) if nb > 1 else 0, M, N, K, nb, mode, _stream()), "fstu_gemm_bf16_ta")
    return out


def gemm_splitk(x2: torch.Tensor, weight: torch.Tensor, ksplit: int, partial: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 partial sums (ksplit, M, N) of x2 (M,K) @ weight (N,K)^T over ksplit slices of K; add_rmsnorm with
    delta_mode=1, nslices=ksplit folds them into the residual stream."""
    _dev(weight, partial)
    if not gemm_supported(x2, weight) or not x2.is_cuda or x2.shape[1] % (64 * ksplit) != 0:
        raise FlashSTUHipError(f"gemm_splitk: unsupported operands {tuple(x2.shape)} x {tuple(weight.shape)} / {ksplit}")
    M, K = x2.shape
    N = weight.shape[0]
    if partial is None:
        partial = torch.empty(ksplit, M, N, dtype=torch.float32, device=x2.device)
    if partial.shape != (ksplit, M, N) or partial.dtype != torch.float32:
        raise FlashSTUHipError("gemm_splitk: partial must be (ksplit, M, N) fp32")
    _check(load().fstu_gemm_bf16_splitk(_p(x2), x2.stride(0), _p(weight), _p(partial), M, N, K, ksplit, _stream()),
           "fstu_gemm_bf16_splitk")
    return partial


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x (..., K) @ weight (N,K)^T (+ bias): the skinny GEMV kernel for up to 16 rows, the bf16 matrix-core GEMM kernel
    for more rows, the general kernel (fstu_gemm_any: fp32, odd shapes, strided weights) for everything else.  No
    library GEMM."""
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    if x2.shape[0] <= MAX_DECODE_ROWS:
        y = linear_decode(x2.contiguous(), weight)
        if bias is not None:
            bias_act(y, bias)
    elif gemm_supported(x2, weight):
        y = gemm(x2, weight)
        if bias is not None:
            bias_act(y, bias)
    else:
        y = gemm_any(x2, weight)
        if bias is not None:
            bias_act(y, bias)
    return y.reshape(*shape[:-1], weight.shape[0])


def stu_step_hist(hist: torch.Tensor, filt: torch.Tensor, t: int, nsplit: int, eo: Optional[torch.Tensor] = None) -> torch.Tensor:
    """hist (B,cap,d), filt (L,d) -> fp32 partial sums (nsplit,2,B,d)."""
    _dev(hist, filt, eo)
    B, cap, d = hist.shape
    L = filt.shape[0]
    assert filt.shape[1] == d and filt.dtype == hist.dtype
    if eo is None:
        eo = torch.empty(nsplit, 2, B, d, dtype=torch.float32, device=hist.device)
    assert eo.dtype == torch.float32 and eo.numel() >= nsplit * 2 * B * d
    _check(load().fstu_stu_step_hist(_p(hist), _p(filt), _p(eo), B, d, t, cap, L, nsplit, _dt(hist), _stream()),
           "fstu_stu_step_hist")
    return eo


def _fir_args(ring, fir, B, d, dtype):
    """(ring pointer, fir pointer, taps) of the optional exact head of the filter."""
    if ring is None and fir is None:
        return None, None, 0
    if ring is None or fir is None:
        raise FlashSTUHipError("ring and fir go together")
    _dev(ring, fir)
    R = fir.shape[0]
    if ring.shape != (B, R, d) or fir.shape != (R, d) or fir.dtype != torch.float32 or ring.dtype != dtype:
        raise FlashSTUHipError(f"ring must be (B,{R},d) in the model dtype and fir ({R},d) fp32")
    return _p(ring), _p(fir), R


def stu_step_lds(state: torch.Tensor, xp: torch.Tensor, a: torch.Tensor, ce: torch.Tensor, t: int,
                 out: Optional[torch.Tensor] = None, co: Optional[torch.Tensor] = None, pair: bool = False,
                 ring: Optional[torch.Tensor] = None, fir: Optional[torch.Tensor] = None,
                 res: Optional[torch.Tensor] = None, ocache: Optional[torch.Tensor] = None) -> torch.Tensor:
    """state fp32 (B,2,S,d) advanced in place; xp (B,d) -> y (B,d) = T(2E), E = ce . bank(t).  With co (S,d) and
    O = co . other bank: the single-branch form y = T(E+O) (use_hankel_L), or with pair=True the two sign branches
    rounded separately, y = T(T(E+O) + T(E-O)).  pair=True with ring (B,R,d) and fir (R,d): the exact head of the
    filter on the first R lags (the ring is updated in place).  pair=True with res (B,d): the step joins the residual
    stream, y = T(res + T(output)); out may be res.  pair=True with ocache (B,d) fp32: O comes from ocache (left by the
    previous step or by stu_step_lds_prime) and the next step's O is left there; the other bank is not read."""
    _dev(state, a, ce, co)
    B, two, S, d = state.shape
    assert two == 2 and state.dtype == torch.float32 and a.dtype == torch.float32 and ce.dtype == torch.float32
    assert a.numel() == S and ce.shape == (S, d)
    rows, ldxp = _rows_view(xp)
    assert rows == B and xp.shape[1] == d
    if out is None:
        out = torch.empty(B, d, dtype=xp.dtype, device=xp.device)
    orow, ldy = _rows_view(out)
    assert orow == B and out.dtype == xp.dtype
    if co is not None:
        assert co.dtype == torch.float32 and co.shape == (S, d)
        if pair:
            rp, fp, R = _fir_args(ring, fir, B, d, xp.dtype)
            if ocache is not None:
                _dev(ocache, res)
                assert ocache.dtype == torch.float32 and ocache.shape == (B, d) and ocache.is_contiguous()
                assert res is None or (res.dtype == xp.dtype and res.shape == (B, d) and _rows_view(res)[1] == ldy)
                _check(load().fstu_stu_step_lds_pair_cached(_p(state), _p(xp), ldxp, _p(a), _p(ce), _p(co), rp, fp, R,
                                                            _p(ocache), _p(res), _p(out), ldy, B, S, d, t, _dt(xp), _stream()),
                       "fstu_stu_step_lds_pair_cached")
                return out
            if res is not None:
                _dev(res)
                assert res.dtype == xp.dtype and res.shape == (B, d) and _rows_view(res)[1] == ldy
                _check(load().fstu_stu_step_lds_pair_add(_p(state), _p(xp), ldxp, _p(a), _p(ce), _p(co), rp, fp, R, _p(res),
                                                         _p(out), ldy, B, S, d, t, _dt(xp), _stream()),
                       "fstu_stu_step_lds_pair_add")
                return out
            _check(load().fstu_stu_step_lds_pair(_p(state), _p(xp), ldxp, _p(a), _p(ce), _p(co), rp, fp, R, _p(out), ldy, B, S, d,
                                                 t, _dt(xp), _stream()), "fstu_stu_step_lds_pair")
            return out
        _check(load().fstu_stu_step_lds_single(_p(state), _p(xp), ldxp, _p(a), _p(ce), _p(co), _p(out), ldy, B, S, d, t,
                                               _dt(xp), _stream()), "fstu_stu_step_lds_single")
        return out
    _check(load().fstu_stu_step_lds(_p(state), _p(xp), ldxp, _p(a), _p(ce), _p(out), ldy, B, S, d, t, _dt(xp), _stream()),
           "fstu_stu_step_lds")
    return out


def stu_step_lds_prime(state: torch.Tensor, a: torch.Tensor, co: torch.Tensor, t: int, dtype: torch.dtype,
                       ring: Optional[torch.Tensor] = None, fir: Optional[torch.Tensor] = None,
                       out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ocache (B,d) fp32 for position t+1 from the state (B,2,S,d) and the ring as they stand after position t: what
    a pair step with ocache at position t would have left.  dtype: the model dtype (of the ring)."""
    _dev(state, a, co)
    B, two, S, d = state.shape
    assert two == 2 and state.dtype == torch.float32 and a.numel() == S and co.shape == (S, d) and co.dtype == torch.float32
    rp, fp, R = _fir_args(ring, fir, B, d, dtype)
    if out is None:
        out = torch.empty(B, d, dtype=torch.float32, device=state.device)
    assert out.shape == (B, d) and out.dtype == torch.float32 and out.is_contiguous() and out.is_cuda
    _check(load().fstu_stu_step_lds_prime(_p(state), _p(a), _p(co), rp, fp, R, _p(out), B, S, d, t,
                                          FSTU_BF16 if dtype == torch.bfloat16 else FSTU_F32, _stream()),
           "fstu_stu_step_lds_prime")
    return out


def stu_scan_lds(xp: torch.Tensor, a: torch.Tensor, ce: torch.Tensor, state: Optional[torch.Tensor] = None,
                 t_start: int = 0, out: Optional[torch.Tensor] = None):
    """xp (B,T,d) -> (y (B,T,d), state fp32 (B,2,S,d)): the recurrence step over a whole sequence in one launch.
    state=None starts from zero; a given state is continued in place (t_start = position of xp[:, 0])."""
    _dev(a, ce, state)
    if not xp.is_cuda or (out is not None and not out.is_cuda):
        raise FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    B, T, d = xp.shape          # batch and token strides are passed on: slices along time need no copy
    S = a.numel()
    assert a.dtype == torch.float32 and ce.dtype == torch.float32 and ce.shape == (S, d) and ce.is_contiguous()
    assert xp.stride(2) == 1
    carry = state is not None
    if state is None:
        state = torch.empty(B, 2, S, d, dtype=torch.float32, device=xp.device)
    assert state.shape == (B, 2, S, d) and state.dtype == torch.float32 and state.is_contiguous()
    if out is None:
        out = torch.empty(B, T, d, dtype=xp.dtype, device=xp.device)
    assert out.shape == xp.shape and out.dtype == xp.dtype and out.stride(2) == 1
    _check(load().fstu_stu_scan_lds(_p(xp), xp.stride(0), xp.stride(1), _p(a), _p(ce), _p(state), _p(out), out.stride(0),
                                    out.stride(1), B, T, S, d, t_start, int(carry), _dt(xp), _stream()), "fstu_stu_scan_lds")
    return out, state


def stu_inproj_step(h: torch.Tensor, Mt: torch.Tensor, state: torch.Tensor, a: torch.Tensor, ce: torch.Tensor, t: int,
                    out: Optional[torch.Tensor] = None, xp_out: Optional[torch.Tensor] = None,
                    co: Optional[torch.Tensor] = None, ring: Optional[torch.Tensor] = None,
                    fir: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h (B,K) bf16, Mt = M_inputs^T (d,K): projection + recurrence step in one launch -> y (B,d); with co the step
    of stu_step_lds(pair=True)."""
    _dev(h, Mt, state, a, ce, out, xp_out, co)
    B, K = h.shape
    d = Mt.shape[0]
    S = a.numel()
    assert h.dtype == Mt.dtype == torch.bfloat16 and Mt.shape[1] == K and state.shape == (B, 2, S, d)
    if out is None:
        out = torch.empty(B, d, dtype=h.dtype, device=h.device)
    rp, fp, R = _fir_args(ring, fir, B, d, h.dtype)
    _check(load().fstu_stu_inproj_step(_p(h), K, _p(Mt), _p(state), _p(a), _p(ce), _p(co), rp, fp, R, _p(out), d, _p(xp_out), B,
                                       S, d, K, t, _stream()), "fstu_stu_inproj_step")
    return out


def stu_res_inproj_step(x: torch.Tensor, partial: torch.Tensor, norm_w: torch.Tensor, eps: float, Mt: torch.Tensor,
                        state: torch.Tensor, a: torch.Tensor, ce: torch.Tensor, t: int, co: Optional[torch.Tensor] = None,
                        ring: Optional[torch.Tensor] = None, fir: Optional[torch.Tensor] = None):
    """(x', y): x' = x + bf16(sum of the fp32 slices); y = projection + recurrence step of rmsnorm(x') * norm_w."""
    _dev(x, partial, norm_w, Mt, state, a, ce, co)
    B, K = x.shape
    d = Mt.shape[0]
    S = a.numel()
    assert x.dtype == Mt.dtype == torch.bfloat16 and partial.dtype == torch.float32 and state.shape == (B, 2, S, d)
    x_out = torch.empty_like(x)
    y = torch.empty(B, d, dtype=x.dtype, device=x.device)
    rp, fp, R = _fir_args(ring, fir, B, d, x.dtype)
    _check(load().fstu_stu_res_inproj_step(_p(x), _p(partial), partial.shape[0], _p(x_out), _p(norm_w), float(eps), _p(Mt),
                                           _p(state), _p(a), _p(ce), _p(co), rp, fp, R, _p(y), d, B, S, d, K, t, _stream()),
           "fstu_stu_res_inproj_step")
    return x_out, y


def stu_lds_state_from_hist(hist: torch.Tensor, a: torch.Tensor, t_last: int, state: Optional[torch.Tensor] = None,
                            ring: Optional[torch.Tensor] = None) -> torch.Tensor:
    """state (B,2,S,d) fp32 of the recurrence after positions 0..t_last of hist (B,cap,d).  ring (B,R,d), optional:
    also receives hist[:, t] in slot t % R for the last R positions (slots a shorter sequence does not reach stay)."""
    _dev(hist, a, state, ring)
    B, cap, d = hist.shape
    S = a.numel()
    assert a.dtype == torch.float32
    if state is None:
        state = torch.empty(B, 2, S, d, dtype=torch.float32, device=hist.device)
    assert state.shape == (B, 2, S, d) and state.dtype == torch.float32
    R = 0
    if ring is not None:
        R = ring.shape[1]
        assert ring.shape == (B, R, d) and ring.dtype == hist.dtype and ring.is_contiguous()
    _check(load().fstu_stu_lds_state_ring_from_hist(_p(hist), _p(a), _p(state), _p(ring), R, B, S, d, t_last, cap, _dt(hist),
                                                    _stream()), "fstu_stu_lds_state_ring_from_hist")
    return state


def stu_bank_step_lds(state: torch.Tensor, x: torch.Tensor, a: torch.Tensor, ce: torch.Tensor,
                      co: Optional[torch.Tensor], t: int):
    """Exact-mode decode step on the recurrence state: returns (U+, U- or None), each (B,K,d) in x's dtype."""
    _dev(state, a, ce, co)
    B, ldx = _rows_view(x)
    d = x.shape[1]
    S, K = ce.shape
    assert state.shape == (B, 2, S, d) and state.dtype == torch.float32 and a.shape == (S,)
    up = torch.empty(B, K, d, dtype=x.dtype, device=x.device)
    um = torch.empty_like(up) if co is not None else None
    _check(load().fstu_stu_bank_step_lds(_p(state), _p(x), ldx, _p(a), _p(ce), _p(co), _p(up), _p(um), B, S, d, K, int(t),
                                         _dt(x), _stream()), "fstu_stu_bank_step_lds")
    return up, um


def stu_conv_direct(xp: torch.Tensor, filt: torch.Tensor, single_branch: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(xp, filt, out)
    B, T, d = xp.shape
    L = filt.shape[0]
    assert filt.shape[1] == d and filt.dtype == xp.dtype
    if out is None:
        out = torch.empty_like(xp)
    _check(load().fstu_stu_conv_direct(_p(xp), _p(filt), _p(out), B, T, d, L, int(single_branch), _dt(xp), _stream()),
           "fstu_stu_conv_direct")
    return out


def fft_length(T: int) -> int:
    """Smallest supported transform length (power of two, 64..16384) with n >= 2T; 0 if T is too long."""
    return int(load().fstu_fft_length(int(T)))


_twiddle_cache = {}


def fft_twiddles(n: int, device) -> torch.Tensor:
    """exp(-2 pi i j / n) as (n, 2) fp32 on `device`, built once per (n, device)."""
    key = (int(n), torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device())
    tw = _twiddle_cache.get(key)
    if tw is None:
        tw = torch.empty(n, 2, dtype=torch.float32, device=device)
        _check(load().fstu_fft_twiddles(_p(tw), n, _stream()), "fstu_fft_twiddles")
        _twiddle_cache[key] = tw
    return tw


def stu_fft_filter(filt: torch.Tensor, n: int, taps: Optional[int] = None, single_branch: bool = False) -> torch.Tensor:
    """Spectra (ncols, n, 2) fp32 of the columns of filt (L, ncols), cut to `taps` <= n/2 taps."""
    _dev(filt)
    L, ncols = filt.shape
    taps = min(L, n // 2) if taps is None else int(taps)
    if not 1 <= taps <= min(L, n // 2):
        raise FlashSTUHipError(f"taps={taps} outside 1..min(L={L}, n/2={n // 2})")
    spec = torch.empty(ncols, n, 2, dtype=torch.float32, device=filt.device)
    _check(load().fstu_stu_fft_filter(_p(filt), ncols, 1, _p(spec), _p(fft_twiddles(n, filt.device)), taps, ncols, n,
                                      int(single_branch), _dt(filt), _stream()), "fstu_stu_fft_filter")
    return spec


def stu_conv_fft(xp: torch.Tensor, spec: torch.Tensor, single_branch: bool = False,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """xp (B,T,d) convolved with the per-channel spectra spec (d,n,2) of stu_fft_filter (same single_branch)."""
    _dev(xp, spec, out)
    B, T, d = xp.shape
    n = spec.shape[1]
    if spec.shape != (d, n, 2) or spec.dtype != torch.float32:
        raise FlashSTUHipError(f"spec must be ({d}, n, 2) float32, got {tuple(spec.shape)} {spec.dtype}")
    if out is None:
        out = torch.empty_like(xp)
    _check(load().fstu_stu_conv_fft(_p(xp), _p(spec), _p(out), _p(fft_twiddles(n, xp.device)), B, T, d, n,
                                    int(single_branch), _dt(xp), _stream()), "fstu_stu_conv_fft")
    return out


def transpose(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """(B,R,C) -> (B,C,R), contiguous."""
    _dev(x, out)
    B, R, C = x.shape
    if out is None:
        out = torch.empty(B, C, R, dtype=x.dtype, device=x.device)
    assert out.shape == (B, C, R) and out.dtype == x.dtype and out.is_contiguous() and out.data_ptr() != x.data_ptr()
    _check(load().fstu_transpose(_p(x), _p(out), B, R, C, _dt(x), _stream()), "fstu_transpose")
    return out


def stu_conv_fft_strided(xp: torch.Tensor, spec: torch.Tensor, out: torch.Tensor, single_branch: bool = False) -> torch.Tensor:
    """xp, out: strided views of logical shape (B,T,d) (e.g. the transposed view of a time-major slab (B,d,T));
    spec (d,n,2) as for stu_conv_fft.  Written into out."""
    _dev(spec)
    if not xp.is_cuda or not out.is_cuda:
        raise FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    B, T, d = xp.shape
    n = spec.shape[1]
    if spec.shape != (d, n, 2) or spec.dtype != torch.float32 or not spec.is_contiguous():
        raise FlashSTUHipError(f"spec must be contiguous ({d}, n, 2) float32")
    if tuple(out.shape) != (B, T, d) or out.dtype != xp.dtype:
        raise FlashSTUHipError("out must have the logical shape and dtype of xp")
    xs = (ctypes.c_int64 * 3)(*xp.stride())
    ys = (ctypes.c_int64 * 3)(*out.stride())
    _check(load().fstu_stu_conv_fft_strided(_p(xp), xs, _p(spec), _p(out), ys, _p(fft_twiddles(n, xp.device)), B, T, d, n,
                                            int(single_branch), _dt(xp), _stream()), "fstu_stu_conv_fft_strided")
    return out


def stu_conv_bank_fft(x: torch.Tensor, spec: torch.Tensor, u_plus: torch.Tensor, u_minus: Optional[torch.Tensor]):
    """x: any strided view of logical shape (B,T,d); spec (K,n,2); u_plus/u_minus: strided views of logical shape
    (B,T,K,d), written in place.  A time stride of 1 makes the stores coalesce."""
    for t in (x, spec, u_plus, u_minus):
        if t is not None and not t.is_cuda:
            raise FlashSTUHipError("tensor is not on the GPU: the HIP path has no CPU fallback")
    B, T, d = x.shape
    K, n = spec.shape[0], spec.shape[1]
    if not spec.is_contiguous() or spec.dtype != torch.float32 or spec.shape[2] != 2:
        raise FlashSTUHipError("spec must be contiguous (K, n, 2) float32")
    if tuple(u_plus.shape) != (B, T, K, d) or u_plus.dtype != x.dtype:
        raise FlashSTUHipError(f"u_plus must have logical shape {(B, T, K, d)} and x's dtype")
    if u_minus is not None and (tuple(u_minus.shape) != (B, T, K, d) or u_minus.stride() != u_plus.stride()
                                or u_minus.dtype != x.dtype):
        raise FlashSTUHipError("u_minus must match u_plus in shape, strides and dtype")
    xs = (ctypes.c_int64 * 3)(*x.stride())
    us = (ctypes.c_int64 * 4)(*u_plus.stride())
    _check(load().fstu_stu_conv_bank_fft(_p(x), xs, _p(spec), _p(u_plus), _p(u_minus), us,
                                         _p(fft_twiddles(n, x.device)), B, T, d, K, n, _dt(x), _stream()),
           "fstu_stu_conv_bank_fft")


def stu_conv_bank(x: torch.Tensor, phi: torch.Tensor, u_plus: torch.Tensor, u_minus: Optional[torch.Tensor]):
    """x (B,T,d), phi (L,K) -> u_plus/u_minus (B,T,K,d) written in place."""
    _dev(x, phi, u_plus, u_minus)
    B, T, d = x.shape
    L, K = phi.shape
    assert u_plus.shape == (B, T, K, d) and phi.dtype == x.dtype == u_plus.dtype
    assert u_minus is None or (u_minus.shape == u_plus.shape and u_minus.dtype == x.dtype)
    _check(load().fstu_stu_conv_bank(_p(x), _p(phi), _p(u_plus), _p(u_minus), B, T, d, L, K, _dt(x), _stream()),
           "fstu_stu_conv_bank")


def kv_fill(qkv: torch.Tensor, kring: torch.Tensor, vring: torch.Tensor, pos0: int):
    """qkv (B,T,3d) -> ring (B,H,cap,hd) slots of positions pos0..pos0+T-1 (the last cap of them)."""
    _dev(qkv, kring, vring)
    B, T, d3 = qkv.shape
    Bk, H, cap, hd = kring.shape
    assert Bk == B and d3 == 3 * H * hd and vring.shape == kring.shape and qkv.dtype == kring.dtype == vring.dtype
    _check(load().fstu_kv_fill(_p(qkv), _p(kring), _p(vring), B, T, H, hd, cap, pos0, _dt(qkv), _stream()), "fstu_kv_fill")


def kv_append(qkv: torch.Tensor, kring: torch.Tensor, vring: torch.Tensor, pos: int):
    _dev(qkv, kring, vring)
    B, d3 = qkv.shape
    Bk, H, cap, hd = kring.shape
    assert Bk == B and d3 == 3 * H * hd and vring.shape == kring.shape and qkv.dtype == kring.dtype == vring.dtype
    _check(load().fstu_kv_append(_p(qkv), _p(kring), _p(vring), B, H, hd, cap, pos, _dt(qkv), _stream()), "fstu_kv_append")


def swa_decode(qkv: torch.Tensor, kring: torch.Tensor, vring: torch.Tensor, slopes: torch.Tensor, pos: int,
               window: int, softcap: float, out: Optional[torch.Tensor] = None, append: bool = False) -> torch.Tensor:
    """One query per (batch, head) at position pos; with append the new k,v are written to the ring first."""
    _dev(qkv, kring, vring, slopes, out)
    B, d3 = qkv.shape
    Bk, H, cap, hd = kring.shape
    assert Bk == B and d3 == 3 * H * hd and slopes.dtype == torch.float32 and slopes.numel() == H
    assert qkv.dtype == kring.dtype == vring.dtype
    if out is None:
        out = torch.empty(B, H * hd, dtype=qkv.dtype, device=qkv.device)
    fn = load().fstu_swa_append_decode if append else load().fstu_swa_decode
    _check(fn(_p(qkv), _p(kring), _p(vring), _p(out), _p(slopes), B, H, hd, cap, pos, window,
              float(softcap or 0.0), _dt(qkv), _stream()), "fstu_swa_decode")
    return out


def swa_prefill(qkv: torch.Tensor, slopes: torch.Tensor, n_heads: int, window: int, softcap: float,
                out: Optional[torch.Tensor] = None, force_valu: bool = False) -> torch.Tensor:
    """Prefill attention: the MFMA kernel for bf16 with head dim 64/128, the wave-per-query kernel otherwise."""
    _dev(qkv, slopes, out)
    B, T, d3 = qkv.shape
    d = d3 // 3
    hd = d // n_heads
    assert slopes.dtype == torch.float32 and slopes.numel() == n_heads
    if out is None:
        out = torch.empty(B, T, d, dtype=qkv.dtype, device=qkv.device)
    if qkv.dtype == torch.bfloat16 and hd in (64, 128) and T >= 16 and not force_valu:
        lib = load()
        ws = torch.empty(lib.fstu_swa_prefill_ws_elems(B, T, n_heads, hd), dtype=qkv.dtype, device=qkv.device)
        _check(lib.fstu_swa_prefill_mfma(_p(qkv), _p(ws), _p(out), _p(slopes), B, T, n_heads, hd, window,
                                         float(softcap or 0.0), _stream()), "fstu_swa_prefill_mfma")
        return out
    _check(load().fstu_swa_prefill(_p(qkv), _p(out), _p(slopes), B, T, n_heads, hd, window, float(softcap or 0.0),
                                   _dt(qkv), _stream()), "fstu_swa_prefill")
    return out


def sample(logits: torch.Tensor, out: torch.Tensor, temperature: float = 1.0, top_k: Optional[int] = None,
           top_p: Optional[float] = None, do_sample: bool = True, seed: int = 0, step: int = 0):
    """logits (B,V); writes one int64 per row into `out`, a (B,) view that may be strided."""
    _dev(logits)
    B, V = logits.shape
    assert out.dtype == torch.int64 and out.is_cuda and out.dim() == 1 and out.shape[0] == B
    _check(load().fstu_sample(_p(logits), out.data_ptr(), out.stride(0), B, V, float(temperature),
                              int(top_k) if top_k else 0, float(top_p) if top_p else 0.0, int(bool(do_sample)),
                              int(seed) & ((1 << 64) - 1), int(step), _dt(logits), _stream()), "fstu_sample")
    return out


def head_argmax(x: torch.Tensor, W: torch.Tensor, out_tokens: torch.Tensor, best_ws: torch.Tensor,
                temperature: float = 1.0, logits: Optional[torch.Tensor] = None) -> torch.Tensor:
    """logits = x @ W^T (rows<=16) and the greedy pick per row written to out_tokens (a strided (rows,) int64 view).
    best_ws: int64 zeros of at least rows*64 elements; it is zero again when the call completes."""
    rows, ldx = _rows_view(x)
    _dev(W, best_ws)
    N, K = W.shape
    assert x.shape[1] == K and x.dtype == W.dtype
    if logits is None:
        logits = torch.empty(rows, N, dtype=x.dtype, device=x.device)
    assert out_tokens.dtype == torch.int64 and out_tokens.dim() == 1 and out_tokens.shape[0] == rows
    assert best_ws.dtype == torch.int64 and best_ws.numel() >= rows * 64
    _check(load().fstu_head_argmax(_p(x), ldx, _p(W), _p(logits), logits.stride(0), rows, N, K, float(temperature),
                                   _p(best_ws), out_tokens.data_ptr(), out_tokens.stride(0), _dt(x), _stream()),
           "fstu_head_argmax")
    return logits


def head_maxima(x: torch.Tensor, W: torch.Tensor, best_ws: torch.Tensor, temperature: float = 1.0,
                logits: Optional[torch.Tensor] = None) -> torch.Tensor:
    """logits = x @ W^T (rows<=16, bf16) and, in best_ws (int64 zeros, rows*64 elements), the packed maxima of 64
    subsets of every row at this temperature: what sample_topk starts from."""
    rows, ldx = _rows_view(x)
    _dev(W, best_ws)
    N, K = W.shape
    assert x.shape[1] == K and x.dtype == W.dtype
    if logits is None:
        logits = torch.empty(rows, N, dtype=x.dtype, device=x.device)
    assert best_ws.dtype == torch.int64 and best_ws.numel() >= rows * 64
    _check(load().fstu_head_maxima(_p(x), ldx, _p(W), _p(logits), logits.stride(0), rows, N, K, float(temperature),
                                   _p(best_ws), _dt(x), _stream()), "fstu_head_maxima")
    return logits


def head_maxima_packed(x: torch.Tensor, wp: torch.Tensor, N: int, best_ws: torch.Tensor, temperature: float = 1.0,
                       logits: Optional[torch.Tensor] = None) -> torch.Tensor:
    """head_maxima over a packed copy of the (N,K) head weight (pack_rows), rows <= 32."""
    rows, ldx = _rows_view(x)
    _dev(wp, best_ws)
    K = x.shape[1]
    if logits is None:
        logits = torch.empty(rows, N, dtype=x.dtype, device=x.device)
    assert x.dtype == torch.bfloat16 and best_ws.dtype == torch.int64 and best_ws.numel() >= rows * 64
    _check(load().fstu_head_maxima_packed(_p(x), ldx, _p(wp), _p(logits), logits.stride(0), rows, N, K, float(temperature),
                                          _p(best_ws), _stream()), "fstu_head_maxima_packed")
    return logits


def sample_ws(device) -> torch.Tensor:
    """Zeroed workspace of sample_topk (allocate once; every call leaves its counters zero again)."""
    return torch.zeros((int(load().fstu_sample_ws_bytes()) + 7) // 8, dtype=torch.int64, device=device)


def sample_topk(logits: torch.Tensor, best_ws: torch.Tensor, samp_ws: torch.Tensor, out: torch.Tensor, top_k: int,
                temperature: float = 1.0, top_p: Optional[float] = None, seed: int = 0, step: int = 0):
    """sample() with do_sample=True for bf16 logits and 1 <= top_k <= 64, every row spread over the chip.  best_ws: the
    maxima head_maxima left for these logits at this temperature; it and samp_ws's counters are zero again afterwards."""
    _dev(best_ws, samp_ws)
    if not logits.is_cuda or logits.dim() != 2 or logits.stride(1) != 1 or logits.dtype != torch.bfloat16:
        raise FlashSTUHipError("sample_topk takes (B,V) bf16 logits with contiguous rows on the GPU")
    B, V = logits.shape
    assert out.dtype == torch.int64 and out.is_cuda and out.dim() == 1 and out.shape[0] == B
    assert best_ws.dtype == torch.int64 and best_ws.numel() >= B * 64
    _check(load().fstu_sample_topk(_p(logits), logits.stride(0), _p(best_ws), _p(samp_ws), out.data_ptr(), out.stride(0),
                                   B, V, float(temperature), int(top_k), float(top_p) if top_p else 0.0,
                                   int(seed) & ((1 << 64) - 1), int(step), _stream()), "fstu_sample_topk")
    return out


def pack_rows(W: torch.Tensor) -> torch.Tensor:
    """(N,K) bf16 row-major -> packed MFMA-fragment order (ceil(N/16)*16*K elements); K % 32 == 0."""
    _dev(W)
    if W.dtype != torch.bfloat16:
        raise FlashSTUHipError("packed weights are bf16 only")
    N, K = W.shape
    lib = load()
    out = torch.empty(lib.fstu_packed_elems(N, K), dtype=W.dtype, device=W.device)
    _check(lib.fstu_pack_rows(_p(W), _p(out), N, K, _stream()), "fstu_pack_rows")
    return out


def glu_packed(x: torch.Tensor, wp_gate: torch.Tensor, wp_up: torch.Tensor, I: int,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Gate/up projection + GLU over packed weights (rows <= 32, bf16): x (rows,d) -> act (rows,I)."""
    _dev(wp_gate, wp_up, out)
    rows, ldx = _rows_view(x)
    d = x.shape[1]
    if x.dtype != torch.bfloat16 or not (load().fstu_glu_packed_supported(rows, d, I) or
                                         load().fstu_mlp_packed_rows32_supported(rows, d, I)):
        raise FlashSTUHipError(f"fstu_glu_packed does not support rows={rows} d={d} I={I} dtype={x.dtype}")
    if out is None:
        out = torch.empty(rows, I, dtype=x.dtype, device=x.device)
    _check(load().fstu_glu_packed(_p(x), ldx, _p(wp_gate), _p(wp_up), _p(out), out.stride(0), rows, I, d, _stream()),
           "fstu_glu_packed")
    return out


def glu_packed_norm(x: torch.Tensor, delta: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                    wp_gate: torch.Tensor, wp_up: torch.Tensor, I: int, out: Optional[torch.Tensor] = None):
    """(x + delta, act) with act = GLU(rmsnorm(x + delta) * norm_w): residual add, norm and gate/up in one launch."""
    _dev(x, delta, norm_w, wp_gate, wp_up)
    rows, d = x.shape
    wide = rows > 16 and delta is None and bool(load().fstu_mlp_packed_rows32_supported(rows, d, I))
    if x.dtype != torch.bfloat16 or not (wide or load().fstu_glu_packed_supported(rows, d, I)):
        raise FlashSTUHipError(f"fstu_glu_packed_norm does not support rows={rows} d={d} I={I} dtype={x.dtype}")
    act = out if out is not None else torch.empty(rows, I, dtype=x.dtype, device=x.device)
    assert act.shape == (rows, I) and act.dtype == x.dtype and act.is_contiguous() and act.is_cuda
    if wide:      # 17..32 rows: x is the summed stream, nothing is stored
        _check(load().fstu_glu_packed_norm(_p(x), None, None, _p(norm_w), float(eps), _p(wp_gate), _p(wp_up),
                                           _p(act), I, rows, I, d, _stream()), "fstu_glu_packed_norm")
        return x, act
    x_out = torch.empty_like(x)
    _check(load().fstu_glu_packed_norm(_p(x), _p(delta), _p(x_out), _p(norm_w), float(eps), _p(wp_gate), _p(wp_up),
                                       _p(act), I, rows, I, d, _stream()), "fstu_glu_packed_norm")
    return x_out, act


def linear_packed(x: torch.Tensor, wp: torch.Tensor, N: int, norm_w: Optional[torch.Tensor] = None, eps: float = 0.0):
    """x (rows,K) @ W^T over packed W (N,K); with norm_w, x is normalised first (rmsnorm * norm_w) in the same launch."""
    _dev(wp, norm_w)
    rows, ldx = _rows_view(x)
    K = x.shape[1]
    out = torch.empty(rows, N, dtype=x.dtype, device=x.device)
    _check(load().fstu_linear_packed(_p(x), ldx, _p(norm_w), float(eps), _p(wp), _p(out), N, rows, N, K, _stream()),
           "fstu_linear_packed")
    return out


def linear_packed_add(x: torch.Tensor, wp: torch.Tensor, res: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """T(res + T(x (rows,K) @ W^T)) over packed W (N,K): the projection joins the residual stream res (rows,N), dense
    rows; out may be res."""
    _dev(wp, res, out)
    rows, ldx = _rows_view(x)
    K = x.shape[1]
    N = res.shape[1]
    assert res.shape == (rows, N) and res.is_contiguous() and res.dtype == x.dtype
    if out is None:
        out = torch.empty_like(res)
    assert out.shape == res.shape and out.is_contiguous() and out.dtype == res.dtype
    _check(load().fstu_linear_packed_add(_p(x), ldx, _p(wp), _p(res), _p(out), rows, N, K, _stream()), "fstu_linear_packed_add")
    return out


def down_packed_splitk(act: torch.Tensor, wp_down: torch.Tensor, d: int, ksplit: int = 16) -> torch.Tensor:
    """Balanced split-K down projection: returns the fp32 slices (ksplit, rows, d); their sum in slice order is the
    result.  ksplit: 4, 8 or 16."""
    _dev(act, wp_down)
    rows, I = act.shape
    partial = torch.empty(ksplit, rows, d, dtype=torch.float32, device=act.device)
    ks = ctypes.c_int(ksplit)
    _check(load().fstu_down_packed_splitk(_p(act), I, _p(wp_down), _p(partial), rows, d, I, ctypes.byref(ks), _stream()),
           "fstu_down_packed_splitk")
    assert ks.value == ksplit
    return partial


def linear_packed_res(x: torch.Tensor, partial: torch.Tensor, norm_w: torch.Tensor, eps: float, wp: torch.Tensor, N: int):
    """(x', y): x' = x + bf16(sum of the fp32 slices), y = (rmsnorm(x') * norm_w) @ W^T over packed W, one launch."""
    _dev(x, partial, norm_w, wp)
    rows, K = x.shape
    ns = partial.shape[0]
    x_out = torch.empty_like(x)
    y = torch.empty(rows, N, dtype=x.dtype, device=x.device)
    _check(load().fstu_linear_packed_res(_p(x), _p(partial), ns, _p(x_out), _p(norm_w), float(eps), _p(wp), _p(y), N, rows,
                                         N, K, _stream()), "fstu_linear_packed_res")
    return x_out, y


def lds_steps(h: torch.Tensor, x: torch.Tensor, A: torch.Tensor, Bm: torch.Tensor, Cm: torch.Tensor,
              out: Optional[torch.Tensor] = None, transposed=None, ws: Optional[torch.Tensor] = None,
              check_status: bool = False) -> torch.Tensor:
    """Dense LDS: h fp32 (Bt,S) carried in place over x (T,Bt,d_in) -> y (T,Bt,d_out).  bf16 with MFMA-friendly shapes
    runs on the matrix cores (fstu_lds_sequence); `transposed` = (Bm^T, Cm^T) contiguous copies and `ws` (fp32,
    lds_sequence_ws_floats elements) may be passed by callers that step position by position, to keep the two
    transposes and the allocation out of every call.  check_status: synchronise and raise if a wait inside the
    sequence kernel ran out."""
    _dev(h, x, A, Bm, Cm, out, ws)
    T, Bt, d_in = x.shape
    S = A.numel()
    d_out = Cm.shape[1]
    assert h.shape == (Bt, S) and h.dtype == torch.float32 and A.dtype == torch.float32
    assert Bm.shape == (d_in, S) and Cm.shape == (S, d_out) and Bm.dtype == Cm.dtype == x.dtype
    if out is None:
        out = torch.empty(T, Bt, d_out, dtype=x.dtype, device=x.device)
    if (x.dtype == torch.bfloat16 and T >= 1 and d_in % 32 == 0 and S % 32 == 0 and S <= 256 and d_out % 16 == 0
            and x.is_contiguous() and out.is_contiguous()):
        # blocks of 128 positions in parallel on the matrix cores (weights passed transposed)
        lib = load()
        need = int(lib.fstu_lds_sequence_ws_floats(T, Bt, S))
        if ws is None:
            ws = torch.empty(need, dtype=torch.float32, device=x.device)
        assert ws.dtype == torch.float32 and ws.numel() >= need and ws.is_contiguous()
        bmt, cmt = transposed if transposed is not None else (Bm.t().contiguous(), Cm.t().contiguous())
        assert bmt.shape == (S, d_in) and cmt.shape == (d_out, S) and bmt.is_contiguous() and cmt.is_contiguous()
        _check(lib.fstu_lds_sequence(_p(h), _p(x), _p(A), _p(bmt), _p(cmt), _p(out), _p(ws), T, Bt, d_in, S, d_out, _stream()),
               "fstu_lds_sequence")
        if check_status:
            err = ctypes.c_int(0)
            _check(lib.fstu_lds_sequence_status(_p(ws), ctypes.byref(err)), "fstu_lds_sequence_status")
            if err.value:
                raise FlashSTUHipError("fstu_lds_sequence: a block waited in vain for the state of the blocks in front of it")
        return out
    _check(load().fstu_lds_steps(_p(h), _p(x), _p(A), _p(Bm), _p(Cm), _p(out), T, Bt, d_in, S, d_out, _dt(x), _stream()),
           "fstu_lds_steps")
    return out
