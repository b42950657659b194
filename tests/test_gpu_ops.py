"""GPU parity of every C-ABI entry point against the CPU oracle on the same
seeded inputs.  All calls go through libflashstu_hip.so (ctypes).

Tolerances: fp32 results differ from the oracle only by summation order
(1e-5 relative to the result scale); bf16 results must equal the oracle's
rounded values except where a different fp32 summation order flips a rounding:
at most one bf16 ulp (2^-7 relative) on a small fraction of elements."""
import math

import numpy as np

import pytest
import torch
import torch.nn.functional as F

from oracle import flashstu_oracle as O

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def hip():
    from flash_stu import _hip
    _hip.load()
    return _hip


def dev(t):
    return t.cuda()


def check(got, ref, dtype, frac=0.02, scale=None, atol=0.0):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    s = float(ref.abs().max()) if scale is None else scale
    diff = (got - ref).abs()
    if dtype == torch.float32:
        assert float(diff.max()) <= 2e-5 * max(s, 1e-30), f"fp32 max diff {float(diff.max())} scale {s}"
    else:
        tol = ref.abs() * 2.0 ** -7 + 1e-3 * 2.0 ** -7 * max(s, 1e-30) + atol
        assert bool((diff <= tol).all()), f"bf16 diff beyond one ulp: {float((diff - tol).max())}"
        assert float((diff > 0).float().mean()) <= frac, f"too many rounding flips: {float((diff > 0).float().mean())}"


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(hip, dtype):
    g = gen(0)
    table = torch.randn(101, 48, generator=g).to(dtype)
    ids = torch.randint(0, 101, (3, 7), generator=g)
    out = hip.embed(dev(ids), dev(table))
    assert torch.equal(out.cpu(), table[ids])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,d", [(8, 768), (3, 100), (64, 2048), (1, 256), (4096, 768), (67, 200), (130, 1000)])
def test_rmsnorm_plain_and_residual(hip, dtype, rows, d):
    g = gen(1)
    x = torch.randn(rows, d, generator=g).to(dtype)
    delta = torch.randn(rows, d, generator=g).to(dtype)
    w = (1 + 0.2 * torch.randn(d, generator=g)).to(dtype)
    y = hip.add_rmsnorm(dev(x), None, dev(w), O.RMS_EPS_DEFAULT)
    check(y, O.rms_norm(x, w), dtype)
    xd = dev(x.clone())
    y2 = hip.add_rmsnorm(xd, dev(delta), dev(w), O.RMS_EPS_DEFAULT)
    xr = x + delta
    assert torch.equal(xd.cpu(), xr)
    check(y2, O.rms_norm(xr, w), dtype)
    xd = dev(x.clone())
    assert hip.add_rmsnorm(xd, dev(delta), None, O.RMS_EPS_DEFAULT, want_norm=False) is None
    assert torch.equal(xd.cpu(), xr)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,N,K", [(8, 768, 768), (8, 2304, 768), (1, 50257, 256), (16, 1000, 320),
                                       (5, 37, 100), (8, 50257, 768)])
def test_linear_decode(hip, dtype, rows, N, K):
    g = gen(2)
    x = torch.randn(rows, K, generator=g).to(dtype)
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    y = hip.linear_decode(dev(x), dev(W))
    check(y, F.linear(x.float(), W.float()).to(dtype), dtype)


def test_linear_decode_strided_rows(hip):
    g = gen(3)
    big = torch.randn(4, 5, 256, generator=g).bfloat16()
    W = (torch.randn(128, 256, generator=g) / 16).bfloat16()
    bd = dev(big)
    out = torch.zeros(4, 3, 128, dtype=torch.bfloat16, device="cuda")
    hip.linear_decode(bd[:, 2, :], dev(W), out[:, 1, :])
    check(out[:, 1].cpu(), F.linear(big[:, 2].float(), W.float()).bfloat16(), torch.bfloat16)
    assert float(out[:, 0].abs().max()) == 0 and float(out[:, 2].abs().max()) == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,d,I", [(8, 768, 3072), (2, 256, 1024), (3, 96, 200)])
def test_mlp_decode_chain(hip, dtype, rows, d, I):
    """glu -> split-K down projection -> residual add equals x + MLP(x)."""
    g = gen(4)
    x = torch.randn(rows, d, generator=g).to(dtype)
    res = torch.randn(rows, d, generator=g).to(dtype)
    p = {"gate_proj.weight": (torch.randn(I, d, generator=g) / math.sqrt(d)).to(dtype),
         "up_proj.weight": (torch.randn(I, d, generator=g) / math.sqrt(d)).to(dtype),
         "down_proj.weight": (torch.randn(d, I, generator=g) / math.sqrt(I)).to(dtype)}
    act = hip.glu_decode(dev(x), dev(p["gate_proj.weight"]), dev(p["up_proj.weight"]))
    ref_act = F.gelu(F.linear(x, p["gate_proj.weight"]), approximate="tanh") * F.linear(x, p["up_proj.weight"])
    check(act, ref_act, dtype)
    for ks in ([1, 4] if I % 256 == 0 else [1, 2]):
        part = hip.linear_decode_splitk(act, dev(p["down_proj.weight"]), ks)
        rd = dev(res.clone())
        hip.add_rmsnorm(rd, part, None, O.RMS_EPS_DEFAULT, delta_mode=1, nslices=ks, want_norm=False)
        down = F.linear(act.cpu(), p["down_proj.weight"])
        ref = res + down
        # a one-ulp flip of the projection survives the residual add at the projection's scale
        check(rd, ref, dtype, frac=0.05, atol=(2.0 ** -7 * float(down.float().abs().max())) if dtype == torch.bfloat16 else 0.0)


# Prompt-pass GEMM kernel: the three tile shapes (128 x 128; 256 x 256 for K >= 1024 on grids that cover the chip
# twice; k tiles of 32 for K % 64 != 0), ragged M and N, one- and many-tile grids.
GEMM_SHAPES = [(4096, 2304, 768), (512, 768, 768), (1000, 772, 96), (17, 4, 32), (300, 200, 1056), (2048, 16384, 1024),
               (257, 132, 64), (32, 2048, 512), (20, 260, 128), (4096, 768, 3072), (1000, 288, 256)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_bf16_plain_and_residual(hip, M, N, K):
    """fstu_gemm_bf16 modes 0 and 2 against F.linear in fp32 rounded once (c_attn / c_proj / down_proj / M_inputs of
    the prompt pass): bf16 results within one ulp, few rounding flips."""
    g = gen(61)
    x = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    res = torch.randn(M, N, generator=g).bfloat16()
    ref = F.linear(x.float(), W.float()).bfloat16()
    xd, Wd = dev(x), dev(W)
    check(hip.gemm(xd, Wd), ref, torch.bfloat16)
    rd = dev(res.clone())
    out = hip.gemm(xd, Wd, residual=rd, out=rd)          # in place, as the MLP's down projection uses it
    assert out.data_ptr() == rd.data_ptr()
    check(rd, (res.float() + ref.float()).bfloat16(), torch.bfloat16, frac=0.05, atol=2.0 ** -7 * float(ref.float().abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(64, 256, 256), (1000, 772, 100), (17, 3, 5), (300, 200, 1056), (1, 1, 1), (129, 65, 33),
                                   (4096, 768, 256)])
def test_gemm_any_against_float64(hip, dtype, M, N, K):
    """fstu_gemm_any (every dense contraction the bf16 prompt GEMM does not take: the fp32 configuration, odd shapes,
    strided operands) against a float64 matmul rounded once: fp32 within summation-order noise, bf16 within one ulp;
    row-major, transposed (k slowest) and padded views of either operand give the same values."""
    g = gen(64)
    x = torch.randn(M, K, generator=g).to(dtype)
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    ref = (x.double() @ W.double().t()).to(dtype)
    xd, Wd = dev(x), dev(W)
    got = hip.gemm_any(xd, Wd)
    check(got, ref, dtype)
    xt = xd.t().contiguous().t()                      # element (m,k) at k*M + m
    Wt = Wd.t().contiguous().t()
    assert torch.equal(hip.gemm_any(xt, Wt), got)
    wide = torch.full((M, K + 3), float("nan"), dtype=dtype, device="cuda")
    wide[:, :K] = xd
    out = torch.full((M, N + 5), float("nan"), dtype=dtype, device="cuda")
    hip.gemm_any(wide[:, :K], Wd, out=out[:, :N])
    assert torch.equal(out[:, :N], got) and bool(torch.isnan(out[:, N:]).all())
    # the dispatcher takes what the bf16 matrix-core kernel refuses (and fp32 beyond 16 rows) to this kernel
    if M > 16:
        check(hip.linear(xd, Wd), ref, dtype)
        b = torch.randn(N, generator=g).to(dtype)
        check(hip.linear(xd, Wd, dev(b)), (ref.float() + b.float()).to(dtype), dtype, frac=0.05,
              atol=2.0 ** -7 * float(ref.float().abs().max()))


@pytest.mark.parametrize("nb,M,N,K", [(1, 128, 64, 64), (3, 256, 132, 192), (2, 1024, 1024, 1536), (4, 512, 260, 2048),
                                      (1, 4096, 768, 3072)])
def test_gemm_bf16_transposed_activations(hip, nb, M, N, K):
    """fstu_gemm_bf16_ta (the exact-mode contraction over time-major slabs, reference stu.py:107-120): every slab
    (K, M) with M contiguous against F.linear of its transpose in fp32 rounded once; the residual form adds in place;
    slab rows that are a view of a wider buffer (row stride > M); and bit-identity with fstu_gemm_bf16 on a row-major
    copy of the same operand (same tiles, same summation order)."""
    g = gen(63)
    A = torch.randn(nb, K, M, generator=g).bfloat16()
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    res = torch.randn(nb, M, N, generator=g).bfloat16()
    ref = torch.stack([F.linear(A[b].t().float(), W.float()) for b in range(nb)]).bfloat16()
    Ad, Wd = dev(A), dev(W)
    got = hip.gemm_ta(Ad, Wd)
    check(got, ref, torch.bfloat16)
    rd = dev(res.clone())
    out = hip.gemm_ta(Ad, Wd, residual=rd, out=rd)
    assert out.data_ptr() == rd.data_ptr()
    check(rd, (res.float() + ref.float()).bfloat16(), torch.bfloat16, frac=0.05, atol=2.0 ** -7 * float(ref.float().abs().max()))
    wide = torch.full((nb, K, M + 256), float("nan"), dtype=torch.bfloat16, device="cuda")
    wide[:, :, :M] = Ad
    assert torch.equal(hip.gemm_ta(wide[:, :, :M], Wd), got)
    if K % 64 == 0 and M > 32:
        rowmajor = torch.stack([hip.gemm(Ad[b].t().contiguous(), Wd) for b in range(nb)])
        frac = float((rowmajor != got).float().mean())
        assert frac <= 1e-3, frac            # another tile shape may be picked: same values up to rare rounding flips
    with pytest.raises(hip.FlashSTUHipError):
        hip.gemm_ta(Ad[:, :, :100], Wd)      # M not a multiple of 128
    with pytest.raises(hip.FlashSTUHipError):
        hip.gemm_ta(Ad.transpose(1, 2), Wd)  # M not the contiguous index


@pytest.mark.parametrize("M,d,I", [(4096, 768, 3072), (300, 256, 1000), (2048, 1024, 8192), (100, 96, 132)])
def test_gemm_bf16_gated_pair(hip, M, d, I):
    """Mode 1: T(T(gelu_tanh(T(x Wg^T))) * T(x Wu^T)) in one kernel equals the three-step bf16 chain of the reference
    MLP (flash_stu/modules/swiglu.py:23-26)."""
    g = gen(62)
    x = torch.randn(M, d, generator=g).bfloat16()
    Wg = (torch.randn(I, d, generator=g) / math.sqrt(d)).bfloat16()
    Wu = (torch.randn(I, d, generator=g) / math.sqrt(d)).bfloat16()
    act = hip.gemm(dev(x), dev(Wg), up_weight=dev(Wu))
    gate = F.linear(x.float(), Wg.float()).bfloat16()
    up = F.linear(x.float(), Wu.float()).bfloat16()
    ref = F.gelu(gate, approximate="tanh") * up
    # a different fp32 summation order may flip the rounding of either projection by one ulp: a flip of `up` and the
    # roundings of gelu and of the product stay within two ulps of the product; a flip of `gate` passes through gelu's
    # slope (<= 1.13), which for negative gates is large against gelu(gate) itself: 1.2 ulp(gate) * |up|
    got, r = act.float().cpu(), ref.float()
    tol = r.abs() * 2.0 ** -6 + 1.2 * 2.0 ** -7 * (gate.float() * up.float()).abs() + 1e-3 * 2.0 ** -7 * float(r.abs().max())
    assert bool(((got - r).abs() <= tol).all()), float(((got - r).abs() - tol).max())
    assert float(((got - r).abs() > 0).float().mean()) <= 0.05


@pytest.mark.parametrize("M,N,K,ks", [(32, 2048, 8192, 16), (17, 768, 3072, 4), (300, 132, 512, 2), (32, 256, 64, 1)])
def test_gemm_bf16_splitk_feeds_the_residual_norm(hip, M, N, K, ks):
    """fstu_gemm_bf16_splitk leaves fp32 slice sums; fstu_add_rmsnorm (delta_mode 1) folds them into the residual stream
    as T(x + T(sum)) and normalises: the down projection of a decode step over 17..32 rows."""
    g = gen(64)
    act = torch.randn(M, K, generator=g).bfloat16()
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    x = torch.randn(M, N, generator=g).bfloat16()
    nw = (1 + 0.1 * torch.randn(N, generator=g)).bfloat16()
    part = hip.gemm_splitk(dev(act), dev(W), ks)
    assert part.shape == (ks, M, N) and part.dtype == torch.float32
    full = F.linear(act.float(), W.float())
    assert float((part.sum(0).cpu() - full).abs().max()) <= 2e-5 * float(full.abs().max()) * math.sqrt(K / 64)
    xd = dev(x.clone())
    h = hip.add_rmsnorm(xd, part, dev(nw), O.RMS_EPS_DEFAULT, delta_mode=1, nslices=ks)
    xr = (x.float() + full.bfloat16().float()).bfloat16()
    check(xd, xr, torch.bfloat16, frac=0.05, atol=2.0 ** -7 * float(full.abs().max()))
    check(h, O.rms_norm(xd.cpu(), nw, O.RMS_EPS_DEFAULT), torch.bfloat16, frac=0.05)


def test_gemm_bf16_strided_operands_and_errors(hip):
    g = gen(63)
    big = torch.randn(200, 3, 128, generator=g).bfloat16()
    W = (torch.randn(64, 128, generator=g) / 11).bfloat16()
    bd = dev(big)
    out = torch.zeros(200, 2, 64, dtype=torch.bfloat16, device="cuda")
    hip.gemm(bd[:, 1, :], dev(W), out=out[:, 1, :])
    check(out[:, 1].cpu(), F.linear(big[:, 1].float(), W.float()).bfloat16(), torch.bfloat16)
    assert float(out[:, 0].abs().max()) == 0
    with pytest.raises(hip.FlashSTUHipError):
        hip.gemm(dev(torch.zeros(32, 40).bfloat16()), dev(torch.zeros(8, 40).bfloat16()))       # K % 32
    with pytest.raises(hip.FlashSTUHipError):
        hip.gemm(dev(torch.zeros(32, 64)), dev(torch.zeros(8, 64)))                               # fp32
    with pytest.raises(hip.FlashSTUHipError):
        hip.gemm(bd[:, 1, :], dev(W), up_weight=dev(W), residual=out[:, 1, :])


@pytest.mark.parametrize("dtype", DTYPES)
def test_gelu_mul(hip, dtype):
    g = gen(5)
    a = (3 * torch.randn(4, 1000, generator=g)).to(dtype)
    b = torch.randn(4, 1000, generator=g).to(dtype)
    check(hip.gelu_mul(dev(a), dev(b)), F.gelu(a, approximate="tanh") * b, dtype)


def _stu_setup(dtype, B, T, d, L, K, seed):
    g = gen(seed)
    phi = torch.tensor(O.get_spectral_filters_f64(L, K)).to(dtype)
    Mf = (torch.randn(K, d, generator=g) / math.sqrt(K)).to(dtype)
    xp = torch.randn(B, T, d, generator=g).to(dtype)
    filt = phi @ Mf
    n = O.nearest_power_of_two(2 * L - 1, True)
    plus, minus = O.convolve(xp, filt, n, use_approx=True)
    return xp, filt, plus + minus, plus


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,T,d,L", [(2, 100, 96, 128), (1, 64, 256, 1024), (3, 120, 100, 128)])
def test_stu_conv_direct(hip, dtype, B, T, d, L):
    xp, filt, ref, plus = _stu_setup(dtype, B, T, d, L, 8, 6)
    # the two branches are rounded before they are added: a flip costs one ulp of a branch
    atol = 2.0 ** -7 * float(plus.float().abs().max()) if dtype == torch.bfloat16 else 0.0
    check(hip.stu_conv_direct(dev(xp), dev(filt)), ref, dtype, frac=0.05, atol=atol)
    check(hip.stu_conv_direct(dev(xp), dev(filt), single_branch=True), plus, dtype, frac=0.05)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,T,d,L", [(2, 100, 96, 128), (1, 64, 256, 1024), (3, 120, 100, 128), (2, 17, 5, 64),
                                     (2, 512, 64, 512), (1, 1000, 48, 1024), (1, 2048, 32, 2048), (1, 4096, 8, 4096),
                                     (1, 3000, 4, 8192), (1, 8192, 2, 8192), (4, 4096, 1024, 4096), (4, 8192, 1024, 8192),
                                     (2, 200, 64, 256), (3, 256, 96, 256), (2, 3500, 2048, 4096)])
def test_stu_conv_fft(hip, dtype, B, T, d, L):
    """The FFT form against the oracle's rfft/irfft convolution, every transform length 64..16384
    (radix splits 4*16, 8*16, 16*16, 2*16*16 ... 4*16*16*16), ragged channel counts, T < L and T == L; the last two
    shapes have enough columns for the row-piece kernel at the two longest lengths."""
    if L <= 1024:
        xp, filt, ref, plus = _stu_setup(dtype, B, T, d, L, 8, 6)
    else:                                  # no eigendecomposition of a large Hankel matrix in a GPU test
        g = gen(6)
        filt = (torch.randn(L, d, generator=g) * torch.linspace(1, 0.02, L)[:, None] / 8).to(dtype)
        xp = torch.randn(B, T, d, generator=g).to(dtype)
        plus, minus = O.convolve(xp, filt, O.nearest_power_of_two(2 * L - 1, True), use_approx=True)
        ref = plus + minus
    n = hip.fft_length(T)
    assert n >= 2 * T and (n == 64 or n < 4 * T)
    atol = 2.0 ** -7 * float(plus.float().abs().max()) if dtype == torch.bfloat16 else 0.0
    spec = hip.stu_fft_filter(dev(filt), n)
    check(hip.stu_conv_fft(dev(xp), spec), ref, dtype, frac=0.05, atol=atol)
    spec1 = hip.stu_fft_filter(dev(filt), n, single_branch=True)
    check(hip.stu_conv_fft(dev(xp), spec1, single_branch=True), plus, dtype, frac=0.05)


def test_stu_conv_fft_equals_direct_fp32(hip):
    """Both forms of the library on the same input: equal to fp32 round-off, and a delta returns the filter."""
    g = gen(21)
    B, T, d, L = 2, 700, 40, 1024
    filt = (torch.randn(L, d, generator=g) * torch.linspace(1, 0.01, L)[:, None]).float()
    xp = torch.randn(B, T, d, generator=g)
    xp[1] = 0
    xp[1, 3, :] = 1.0
    n = hip.fft_length(T)
    yf = hip.stu_conv_fft(dev(xp), hip.stu_fft_filter(dev(filt), n, single_branch=True), single_branch=True).cpu()
    yd = hip.stu_conv_direct(dev(xp), dev(filt), single_branch=True).cpu()
    s = float(yd.abs().max())
    assert float((yf - yd).abs().max()) <= 5e-6 * s
    assert float((yf[1, 3:] - filt[: T - 3]).abs().max()) <= 5e-6 * float(filt.abs().max())
    assert float(yf[1, :3].abs().max()) <= 5e-6 * float(filt.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,T,d,L,K", [(2, 100, 24, 128, 5), (1, 600, 6, 1024, 24), (1, 5000, 2, 8192, 3)])
def test_stu_conv_bank_fft(hip, dtype, B, T, d, L, K):
    """Exact-mode bank by FFT == the time-domain bank kernel == the oracle's convolve(use_approx=False),
    in the (B,T,K,d) layout and in the time-major layout the contraction consumes."""
    g = gen(22)
    phi = O.get_spectral_filters(L, K, dtype=dtype) if L <= 1024 else \
        (torch.randn(L, K, generator=g) * torch.linspace(1, 0.01, L)[:, None]).to(dtype)
    x = torch.randn(B, T, d, generator=g).to(dtype)
    n_ref = O.nearest_power_of_two(2 * L - 1, True)
    rp, rm = O.convolve(x, phi, n_ref, use_approx=False)
    n = hip.fft_length(T)
    spec = hip.stu_fft_filter(dev(phi), n)
    up = torch.empty(B, T, K, d, dtype=dtype, device="cuda")
    um = torch.empty_like(up)
    hip.stu_conv_bank_fft(dev(x), spec, up, um)
    sc = float(rp.float().abs().max())
    check(up, rp, dtype, frac=0.05, scale=sc)
    check(um, rm, dtype, frac=0.05, scale=sc)
    # time-major outputs (B,K,d,T) viewed as (B,T,K,d), time-major input
    upt = torch.empty(B, K, d, T, dtype=dtype, device="cuda")
    xt = dev(x).transpose(1, 2).contiguous().transpose(1, 2)
    hip.stu_conv_bank_fft(xt, spec, upt.permute(0, 3, 1, 2), None)
    assert torch.equal(upt.permute(0, 3, 1, 2), up)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,T,d,L,nsplit", [(2, 100, 96, 128, 3), (8, 257, 768, 512, 4), (1, 50, 100, 64, 1),
                                             (2, 128, 2048, 128, 2)])  # T <= L: the reference's FFT length assumes it
def test_stu_step_hist(hip, dtype, B, T, d, L, nsplit):
    """Newest-position output of the history step == last row of the oracle's
    FFT convolution, at several t including t >= L-1."""
    xp, filt, ref, plus = _stu_setup(dtype, B, T, d, L, 8, 7)
    atol = 2.0 ** -7 * float(plus.float().abs().max()) if dtype == torch.bfloat16 else 0.0
    cap = T + 3
    hist = torch.zeros(B, cap, d, dtype=dtype)
    hist[:, :T] = xp
    hd_, fd = dev(hist), dev(filt)
    for t in (0, 1, T // 2, T - 1):
        eo = hip.stu_step_hist(hd_, fd, t, nsplit)
        x = torch.zeros(B, d, dtype=dtype, device="cuda")
        hip.add_rmsnorm(x, eo, None, O.RMS_EPS_DEFAULT, delta_mode=2, nslices=nsplit, want_norm=False)
        check(x, ref[:, t], dtype, frac=0.05, scale=float(ref.abs().max()), atol=atol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,T,d,L", [(2, 100, 96, 128), (1, 20, 8, 64), (2, 64, 40, 64)])
def test_convolve_operator_matches_oracle(hip, dtype, B, T, d, L):
    """flash_stu.utils.stu_utils.convolve with the reference's signature: both branches, one branch, exact mode."""
    from flash_stu.utils.stu_utils import convolve, nearest_power_of_two
    xp, filt, _, _ = _stu_setup(dtype, B, T, d, L, 8, 6)
    n = nearest_power_of_two(2 * L - 1, round_up=True)
    assert n == O.nearest_power_of_two(2 * L - 1, True)
    rp, rm = O.convolve(xp, filt, n, use_approx=True)
    gp, gm = convolve(dev(xp), dev(filt), n, use_approx=True)
    check(gp, rp, dtype, frac=0.05)
    check(gm, rm, dtype, frac=0.05)
    only, none = convolve(dev(xp), dev(filt), n, use_approx=True, return_both=False)
    assert none is None and torch.equal(only, gp)
    phi = torch.tensor(O.get_spectral_filters_f64(L, 6)).to(dtype)
    ep, em = O.convolve(xp, phi, n, use_approx=False)
    bp, bm = convolve(dev(xp), dev(phi), n, use_approx=False)
    check(bp, ep, dtype, frac=0.05)
    check(bm, em, dtype, frac=0.05)
    with pytest.raises(ValueError):
        convolve(dev(xp), dev(filt), T, use_approx=True)          # n shorter than the linear convolution


@pytest.mark.parametrize("B,T,d,L,both", [(2, 70, 24, 70, True), (3, 40, 16, 64, True), (2, 20, 8, 32, False), (2, 50, 12, 30, True)])
def test_convolve_operator_gradients(hip, B, T, d, L, both):
    """Backward of the approx-mode convolution (every piece is the forward kernel on time-reversed operands) against
    autograd through the oracle's FFT convolution, fp32; filters longer and shorter than the input."""
    from flash_stu.utils.stu_utils import convolve
    g = gen(31)
    u = torch.randn(B, T, d, generator=g)
    v = torch.randn(L, d, generator=g) / math.sqrt(L)
    wp, wm = torch.randn(B, T, d, generator=g), torch.randn(B, T, d, generator=g)
    n = O.nearest_power_of_two(2 * max(L, T) - 1, True)
    uo, vo = u.clone().requires_grad_(True), v.clone().requires_grad_(True)
    rp, rm = O.convolve(uo, vo, n, use_approx=True)
    loss = (rp * wp).sum() + ((rm * wm).sum() if both else 0.0)
    loss.backward()
    ud, vd = dev(u).requires_grad_(True), dev(v).requires_grad_(True)
    gp, gm = convolve(ud, vd, n, use_approx=True, return_both=both)
    lossd = (gp * dev(wp)).sum() + ((gm * dev(wm)).sum() if both else 0.0)
    lossd.backward()
    su, sv = float(uo.grad.abs().max()), float(vo.grad.abs().max())
    assert float((ud.grad.cpu() - uo.grad).abs().max()) <= 1e-4 * su
    assert float((vd.grad.cpu() - vo.grad).abs().max()) <= 1e-4 * sv
    with pytest.raises(NotImplementedError):
        convolve(ud, dev(torch.randn(L, 4)), n, use_approx=False)


def _fit_lds(filt_even, S):
    """ridge fit of the even-lag filter by S real poles (host-side helper of the product)."""
    from flash_stu.utils.lds_fit import fit_even_lag_lds
    return fit_even_lag_lds(filt_even, S)


@pytest.mark.parametrize("dtype", DTYPES)
def test_stu_step_lds_recurrence(hip, dtype):
    """The kernel's recurrence equals a float64 evaluation of the same
    recurrence, and the state builder equals stepping from zero."""
    g = gen(8)
    B, S, d, T = 3, 64, 256, 41
    a = (0.5 + 0.49 * torch.rand(S, generator=g)).float()
    ce = (torch.randn(S, d, generator=g) / S).float()
    xs = torch.randn(T, B, d, generator=g).to(dtype)
    state = torch.zeros(B, 2, S, d, device="cuda")
    h64 = torch.zeros(B, 2, S, d, dtype=torch.float64)
    ad, ced = dev(a), dev(ce)
    for t in range(T):
        y = hip.stu_step_lds(state, dev(xs[t]), ad, ced, t)
        p = t & 1
        h64[:, p] = a.double()[None, :, None] * h64[:, p] + xs[t].double()[:, None, :]
        ref = 2 * (ce.double()[None] * h64[:, p]).sum(1)
        check(y, ref.to(dtype), dtype, frac=0.05, scale=float(ref.abs().max()))
    assert float((state.cpu().double() - h64).abs().max()) < 1e-4 * float(h64.abs().max())
    hist = torch.zeros(B, T + 5, d, dtype=dtype)
    hist[:, :T] = xs.transpose(0, 1)
    st2 = hip.stu_lds_state_from_hist(dev(hist), ad, T - 1)
    assert float((st2.cpu().double() - h64).abs().max()) < 1e-4 * float(h64.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,S,d,T,t_start", [(3, 64, 256, 41, 0), (2, 64, 768, 512, 0), (2, 40, 200, 37, 5), (1, 128, 64, 130, 1),
                                             (2, 64, 128, 1, 3), (2, 8, 72, 16, 0)])
def test_stu_scan_lds_equals_steps_and_float64(hip, dtype, B, S, d, T, t_start):
    """The whole-sequence recurrence: outputs equal a float64 evaluation of the recurrence, the final state equals
    T single-token steps bit for bit; ragged channel counts, odd start positions, S not a multiple of 8, and a
    sequence continued from a carried state in two pieces of odd length."""
    g = gen(8)
    a = (0.5 + 0.49 * torch.rand(S, generator=g)).float()
    ce = (torch.randn(S, d, generator=g) / S).float()
    xs = torch.randn(B, T, d, generator=g).to(dtype)
    h64 = torch.zeros(B, 2, S, d, dtype=torch.float64)
    ref = torch.zeros(B, T, d, dtype=torch.float64)
    for t in range(T):
        p = (t_start + t) & 1
        h64[:, p] = a.double()[None, :, None] * h64[:, p] + xs[:, t].double()[:, None, :]
        ref[:, t] = 2 * (ce.double()[None] * h64[:, p]).sum(1)
    ad, ced, xd = dev(a), dev(ce), dev(xs)
    y, st = hip.stu_scan_lds(xd, ad, ced, t_start=t_start)
    check(y, ref.to(dtype), dtype, frac=0.05, scale=float(ref.abs().max()))
    assert float((st.cpu().double() - h64).abs().max()) <= 1e-4 * float(h64.abs().max())
    if T <= 64:
        step_state = torch.zeros(B, 2, S, d, device="cuda")
        ys = [hip.stu_step_lds(step_state, xd[:, t].contiguous(), ad, ced, t_start + t) for t in range(T)]
        assert torch.equal(st, step_state)
        check(y, torch.stack(ys, 1).float().cpu().to(dtype), dtype, frac=0.05, scale=float(ref.abs().max()))
    if T >= 3:
        cut = (T // 2) | 1
        y1, st1 = hip.stu_scan_lds(xd[:, :cut], ad, ced, t_start=t_start)
        y2, st2 = hip.stu_scan_lds(xd[:, cut:], ad, ced, state=st1, t_start=t_start + cut)
        assert st2.data_ptr() == st1.data_ptr()
        assert torch.equal(torch.cat([y1, y2], 1), y) and torch.equal(st2, st)


def test_stu_scan_lds_rejects_bad_arguments(hip):
    a = torch.full((200,), 0.9, device="cuda")
    x = torch.zeros(1, 4, 64, device="cuda")
    with pytest.raises(RuntimeError):
        hip.stu_scan_lds(x, a, torch.zeros(200, 64, device="cuda"))          # S > 128
    with pytest.raises(RuntimeError):
        hip.stu_scan_lds(torch.zeros(1, 4, 66, device="cuda", dtype=torch.bfloat16), a[:8], torch.zeros(8, 66, device="cuda"))


def test_stu_inproj_step_equals_projection_then_step(hip):
    g = gen(21)
    B, S, d = 8, 64, 768
    a = dev((0.5 + 0.49 * torch.rand(S, generator=g)).float())
    ce = dev((torch.randn(S, d, generator=g) / S).float())
    Mt = dev((torch.randn(d, d, generator=g) / math.sqrt(d)).bfloat16())
    st1 = dev(torch.randn(B, 2, S, d, generator=g))
    st2 = st1.clone()
    co = dev((torch.randn(S, d, generator=g) / S).float())
    for t in range(5):
        h = dev(torch.randn(B, d, generator=g).bfloat16())
        xp = hip.linear_decode(h, Mt)
        y_ref = hip.stu_step_lds(st1, xp, a, ce, t)
        xp2 = torch.empty_like(xp)
        y = hip.stu_inproj_step(h, Mt, st2, a, ce, t, xp_out=xp2)
        assert torch.equal(xp2, xp)
        check(y, y_ref, torch.bfloat16, frac=0.02)
        assert float((st1 - st2).abs().max()) == 0.0
        # with odd-lag weights: the step of stu_step_lds(pair=True)
        y_pair_ref = hip.stu_step_lds(st1.clone(), xp, a, ce, t, co=co, pair=True)
        y_pair = hip.stu_inproj_step(h, Mt, st2.clone(), a, ce, t, co=co)
        check(y_pair, y_pair_ref, torch.bfloat16, frac=0.03, atol=2.0 ** -8 * float(y_pair_ref.float().abs().max()))


@pytest.mark.parametrize("B,ns", [(8, 4), (3, 2), (1, 1)])
def test_stu_res_inproj_step_equals_add_norm_then_step(hip, B, ns):
    """Split-K slices + residual + RMSNorm as the prologue of the projection+step launch == fstu_add_rmsnorm followed
    by the plain launch: the residual bit for bit, the output up to the summation order of the row statistics."""
    g = gen(22)
    S, d = 64, 768
    a = dev((0.5 + 0.49 * torch.rand(S, generator=g)).float())
    ce = dev((torch.randn(S, d, generator=g) / S).float())
    Mt = dev((torch.randn(d, d, generator=g) / math.sqrt(d)).bfloat16())
    nw = dev((1 + 0.1 * torch.randn(d, generator=g)).bfloat16())
    st1 = dev(torch.randn(B, 2, S, d, generator=g))
    st2 = st1.clone()
    for t in range(4):
        x = dev(torch.randn(B, d, generator=g).bfloat16())
        part = dev(0.3 * torch.randn(ns, B, d, generator=g))
        x_ref = x.clone()
        h = hip.add_rmsnorm(x_ref, part, nw, O.RMS_EPS_DEFAULT, delta_mode=1, nslices=ns)
        y_ref = hip.stu_inproj_step(h, Mt, st1, a, ce, t)
        x_out, y = hip.stu_res_inproj_step(x, part, nw, O.RMS_EPS_DEFAULT, Mt, st2, a, ce, t)
        assert torch.equal(x_out, x_ref)
        check(y, y_ref, torch.bfloat16, frac=0.05)
        assert float((st1 - st2).abs().max()) <= 2.0 ** -7 * float(st1.abs().max())


@pytest.mark.parametrize("L", [128, 1024])
def test_stu_step_lds_tracks_the_convolution(hip, L):
    """With poles/weights fitted to the effective filter, the recurrence
    reproduces the oracle's convolution output to well below one bf16 ulp."""
    dtype = torch.float32
    B, d, K, S = 2, 128, 24 if L >= 256 else 8, 64
    T = L
    xp, filt, ref, _ = _stu_setup(dtype, B, T, d, L, K, 9)
    a, ce, err = _fit_lds(filt.double()[0::2], S)
    state = torch.zeros(B, 2, S, d, device="cuda")
    ad, ced = dev(a), dev(ce)
    worst = 0.0
    for t in range(T):
        y = hip.stu_step_lds(state, dev(xp[:, t].contiguous()), ad, ced, t)
        worst = max(worst, float((y.cpu() - ref[:, t]).abs().max()))
    assert worst < 1e-3 * float(ref.abs().max()), (worst, float(ref.abs().max()), err)


def test_stu_step_lds_pair_keeps_the_reference_rounding_points(hip):
    """bf16, two sign branches: the reference rounds plus = E+O and minus = E-O separately before adding them
    (stu_utils.py:226-228, stu.py:120).  The pair step forms E on the bank of the token's parity and O on the other
    bank and rounds the same way: the kernel equals a float64 evaluation of that recurrence with those roundings, and
    its outputs differ from the oracle's convolution on far fewer elements than T(2E), which drops O."""
    dtype = torch.bfloat16
    B, d, L, K, S = 2, 128, 1024, 24, 64
    T = 600
    xp, filt, ref, _ = _stu_setup(dtype, B, T, d, L, K, 9)
    a, ce, _ = _fit_lds(filt[0::2], S)
    a2, co, _ = _fit_lds(filt[1::2], S)
    assert torch.equal(a, a2)
    st_pair = torch.zeros(B, 2, S, d, device="cuda")
    st_2e = torch.zeros(B, 2, S, d, device="cuda")
    h64 = torch.zeros(B, 2, S, d, dtype=torch.float64)
    ad, ced, cod = dev(a), dev(ce), dev(co)
    bad_pair = bad_2e = bad_model = total = 0
    rb = lambda v: v.float().to(dtype).double()
    for t in range(T):
        xt = dev(xp[:, t].contiguous())
        y = hip.stu_step_lds(st_pair, xt, ad, ced, t, co=cod, pair=True).cpu()
        y2 = hip.stu_step_lds(st_2e, xt, ad, ced, t).cpu()
        p = t & 1
        h64[:, p] = a.double()[None, :, None] * h64[:, p] + xp[:, t].double()[:, None, :]
        E = (ce.double()[None] * h64[:, p]).sum(1)
        Od = (co.double()[None] * h64[:, p ^ 1]).sum(1)
        model = rb(rb(E + Od) + rb(E - Od))
        bad_model += int((y.double() != model).sum())
        if t >= 64:
            bad_pair += int((y != ref[:, t]).sum())
            bad_2e += int((y2 != ref[:, t]).sum())
            total += y.numel()
    assert torch.equal(st_pair, st_2e)
    assert bad_model <= 0.03 * T * B * d, bad_model           # fp32 vs float64 accumulation flips a rounding now and then
    print(f"elements differing from the oracle: pair {bad_pair / total:.3f}, T(2E) {bad_2e / total:.3f}")
    assert bad_pair <= 0.22 * total and bad_pair < 0.6 * bad_2e, (bad_pair / total, bad_2e / total)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_stu_step_lds_pair_joins_the_residual_stream(hip, dtype):
    """The pair step with a residual row: y = T(res + T(step output)), bit for bit the plain step followed by an add
    in the model dtype, in place on the stream and with identical states."""
    B, d, S = 3, 384, 64
    g = gen(91)
    a = dev(torch.rand(S, generator=g) * 0.9)
    ce, co = dev(torch.randn(S, d, generator=g) / 8), dev(torch.randn(S, d, generator=g) / 8)
    st1 = torch.zeros(B, 2, S, d, device="cuda")
    st2 = torch.zeros(B, 2, S, d, device="cuda")
    stream = dev(torch.randn(B, d, generator=g).to(dtype))
    for t in range(5):
        xt = dev(torch.randn(B, d, generator=g).to(dtype))
        want = stream + hip.stu_step_lds(st1, xt, a, ce, t, co=co, pair=True)
        got = hip.stu_step_lds(st2, xt, a, ce, t, co=co, pair=True, res=stream, out=stream)
        assert got is stream and torch.equal(stream, want)
    assert torch.equal(st1, st2)


@pytest.mark.parametrize("dtype,S,R,T0", [(torch.bfloat16, 64, 64, 70), (torch.bfloat16, 64, 64, 1), (torch.bfloat16, 80, 128, 5),
                                          (torch.float32, 64, 8, 3), (torch.bfloat16, 24, 0, 9), (torch.float32, 72, 256, 300)])
def test_stu_step_lds_pair_with_the_odd_lag_sum_handed_on(hip, dtype, S, R, T0):
    """The pair step that takes O from the previous step (or from the priming launch after a prompt of T0 positions)
    and never reads the other bank equals the plain pair step bit for bit: outputs, both banks and the ring, with and
    without the exact head (R taps; beyond 64 modes / 64 taps the kernels' loops), with and without a residual row."""
    B, d = 3, 256
    g = gen(93)
    a = dev(torch.rand(S, generator=g) * 0.95)
    ce, co = dev(torch.randn(S, d, generator=g) / 8), dev(torch.randn(S, d, generator=g) / 8)
    fir = dev(torch.randn(R, d, generator=g) / 16) if R else None
    ring_p = torch.zeros(B, R, d, dtype=dtype, device="cuda") if R else None
    st_p = torch.zeros(B, 2, S, d, device="cuda")
    xs = torch.randn(T0 + 12, B, d, generator=g).to(dtype)
    for t in range(T0):                                   # the "prompt", stepped by the plain kernel
        hip.stu_step_lds(st_p, dev(xs[t]), a, ce, t, co=co, pair=True, ring=ring_p, fir=fir)
    st_c, ring_c = st_p.clone(), (ring_p.clone() if R else None)
    oc = hip.stu_step_lds_prime(st_c, a, co, T0 - 1, dtype, ring=ring_c, fir=fir)
    assert torch.equal(st_c, st_p) and (not R or torch.equal(ring_c, ring_p))      # priming writes nothing else
    stream = dev(torch.randn(B, d, generator=g).to(dtype))
    for t in range(T0, T0 + 12):
        xt = dev(xs[t])
        want = hip.stu_step_lds(st_p, xt, a, ce, t, co=co, pair=True, ring=ring_p, fir=fir)
        if t % 3 == 0:                                    # joined with the residual stream now and then
            got = hip.stu_step_lds(st_c, xt, a, ce, t, co=co, pair=True, ring=ring_c, fir=fir, ocache=oc, res=stream)
            assert torch.equal(got, stream + want), t
        else:
            got = hip.stu_step_lds(st_c, xt, a, ce, t, co=co, pair=True, ring=ring_c, fir=fir, ocache=oc)
            assert torch.equal(got, want), t
        assert torch.equal(st_c[:, t & 1], st_p[:, t & 1])
    assert torch.equal(st_c, st_p) and (not R or torch.equal(ring_c, ring_p))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,R,C", [(1, 4096, 2048), (3, 100, 70), (2, 64, 64), (1, 1, 5), (2, 129, 1)])
def test_transpose(hip, dtype, B, R, C):
    x = dev(torch.randn(B, R, C, generator=gen(95)).to(dtype))
    assert torch.equal(hip.transpose(x), x.transpose(1, 2).contiguous())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,T,d", [(1, 4096, 256), (2, 2100, 64), (1, 600, 40)])
def test_stu_conv_fft_on_time_major_slabs(hip, dtype, B, T, d):
    """The strided entry on time-major slabs gives the bits of the channel-contiguous call (every transform length,
    both kernels behind them)."""
    g = gen(96)
    xp = dev(torch.randn(B, T, d, generator=g).to(dtype))
    filt = dev((torch.randn(T, d, generator=g) / 30).to(dtype))
    n = hip.fft_length(T)
    spec = hip.stu_fft_filter(filt, n)
    want = hip.stu_conv_fft(xp, spec)
    xt = hip.transpose(xp)
    yt = torch.empty_like(xt)
    hip.stu_conv_fft_strided(xt.transpose(1, 2), spec, yt.transpose(1, 2))
    assert torch.equal(hip.transpose(yt), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,R", [(600, 64), (64, 64), (65, 64), (40, 64), (1, 8), (300, 256), (1000, 8)])
def test_state_from_hist_also_leaves_the_ring(hip, dtype, T, R):
    """The launch that scans a prompt's projected inputs into the recurrence state also writes the exact head's ring:
    position t in slot t % R for the last R positions, zeros (the caller's) where a short prompt has none; the state
    is the one the launch without a ring leaves."""
    B, d, S = 3, 200, 64
    g = gen(94)
    xp = dev(torch.randn(B, T, d, generator=g).to(dtype))
    a = dev(torch.rand(S, generator=g) * 0.95)
    ring = torch.zeros(B, R, d, dtype=dtype, device="cuda") if T < R else torch.full((B, R, d), float("nan"), dtype=dtype, device="cuda")
    st = hip.stu_lds_state_from_hist(xp, a, T - 1, ring=ring)
    assert torch.equal(st, hip.stu_lds_state_from_hist(xp, a, T - 1))
    want = torch.zeros(B, R, d, dtype=dtype, device="cuda")
    for t in range(max(0, T - R), T):
        want[:, t % R] = xp[:, t]
    assert torch.equal(ring, want)


@pytest.mark.parametrize("R", [8, 32, 128, 256])
def test_stu_step_lds_exact_head(hip, R):
    """The exact head of the distilled filter: fir[s] = phi_proj[s] - fitted filter for the first R lags, applied to a
    ring of the last R projected inputs, even lags into E and odd lags into O.  The kernel equals a float64 evaluation
    of recurrence + head with the reference's two roundings, the ring ends up holding the last R inputs, and the
    outputs differ from the oracle's convolution on fewer elements than without the head.  The fused
    projection + step launch gives the same values."""
    dtype = torch.bfloat16
    B, d, L, K, S = 2, 256, 1024, 24, 64
    T = 300
    xp, filt, ref, _ = _stu_setup(dtype, B, T, d, L, K, 9)
    a, ce, _ = _fit_lds(filt[0::2], S)
    a2, co, _ = _fit_lds(filt[1::2], S)
    m = torch.arange(R // 2, dtype=torch.float64)
    V = a.double()[None, :] ** m[:, None]
    fit = torch.empty(R, d, dtype=torch.float64)
    fit[0::2] = V @ ce.double()
    fit[1::2] = V @ co.double()
    fir = (filt[:R].double() - fit).float()
    g = gen(77)
    Kin = 256
    Mt = (torch.randn(d, Kin, generator=g) / 16).to(dtype)          # a projection whose outputs are the test's x_proj
    st = torch.zeros(B, 2, S, d, device="cuda")
    st0 = torch.zeros(B, 2, S, d, device="cuda")
    st_f = torch.zeros(B, 2, S, d, device="cuda")
    ring = torch.zeros(B, R, d, dtype=dtype, device="cuda")
    ring_f = torch.zeros(B, R, d, dtype=dtype, device="cuda")
    h64 = torch.zeros(B, 2, S, d, dtype=torch.float64)
    ad, ced, cod, fird, Mtd = dev(a), dev(ce), dev(co), dev(fir), dev(Mt)
    rb = lambda v: v.float().to(dtype).double()
    bad_model = bad_head = bad_plain = total = fused_diff = 0
    hs = torch.randn(T, B, Kin, generator=g).to(dtype)
    xf_hist = []
    for t in range(T):
        xt = dev(xp[:, t].contiguous())
        y = hip.stu_step_lds(st, xt, ad, ced, t, co=cod, pair=True, ring=ring, fir=fird).cpu()
        y0 = hip.stu_step_lds(st0, xt, ad, ced, t, co=cod, pair=True).cpu()
        p = t & 1
        h64[:, p] = a.double()[None, :, None] * h64[:, p] + xp[:, t].double()[:, None, :]
        E = (ce.double()[None] * h64[:, p]).sum(1)
        Od = (co.double()[None] * h64[:, p ^ 1]).sum(1)
        for s_ in range(min(R, t + 1)):
            term = fir[s_].double()[None] * xp[:, t - s_].double()
            if s_ & 1:
                Od = Od + term
            else:
                E = E + term
        model = rb(rb(E + Od) + rb(E - Od))
        bad_model += int((y.double() != model).sum())
        if t >= 64:
            bad_head += int((y != ref[:, t]).sum())
            bad_plain += int((y0 != ref[:, t]).sum())
            total += y.numel()
        # fused launch on its own inputs: same values as projection + step
        hd = dev(hs[t])
        st_b, ring_b = st_f.clone(), ring_f.clone()
        xpf = torch.empty(B, d, dtype=dtype, device="cuda")
        got = hip.stu_inproj_step(hd, Mtd, st_f, ad, ced, t, xp_out=xpf, co=cod, ring=ring_f, fir=fird)
        xf_hist.append(xpf.cpu())
        want = hip.stu_step_lds(st_b, xpf, ad, ced, t, co=cod, pair=True, ring=ring_b, fir=fird)
        fused_diff += int((got != want).sum())
    assert bad_model <= 0.03 * T * B * d, bad_model
    # the fused launch reduces the mode groups in another order: a rounding of E+O or E-O flips now and then
    assert fused_diff <= 0.03 * T * B * d, fused_diff
    want_ring = torch.zeros(B, R, d, dtype=dtype)
    for t in range(max(0, T - R), T):
        want_ring[:, t % R] = xp[:, t]
    assert torch.equal(ring.cpu(), want_ring)
    want_ring_f = torch.zeros(B, R, d, dtype=dtype)
    for t in range(max(0, T - R), T):
        want_ring_f[:, t % R] = xf_hist[t]
    assert torch.equal(ring_f.cpu(), want_ring_f)
    print(f"R={R}: elements differing from the oracle: with the head {bad_head / total:.3f}, without {bad_plain / total:.3f}")
    # 4 lags per parity hardly matter; 16 and 64 do (256 taps: beyond the lags the kernels request ahead of time)
    assert bad_head <= (1.01 if R < 32 else 0.9) * bad_plain, (bad_head / total, bad_plain / total)


@pytest.mark.parametrize("dtype", DTYPES)
def test_stu_step_lds_single_branch(hip, dtype):
    """use_hankel_L on the recurrence state: even lags from the bank of the token's parity, odd lags from the other
    bank.  The kernel equals a float64 evaluation of that recurrence, and with weights fitted to the even / odd
    halves of a filter it tracks the oracle's single-branch convolution."""
    B, d, L, K, S = 2, 128, 128, 8, 64
    xp, filt, _, plus = _stu_setup(dtype, B, L, d, L, K, 9)
    a, ce, _ = _fit_lds(filt.double()[0::2], S)
    a2, co, _ = _fit_lds(filt.double()[1::2], S)
    assert torch.equal(a, a2)
    state = torch.zeros(B, 2, S, d, device="cuda")
    h64 = torch.zeros(B, 2, S, d, dtype=torch.float64)
    ad, ced, cod = dev(a), dev(ce), dev(co)
    worst = 0.0
    for t in range(L):
        y = hip.stu_step_lds(state, dev(xp[:, t].contiguous()), ad, ced, t, co=cod)
        p = t & 1
        h64[:, p] = a.double()[None, :, None] * h64[:, p] + xp[:, t].double()[:, None, :]
        ref = (ce.double()[None] * h64[:, p]).sum(1) + (co.double()[None] * h64[:, p ^ 1]).sum(1)
        # the two bank sums cancel in part: fp32 error relative to the larger of them, not to their sum
        check(y, ref.to(dtype), dtype, frac=0.12, scale=float(ref.abs().max()), atol=2.0 ** -10 * float(ref.abs().max()))
        worst = max(worst, float((y.float().cpu() - plus[:, t].float()).abs().max()))
    assert float((state.cpu().double() - h64).abs().max()) < 1e-4 * float(h64.abs().max())
    tol = 1e-3 if dtype == torch.float32 else 2.0 ** -6
    assert worst < tol * float(plus.float().abs().max()), worst


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,hd,W,T", [(2, 4, 64, 16, 50), (8, 12, 64, 512, 600), (1, 16, 128, 32, 40),
                                         (2, 2, 32, 7, 20)])
def test_swa_ring_decode_and_prefill(hip, dtype, B, H, hd, W, T):
    g = gen(10)
    d = H * hd
    qkv = torch.randn(B, T, 3 * d, generator=g).to(dtype)
    slopes = O.alibi_slopes(H)
    q, k, v = (t.reshape(B, T, H, hd) for t in torch.chunk(qkv, 3, dim=2))
    full = O.attention_core(q, k, v, W, slopes, 50.0).reshape(B, T, d)
    out = hip.swa_prefill(dev(qkv), dev(slopes), H, W, 50.0)
    check(out, full, dtype, frac=0.05)
    # ring: prefill P positions, then append/decode the rest one by one
    cap = W + 1
    P = T // 2
    kr = torch.zeros(B, H, cap, hd, dtype=dtype, device="cuda")
    vr = torch.zeros_like(kr)
    qd = dev(qkv)
    hip.kv_fill(qd[:, :P].contiguous(), kr, vr, 0)
    sd = dev(slopes)
    for pos in range(P, T):
        row = qd[:, pos].contiguous()
        hip.kv_append(row, kr, vr, pos)
        o = hip.swa_decode(row, kr, vr, sd, pos, W, 50.0)
        check(o, full[:, pos], dtype, frac=0.05, scale=float(full.abs().max()))
    # fused append + decode gives the same result as the two separate calls
    kr2, vr2 = torch.zeros_like(kr), torch.zeros_like(vr)
    hip.kv_fill(qd[:, :T - 1].contiguous(), kr2, vr2, 0)
    o3 = hip.swa_decode(qd[:, T - 1].contiguous(), kr2, vr2, sd, T - 1, W, 50.0, append=True)
    check(o3, full[:, T - 1], dtype, frac=0.05, scale=float(full.abs().max()))   # the own key is taken from the qkv row
    assert torch.equal(kr2, kr) and torch.equal(vr2, vr)
    # softcap disabled
    o2 = hip.swa_decode(qd[:, T - 1].contiguous(), kr, vr, sd, T - 1, W, 0.0)
    ref2 = O.attention_core(q[:, -1:], k, v, W, slopes, 0.0).reshape(B, d)
    check(o2, ref2, dtype, frac=0.05)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,hd,W,T", [(8, 16, 128, 1024, 1100), (2, 16, 128, 512, 560), (4, 12, 64, 512, 540)])
def test_swa_decode_long_window_past_the_ring_wrap(hip, dtype, B, H, hd, W, T):
    """The long-window instances of the decode kernel (8 waves per head; head dim 128 deals a 256-byte ring row to
    the 8 lanes of a key in 16-byte pieces) on a ring that has wrapped, against the oracle on the last queries
    only.  B=8, H=16, hd=128, W=1024 is config 5's attention shape at a quarter of its batch: one launch reads
    2*B*H*(W+1)*hd elements = 64 MB or more in either dtype, which selects the instance with streamed
    (non-temporal) ring loads.  The rings start out filled with NaN: no slot may be read before it is written."""
    g = gen(31)
    d = H * hd
    nq = 6
    qkv = torch.randn(B, T, 3 * d, generator=g).to(dtype)
    slopes = O.alibi_slopes(H)
    q, k, v = (t.reshape(B, T, H, hd) for t in torch.chunk(qkv, 3, dim=2))
    lo = T - nq - W - 1          # the oldest key any of the checked queries sees is at T - nq - W
    full = O.attention_core(q[:, T - nq:], k[:, lo:], v[:, lo:], W, slopes, 50.0).reshape(B, nq, d)
    cap = W + 1
    assert T - nq > cap          # the prompt alone wraps the ring
    if hd == 128 and W == 1024:
        assert 2 * B * H * cap * hd * qkv.element_size() >= 64 << 20
    kr = torch.full((B, H, cap, hd), float("nan"), dtype=dtype, device="cuda")
    vr = torch.full_like(kr, float("nan"))
    qd = dev(qkv)
    hip.kv_fill(qd[:, :T - nq].contiguous(), kr, vr, 0)
    sd = dev(slopes)
    scale = float(full.abs().max())
    for i, pos in enumerate(range(T - nq, T)):
        row = qd[:, pos].contiguous()
        if i % 2 == 0:           # fused append + decode and the two separate calls in turn
            o = hip.swa_decode(row, kr, vr, sd, pos, W, 50.0, append=True)
        else:
            hip.kv_append(row, kr, vr, pos)
            o = hip.swa_decode(row, kr, vr, sd, pos, W, 50.0)
        assert bool(torch.isfinite(o).all())
        check(o, full[:, i], dtype, frac=0.05, scale=scale)
    # the ring holds exactly the last cap positions, each in slot position % cap
    want = torch.empty(B, H, cap, hd, dtype=dtype)
    pos = torch.arange(T - cap, T)
    want[:, :, pos % cap] = k[:, T - cap:].transpose(1, 2)
    assert torch.equal(kr.cpu(), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,hd,W", [(2, 4, 64, 16), (1, 16, 128, 160), (8, 12, 64, 512)])
def test_swa_decode_never_reads_a_slot_before_it_is_written(hip, dtype, B, H, hd, W):
    """Rings are allocated uninitialised by the attention module.  A prompt shorter than the window leaves most
    slots unwritten; with those slots set to NaN every decode step up to and past the wrap must give the finite
    values of a zero-filled ring, bit for bit (a masked slot read with weight 0 would give 0 * NaN)."""
    g = gen(32)
    d = H * hd
    P, T = 5, W + 9
    qkv = dev(torch.randn(B, T, 3 * d, generator=g).to(dtype))
    sd = dev(O.alibi_slopes(H))
    rings = []
    for fill in (0.0, float("nan")):
        kr = torch.full((B, H, W + 1, hd), fill, dtype=dtype, device="cuda")
        vr = torch.full_like(kr, fill)
        hip.kv_fill(qkv[:, :P].contiguous(), kr, vr, 0)
        rings.append((kr, vr))
    for pos in range(P, T):
        row = qkv[:, pos].contiguous()
        o0 = hip.swa_decode(row, *rings[0], sd, pos, W, 50.0, append=True)
        o1 = hip.swa_decode(row, *rings[1], sd, pos, W, 50.0, append=True)
        assert bool(torch.isfinite(o1).all()), pos
        assert torch.equal(o0, o1), pos
    assert torch.equal(rings[0][0], rings[1][0]) and torch.equal(rings[0][1], rings[1][1])


@pytest.mark.parametrize("dtype", DTYPES)
def test_sample_greedy_matches_oracle_ties_included(hip, dtype):
    g = gen(11)
    B, V = 8, 50257
    logits = torch.randn(B, V, generator=g).to(dtype)
    logits[0, 100] = logits[0, 40000] = 9.0        # tie -> lowest index
    logits[1, :] = 0.0                               # all equal -> 0
    out = torch.full((B, 4), -1, dtype=torch.int64, device="cuda")
    hip.sample(dev(logits), out[:, 2], do_sample=False)
    ref = O.next_token(logits, do_sample=False)
    assert torch.equal(out[:, 2].cpu(), ref[:, 0])
    assert int(out[0, 2]) == 100 and int(out[1, 2]) == 0
    assert bool((out[:, [0, 1, 3]] == -1).all())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_head_with_fused_greedy_pick(hip, dtype, temperature):
    """logits as linear_decode; the pick equals the oracle's argmax of the filtered logits, ties to the lowest id."""
    g = gen(14)
    B, V, K = 8, 50257, 256
    x = torch.randn(B, K, generator=g).to(dtype)
    W = (torch.randn(V, K, generator=g) / 16).to(dtype)
    W[40000] = W[123]                      # exact tie between ids 123 and 40000 in every row
    x[0] = W[123].float().sign().to(dtype) * 3    # make that tied pair the maximum of row 0
    ws = torch.zeros(16 * 64, dtype=torch.int64, device="cuda")
    toks = torch.full((B, 3), -7, dtype=torch.int64, device="cuda")
    logits = hip.head_argmax(dev(x), dev(W), toks[:, 1], ws, temperature)
    ref_logits = F.linear(x.float(), W.float()).to(dtype)
    check(logits, ref_logits, dtype)
    ref = O.next_token(logits.cpu(), temperature=temperature, do_sample=False)[:, 0]
    assert torch.equal(toks[:, 1].cpu(), ref)
    assert int(toks[0, 1]) == 123
    assert bool((ws == 0).all()) and bool((toks[:, [0, 2]] == -7).all())


def _nucleus_fp32(logits_bf16, temperature, top_k, top_p):
    """The kernel's own top-p rule restated in numpy (fstu_sample): transformed logits rounded to bf16; survivors
    of top-k; fp32 exponentials relative to the row maximum, summed in float64; descending value order with ties by
    lower index; a token is kept iff the probability mass ranked before it is <= top_p.  Returns the filtered
    logits (fp32, -inf outside the nucleus) and the set of boundary tokens whose mass-before is within 1e-6 of top_p
    (their membership may depend on the last bit of an exponential)."""
    l = (logits_bf16.float() / temperature).to(torch.bfloat16).float().clamp(-1e4, 1e4).to(torch.bfloat16).float()
    B, V = l.shape
    out = torch.full_like(l, float("-inf"))
    slack = []
    for b in range(B):
        row = l[b].numpy()
        alive = np.ones(V, bool)
        if top_k:
            kth = np.sort(row)[::-1][top_k - 1]
            alive = row >= kth
        e = np.exp((row - row.max()).astype(np.float32)).astype(np.float64) * alive
        order = np.lexsort((np.arange(V), -row))            # value descending, index ascending inside ties
        order = order[alive[order]]
        before = (np.cumsum(e[order]) - e[order]) / e.sum()
        keep = before <= top_p
        kept = order[keep]
        out[b, kept] = torch.from_numpy(row[kept])
        slack.append(set(order[np.abs(before - top_p) < 1e-6].tolist()))
    return out, slack


@pytest.mark.parametrize("V", [3001, 50257])
@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, None, 0.7), (0.8, None, 0.9), (1.0, 40, 0.7), (1.3, 200, 0.9)])
def test_sample_top_p_bf16_nucleus(hip, V, temperature, top_k, top_p):
    """bf16 rows through the two-pass radix selects and the LDS logits cache of the sampler: every draw lies in the
    nucleus of the kernel's rule (fp32 exponentials, float64 sums over the bf16 transformed logits) and equals the
    oracle's inverse-CDF pick from the counter stream over that nucleus.  Row 0 carries a plateau of tied bf16 values
    that the boundary cuts through (tie ranks in index order)."""
    g = gen(31 + V)
    B = 4
    logits = (2.5 * torch.randn(B, V, generator=g)).to(torch.bfloat16)
    big = logits[0].float().topk(3)[0][-1]
    tied = torch.randperm(V, generator=g)[:300]
    logits[0, tied] = big.to(torch.bfloat16)                 # 300 tokens tied near the top of row 0
    ld = dev(logits)
    filt, slack = _nucleus_fp32(logits, temperature, top_k, top_p)
    sizes = torch.isfinite(filt).sum(-1)
    assert int(sizes.min()) >= 1 and int(sizes.max()) < V
    if not top_k:
        assert 3 < int(sizes[0]) < 303 + 40, int(sizes[0])   # the boundary lies inside the plateau of row 0
    agree = total = 0
    for step in range(40):
        out = torch.empty(B, dtype=torch.int64, device="cuda")
        hip.sample(ld, out, temperature, top_k, top_p, True, seed=91, step=step)
        got = out.cpu()
        ref = O.sample_from_logits(filt, 91, step)[:, 0]
        for b in range(B):
            inside = bool(torch.isfinite(filt[b, got[b]])) or int(got[b]) in slack[b]
            assert inside, f"row {b} step {step}: drew token {int(got[b])} outside the nucleus"
        agree += int((got == ref).sum())
        total += B
    assert agree >= total - 1, (agree, total)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("temperature,top_k,top_p", [(0.8, 40, None), (1.0, None, None), (1.0, 5, 0.7),
                                                      (1.3, None, 0.9), (0.7, 1, None)])
def test_sample_draws_match_oracle(hip, dtype, temperature, top_k, top_p):
    """Same counter-based stream, same filters: ids equal the oracle's draw.  With top-p in bf16 the reference takes
    softmax and cumsum in the model dtype while the kernel evaluates its nucleus in fp32/float64 (documented in the
    header): there the expected pick is the oracle's draw over the kernel's own nucleus rule (_nucleus_fp32)."""
    g = gen(12)
    B, V = 4, 3001
    logits = (2.5 * torch.randn(B, V, generator=g)).to(dtype)
    ld = dev(logits)
    own_rule = top_p is not None and dtype == torch.bfloat16
    if own_rule:
        filt = _nucleus_fp32(logits, temperature, top_k, top_p)[0]
    else:
        filt = O.filter_logits(logits.float() if dtype == torch.float32 else logits, temperature, top_k, top_p)
    agree = total = 0
    for step in range(40):
        out = torch.empty(B, dtype=torch.int64, device="cuda")
        hip.sample(ld, out, temperature, top_k, top_p, True, seed=77, step=step)
        ref = (O.sample_from_logits(filt, 77, step) if own_rule else
               O.next_token(logits, temperature, top_k, top_p, True, seed=77, step=step))[:, 0]
        agree += int((out.cpu() == ref).sum())
        total += B
        assert bool(torch.isfinite(filt.float().gather(1, out.cpu()[:, None])).all()), "drew a filtered token"
    assert agree >= total - 1, (agree, total)


SAMP_COUNTER_WORDS = (32 * 32 + 32 + 32 * 32) // 2     # tickets (a line per row), launch counter, per-chunk counts: 32-bit each


@pytest.mark.parametrize("V", [50257, 4096, 1031])
@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 40, None), (0.8, 40, None), (0.8, 1, None), (1.3, 64, None),
                                                     (0.8, 40, 0.9), (1.0, 7, 0.5)])
def test_sample_topk_spread_equals_one_workgroup_per_row_and_oracle(hip, V, temperature, top_k, top_p):
    """The sampler that spreads a row over the chip (head maxima -> candidates -> short-list draw) picks what
    fstu_sample picks on the same logits, and (without top-p, where the bf16 nucleus rule is the kernel's own) what the
    oracle's draw picks.  Rows start at odd element offsets (odd V); the maxima and the sampler's counters come back zeroed."""
    g = gen(41)
    B, K = 8, 256
    x = dev((torch.randn(B, K, generator=g)).bfloat16())
    W = dev((torch.randn(V, K, generator=g) * (3.0 / K ** 0.5)).bfloat16())
    best = torch.zeros(B * 64, dtype=torch.int64, device="cuda")
    ws = hip.sample_ws("cuda")
    agree = total = 0
    for step in range(12):
        logits = hip.head_maxima(x, W, best, temperature)
        assert int((best != 0).sum()) > 0
        out = torch.empty(B, dtype=torch.int64, device="cuda")
        hip.sample_topk(logits, best, ws, out, top_k, temperature, top_p, seed=5, step=step)
        ref = torch.empty(B, dtype=torch.int64, device="cuda")
        hip.sample(logits, ref, temperature, top_k, top_p, True, seed=5, step=step)
        assert torch.equal(out, ref), (step, out.tolist(), ref.tolist())
        assert int((best != 0).sum()) == 0 and int((ws[:SAMP_COUNTER_WORDS] != 0).sum()) == 0
        if top_p is None:
            o = O.next_token(logits.cpu(), temperature, top_k, None, True, seed=5, step=step)[:, 0]
            agree += int((out.cpu() == o).sum())
            total += B
    assert agree >= total - 1, (agree, total)


@pytest.mark.parametrize("rows,K,V,temperature", [(32, 2048, 50257, 0.8), (8, 768, 50257, 1.0), (19, 1024, 4099, 1.3),
                                                  (1, 256, 1031, 1.0), (16, 512, 6000, 0.7)])
def test_head_maxima_over_packed_embedding(hip, rows, K, V, temperature):
    """The head over a packed copy of the embedding (rows <= 32): logits within bf16 rounding of the float64 product;
    the packed maxima name, per row, the first index of the largest transformed logit and every slot holds an element
    of its row; fed to the spread sampler they give what fstu_sample draws from the same logits."""
    g = gen(43)
    x = dev(torch.randn(rows, K, generator=g).bfloat16())
    Wc = (torch.randn(V, K, generator=g) * (3.0 / K ** 0.5)).bfloat16()
    W = dev(Wc)
    wp = hip.pack_rows(W)
    best = torch.zeros(32 * 64, dtype=torch.int64, device="cuda")
    logits = hip.head_maxima_packed(x, wp, V, best, temperature)
    ref = x.double() @ W.double().t()
    assert float((logits.double() - ref).abs().max()) <= 2.0 ** -8 * float(ref.abs().max()) * 1.01
    t = logits.float()
    if temperature != 1.0:
        t = (t / temperature).bfloat16().float()
    t = t.clamp(-1e4, 1e4).bfloat16().float()
    b = best.view(32, 64)
    assert int((b[rows:] != 0).sum()) == 0
    idx_of = lambda w: 0xffffffff - (w & 0xffffffff)
    top = b[:rows].max(dim=1).values
    for r in range(rows):
        i = int(idx_of(top[r]))
        assert float(t[r, i]) == float(t[r].max()) and i == int((t[r] == t[r].max()).nonzero()[0])
        slots = b[r][b[r] != 0]
        ids = idx_of(slots)
        assert int(ids.max()) < V and len(set(ids.tolist())) == len(ids)
    if V >= 1024:
        ws = hip.sample_ws("cuda")
        out = torch.empty(rows, dtype=torch.int64, device="cuda")
        hip.sample_topk(logits, best, ws, out, 40, temperature, None, seed=11, step=3)
        want = torch.empty(rows, dtype=torch.int64, device="cuda")
        hip.sample(logits, want, temperature, 40, None, True, seed=11, step=3)
        assert torch.equal(out, want)
        assert int((best != 0).sum()) == 0


def test_sample_topk_spread_plateaus_and_errors(hip):
    """Long runs of equal logits overflow the per-chunk candidate lists: the row's last workgroup then draws from the
    whole row, with the same result as fstu_sample.  Arguments outside the fast path are refused."""
    g = gen(42)
    B, K, V = 5, 256, 6000
    x = dev(torch.randn(B, K, generator=g).bfloat16())
    Wc = (torch.randn(V, K, generator=g) * 0.2).bfloat16()
    Wc[1000:3000] = Wc[1000]          # 2000 tokens share one logit per row
    Wc[3500:3600] = Wc[3500]
    W = dev(Wc)
    best = torch.zeros(B * 64, dtype=torch.int64, device="cuda")
    ws = hip.sample_ws("cuda")
    for step, (top_k, temperature, top_p) in enumerate([(40, 1.0, None), (64, 0.7, None), (40, 0.9, 0.8), (3, 1.0, None)]):
        logits = hip.head_maxima(x, W, best, temperature)
        out = torch.empty(B, dtype=torch.int64, device="cuda")
        hip.sample_topk(logits, best, ws, out, top_k, temperature, top_p, seed=9, step=step)
        ref = torch.empty(B, dtype=torch.int64, device="cuda")
        hip.sample(logits, ref, temperature, top_k, top_p, True, seed=9, step=step)
        assert torch.equal(out, ref), (step, out.tolist(), ref.tolist())
        assert int((best != 0).sum()) == 0 and int((ws[:SAMP_COUNTER_WORDS] != 0).sum()) == 0
    # all logits equal: every token is a candidate everywhere
    xz = torch.zeros(B, K, dtype=torch.bfloat16, device="cuda")
    logits = hip.head_maxima(xz, W, best, 1.0)
    out = torch.empty(B, dtype=torch.int64, device="cuda")
    hip.sample_topk(logits, best, ws, out, 40, 1.0, None, seed=3, step=0)
    ref = torch.empty(B, dtype=torch.int64, device="cuda")
    hip.sample(logits, ref, 1.0, 40, None, True, seed=3, step=0)
    assert torch.equal(out, ref)
    for bad_k in (0, 65):
        with pytest.raises(hip.FlashSTUHipError, match="top_k"):
            hip.sample_topk(logits, best, ws, out, bad_k)
    with pytest.raises(hip.FlashSTUHipError, match="V="):
        hip.sample_topk(logits[:, :512].contiguous(), best, ws, out, 40)


@pytest.mark.parametrize("dtype", DTYPES)
def test_lds_steps_dense(hip, dtype):
    g = gen(13)
    T, Bt, din, S, dout = 12, 5, 96, 40, 72
    A = (0.9 + 0.099 * torch.rand(S, generator=g)).float()
    Bm = (torch.randn(din, S, generator=g) / din).to(dtype)
    Cm = (torch.randn(S, dout, generator=g) / S).to(dtype)
    x = torch.randn(T, Bt, din, generator=g).to(dtype)
    yref, href = O.lds_sequence(x, A, Bm, Cm)
    h = torch.zeros(Bt, S, device="cuda")
    y = hip.lds_steps(h, dev(x[:7]), dev(A), dev(Bm), dev(Cm))
    y2 = hip.lds_steps(h, dev(x[7:]), dev(A), dev(Bm), dev(Cm))     # state carried across launches
    check(torch.cat([y, y2]), yref, dtype, frac=0.05)
    assert float((h.cpu() - href).abs().max()) < 1e-5 * max(1.0, float(href.abs().max()))


@pytest.mark.parametrize("T,Bt,din,S,dout", [(300, 3, 96, 32, 48), (200, 2, 128, 64, 80), (130, 2, 64, 192, 64),
                                             (257, 1, 256, 256, 144), (129, 4, 160, 160, 16)])
def test_lds_sequence_on_the_matrix_cores(hip, T, Bt, din, S, dout):
    """The block-parallel form (bf16, S a multiple of 32: fstu_lds_sequence) at state sizes of every register variant,
    ragged block counts, d_in of an odd number of 32-wide k steps and output widths that are not whole groups of 64:
    against the oracle's literal loop, and bit-identical when the sequence is cut at a multiple of 128 positions."""
    g = gen(15)
    dtype = torch.bfloat16
    A = (0.9 + 0.099 * torch.rand(S, generator=g)).float()
    Bm = (torch.randn(din, S, generator=g) / din ** 0.5).to(dtype)
    Cm = (torch.randn(S, dout, generator=g) / S).to(dtype)
    x = torch.randn(T, Bt, din, generator=g).to(dtype)
    yref, href = O.lds_sequence(x, A, Bm, Cm)
    Ad, Bd, Cd, xd = dev(A), dev(Bm), dev(Cm), dev(x)
    h = torch.zeros(Bt, S, device="cuda")
    y = hip.lds_steps(h, xd, Ad, Bd, Cd, check_status=True)
    diff = (y.float().cpu() - yref.float()).abs()
    assert float(diff.max()) <= 2.0 ** -7 * float(yref.float().abs().max())
    assert float((diff > 0).float().mean()) < 0.05
    assert float((h.cpu() - href).abs().max()) <= 1e-4 * float(href.abs().max())
    h2 = torch.zeros(Bt, S, device="cuda")
    ya = hip.lds_steps(h2, xd[:128], Ad, Bd, Cd, check_status=True)
    yb = hip.lds_steps(h2, xd[128:], Ad, Bd, Cd, check_status=True)
    assert torch.equal(torch.cat([ya, yb]), y) and torch.equal(h2, h)


def test_argument_errors_do_not_launch(hip):
    x = torch.zeros(17, 64, dtype=torch.bfloat16, device="cuda")
    W = torch.zeros(32, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(hip.FlashSTUHipError, match="rows=17"):
        hip.linear_decode(x, W)
    with pytest.raises(hip.FlashSTUHipError):
        hip.linear_decode(torch.zeros(2, 64), W.cpu())
    kr = torch.zeros(1, 2, 4, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(hip.FlashSTUHipError, match="ring capacity"):
        hip.swa_decode(torch.zeros(1, 384, dtype=torch.bfloat16, device="cuda"), kr, kr.clone(),
                       torch.zeros(2, device="cuda"), 3, 8, 50.0)


@pytest.mark.parametrize("B,H,hd,W,T", [(2, 4, 64, 16, 50), (2, 12, 64, 512, 700), (1, 4, 128, 32, 100),
                                         (1, 2, 64, 1000, 333), (1, 2, 128, 64, 17)])
def test_swa_prefill_mfma(hip, B, H, hd, W, T):
    """Matrix-core prefill attention (bf16): against the oracle's explicit softmax and against the wave-per-query
    kernel; ragged T (not a multiple of the 16-query / 32-key tiles), window smaller and larger than T."""
    dtype = torch.bfloat16
    g = gen(40)
    d = H * hd
    qkv = torch.randn(B, T, 3 * d, generator=g).to(dtype)
    slopes = O.alibi_slopes(H)
    q, k, v = (t.reshape(B, T, H, hd) for t in torch.chunk(qkv, 3, dim=2))
    full = O.attention_core(q, k, v, W, slopes, 50.0).reshape(B, T, d)
    out = hip.swa_prefill(dev(qkv), dev(slopes), H, W, 50.0)
    check(out, full, dtype, frac=0.05)
    valu = hip.swa_prefill(dev(qkv), dev(slopes), H, W, 50.0, force_valu=True)
    check(out, valu, dtype, frac=0.05)
    out0 = hip.swa_prefill(dev(qkv), dev(slopes), H, W, 0.0)
    check(out0, O.attention_core(q, k, v, W, slopes, 0.0).reshape(B, T, d), dtype, frac=0.05)


def test_stu_step_lds_with_the_reference_lds_fixture(hip):
    """The reference's own distilled LDS (mini_stu/phi_lds.pt: 160 poles A, A[80:] = -A[:80], output map C (160,48),
    exact for L=8192) driven through the decode-step kernel: the 80 two-step poles A^2 and the merged output weights
    C[:80,:24] @ M_filters reproduce the spectral convolution with phi @ M_filters (stu.py:87-98,120), phi being the
    fixture's own impulse responses sum_j A_j^t C[j,k].  The fixture's output weights reach +-280 and cancel, which
    is why the reference runs this LDS in float64: the same recurrence evaluated on the CPU is exact to 1.5e-11 in
    float64 and off by 3.6e-3 of the output scale in float32, and the kernel (fp32 state) lands on the float32
    figure, just under one bf16 ulp.  The product's own fit (flash_stu/utils/lds_fit.py) keeps the weights small
    and stays at 5e-5 in fp32 (test_stu_step_lds_tracks_the_convolution)."""
    import os
    fx = torch.load(os.path.join(os.path.dirname(__file__), "golden", "phi_lds.pt"), weights_only=True)["model_state_dict"]
    A, C = fx["A"].double(), fx["C"].double()
    assert torch.equal(A[80:], -A[:80])
    K, S, B, d, T, L = 24, 80, 2, 64, 400, 8192
    g = gen(50)
    Mf = (torch.randn(K, d, generator=g, dtype=torch.float64) / math.sqrt(K))
    # filters from the fixture: phi[t,k] = sum_j A_j^t C[j,k] (k < 24, poles j < 80), built by repeated multiplication
    phi = torch.empty(L, K, dtype=torch.float64)
    pw = torch.ones(80, dtype=torch.float64)
    for t in range(L):
        phi[t] = pw @ C[:80, :K]
        pw = pw * A[:80]
    filt = (phi @ Mf).float()
    xp = torch.randn(B, T, d, generator=g)
    plus, minus = O.convolve(xp, filt, O.nearest_power_of_two(2 * L - 1, True), use_approx=True)
    ref = plus + minus
    a = (A[:80] ** 2).float()
    ce = (C[:80, :K] @ Mf).float().contiguous()
    state = torch.zeros(B, 2, S, d, device="cuda")
    ad, ced = dev(a), dev(ce)
    worst = 0.0
    for t in range(T):
        y = hip.stu_step_lds(state, dev(xp[:, t].contiguous()), ad, ced, t)
        worst = max(worst, float((y.cpu() - ref[:, t]).abs().max()))
    scale = float(ref.abs().max())
    print(f"fixture LDS through the step kernel: max error {worst:.3e} of scale {scale:.3e}")
    assert worst <= 2.0 ** -8 * scale * 1.5


@pytest.mark.parametrize("rows,d,I", [(8, 768, 9216), (1, 256, 512), (16, 512, 1000), (5, 1024, 4096), (8, 2048, 24576),
                                      (3, 768, 20), (32, 768, 9216), (17, 256, 512), (24, 2048, 8192), (32, 1024, 4096)])
def test_glu_packed_balanced(hip, rows, d, I):
    """Balanced packed gate/up GEMV == the row-major GLU kernel bit for bit is not required (other K split), but both
    must match the oracle within one bf16 ulp; ragged I (not a multiple of 16 or of the grid).  17..32 rows run as two
    row tiles per weight fragment and equal two launches of 16 rows bit for bit."""
    dtype = torch.bfloat16
    g = gen(60)
    x = torch.randn(rows, d, generator=g).to(dtype)
    wg = (torch.randn(I, d, generator=g) / math.sqrt(d)).to(dtype)
    wu = (torch.randn(I, d, generator=g) / math.sqrt(d)).to(dtype)
    # the specification with exact (float64) accumulation and the model's rounding points
    gate = (x.double() @ wg.double().t()).to(dtype)
    up = (x.double() @ wu.double().t()).to(dtype)
    ref = torch.nn.functional.gelu(gate.float(), approximate="tanh").to(dtype) * up
    out = hip.glu_packed(dev(x), hip.pack_rows(dev(wg)), hip.pack_rows(dev(wu)), I)
    # act is a product of two rounded factors: a flip of gate (one ulp, stretched by gelu' <= 1.13) and a flip of up
    # can coincide, so single elements may sit two ulps away; almost all are exact
    def close(a, b, frac):
        a, b = a.float().cpu(), b.float().cpu()
        diff = (a - b).abs()
        assert bool((diff <= b.abs() * 2.0 ** -6 + 1e-3 * 2.0 ** -7 * float(b.abs().max())).all())
        assert float((diff > 0).float().mean()) <= frac
    close(out, ref, 0.05)
    if rows <= 16:
        close(out, hip.glu_decode(dev(x), dev(wg), dev(wu)), 0.02)     # the row-major kernel, other K split
    else:
        pg, pu = hip.pack_rows(dev(wg)), hip.pack_rows(dev(wu))
        halves = torch.cat([hip.glu_packed(dev(x[:16]), pg, pu, I), hip.glu_packed(dev(x[16:]), pg, pu, I)])
        assert torch.equal(out, halves)


@pytest.mark.parametrize("rows,d,I", [(8, 768, 9216), (3, 256, 512), (16, 1024, 4096), (8, 2048, 8192),
                                      (16, 2048, 4096)])     # the last: more chunks than threads x 4, wave-per-row norm
def test_glu_packed_norm_prologue(hip, rows, d, I):
    """Residual add + RMSNorm as the prologue of the balanced gate/up launch == the separate add+norm kernel followed
    by the plain balanced launch (same arithmetic, bit for bit), and the sum is stored."""
    dtype = torch.bfloat16
    g = gen(61)
    x = torch.randn(rows, d, generator=g).to(dtype)
    delta = (0.5 * torch.randn(rows, d, generator=g)).to(dtype)
    nw = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype)
    wg = (torch.randn(I, d, generator=g) / math.sqrt(d)).to(dtype)
    wu = (torch.randn(I, d, generator=g) / math.sqrt(d)).to(dtype)
    pg, pu = hip.pack_rows(dev(wg)), hip.pack_rows(dev(wu))
    x_out, act = hip.glu_packed_norm(dev(x), dev(delta), dev(nw), O.RMS_EPS_DEFAULT, pg, pu, I)
    assert torch.equal(x_out.cpu(), x + delta)
    h_ref = O.rms_norm(x + delta, nw, O.RMS_EPS_DEFAULT)
    gate = (h_ref.double() @ wg.double().t()).to(dtype)
    up = (h_ref.double() @ wu.double().t()).to(dtype)
    ref = torch.nn.functional.gelu(gate.float(), approximate="tanh").to(dtype) * up
    diff = (act.float().cpu() - ref.float()).abs()
    assert bool((diff <= ref.float().abs() * 2.0 ** -6 + 2.0 ** -7 * 2e-2 * float(ref.float().abs().max())).all())
    assert float((diff > 0).float().mean()) <= 0.10
    x_out2, act2 = hip.glu_packed_norm(dev(x), None, dev(nw), O.RMS_EPS_DEFAULT, pg, pu, I)
    assert torch.equal(x_out2.cpu(), x)


@pytest.mark.parametrize("rows,d,I", [(32, 2048, 4096), (17, 2048, 1024), (24, 1024, 2048), (32, 768, 1536), (29, 256, 512)])
def test_glu_packed_norm_two_row_tiles(hip, rows, d, I):
    """17..32 rows: the RMSNorm of the (already summed) residual stream formed in the matrix-core fragments of the
    gate/up launch.  The activations meet the float64 reference like the 16-row prologue's, and the separate norm
    launch followed by the plain gate/up launch almost everywhere bit for bit (the row's sum of squares is gathered in
    another order, so a normalised value may round the other way now and then)."""
    dtype = torch.bfloat16
    g = gen(67)
    x = torch.randn(rows, d, generator=g).to(dtype)
    nw = (1 + 0.1 * torch.randn(d, generator=g)).to(dtype)
    wg = (torch.randn(I, d, generator=g) / math.sqrt(d)).to(dtype)
    wu = (torch.randn(I, d, generator=g) / math.sqrt(d)).to(dtype)
    pg, pu = hip.pack_rows(dev(wg)), hip.pack_rows(dev(wu))
    xd = dev(x)
    x_out, act = hip.glu_packed_norm(xd, None, dev(nw), O.RMS_EPS_DEFAULT, pg, pu, I)
    assert x_out is xd and torch.equal(xd.cpu(), x)
    h_ref = O.rms_norm(x, nw, O.RMS_EPS_DEFAULT)
    gate = (h_ref.double() @ wg.double().t()).to(dtype)
    up = (h_ref.double() @ wu.double().t()).to(dtype)
    ref = torch.nn.functional.gelu(gate.float(), approximate="tanh").to(dtype) * up
    diff = (act.float().cpu() - ref.float()).abs()
    assert bool((diff <= ref.float().abs() * 2.0 ** -6 + 2.0 ** -7 * 2e-2 * float(ref.float().abs().max())).all())
    assert float((diff > 0).float().mean()) <= 0.10
    h = hip.add_rmsnorm(xd.clone(), None, dev(nw), O.RMS_EPS_DEFAULT)
    two = hip.glu_packed(h, pg, pu, I)
    assert float((two != act).float().mean()) <= 0.01


@pytest.mark.parametrize("rows,d,ns", [(32, 2048, 16), (17, 768, 4), (5, 260, 3)])
def test_add_slices_equals_the_residual_update_of_add_rmsnorm(hip, rows, d, ns):
    g = gen(69)
    x = dev(torch.randn(rows, d, generator=g).bfloat16())
    sl = dev(0.3 * torch.randn(ns, rows, d, generator=g))
    want = x.clone()
    hip.add_rmsnorm(want, sl, None, 0.0, delta_mode=1, nslices=ns, want_norm=False)
    got = hip.add_slices(x.clone(), sl)
    assert torch.equal(got, want)
    ref = (x.double() + sl.double().sum(0).bfloat16().double()).bfloat16()
    assert float((got != ref).float().mean()) <= 0.01          # fp32 against float64 summation of the slices


@pytest.mark.parametrize("rows,K,N", [(32, 2048, 6144), (20, 1024, 1024), (17, 256, 768)])
def test_linear_packed_norm_two_row_tiles(hip, rows, K, N):
    """17..32 rows: y = rmsnorm(x) W^T with the norm formed in the launch's matrix-core fragments: almost everywhere
    the bits of the norm launch followed by the plain packed projection, and within the bf16 tolerance of float64."""
    dtype = torch.bfloat16
    g = gen(70)
    x = dev(torch.randn(rows, K, generator=g).to(dtype))
    nw = dev((1 + 0.1 * torch.randn(K, generator=g)).to(dtype))
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    wp = hip.pack_rows(dev(W))
    got = hip.linear_packed(x, wp, N, nw, O.RMS_EPS_DEFAULT)
    h = hip.add_rmsnorm(x.clone(), None, nw, O.RMS_EPS_DEFAULT)
    two = hip.linear_packed(h, wp, N)
    assert float((two != got).float().mean()) <= 0.01
    ref = (O.rms_norm(x.cpu(), nw.cpu(), O.RMS_EPS_DEFAULT).double() @ W.double().t()).to(dtype)
    check(got, ref, dtype, frac=0.05, atol=2.0 ** -7 * 2e-2 * float(ref.float().abs().max()))   # fp32 against float64 sums of K terms


@pytest.mark.parametrize("rows,K,N", [(32, 2048, 2048), (8, 768, 768), (19, 1024, 512), (32, 256, 64)])
def test_linear_packed_add_joins_the_residual_stream(hip, rows, K, N):
    """res_out = T(res + T(x W^T)) == the plain packed projection followed by a bf16 add, bit for bit; in place too."""
    dtype = torch.bfloat16
    g = gen(68)
    x = dev(torch.randn(rows, K, generator=g).to(dtype))
    res = dev(torch.randn(rows, N, generator=g).to(dtype))
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    wp = hip.pack_rows(dev(W))
    want = res + hip.linear_packed(x, wp, N)
    assert torch.equal(hip.linear_packed_add(x, wp, res), want)
    r2 = res.clone()
    assert hip.linear_packed_add(x, wp, r2, out=r2) is r2 and torch.equal(r2, want)
    ref = (res.double().cpu() + (x.double().cpu() @ W.double().t()).to(dtype).double()).to(dtype)
    check(want, ref, dtype)


@pytest.mark.parametrize("rows,K,N,ns", [(8, 768, 2304, 4), (4, 256, 96, 3), (2, 1024, 3072, 1)])
def test_linear_packed_res_equals_add_norm_then_linear(hip, rows, K, N, ns):
    dtype = torch.bfloat16
    g = gen(64)
    x = dev(torch.randn(rows, K, generator=g).to(dtype))
    part = dev(0.3 * torch.randn(ns, rows, K, generator=g))
    nw = dev((1 + 0.1 * torch.randn(K, generator=g)).to(dtype))
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    wp = hip.pack_rows(dev(W))
    x_ref = x.clone()
    h = hip.add_rmsnorm(x_ref, part, nw, O.RMS_EPS_DEFAULT, delta_mode=1, nslices=ns)
    y_ref = hip.linear_packed(h, wp, N)
    x_out, y = hip.linear_packed_res(x, part, nw, O.RMS_EPS_DEFAULT, wp, N)
    assert torch.equal(x_out, x_ref)
    check(y, y_ref, dtype, frac=0.05)
    # against the float64-accumulated specification
    xs = x.cpu() + part.cpu().sum(0).to(dtype)
    ref = (O.rms_norm(xs, nw.cpu(), O.RMS_EPS_DEFAULT).double() @ W.double().t()).to(dtype)
    check(y, ref, dtype, frac=0.05, atol=2.0 ** -8 * float(ref.float().abs().max()))


@pytest.mark.parametrize("rows,K,N", [(8, 768, 2304), (8, 768, 768), (4, 256, 96), (16, 1024, 3072)])
def test_linear_packed_with_and_without_norm(hip, rows, K, N):
    dtype = torch.bfloat16
    g = gen(63)
    x = torch.randn(rows, K, generator=g).to(dtype)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(dtype)
    W = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    wp = hip.pack_rows(dev(W))
    ref = (x.double() @ W.double().t()).to(dtype)
    check(hip.linear_packed(dev(x), wp, N), ref, dtype, frac=0.05)
    h = O.rms_norm(x, nw, O.RMS_EPS_DEFAULT)
    refn = (h.double() @ W.double().t()).to(dtype)
    check(hip.linear_packed(dev(x), wp, N, dev(nw), O.RMS_EPS_DEFAULT), refn, dtype, frac=0.10,
          atol=2.0 ** -7 * 0.05 * float(refn.float().abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
def test_stu_bank_step_lds(hip, dtype):
    """Exact-mode step on the recurrence state == a float64 evaluation of the same recurrence and output maps, and ==
    the oracle's exact-mode filter-bank convolution when ce/co are fitted to the filters."""
    from flash_stu.utils.lds_fit import fit_even_lag_lds
    g = gen(70)
    B, d, K, S, L, T = 2, 96, 6, 64, 128, 60
    phi = torch.tensor(O.get_spectral_filters_f64(L, K))
    a, ce, _ = fit_even_lag_lds(phi[0::2], S)
    a2, co, _ = fit_even_lag_lds(phi[1::2], S)
    assert torch.equal(a, a2)
    x = torch.randn(B, T, d, generator=g).to(dtype)
    rp, rm = O.convolve(x, phi.to(dtype), O.nearest_power_of_two(2 * L - 1, True), use_approx=False)   # (B,T,K,d)
    state = torch.zeros(B, 2, S, d, device="cuda")
    st64 = torch.zeros(B, 2, S, d, dtype=torch.float64)
    worst = 0.0
    for t in range(T):
        up, um = hip.stu_bank_step_lds(state, dev(x[:, t].contiguous()), dev(a), dev(ce), dev(co), t)
        p = t & 1
        st64[:, p] = st64[:, p] * a.double()[None, :, None] + x[:, t].double()[:, None, :]
        E = torch.einsum("jk,bjc->bkc", ce.double(), st64[:, p])
        Od = torch.einsum("jk,bjc->bkc", co.double(), st64[:, 1 - p])
        check(up, (E + Od).to(dtype), dtype, frac=0.05, scale=float(rp.float().abs().max()))
        check(um, (E - Od).to(dtype), dtype, frac=0.05, scale=float(rp.float().abs().max()))
        worst = max(worst, float((up.float().cpu() - rp[:, t].float()).abs().max()), float((um.float().cpu() - rm[:, t].float()).abs().max()))
    tol = 1e-3 if dtype == torch.float32 else 2.0 ** -7
    assert worst <= tol * float(rp.float().abs().max()), worst


def test_packed_kernels_refuse_rows_and_shapes_they_do_not_take(hip):
    """More than 32 rows, 17..32 rows with a norm prologue that would have to add a delta, and widths outside the packed
    kernels' set are refused on the host before any launch."""
    g = gen(66)
    d, I = 256, 512
    wg = dev((torch.randn(I, d, generator=g) / 16).bfloat16())
    pg = hip.pack_rows(wg)
    pd = hip.pack_rows(dev((torch.randn(d, I, generator=g) / 16).bfloat16()))
    nw = dev(torch.ones(d).bfloat16())
    x33 = dev(torch.randn(33, d, generator=g).bfloat16())
    x20 = dev(torch.randn(20, d, generator=g).bfloat16())
    best = torch.zeros(64 * 64, dtype=torch.int64, device="cuda")
    with pytest.raises(hip.FlashSTUHipError):
        hip.glu_packed(x33, pg, pg, I)
    with pytest.raises(hip.FlashSTUHipError):
        hip.down_packed_splitk(dev(torch.randn(33, I, generator=g).bfloat16()), pd, d, 16)
    with pytest.raises(hip.FlashSTUHipError):
        hip.linear_packed(x33, pg, I)
    with pytest.raises(hip.FlashSTUHipError):
        hip.glu_packed_norm(x20, x20, nw, 1e-6, pg, pg, I)  # 17..32 rows take the summed stream only: no delta
    with pytest.raises(hip.FlashSTUHipError):
        hip.glu_packed_norm(x33, None, nw, 1e-6, pg, pg, I)
    with pytest.raises(hip.FlashSTUHipError):
        hip.linear_packed_add(x33, pg, dev(torch.zeros(33, I).bfloat16()))
    with pytest.raises(hip.FlashSTUHipError):
        hip.head_maxima_packed(x33, pg, I, best)
    x320 = dev(torch.randn(20, 320, generator=g).bfloat16())    # K = 320 is not one of the packed kernels' widths
    w320 = hip.pack_rows(dev((torch.randn(I, 320, generator=g) / 16).bfloat16()))
    with pytest.raises(hip.FlashSTUHipError):
        hip.linear_packed(x320, w320, I)
    # and what they do take at 20 rows still runs
    assert hip.linear_packed(x20, pg, I).shape == (20, I)
    assert hip.glu_packed(x20, pg, pg, I).shape == (20, I)
    assert hip.glu_packed_norm(x20, None, nw, 1e-6, pg, pg, I)[1].shape == (20, I)
    assert hip.linear_packed(x20, pg, I, nw, 1e-6).shape == (20, I)


@pytest.mark.parametrize("rows,d,I,ks", [(8, 768, 9216, 16), (3, 256, 512, 4), (16, 1024, 4096, 8), (8, 2048, 24576, 16), (5, 48, 1024, 4), (8, 768, 9216, 4), (8, 768, 9216, 8),
                                         (32, 768, 9216, 16), (19, 1024, 4096, 8), (32, 2048, 24576, 16), (17, 48, 1024, 4)])
def test_down_packed_splitk(hip, rows, d, I, ks):
    """Balanced split-K down projection: the 4, 8 or 16 slices sum to the float64-accumulated product (17..32 rows: two
    row tiles per weight fragment, slice for slice equal to two launches of 16 rows)."""
    dtype = torch.bfloat16
    g = gen(64)
    act = torch.randn(rows, I, generator=g).to(dtype)
    wd = (torch.randn(d, I, generator=g) / math.sqrt(I)).to(dtype)
    ref = act.double() @ wd.double().t()
    part = hip.down_packed_splitk(dev(act), hip.pack_rows(dev(wd)), d, ks)
    assert part.shape[0] == ks
    got = part.double().sum(0).cpu()
    assert float((got - ref).abs().max()) <= 2e-5 * float(ref.abs().max())
    if rows > 16:
        wp = hip.pack_rows(dev(wd))
        halves = torch.cat([hip.down_packed_splitk(dev(act[:16]), wp, d, ks), hip.down_packed_splitk(dev(act[16:]), wp, d, ks)], 1)
        assert torch.equal(part, halves)


def test_kernels_against_committed_known_answers(hip):
    """The HIP kernels against tests/golden/kat_small.npz (first-principles float64 vectors, made by
    tests/golden/make_fixtures.py without any oracle code): both convolution forms, decode and prefill attention,
    the dense LDS loop and the top-k / top-p survivor sets of the sampler."""
    import os
    import numpy as np
    k = np.load(os.path.join(os.path.dirname(__file__), "golden", "kat_small.npz"))
    f32 = lambda a: torch.tensor(a, dtype=torch.float32)
    # convolution: time-domain and FFT form, both branches (mode: single branch = plus; sum = plus + minus)
    x, f = f32(k["conv_x"])[None], f32(k["conv_f"])
    plus, both = f32(k["conv_plus"]), f32(k["conv_plus"] + k["conv_minus"])
    assert float((hip.stu_conv_direct(dev(x), dev(f), single_branch=True)[0].cpu() - plus).abs().max()) < 2e-5
    assert float((hip.stu_conv_direct(dev(x), dev(f))[0].cpu() - both).abs().max()) < 4e-5
    n = hip.fft_length(12)
    assert float((hip.stu_conv_fft(dev(x), hip.stu_fft_filter(dev(f), n, single_branch=True), single_branch=True)[0].cpu()
                  - plus).abs().max()) < 2e-5
    assert float((hip.stu_conv_fft(dev(x), hip.stu_fft_filter(dev(f), n))[0].cpu() - both).abs().max()) < 4e-5
    # attention: prefill kernel and ring decode of the last position
    q, kk, v = (f32(k[n_]) for n_ in ("att_q", "att_k", "att_v"))          # (T,H,hd)
    T, H, hd = q.shape
    qkv = torch.cat([q.reshape(T, H * hd), kk.reshape(T, H * hd), v.reshape(T, H * hd)], dim=1)[None].contiguous()
    slopes = O.alibi_slopes(H)
    out = hip.swa_prefill(dev(qkv), dev(slopes), H, 3, 50.0)[0].cpu().reshape(T, H, hd)
    assert float((out - f32(k["att_out"])).abs().max()) < 5e-6
    kr = torch.zeros(1, H, 4, hd, device="cuda")
    vr = torch.zeros_like(kr)
    hip.kv_fill(dev(qkv[:, : T - 1].contiguous()), kr, vr, 0)
    o = hip.swa_decode(dev(qkv[:, T - 1].contiguous()), kr, vr, dev(slopes), T - 1, 3, 50.0, append=True)
    assert float((o.cpu().reshape(H, hd) - f32(k["att_out"])[T - 1]).abs().max()) < 5e-6
    # dense LDS loop
    h = torch.zeros(2, 5, device="cuda")
    y = hip.lds_steps(h, dev(f32(k["lds_x"])), dev(f32(k["lds_A"])), dev(f32(k["lds_B"])), dev(f32(k["lds_C"])))
    assert float((y.cpu() - f32(k["lds_y"])).abs().max()) < 5e-6
    # sampler survivor sets: with many seeds every draw must land inside the set, and every member gets drawn
    lg = f32(k["samp_logits"])
    for kw, keep in ((dict(top_k=3), k["samp_topk_keep"]), (dict(top_p=0.8), k["samp_topp_keep"])):
        seen = np.zeros_like(keep)
        for seed in range(300):
            out_ids = torch.zeros(2, dtype=torch.int64, device="cuda")
            hip.sample(dev(lg), out_ids, 1.0, kw.get("top_k"), kw.get("top_p"), True, seed, 0)
            for b, t in enumerate(out_ids.cpu().tolist()):
                assert keep[b, t], (kw, b, t)
                seen[b, t] = True
        assert np.array_equal(seen, keep)
