"""CPU-only checks of the host side: the C-ABI library loads and exports every
symbol the header declares, configuration / filters / distillation helpers
behave as the reference's, and the product refuses to run without the GPU
path instead of falling back."""
import os
import re
import ctypes

import numpy as np
import pytest
import torch

from oracle import flashstu_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from flash_stu import _hip
    header = open(os.path.join(ROOT, "include", "flashstu_hip.h")).read()
    declared = set(re.findall(r"^\s*(?:int|const char\*|int64_t|size_t)\s+(fstu_\w+)\s*\(", header, flags=re.M))
    assert {"fstu_version", "fstu_last_error", "fstu_decode_step", "fstu_swa_decode", "fstu_stu_step_lds"} <= declared
    lib = ctypes.CDLL(_hip.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    # every entry point must have its argument types declared: an undeclared pointer argument would be
    # truncated to a 32-bit int by ctypes
    bound = set(_hip.SIGNATURES) | {"fstu_version", "fstu_last_error"}
    assert declared == bound, declared ^ bound
    assert _hip.load().fstu_version() == 100


def test_argument_validation_happens_on_the_host():
    """Null pointers and bad shapes are rejected before any launch, so this runs without a GPU."""
    from flash_stu import _hip
    lib = _hip.load()
    assert lib.fstu_linear_decode(None, 8, None, None, 8, 1, 8, 8, 1, None) == -1
    assert b"null" in lib.fstu_last_error()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.fstu_linear_decode(p, 8, p, p, 8, 17, 8, 8, 1, None) == -3
    assert b"rows=17" in lib.fstu_last_error()
    assert lib.fstu_add_rmsnorm(p, None, 0, 1, 0, None, None, 1, 8, 1e-6, 1, None) == -5
    assert lib.fstu_swa_decode(p, p, p, p, p, 1, 2, 48, 9, 0, 8, 50.0, 1, None) == -3      # head dim 48
    assert lib.fstu_sample(p, p, 1, 1, 10, 0.0, 0, 0.0, 0, 0, 0, 1, None) == -5             # temperature 0
    assert lib.fstu_embed(p, p, p, 1, 8, 4, 7, None) == -2                                   # unknown dtype


def test_config_surface_matches_reference_defaults(tmp_path):
    from flash_stu import FlashSTUConfig
    c = FlashSTUConfig()
    assert (c.n_embd, c.n_heads, c.n_layers, c.seq_len, c.window_size, c.vocab_size, c.mlp_scale) == \
        (1536, 8, 26, 8192, 1024, 200064, 12)
    assert c.use_approx and c.use_attn and c.use_cache and c.softcap == 50.0 and c.torch_dtype == torch.bfloat16
    assert c.hidden_size == 1536 and c.intermediate_size == 1536 * 12 and c.hidden_act == "swish"
    assert FlashSTUConfig(torch_dtype="float32").torch_dtype == torch.float32
    assert FlashSTUConfig(torch_dtype=None).torch_dtype == torch.float32
    d = c.to_dict()
    assert d["torch_dtype"] == "bfloat16" and d["model_type"] == "FlashSTU"
    c2 = FlashSTUConfig(n_embd=64, window_size=(32, 0), torch_dtype=torch.float32, my_extra=5)
    c2.save_pretrained(str(tmp_path))
    c3 = FlashSTUConfig.from_pretrained(str(tmp_path))
    assert c3.n_embd == 64 and c3.window_size == (32, 0) and c3.torch_dtype == torch.float32 and c3.my_extra == 5
    assert c3.window_left == 32
    assert FlashSTUConfig(torch_dtype=torch.bfloat16).resolved_stu_decode_mode() == "lds"
    assert FlashSTUConfig(torch_dtype=torch.float32).resolved_stu_decode_mode() == "history"
    with pytest.raises(ValueError):
        FlashSTUConfig(stu_decode_mode="fft")


def test_product_filters_equal_oracle_filters():
    from flash_stu import get_spectral_filters
    from flash_stu.utils.stu_utils import get_hankel, load_spectral_filters, save_spectral_filters
    from flash_stu.utils.numerics import nearest_power_of_two
    for hl in (False, True):
        assert np.array_equal(get_hankel(16, hl), O.get_hankel(16, hl))
    a = get_spectral_filters(64, 8, device="cpu", dtype=torch.float32)
    assert torch.equal(a, O.get_spectral_filters(64, 8, dtype=torch.float32))
    assert [nearest_power_of_two(x, True) for x in (3, 2047, 4096)] == [4, 2048, 4096]


def test_filter_files_roundtrip(tmp_path):
    from flash_stu import get_spectral_filters
    from flash_stu.utils.stu_utils import save_spectral_filters
    phi = get_spectral_filters(32, 4, device="cpu", dtype=torch.float32)
    path = str(tmp_path / "f" / "phi.pt")
    save_spectral_filters(phi, path)
    back = get_spectral_filters(32, 4, device="cpu", dtype=torch.float32, load_from=path)
    assert torch.equal(back, phi)
    with pytest.raises(ValueError):
        get_spectral_filters(32, 5, device="cpu", load_from=path)


@pytest.mark.parametrize("L", [128, 1024])
def test_lds_distillation_reproduces_even_lag_filter(L):
    """float64 recurrence with the fitted poles/weights == direct convolution
    with 2*f on even lags, far below one bf16 ulp (2^-8)."""
    from flash_stu.utils.lds_fit import fit_even_lag_lds
    K = 8 if L < 256 else 24
    phi = O.get_spectral_filters_f64(L, K)
    g = torch.Generator().manual_seed(0)
    Mf = torch.randn(K, 16, generator=g, dtype=torch.float64) / K ** 0.5
    f = torch.tensor(phi) @ Mf
    a, ce, err = fit_even_lag_lds(f[0::2], 64)
    assert err < 2e-4 * float(f.abs().max())
    x = torch.randn(1, L, 16, generator=g, dtype=torch.float64)
    geff = f.clone()
    geff[1::2] = 0
    geff[0::2] *= 2
    ref = O.convolve_direct(x, geff)[0]
    h = torch.zeros(2, 64, 16, dtype=torch.float64)
    worst = 0.0
    for t in range(L):
        p = t & 1
        h[p] = a.double()[:, None] * h[p] + x[0, t][None, :]
        y = 2 * (ce.double() * h[p]).sum(0)
        worst = max(worst, float((y - ref[t]).abs().max()))
    assert worst < 5e-4 * float(ref.abs().max())


def test_model_builds_on_cpu_but_refuses_to_compute_there():
    from flash_stu import FlashSTU, FlashSTUConfig
    from flash_stu._hip import FlashSTUHipError
    cfg = FlashSTUConfig(n_embd=64, n_heads=1, n_layers=2, seq_len=32, window_size=4, vocab_size=50, mlp_scale=2,
                         num_eigh=4, torch_dtype=torch.float32)
    m = FlashSTU(cfg)
    names = set(m.state_dict().keys())
    assert {"phi", "tok_emb.weight", "lm_head.weight", "norm.weight", "layers.0.stu_norm.weight",
            "layers.0.stu.M_inputs", "layers.0.stu.M_filters", "layers.0.mlp_norm.weight",
            "layers.0.mlp.gate_proj.weight", "layers.0.mlp.up_proj.weight", "layers.0.mlp.down_proj.weight",
            "layers.1.attn_norm.weight", "layers.1.attn.c_attn.weight", "layers.1.attn.c_proj.weight"} <= names
    assert m.tok_emb.weight is m.lm_head.weight
    assert m.get_num_params() == sum(p.numel() for p in m.parameters())
    with pytest.raises(FlashSTUHipError):
        m(torch.zeros(1, 4, dtype=torch.int64))
    with pytest.raises(FlashSTUHipError):
        m.generate(torch.zeros(1, 4, dtype=torch.int64), max_length=8)
    # cumulative-std quirk of the reference's init: the tied embedding is drawn last
    exp = 64 ** -0.5 * (4 ** -0.5)
    assert float(m.tok_emb.weight.std()) == pytest.approx(exp, rel=0.15)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "flash-stu-2_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.replace("load_named_tensors", ""), f"{f} mentions the oracle"


@pytest.mark.parametrize("L,K", [(128, 8), (2048, 24), (8192, 24)])
def test_lds_fit_reproduces_hankel_filters_and_rejects_what_it_cannot_fit(L, K):
    """The recurrence that replaces the STU filter in bf16 decode must reproduce it: fit error of the even- and the
    odd-lag halves below one bf16 step of the filters' largest taps, for random and for structured (all-ones,
    single-filter) M_filters; a filter that is no sum of decaying exponentials is refused."""
    from flash_stu.utils.lds_fit import check_lds_fit, fit_even_lag_lds
    phi = torch.tensor(O.get_spectral_filters_f64(L, K)).to(torch.bfloat16)
    g = torch.Generator().manual_seed(L)
    d = 16
    cases = {"random": torch.randn(K, d, generator=g) / K ** 0.5, "ones": torch.ones(K, d) / K,
             "one filter": torch.eye(K)[:, :d] if K >= d else torch.eye(K).repeat(1, 2)[:, :d]}
    for name, Mf in cases.items():
        f = torch.matmul(phi, Mf.to(torch.bfloat16))
        refused = False
        for half in (f[0::2], f[1::2]):
            a, c, err = fit_even_lag_lds(half, 64, per_channel=True)
            assert a.shape == (64,) and c.shape == (64, d) and err.shape == (d,)
            try:
                check_lds_fit(err, f[0::2])
            except ValueError as e:
                assert "history" in str(e)
                refused = True
        # mixtures led by the large eigenvectors fit; the 16 smallest, oscillating eigenvectors on channels of their
        # own ("one filter": the first columns of phi) do not once the filters are long
        assert refused == (name == "one filter" and L >= 2048), (name, L, refused)
    noise = torch.randn(L // 2, d, generator=g)
    _, _, err = fit_even_lag_lds(noise, 64, per_channel=True)
    with pytest.raises(ValueError, match="history"):
        check_lds_fit(err, noise)


def test_lds_exact_head_closes_the_fit_on_the_first_lags():
    """STU.lds_fir(): the taps added to the fitted recurrence make the first R lags of the decode filter equal to
    phi_proj itself (to fp32), for R below and above the filter length; off for Hankel-L, history mode and R = 0."""
    from flash_stu import FlashSTUConfig
    from flash_stu.modules.stu import STU
    for L, R in ((256, 32), (64, 128)):
        cfg = FlashSTUConfig(n_embd=16, n_heads=2, n_layers=2, seq_len=L, num_eigh=8, vocab_size=11,
                             torch_dtype=torch.bfloat16, stu_decode_mode="lds", stu_lds_fir_taps=R)
        phi = torch.tensor(O.get_spectral_filters_f64(L, 8)).to(torch.bfloat16)
        torch.manual_seed(L)
        stu = STU(cfg, phi, L)
        with torch.no_grad():
            stu.M_filters.copy_(torch.randn_like(stu.M_filters) / 8 ** 0.5)
        fir = stu.lds_fir()
        a, ce, co = stu.lds_params()
        assert fir.shape == (R, 16) and fir.dtype == torch.float32
        f = stu.effective_filter().detach().double()
        want = torch.zeros(R, 16, dtype=torch.float64)
        want[: min(R, L)] = f[: min(R, L)]
        m = torch.arange(R // 2, dtype=torch.float64)
        V = a.double()[None, :] ** m[:, None]
        got = fir.double()
        got[0::2] += V @ ce.double()
        got[1::2] += V @ co.double()
        assert float((got - want).abs().max()) <= 1e-6 * float(f.abs().max())
        for off in (dict(stu_lds_fir_taps=0), dict(use_hankel_L=True), dict(stu_decode_mode="history")):
            kw = dict(n_embd=16, n_heads=2, n_layers=2, seq_len=L, num_eigh=8, vocab_size=11, torch_dtype=torch.bfloat16,
                      stu_decode_mode="lds", stu_lds_fir_taps=R)
            kw.update(off)
            assert STU(FlashSTUConfig(**kw), phi, L).lds_fir() is None
    with pytest.raises(ValueError):
        FlashSTUConfig(n_embd=16, n_heads=2, n_layers=2, seq_len=64, num_eigh=8, vocab_size=11, stu_lds_fir_taps=48)


def test_generate_beyond_seq_len_leaves_the_stateful_paths():
    """prompt + new tokens > seq_len: the decode engine refuses (its state has no counterpart in the reference's
    truncated re-run, model.py:250-255) and FlashSTU.generate takes the recompute loop instead of the engine."""
    from flash_stu import FlashSTU, FlashSTUConfig
    from flash_stu.engine import DecodeEngine
    cfg = FlashSTUConfig(n_embd=64, n_heads=2, n_layers=2, seq_len=32, window_size=8, vocab_size=50, num_eigh=4,
                         torch_dtype=torch.bfloat16)
    model = FlashSTU(cfg)
    eng = DecodeEngine(model)
    with pytest.raises(Exception, match="seq_len|GPU"):
        eng.generate(torch.zeros(1, 30, dtype=torch.int64), 8)
    import inspect
    src = inspect.getsource(FlashSTU.generate)
    assert "max_length <= self.config.seq_len and DecodeEngine.supports" in src


def test_lm_head_follows_config_bias():
    """model.py:100-102: lm_head is built with bias=config.bias, so a bias=True checkpoint carries lm_head.bias."""
    from flash_stu import FlashSTU, FlashSTUConfig
    kw = dict(n_embd=64, n_heads=2, n_layers=2, seq_len=32, window_size=8, vocab_size=50, num_eigh=4)
    assert FlashSTU(FlashSTUConfig(bias=False, **kw)).lm_head.bias is None
    m = FlashSTU(FlashSTUConfig(bias=True, **kw))
    assert m.lm_head.bias is not None and "lm_head.bias" in m.state_dict()
    assert float(m.lm_head.bias.abs().max()) == 0.0
