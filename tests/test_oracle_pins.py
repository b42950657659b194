"""Independent checks that pin the CPU oracle (oracle/flashstu_oracle.py).

None of these re-type the oracle's formulas: each compares against a closed
form, a library routine, brute force, or the reference's own data file
mini_stu/phi_lds.pt (committed as tests/golden/phi_lds.pt)."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import flashstu_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")


# ---------------- filters ----------------
def test_nearest_power_of_two_table():
    assert [O.nearest_power_of_two(x) for x in (1, 2, 3, 12, 16, 17)] == [1, 2, 2, 8, 16, 16]
    assert [O.nearest_power_of_two(x, True) for x in (1, 2, 3, 12, 16, 17, 2047, 4095, 16383)] == \
        [1, 2, 4, 16, 16, 32, 2048, 4096, 16384]


def test_hankel_closed_form_entries():
    Z = O.get_hankel(5)
    # Z[i,j] = 2/((i+j)^3-(i+j)) with 1-based i,j: Z[0,0] -> s=2 -> 2/6
    assert Z[0, 0] == pytest.approx(1 / 3)
    assert Z[0, 1] == pytest.approx(2 / 24)
    assert Z[4, 4] == pytest.approx(2 / 990)
    assert np.allclose(Z, Z.T)
    ZL = O.get_hankel(4, use_hankel_L=True)
    # s=2: sgn=2, 8/((5)(1)(3)) -> 16/15 ; odd s -> 0
    assert ZL[0, 0] == pytest.approx(16 / 15)
    assert ZL[0, 1] == 0.0


@pytest.mark.parametrize("L,K", [(16, 4), (64, 8), (256, 24)])
def test_filters_eigen_equation(L, K):
    phi = O.get_spectral_filters_f64(L, K)
    Z = O.get_hankel(L)
    G = phi.T @ phi                        # = diag(sigma^(1/2))
    sig = np.diag(G) ** 2
    assert np.allclose(G, np.diag(np.diag(G)), atol=1e-10)
    assert np.all(np.diff(sig) > 0)        # ascending order kept
    assert np.allclose(Z @ phi, phi * sig[None, :], atol=1e-9)
    top = np.linalg.eigvalsh(Z)[-K:]
    assert np.allclose(sig, top, rtol=1e-6, atol=1e-12)


def test_filters_against_reference_lds_fixture():
    """The reference ships an LDS whose impulse response reproduces its
    L=8192 filters: sum_j A_j^t C[j,k] = phi_k[t] (k<24) and (-1)^t phi_k[t]
    (k>=24), up to the eigenvector sign."""
    d = torch.load(os.path.join(GOLD, "phi_lds.pt"), weights_only=True)
    sd = d["model_state_dict"]
    A, C = sd["A"].double().numpy(), sd["C"].double().numpy()
    L = 8192
    phi = O.get_spectral_filters_f64(L, 24)
    t = np.arange(L)[:, None]
    imp = (A[None, :80] ** t) @ C[:80, :24]
    sgn = np.sign((imp * phi).sum(0))
    assert np.abs(imp * sgn - phi).max() < 5e-7
    imp_minus = (A[None, 80:] ** t) @ C[80:, 24:]
    assert np.abs(imp_minus * sgn - phi * ((-1.0) ** t)).max() < 5e-7


# ---------------- convolution ----------------
def test_convolve_matches_numpy_and_bruteforce():
    torch.manual_seed(0)
    B, T, d, L = 2, 37, 5, 64
    u = torch.randn(B, T, d)
    f = torch.randn(L, d)
    n = O.nearest_power_of_two(2 * L - 1, True)
    plus, minus = O.convolve(u, f, n, use_approx=True)
    ref = np.zeros((B, T, d))
    sg = (-1.0) ** np.arange(L)
    refm = np.zeros((B, T, d))
    for b in range(B):
        for c in range(d):
            ref[b, :, c] = np.convolve(u[b, :, c].double().numpy(), f[:, c].double().numpy())[:T]
            refm[b, :, c] = np.convolve(u[b, :, c].double().numpy(), (f[:, c].double().numpy() * sg))[:T]
    assert np.abs(plus.double().numpy() - ref).max() < 2e-5
    assert np.abs(minus.double().numpy() - refm).max() < 2e-5      # sgn*conv(sgn*u,f) = conv(u,(-1)^s f)
    assert np.abs(O.convolve_direct(u, f).numpy() - ref).max() < 1e-12


def test_convolve_delta_returns_filter_and_exact_mode():
    L, K, d = 32, 6, 3
    phi = torch.randn(L, K)
    n = 64
    u = torch.zeros(1, L, d)
    u[0, 0, :] = 1.0
    Up, Um = O.convolve(u, phi, n, use_approx=False)
    assert Up.shape == (1, L, K, d)
    assert torch.allclose(Up[0, :, :, 1], phi, atol=1e-5)
    sg = ((-1.0) ** torch.arange(L))[:, None]
    assert torch.allclose(Um[0, :, :, 2], phi * sg, atol=1e-5)
    # delayed delta: causal shift
    u2 = torch.zeros(1, L, d)
    u2[0, 5, 0] = 2.0
    Up2, _ = O.convolve(u2, phi, n, use_approx=False)
    assert torch.allclose(Up2[0, 5:, :, 0], 2 * phi[: L - 5], atol=1e-5)
    assert Up2[0, :5].abs().max() < 1e-5
    # single branch
    P, none = O.convolve(u, phi, n, use_approx=False, return_both=False)
    assert none is None and torch.allclose(P, Up, atol=1e-5)


def test_stu_forward_approx_is_even_lag_filter():
    """plus+minus = causal conv with 2*f on even lags, 0 on odd lags."""
    torch.manual_seed(1)
    B, T, d, L, K = 2, 48, 8, 64, 6
    phi = torch.tensor(O.get_spectral_filters_f64(L, K), dtype=torch.float32)
    p = {"M_inputs": torch.randn(d, d) / d ** 0.5, "M_filters": torch.randn(K, d) / K ** 0.5}
    x = torch.randn(B, T, d)
    y = O.stu_forward(x, phi, p, 128, use_approx=True)
    f = (phi @ p["M_filters"]).double()
    g = f.clone()
    g[1::2] = 0
    g[0::2] *= 2
    ref = O.convolve_direct(x @ p["M_inputs"], g)
    assert (y.double() - ref).abs().max() < 5e-5


def test_stu_forward_exact_is_einsum():
    torch.manual_seed(2)
    B, T, d, L, K = 2, 24, 6, 32, 5
    phi = torch.tensor(O.get_spectral_filters_f64(L, K), dtype=torch.float32)
    p = {"M_phi_plus": torch.randn(K, d, d) / d, "M_phi_minus": torch.randn(K, d, d) / d}
    x = torch.randn(B, T, d)
    y = O.stu_forward(x, phi, p, 64, use_approx=False)
    sg = ((-1.0) ** torch.arange(L))[:, None]
    ref = torch.zeros(B, T, d, dtype=torch.float64)
    for k in range(K):
        up = O.convolve_direct(x, phi[:, k:k + 1].expand(L, d))
        um = O.convolve_direct(x, (phi * sg)[:, k:k + 1].expand(L, d))
        ref += up @ p["M_phi_plus"][k].double() + um @ p["M_phi_minus"][k].double()
    assert (y.double() - ref).abs().max() < 5e-5


# ---------------- LDS ----------------
def test_lds_sequence_equals_impulse_response_convolution():
    torch.manual_seed(3)
    T, Bt, din, S, dout = 40, 3, 7, 11, 5
    A = torch.rand(S) * 0.9
    Bm, Cm = torch.randn(din, S), torch.randn(S, dout)
    x = torch.randn(T, Bt, din)
    y, h = O.lds_sequence(x, A, Bm, Cm)
    # y_t = sum_s x_{t-s} @ (B diag(A^s) C)
    ref = torch.zeros(T, Bt, dout, dtype=torch.float64)
    for s in range(T):
        G = (Bm.double() * (A.double() ** s)[None, :]) @ Cm.double()
        ref[s:] += x[: T - s].double() @ G
    assert (y.double() - ref).abs().max() < 1e-4


def test_distilled_lds_reproduces_reference_filters_on_a_signal():
    d = torch.load(os.path.join(GOLD, "phi_lds.pt"), weights_only=True)["model_state_dict"]
    A, Bv, C = d["A"], d["B"].reshape(-1), d["C"]
    T = 64
    u = torch.randn(2, T, dtype=torch.float64)
    out = O.lds_distilled_sequence(u, A, Bv, C)               # (2,T,48)
    t = torch.arange(T, dtype=torch.float64)[:, None]
    imp = (A[None, :] ** t) @ C                                 # (T,48)
    ref = torch.zeros(2, T, 48, dtype=torch.float64)
    for s in range(T):
        ref[:, s:] += u[:, : T - s, None] * imp[s]
    assert (out - ref).abs().max() < 1e-9


# ---------------- attention ----------------
def test_alibi_slopes_values():
    s4 = O.alibi_slopes(4)
    assert torch.allclose(s4, 0.25 * torch.tensor([2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8]))
    s12 = O.alibi_slopes(12)
    exp = [2.0 ** -(i + 1) for i in range(8)] + [2.0 ** -0.5, 2.0 ** -1.5, 2.0 ** -2.5, 2.0 ** -3.5]
    assert torch.allclose(s12, 0.25 * torch.tensor(exp))
    s16 = O.alibi_slopes(16)
    assert torch.allclose(s16, 0.25 * torch.tensor([2.0 ** (-(i + 1) / 2) for i in range(16)]))


def test_attention_softcap_off_equals_sdpa_with_bias_mask():
    torch.manual_seed(4)
    B, T, H, hd, W = 2, 19, 4, 8, 5
    q, k, v = (torch.randn(B, T, H, hd) for _ in range(3))
    slopes = O.alibi_slopes(H)
    out = O.attention_core(q, k, v, W, slopes, softcap=0.0)
    i = torch.arange(T)
    dist = i[:, None] - i[None, :]
    bias = -slopes.view(H, 1, 1) * dist.abs().float()
    bias = bias.masked_fill(((dist < 0) | (dist > W))[None], float("-inf"))
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                         attn_mask=bias[None]).transpose(1, 2)
    assert torch.allclose(out, ref, atol=2e-6)


def test_attention_softcap_single_key_and_wide_window():
    torch.manual_seed(5)
    B, T, H, hd = 1, 9, 2, 4
    q, k, v = (torch.randn(B, T, H, hd) for _ in range(3))
    slopes = torch.zeros(H)
    # window 0 -> every query sees only itself -> output = v
    assert torch.allclose(O.attention_core(q, k, v, 0, slopes, 50.0), v, atol=1e-6)
    # window >= T and tiny scores: tanh(x) ~ x, so softcap 1e6 == plain causal SDPA
    big = O.attention_core(q, k, v, 100, slopes, 1e6)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                         is_causal=True).transpose(1, 2)
    assert torch.allclose(big, ref, atol=1e-5)
    # softcap bounds the score: with q.k huge, all visible keys get score ~cap -> uniform average
    qh = torch.ones(1, 1, 1, 4) * 1e3
    kh = torch.ones(1, 3, 1, 4) * 1e3
    vh = torch.tensor([1.0, 2.0, 6.0]).view(1, 3, 1, 1).expand(1, 3, 1, 4)
    o = O.attention_core(qh, kh, vh, 10, torch.zeros(1), 50.0)
    assert torch.allclose(o, torch.full_like(o, 3.0), atol=1e-5)


def test_attention_decode_alignment_and_ring_equals_full():
    """A single query against a cache sits at the END of the keys; dropping
    keys older than window changes nothing."""
    torch.manual_seed(6)
    B, T, H, hd, W = 2, 30, 4, 8, 7
    q, k, v = (torch.randn(B, T, H, hd) for _ in range(3))
    slopes = O.alibi_slopes(H)
    full = O.attention_core(q, k, v, W, slopes, 50.0)
    for t in (0, 5, 29):
        one = O.attention_core(q[:, t:t + 1], k[:, : t + 1], v[:, : t + 1], W, slopes, 50.0)
        assert torch.allclose(one, full[:, t:t + 1], atol=1e-6)
        lo = max(0, t - W)
        ring = O.attention_core(q[:, t:t + 1], k[:, lo: t + 1], v[:, lo: t + 1], W, slopes, 50.0)
        assert torch.allclose(ring, full[:, t:t + 1], atol=1e-6)


# ---------------- norm / mlp ----------------
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_rms_norm_is_torch_rms_norm(dt):
    torch.manual_seed(7)
    x = torch.randn(3, 5, 96).to(dt)
    w = (1 + 0.3 * torch.randn(96)).to(dt)
    ref = F.rms_norm(x, (96,), w, O.RMS_EPS_DEFAULT)
    assert torch.equal(O.rms_norm(x, w), ref) if dt == torch.bfloat16 else torch.allclose(O.rms_norm(x, w), ref, atol=1e-6)
    m = torch.nn.RMSNorm(96, dtype=dt)
    m.weight.data.copy_(w)
    assert torch.allclose(m(x).float(), O.rms_norm(x, w).float(), atol=1e-6)


def test_mlp_is_gelu_tanh_glu():
    torch.manual_seed(8)
    x = torch.randn(4, 16)
    p = {"gate_proj.weight": torch.randn(32, 16), "up_proj.weight": torch.randn(32, 16),
         "down_proj.weight": torch.randn(16, 32)}
    g = x @ p["gate_proj.weight"].T
    gelu = 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3)))
    ref = (gelu * (x @ p["up_proj.weight"].T)) @ p["down_proj.weight"].T
    assert torch.allclose(O.mlp_forward(x, p), ref, atol=1e-4)


# ---------------- sampling ----------------
def _filter_bruteforce(row, temperature, top_k, top_p):
    l = [min(max(x / temperature, -1e4), 1e4) for x in row]
    V = len(l)
    if top_k is not None:
        kth = sorted(l, reverse=True)[top_k - 1]
        l = [x if x >= kth else -math.inf for x in l]
    if top_p is not None:
        order = sorted(range(V), key=lambda i: -l[i])
        m = max(l)
        e = [math.exp(l[i] - m) if l[i] > -math.inf else 0.0 for i in order]
        Z = sum(e)
        cum, acc = [], 0.0
        for x in e:
            acc += x / Z
            cum.append(acc)
        rem = [c > top_p for c in cum]
        rem = [False] + rem[:-1]
        for r, i in zip(rem, order):
            if r:
                l[i] = -math.inf
    return l


@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, None, None), (0.7, 3, None), (1.3, None, 0.6),
                                                      (0.9, 5, 0.8), (1.0, 1, None)])
def test_filter_logits_bruteforce(temperature, top_k, top_p):
    g = torch.Generator().manual_seed(9)
    logits = torch.randn(6, 11, generator=g, dtype=torch.float64) * 3
    got = O.filter_logits(logits, temperature, top_k, top_p)
    for b in range(6):
        exp = _filter_bruteforce(logits[b].tolist(), temperature, top_k, top_p)
        for a, e in zip(got[b].tolist(), exp):
            assert (a == e) or abs(a - e) < 1e-9


def test_topk_keeps_ties_and_argmax_lowest_index():
    l = torch.tensor([[1.0, 5.0, 5.0, 3.0, 5.0, 0.0]])
    f = O.filter_logits(l, 1.0, top_k=2)
    assert torch.isinf(f[0, [0, 3, 5]]).all() and (f[0, [1, 2, 4]] == 5).all()
    assert O.next_token(l, do_sample=False).item() == 1
    assert O.filter_logits(torch.tensor([[2e4, -3e4]]), 1.0).tolist() == [[1e4, -1e4]]


def test_counter_sampler_distribution_and_determinism():
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]])
    p = torch.softmax(logits.double(), -1)[0]
    N = 4000
    counts = torch.zeros(5)
    for s in range(N):
        counts[O.next_token(logits, do_sample=True, seed=123, step=s).item()] += 1
    chi2 = float((((counts - N * p) ** 2) / (N * p)).sum())
    assert chi2 < 18.5                      # chi-square, 4 dof, p ~ 1e-3
    a = O.next_token(logits, do_sample=True, seed=5, step=7)
    assert torch.equal(a, O.next_token(logits, do_sample=True, seed=5, step=7))
    us = [O.counter_uniform(1, s, 0) for s in range(2000)]
    assert 0.0 <= min(us) and max(us) < 1.0 and abs(sum(us) / 2000 - 0.5) < 0.03
    # filtered tokens are never drawn
    fl = O.filter_logits(logits, 1.0, top_k=2)
    assert all(O.sample_from_logits(fl, 3, s).item() in (1, 2) for s in range(200))


# ---------------- whole model ----------------
def _tiny_cfg(dtype=torch.float32, **kw):
    base = dict(n_embd=32, n_heads=4, n_layers=4, seq_len=64, window_size=6, vocab_size=101,
                mlp_scale=2, num_eigh=6, dtype=dtype)
    base.update(kw)
    return O.OracleConfig(**base)


@pytest.mark.parametrize("use_approx", [True, False])
def test_generate_stateful_equals_recompute_fp32(use_approx):
    cfg = _tiny_cfg(use_approx=use_approx)
    w = O.init_weights(cfg, seed=0, mode="healthy")
    ids = torch.randint(0, cfg.vocab_size, (2, 9), generator=torch.Generator().manual_seed(1))
    a, la = O.generate(w, cfg, ids, max_length=30, do_sample=False, mode="recompute", return_logits=True)
    b, lb = O.generate(w, cfg, ids, max_length=30, do_sample=False, mode="stateful", return_logits=True)
    assert torch.equal(a, b)
    assert (la - lb).abs().max() < 1e-4
    assert a.shape == (2, 30) and torch.equal(a[:, :9], ids)


def test_forward_cache_layout_and_causality():
    cfg = _tiny_cfg()
    w = O.init_weights(cfg, seed=3, mode="healthy")
    ids = torch.randint(0, cfg.vocab_size, (2, 12), generator=torch.Generator().manual_seed(2))
    logits, cache = O.model_forward(w, cfg, ids, use_cache=True)
    assert logits.shape == (2, 12, cfg.vocab_size)
    assert cache[0] is None and cache[2] is None
    assert cache[1][0].shape == (2, 12, 4, 8)
    # causal: logits at position 6 do not depend on later tokens
    l2, _ = O.model_forward(w, cfg, ids[:, :7])
    assert (l2[:, -1] - logits[:, 6]).abs().max() < 1e-4


def test_reference_init_cumulative_std():
    cfg = _tiny_cfg(n_embd=64, vocab_size=4000, n_layers=4)
    w = O.init_weights(cfg, seed=0, mode="reference")
    exp = O.expected_reference_stds(cfg)
    assert exp["tok_emb"] == pytest.approx(64 ** -0.5 * (8 ** -0.5) ** 2)
    assert float(w["tok_emb.weight"].float().std()) == pytest.approx(exp["tok_emb"], rel=0.05)
    assert float(w["layers.0.mlp.gate_proj.weight"].float().std()) == pytest.approx(64 ** -0.5, rel=0.05)
    assert float(w["layers.3.mlp.down_proj.weight"].float().std()) == pytest.approx(exp["layers.3.mlp"], rel=0.05)
    # xavier for STU / attention projections
    assert float(w["layers.1.attn.c_attn.weight"].float().std()) == pytest.approx(math.sqrt(2 / (64 + 192)), rel=0.05)
    assert w["tok_emb.weight"] is w["lm_head.weight"]


def test_decode_step_bytes_matches_worked_example():
    cfg = O.OracleConfig(n_embd=768, n_heads=12, n_layers=12, seq_len=2048, window_size=512, vocab_size=50257,
                         mlp_scale=12)
    b = O.decode_step_bytes(cfg, 8, 2048, state_dim=160)
    assert abs(b / 1e6 - 749.8) < 3.0


# ----------------------------------------------------------------- committed known-answer vectors
def _kat():
    return np.load(os.path.join(GOLD, "kat_small.npz"))


def test_kat_filters_convolution_attention_lds_sampling():
    """The oracle against tests/golden/kat_small.npz (first-principles float64 loops, tests/golden/make_fixtures.py)."""
    k = _kat()
    for name, L, K in (("phi_L8_K3", 8, 3), ("phi_L64_K6", 64, 6)):
        phi = np.asarray(O.get_spectral_filters_f64(L, K))
        ref = k[name]
        for c in range(K):                                    # eigenvector sign is a convention
            err = min(np.abs(phi[:, c] - ref[:, c]).max(), np.abs(phi[:, c] + ref[:, c]).max())
            assert err < 1e-9
    x = torch.tensor(k["conv_x"], dtype=torch.float32)[None]
    f = torch.tensor(k["conv_f"], dtype=torch.float32)
    plus, minus = O.convolve(x, f, O.nearest_power_of_two(2 * 12 - 1, True), use_approx=True)
    assert np.abs(plus[0].numpy() - k["conv_plus"]).max() < 2e-5
    assert np.abs(minus[0].numpy() - k["conv_minus"]).max() < 2e-5
    q, kk, v = (torch.tensor(k[n], dtype=torch.float32)[None] for n in ("att_q", "att_k", "att_v"))
    out = O.attention_core(q, kk, v, 3, O.alibi_slopes(4), 50.0)
    assert np.abs(out[0].numpy() - k["att_out"]).max() < 2e-6
    y, _ = O.lds_sequence(torch.tensor(k["lds_x"], dtype=torch.float32), torch.tensor(k["lds_A"], dtype=torch.float32),
                          torch.tensor(k["lds_B"], dtype=torch.float32), torch.tensor(k["lds_C"], dtype=torch.float32))
    assert np.abs(y.numpy() - k["lds_y"]).max() < 2e-6
    lg = torch.tensor(k["samp_logits"], dtype=torch.float32)
    assert np.array_equal(torch.isfinite(O.filter_logits(lg, top_k=3)).numpy(), k["samp_topk_keep"])
    assert np.array_equal(torch.isfinite(O.filter_logits(lg, top_p=0.8)).numpy(), k["samp_topp_keep"])
