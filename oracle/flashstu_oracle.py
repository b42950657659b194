"""CPU oracle for Flash STU's autoregressive token loop.

TEST INFRASTRUCTURE ONLY.  This module is the checker the HIP path is compared
against; nothing in the product package imports it.  Only tests, the smoke
entry and the benchmark's CPU-baseline leg may call it.

It restates, in plain PyTorch on whatever device the inputs live on (CPU in
the tests), the arithmetic of the reference files listed below, including the
points where the reference rounds to the model dtype.  Every function cites
the reference lines it follows (paths relative to the reference checkout).

Two deliberate departures from the reference text, both needed to make the
reference's own loop runnable:
  * `convolve` slices the cached sign vector to the input length
    (flash_stu/modules/stu.py:30-33 caches it at seq_len and
    flash_stu/utils/stu_utils.py:223 then fails to broadcast for T != seq_len;
    the un-cached branch at stu_utils.py:204-206 builds it from the input
    length, which is what is restated here).
  * attention is an explicit-softmax statement of the flash-attn call at
    flash_stu/modules/attention.py:90-99 (the reference has no other attention
    implementation): scale -> tanh soft-cap -> ALiBi bias -> causal band mask
    -> fp32 softmax -> P @ V.

Pinning status (which independent check fixes each function; see tests/):
  get_hankel / get_spectral_filters : closed form, eigen-equation, and the
      reference's data file mini_stu/phi_lds.pt (golden fixture)      PINNED
  convolve / stu_forward            : O(T^2) brute force, numpy.convolve,
      delta input, minus-branch identity                              PINNED
  lds_step / lds_distilled_step     : equality with convolution by the
      impulse response, literal loop                                  PINNED
  attention_core                    : SDPA special cases (softcap off),
      single key, window >= t, ring == full history                   PINNED up
      to flash-attn's internal rounding of P, which no reference test fixes:
      "parity unpinned" for that rounding point only
  rms_norm / mlp_forward            : torch.nn.functional.rms_norm / gelu PINNED
  filter_logits / greedy            : brute force on tiny vocabularies  PINNED
  sample_from_logits (do_sample)    : own counter-based stream; agrees with
      torch.multinomial only in distribution (chi-square test).  The
      reference's ids from the global torch generator: parity unpinned.
  init_weights                      : distribution and order restated;
      seeded bit-identity with the reference: parity unpinned.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

RMS_EPS_DEFAULT = 1.1920929e-07  # what torch.nn.RMSNorm(eps=None) resolves to


# --------------------------------------------------------------------------
# configuration (flash_stu/config.py:71-132)
# --------------------------------------------------------------------------
@dataclass
class OracleConfig:
    n_embd: int = 1536
    n_heads: int = 8
    n_layers: int = 26
    seq_len: int = 8192
    window_size: int = 1024
    vocab_size: int = 200064
    mlp_scale: int = 12
    num_eigh: int = 24
    use_hankel_L: bool = False
    use_approx: bool = True
    use_attn: bool = True
    softcap: float = 50.0
    dtype: torch.dtype = torch.bfloat16
    rms_eps: float = RMS_EPS_DEFAULT

    @property
    def intermediate_size(self) -> int:  # config.py:109
        return self.n_embd * self.mlp_scale

    @property
    def n_fft(self) -> int:  # model.py:56
        return nearest_power_of_two(self.seq_len * 2 - 1, round_up=True)

    def is_attention_layer(self, idx: int) -> bool:  # model.py:77-87
        return (idx % 2 == 1) and self.use_attn


# --------------------------------------------------------------------------
# filters (flash_stu/utils/numerics.py:3-6, stu_utils.py:18-31,146-193)
# --------------------------------------------------------------------------
def nearest_power_of_two(x: int, round_up: bool = False) -> int:
    """numerics.py:3-6."""
    return 1 << (math.ceil(math.log2(x)) if round_up else math.floor(math.log2(x)))


def get_hankel(seq_len: int, use_hankel_L: bool = False) -> np.ndarray:
    """stu_utils.py:18-31.  Z[i,j] for i,j = 1..L (float64)."""
    e = np.arange(1, seq_len + 1, dtype=np.float64)
    s = e[:, None] + e[None, :]
    if use_hankel_L:
        sgn = (-1.0) ** (s - 2.0) + 1.0
        return sgn * (8.0 / ((s + 3.0) * (s - 1.0) * (s + 1.0)))
    return 2.0 / (s ** 3 - s)


def get_spectral_filters_f64(seq_len: int, K: int, use_hankel_L: bool = False) -> np.ndarray:
    """stu_utils.py:188-192 before the cast: top-K eigenpairs (ascending),
    eigenvectors scaled by sigma**0.25.  Returns (L, K) float64."""
    Z = get_hankel(seq_len, use_hankel_L)
    sigma, phi = np.linalg.eigh(Z)
    sigma, phi = sigma[-K:], phi[:, -K:]
    return phi * sigma ** 0.25


def get_spectral_filters(seq_len: int, K: int, use_hankel_L: bool = False,
                         dtype: torch.dtype = torch.bfloat16, device="cpu") -> torch.Tensor:
    """stu_utils.py:146-193 (without the CUDA assertion at :185)."""
    return torch.tensor(get_spectral_filters_f64(seq_len, K, use_hankel_L), device=device, dtype=dtype)


# --------------------------------------------------------------------------
# convolution (stu_utils.py:195-246)
# --------------------------------------------------------------------------
def _sgn(T: int, device) -> torch.Tensor:
    s = torch.ones(1, T, 1, device=device, dtype=torch.int64)
    s[:, 1::2] *= -1
    return s


def convolve(u: torch.Tensor, v: torch.Tensor, n: int, use_approx: bool = True,
             return_both: bool = True, v_fft: Optional[torch.Tensor] = None
             ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """stu_utils.py:195-246.  u (B,T,d); v is the (L,d) per-channel filter in
    approx mode or the (L,K) filter bank otherwise.  fp32 FFT of length n,
    result truncated to T and cast back to u's dtype.  The filter is cut to
    its first n taps by rfft exactly as torch does (n >= L always holds)."""
    B, T, d_in = u.shape
    dt = u.dtype
    sgn = _sgn(T, u.device)
    if use_approx:
        if v_fft is None:
            v_fft = torch.fft.rfft(v.reshape(1, -1, v.shape[1], 1).to(torch.float32), n=n, dim=1)
        elif v_fft.dim() == 3:
            v_fft = v_fft.unsqueeze(-1)
    else:
        K = v.shape[1]
        if v_fft is None:
            v_fft = torch.fft.rfft(v.reshape(1, -1, K, 1, 1).to(torch.float32), n=n, dim=1)
        elif v_fft.dim() == 4:
            v_fft = v_fft.unsqueeze(-1)
        u = u.reshape(B, T, 1, d_in).expand(B, T, K, d_in)
        sgn = sgn.unsqueeze(-1)
    if return_both:
        U = torch.stack([u, u * sgn], dim=-1).to(torch.float32)
        U = torch.fft.rfft(U, n=n, dim=1)
        Uc = torch.fft.irfft(v_fft * U, n=n, dim=1)[:, :T]
        plus, minus = torch.unbind(Uc, dim=-1)
        minus = minus * sgn
        return plus.to(dt), minus.to(dt)
    if not use_approx:
        v_fft = v_fft.squeeze(-1)
    else:
        v_fft = v_fft.squeeze(-1)
    U = torch.fft.rfft(u.to(torch.float32), n=n, dim=1)
    plus = torch.fft.irfft(v_fft * U, n=n, dim=1)[:, :T]
    return plus.to(dt), None


def convolve_direct(u: torch.Tensor, f: torch.Tensor) -> torch.Tensor:
    """O(T^2) time-domain statement of one causal branch (float64):
    y[b,t,c] = sum_{s<=t} f[s,c] u[b,t-s,c].  Used to pin `convolve`."""
    B, T, d = u.shape
    u64, f64 = u.double(), f.double()
    y = torch.zeros(B, T, d, dtype=torch.float64, device=u.device)
    for s in range(min(T, f.shape[0])):
        y[:, s:] += f64[s] * u64[:, : T - s]
    return y


# --------------------------------------------------------------------------
# STU module (flash_stu/modules/stu.py:81-120)
# --------------------------------------------------------------------------
def stu_forward(x: torch.Tensor, phi: torch.Tensor, p: Dict[str, torch.Tensor], n: int,
                use_approx: bool = True, use_hankel_L: bool = False) -> torch.Tensor:
    """stu.py:81-120 (_forward_standard, torch.fft path).  `p` holds
    M_inputs/M_filters (approx) or M_phi_plus[/M_phi_minus] (exact); phi is
    already in the model dtype (model.py:61-68), so phi_fft in exact mode is
    the FFT of the rounded filters (stu.py:43-53)."""
    both = not use_hankel_L
    if use_approx:
        x_proj = x @ p["M_inputs"]                      # stu.py:87
        phi_proj = phi @ p["M_filters"]                 # stu.py:88
        plus, minus = convolve(x_proj, phi_proj, n, True, both)
    else:
        Up, Um = convolve(x, phi, n, False, both)
        plus = torch.tensordot(Up, p["M_phi_plus"], dims=([2, 3], [0, 1]))   # stu.py:112-114
        minus = torch.tensordot(Um, p["M_phi_minus"], dims=([2, 3], [0, 1])) if both else None
    return plus if use_hankel_L else plus + minus


# --------------------------------------------------------------------------
# LDS forms (mini_stu/lds.py:79-103, mini_stu/stu_lds.py:213-338,379-411)
# --------------------------------------------------------------------------
def lds_step(h: torch.Tensor, x_t: torch.Tensor, A: torch.Tensor, Bm: torch.Tensor,
             Cm: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """One iteration of the loop at mini_stu/lds.py:95-101 with the state in
    fp32: h (Bt,S) <- h*A + x_t (Bt,d_in) @ B (d_in,S); y = h @ C (S,d_out).
    B, C and x may be bf16; products accumulate in fp32; y is returned in
    x_t's dtype."""
    h = h.float() * A.float() + x_t.float() @ Bm.float()
    y = h @ Cm.float()
    return h, y.to(x_t.dtype)


def lds_sequence(x: torch.Tensor, A, Bm, Cm, h0: Optional[torch.Tensor] = None
                 ) -> Tuple[torch.Tensor, torch.Tensor]:
    """mini_stu/lds.py:79-103 over x (T,Bt,d_in) -> y (T,Bt,d_out), final h."""
    T, Bt, _ = x.shape
    h = torch.zeros(Bt, A.shape[0], dtype=torch.float32, device=x.device) if h0 is None else h0.float()
    ys = []
    for t in range(T):
        h, y = lds_step(h, x[t], A, Bm, Cm)
        ys.append(y)
    return torch.stack(ys), h


def lds_distilled_sequence(u: torch.Tensor, A: torch.Tensor, Bv: torch.Tensor, C: torch.Tensor,
                           h0: Optional[torch.Tensor] = None) -> torch.Tensor:
    """mini_stu/stu_lds.py:213-338 (FixedDiagonalLDS), sequential statement:
    per scalar stream u (N,T): h <- A*h + Bv*u_t ; y_t = h @ C, using the
    *updated* state (stu_lds.py:218-219).  float64 throughout."""
    N, T = u.shape
    D = A.shape[0]
    h = torch.zeros(N, D, dtype=torch.float64) if h0 is None else h0.double().expand(N, D).clone()
    out = torch.empty(N, T, C.shape[1], dtype=torch.float64)
    A, Bv, C, u = A.double(), Bv.double(), C.double(), u.double()
    for t in range(T):
        h = A * h + Bv * u[:, t:t + 1]
        out[:, t] = h @ C
    return out


# --------------------------------------------------------------------------
# attention (flash_stu/modules/attention.py:38-105)
# --------------------------------------------------------------------------
def alibi_slopes(n_heads: int, interpolation_factor: float = 0.25) -> torch.Tensor:
    """attention.py:38-57 (fp32)."""
    def gen(n):
        start = 2 ** (-(2 ** -(math.log2(n) - 3)))
        return [start * (start ** i) for i in range(n)]
    if math.log2(n_heads).is_integer():
        s = gen(n_heads)
    else:
        n = nearest_power_of_two(n_heads, round_up=False)
        s = gen(n) + gen(2 * n)[0::2][: n_heads - n]
    return torch.tensor(s, dtype=torch.float32) * interpolation_factor


def attention_core(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int,
                   slopes: torch.Tensor, softcap: float) -> torch.Tensor:
    """The flash-attn call at attention.py:90-99 restated: q (B,Tq,H,hd),
    k,v (B,Tk,H,hd) with the queries aligned to the END of the keys (causal,
    bottom-right).  Query i sits at absolute position p = i + Tk - Tq; key j is
    visible iff p - window <= j <= p.  score = softcap*tanh(q.k*hd^-0.5/softcap)
    - slope_h*(p-j); softmax and P@V in fp32; output in q's dtype."""
    B, Tq, H, hd = q.shape
    Tk = k.shape[1]
    qf, kf, vf = q.float(), k.float(), v.float()
    s = torch.einsum("bqhd,bkhd->bhqk", qf, kf) * (hd ** -0.5)
    if softcap and softcap > 0:
        s = softcap * torch.tanh(s / softcap)
    pos_q = torch.arange(Tq, device=q.device) + (Tk - Tq)
    pos_k = torch.arange(Tk, device=q.device)
    dist = (pos_q[:, None] - pos_k[None, :])                         # (Tq,Tk)
    s = s - slopes.to(q.device).view(1, H, 1, 1) * dist.abs().float()
    visible = (dist >= 0) & (dist <= window)
    s = s.masked_fill(~visible, float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("bhqk,bkhd->bqhd", p, vf)
    return o.to(q.dtype)


def attention_forward(x: torch.Tensor, p: Dict[str, torch.Tensor], n_heads: int, window: int,
                      softcap: float, past: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
                      ) -> Tuple[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """attention.py:59-105: fused QKV linear, split q,k,v, concatenate the
    cache along time, attention, output projection.  Returns (y, (k, v))."""
    B, T, d = x.shape
    qkv = F.linear(x, p["c_attn.weight"])
    q, k, v = torch.chunk(qkv, 3, dim=2)
    hd = d // n_heads
    q, k, v = (t.reshape(B, T, n_heads, hd) for t in (q, k, v))
    if past is not None:
        k = torch.cat([past[0], k], dim=1)
        v = torch.cat([past[1], v], dim=1)
    y = attention_core(q, k, v, window, alibi_slopes(n_heads), softcap)
    y = F.linear(y.reshape(B, T, d), p["c_proj.weight"])
    return y, (k, v)


# --------------------------------------------------------------------------
# norm / MLP / layers
# --------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float = RMS_EPS_DEFAULT) -> torch.Tensor:
    """torch.nn.RMSNorm fallback at stu_layer.py:32-36,81: fp32 statistics,
    one rounding to the input dtype after the weight multiply."""
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return ((xf * r) * w.float()).to(x.dtype)


def mlp_forward(x: torch.Tensor, p: Dict[str, torch.Tensor]) -> torch.Tensor:
    """swiglu.py:22-29: down(gelu_tanh(gate(x)) * up(x)), each op rounding to
    the model dtype."""
    gate = F.gelu(F.linear(x, p["gate_proj.weight"]), approximate="tanh")
    gate = gate * F.linear(x, p["up_proj.weight"])
    return F.linear(gate, p["down_proj.weight"])


def _sub(w: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    n = len(prefix)
    return {k[n:]: v for k, v in w.items() if k.startswith(prefix)}


def stu_layer_forward(x, w, cfg: OracleConfig, phi) -> torch.Tensor:
    """stu_layer.py:78-97 (no sandwich): x += stu(norm(x)); x += mlp(norm(x))."""
    h = rms_norm(x, w["stu_norm.weight"], cfg.rms_eps)
    h = stu_forward(h, phi, _sub(w, "stu."), cfg.n_fft, cfg.use_approx, cfg.use_hankel_L)
    x = x + h
    return x + mlp_forward(rms_norm(x, w["mlp_norm.weight"], cfg.rms_eps), _sub(w, "mlp."))


def attention_layer_forward(x, w, cfg: OracleConfig, past=None):
    """attention_layer.py:50-66."""
    a = rms_norm(x, w["attn_norm.weight"], cfg.rms_eps)
    y, present = attention_forward(a, _sub(w, "attn."), cfg.n_heads, cfg.window_size, cfg.softcap, past)
    x = x + y
    x = x + mlp_forward(rms_norm(x, w["mlp_norm.weight"], cfg.rms_eps), _sub(w, "mlp."))
    return x, present


# --------------------------------------------------------------------------
# model forward (flash_stu/model.py:108-205)
# --------------------------------------------------------------------------
def model_forward(w: Dict[str, torch.Tensor], cfg: OracleConfig, input_ids: torch.Tensor,
                  past_key_values=None, use_cache: bool = False, last_only: bool = False):
    """model.py:152-176.  Returns (logits, cache-tuple|None).  `w` uses the
    reference's state-dict names.  With last_only the head is applied to the
    final position only (same values as logits[:, -1:])."""
    x = w["tok_emb.weight"][input_ids]
    phi = w["phi"]
    cache = []
    for i in range(cfg.n_layers):
        lw = _sub(w, f"layers.{i}.")
        if cfg.is_attention_layer(i):
            past = past_key_values[i] if past_key_values is not None else None
            x, present = attention_layer_forward(x, lw, cfg, past)
            cache.append(present)
        else:
            x = stu_layer_forward(x, lw, cfg, phi)
            cache.append(None)
    x = rms_norm(x, w["norm.weight"], cfg.rms_eps)
    if last_only:
        x = x[:, -1:]
    logits = F.linear(x, w["tok_emb.weight"])
    return logits, (tuple(cache) if use_cache else None)


# --------------------------------------------------------------------------
# sampling (flash_stu/model.py:267-299)
# --------------------------------------------------------------------------
def filter_logits(logits: torch.Tensor, temperature: float = 1.0, top_k: Optional[int] = None,
                  top_p: Optional[float] = None) -> torch.Tensor:
    """model.py:268-289 on (B,V) last-position logits, in the logits' dtype."""
    l = logits / temperature
    l = torch.clamp(l, min=-1e4, max=1e4)
    if top_k is not None:
        kth = torch.topk(l, top_k)[0][..., -1, None]
        l = l.masked_fill(l < kth, float("-inf"))
    if top_p is not None:
        sl, si = torch.sort(l, descending=True)
        cum = torch.cumsum(F.softmax(sl, dim=-1), dim=-1)
        rem = cum > top_p
        rem[..., 1:] = rem[..., :-1].clone()
        rem[..., 0] = False
        l = l.masked_fill(rem.scatter(1, si, rem), float("-inf"))
    return l


_M64 = (1 << 64) - 1


def counter_uniform(seed: int, step: int, row: int) -> float:
    """Counter-based uniform in [0,1) with 24 random bits: a splitmix64
    finaliser over (seed, step, row).  The device sampler evaluates the same
    integer function, so draws are reproducible without a generator state.
    (Stands in for the global-generator torch.multinomial at model.py:297.)"""
    z = (seed * 0x9E3779B97F4A7C15 + step * 0xBF58476D1CE4E5B9 + row * 0x94D049BB133111EB + 0x2545F4914F6CDD1D) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    z = z ^ (z >> 31)
    return (z >> 40) / float(1 << 24)


def sample_from_logits(l: torch.Tensor, seed: int, step: int) -> torch.Tensor:
    """Inverse-CDF draw over softmax(l) per row, tokens walked in index order:
    the first index whose running probability sum exceeds u * total.
    fp32 exponentials relative to the row maximum, float64 running sum."""
    B, V = l.shape
    out = torch.empty(B, 1, dtype=torch.int64)
    lf = l.float().cpu()
    for b in range(B):
        row = lf[b]
        m = row.max()
        e = torch.exp(row - m).double()
        e[torch.isinf(row) & (row < 0)] = 0.0
        c = torch.cumsum(e, 0)
        u = counter_uniform(seed, step, b) * float(c[-1])
        idx = int(torch.searchsorted(c, torch.tensor(u, dtype=torch.float64), right=True))
        idx = min(idx, V - 1)
        while e[idx] == 0.0 and idx > 0:   # never land on a filtered token
            idx -= 1
        out[b, 0] = idx
    return out.to(l.device)


def next_token(logits_last: torch.Tensor, temperature=1.0, top_k=None, top_p=None,
               do_sample=True, seed: int = 0, step: int = 0) -> torch.Tensor:
    """model.py:267-299 -> (B,1) int64."""
    l = filter_logits(logits_last, temperature, top_k, top_p)
    if do_sample:
        return sample_from_logits(l, seed, step)
    return torch.argmax(l, dim=-1, keepdim=True)


# --------------------------------------------------------------------------
# generate (flash_stu/model.py:207-304)
# --------------------------------------------------------------------------
@torch.no_grad()
def generate(w, cfg: OracleConfig, input_ids: torch.Tensor, max_length: int = 100,
             temperature: float = 1.0, top_k=None, top_p=None, do_sample: bool = True,
             mode: str = "recompute", seed: int = 0, return_logits: bool = False):
    """model.py:245-302.  mode="recompute" is the reference's use_cache=False
    branch (:251-257): the whole sequence, cut to the last seq_len tokens, is
    re-run every step; it is the ground truth for an STU model because the
    reference's STU layers carry no decode state (stu_layer.py:99-120).
    mode="stateful" feeds one token per step against a bounded state (see
    DecodeState) and must produce the same tokens."""
    gen = input_ids
    all_logits = []
    state = None
    for step in range(max_length - input_ids.shape[1]):
        if mode == "recompute":
            seq = gen[:, -cfg.seq_len:] if gen.shape[1] > cfg.seq_len else gen
            logits, _ = model_forward(w, cfg, seq, last_only=True)
        else:
            if state is None:
                state = DecodeState(w, cfg, gen.shape[0])
                logits = state.prefill(gen)
            else:
                logits = state.step(gen[:, -1])
        last = logits[:, -1, :]
        if return_logits:
            all_logits.append(last.clone())
        nxt = next_token(last, temperature, top_k, top_p, do_sample, seed, step)
        gen = torch.cat([gen, nxt], dim=-1)
    return (gen, torch.stack(all_logits, 1)) if return_logits else gen


# --------------------------------------------------------------------------
# bounded-state decode: what the device path implements
# --------------------------------------------------------------------------
def stu_effective_filter(phi: torch.Tensor, M_filters: torch.Tensor) -> torch.Tensor:
    """phi_proj of stu.py:88, in the model dtype: (L,d)."""
    return phi @ M_filters


class DecodeState:
    """One-token-per-step evaluation with bounded state, equal (up to fp32
    summation order) to re-running the whole sequence:
      * attention layers keep the last window+1 keys/values in a ring
        (only those are visible through the band mask of attention.py:96);
      * STU layers (approx mode) keep the x_proj history and evaluate the
        causal convolution at the newest position directly, both sign
        branches rounded separately as stu_utils.py:227-228 does.
    """

    def __init__(self, w, cfg: OracleConfig, batch: int):
        self.w, self.cfg, self.B = w, cfg, batch
        self.t = 0
        self.kv: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
        self.hist: Dict[int, torch.Tensor] = {}
        self.filt: Dict[int, torch.Tensor] = {}
        for i in range(cfg.n_layers):
            if not cfg.is_attention_layer(i) and cfg.use_approx:
                self.filt[i] = stu_effective_filter(w["phi"], w[f"layers.{i}.stu.M_filters"]).float()

    def prefill(self, ids: torch.Tensor) -> torch.Tensor:
        w, cfg = self.w, self.cfg
        x = w["tok_emb.weight"][ids]
        T = ids.shape[1]
        for i in range(cfg.n_layers):
            lw = _sub(w, f"layers.{i}.")
            if cfg.is_attention_layer(i):
                x, (k, v) = attention_layer_forward(x, lw, cfg, None)
                keep = cfg.window_size + 1
                self.kv[i] = (k[:, -keep:].clone(), v[:, -keep:].clone())
            else:
                h = rms_norm(x, lw["stu_norm.weight"], cfg.rms_eps)
                if cfg.use_approx:
                    self.hist[i] = (h @ lw["stu.M_inputs"]).clone()
                else:
                    self.hist[i] = h.clone()
                x = stu_layer_forward(x, lw, cfg, w["phi"])
        self.t = T
        x = rms_norm(x, w["norm.weight"], cfg.rms_eps)[:, -1:]
        return F.linear(x, w["tok_emb.weight"])

    def _stu_step(self, i: int, h: torch.Tensor, lw) -> torch.Tensor:
        cfg, dt = self.cfg, h.dtype
        if cfg.use_approx:
            xp = h @ lw["stu.M_inputs"]                                   # (B,1,d)
            self.hist[i] = torch.cat([self.hist[i], xp], dim=1)
            H = self.hist[i].float()                                      # (B,t+1,d)
            t1 = H.shape[1]
            f = self.filt[i][:t1]                                         # (t+1,d)
            Hr = torch.flip(H, dims=[1])                                  # lag s -> x[t-s]
            prod = Hr * f.unsqueeze(0)
            even, odd = prod[:, 0::2].sum(1), prod[:, 1::2].sum(1)
            if cfg.use_hankel_L:
                return (even + odd).to(dt).unsqueeze(1)
            # minus branch: sgn[t] * sum_s f[s] sgn[t-s] x[t-s] = sum_s (-1)^s f[s] x[t-s]
            return ((even + odd).to(dt) + (even - odd).to(dt)).unsqueeze(1)
        self.hist[i] = torch.cat([self.hist[i], h], dim=1)
        H = torch.flip(self.hist[i].float(), dims=[1])                    # (B,t+1,d) by lag
        t1 = H.shape[1]
        ph = self.w["phi"].float()[:t1]                                   # (t+1,K)
        Up = torch.einsum("bsd,sk->bkd", H, ph).to(dt)
        y = torch.tensordot(Up, lw["stu.M_phi_plus"], dims=([1, 2], [0, 1]))
        if not cfg.use_hankel_L:
            sg = torch.ones(t1, 1, device=H.device)
            sg[1::2] = -1
            Um = torch.einsum("bsd,sk->bkd", H, ph * sg).to(dt)
            y = y + torch.tensordot(Um, lw["stu.M_phi_minus"], dims=([1, 2], [0, 1]))
        return y.unsqueeze(1)

    def step(self, tok: torch.Tensor) -> torch.Tensor:
        w, cfg = self.w, self.cfg
        x = w["tok_emb.weight"][tok].unsqueeze(1)
        for i in range(cfg.n_layers):
            lw = _sub(w, f"layers.{i}.")
            if cfg.is_attention_layer(i):
                a = rms_norm(x, lw["attn_norm.weight"], cfg.rms_eps)
                y, (k, v) = attention_forward(a, _sub(lw, "attn."), cfg.n_heads, cfg.window_size,
                                              cfg.softcap, self.kv[i])
                keep = cfg.window_size + 1
                self.kv[i] = (k[:, -keep:], v[:, -keep:])
                x = x + y
            else:
                h = rms_norm(x, lw["stu_norm.weight"], cfg.rms_eps)
                x = x + self._stu_step(i, h, lw)
            x = x + mlp_forward(rms_norm(x, lw["mlp_norm.weight"], cfg.rms_eps), _sub(lw, "mlp."))
        self.t += 1
        x = rms_norm(x, w["norm.weight"], cfg.rms_eps)
        return F.linear(x, w["tok_emb.weight"])


# --------------------------------------------------------------------------
# weights (flash_stu/model.py:52-106,428-452)
# --------------------------------------------------------------------------
def _xavier_normal_(t: torch.Tensor, gen: torch.Generator) -> None:
    """torch.nn.init.xavier_normal_: fan_in = size(1)*receptive, fan_out =
    size(0)*receptive for tensors of any rank >= 2."""
    rec = 1
    for s in t.shape[2:]:
        rec *= s
    fan_in, fan_out = t.shape[1] * rec, t.shape[0] * rec
    std = math.sqrt(2.0 / (fan_in + fan_out))
    t.copy_(torch.randn(t.shape, generator=gen) * std)


def init_weights(cfg: OracleConfig, seed: int = 0, mode: str = "reference",
                 phi: Optional[torch.Tensor] = None) -> Dict[str, torch.Tensor]:
    """Random-init weights under the reference's state-dict names.

    mode="reference" restates model.py:104-106,428-452: module.apply visits
    modules post-order in registration order (tok_emb, dropout, layers..., norm,
    lm_head); every Linear/Embedding draws normal(0, std) with the model-level
    std, which each SCALE_INIT linear (attention c_proj, attention.py:31) first
    multiplies by (2*n_layers)**-0.5 -- cumulatively; STU parameters and the
    attention c_attn/c_proj are then re-drawn xavier-normal when their parent
    module is visited.  tok_emb and lm_head share one tensor and lm_head is
    visited last, so its draw is the one that survives.
    mode="healthy" uses a fixed std of 0.02 for Linear/Embedding instead (same
    xavier rules), which keeps late layers numerically alive.
    The draws come from a private generator: the reference's own global-RNG
    stream is not reproduced (parity unpinned), only its procedure."""
    g = torch.Generator().manual_seed(seed)
    d, I, V, K = cfg.n_embd, cfg.intermediate_size, cfg.vocab_size, cfg.num_eigh
    dt = cfg.dtype
    w: Dict[str, torch.Tensor] = {}
    std = [d ** -0.5]

    def normal(shape, scale_init=False):
        if mode == "reference":
            if scale_init:
                std[0] *= (2 * cfg.n_layers) ** -0.5
            s = std[0]
        else:
            s = 0.02
        return (torch.randn(shape, generator=g) * s).to(dt)

    def xavier(shape):
        t = torch.empty(shape)
        _xavier_normal_(t, g)
        return t.to(dt)

    w["phi"] = (phi if phi is not None else get_spectral_filters(cfg.seq_len, K, cfg.use_hankel_L, dt)).to(dt)
    emb_first = normal((V, d))                       # tok_emb visit (overwritten by lm_head's)
    del emb_first
    for i in range(cfg.n_layers):
        pre = f"layers.{i}."
        if cfg.is_attention_layer(i):
            w[pre + "attn_norm.weight"] = torch.ones(d, dtype=dt)
            normal((3 * d, d))                               # c_attn as a Linear (re-drawn below)
            normal((d, d), scale_init=True)                  # c_proj: shrinks the running std
            w[pre + "attn.c_attn.weight"] = xavier((3 * d, d))
            w[pre + "attn.c_proj.weight"] = xavier((d, d))
        else:
            w[pre + "stu_norm.weight"] = torch.ones(d, dtype=dt)
            if cfg.use_approx:
                w[pre + "stu.M_inputs"] = xavier((d, d))
                w[pre + "stu.M_filters"] = xavier((K, d))
            else:
                w[pre + "stu.M_phi_plus"] = xavier((K, d, d))
                if not cfg.use_hankel_L:
                    w[pre + "stu.M_phi_minus"] = xavier((K, d, d))
        w[pre + "mlp_norm.weight"] = torch.ones(d, dtype=dt)
        w[pre + "mlp.gate_proj.weight"] = normal((I, d))
        w[pre + "mlp.up_proj.weight"] = normal((I, d))
        w[pre + "mlp.down_proj.weight"] = normal((d, I))
    w["norm.weight"] = torch.ones(d, dtype=dt)
    w["tok_emb.weight"] = normal((V, d))                     # lm_head visit; tied
    w["lm_head.weight"] = w["tok_emb.weight"]
    return w


def expected_reference_stds(cfg: OracleConfig) -> Dict[str, float]:
    """Closed-form std of each normal() draw under mode="reference"."""
    out, s = {}, cfg.n_embd ** -0.5
    shrink = (2 * cfg.n_layers) ** -0.5
    for i in range(cfg.n_layers):
        if cfg.is_attention_layer(i):
            s *= shrink
        out[f"layers.{i}.mlp"] = s
    out["tok_emb"] = s
    return out


def decode_step_bytes(cfg: OracleConfig, batch: int, t: int, state_dim: int = 0) -> int:
    """Algorithmic HBM bytes of one decode step at position t: every weight
    once, the visible KV window read plus one row written, the STU state read
    and written (state_dim fp32 values per (batch, channel); 0 = history form:
    the x_proj history up to t is read instead), fp32 logits written."""
    d, I, V = cfg.n_embd, cfg.intermediate_size, cfg.vocab_size
    wb = 2 if cfg.dtype == torch.bfloat16 else 4
    n_att = sum(cfg.is_attention_layer(i) for i in range(cfg.n_layers))
    n_stu = cfg.n_layers - n_att
    weights = (cfg.n_layers * (3 * d * I + 2 * d) + n_att * 4 * d * d + n_stu * d * d + d + V * d) * wb
    kv = n_att * batch * 2 * d * wb * (min(t, cfg.window_size + 1) + 1)
    if state_dim:
        stu = n_stu * (batch * state_dim * d * 4 * 2 + state_dim * d * 4)
    else:
        stu = n_stu * (batch * t * d * wb + (t + 1) // 2 * d * 4)
    return weights + kv + stu + batch * V * 4
