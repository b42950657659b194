"""Writes tests/golden/kat_small.npz: small known-answer vectors for the hot path, computed here from first
principles in float64 with plain numpy loops (no oracle code, no FFT, no library attention), so that they pin the
CPU oracle and the HIP path independently.  Run once:  python tests/golden/make_fixtures.py

Contents (reference statements they follow):
  phi_L8_K3, phi_L64_K6      Hankel filters: Z[i,j] = 2/((i+j)^3-(i+j)), top-K eigenpairs ascending, phi = v*sigma^(1/4),
                             column sign fixed so that the largest-magnitude entry is positive
                             (flash_stu/utils/stu_utils.py:18-31,146-193)
  conv_x, conv_f, conv_plus, conv_minus
                             plus[t,c] = sum_{s<=t} f[s,c] x[t-s,c];  minus[t,c] = sum_s (-1)^s f[s,c] x[t-s,c]
                             (flash_stu/utils/stu_utils.py:195-228, time-domain statement)
  att_q, att_k, att_v, att_out
                             sliding-window attention with ALiBi and tanh soft-capping, W+1 keys incl. self
                             (flash_stu/modules/attention.py:59-105, flash-attn's documented semantics)
  lds_A, lds_B, lds_C, lds_x, lds_y
                             h <- h*A + x_t B ; y_t = h C  (mini_stu/lds.py:95-101)
  samp_logits, samp_topk_keep, samp_topp_keep
                             survivors of top-k (all values >= k-th) and top-p (sorted cumsum > p shifted right by one)
                             (flash_stu/model.py:268-289)
"""
import math
import os

import numpy as np


def hankel_filters(L, K):
    i = np.arange(1, L + 1, dtype=np.float64)
    s = i[:, None] + i[None, :]
    Z = 2.0 / (s ** 3 - s)
    sig, vec = np.linalg.eigh(Z)
    sig, vec = sig[-K:], vec[:, -K:]
    phi = vec * sig ** 0.25
    for k in range(K):
        if phi[np.abs(phi[:, k]).argmax(), k] < 0:
            phi[:, k] = -phi[:, k]
    return phi


def conv_branches(x, f):
    T, d = x.shape
    plus = np.zeros((T, d))
    minus = np.zeros((T, d))
    for t in range(T):
        for s in range(min(t + 1, f.shape[0])):
            plus[t] += f[s] * x[t - s]
            minus[t] += (-1.0) ** s * f[s] * x[t - s]
    return plus, minus


def alibi_slopes(H):
    def gen(n):
        start = 2.0 ** (-(2.0 ** -(math.log2(n) - 3)))
        return [start * start ** i for i in range(n)]
    if math.log2(H).is_integer():
        sl = gen(H)
    else:
        n = 2 ** math.floor(math.log2(H))
        sl = gen(n) + gen(2 * n)[0::2][: H - n]
    return np.array(sl) * 0.25


def swa(q, k, v, W, softcap):
    T, H, hd = q.shape
    sl = alibi_slopes(H)
    out = np.zeros((T, H, hd))
    for h in range(H):
        for p in range(T):
            js = [j for j in range(max(0, p - W), p + 1)]
            s = np.array([q[p, h] @ k[j, h] / math.sqrt(hd) for j in js])
            s = softcap * np.tanh(s / softcap)
            s = s - sl[h] * np.array([p - j for j in js])
            e = np.exp(s - s.max())
            pr = e / e.sum()
            out[p, h] = sum(pr[i] * v[j, h] for i, j in enumerate(js))
    return out


def main():
    rng = np.random.default_rng(20240517)
    out = {}
    out["phi_L8_K3"] = hankel_filters(8, 3)
    out["phi_L64_K6"] = hankel_filters(64, 6)
    x = rng.standard_normal((12, 3))
    f = rng.standard_normal((12, 3)) * np.linspace(1.0, 0.1, 12)[:, None]
    out["conv_x"], out["conv_f"] = x, f
    out["conv_plus"], out["conv_minus"] = conv_branches(x, f)
    q, k, v = (rng.standard_normal((9, 4, 32)) for _ in range(3))
    out["att_q"], out["att_k"], out["att_v"] = q, k, v
    out["att_out"] = swa(q, k, v, W=3, softcap=50.0)
    A = rng.uniform(0.5, 0.99, 5)
    B = rng.standard_normal((4, 5)) / 4
    C = rng.standard_normal((5, 3)) / 5
    xs = rng.standard_normal((7, 2, 4))
    h = np.zeros((2, 5))
    ys = np.zeros((7, 2, 3))
    for t in range(7):
        h = h * A + xs[t] @ B
        ys[t] = h @ C
    out.update(lds_A=A, lds_B=B, lds_C=C, lds_x=xs, lds_y=ys)
    logits = np.round(rng.standard_normal((2, 11)) * 2, 2)
    logits[0, 3] = logits[0, 7]                      # a tie at the boundary region
    keep_k = np.zeros_like(logits, dtype=bool)
    keep_p = np.zeros_like(logits, dtype=bool)
    for b in range(2):
        kth = np.sort(logits[b])[-3]
        keep_k[b] = logits[b] >= kth
        order = np.argsort(-logits[b], kind="stable")
        pr = np.exp(logits[b][order] - logits[b].max())
        pr /= pr.sum()
        cum = np.cumsum(pr)
        rem = cum > 0.8
        rem[1:] = rem[:-1].copy()
        rem[0] = False
        keep_p[b, order] = ~rem
    out.update(samp_logits=logits, samp_topk_keep=keep_k, samp_topp_keep=keep_p)
    np.savez(os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat_small.npz"), **out)
    print({k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
