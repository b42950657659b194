#!/usr/bin/env python3
"""Benchmarks of the Flash STU token loop on one MI355X.

Default workload (BASELINE config 2, `--config c2`): FlashSTU 768-d / 12 layers (STU, SWA alternating) / 12 heads /
window 512 / 24 filters / seq_len 2048 / vocab 50257, random-init bf16 (seed 1), batch 8, 512-token prompts of uniform
random ids, greedy decode.  One "step" is one decode step of the whole batch (8 tokens).  The prompt is prefilled
(untimed, reported separately), W warm-up steps run, then exactly K steps are timed with the inputs, weights and decode
state resident in HBM.  The steps replay as HIP graphs of `--graph-steps` steps; what does not divide runs as
single-step graphs, so any --steps / --warmup keeps the long graphs.

Prints one JSON line.  `roofline` is the dominant kernel (the gate/up GLU projection, the largest weight stream of a
step), timed live with HIP events on the launch stream; `step_roofline` is the whole step against the HBM roofline;
`cpu_baseline` is the CPU oracle on a bounded sample of the same workload (BASELINE config 1 in full and a shortened
config 2, stateful and full-recompute decode, median of three).

Other workloads of BASELINE.json, same JSON keys:
  --config c5   FlashSTU 2048-d / 24 layers / 16 heads of 128 / window 1024, batch 32, 4096-token prompt, top-k 40 /
                temperature 0.8 sampling with the seeded stream (decode tokens/s, HBM roofline)
  --config c3   the exact-mode STU operator (use_approx=False) on x (4, 8192, 1024), K=24 (MFMA roofline)
  --config c4   the dense LDS step, batch 64, d=1024, state 160, 4096 steps with the state carried (HBM roofline of the
                one-launch form, microseconds per step of the per-launch form)
  --config c1   the tiny fp32 parity model, batch 1, 64-token prompt, 64 greedy tokens
  --config ref  the one shape the reference itself records a time for: STU.forward, approx mode, B=1, L=4096,
                d=2048, K=24, bf16 (tests/benchmark_tilling.py:157-165 of the reference; 2.43 ms per call on an H100 PCIe,
                tests/tilling/standard_memory_profile.txt:48-59)
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "flash-stu-2_amd"))

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
METRIC_C2 = "decode tokens/sec at 1 GPU (768-d FlashSTU, bs=8) + achieved HBM GB/s"


def decode_step_bytes(cfg, B, t, mode, S):
    """Algorithmic HBM bytes of one decode step at position t (every weight once, visible KV window + one row
    written, STU state or history, logits)."""
    d, I, V, w = cfg.n_embd, cfg.n_embd * cfg.mlp_scale, cfg.vocab_size, 2 if str(cfg.torch_dtype).endswith("bfloat16") else 4
    n_att = sum(1 for i in range(cfg.n_layers) if i % 2 == 1 and cfg.use_attn)
    n_stu = cfg.n_layers - n_att
    weights = (cfg.n_layers * (3 * d * I + 2 * d) + n_att * 4 * d * d + n_stu * d * d + d + V * d) * w
    kv = n_att * B * 2 * d * w * (min(t, cfg.window_left + 1) + 1)
    if mode == "lds":
        R = int(getattr(cfg, "stu_lds_fir_taps", 0) or 0)
        if B > 16 and w == 2 and not cfg.use_hankel_L:
            # 17..32 rows: the odd-lag sum is handed from step to step, so a step reads and writes ONE parity bank
            # (plus that sum, B x d fp32 read and written) and the even-lag half of the ring
            stu = n_stu * (B * S * d * 4 * 2 + 2 * B * d * 4 + 2 * S * d * 4)
            if R:
                stu += n_stu * (B * (R // 2) * d * w + B * d * w + R * d * 4)
        else:
            stu = n_stu * (B * S * d * 4 * 3 + 2 * S * d * 4)      # both parity banks read, one written; ce and co
            if R and not cfg.use_hankel_L:
                stu += n_stu * (B * R * d * w + B * d * w + R * d * 4)   # ring of the last R inputs read, one row written; taps
    else:
        stu = n_stu * (B * (t + 1) * d * w + (t + 1) * d * w)
    return weights + kv + stu + B * V * w


def timed_decode(eng, tokens, pos, step_idx, W, K, S, torch, temperature=1.0, top_k=None, top_p=None, do_sample=False, seed=0,
                 use_graph=True):
    """W warm-up steps, then K timed steps starting at position `pos`.  Returns (seconds for the K steps, next position).
    Graph replay: graphs of S steps; the warm-up's remainder (W % S) as single-step graphs, the timed steps' remainder
    (K % S) as one more graph of that many steps."""
    if not use_graph:
        def run(n, p):
            for i in range(n):
                eng.step(tokens, p + i, temperature, top_k, top_p, do_sample, seed, step_idx + (p + i - pos))
        run(W, pos)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(K, pos + W)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, pos + W + K
    w1, w8, k8, k1 = W % S, W // S, K // S, K % S
    eng.graph_begin(tokens, pos, step_idx, temperature, top_k, top_p, do_sample, seed, steps_per_graph=1)
    if w8 + k8 > 0 and S > 1:
        eng.graph_begin(tokens, pos + w1, step_idx + w1, temperature, top_k, top_p, do_sample, seed, steps_per_graph=S, keep=True)
    if k1 > 1:
        eng.graph_begin(tokens, pos + W + k8 * S, step_idx + W + k8 * S, temperature, top_k, top_p, do_sample, seed,
                        steps_per_graph=k1, keep=True)
    for _ in range(w1):
        eng.graph_step(1)
    for _ in range(w8):
        eng.graph_step(S)
    eng.graph_seek(1, pos + W + k8 * S)
    eng.graph_sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(k8):
        eng.graph_step(S)
    if k1:
        eng.graph_step(k1)
    eng.graph_sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    eng.graph_end()
    return dt, pos + W + K


def median_time(fn, reps=3):
    fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return statistics.median(ts)


def cpu_baseline(args, torch):
    """The CPU oracle on the box's host cores, a bounded sample (about 20 s): BASELINE config 1 in full (fp32,
    batch 1, 64-token prompt, 64 greedy tokens) and config 2 shortened (bf16, batch 8, 32-token prompt; 8 stateful
    decode steps, one full-recompute step); medians of three runs after one warm-up, except config 2's prompt pass and
    full-recompute step (seconds each), which are timed once.  `value` is config 2's
    stateful decode rate; the real Hankel filters are used."""
    from oracle import flashstu_oracle as O
    out = {}
    with torch.no_grad():
        # ---- config 1 in full
        c1 = O.OracleConfig(n_embd=256, n_heads=4, n_layers=4, seq_len=1024, window_size=128, vocab_size=50257,
                            mlp_scale=args.mlp_scale, num_eigh=24, dtype=torch.float32)
        w1 = O.init_weights(c1, seed=0, mode="reference")
        ids1 = torch.randint(0, 50257, (1, 64), generator=torch.Generator().manual_seed(0))
        t_rec = median_time(lambda: O.generate(w1, c1, ids1, max_length=128, do_sample=False, mode="recompute"))
        t_sta = median_time(lambda: O.generate(w1, c1, ids1, max_length=128, do_sample=False, mode="stateful"))
        out["c1_full"] = {"recompute_tokens_per_s": 64 / t_rec, "stateful_tokens_per_s": 64 / t_sta}
        # ---- config 2, shortened
        c2 = O.OracleConfig(n_embd=768, n_heads=12, n_layers=12, seq_len=2048, window_size=512, vocab_size=50257,
                            mlp_scale=args.mlp_scale, num_eigh=24, dtype=torch.bfloat16)
        w2 = O.init_weights(c2, seed=1, mode="reference")
        B, P, N = 8, 32, 8
        ids2 = torch.randint(0, 50257, (B, P), generator=torch.Generator().manual_seed(0))
        # the prompt pass and the full-recompute step cost seconds each on the CPU: timed once; the decode steps
        # (tens of milliseconds) are the median of three passes of N steps after one warm-up pass
        st = O.DecodeState(w2, c2, B)
        t0 = time.perf_counter()
        tok = st.prefill(ids2)[:, -1].argmax(-1)
        t_pre = time.perf_counter() - t0
        decs = []
        for rep in range(4):
            t1 = time.perf_counter()
            for _ in range(N):
                tok = st.step(tok)[:, -1].argmax(-1)
            if rep:
                decs.append(time.perf_counter() - t1)
        t_dec = statistics.median(decs)
        seq = torch.cat([ids2, ids2[:, :1]], 1)
        t0 = time.perf_counter()
        O.model_forward(w2, c2, seq)                  # one full-recompute step = one forward over prompt + 1 tokens
        t_rec2 = time.perf_counter() - t0
        out["c2_short"] = {"prefill_tokens_per_s": B * P / t_pre, "stateful_tokens_per_s": B * N / t_dec,
                           "recompute_tokens_per_s": B / t_rec2}
    return {"value": out["c2_short"]["stateful_tokens_per_s"], "unit": "tokens/s", "cores": torch.get_num_threads(),
            "os_cpu_count": os.cpu_count(), "kind": "port",
            "sample": f"CPU oracle, median of 3: config 1 in full (fp32, 1x64 prompt, 64 tokens) and config 2 shortened (bf16, "
                      f"{B}x{P} prompt, {N} stateful decode steps, one full-recompute step), mlp_scale {args.mlp_scale}; value = config 2 stateful",
            "detail": out}


def glu_roofline(eng, cfg, B, K, lib, torch, _hip):
    """The gate/up GLU projection of every layer launched back to back on one stream between two HIP events (the
    same kernel, weights and activations as inside the step; cycling through the layers' weights keeps them from
    being served out of the 256 MB Infinity Cache)."""
    d, I = cfg.n_embd, cfg.n_embd * cfg.mlp_scale
    if eng.desc.B > _hip.MAX_DECODE_ROWS:
        # 17..32 rows: the step's gate/up launch covers all rows and reads every weight once: the balanced kernel over
        # packed weights with two row tiles per weight fragment where the shape allows it, else the tiled GEMM kernel
        rows = eng.desc.B
        h = torch.randn(rows, d, device="cuda", dtype=torch.bfloat16)
        act = torch.empty(rows, I, device="cuda", dtype=torch.bfloat16)
        mlps = [l.mlp for l in eng.model.layers]
        packed = bool(lib.fstu_mlp_packed_rows32_supported(rows, d, I))
        if packed:
            # as the step launches it: mlp_norm of the summed residual stream formed in the launch's own fragments
            ops = [(eng._pack(l.mlp.gate_proj.weight), eng._pack(l.mlp.up_proj.weight), l.mlp_norm.weight) for l in eng.model.layers]
            launch = lambda o: _hip.glu_packed_norm(h, None, o[2], cfg.rms_norm_eps, o[0], o[1], I, out=act)
            name = ("glu_balanced_kernel<two row tiles, norm in the fragments> (mlp_norm + gate/up projection + gelu*up over "
                    "all rows, packed weights, one workgroup per compute unit)")
        else:
            ops = [(m_.gate_proj.weight, m_.up_proj.weight) for m_ in mlps]
            launch = lambda o: _hip.gemm(h, o[0], up_weight=o[1], out=act)
            name = "gemm_bf16_kernel<128 features x 32 rows, gated pair> (gate/up projection + gelu*up over all rows)"
        for o in ops[:2]:
            launch(o)
        reps = max(1, 96 // len(mlps))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for o in ops:
                launch(o)
        e1.record()
        torch.cuda.synchronize()
        n = reps * len(mlps)
        us = e0.elapsed_time(e1) * 1e3 / n
        glu_bytes = 2 * I * d * 2 + rows * d * 2 + rows * I * 2
        gbps = glu_bytes / (us * 1e-6) / 1e9
        # HBM bytes per launch from two rocprofv3 --pmc runs (FETCH_SIZE x2.000, WRITE_SIZE x1.000 against the library's
        # plain copy kernel), measured offline for config 5's shape: profiles/decode_c5_hbm_traffic_pmc.txt
        traffic = 204146262 if packed and (d, I, rows) == (2048, 24576, 32) else None
        return {"bound": "hbm", "kernel": name,
                "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": traffic,
                "traffic_source": "profiles/decode_c5_hbm_traffic_pmc.txt (counter runs of this kernel, not of this run)" if traffic else None,
                "bytes_per_launch": glu_bytes, "avg_launch_us": us, "launches_timed": n, "rows_per_launch": rows}
    ms_c, n_c = ctypes.c_double(), ctypes.c_int()
    torch.cuda.synchronize()
    _hip._check(lib.fstu_prof_glu_loop(ctypes.byref(eng.desc), max(4, K // 8), ctypes.byref(ms_c), ctypes.byref(n_c),
                                       torch.cuda.current_stream().cuda_stream), "fstu_prof_glu_loop")
    rows = eng.desc.B
    glu_bytes = 2 * I * d * 2 + rows * d * 2 + rows * I * 2   # gate+up weights, x in, act out (the prologue adds 0.1 %)
    us = ms_c.value / n_c.value * 1e3
    gbps = glu_bytes / (us * 1e-6) / 1e9
    # HBM bytes per launch from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE, each scaled by what the same counter
    # reads for the library's plain 256 MiB copy kernel: x2.000 and x1.000); measured offline for the default workload,
    # summary and commands in profiles/glu_c2_hbm_traffic_pmc.txt
    default_shape = (cfg.n_embd, cfg.mlp_scale, rows) == (768, 12, 8)
    traffic = 28870625 if default_shape else None
    return {"bound": "hbm", "kernel": "glu_balanced_kernel<PRO> (residual add + mlp_norm + gate/up projection + gelu*up)",
            "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": traffic,
            "traffic_source": "profiles/glu_c2_hbm_traffic_pmc.txt (counter runs of this kernel, not of this run)" if default_shape else None,
            "bytes_per_launch": glu_bytes, "avg_launch_us": us, "launches_timed": n_c.value, "rows_per_launch": rows}


def run_lm(args, torch, _hip, which):
    """configs 2 and 5 (and 1): prefill, warm-up, timed decode steps of a FlashSTU language model."""
    from flash_stu import FlashSTU, FlashSTUConfig
    if which == "c5":
        kw = dict(n_embd=2048, n_layers=24, n_heads=16, window_size=1024, num_eigh=24, seq_len=8192, vocab_size=50257)
        B, P, seed, dt = args.batch or 32, args.prompt or 4096, 2, torch.bfloat16
        sampling = dict(temperature=0.8, top_k=40, top_p=None, do_sample=True, seed=2)
        label = ("BASELINE config 5: FlashSTU 2048-d/24-layer/16-head, window 1024, K=24, seq_len 8192, vocab 50257, random-init "
                 "bf16 seed 2, batch 32, 4096-token prompt, top-k 40 / temperature 0.8 sampling with the seeded stream")
        metric = "decode tokens/sec at 1 GPU (2048-d FlashSTU, bs=32, top-k 40 sampling) + achieved HBM GB/s"
    elif which == "c1":
        kw = dict(n_embd=256, n_layers=4, n_heads=4, window_size=128, num_eigh=24, seq_len=1024, vocab_size=50257)
        B, P, seed, dt = args.batch or 1, args.prompt or 64, 0, torch.float32
        sampling = dict(temperature=1.0, top_k=None, top_p=None, do_sample=False, seed=0)
        label = ("BASELINE config 1: FlashSTU 256-d/4-layer/4-head, window 128, K=24, seq_len 1024, vocab 50257, random-init "
                 "fp32 seed 0, batch 1, 64-token prompt, greedy decode")
        metric = "decode tokens/sec at 1 GPU (256-d FlashSTU fp32, bs=1) + achieved HBM GB/s"
    else:
        kw = dict(n_embd=768, n_layers=12, n_heads=12, window_size=512, num_eigh=24, seq_len=2048, vocab_size=50257)
        B, P, seed, dt = args.batch or 8, args.prompt or 512, 1, torch.bfloat16
        sampling = dict(temperature=1.0, top_k=None, top_p=None, do_sample=False, seed=0)
        label = ("BASELINE config 2: FlashSTU 768-d/12-layer/12-head, window 512, K=24, seq_len 2048, vocab 50257, random-init "
                 "bf16 seed 1, batch 8, 512-token prompt, greedy decode")
        metric = METRIC_C2
        if args.top_k:
            # not the headline workload: the same model with config 5's sampling, to price the sampler against greedy
            sampling = dict(temperature=0.8, top_k=args.top_k, top_p=None, do_sample=True, seed=2)
            label = label.replace("greedy decode", f"top-k {args.top_k} / temperature 0.8 sampling with the seeded stream")
    stu_mode = args.stu_mode if dt == torch.bfloat16 else "history"
    K, W = args.steps, args.warmup

    def build(mlp_scale):
        fir = {} if args.fir_taps is None else {"stu_lds_fir_taps": args.fir_taps}
        cfg = FlashSTUConfig(mlp_scale=mlp_scale, torch_dtype=dt, stu_decode_mode=stu_mode, stu_prefill_mode=args.stu_prefill, **fir, **kw)
        torch.manual_seed(seed)
        with torch.device("cuda"):
            model = FlashSTU(cfg)
        return cfg, model.cuda().eval()

    def measure(cfg, model, full):
        total = P + W + 2 * K + 16
        assert total <= cfg.seq_len, (total, cfg.seq_len)
        ids = torch.randint(0, cfg.vocab_size, (B, P), generator=torch.Generator().manual_seed(seed)).cuda()
        eng = model.decode_engine()
        tokens = torch.zeros(B, total, dtype=torch.int64, device="cuda")
        tokens[:, :P] = ids
        res = {}
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = eng.prefill(ids, total)
        _hip.sample(logits, tokens[:, P], sampling["temperature"], sampling["top_k"], sampling["top_p"], sampling["do_sample"], sampling["seed"], 0)
        torch.cuda.synchronize()
        res["prefill_first_call_ms"] = (time.perf_counter() - t0) * 1e3
        if full:
            warm = []
            for _ in range(5 if which != "c5" else 2):      # warm prefill: median (the second call still loads code objects)
                t0 = time.perf_counter()
                logits = eng.prefill(ids, total)
                _hip.sample(logits, tokens[:, P], sampling["temperature"], sampling["top_k"], sampling["top_p"], sampling["do_sample"], sampling["seed"], 0)
                torch.cuda.synchronize()
                warm.append(time.perf_counter() - t0)
            res["prefill_ms"] = statistics.median(warm) * 1e3
            res["prefill_tokens_per_s"] = B * P / statistics.median(warm)
        use_graph = eng.graph_supported() and not args.no_graph
        dt_s, pos = timed_decode(eng, tokens, P, 1, W, K, args.graph_steps, torch, use_graph=use_graph, **sampling)
        res["ms_per_step"] = dt_s / K * 1e3
        res["value"] = B * K / dt_s
        S = cfg.stu_lds_state_dim
        step_bytes = decode_step_bytes(cfg, B, P + W + K // 2, stu_mode, S)
        res["step_roofline"] = {"bound": "hbm", "bytes_per_step": step_bytes, "achieved": step_bytes / (res["ms_per_step"] * 1e-3) / 1e9,
                                "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": step_bytes / (res["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        res["hip_graph"] = bool(use_graph)
        res["params"] = model.get_num_params()
        return res, eng, tokens, pos

    cfg, model = build(args.mlp_scale)
    res, eng, tokens, pos = measure(cfg, model, True)
    lib = _hip.load()
    out = {
        "metric": metric, "value": res["value"], "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if dt == torch.bfloat16 else "f32", "data": "synthetic",
        "config": {"workload": label, "mlp_scale": cfg.mlp_scale, "params": res["params"], "batch": B, "prompt": P,
                   "stu_decode_mode": stu_mode, "stu_prefill_mode": args.stu_prefill, "hip_graph": res["hip_graph"],
                   "graph_steps": args.graph_steps, "stu_state_dim": cfg.stu_lds_state_dim if stu_mode == "lds" else None,
                   "stu_fir_taps": cfg.stu_lds_fir_taps if stu_mode == "lds" else None},
        "step_roofline": res["step_roofline"],
        "prefill_tokens_per_s": res.get("prefill_tokens_per_s"), "prefill_ms": res.get("prefill_ms"),
        "prefill_first_call_ms": res["prefill_first_call_ms"],
    }
    if dt == torch.bfloat16:
        out["roofline"] = glu_roofline(eng, cfg, B, K, lib, torch, _hip)
    else:
        out["roofline"] = dict(res["step_roofline"], kernel="whole decode step (fp32 parity path)", traffic=None)
    if args.pmc_calibrate:
        a_ = torch.zeros(256 << 20, dtype=torch.uint8, device="cuda")
        b_ = torch.empty_like(a_)
        for _ in range(4):
            _hip._check(lib.fstu_prof_copy(b_.data_ptr(), a_.data_ptr(), a_.numel(), torch.cuda.current_stream().cuda_stream), "fstu_prof_copy")
        torch.cuda.synchronize()
        del a_, b_
    if which == "c2":
        # MFMA rates of the prompt pass's two largest contractions as the MLP runs them (hand-written kernel
        # fstu_gemm_bf16): gate+up with the gelu*up epilogue, and the down projection with the residual add
        gm, gi, gd = B * P, cfg.n_embd * cfg.mlp_scale, cfg.n_embd
        ga = torch.randn(gm, gd, device="cuda", dtype=torch.bfloat16)
        mlp0 = model.layers[0].mlp
        gres = torch.zeros(gm, gd, device="cuda", dtype=torch.bfloat16)

        def _rate(fn, flops):
            for _ in range(3):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                fn()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 20
            tf = flops / (us * 1e-6) / 1e12
            return {"us": us, "achieved": tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tf / MFMA_BF16_PEAK_TFLOPS}
        gact = _hip.gemm(ga, mlp0.gate_proj.weight, up_weight=mlp0.up_proj.weight)
        out["prefill_gemm"] = dict(_rate(lambda: _hip.gemm(ga, mlp0.gate_proj.weight, up_weight=mlp0.up_proj.weight, out=gact),
                                         4.0 * gm * gi * gd),
                                   what="gate+up projection of the prompt with the gelu*up epilogue (M, 2N, K)", shape=[gm, 2 * gi, gd])
        out["prefill_gemm_down"] = dict(_rate(lambda: _hip.gemm(gact, mlp0.down_proj.weight, residual=gres, out=gres),
                                              2.0 * gm * gi * gd),
                                        what="down projection of the prompt with the residual add (M, N, K)", shape=[gm, gd, gi])
        del gact, gres
        del ga
    if args.breakdown:
        names = {1: "glu", 2: "down", 3: "head", 4: "attention", 5: "stu_step", 6: "proj_qkv", 7: "embed_add_norm", 8: "sample"}
        n = min(K, 32)
        br = {}
        for c, nm in names.items():
            _hip._check(lib.fstu_prof_begin(c, n * cfg.n_layers * 2 + 8), "fstu_prof_begin")
            for i in range(n):
                eng.step(tokens, pos + i, 1.0, None, None, False, 0, pos + i - P + 1)
            ms, cnt = ctypes.c_double(), ctypes.c_int()
            _hip._check(lib.fstu_prof_end(ctypes.byref(ms), ctypes.byref(cnt)), "fstu_prof_end")
            br[nm] = ms.value / n * 1e3
        out["kernel_us_per_step"] = br
    if which == "c2" and args.mlp_scale == 12 and not args.no_mlp4:
        # BASELINE.json leaves mlp_scale open: 12 is the reference config's default, 4 matches the "~125M" label
        del eng, model
        torch.cuda.empty_cache()
        cfg4, model4 = build(4)
        r4, eng4, _, _ = measure(cfg4, model4, False)
        out["mlp_scale_4"] = {"params": r4["params"], "ms_per_step": r4["ms_per_step"], "value": r4["value"], "unit": "tokens/s",
                              "step_roofline": r4["step_roofline"]}
        del eng4, model4
        torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args, torch)
    return out


def run_c3(args, torch, _hip):
    """The exact-mode STU operator (use_approx=False; flash_stu/modules/stu.py:99-120 of the reference) at BASELINE
    config 3's shape.  A step is one forward of the operator; the bound is the MFMA rate of its contraction
    (2 * B * L * (2K d) * d flops), the FFT part being small beside it."""
    from flash_stu import STU, FlashSTUConfig
    from flash_stu.utils.stu_utils import get_spectral_filters
    B, L, d, Kf = args.batch or 4, 8192, 1024, 24
    cfg = FlashSTUConfig(n_embd=d, n_heads=16, n_layers=2, seq_len=L, num_eigh=Kf, vocab_size=64, torch_dtype=torch.bfloat16,
                         use_approx=False)
    phi = get_spectral_filters(L, Kf, device=torch.device("cpu"), dtype=torch.bfloat16).cuda()
    g = torch.Generator().manual_seed(3)
    stu = STU(cfg, phi, 2 * L).cuda()
    with torch.no_grad():
        stu.M_phi_plus.copy_((torch.randn(Kf, d, d, generator=g) / d ** 0.5).to(torch.bfloat16))
        stu.M_phi_minus.copy_((torch.randn(Kf, d, d, generator=g) / d ** 0.5).to(torch.bfloat16))
    x = torch.randn(B, L, d, generator=g).to(torch.bfloat16).cuda()
    K, W = args.steps, args.warmup
    for _ in range(max(W, 1)):
        y = stu(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        y = stu(x)
    torch.cuda.synchronize()
    dt_s = time.perf_counter() - t0
    ms = dt_s / K * 1e3
    flops = 2.0 * B * L * (2 * Kf * d) * d
    tf = flops / (ms * 1e-3) / 1e12
    alg_bytes = 2 * B * L * d * 2 + 2 * Kf * d * d * 2
    out = {"metric": "exact-mode STU operator (use_approx=False) tokens/sec at 1 GPU + MFMA utilisation", "value": B * L / (ms * 1e-3),
           "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "BASELINE config 3: STU exact mode, x (4, 8192, 1024) bf16 ~ N(0,1), K=24 Hankel filters (L=8192), "
                                  "M_phi+- (24,1024,1024) ~ N(0, 1/sqrt(d)), FFT length 16384", "batch": B, "L": L, "d": d, "K": Kf},
           "roofline": {"bound": "mfma", "kernel": "contraction of U+- (B*L, 2*K*d) with M_phi+- (2*K*d, d), whole operator timed",
                        "achieved": tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tf / MFMA_BF16_PEAK_TFLOPS,
                        "traffic": None, "flops_per_step": flops, "algorithmic_bytes": alg_bytes}}
    assert bool(torch.isfinite(y.float()).all())
    return out


def run_c4(args, torch, _hip):
    """The dense LDS step of mini_stu/lds.py:95-101 at BASELINE config 4's shape: 4096 consecutive steps with the
    state carried, as ONE launch over pre-staged inputs (HBM-bound: x in, y out) and launch by launch."""
    g = torch.Generator().manual_seed(4)
    T, Bt, d, S = 4096, args.batch or 64, 1024, 160
    A = (0.9 + 0.099 * torch.rand(S, generator=g)).float().cuda()
    Bm = (torch.randn(d, S, generator=g) / d).to(torch.bfloat16).cuda()
    Cm = (torch.randn(S, d, generator=g) / S).to(torch.bfloat16).cuda()
    x = torch.randn(T, Bt, d, generator=g).to(torch.bfloat16).cuda()
    y = torch.empty_like(x)
    h = torch.zeros(Bt, S, dtype=torch.float32, device="cuda")
    K, W = max(1, args.steps // 64), max(1, args.warmup // 16)      # a "step" here is one launch over all 4096 positions
    for _ in range(W):
        h.zero_()
        _hip.lds_steps(h, x, A, Bm, Cm, y)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        _hip.lds_steps(h, x, A, Bm, Cm, y)
    torch.cuda.synchronize()
    dt_s = time.perf_counter() - t0
    ms = dt_s / K * 1e3
    _hip.lds_steps(h, x, A, Bm, Cm, y, check_status=True)      # raises if a block's wait for its predecessors ran out
    assert bool(torch.isfinite(y.float()).all())
    alg = 2 * T * Bt * d * 2 + (2 * d * S * 2 + S * 4) + 2 * Bt * S * 4      # x in, y out, weights, state
    gbps = alg / (ms * 1e-3) / 1e9
    # launch by launch (one position per launch, state carried in HBM)
    n1 = 512
    h.zero_()
    tr = (Bm.t().contiguous(), Cm.t().contiguous())
    ws1 = torch.empty(int(_hip.load().fstu_lds_sequence_ws_floats(1, Bt, S)), dtype=torch.float32, device="cuda")
    for t in range(16):
        _hip.lds_steps(h, x[t:t + 1], A, Bm, Cm, y[t:t + 1], transposed=tr, ws=ws1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(n1):
        _hip.lds_steps(h, x[t:t + 1], A, Bm, Cm, y[t:t + 1], transposed=tr, ws=ws1)
    torch.cuda.synchronize()
    us_launch = (time.perf_counter() - t0) / n1 * 1e6
    return {"metric": "dense LDS steps/sec at 1 GPU (batch 64, d=1024, state 160, state carried) + achieved HBM GB/s",
            "value": T / (ms * 1e-3), "unit": "steps/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "BASELINE config 4: dense LDS step, batch 64, d_in=d_out=1024, state 160, A~U(0.9,0.999) fp32, "
                                   "B~N(0,1/d), C~N(0,1/160) bf16, 4096 consecutive steps in one launch (a bench step = one launch)",
                       "positions_per_launch": T, "us_per_position_one_launch": ms * 1e3 / T, "us_per_position_launch_by_launch": us_launch},
            "roofline": {"bound": "hbm", "kernel": "lds_seq_kernel (blocks of 128 positions on the matrix cores, the state handed from block to block inside the launch; x is read once)", "achieved": gbps,
                         "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": None, "bytes_per_launch": alg}}


def run_ref(args, torch, _hip):
    """STU.forward in approx mode at the shape of the reference's own benchmark (tests/benchmark_tilling.py:157-165:
    n_embd 2048, seq_len 4096, num_eigh 24, use_approx, bf16, batch 1; x ~ N(0,1)): x @ M_inputs on the matrix cores,
    then the spectral convolution with phi @ M_filters, both sign branches.  A step is one call of the operator."""
    from flash_stu import STU, FlashSTUConfig
    from flash_stu.utils.stu_utils import get_spectral_filters
    B, L, d, Kf = args.batch or 1, 4096, 2048, 24
    cfg = FlashSTUConfig(n_embd=d, n_heads=16, n_layers=2, seq_len=L, num_eigh=Kf, vocab_size=64, torch_dtype=torch.bfloat16,
                         use_approx=True, use_hankel_L=False)
    phi = get_spectral_filters(L, Kf, device=torch.device("cpu"), dtype=torch.bfloat16).cuda()
    g = torch.Generator().manual_seed(5)
    stu = STU(cfg, phi, 2 * L).cuda()
    with torch.no_grad():
        stu.M_inputs.copy_((torch.randn(d, d, generator=g) / d ** 0.5).to(torch.bfloat16))
        stu.M_filters.copy_((torch.randn(Kf, d, generator=g) / Kf ** 0.5).to(torch.bfloat16))
    x = torch.randn(B, L, d, generator=g).to(torch.bfloat16).cuda()
    K, W = args.steps, args.warmup

    def timed(fn, n):
        for _ in range(max(W, 2)):
            out = fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(n):
            out = fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n, out
    for _ in range(max(W, 1)):
        y = stu(x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        y = stu(x)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / K * 1e3
    assert bool(torch.isfinite(y.float()).all())
    # the two launches of the operator on their own (HIP events on the launch stream)
    # (x @ M_inputs as time-major slabs, the convolution on them, the transpose of its result)
    ms_proj, xt = timed(lambda: stu._project_time_major(x), K)
    yt = torch.empty_like(xt)
    spec = stu.filter_spectrum(_hip.fft_length(L))
    ms_conv, _ = timed(lambda: _hip.stu_conv_fft_strided(xt.transpose(1, 2), spec, yt.transpose(1, 2)), K)
    ms_tr, _ = timed(lambda: _hip.transpose(yt), K)
    conv_bytes = 2 * B * L * d * 2 + L * d * 2          # x_proj in, y out, the filter once
    conv_gbps = conv_bytes / (ms_conv * 1e-3) / 1e9
    flops = 2.0 * B * L * d * d
    published_ms = 2.43
    return {"metric": "STU.forward (approx mode, B=1, L=4096, d=2048, K=24, bf16) tokens/sec at 1 GPU", "value": B * L / (ms * 1e-3),
            "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": published_ms / ms, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "the reference's own recorded benchmark shape: STU.forward, approx mode, batch 1, L=4096, "
                                   "d=2048, K=24 Hankel filters, bf16, x ~ N(0,1) (tests/benchmark_tilling.py:157-165)",
                       "batch": B, "L": L, "d": d, "K": Kf,
                       "published": {"ms_per_call": published_ms, "hardware": "NVIDIA H100 PCIe (another GPU: context, not a like-for-like bar)",
                                     "source": "tests/tilling/standard_memory_profile.txt:48-59"}},
            "kernels_ms": {"x @ M_inputs (gemm_bf16_kernel, time-major output)": ms_proj,
                           "spectral convolution (fft_conv_kernel on time-major slabs)": ms_conv,
                           "result back to (L, d) (transpose_tiles_kernel)": ms_tr,
                           "projection_tflops": flops / (ms_proj * 1e-3) / 1e12},
            "roofline": {"bound": "hbm", "kernel": "fft_conv_kernel (spectral convolution of the projected inputs, both sign branches, one column per workgroup)",
                         "achieved": conv_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": conv_gbps / HBM_PEAK_GBPS,
                         "traffic": None, "bytes_per_launch": conv_bytes, "avg_launch_us": ms_conv * 1e3}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", default="c2", choices=["c1", "c2", "c3", "c4", "c5", "ref"], help="BASELINE.json workload (default: config 2)")
    ap.add_argument("--mlp-scale", type=int, default=12, dest="mlp_scale")
    ap.add_argument("--stu-mode", default="lds", choices=["lds", "history"], dest="stu_mode")
    ap.add_argument("--fir-taps", type=int, default=None, dest="fir_taps",
                    help="exact head of the distilled STU filter: first lags taken from phi_proj itself (0: off; default: the config's)")
    ap.add_argument("--stu-prefill", default="fft", choices=["fft", "scan"], dest="stu_prefill",
                    help="prompt pass of the STU layers: the reference's FFT convolution, or the distilled recurrence as a scan")
    ap.add_argument("--batch", type=int, default=0, help="batch rows (default: the workload's own)")
    ap.add_argument("--prompt", type=int, default=0, help="prompt length (default: the workload's own)")
    ap.add_argument("--top-k", type=int, default=0, dest="top_k",
                    help="config 2 only: sample with this top-k at temperature 0.8 instead of the greedy pick")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-mlp4", action="store_true", dest="no_mlp4", help="skip the second measurement of config 2 at mlp_scale 4")
    ap.add_argument("--graph-steps", type=int, default=8, dest="graph_steps", help="decode steps captured per HIP graph")
    ap.add_argument("--no-graph", action="store_true", help="launch every step kernel by kernel instead of replaying HIP graphs")
    ap.add_argument("--pmc-calibrate", action="store_true", dest="pmc_calibrate",
                    help="also launch the library's plain 256 MiB copy kernel 4 times (reference for traffic counters)")
    ap.add_argument("--breakdown", action="store_true", help="time every kernel class with HIP events")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (decode shards by batch: every GPU would hold the full weights "
              "and its own sequences, with no exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from flash_stu import _hip
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    if args.config in ("c1", "c2", "c5"):
        out = run_lm(args, torch, _hip, args.config)
    elif args.config == "c3":
        out = run_c3(args, torch, _hip)
    elif args.config == "ref":
        out = run_ref(args, torch, _hip)
    else:
        out = run_c4(args, torch, _hip)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
