#!/usr/bin/env python3
"""Decode-throughput benchmark of the Flash STU token loop on one MI355X.

Workload (BASELINE config 2): FlashSTU 768-d / 12 layers (STU, SWA alternating)
/ 12 heads / window 512 / 24 filters / seq_len 2048 / vocab 50257, random-init
bf16 (seed 1), batch 8, 512-token prompts of uniform random ids, greedy decode.
One "step" is one decode step of the whole batch (8 tokens).  The prompt is
prefilled (untimed, reported separately), W warm-up steps run, then exactly K
steps are timed with the inputs, weights and decode state resident in HBM.

Prints one JSON line; see the keys below.  `roofline` is the dominant kernel
(the gate/up GLU projection, the largest weight stream of a step), timed live
with HIP events on the launch stream in a second pass over the same K steps;
`step_roofline` is the whole step against the HBM roofline; `cpu_baseline` is
the CPU oracle on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "flash-stu-2_amd"))

HBM_PEAK_GBPS = 8000.0


def build_model(args, torch):
    from flash_stu import FlashSTU, FlashSTUConfig
    cfg = FlashSTUConfig(n_embd=768, n_layers=12, n_heads=12, window_size=512, num_eigh=24, seq_len=2048,
                         vocab_size=50257, mlp_scale=args.mlp_scale, torch_dtype=torch.bfloat16,
                         stu_decode_mode=args.stu_mode, stu_prefill_mode=args.stu_prefill)
    torch.manual_seed(1)
    model = FlashSTU(cfg).cuda().eval()
    return cfg, model


def decode_step_bytes(cfg, B, t, mode, S):
    """Algorithmic HBM bytes of one decode step at position t (every weight
    once, visible KV window + one row written, STU state or history, logits)."""
    d, I, V, w = cfg.n_embd, cfg.n_embd * cfg.mlp_scale, cfg.vocab_size, 2
    n_att = sum(1 for i in range(cfg.n_layers) if i % 2 == 1 and cfg.use_attn)
    n_stu = cfg.n_layers - n_att
    weights = (cfg.n_layers * (3 * d * I + 2 * d) + n_att * 4 * d * d + n_stu * d * d + d + V * d) * w
    kv = n_att * B * 2 * d * w * (min(t, cfg.window_left + 1) + 1)
    if mode == "lds":
        stu = n_stu * (B * S * d * 4 * 2 + S * d * 4)
    else:
        stu = n_stu * (B * (t + 1) * d * w + (t + 1) * d * w)
    return weights + kv + stu + B * V * w


def cpu_baseline(args, torch):
    """CPU oracle (stateful decode) on a bounded sample: batch 8, 32-token
    prompt, 6 decode steps, same architecture and dtype."""
    from oracle import flashstu_oracle as O
    ocfg = O.OracleConfig(n_embd=768, n_heads=12, n_layers=12, seq_len=2048, window_size=512, vocab_size=50257,
                          mlp_scale=args.mlp_scale, num_eigh=24, dtype=torch.bfloat16)
    phi = torch.zeros(2048, 24, dtype=torch.bfloat16)       # filter values do not change the cost
    phi[:, :] = torch.linspace(0.1, 1.0, 24, dtype=torch.float32).bfloat16()
    w = O.init_weights(ocfg, seed=1, mode="reference", phi=phi)
    B, P, N = 8, 32, 6
    ids = torch.randint(0, 50257, (B, P), generator=torch.Generator().manual_seed(0))
    with torch.no_grad():
        st = O.DecodeState(w, ocfg, B)
        t0 = time.perf_counter()
        logits = st.prefill(ids)
        t_pre = time.perf_counter() - t0
        tok = logits[:, -1].argmax(-1)
        st.step(tok)                                   # warm-up step
        t0 = time.perf_counter()
        for _ in range(N):
            tok = st.step(tok)[:, -1].argmax(-1)
        t_dec = time.perf_counter() - t0
    return {"value": B * N / t_dec, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"CPU oracle, bf16, batch {B}, {P}-token prompt, {N} stateful decode steps "
                      f"(prefill {B * P / t_pre:.0f} tokens/s)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--mlp-scale", type=int, default=12, dest="mlp_scale")
    ap.add_argument("--stu-mode", default="lds", choices=["lds", "history"], dest="stu_mode")
    ap.add_argument("--stu-prefill", default="fft", choices=["fft", "scan"], dest="stu_prefill",
                    help="prompt pass of the STU layers: the reference's FFT convolution, or the distilled recurrence as a scan")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph-steps", type=int, default=8, dest="graph_steps",
                    help="decode steps captured per HIP graph (used when it divides --steps and --warmup)")
    ap.add_argument("--no-graph", action="store_true", help="launch every step kernel by kernel instead of replaying a HIP graph")
    ap.add_argument("--warm-wgs", type=int, default=-1, help="workgroups of the graph's cache warm-up branch (0 = off)")
    ap.add_argument("--pmc-calibrate", action="store_true", dest="pmc_calibrate",
                    help="also launch the library's plain 256 MiB copy kernel 4 times (reference for traffic counters)")
    ap.add_argument("--breakdown", action="store_true", help="time every kernel class with HIP events")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (decode shards by batch: every GPU would hold the full weights "
              "and its own sequences, with no exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import ctypes
    import torch
    from flash_stu import _hip
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    if args.warm_wgs >= 0:
        _hip._check(_hip.load().fstu_set_warm_workgroups(args.warm_wgs), "fstu_set_warm_workgroups")
    cfg, model = build_model(args, torch)
    B, P, K, W = args.batch, args.prompt, args.steps, args.warmup
    total = P + W + 2 * K + 8
    assert total <= cfg.seq_len or args.stu_mode == "lds"
    ids = torch.randint(0, cfg.vocab_size, (B, P), generator=torch.Generator().manual_seed(1)).cuda()
    eng = model.decode_engine()
    tokens = torch.zeros(B, total, dtype=torch.int64, device="cuda")
    tokens[:, :P] = ids
    # ---- prefill (untimed for `value`, reported on its own)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits = eng.prefill(ids, total)
    _hip.sample(logits, tokens[:, P], do_sample=False)
    torch.cuda.synchronize()
    t_prefill_cold = time.perf_counter() - t0
    warm = []
    for _ in range(5):          # warm prefill: median of five calls (the second call still loads code objects)
        t0 = time.perf_counter()
        logits = eng.prefill(ids, total)
        _hip.sample(logits, tokens[:, P], do_sample=False)
        torch.cuda.synchronize()
        warm.append(time.perf_counter() - t0)
    t_prefill = sorted(warm)[len(warm) // 2]
    # MFMA rate of the prefill's largest GEMM (the gate projection of the whole prompt through the library GEMM the
    # module path uses), timed with events on torch's stream
    gm, gn, gk = B * P, cfg.n_embd * cfg.mlp_scale, cfg.n_embd
    ga = torch.randn(gm, gk, device="cuda", dtype=torch.bfloat16)
    gw = model.layers[0].mlp.gate_proj.weight
    for _ in range(3):
        torch.matmul(ga, gw.t())
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        torch.matmul(ga, gw.t())
    e1.record()
    torch.cuda.synchronize()
    gemm_tflops = 2.0 * gm * gn * gk * 20 / (e0.elapsed_time(e1) * 1e-3) / 1e12
    del ga
    pos = P

    def run(n):
        nonlocal pos
        for _ in range(n):
            eng.step(tokens, pos, 1.0, None, None, False, 0, pos - P + 1)
            pos += 1

    use_graph = eng.graph_supported() and not args.no_graph
    if use_graph:
        # one decode step captured once; every replay reads its position from device memory
        S = args.graph_steps if (W % args.graph_steps == 0 and K % args.graph_steps == 0) else 1
        eng.graph_begin(tokens, pos, pos - P + 1, 1.0, None, None, False, 0, steps_per_graph=S)
        for _ in range(W // S):
            eng.graph_step()
        eng.graph_sync()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(K // S):
            eng.graph_step()
        eng.graph_sync()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        eng.graph_end()
        pos += W + K
    else:
        run(W)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(K)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    ms_per_step = dt / K * 1e3
    value = B * K / dt
    t_mid = P + W + K // 2
    S = cfg.stu_lds_state_dim
    step_bytes = decode_step_bytes(cfg, B, t_mid, args.stu_mode, S)
    lib = _hip.load()

    def timed_class(cls, n):
        nonlocal pos
        save = pos
        _hip._check(lib.fstu_prof_begin(cls, n * cfg.n_layers * 2 + 8), "fstu_prof_begin")
        run(n)
        ms, cnt = ctypes.c_double(), ctypes.c_int()
        _hip._check(lib.fstu_prof_end(ctypes.byref(ms), ctypes.byref(cnt)), "fstu_prof_end")
        pos = save
        return ms.value, cnt.value

    # ---- dominant kernel, timed live: the gate/up GLU projection of all 12 layers launched back to back on one
    # stream between two HIP events (the same kernel, weights and activations as inside the step; cycling through
    # the layers' 340 MB of gate/up weights keeps them from being served out of the 256 MB Infinity Cache).
    d, I = cfg.n_embd, cfg.n_embd * cfg.mlp_scale
    ms_c, n_c = ctypes.c_double(), ctypes.c_int()
    torch.cuda.synchronize()
    _hip._check(lib.fstu_prof_glu_loop(ctypes.byref(eng.desc), max(4, K // 8), ctypes.byref(ms_c), ctypes.byref(n_c),
                                       torch.cuda.current_stream().cuda_stream), "fstu_prof_glu_loop")
    glu_ms, glu_n = ms_c.value, n_c.value
    if args.pmc_calibrate:
        a_ = torch.zeros(256 << 20, dtype=torch.uint8, device="cuda")
        b_ = torch.empty_like(a_)
        for _ in range(4):
            _hip._check(lib.fstu_prof_copy(b_.data_ptr(), a_.data_ptr(), a_.numel(), torch.cuda.current_stream().cuda_stream),
                        "fstu_prof_copy")
        torch.cuda.synchronize()
    glu_bytes = 2 * I * d * 2 + B * d * 2 + B * I * 2          # gate+up weights, x in, act out (the fused prologue adds 3*B*d*2 + d*2 bytes: 0.1 %)
    glu_avg_us = glu_ms / glu_n * 1e3
    glu_gbps = glu_bytes / (glu_avg_us * 1e-6) / 1e9
    # HBM bytes per GLU launch from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE; each scaled by what the same
    # counter reads for the library's plain 256 MiB copy kernel: x2.000 and x1.000).  Measured offline for the default
    # workload only; summary and commands in profiles/glu_c2_hbm_traffic_pmc.txt.
    traffic = 28876800 if (cfg.n_embd, cfg.mlp_scale, B) == (768, 12, 8) else None
    out = {
        "metric": "decode tokens/sec at 1 GPU (768-d FlashSTU, bs=8) + achieved HBM GB/s",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE config 2: FlashSTU 768-d/12-layer/12-head, window 512, K=24, seq_len 2048, "
                               "vocab 50257, random-init bf16 seed 1, batch 8, 512-token prompt, greedy decode",
                   "mlp_scale": cfg.mlp_scale, "params": model.get_num_params(), "batch": B, "prompt": P,
                   "stu_decode_mode": args.stu_mode, "stu_prefill_mode": args.stu_prefill, "hip_graph": bool(use_graph), "stu_state_dim": S if args.stu_mode == "lds" else None},
        "roofline": {"bound": "hbm", "kernel": ("glu_balanced_kernel<PRO> (residual add + mlp_norm + gate/up projection + gelu*up)"
                                if getattr(eng.desc, "glu_packed", 0) and eng.desc.x2 else
                                "glu_balanced_kernel (gate/up projection + gelu*up)" if getattr(eng.desc, "glu_packed", 0)
                                else "linear_mfma_bf16_kernel<GLU> (gate/up projection + gelu*up)"),
                     "achieved": glu_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": glu_gbps / HBM_PEAK_GBPS,
                     "traffic": traffic, "bytes_per_launch": glu_bytes, "avg_launch_us": glu_avg_us,
                     "launches_timed": glu_n},
        "step_roofline": {"bound": "hbm", "bytes_per_step": step_bytes, "achieved": step_bytes / (ms_per_step * 1e-3) / 1e9,
                          "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                          "frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "prefill_tokens_per_s": B * P / t_prefill, "prefill_ms": t_prefill * 1e3, "prefill_first_call_ms": t_prefill_cold * 1e3,
        "prefill_gemm": {"what": "gate projection of the prompt, library GEMM (M, N, K)", "shape": [gm, gn, gk],
                         "achieved": gemm_tflops, "peak": 2500.0, "unit": "TFLOP/s", "frac": gemm_tflops / 2500.0},
    }
    if args.breakdown:
        names = {1: "glu", 2: "down", 3: "head", 4: "attention", 5: "stu_step", 6: "proj_qkv", 7: "embed_add_norm", 8: "sample"}
        n = min(K, 32)
        out["kernel_us_per_step"] = {names[c]: timed_class(c, n)[0] / n * 1e3 for c in names}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args, torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
