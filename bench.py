#!/usr/bin/env python3
"""Benchmark of the fused-MoE forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME] [--split 0|1] [--headline-only]
    python bench.py --sweep [--sweep-out FILE.csv]

A "step" is one call of the fused op over one batch of synthetic input that is already
resident in HBM (routing, moe_align and quantisation happen before the timed region, as in the
reference's benchmark/benchmark.py:19-22).  The headline workload is the Mixtral-8x7B-like bf16
prefill shape with split=True.  The last line printed is one JSON object: whole-op throughput
(`value`), the roofline figure of the dominant kernel measured with HIP events in this run, the
CPU oracle timed on the host cores on a bounded sample of the same workload, and `config.all`: the
same measurements (time, TFLOP/s, GB/s, % of roofline, per-kernel times) for every benchmark
configuration and both values of `split` where the specification names both, taken before the
headline run (`--headline-only` skips them), plus the router front-end next to the unfused sequence.

`--sweep` runs the reference benchmark's token sweep against torch's grouped GEMM on this GPU and
writes a CSV with the reference's columns (prime_moe/sweep.py); it takes the reference benchmark's
knobs (--sweep-tokens, --sweep-dtypes, --experts, --top-k, --hidden, --inter, --balancedness, --seed,
--graphs, --skip-naive).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "prime-flash-moe_amd"))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

# MI355X published dense peaks
PEAK_TFLOPS = {"bf16": 2500.0, "mxfp8": 5000.0}
PEAK_HBM_GBS = 8000.0

PHASE_PROLOGUE, PHASE_UP, PHASE_DOWN, PHASE_FINALIZE, PHASE_ALL = 1, 2, 4, 8, 15


def build_case(cfg, device, seed=0):
    import prime_moe  # noqa: F401
    from prime_moe.workloads import make_inputs
    inp = make_inputs(cfg, device, seed=seed, keep_row_major_scales=cfg.dtype != "bf16")  # (for the CPU leg)
    sched = torch.ops.prime_moe.moe_align(inp["topk_ids"], cfg.E, cfg.block_m, 1)
    out = torch.zeros((cfg.T, cfg.K), dtype=torch.bfloat16, device=device)
    return inp, sched, out


def make_step(cfg, inp, sched, out, split):
    import prime_moe
    if cfg.dtype == "bf16":
        def op():
            prime_moe.fused_moe_bf16(inp["x"], inp["w1"], inp["w2"], *sched, inp["topk_weights"], out,
                                     cfg.top_k, cfg.block_m, 64, 4, 2, 1, 1, split)
    else:
        def op():
            prime_moe.fused_moe_mxfp8(inp["x"], inp["x_scales"], inp["w1"], inp["w1_scales"], inp["w2"],
                                      inp["w2_scales"], *sched, inp["topk_weights"], out, cfg.top_k,
                                      cfg.block_m, 64, 4, 2, 1, split)
    if split:
        return op

    def step():  # the fused pipeline accumulates into `out`: zeroing it is part of the step
        out.zero_()
        op()
    return step


def time_steps(step, steps, warmup):
    """Wall clock over exactly `steps` calls, synchronised on both sides; returns seconds/step.

    The default of 20 warm-up calls is not caution: after the set-up work the first call runs at the
    boost clock, the next few under a power controller that overshoots (the Qwen3-like shape goes
    753 -> 963 us), and the time settles over about 20 calls (790 us)."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def time_events(step, steps):
    """Average duration of `step` from HIP events recorded on the stream the kernels run on."""
    start = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stop = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    for i in range(steps):
        start[i].record()
        step()
        stop[i].record()
    torch.cuda.synchronize()
    ms = sorted(s.elapsed_time(e) for s, e in zip(start, stop))
    return sum(ms) / len(ms) * 1e-3, ms[len(ms) // 2] * 1e-3


def phase_time(step, mask, steps, inner=1):
    """Duration of the kernels that `mask` leaves of one call, from replays of a HIP graph captured under that mask
    (the mask acts when the kernels are enqueued, that is at capture): the time of the kernels themselves, without
    the host's launch path, which at a few tens of microseconds per call would drown the small shapes."""
    from prime_moe import _native
    lib = _native.load()
    lib.pmoe_set_phase_mask(mask)
    try:
        return graph_time(step, steps, inner)
    finally:
        lib.pmoe_set_phase_mask(PHASE_ALL)


def graph_time(step, replays=20, inner=1):
    """Median duration of `step` in a replayed HIP graph (the reference benchmark's method,
    benchmark/benchmark.py:355-386): what the call costs without the host's launch path.  `inner` calls are
    captured back to back in one graph, so that replays of very short calls measure the GPU and not the launch of
    the graph."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(inner):
            step()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    return time_events(graph.replay, replays)[1] / inner


def recorded_traffic(config: str, kernel: str = "moe_up_kernel"):
    """HBM-side bytes per launch of `kernel` on `config` as the last counter run recorded them in
    profiles/kernel_figures.txt (written by prime_moe/profiling.py: FETCH_SIZE + WRITE_SIZE of two
    rocprofv3 --pmc runs, scaled by a plain copy of known size).  A counter run cannot share a process
    with the timed run, so the line carries the recorded figure and says where it comes from."""
    path = os.path.join(ROOT, "profiles", "kernel_figures.txt")
    try:
        for line in open(path):
            f = line.split()
            if len(f) >= 8 and f[0] == config and f[1] == kernel:
                kv = dict(zip(f[2::2], f[3::2]))
                return float(kv["fetch_bytes"]) + float(kv["write_bytes"]), float(kv.get("mfma_busy", "nan"))
    except OSError:
        pass
    return None, None


def hbm_bytes(cfg, inp):
    """Algorithmic bytes of one call: weights (+scales) of the touched experts, x, out, routing."""
    from prime_moe.workloads import touched_weight_bytes
    wb = touched_weight_bytes(cfg, inp["topk_ids"])
    xb = cfg.T * cfg.K * (2 if cfg.dtype == "bf16" else 1 + 1 / 32)
    return wb, int(wb + xb + cfg.T * cfg.K * 2 + cfg.T * cfg.top_k * 8)


def cpu_baseline_mx(cfg, inp, cores):
    """mxfp8 leg of the CPU baseline: the oracle's dataflow (dequantise, fp32 GEMMs, SwiGLU, activation
    quantise->dequantise, down GEMM, weighted sum) expert by expert over the routed rows of the first
    experts, as many as about ten seconds of CPU work take (one expert's weights are dequantised at a
    time, so the sample needs well under 1 GB)."""
    from oracle import moe_oracle as O
    ids = inp["topk_ids"].cpu()
    wts = inp["topk_weights"].cpu()
    xq, xs = inp["x"].cpu(), inp["x_scales"].cpu().view(torch.uint8)
    H = cfg.H
    flops, wbytes, rows_done, n_e = 0.0, 0, 0, 0
    t0 = time.perf_counter()
    acc = torch.zeros((cfg.T, cfg.K), dtype=torch.float32)
    for e in range(cfg.E):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        w1 = O.dequantize_mx_torch(inp["w1"][e].cpu(), inp["w1_scales_rm"][e].cpu())
        w2 = O.dequantize_mx_torch(inp["w2"][e].cpu(), inp["w2_scales_rm"][e].cpu())
        x = O.dequantize_mx_torch(xq[tok], xs[tok])
        h = x @ w1.t()
        act = O.swiglu(h[:, :H], h[:, H:])
        aq, asc = O.quantize_mx_torch(act)
        y = O.dequantize_mx_torch(aq, asc) @ w2.t()
        acc.index_add_(0, tok, y * wts[tok, slot].unsqueeze(1))
        flops += 3.0 * tok.numel() * cfg.K * cfg.N
        wbytes += cfg.weight_bytes_per_expert()
        rows_done += tok.numel()
        n_e += 1
        if time.perf_counter() - t0 >= 10.0:
            break
    dt = time.perf_counter() - t0
    sample = (f"the {rows_done} routed rows of the first {n_e} experts with tokens (of {cfg.E}), fp32 torch oracle on "
              f"dequantised operands, {dt:.1f} s of CPU time on the clock")
    if cfg.name.startswith("c5"):
        return {"value": wbytes / dt / 1e9, "unit": "GB/s", "cores": cores, "kind": "port", "sample": sample}, None
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port", "sample": sample}, None


def cpu_baseline(cfg, inp, gpu_out, budget_tokens):
    """The CPU oracle (fp32 torch on the host cores) on the first `budget_tokens` tokens."""
    from oracle import moe_oracle as O
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    if cfg.dtype != "bf16":
        return cpu_baseline_mx(cfg, inp, cores)
    n = min(cfg.T, budget_tokens)
    ids = inp["topk_ids"][:n].cpu()
    wts = inp["topk_weights"][:n].cpu()
    x, w1, w2 = inp["x"][:n].cpu(), inp["w1"].cpu(), inp["w2"].cpu()
    run = lambda: O.fused_moe_dense(x, w1, w2, ids, wts)
    O.fused_moe_dense(x[:32], w1, w2, ids[:32], wts[:32])  # warm-up (thread pool, page faults)
    passes, t0 = 0, time.perf_counter()
    while True:  # whole passes over the sample until about ten seconds of CPU work are on the clock
        ref = run()
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= 10.0 or passes >= 50:
            break
    flops = 3.0 * n * cfg.top_k * cfg.K * cfg.N * passes
    err = None
    if gpu_out is not None:
        got = gpu_out[:n].float().cpu()
        err = float(((got - ref).abs() / ref.abs().clamp_min(1.0)).max())
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{passes} passes over the first {n} of {cfg.T} tokens through all {cfg.E} experts, "
                      f"fp32 torch oracle, {dt:.1f} s of CPU time on the clock"}, err


def run_config(cfg, split, steps, warmup, device, with_cpu, log):
    inp, sched, out = build_case(cfg, device)
    step = make_step(cfg, inp, sched, out, split)
    sec = time_steps(step, steps, warmup)
    ev_mean, ev_med = time_events(step, steps)
    # the part of the prologue that builds the schedule runs whatever the mask: it is timed alone and taken off
    # the two kernels' times, so that they are the kernels' own
    inner = 8 if sec < 200e-6 else 1
    t_plan = phase_time(step, 0, steps, inner)
    t_up = max(phase_time(step, PHASE_UP, steps, inner) - t_plan, 1e-9)
    t_down = max(phase_time(step, PHASE_DOWN, steps, inner) - t_plan, 1e-9)
    t_graph = graph_time(step, steps, inner)
    step()
    torch.cuda.synchronize()
    P = cfg.T * cfg.top_k
    flops_up = 2.0 * P * cfg.K * cfg.N
    flops_down = 1.0 * P * cfg.K * cfg.N
    wb, total_b = hbm_bytes(cfg, inp)
    peak = PEAK_TFLOPS[cfg.dtype]
    res = {
        "name": cfg.name, "split": bool(split), "sec": sec, "ev_mean": ev_mean, "ev_med": ev_med,
        "t_up": t_up, "t_down": t_down, "t_graph": t_graph, "tflops": cfg.flops / sec / 1e12,
        "pct_mfma": 100 * cfg.flops / sec / 1e12 / peak, "weight_gbs": wb / sec / 1e9,
        "pct_hbm": 100 * total_b / sec / 1e9 / PEAK_HBM_GBS, "weight_bytes": wb, "bytes": total_b,
        "up_tflops": flops_up / t_up / 1e12 if t_up else 0.0,
        "down_tflops": flops_down / t_down / 1e12 if t_down else 0.0, "topk_ids": inp["topk_ids"],
    }
    log(f"{cfg.name:18s} split={int(split)}  {sec * 1e6:10.1f} us/call  {res['tflops']:8.1f} TFLOP/s "
        f"({res['pct_mfma']:5.1f}% {cfg.dtype} MFMA peak)  weights {res['weight_gbs']:7.1f} GB/s  "
        f"all-bytes {res['pct_hbm']:5.1f}% of 8 TB/s | up {t_up * 1e6:9.1f} us ({res['up_tflops']:7.1f} TF) "
        f"down {t_down * 1e6:9.1f} us ({res['down_tflops']:7.1f} TF) | graph replay {t_graph * 1e6:9.1f} us")
    # algorithmic bytes of one launch of each kernel: weights (+ scales) of the touched experts once, the routed
    # rows of the token-side operand once, the output written once
    sx = 2 if cfg.dtype == "bf16" else 33 / 32
    n_touched = wb / cfg.weight_bytes_per_expert()
    alg = {"moe_up_kernel": n_touched * cfg.N * cfg.K * sx + P * cfg.K * sx + P * cfg.H * sx,
           "moe_down_kernel": n_touched * cfg.K * cfg.H * sx + P * cfg.H * sx + P * cfg.K * 2,
           "finalize_kernel": P * cfg.K * 2 + cfg.T * cfg.K * 2}
    res["algorithmic_bytes"] = alg
    log("  algorithmic bytes per launch: " + " ".join(f"{k} {v:.0f}" for k, v in alg.items()))
    cpu, err = (None, None)
    if with_cpu:
        cpu, err = cpu_baseline(cfg, inp, out, budget_tokens=4096)
        log(f"  cpu oracle: {cpu['value']:.3f} {cpu['unit']} on {cpu['cores']} cores ({cpu['sample']})"
            + (f"; GPU vs oracle rel_clamp_1 = {err:.3g}" if err is not None else ""))
    res["cpu"], res["parity"] = cpu, err
    return res


def router_times(device, steps):
    """The router front-end (top-k + softmax + moe_align, prime_moe.route) next to the unfused torch
    sequence in front of the moe_align op, on the gate logits of the Qwen3-like configuration."""
    import prime_moe
    from prime_moe.workloads import CONFIGS
    cfg = CONFIGS["c3_qwen3_bf16"]
    g = torch.Generator(device=device).manual_seed(0)
    logits = torch.randn((cfg.T, cfg.E), generator=g, device=device)

    def unfused():
        vals, ids = torch.topk(logits, cfg.top_k, dim=-1)
        w = torch.softmax(vals.float(), dim=-1)
        return (ids.to(torch.int32), w) + tuple(torch.ops.prime_moe.moe_align(ids.to(torch.int32), cfg.E, cfg.block_m, 1))

    fused = lambda: prime_moe.route(logits, cfg.top_k, cfg.block_m, 1)
    out = {}
    for name, fn in (("fused_us", fused), ("unfused_us", unfused)):
        for _ in range(5):
            fn()
        out[name] = time_events(fn, steps)[1] * 1e6
    out["workload"] = f"gate logits ({cfg.T}, {cfg.E}) fp32, top_k={cfg.top_k}, block_m=128"
    return out


def summary(r):
    """One entry of `config.all`."""
    return {"config": r["name"], "split": r["split"], "us_per_call": round(r["sec"] * 1e6, 1),
            "tflops": round(r["tflops"], 1), "pct_mfma_peak": round(r["pct_mfma"], 2),
            "weight_gbs": round(r["weight_gbs"], 1), "pct_hbm_all_bytes": round(r["pct_hbm"], 2),
            "graph_us_per_call": round(r["t_graph"] * 1e6, 1),
            "up_kernel_us": round(r["t_up"] * 1e6, 1), "down_kernel_us": round(r["t_down"] * 1e6, 1),
            "other_us": round((r["ev_mean"] - r["t_up"] - r["t_down"]) * 1e6, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="c2_mixtral_bf16")
    ap.add_argument("--split", type=int, default=1)
    ap.add_argument("--headline-only", action="store_true",
                    help="time only --config (skips the other configurations and the router)")
    ap.add_argument("--all", action="store_true", help="(accepted for compatibility: every configuration is timed by default)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU oracle leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (a kernel of known traffic, to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run); implies --headline-only")
    ap.add_argument("--sweep", action="store_true", help="token sweep against torch's grouped GEMM, CSV output")
    ap.add_argument("--sweep-out", default=os.path.join(ROOT, "gpurun_out", "sweep.csv"))
    ap.add_argument("--sweep-tokens", type=int, nargs="+", default=[4096, 8192, 16384, 32768, 65536, 131072])
    # the reference benchmark's knobs (benchmark/benchmark.py:695-721), for --sweep only
    ap.add_argument("--sweep-dtypes", nargs="+", choices=["bf16", "mxfp8"], default=["bf16", "mxfp8"])
    ap.add_argument("--experts", type=int, default=32)
    ap.add_argument("--top-k", type=int, default=4)
    ap.add_argument("--hidden", type=int, default=2048, help="K, the model dim")
    ap.add_argument("--inter", type=int, default=1024, help="per expert intermediate dim H; w1 has N = 2H rows")
    ap.add_argument("--balancedness", type=float, default=1.0, help="1.0 = uniform routing, 0.0 = everything to expert 0")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--graphs", action=argparse.BooleanOptionalAction, default=False,
                    help="time graph replays instead of eager calls (the reference's --cuda-graphs)")
    ap.add_argument("--skip-naive", action="store_true", help="skip the per-expert loop baseline")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (the path is single-device, "
                 "there is no collective to scale)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from prime_moe.workloads import CONFIGS
    device = torch.device("cuda:0")
    log = lambda *a: print(*a, file=sys.stderr, flush=True)
    log(f"device: {torch.cuda.get_device_name(0)}; peaks used: bf16 {PEAK_TFLOPS['bf16']} / "
        f"mxfp8 {PEAK_TFLOPS['mxfp8']} TFLOP/s dense, HBM {PEAK_HBM_GBS} GB/s")
    if args.sweep:
        from prime_moe.sweep import run_sweep
        os.makedirs(os.path.dirname(os.path.abspath(args.sweep_out)), exist_ok=True)
        rows = run_sweep(args.sweep_out, tokens=tuple(args.sweep_tokens), dtypes=tuple(args.sweep_dtypes), E=args.experts,
                         top_k=args.top_k, K=args.hidden, H=args.inter, warmup=min(args.warmup, 10), iters=args.steps,
                         log=log, seed=args.seed, balancedness=args.balancedness, graphs=args.graphs,
                         skip_naive=args.skip_naive)
        print(json.dumps({"sweep_csv": args.sweep_out, "rows": len(rows),
                          "speedup_min": min(r["speedup"] for r in rows), "speedup_max": max(r["speedup"] for r in rows)}))
        return
    if args.calibrate_copy:
        from prime_moe import _native
        src = torch.empty(1 << 28, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):  # copy_calibration_kernel: reads 1 GiB, writes 1 GiB
            _native.check(_native.load().pmoe_copy_calibration(src.data_ptr(), dst.data_ptr(), src.numel() * 4,
                                                               torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    everything, router = [], None
    if not (args.headline_only or args.calibrate_copy or args.config != "c2_mixtral_bf16" or args.split != 1):
        # every configuration, both pipelines where the specification names both; also brings the chip to
        # its steady clocks before the headline run
        for name, cfg in CONFIGS.items():
            for split in ((1, 0) if name.startswith(("c2", "c5")) else (1,)):
                if name == args.config and split == args.split:
                    continue
                everything.append(summary(run_config(cfg, split, args.steps, args.warmup, device, False, log)))
                torch.cuda.empty_cache()
        from prime_moe.workloads import GRID_CONFIGS
        for cfg in GRID_CONFIGS.values():
            everything.append(summary(run_config(cfg, 1, args.steps, args.warmup, device, False, log)))
            torch.cuda.empty_cache()
        router = router_times(device, 20)
        log(f"router front-end on {router['workload']}: fused {router['fused_us']:.1f} us, "
            f"torch top-k + softmax + moe_align op {router['unfused_us']:.1f} us")
    cfg = CONFIGS[args.config]
    r = run_config(cfg, args.split, args.steps, args.warmup, device,
                   with_cpu=not args.no_cpu, log=log)
    everything.insert(0, summary(r))
    memory_bound = cfg.name.startswith("c5")
    if cfg.dtype != "bf16":
        # the mxfp8 shapes stream every touched weight once (arithmetic intensity below the ridge): the up
        # kernel, the longer of the two, against HBM.  Algorithmic bytes of one launch: W1 and its scales
        # of the touched experts, the routed x rows and their scales once, the activation written.
        P = cfg.T * cfg.top_k
        n_touched = int(torch.unique(r["topk_ids"]).numel())
        up_bytes = (n_touched * cfg.N * cfg.K + P * cfg.K + P * cfg.H) * 33 // 32
        roofline = {"bound": "hbm", "achieved": up_bytes / r["t_up"] / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "kernel": "moe_up_kernel<1> (mxfp8 gate/up GEMM + SwiGLU + requantisation)",
                    "launch_us": r["t_up"] * 1e6, "bytes_per_launch": up_bytes}
    else:
        P = cfg.T * cfg.top_k
        roofline = {"bound": "mfma", "achieved": 2.0 * P * cfg.K * cfg.N / r["t_up"] / 1e12,
                    "peak": PEAK_TFLOPS[cfg.dtype], "unit": "TFLOP/s",
                    "kernel": "moe_up_kernel_bf16 (gate/up GEMM + SwiGLU)", "launch_us": r["t_up"] * 1e6}
    roofline["frac"] = roofline["achieved"] / roofline["peak"]
    traffic, mfma_busy = recorded_traffic(cfg.name)  # the kernels do not depend on --split
    roofline["traffic"] = traffic
    roofline["traffic_source"] = ("profiles/kernel_figures.txt (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of an earlier run of "
                                  "this workload, prime_moe/profiling.py)") if traffic is not None else None
    roofline["mfma_busy_recorded"] = mfma_busy
    # the per-configuration table once more as flat keys (config.<name>.split<0|1>.<figure>), for readers that keep
    # only the scalar members of `config`
    flat = {}
    for e in everything:
        for k, v in e.items():
            if k not in ("config", "split"):
                flat[f"{e['config']}.split{int(e['split'])}.{k}"] = v
    line = {
        "metric": "Fused-MoE TFLOP/s & % MFMA peak (bf16/mxfp8); decode-shape HBM GB/s",
        "value": r["weight_gbs"] if memory_bound else r["tflops"],
        "unit": "GB/s" if memory_bound else "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": r["sec"] * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": cfg.dtype, "data": "synthetic",
        "config": {"workload": f"{cfg.name}: T={cfg.T} K={cfg.K} E={cfg.E} N={cfg.N} top_k={cfg.top_k} "
                               f"block_m=128 split={bool(args.split)}",
                   "flops_per_step": cfg.flops, "pct_mfma_peak": r["pct_mfma"],
                   "weight_gbs": r["weight_gbs"], "parity_rel_clamp_1": r["parity"],
                   **flat, "all": everything, "router": router},
        "roofline": roofline,
        "cpu_baseline": r["cpu"],
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
