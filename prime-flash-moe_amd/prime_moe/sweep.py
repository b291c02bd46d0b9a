"""Token sweep of the fused op against torch baselines on the same GPU, written as CSV.

The counterpart of the reference's benchmark harness (benchmark/benchmark.py:393-547): for every
token count of the sweep, the fused op is timed next to
  * the grouped baseline: rows gathered in expert order -> ``torch.nn.functional.grouped_mm`` ->
    SwiGLU -> ``grouped_mm`` -> routing weight (dataflow of the reference's test/test.py:13-48 and
    benchmark.py:219-224; gather and scatter-add stay outside the timed region, as there), and
  * the naive per-expert loop (benchmark.py:191-200),
and the CSV has the reference's columns (benchmark.py:523-543).  The reference's mxfp8 baseline is
``scaled_grouped_mm`` with MX scales, which this ROCm build of torch does not provide for gfx950; the
mxfp8 rows therefore use the same bf16 grouped baseline on the dequantised operands (column
``baseline_kind`` says which), and ``noreq_ms`` stays empty.

Default grid = the reference's (benchmark.py:695-718): E=32, top_k=4, K=2048, H=1024,
tokens 4096 ... 131072, both dtypes, split=True, median of per-iteration event timings.  Like the
reference's, the run can be shaped from the command line (``bench.py --sweep``): experts, top_k, hidden and
intermediate size, ``balancedness`` of the routing (benchmark.py:116-121: every (token, slot) draws its
expert from ``b * uniform + (1 - b) * all-to-expert-0``, with replacement), seed, and whether the timed
callables are graph replays (benchmark.py:355-370, the reference's default) or eager calls.  A row never mixes
the two: if one of its callables cannot be captured (or its replay does not reproduce the eager result), every
callable of the row is timed eagerly, and the columns ``timed_as`` / ``timed_note`` say so and why.
"""
from __future__ import annotations

import csv
import math
import statistics
import sys
import warnings

import torch
import torch.nn.functional as F

import prime_moe

COLUMNS = ["dtype", "tokens", "E", "K", "N", "top_k", "naive_ms", "baseline_ms", "noreq_ms", "fused_ms", "speedup",
           "speedup_noreq", "speedup_naive", "naive_tflops", "baseline_tflops", "fused_tflops", "max_abs", "rel",
           "naive_max_abs", "baseline_kind", "split", "timed_as", "timed_note"]


def median_ms(fn, warmup: int, iters: int) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b))
    return statistics.median(times)


def capture_replay(fn, reproduces=None):
    """Records one call of `fn` in a HIP graph.  Returns (replay, None), or (None, reason) when the call cannot
    be recorded: it raises under capture (a host synchronisation, an allocation the capture forbids), it records
    nothing (torch warns of an empty graph: the work went to another stream), or `reproduces(replay)`, the
    caller's check that a replay gives what an eager call gives, says no."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    reason = None
    try:
        with torch.cuda.stream(stream):  # first calls outside the capture: lazy initialisation, allocator warm-up
            fn()
            fn()
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        with warnings.catch_warnings():
            warnings.simplefilter("error")  # "The CUDA Graph is empty" must not pass for a recording
            with torch.cuda.graph(graph):
                fn()
    except (RuntimeError, Warning) as exc:
        text = str(exc).strip()
        reason = f"{type(exc).__name__}: {text.splitlines()[0] if text else 'no message'}"
    torch.cuda.synchronize()
    if reason is None and reproduces is not None and not reproduces(graph.replay):
        reason = "a replay does not reproduce the eager result"
    return (graph.replay, None) if reason is None else (None, reason)


def generate_topk_ids(E: int, tokens: int, top_k: int, balancedness: float, gen: torch.Generator) -> torch.Tensor:
    """The reference benchmark's routing (benchmark.py:116-121): 1.0 = uniform, 0.0 = everything to expert 0;
    slots are drawn independently, so a token may name an expert twice."""
    dev = gen.device
    uniform = torch.ones(E, device=dev) / E
    skewed = torch.zeros(E, device=dev)
    skewed[0] = 1.0
    probs = balancedness * uniform + (1.0 - balancedness) * skewed
    return torch.multinomial(probs, tokens * top_k, replacement=True, generator=gen).view(tokens, top_k).to(torch.int32)


def grouped_inputs(x, topk_ids, topk_weights, E):
    """Rows in expert order (stable), their tokens, routing weights and the group ends."""
    top_k = topk_ids.shape[1]
    order = torch.argsort(topk_ids.flatten().long(), stable=True)
    tok = order // top_k
    counts = torch.bincount(topk_ids.flatten().long(), minlength=E)
    offs = torch.cumsum(counts, 0).to(torch.int32)
    wg = topk_weights.flatten()[order].to(torch.bfloat16)
    return x[tok].contiguous(), wg, offs, tok, counts.tolist()


def grouped_forward(xg, w1t, w2t, offs, wg):
    gate_up = F.grouped_mm(xg, w1t, offs=offs, out_dtype=torch.bfloat16)
    gate, up = gate_up.chunk(2, dim=-1)
    act = F.silu(gate) * up
    return wg.unsqueeze(1) * F.grouped_mm(act, w2t, offs=offs, out_dtype=torch.bfloat16)


def naive_forward(xg, w1, w2, counts, wg):
    out = torch.empty((xg.shape[0], w2.shape[1]), dtype=torch.bfloat16, device=xg.device)
    s = 0
    for e, c in enumerate(counts):
        if c:
            gate, up = (xg[s:s + c] @ w1[e].T).chunk(2, dim=-1)
            out[s:s + c] = wg[s:s + c].unsqueeze(1) * ((F.silu(gate) * up) @ w2[e].T)
        s += c
    return out


def run_one(dtype: str, tokens: int, E: int, K: int, H: int, top_k: int, split: bool, warmup: int, iters: int,
            check: bool, seed: int = 0, skip_naive: bool = False, balancedness: float = 1.0, graphs: bool = False,
            log=None) -> dict:
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(seed)
    N = 2 * H
    x = (torch.randn((tokens, K), device=dev, generator=g) * 0.05).to(torch.bfloat16)
    w1 = (torch.randn((E, N, K), device=dev, generator=g) * 0.05).to(torch.bfloat16)
    w2 = (torch.randn((E, K, H), device=dev, generator=g) * 0.05).to(torch.bfloat16)
    topk_ids = generate_topk_ids(E, tokens, top_k, balancedness, g)
    topk_weights = torch.softmax(torch.randn((tokens, top_k), device=dev, generator=g), -1)
    sched = torch.ops.prime_moe.moe_align(topk_ids, E, 128, 1)
    out = torch.zeros((tokens, K), dtype=torch.bfloat16, device=dev)
    kind = "grouped_mm bf16"
    if dtype == "bf16":
        def fused():
            return prime_moe.fused_moe_bf16(x, w1, w2, *sched, topk_weights, out, top_k, 128, 64, 4, 2, 1, 1, split)
        bx, bw1, bw2 = x, w1, w2
    else:
        xq, xs = prime_moe.quantize_mx(x)
        w1q, w1s = prime_moe.quantize_mx(w1)
        w2q, w2s = prime_moe.quantize_mx(w2)
        w1p, w2p = prime_moe.pack_scales_blocked(w1s), prime_moe.pack_scales_blocked(w2s)

        def fused():
            return prime_moe.fused_moe_mxfp8(xq, xs, w1q, w1p, w2q, w2p, *sched, topk_weights, out, top_k, 128, 64, 4, 4,
                                             1, split)

        def deq(q, s):  # e4m3 x 2^(e8m0 - 127), exact in bf16
            v = q.float().reshape(*q.shape[:-1], -1, 32) * torch.exp2(s.view(torch.uint8).float() - 127.0).unsqueeze(-1)
            return v.reshape(q.shape).to(torch.bfloat16)
        bx, bw1, bw2 = deq(xq, xs), deq(w1q, w1s), deq(w2q, w2s)
        kind = "grouped_mm bf16 on dequantised mxfp8 operands"
    step = fused if split else (lambda: (out.zero_(), fused()))
    xg, wg, offs, tok, counts = grouped_inputs(bx, topk_ids, topk_weights, E)
    w1t, w2t = bw1.transpose(1, 2), bw2.transpose(1, 2)
    baseline = lambda: grouped_forward(xg, w1t, w2t, offs, wg)
    try:
        baseline()
        torch.cuda.synchronize()
    except Exception as exc:  # this torch build has no grouped GEMM for the device: the loop is the baseline
        print(f"  note: grouped_mm unavailable ({type(exc).__name__}: {exc}); baseline = per-expert loop", file=sys.stderr)
        baseline = lambda: naive_forward(xg, bw1, bw2, counts, wg)
        kind = "per-expert loop"
    naive = lambda: naive_forward(xg, bw1, bw2, counts, wg)
    max_abs = rel = naive_max_abs = float("nan")
    if check:
        base_out = baseline()
        if not skip_naive:
            naive_max_abs = float((base_out.float() - naive().float()).abs().max())
        ref = torch.zeros_like(x).index_add_(0, tok, base_out)
        if not split:
            out.zero_()
        got = fused().float()
        torch.cuda.synchronize()
        diff = (ref.float() - got).abs()
        max_abs, rel = float(diff.max()), float((diff / ref.float().abs().clamp_min(1.0)).max())
    timed = {"baseline": baseline, "naive": naive, "fused": step}
    timed_as, timed_note = "eager", ""
    if graphs:
        def fused_reproduces(replay):
            # one replay must rewrite a poisoned `out` to the bits of an eager call
            step()
            torch.cuda.synchronize()
            want = out.clone()
            out.fill_(float("nan"))
            replay()
            torch.cuda.synchronize()
            return bool(torch.equal(out.view(torch.int16), want.view(torch.int16)))

        replays, why = {}, []
        for name in ("baseline", "fused") + (() if skip_naive else ("naive",)):
            replays[name], reason = capture_replay(timed[name], fused_reproduces if name == "fused" else None)
            if reason is not None:
                why.append(f"{name}: {reason}")
        if why:  # never a replayed callable next to an eager one
            timed_note = "graph replays asked for, all callables timed eagerly; " + "; ".join(why)
            if log is not None:
                log("  note: " + timed_note)
        else:
            timed.update(replays)
            timed_as = "replay"
    baseline_ms = median_ms(timed["baseline"], warmup, iters)
    naive_ms = float("nan") if skip_naive else median_ms(timed["naive"], warmup, iters)
    fused_ms = median_ms(timed["fused"], warmup, iters)
    flops = 3.0 * tokens * top_k * K * N  # reference's model, benchmark.py:389-391
    tf = lambda ms: flops / (ms * 1e-3) / 1e12
    return {"dtype": dtype, "tokens": tokens, "E": E, "K": K, "N": N, "top_k": top_k, "naive_ms": naive_ms,
            "baseline_ms": baseline_ms, "noreq_ms": float("nan"), "fused_ms": fused_ms, "speedup": baseline_ms / fused_ms,
            "speedup_noreq": float("nan"), "speedup_naive": naive_ms / fused_ms, "naive_tflops": tf(naive_ms),
            "baseline_tflops": tf(baseline_ms), "fused_tflops": tf(fused_ms), "max_abs": max_abs, "rel": rel,
            "naive_max_abs": naive_max_abs, "baseline_kind": kind, "split": int(split), "timed_as": timed_as,
            "timed_note": timed_note}


def run_sweep(path: str, tokens=(4096, 8192, 16384, 32768, 65536, 131072), dtypes=("bf16", "mxfp8"), E=32, top_k=4,
              K=2048, H=1024, split=True, warmup=10, iters=50, check=True, log=print, seed=0, balancedness=1.0,
              graphs=False, skip_naive=False):
    rows = []
    for dtype in dtypes:
        for t in tokens:
            r = run_one(dtype, t, E, K, H, top_k, split, warmup, iters, check, seed=seed, skip_naive=skip_naive,
                        balancedness=balancedness, graphs=graphs, log=log)
            rows.append(r)
            log(f"{dtype:6s} tokens {t:7d}: fused {r['fused_ms']:8.3f} ms ({r['fused_tflops']:7.1f} TFLOP/s)  "
                f"{r['baseline_kind']} {r['baseline_ms']:8.3f} ms  speedup {r['speedup']:.2f}x  "
                f"naive loop {r['naive_ms']:8.3f} ms  max_abs {r['max_abs']:.3g} rel {r['rel']:.3g}"
                + f"  ({r['timed_as']})")
            torch.cuda.empty_cache()
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=COLUMNS)
        w.writeheader()
        for r in rows:
            w.writerow({k: (f"{v:.6g}" if isinstance(v, float) and not math.isnan(v) else ("" if isinstance(v, float) else v))
                        for k, v in r.items()})
    return rows
