"""rocprofv3 summaries of the fused-MoE pipeline on one benchmark configuration.

    python prime-flash-moe_amd/prime_moe/profiling.py --config c2_mixtral_bf16 [--split 1] [--out profiles]

Run from the repository root on a machine with the GPU.  Five profiler runs of ``bench.py`` on the same
workload, each a process of its own (the counter runs cannot share a process with a timed run):

  1. ``--kernel-trace --stats``                     average duration of every kernel
  2. ``--pmc FETCH_SIZE``  (+ ``--calibrate-copy``)  bytes fetched past the per-XCD L2s, per dispatch
  3. ``--pmc WRITE_SIZE``  (+ ``--calibrate-copy``)  bytes written past them
  4. ``--pmc`` eight SQ counters                    matrix-pipe busy cycles, LDS activity and conflicts, waits
  5. ``--pmc`` four L2 (TCC) counters               reads past L2: requests, summed queue level, DRAM credit stalls

``--calibrate-copy`` adds launches of a plain 1 GiB copy kernel whose known traffic scales the two
size counters.  The script writes ``<out>/split_pipeline_<config>.md`` (the commands, the raw per-kernel
figures, the derived table) and replaces the config's lines in ``<out>/kernel_figures.txt``, the small
table ``bench.py`` reads its ``roofline.traffic`` from:

    <config> <kernel> avg_us <float> fetch_bytes <int> write_bytes <int> mfma_busy <float> lds_conflict <float>
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
KERNELS = ("moe_up_kernel", "moe_up_join_kernel", "moe_down_kernel", "finalize_kernel", "moe_prologue_kernel",
           "copy_calibration_kernel")
SQ_COUNTERS = ["SQ_BUSY_CYCLES", "SQ_VALU_MFMA_BUSY_CYCLES", "SQ_INSTS_VALU_MFMA_MOPS_{DT}", "SQ_LDS_BANK_CONFLICT",
               "SQ_ACTIVE_INST_LDS", "SQ_WAIT_INST_LDS", "SQ_WAVE_CYCLES", "SQ_WAIT_ANY"]
EA_COUNTERS = ["TCC_EA0_RDREQ_sum", "TCC_EA0_RDREQ_LEVEL_sum", "TCC_EA0_RDREQ_DRAM_CREDIT_STALL_sum", "TCC_BUSY_sum"]
GIB_KIB = 1048576.0


def short(name: str) -> str:
    for k in KERNELS:
        if k in name:
            return k
    return ""


def run_pass(tag, prof_args, bench_args, workdir, log):
    out_dir = os.path.join(workdir, tag)
    shutil.rmtree(out_dir, ignore_errors=True)
    cmd = ["rocprofv3", *prof_args, "-d", out_dir, "-o", "out", "--output-format", "csv", "--",
           "python3", os.path.join(ROOT, "bench.py"), *bench_args]
    log.append(" ".join(cmd).replace(ROOT, "$R").replace(workdir.replace(ROOT, "$R"), "$R/gpurun_out/prof"))
    env = dict(os.environ, TMPDIR="/tmp")
    res = subprocess.run(["timeout", "-s", "KILL", "240", *cmd], cwd="/tmp", env=env, capture_output=True, text=True)
    if res.returncode != 0:
        sys.exit(f"profiler pass {tag} failed (rc {res.returncode}):\n{res.stdout[-2000:]}\n{res.stderr[-2000:]}")
    lines = res.stderr.splitlines() + res.stdout.splitlines()
    bench_line = [l for l in lines if l[:2] in ("c1", "c2", "c3", "c4", "c5")]
    alg = [l for l in lines if "algorithmic bytes per launch:" in l]
    algorithmic = {}
    if alg:
        f = alg[-1].split(":", 1)[1].split()
        algorithmic = {f[i]: float(f[i + 1]) for i in range(0, len(f) - 1, 2)}
    return out_dir, (bench_line[-1] if bench_line else ""), algorithmic


def kernel_stats(out_dir):
    stats = {}
    for f in glob.glob(os.path.join(out_dir, "**", "*kernel_stats.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            k = short(r["Name"])
            if k:
                stats[k] = dict(calls=int(r["Calls"]), avg_ns=float(r["AverageNs"]), min_ns=float(r["MinNs"]),
                                max_ns=float(r["MaxNs"]))
    return stats


def counters(out_dir):
    """kernel -> counter -> (mean per dispatch, dispatches)"""
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    for f in glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            k = short(r["Kernel_Name"])
            if k:
                agg[k][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return {k: {c: (sum(v) / len(v), len(v)) for c, v in d.items()} for k, d in agg.items()}


def simds_per_shader_engine(out_dir) -> float:
    """SIMD count / shader engine count of the GPU agent, from the profiler's agent table (MI355X: 1024 / 32)."""
    for f in glob.glob(os.path.join(out_dir, "**", "*agent_info.csv"), recursive=True):
        for r in csv.DictReader(open(f)):
            try:
                if int(r.get("Simd_Count", 0)) > 0 and int(r.get("Num_Shader_Banks", 0)) > 0:
                    return int(r["Simd_Count"]) / int(r["Num_Shader_Banks"])
            except ValueError:
                pass
    return 32.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", required=True)
    ap.add_argument("--split", type=int, default=1)
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles"))
    ap.add_argument("--workdir", default=os.path.join(ROOT, "gpurun_out", "prof"))
    a = ap.parse_args()
    sys.path.insert(0, os.path.join(ROOT, "prime-flash-moe_amd"))
    dt = "bf16" if "bf16" in a.config else "mxfp8"
    sq = [c.replace("{DT}", "BF16" if dt == "bf16" else "F8") for c in SQ_COUNTERS]
    common = ["--no-cpu", "--headline-only", "--config", a.config, "--split", str(a.split)]
    cmds = []
    d_stats, bench_line, algorithmic = run_pass("stats", ["--kernel-trace", "--stats"], ["--steps", "10", "--warmup", "3", *common],
                                   a.workdir, cmds)
    d_fetch, _, _ = run_pass("fetch", ["--pmc", "FETCH_SIZE"], ["--steps", "3", "--warmup", "1", "--calibrate-copy", *common],
                          a.workdir, cmds)
    d_write, _, _ = run_pass("write", ["--pmc", "WRITE_SIZE"], ["--steps", "3", "--warmup", "1", "--calibrate-copy", *common],
                          a.workdir, cmds)
    d_sq, _, _ = run_pass("sq", ["--pmc", *sq], ["--steps", "3", "--warmup", "1", *common], a.workdir, cmds)
    d_ea, _, _ = run_pass("ea", ["--pmc", *EA_COUNTERS], ["--steps", "3", "--warmup", "1", *common], a.workdir, cmds)
    stats, fetch, write, sqc = kernel_stats(d_stats), counters(d_fetch), counters(d_write), counters(d_sq)
    eac = counters(d_ea)
    cal_f = fetch.get("copy_calibration_kernel", {}).get("FETCH_SIZE", (GIB_KIB, 0))[0]
    cal_w = write.get("copy_calibration_kernel", {}).get("WRITE_SIZE", (GIB_KIB, 0))[0]
    f_scale, w_scale = GIB_KIB / cal_f, GIB_KIB / cal_w
    simds_per_se = simds_per_shader_engine(d_sq)

    lines = [f"# rocprofv3 summary: fused-MoE pipeline, {a.config}", "",
             f"Workload `{a.config}` of `prime_moe/workloads.py`, `split={bool(a.split)}`, one MI355X.  Written by",
             f"`python prime-flash-moe_amd/prime_moe/profiling.py --config {a.config} --split {a.split}`, which runs (from `/tmp`,",
             "`TMPDIR=/tmp`, `$R` = repository root):", ""]
    lines += ["    " + c for c in cmds]
    lines += ["", "`--calibrate-copy` adds launches of `copy_calibration_kernel`, a plain copy that reads 1 GiB and writes 1 GiB:",
              f"FETCH_SIZE reads {cal_f:,.0f} KiB for it (scale factor {f_scale:.2f}), WRITE_SIZE {cal_w:,.0f} KiB (scale factor {w_scale:.2f}).",
              "", "bench.py's own line of the traced run (profiler attached):", "", "    " + bench_line, "",
              "## Per kernel (means per dispatch)", "",
              "| kernel | avg duration | fetched past L2 | written past L2 | sum | algorithmic bytes | rate | MFMA busy | LDS conflict cycles / LDS active | waiting on LDS | read latency past L2 | DRAM credit stalls |",
              "|---|---|---|---|---|---|---|---|---|---|---|---|"]
    figs = []
    for k in KERNELS[:5]:
        if k not in stats:
            continue
        us = stats[k]["avg_ns"] / 1e3
        fb = fetch.get(k, {}).get("FETCH_SIZE", (0.0, 0))[0] * 1024 * f_scale
        wb = write.get(k, {}).get("WRITE_SIZE", (0.0, 0))[0] * 1024 * w_scale
        c = {n: v[0] for n, v in sqc.get(k, {}).items()}
        busy = c.get("SQ_BUSY_CYCLES", 0.0)
        # SQ_VALU_MFMA_BUSY_CYCLES is summed over the SIMDs, SQ_BUSY_CYCLES over the shader engines: with the
        # SIMDs per shader engine in the denominator, a kernel whose every SIMD keeps its matrix pipe busy reads 1
        mfma = c.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) / simds_per_se
        lds_act = c.get("SQ_ACTIVE_INST_LDS", 0.0)
        conflict = c.get("SQ_LDS_BANK_CONFLICT", 0.0) / lds_act if lds_act else 0.0
        wait_lds = c.get("SQ_WAIT_INST_LDS", 0.0) / c["SQ_WAVE_CYCLES"] if c.get("SQ_WAVE_CYCLES") else 0.0
        mfma_frac = mfma / busy if busy else 0.0
        ab = algorithmic.get(k)
        e = {n.replace("_sum", ""): v[0] for n, v in eac.get(k, {}).items()}
        ea_lat = e.get("TCC_EA0_RDREQ_LEVEL", 0.0) / e["TCC_EA0_RDREQ"] if e.get("TCC_EA0_RDREQ") else 0.0
        ea_stall = e.get("TCC_EA0_RDREQ_DRAM_CREDIT_STALL", 0.0) / e["TCC_BUSY"] if e.get("TCC_BUSY") else 0.0
        lines.append(f"| {k} | {us:.1f} us | {fb / 1e9:.3f} GB | {wb / 1e9:.3f} GB | {(fb + wb) / 1e9:.3f} GB | "
                     f"{(f'{ab / 1e9:.3f} GB' if ab else '')} | {(fb + wb) / us / 1e6:.2f} TB/s | {mfma_frac:.3f} | {conflict:.3f} | {wait_lds:.3f} | "
                     f"{ea_lat:.0f} L2 clk | {ea_stall:.4f} |")
        figs.append(f"{a.config} {k} avg_us {us:.1f} fetch_bytes {fb:.0f} write_bytes {wb:.0f} mfma_busy {mfma_frac:.4f} "
                    f"lds_conflict {conflict:.4f}")
    lines += ["", "MFMA busy = SQ_VALU_MFMA_BUSY_CYCLES (summed over SIMDs) / (SQ_BUSY_CYCLES (summed over shader engines) x SIMDs per",
              f"shader engine = {simds_per_se:.0f}): the share of the cycles a SIMD is busy in which its matrix pipe is.",
              "Read latency past L2 = TCC_EA0_RDREQ_LEVEL / TCC_EA0_RDREQ (mean time a read that missed L2 is outstanding, in L2",
              "clocks); DRAM credit stalls = TCC_EA0_RDREQ_DRAM_CREDIT_STALL / TCC_BUSY (share of the L2-busy cycles in which a",
              "read could not be sent on for lack of DRAM credits: the memory side saturated).",
              "FETCH_SIZE counts what misses the per-XCD L2s, whether the memory-side cache or HBM serves it.  Algorithmic bytes:",
              "weights (+ scales) of the touched experts once, the routed rows of the token-side operand once, the output once.", "",
              "## Raw figures", ""]
    for k in KERNELS:
        if k in stats:
            s = stats[k]
            lines.append(f"    {k}: calls {s['calls']} avg_ns {s['avg_ns']:.0f} min_ns {s['min_ns']:.0f} max_ns {s['max_ns']:.0f}")
        for src in (fetch, write, sqc, eac):
            for cname, (v, n) in sorted(src.get(k, {}).items()):
                lines.append(f"    {k}: {cname} {v:.1f} (mean of {n} dispatches)")
    os.makedirs(a.out, exist_ok=True)
    with open(os.path.join(a.out, f"split_pipeline_{a.config}.md"), "w") as f:
        f.write("\n".join(lines) + "\n")
    table = os.path.join(a.out, "kernel_figures.txt")
    old = [l for l in open(table).read().splitlines() if l and not l.startswith(a.config + " ")] if os.path.exists(table) else []
    with open(table, "w") as f:
        f.write("\n".join(sorted(old + figs)) + "\n")
    print("\n".join(lines[-40:]))


if __name__ == "__main__":
    main()
