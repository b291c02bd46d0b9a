"""The benchmark harness (prime_moe/sweep.py, the counterpart of the reference's benchmark/benchmark.py):
one small row per dtype, eager and as graph replays, with skewed routing; the row's own check compares
the fused op with the grouped-GEMM baseline on the same GPU."""
import csv
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.filterwarnings("error::UserWarning")  # (an empty graph must not slip through as a warning)
@pytest.mark.parametrize("dtype,graphs", [("bf16", False), ("bf16", True), ("mxfp8", True)])
def test_sweep_row(dtype, graphs, device):
    from prime_moe import sweep
    r = sweep.run_one(dtype, 512, 8, 512, 256, 2, True, 2, 5, True, seed=3, balancedness=0.6, graphs=graphs)
    assert r["fused_ms"] > 0 and r["baseline_ms"] > 0 and r["naive_ms"] > 0
    # one way of timing per row, and the row says which: replays only if every callable could be recorded (and the
    # fused one's replay reproduced the eager bits), otherwise eager calls with the reason
    if not graphs:
        assert r["timed_as"] == "eager" and r["timed_note"] == ""
    else:
        assert r["timed_as"] in ("replay", "eager")
        assert (r["timed_note"] == "") == (r["timed_as"] == "replay"), r["timed_note"]
        assert "fused:" not in r["timed_note"], r["timed_note"]  # the fused op itself is always capturable
    assert math.isfinite(r["rel"]) and r["rel"] <= (2e-2 if dtype == "bf16" else 5e-2), r
    assert r["naive_max_abs"] <= 2e-2  # the two torch baselines agree with each other


def test_routing_balancedness(device):
    from prime_moe import sweep
    g = torch.Generator(device=device).manual_seed(0)
    ids = sweep.generate_topk_ids(16, 4096, 4, 0.0, g)
    assert int(ids.max()) == 0  # everything to expert 0
    ids = sweep.generate_topk_ids(16, 4096, 4, 1.0, g)
    counts = torch.bincount(ids.flatten().long(), minlength=16).float()
    assert float(counts.min()) > 0.8 * 1024 and float(counts.max()) < 1.2 * 1024
    ids = sweep.generate_topk_ids(16, 4096, 4, 0.5, g)
    share0 = float((ids == 0).float().mean())
    assert 0.48 < share0 < 0.58  # 0.5 + 0.5 / 16


def test_sweep_csv_columns(tmp_path, device):
    from prime_moe import sweep
    path = tmp_path / "sweep.csv"
    sweep.run_sweep(str(path), tokens=(256,), dtypes=("bf16",), E=4, top_k=2, K=256, H=128, warmup=1, iters=2,
                    log=lambda *a: None, skip_naive=True)
    rows = list(csv.DictReader(open(path)))
    assert len(rows) == 1
    # the reference's columns (benchmark/benchmark.py:523-543), in its order, then this harness's own
    assert list(rows[0].keys()) == sweep.COLUMNS
    assert list(rows[0].keys())[:19] == ["dtype", "tokens", "E", "K", "N", "top_k", "naive_ms", "baseline_ms", "noreq_ms",
                                         "fused_ms", "speedup", "speedup_noreq", "speedup_naive", "naive_tflops",
                                         "baseline_tflops", "fused_tflops", "max_abs", "rel", "naive_max_abs"]
    assert rows[0]["naive_ms"] == "" and float(rows[0]["fused_ms"]) > 0
    assert rows[0]["timed_as"] == "eager" and rows[0]["timed_note"] == ""
