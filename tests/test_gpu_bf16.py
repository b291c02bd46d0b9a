"""fused_moe_bf16 on the GPU vs the fp32 CPU oracle on identical seeded inputs.
Gate: max |got - ref| / max(|ref|, 1) <= 2e-2."""
import math

import pytest
import torch

from helpers import BF16_GATE, oracle_schedule, reference_routing, rel_clamp
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _inputs(T, K, E, N, device, seed, x_std=1.0):
    g = torch.Generator(device=device).manual_seed(seed)
    x = (torch.randn((T, K), device=device, generator=g) * x_std).to(torch.bfloat16)
    w1 = (torch.randn((E, N, K), device=device, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    w2 = (torch.randn((E, K, N // 2), device=device, generator=g) / math.sqrt(N // 2)).to(torch.bfloat16)
    return g, x, w1, w2


def _run_case(T, K, E, N, top_k, split, device, seed=0, use_op_align=True, exact=False, hot_last=True,
              prefill_out=None):
    import prime_moe
    g, x, w1, w2 = _inputs(T, K, E, N, device, seed)
    ids, wts = reference_routing(T, E, top_k, device, g, hot_last=hot_last)
    if use_op_align:
        sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    else:
        sched = oracle_schedule(ids, E, 128, exact=exact)
    if prefill_out is None:
        out = torch.zeros((T, K), dtype=torch.bfloat16, device=device) if not split else \
            torch.full((T, K), float("nan"), dtype=torch.bfloat16, device=device)
    else:
        out = prefill_out.clone()
    ret = prime_moe.fused_moe_bf16(x, w1, w2, *sched, wts, out, top_k, 128, 64, 4, 2, 1, 1, split)
    torch.cuda.synchronize()
    assert ret is out
    ref = O.fused_moe_dense(x.cpu(), w1.cpu(), w2.cpu(), ids.cpu(), wts.cpu())
    if prefill_out is not None and not split:
        ref = ref + prefill_out.float().cpu()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    err = rel_clamp(got, ref, 1.0)
    assert err <= BF16_GATE, f"rel_clamp_1 {err:.4g} > {BF16_GATE}"
    return err


@pytest.mark.parametrize("split", [True, False])
def test_readme_shape(split, device):
    # T=256 K=4096 E=8 N=512 top_k=4 with top-4 of N(0,1) logits and softmax weights
    import prime_moe
    from prime_moe.workloads import CONFIGS, make_inputs
    cfg = CONFIGS["c1_readme_bf16"]
    inp = make_inputs(cfg, device, seed=1)
    sched = torch.ops.prime_moe.moe_align(inp["topk_ids"], cfg.E, 128, 1)
    out = torch.zeros((cfg.T, cfg.K), dtype=torch.bfloat16, device=device)
    prime_moe.fused_moe_bf16(inp["x"], inp["w1"], inp["w2"], *sched, inp["topk_weights"], out, cfg.top_k,
                             128, 64, 4, 2, 1, 1, split)
    torch.cuda.synchronize()
    ref = O.fused_moe_dense(inp["x"].cpu(), inp["w1"].cpu(), inp["w2"].cpu(), inp["topk_ids"].cpu(),
                            inp["topk_weights"].cpu())
    err = rel_clamp(out.float().cpu(), ref, 1.0)
    assert err <= BF16_GATE, err


@pytest.mark.parametrize("split", [True, False])
@pytest.mark.parametrize("T,K,E,N", [
    (8, 4096, 257, 256), (32, 7168, 8, 512), (128, 4096, 37, 256), (256, 7168, 37, 512),
    (200, 1024, 8, 768), (1, 128, 1, 256), (130, 384, 3, 256),
])
def test_reference_sweep_shapes(T, K, E, N, split, device):
    # the reference's own sweep grid (test/test.py:133-146), top_k = 9 with a hot last expert,
    # plus ragged cases: K % 256 == 128, a single token, one expert
    top_k = 9 if E > 1 else 1
    _run_case(T, K, E, N, top_k, split, device, seed=T + E)


@pytest.mark.parametrize("split", [True, False])
def test_exact_size_schedule_from_python_restatement(split, device):
    _run_case(64, 1024, 8, 512, 4, split, device, use_op_align=False, exact=True)
    _run_case(64, 1024, 8, 512, 4, split, device, use_op_align=False, exact=False)


def test_split_overwrites_and_fused_accumulates(device):
    T, K = 96, 512
    pre = torch.randn((T, K), device=device).to(torch.bfloat16)
    _run_case(T, K, 4, 256, 2, True, device, prefill_out=pre, hot_last=False)   # overwritten
    _run_case(T, K, 4, 256, 2, False, device, prefill_out=pre, hot_last=False)  # added to


def test_tokens_beyond_m_are_dropped(device):
    import prime_moe
    T, K, E, N, top_k = 64, 512, 4, 256, 2
    g, x, w1, w2 = _inputs(T, K, E, N, device, 3)
    ids, wts = reference_routing(T, E, top_k, device, g, hot_last=False)
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    keep = 40  # x with fewer rows than the schedule refers to: rows of tokens >= keep are skipped
    out = torch.zeros((keep, K), dtype=torch.bfloat16, device=device)
    prime_moe.fused_moe_bf16(x[:keep].contiguous(), w1, w2, *sched, wts, out, top_k, 128, 32, 8, 1, 1, 1, True)
    torch.cuda.synchronize()
    ref = O.fused_moe_dense(x.cpu(), w1.cpu(), w2.cpu(), ids.cpu(), wts.cpu())[:keep]
    assert rel_clamp(out.float().cpu(), ref, 1.0) <= BF16_GATE


def test_validation_errors(device):
    import prime_moe
    T, K, E, N, top_k = 16, 256, 2, 256, 2
    g, x, w1, w2 = _inputs(T, K, E, N, device, 0)
    ids, wts = reference_routing(T, E, top_k, device, g, hot_last=False)
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    out = torch.zeros((T, K), dtype=torch.bfloat16, device=device)
    ok = dict(top_k=top_k, block_m=128, block_n=64, warp_n=4, stages=2, bpc=1, cpc=1, split=True)

    def call(**kw):
        a = dict(ok)
        a.update(kw)
        prime_moe.fused_moe_bf16(kw.pop("x", x), w1, w2, *sched, kw.pop("wts", wts), kw.pop("out", out),
                                 a["top_k"], a["block_m"], a["block_n"], a["warp_n"], a["stages"], a["bpc"],
                                 a["cpc"], a["split"])

    call()
    for bad in (dict(block_m=64), dict(block_n=64, warp_n=8), dict(stages=0), dict(stages=6),
                dict(stages=5, split=True), dict(bpc=2), dict(cpc=2)):
        with pytest.raises(RuntimeError):
            call(**bad)
    call(stages=5, split=False)
    with pytest.raises(RuntimeError):
        call(x=x.float())
    with pytest.raises(RuntimeError):
        call(out=out.float())
    with pytest.raises(RuntimeError):
        call(wts=wts.double())
    with pytest.raises(RuntimeError):
        call(x=x.t().contiguous().t())
    with pytest.raises(RuntimeError):
        call(x=x[:, :192].contiguous())
    # a tensor that is not on x's GPU is rejected on the host (its pointer never reaches a kernel)
    with pytest.raises(RuntimeError, match="is on cpu"):
        call(wts=wts.cpu())
    with pytest.raises(RuntimeError, match="is on cpu"):
        call(out=out.cpu())
    with pytest.raises(RuntimeError, match="is on cpu"):
        prime_moe.fused_moe_bf16(x, w1, w2, sched[0].cpu(), sched[1], sched[2], wts, out, top_k, 128, 64, 4, 2, 1, 1, True)
    # x starting 2 bytes into an allocation: the 16-byte copies of the loaders would be misaligned
    shifted = torch.empty((T * K + 1,), dtype=torch.bfloat16, device=device)[1:].view(T, K)
    with pytest.raises(RuntimeError, match="aligned"):
        call(x=shifted)


def test_result_is_bitwise_reproducible(device):
    """No atomics anywhere in the pipeline: two calls on the same inputs agree bit for bit."""
    import prime_moe
    g, x, w1, w2 = _inputs(300, 512, 8, 512, device, seed=5)
    ids, wts = reference_routing(300, 8, 4, device, g)
    sched = torch.ops.prime_moe.moe_align(ids, 8, 128, 1)
    outs = []
    for _ in range(3):
        out = torch.empty((300, 512), dtype=torch.bfloat16, device=device)
        prime_moe.fused_moe_bf16(x, w1, w2, *sched, wts, out, 4, 128, 64, 4, 2, 1, 1, True)
        outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


def test_experts_with_one_and_with_several_row_tiles(device):
    # expert 0: 276 rows = a full row tile and a tail of 20 rows that reads the same weight rows; expert 1:
    # 200 rows in one tile of two blocks; expert 2: 56 rows; expert 3: 20 rows, alone on its weight rows
    # (decode-style tile, other cache policy of the weight copies); expert 4: none
    import prime_moe
    from test_gpu_mxfp8 import _routing_by_counts
    counts, top_k = [276, 200, 56, 20, 0], 2
    K, E, N = 1024, 5, 512
    ids, wts = _routing_by_counts(counts, top_k, device, seed=6)
    T = ids.shape[0]
    g, x, w1, w2 = _inputs(T, K, E, N, device, seed=22)
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    for split in (True, False):
        out = torch.zeros((T, K), dtype=torch.bfloat16, device=device)
        prime_moe.fused_moe_bf16(x, w1, w2, *sched, wts, out, top_k, 128, 64, 4, 2, 1, 1, split)
        torch.cuda.synchronize()
        ref = O.fused_moe_dense(x.cpu(), w1.cpu(), w2.cpu(), ids.cpu(), wts.cpu())
        assert rel_clamp(out.float().cpu(), ref, 1.0) <= BF16_GATE


def test_block_without_expert_and_duplicate_pair(device):
    """Schedules the fused op must survive: a block whose expert id is out of range is not computed and
    its pairs contribute nothing (never whatever the workspace held); a pair id listed twice in one block
    contributes once; listed again in a block of another expert, one of the two experts' rows (unspecified
    which) stands for the pair, and nothing faults."""
    import prime_moe
    T, K, E, N, top_k = 300, 512, 6, 512, 2
    g, x, w1, w2 = _inputs(T, K, E, N, device, seed=9)
    ids, wts = reference_routing(T, E, top_k, device, g, hot_last=False)
    s, e, n = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    dropped = 1  # second block of the schedule loses its expert
    e_bad = e.clone()
    e_bad[dropped] = -1
    pairs = s[dropped * 128:(dropped + 1) * 128]
    pairs = pairs[pairs >= 0].long()
    w_ref = wts.clone().flatten()
    w_ref[pairs] = 0.0  # the oracle drops the same pairs through their routing weights
    ref = O.fused_moe_dense(x.cpu(), w1.cpu(), w2.cpu(), ids.cpu(), w_ref.view(T, top_k).cpu())
    for fill in (float("nan"), 1e30):  # whatever an earlier call left in the caching allocator's blocks
        junk = torch.full((64 << 20,), fill, dtype=torch.bfloat16, device=device)
        del junk
        out = torch.empty((T, K), dtype=torch.bfloat16, device=device)
        prime_moe.fused_moe_bf16(x, w1, w2, s, e_bad, n, wts, out, top_k, 128, 64, 4, 2, 1, 1, True)
        torch.cuda.synchronize()
        got = out.float().cpu()
        assert torch.isfinite(got).all()
        assert rel_clamp(got, ref, 1.0) <= BF16_GATE
    # a pair id listed twice (in a padding slot of its own block): counted once
    s_dup = s.clone()
    blk = int((s[:128] < 0).nonzero()[0]) if bool((s[:128] < 0).any()) else None
    if blk is not None:
        s_dup[blk] = s[0]
        ref = O.fused_moe_dense(x.cpu(), w1.cpu(), w2.cpu(), ids.cpu(), wts.cpu())
        out = torch.empty((T, K), dtype=torch.bfloat16, device=device)
        prime_moe.fused_moe_bf16(x, w1, w2, s_dup, e, n, wts, out, top_k, 128, 64, 4, 2, 1, 1, True)
        torch.cuda.synchronize()
        assert rel_clamp(out.float().cpu(), ref, 1.0) <= BF16_GATE
    # the same pair id once more in a padding slot of another expert's block: two workgroups write y[pair]; the
    # result for that token is one of the two candidates, the rest of the output is untouched
    other = [b for b in range(1, int(n[0]) // 128) if int(e[b]) != int(e[0]) and bool((s[b * 128:(b + 1) * 128] < 0).any())]
    if other:
        b = other[0]
        slot = b * 128 + int((s[b * 128:(b + 1) * 128] < 0).nonzero()[0])
        s_far = s.clone()
        s_far[slot] = s[0]
        ref = O.fused_moe_dense(x.cpu(), w1.cpu(), w2.cpu(), ids.cpu(), wts.cpu())
        out = torch.empty((T, K), dtype=torch.bfloat16, device=device)
        prime_moe.fused_moe_bf16(x, w1, w2, s_far, e, n, wts, out, top_k, 128, 64, 4, 2, 1, 1, True)
        torch.cuda.synchronize()
        got = out.float().cpu()
        assert torch.isfinite(got).all()
        tok = int(s[0]) // top_k
        keep = torch.ones(T, dtype=torch.bool)
        keep[tok] = False
        assert rel_clamp(got[keep], ref[keep], 1.0) <= BF16_GATE


@pytest.mark.parametrize("T,K,E,N,top_k,exact", [
    (256, 4096, 8, 512, 4, False),   # the README shape: 8 - 16 row tiles x 2 weight tiles, every tile split 8 ways
    (40, 2048, 4, 256, 2, False),    # one weight tile, tiles of one or two fragments
    (130, 6144, 3, 512, 3, True),    # exact-size schedule, a second block with two live rows
    (1, 2048, 1, 256, 1, False),     # one row
    (300, 2176, 2, 1024, 2, False),  # 17 slabs: parts of unequal length
])
def test_few_jobs_deep_split_and_join_kernel(T, K, E, N, top_k, exact, device):
    """Few up jobs for the chip and a long contraction: every up tile is split over up to 8 workgroups that
    only store their partial sums, and a kernel of its own joins them and applies SwiGLU.  Against the
    oracle, and bit for bit the same on a second call (the join adds the parts in part order)."""
    import prime_moe
    for split in (True, False):
        _run_case(T, K, E, N, top_k, split, device, seed=T + K, use_op_align=not exact, exact=exact, hot_last=False)
    g, x, w1, w2 = _inputs(T, K, E, N, device, T + K)
    ids, wts = reference_routing(T, E, top_k, device, g, hot_last=False)
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    outs = []
    for _ in range(2):
        torch.empty((32 << 20,), dtype=torch.float32, device=device).fill_(float("nan"))  # dirty the allocator's blocks
        out = torch.empty((T, K), dtype=torch.bfloat16, device=device)
        prime_moe.fused_moe_bf16(x, w1, w2, *sched, wts, out, top_k, 128, 64, 4, 2, 1, 1, True)
        outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
