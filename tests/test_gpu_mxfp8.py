"""fused_moe_mxfp8 on the GPU vs the fp32 CPU oracle evaluated on the dequantised inputs with
the activation quantise->dequantise modelled.  Gates: cosine >= 0.999, rel-L2 <= 2e-2."""
import math

import numpy as np
import pytest
import torch

from helpers import MX_COS_GATE, MX_RELL2_GATE, cosine, oracle_schedule, reference_routing, rel_clamp, rel_l2
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _quantised_inputs(T, K, E, N, device, seed, x_std=1.0):
    """bf16 masters on the device, quantised by the CPU oracle (so the op's inputs do not depend
    on the GPU quantiser), packed with the product's pack_scales_blocked."""
    import prime_moe
    g = torch.Generator(device=device).manual_seed(seed)
    x = (torch.randn((T, K), device=device, generator=g) * x_std).to(torch.bfloat16)
    w1 = (torch.randn((E, N, K), device=device, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    w2 = (torch.randn((E, K, N // 2), device=device, generator=g) / math.sqrt(N // 2)).to(torch.bfloat16)
    q = {}
    for name, t in (("x", x), ("w1", w1), ("w2", w2)):
        qt, st = O.quantize_mx_torch(t.float().cpu())
        q[name] = (qt, st)
    dev = lambda t: t.to(device)
    e8 = lambda s: s.view(torch.float8_e8m0fnu)
    args = dict(
        x=dev(q["x"][0]), x_scales=dev(e8(q["x"][1])),
        w1=dev(q["w1"][0]), w1_scales=prime_moe.pack_scales_blocked(dev(e8(q["w1"][1]))),
        w2=dev(q["w2"][0]), w2_scales=prime_moe.pack_scales_blocked(dev(e8(q["w2"][1]))),
    )
    deq = {k: O.dequantize_mx_torch(*v) for k, v in q.items()}
    return g, args, deq


def _run_case(T, K, E, N, top_k, split, device, seed=0, use_op_align=True, exact=False, hot_last=True):
    import prime_moe
    g, a, deq = _quantised_inputs(T, K, E, N, device, seed)
    ids, wts = reference_routing(T, E, top_k, device, g, hot_last=hot_last)
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1) if use_op_align else oracle_schedule(ids, E, 128, exact)
    out = torch.zeros((T, K), dtype=torch.bfloat16, device=device) if not split else \
        torch.full((T, K), float("nan"), dtype=torch.bfloat16, device=device)
    ret = prime_moe.fused_moe_mxfp8(a["x"], a["x_scales"], a["w1"], a["w1_scales"], a["w2"], a["w2_scales"],
                                    *sched, wts, out, top_k, 128, 64, 4, 2, 1, split)
    torch.cuda.synchronize()
    assert ret is out
    ref = O.fused_moe_dense(deq["x"], deq["w1"], deq["w2"], ids.cpu(), wts.cpu(), act_mx=True)
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    c, l2 = cosine(got, ref), rel_l2(got, ref)
    assert c >= MX_COS_GATE, f"cosine {c}"
    assert l2 <= MX_RELL2_GATE, f"rel-L2 {l2}"
    return c, l2


@pytest.mark.parametrize("split", [True, False])
@pytest.mark.parametrize("T,K,E,N", [
    (8, 4096, 257, 256), (32, 7168, 8, 512), (128, 4096, 37, 256), (256, 7168, 37, 512),
    (1, 256, 1, 256), (130, 768, 3, 512),
])
def test_reference_sweep_shapes(T, K, E, N, split, device):
    top_k = 9 if E > 1 else 1
    _run_case(T, K, E, N, top_k, split, device, seed=T + E)


@pytest.mark.parametrize("split", [True, False])
def test_exact_size_schedule(split, device):
    _run_case(64, 1024, 8, 512, 4, split, device, use_op_align=False, exact=True)


def test_public_wrapper_matches_raw_op(device):
    # mirrors the reference's wrapper test (test/test_mxfp8.py:203-239)
    import prime_moe
    T, K, E, N, top_k = 128, 4096, 8, 256, 4
    g, a, _ = _quantised_inputs(T, K, E, N, device, 5, x_std=0.05)
    ids, wts = reference_routing(T, E, top_k, device, g, hot_last=False)
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    args = (a["x"], a["x_scales"], a["w1"], a["w1_scales"], a["w2"], a["w2_scales"], *sched, wts)
    tail = (top_k, 128, 32, 8, 1, 1, False)
    raw = torch.zeros((T, K), dtype=torch.bfloat16, device=device)
    torch.ops.prime_moe.fused_moe_mxfp8(*args, raw, *tail)
    wrapped = torch.zeros((T, K), dtype=torch.bfloat16, device=device)
    ret = prime_moe.fused_moe_mxfp8(*args, wrapped, *tail)
    torch.cuda.synchronize()
    assert ret is wrapped
    assert torch.allclose(raw.float(), wrapped.float(), rtol=1e-2, atol=2e-3)


def test_validation_errors(device):
    import prime_moe
    T, K, E, N, top_k = 16, 256, 2, 256, 2
    g, a, _ = _quantised_inputs(T, K, E, N, device, 0)
    ids, wts = reference_routing(T, E, top_k, device, g, hot_last=False)
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    out = torch.zeros((T, K), dtype=torch.bfloat16, device=device)

    def call(x=a["x"], xs=a["x_scales"], w1s=a["w1_scales"], block_m=128, bn=64, wn=4, stages=2, bpc=1, split=True):
        prime_moe.fused_moe_mxfp8(x, xs, a["w1"], w1s, a["w2"], a["w2_scales"], *sched, wts, out, top_k,
                                  block_m, bn, wn, stages, bpc, split)

    call()
    for bad in (dict(block_m=64), dict(bn=32, wn=4), dict(stages=0), dict(stages=5), dict(bpc=2)):
        with pytest.raises(RuntimeError):
            call(**bad)
    with pytest.raises(RuntimeError):
        call(x=a["x"].view(torch.uint8))
    with pytest.raises(RuntimeError):
        call(xs=a["x_scales"].view(torch.uint8))
    with pytest.raises(RuntimeError):
        call(xs=a["x_scales"][:, :4].contiguous())
    with pytest.raises(RuntimeError):
        call(w1s=a["w1_scales"].reshape(-1)[:-1].contiguous())
    # tensors that are not on x's GPU are rejected on the host (their pointers never reach a kernel)
    with pytest.raises(RuntimeError, match="is on cpu"):
        call(xs=a["x_scales"].cpu())
    with pytest.raises(RuntimeError, match="is on cpu"):
        call(w1s=a["w1_scales"].cpu())
    # x scales starting 1 byte into an allocation: the kernels read them as 32-bit words
    n_xs = a["x_scales"].numel()
    shifted = torch.empty((n_xs + 1,), dtype=torch.uint8, device=device)[1:].view(torch.float8_e8m0fnu).view(T, K // 32)
    with pytest.raises(RuntimeError, match="aligned"):
        call(xs=shifted)


@pytest.mark.parametrize("per", [2, 3, 16])
@pytest.mark.parametrize("T,K,E,N,top_k", [
    (300, 1280, 4, 1280, 2),   # wide tiles of every kind; 5 up and 5 down weight tiles (not a multiple of 2 or 3)
    (24, 768, 6, 768, 3),      # tiles of one fragment: the down tile stores from registers
])
def test_several_weight_tiles_per_workgroup(T, K, E, N, top_k, per, device):
    # a workgroup that walks `per` weight tiles with its token rows must give the bits of one tile per
    # workgroup (same sums in the same order), and both must pass the oracle gates
    import prime_moe
    from prime_moe import _native
    lib = _native.load()
    g, a, deq = _quantised_inputs(T, K, E, N, device, seed=per)
    ids, wts = reference_routing(T, E, top_k, device, g)
    sched = torch.ops.prime_moe.moe_align(ids, E, 128, 1)
    outs = []
    try:
        for n in (1, per):
            lib.pmoe_set_tiles_per_workgroup(n)
            out = torch.full((T, K), float("nan"), dtype=torch.bfloat16, device=device)
            prime_moe.fused_moe_mxfp8(a["x"], a["x_scales"], a["w1"], a["w1_scales"], a["w2"], a["w2_scales"],
                                      *sched, wts, out, top_k, 128, 64, 4, 2, 1, True)
            torch.cuda.synchronize()
            outs.append(out)
    finally:
        lib.pmoe_set_tiles_per_workgroup(0)
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    ref = O.fused_moe_dense(deq["x"], deq["w1"], deq["w2"], ids.cpu(), wts.cpu(), act_mx=True)
    got = outs[1].float().cpu()
    assert cosine(got, ref) >= MX_COS_GATE and rel_l2(got, ref) <= MX_RELL2_GATE
