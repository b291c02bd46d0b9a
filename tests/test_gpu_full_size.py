"""The five benchmark configurations at their full sizes.

The CPU oracle cannot evaluate a whole configuration in seconds, so each one is checked through
(a) the CPU oracle on every routed row of a set of experts that includes the hottest and the coldest
    touched one: the op runs with the routing weights of all other pairs set to zero, so `out` holds
    exactly those experts' contributions (hundreds of tokens, every kernel at its full-size shape);
(b) the CPU oracle on a seeded sample of whole tokens (all their experts);
(c) the oracle's dataflow evaluated in fp32 on the device (the same oracle function on device tensors,
    weights fetched and, for mxfp8, dequantised one expert at a time): every element of the full
    output.  (a) ties this evaluation to the CPU one on the same subset;
(d) properties that do not depend on the size: doubling the routing weights doubles the result, and
    split=False adds the same result into a prefilled `out`.
Gates as for the small cases, plus the element-wise rel_clamp_1 for mxfp8.
"""
import pytest
import torch

import test_gpu_mxfp8 as M
from helpers import BF16_GATE, MX_COS_GATE, MX_FLIP_DELTA, MX_RELL2_GATE, cosine, mx_elementwise_gates, rel_clamp, rel_l2
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _run(cfg, inp, sched, out, split, weights=None):
    import prime_moe
    w = inp["topk_weights"] if weights is None else weights
    if cfg.dtype == "bf16":
        prime_moe.fused_moe_bf16(inp["x"], inp["w1"], inp["w2"], *sched, w, out, cfg.top_k, cfg.block_m,
                                 64, 4, 2, 1, 1, split)
    else:
        prime_moe.fused_moe_mxfp8(inp["x"], inp["x_scales"], inp["w1"], inp["w1_scales"], inp["w2"],
                                  inp["w2_scales"], *sched, w, out, cfg.top_k, cfg.block_m, 64, 4, 2, 1, split)
    torch.cuda.synchronize()
    return out


def _oracle(cfg, inp, device, tokens=None, experts=None):
    """The oracle on `device` ("cpu" or the GPU) for the tokens `tokens` (all if None), restricted to
    `experts` (all if None); fp32 throughout, one expert's weights at a time.  Returns (ref, bound): for mxfp8
    the oracle's bound on boundary flips of the activation quantisation (from the fp32 activations: a full-size
    configuration in fp64 would take too long), for bf16 None."""
    mx = cfg.dtype != "bf16"
    to = lambda t: t.to(device)
    sel = slice(None) if tokens is None else tokens.to(inp["x"].device)
    ids, wts = to(inp["topk_ids"][sel]), to(inp["topk_weights"][sel])
    if mx:
        x = O.dequantize_mx_torch(to(inp["x"][sel]), to(inp["x_scales"][sel].view(torch.uint8)))
        fetch = lambda e: (O.dequantize_mx_torch(to(inp["w1"][e]), to(inp["w1_scales_rm"][e])),
                           O.dequantize_mx_torch(to(inp["w2"][e]), to(inp["w2_scales_rm"][e])))
    else:
        x = to(inp["x"][sel]).float()
        fetch = lambda e: (to(inp["w1"][e]).float(), to(inp["w2"][e]).float())
    if mx:
        return O.fused_moe_by_expert(x, fetch, ids, wts, cfg.E, act_mx=True, experts=experts, flip_delta=MX_FLIP_DELTA)
    return O.fused_moe_by_expert(x, fetch, ids, wts, cfg.E, experts=experts), None


def _gate(cfg, got, ref, bound, what):
    """The gates of the small cases on `got` vs `ref` (CPU float tensors)."""
    if cfg.dtype == "bf16":
        err = rel_clamp(got, ref, 1.0)
        assert err <= BF16_GATE, f"{cfg.name} {what}: rel_clamp_1 {err:.4g}"
        return f"rel_clamp_1 {err:.3g}"
    c, l2 = cosine(got, ref), rel_l2(got, ref)
    assert c >= MX_COS_GATE and l2 <= MX_RELL2_GATE, f"{cfg.name} {what}: cosine {c}, rel-L2 {l2}"
    rc1, rc10, needed = mx_elementwise_gates(got, ref, bound.cpu())
    return (f"cosine {c:.6f} rel-L2 {l2:.3g}, beyond the flip bound rel_clamp_1 {rc1:.3g} rel_clamp_10 {rc10:.3g} "
            f"({needed} elements needed the bound)")


@pytest.mark.parametrize("name,n_tokens", [
    ("c1_readme_bf16", 64), ("c2_mixtral_bf16", 32), ("c3_qwen3_bf16", 32),
    ("c4_dsv3_mxfp8", 4), ("c5_decode_mxfp8", 4),
])
def test_full_size_config(name, n_tokens, device):
    import prime_moe  # noqa: F401
    from prime_moe.workloads import CONFIGS, make_inputs
    cfg = CONFIGS[name]
    inp = make_inputs(cfg, device, seed=1, keep_row_major_scales=True)
    sched = torch.ops.prime_moe.moe_align(inp["topk_ids"], cfg.E, cfg.block_m, 1)
    out = torch.full((cfg.T, cfg.K), float("nan"), dtype=torch.bfloat16, device=device)
    _run(cfg, inp, sched, out, True)
    got = out.float()
    assert torch.isfinite(got).all()
    report = []

    # (a) all rows of the hottest, the coldest touched and two more experts, against the CPU oracle
    counts = torch.bincount(inp["topk_ids"].flatten().long(), minlength=cfg.E).cpu()
    touched = torch.nonzero(counts > 0).flatten()
    hottest = int(counts.argmax())
    coldest = int(touched[counts[touched].argmin()])
    g = torch.Generator().manual_seed(7)
    extra = touched[torch.randperm(touched.numel(), generator=g)[:2]].tolist()
    subset = sorted({hottest, coldest, *extra})
    keep = torch.zeros((cfg.E,), dtype=torch.bool, device=device)
    keep[subset] = True
    masked_w = inp["topk_weights"] * keep[inp["topk_ids"].long()]
    out_s = torch.full_like(out, float("nan"))
    _run(cfg, inp, sched, out_s, True, weights=masked_w)
    ref_cpu, bound_cpu = _oracle(cfg, inp, "cpu", experts=subset)
    n_rows = int((ref_cpu.abs().sum(1) > 0).sum())
    assert n_rows >= min(32, cfg.T), f"{name}: only {n_rows} tokens reach the checked experts"
    report.append(f"(a) experts {subset} ({n_rows} tokens, hottest {int(counts[hottest])} / coldest "
                  f"{int(counts[coldest])} rows): " + _gate(cfg, out_s.float().cpu(), ref_cpu, bound_cpu, "expert subset vs CPU oracle"))

    # (b) whole tokens against the CPU oracle (every expert they use)
    sel = torch.randperm(cfg.T, generator=g)[:n_tokens].sort().values
    ref_tok, bound_tok = _oracle(cfg, inp, "cpu", tokens=sel)
    report.append(f"(b) {n_tokens} whole tokens: " + _gate(cfg, got[sel.to(device)].cpu(), ref_tok, bound_tok, "token sample vs CPU oracle"))

    # (c) every element against the oracle's dataflow evaluated on the device, which (a) and (b) tie
    # to the CPU evaluation
    ref_dev, bound_dev = _oracle(cfg, inp, device)
    # (fp32 sums in another order; for mxfp8 an activation that sits on a rounding boundary of e4m3 may
    # land on the neighbouring code: the two evaluations agree to within the bound on that)
    if cfg.dtype == "bf16":
        tie = rel_clamp(ref_dev[sel.to(device)].cpu(), ref_tok, 1.0)
    else:
        rest = ((ref_dev[sel.to(device)].cpu().double() - ref_tok.double()).abs() - bound_tok).clamp_min(0.0)
        tie = float((rest / ref_tok.double().abs().clamp_min(1.0)).max())
    assert tie <= 1e-4, f"{name}: device and CPU evaluation of the oracle differ by {tie:.3g}"
    report.append("(c) all elements: " + _gate(cfg, got.cpu(), ref_dev.cpu(), bound_dev, "all elements vs the oracle on the device"))
    print(f"\n{name}: " + "; ".join(report))

    # (d) linear in the routing weights (up to the bf16 rounding of `out`)
    out2 = torch.empty_like(out)
    _run(cfg, inp, sched, out2, True, weights=inp["topk_weights"] * 2.0)
    scale = float(got.abs().max())
    assert float((out2.float() - 2.0 * got).abs().max()) <= 2e-2 * scale

    # split=False adds the same result into `out`
    out3 = torch.ones_like(out)
    _run(cfg, inp, sched, out3, False)
    assert float((out3.float() - (1.0 + got)).abs().max()) <= 2e-2 * max(scale, 1.0)
