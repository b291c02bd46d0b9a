"""The five benchmark configurations at their full sizes.

The CPU oracle cannot evaluate a whole configuration in seconds, so each one is checked through
(a) the oracle on a seeded sample of tokens (tokens are independent given the routing; for mxfp8
the experts of the sample are dequantised on the host one sample at a time), with the same gates
as the small cases, and (b) properties that do not depend on the size: doubling the routing
weights doubles the result, and split=False adds the same result into a prefilled `out`.
"""
import dataclasses

import pytest
import torch

from helpers import BF16_GATE, MX_COS_GATE, MX_RELL2_GATE, cosine, rel_clamp, rel_l2
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


def _sample_oracle(cfg, inp, sel):
    """fp32 oracle rows for the tokens `sel` (CPU tensor of indices)."""
    ids = inp["topk_ids"].cpu()[sel]
    wts = inp["topk_weights"].cpu()[sel]
    if cfg.dtype == "bf16":
        return O.fused_moe_dense(inp["x"].cpu()[sel], inp["w1"].cpu(), inp["w2"].cpu(), ids, wts)
    # mxfp8: only the experts the sample uses are dequantised, renumbered 0..U-1
    used, remap = torch.unique(ids, return_inverse=True)
    u8 = lambda t: t.cpu().view(torch.uint8)
    x = O.dequantize_mx_torch(inp["x"].cpu()[sel], u8(inp["x_scales"])[sel])
    w1 = torch.stack([O.dequantize_mx_torch(inp["w1"][int(e)].cpu(), inp["w1_scales_rm"][int(e)].cpu()) for e in used])
    w2 = torch.stack([O.dequantize_mx_torch(inp["w2"][int(e)].cpu(), inp["w2_scales_rm"][int(e)].cpu()) for e in used])
    return O.fused_moe_dense(x, w1, w2, remap.reshape(ids.shape), wts, act_mx=True)


@pytest.mark.parametrize("name,n_sample", [
    ("c1_readme_bf16", 64), ("c2_mixtral_bf16", 48), ("c3_qwen3_bf16", 64),
    ("c4_dsv3_mxfp8", 3), ("c5_decode_mxfp8", 3),
])
def test_full_size_config(name, n_sample, device):
    import prime_moe  # noqa: F401
    from prime_moe.workloads import CONFIGS, make_inputs
    cfg = CONFIGS[name]
    inp = make_inputs(cfg, device, seed=1, keep_row_major_scales=True)
    sched = torch.ops.prime_moe.moe_align(inp["topk_ids"], cfg.E, cfg.block_m, 1)
    out = torch.full((cfg.T, cfg.K), float("nan"), dtype=torch.bfloat16, device=device)
    _run(cfg, inp, sched, out, True)
    got = out.float()
    assert torch.isfinite(got).all()

    # (a) sampled tokens against the oracle
    g = torch.Generator().manual_seed(7)
    sel = torch.randperm(cfg.T, generator=g)[:n_sample].sort().values
    ref = _sample_oracle(cfg, inp, sel)
    got_s = got[sel.to(device)].cpu()
    if cfg.dtype == "bf16":
        err = rel_clamp(got_s, ref, 1.0)
        assert err <= BF16_GATE, f"{name}: rel_clamp_1 {err:.4g}"
    else:
        c, l2 = cosine(got_s, ref), rel_l2(got_s, ref)
        assert c >= MX_COS_GATE and l2 <= MX_RELL2_GATE, f"{name}: cosine {c}, rel-L2 {l2}"

    # (b) linear in the routing weights (up to the bf16 rounding of `out`)
    out2 = torch.empty_like(out)
    _run(cfg, inp, sched, out2, True, weights=inp["topk_weights"] * 2.0)
    scale = float(got.abs().max())
    assert float((out2.float() - 2.0 * got).abs().max()) <= 2e-2 * scale

    # (c) split=False adds the same result into `out`
    out3 = torch.ones_like(out)
    _run(cfg, inp, sched, out3, False)
    assert float((out3.float() - (1.0 + got)).abs().max()) <= 2e-2 * max(scale, 1.0)
