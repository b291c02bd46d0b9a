"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

from oracle import moe_oracle as O

BF16_GATE = 2e-2        # max |got - ref| / max(|ref|, 1) for the bf16 path
MX_COS_GATE = 0.999     # cosine similarity floor for the mxfp8 path
MX_RELL2_GATE = 2e-2    # ||got - ref|| / ||ref|| ceiling for the mxfp8 path
# element-wise gates of the mxfp8 path, the reference's own metric and values (test/test_mxfp8.py:14-15,
# :168-191): max |got - ref| / max(|ref|, c) for c = 1 and c = 10
MX_REL_CLAMP_1_GATE = 2e-2
MX_REL_CLAMP_10_GATE = 2e-3


def rel_clamp(got: torch.Tensor, ref: torch.Tensor, c: float) -> float:
    d = (got.double() - ref.double()).abs()
    return float((d / ref.double().abs().clamp_min(c)).max())


def cosine(got: torch.Tensor, ref: torch.Tensor) -> float:
    g, r = got.double().reshape(-1), ref.double().reshape(-1)
    return float((g @ r) / (g.norm() * r.norm()).clamp_min(1e-300))


def rel_l2(got: torch.Tensor, ref: torch.Tensor) -> float:
    return float((got.double() - ref.double()).norm() / ref.double().norm().clamp_min(1e-300))


def reference_routing(T, E, top_k, device, gen, hot_last=True):
    """Routing of the reference's sweeps (test/test.py:155-157): top_k-1 experts drawn with
    replacement from the first E-1 plus expert E-1 for every token; softmax(N(0,1)) weights."""
    if hot_last and E > 1:
        probs = torch.ones(E - 1, device=device)
        ids = torch.multinomial(probs, T * (top_k - 1), replacement=True, generator=gen).view(T, top_k - 1)
        ids = torch.cat([ids, torch.full((T, 1), E - 1, device=device, dtype=ids.dtype)], 1)
    else:
        ids = torch.randint(0, E, (T, top_k), device=device, generator=gen)
    w = torch.softmax(torch.randn((T, top_k), device=device, generator=gen), -1)
    return ids.to(torch.int32).contiguous(), w.contiguous()


def oracle_schedule(topk_ids: torch.Tensor, E: int, block_m: int = 128, exact: bool = False):
    """Schedule from the CPU oracle, as device tensors (exact=True: the exact-size arrays the
    reference's Python restatement returns, test/test.py:81-120)."""
    s, e, t = O.moe_align_fast(topk_ids.cpu().numpy(), E, block_m, 1)
    if exact:
        tot = int(t[0])
        s, e = s[:tot], e[: tot // block_m]
    dev = topk_ids.device
    return (torch.from_numpy(s.copy()).to(dev), torch.from_numpy(e.copy()).to(dev), torch.from_numpy(t.copy()).to(dev))
