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
# An activation within this relative distance of a rounding boundary of its MX quantisation may come out on the
# neighbouring code in two evaluations that add the same fp32 products in different orders (kernel and oracle);
# the oracle bounds what that does to every output element (oracle.mx_flip_spacing), and the element-wise gates
# allow that much on top of the reference's thresholds, and nothing else.
MX_FLIP_DELTA = 1e-4


def rel_clamp(got: torch.Tensor, ref: torch.Tensor, c: float) -> float:
    d = (got.double() - ref.double()).abs()
    return float((d / ref.double().abs().clamp_min(c)).max())


def mx_elementwise_gates(got: torch.Tensor, ref: torch.Tensor, bound: torch.Tensor):
    """The reference's element-wise gates (test/test_mxfp8.py:168-191) on what is left of |got - ref| after the
    oracle's bound on boundary flips of the activation quantisation (MX_FLIP_DELTA) is taken off: elements that no
    such flip can reach (bound 0: most of them) face the reference's thresholds exactly.  Returns
    (rel_clamp_1, rel_clamp_10, elements that needed the bound)."""
    d = (got.double() - ref.double()).abs()
    rest = (d - bound.double().to(d.device)).clamp_min(0.0)
    a = ref.double().abs()
    rc1 = float((rest / a.clamp_min(1.0)).max())
    rc10 = float((rest / a.clamp_min(10.0)).max())
    needed = int(((d > MX_REL_CLAMP_1_GATE * a.clamp_min(1.0)) | (d > MX_REL_CLAMP_10_GATE * a.clamp_min(10.0))).sum())
    assert rc1 <= MX_REL_CLAMP_1_GATE, f"rel_clamp_1 {rc1} beyond what boundary flips explain ({needed} elements over the plain gates)"
    assert rc10 <= MX_REL_CLAMP_10_GATE, f"rel_clamp_10 {rc10} beyond what boundary flips explain ({needed} elements over the plain gates)"
    return rc1, rc10, needed


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
