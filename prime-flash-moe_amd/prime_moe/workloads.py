"""Synthetic workloads of the fused-MoE forward: the five benchmark configurations.

Shapes, input distributions and routing rules are the ones the benchmark specification
names; everything is generated on the device from one seeded generator, expert by expert,
so the largest configuration never holds bf16 masters of all experts at once.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Dict, Optional

import torch

from . import pack_scales_blocked, quantize_mx


@dataclasses.dataclass(frozen=True)
class MoeConfig:
    name: str
    dtype: str          # "bf16" | "mxfp8"
    T: int
    K: int
    E: int
    N: int
    top_k: int
    routing: str        # "topk" | "topk_bias" | "uniform" | "zipf"
    block_m: int = 128

    @property
    def H(self) -> int:
        return self.N // 2

    @property
    def flops(self) -> float:
        """3*P*K*N with P = T*top_k unpadded pairs (the reference benchmark's FLOP model,
        benchmark/benchmark.py:389-391)."""
        return 3.0 * self.T * self.top_k * self.K * self.N

    def weight_bytes_per_expert(self) -> int:
        elems = self.N * self.K + self.K * self.H
        if self.dtype == "bf16":
            return 2 * elems
        return elems + elems // 32


CONFIGS: Dict[str, MoeConfig] = {
    "c1_readme_bf16": MoeConfig("c1_readme_bf16", "bf16", 256, 4096, 8, 512, 4, "topk"),
    "c2_mixtral_bf16": MoeConfig("c2_mixtral_bf16", "bf16", 4096, 4096, 8, 28672, 2, "topk"),
    "c3_qwen3_bf16": MoeConfig("c3_qwen3_bf16", "bf16", 8192, 2048, 128, 1536, 8, "topk_bias"),
    "c4_dsv3_mxfp8": MoeConfig("c4_dsv3_mxfp8", "mxfp8", 4096, 7168, 256, 4096, 8, "uniform"),
    "c5_decode_mxfp8": MoeConfig("c5_decode_mxfp8", "mxfp8", 64, 7168, 256, 4096, 8, "zipf"),
}

# The compute-bound end of the reference benchmark's own grid (benchmark/benchmark.py:695-718: E=32, top_k=4,
# K=2048, H=1024, 131072 tokens, 16384 rows per expert): reported next to the five specification workloads.
GRID_CONFIGS: Dict[str, MoeConfig] = {
    "g1_grid_bf16_131072": MoeConfig("g1_grid_bf16_131072", "bf16", 131072, 2048, 32, 2048, 4, "topk"),
    "g2_grid_mxfp8_131072": MoeConfig("g2_grid_mxfp8_131072", "mxfp8", 131072, 2048, 32, 2048, 4, "topk"),
}


def make_routing(cfg: MoeConfig, gen: torch.Generator, device) -> Dict[str, torch.Tensor]:
    """topk_ids (T, top_k) int32 and topk_weights (T, top_k) fp32 for the config's routing rule."""
    T, E, k = cfg.T, cfg.E, cfg.top_k
    if cfg.routing in ("topk", "topk_bias", "uniform"):
        if cfg.routing == "uniform":
            logits = torch.rand((T, E), generator=gen, device=device)
        else:
            logits = torch.randn((T, E), generator=gen, device=device)
        if cfg.routing == "topk_bias":
            logits = logits + 0.5 * torch.randn((E,), generator=gen, device=device)
        vals, ids = torch.topk(logits, k, dim=-1)
        weights = torch.softmax(vals.float(), dim=-1)
    elif cfg.routing == "zipf":
        pop = torch.arange(1, E + 1, device=device, dtype=torch.float32).pow(-1.2)
        ids = torch.multinomial(pop.expand(T, E).contiguous(), k, replacement=False, generator=gen)
        weights = torch.softmax(torch.randn((T, k), generator=gen, device=device), dim=-1)
    else:
        raise ValueError(cfg.routing)
    return {"topk_ids": ids.to(torch.int32).contiguous(), "topk_weights": weights.contiguous()}


def _randn_bf16(shape, std, gen, device):
    return (torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * std).to(torch.bfloat16)


def make_inputs(cfg: MoeConfig, device="cuda:0", seed: int = 0, keep_row_major_scales: bool = False,
                scale: Optional[float] = None) -> Dict[str, torch.Tensor]:
    """Tensors of one configuration: x ~ N(0,1), w1 ~ N(0,1/K), w2 ~ N(0,1/H), routing per config.

    mxfp8: the bf16 masters are quantised with the OCP-MX quantiser (e4m3 + e8m0 per 32 along the
    contraction dim); x scales stay row major, weight scales are packed into the blocked layout.
    """
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    T, K, E, N, H = cfg.T, cfg.K, cfg.E, cfg.N, cfg.H
    xs = 1.0 if scale is None else scale
    out: Dict[str, torch.Tensor] = {}
    x = _randn_bf16((T, K), xs, gen, device)
    out.update(make_routing(cfg, gen, device))
    s1, s2 = 1.0 / math.sqrt(K), 1.0 / math.sqrt(H)
    if cfg.dtype == "bf16":
        w1 = torch.empty((E, N, K), dtype=torch.bfloat16, device=device)
        w2 = torch.empty((E, K, H), dtype=torch.bfloat16, device=device)
        for e in range(E):
            w1[e] = _randn_bf16((N, K), s1, gen, device)
            w2[e] = _randn_bf16((K, H), s2, gen, device)
        out.update(x=x, w1=w1, w2=w2)
        return out
    xq, xsc = quantize_mx(x)
    w1q = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device=device)
    w2q = torch.empty((E, K, H), dtype=torch.float8_e4m3fn, device=device)
    w1s = torch.empty((E, N, K // 32), dtype=torch.uint8, device=device)
    w2s = torch.empty((E, K, H // 32), dtype=torch.uint8, device=device)
    for e in range(E):
        q, s = quantize_mx(_randn_bf16((N, K), s1, gen, device))
        w1q[e], w1s[e] = q, s.view(torch.uint8)
        q, s = quantize_mx(_randn_bf16((K, H), s2, gen, device))
        w2q[e], w2s[e] = q, s.view(torch.uint8)
    out.update(x=xq, x_scales=xsc, w1=w1q, w2=w2q,
               w1_scales=pack_scales_blocked(w1s.view(torch.float8_e8m0fnu)),
               w2_scales=pack_scales_blocked(w2s.view(torch.float8_e8m0fnu)))
    if keep_row_major_scales:
        out.update(w1_scales_rm=w1s, w2_scales_rm=w2s)
    return out


def touched_weight_bytes(cfg: MoeConfig, topk_ids: torch.Tensor) -> int:
    """Weight (+scale) bytes of the experts the routing actually uses (decode-shape GB/s figure)."""
    n_touched = int(torch.unique(topk_ids).numel())
    return n_touched * cfg.weight_bytes_per_expert()
