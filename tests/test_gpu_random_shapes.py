"""Seeded random shapes through both fused ops against the CPU oracle.

The kernels choose among many tile paths from the routing (two paired blocks or one, 1 / 2 / 4 live
fragments, complete tiles, jobs of the tail split 2 to 4 ways in the bf16 kernels, several weight tiles
per workgroup in the mxfp8 kernels); the fixed cases of the other files pin the ones the reference
tests, these walk the space between them.  Same gates as everywhere else.
"""
import random

import pytest
import torch

import test_gpu_bf16 as B
import test_gpu_mxfp8 as M

pytestmark = pytest.mark.gpu


def _draw(seed, mx):
    r = random.Random(seed)
    E = r.choice([1, 2, 3, 5, 8, 17, 40])
    top_k = r.randint(1, min(E, 6)) if E > 1 else 1
    T = r.choice([1, 7, 33, 100, 129, 257, 400, 700])
    K = r.choice([256, 512, 768, 1280] if mx else [128, 256, 384, 640, 1152])
    N = r.choice([256, 512, 768, 1280])
    split, hot_last = r.random() < 0.5, top_k > 1 and r.random() < 0.5  # (the hot expert takes one of >= 2 picks)
    return T, K, E, N, top_k, split, hot_last, r.choice([0, 0, 1, 2, 3])


@pytest.mark.parametrize("seed", range(16))
def test_bf16_random_shape(seed, device):
    T, K, E, N, top_k, split, hot_last, _ = _draw(seed, mx=False)
    B._run_case(T, K, E, N, top_k, split, device, seed=100 + seed, hot_last=hot_last)


@pytest.mark.parametrize("seed", range(16))
def test_mxfp8_random_shape(seed, device):
    from prime_moe import _native
    T, K, E, N, top_k, split, hot_last, per = _draw(1000 + seed, mx=True)
    lib = _native.load()
    lib.pmoe_set_tiles_per_workgroup(per)
    try:
        M._run_case(T, K, E, N, top_k, split, device, seed=200 + seed, hot_last=hot_last)
    finally:
        lib.pmoe_set_tiles_per_workgroup(0)
