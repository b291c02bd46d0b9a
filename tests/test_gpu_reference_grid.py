"""The reference's whole sweep grid (test/test.py:133-146 and the same grid in test/test_mxfp8.py):
T in {8, 32, 128, 256} x N in {256, 512} x K in {7168, 4096} x E in {257, 8, 37}, top_k = 9 with the
last expert hot, both values of `split`.  96 + 96 cases whose CPU oracle takes minutes in total, so
they only run when PMOE_FULL_GRID=1 is set; the everyday suite keeps one case per (T, K, E) diagonal
(test_reference_sweep_shapes in the two per-dtype files)."""
import itertools
import os

import pytest

import test_gpu_bf16 as B
import test_gpu_mxfp8 as M

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("PMOE_FULL_GRID") != "1", reason="set PMOE_FULL_GRID=1 to run the whole grid")]

GRID = list(itertools.product([8, 32, 128, 256], [256, 512], [7168, 4096], [257, 8, 37], [True, False]))


@pytest.mark.parametrize("T,N,K,E,split", GRID)
def test_bf16_grid(T, N, K, E, split, device):
    B._run_case(T, K, E, N, 9, split, device, seed=T + N + E)


@pytest.mark.parametrize("T,N,K,E,split", GRID)
def test_mxfp8_grid(T, N, K, E, split, device):
    M._run_case(T, K, E, N, 9, split, device, seed=T + N + E)
