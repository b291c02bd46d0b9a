"""The direct-to-LDS copies of the GEMM kernels are issued from inline assembly that sets M0 itself (csrc/moe_ring.h).
If a compiler ever kept a value of its own in M0 across such a statement, copies would land in the wrong place.  These
cases run the tile paths with the longest runs of copies between two barriers (bf16: tiles of 384 token rows, ten
copies per wave and slab; mxfp8: row tiles of two full blocks, nine per wave and stage, with two to four stages in
flight) right after every CU's LDS has been filled with NaN patterns, so a misplaced copy shows up here, by name, as
a NaN or a parity failure, and not somewhere in the grids."""
import pytest
import torch

import test_gpu_bf16 as B
import test_gpu_mxfp8 as M

pytestmark = pytest.mark.gpu


def _poison(device):
    from prime_moe import _native
    word = torch.zeros(1, dtype=torch.int32, device=device)
    _native.check(_native.load().pmoe_poison_lds(word.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert int(word[0]) == 0


@pytest.mark.parametrize("split", [True, False])
@pytest.mark.parametrize("K,N", [(256, 256), (2048, 512)])
def test_bf16_tall_tiles_on_poisoned_lds(K, N, split, device):
    # 2 experts x ~800 rows: tiles of 5 and 6 pairs of fragments; K = 256 has four slabs (the ring's first and last
    # stages only), K = 2048 runs the steady state
    _poison(device)
    B._run_case(800, K, 2, N, 2, split, device, seed=11, hot_last=False)


@pytest.mark.parametrize("split", [True, False])
@pytest.mark.parametrize("K,N", [(256, 256), (2048, 512)])
def test_mxfp8_full_tiles_on_poisoned_lds(K, N, split, device):
    _poison(device)
    M._run_case(800, K, 2, N, 2, split, device, seed=12, hot_last=False)
