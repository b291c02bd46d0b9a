"""moe_align on the GPU vs the CPU oracle: bit-exact int32 outputs, through the torch op
(which calls the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _run(ids_np, E, block_m, bpc, device):
    import prime_moe  # noqa: F401  (registers the ops)
    ids = torch.from_numpy(np.ascontiguousarray(ids_np, dtype=np.int32)).to(device)
    s, e, t = torch.ops.prime_moe.moe_align(ids, E, block_m, bpc)
    torch.cuda.synchronize()
    ref = O.moe_align_fast(ids_np, E, block_m, bpc)
    for got, want, name in zip((s, e, t), ref, ("sorted_token_ids", "expert_ids", "num_tokens_post_padded")):
        assert got.dtype == torch.int32
        np.testing.assert_array_equal(got.cpu().numpy(), want, err_msg=name)


@pytest.mark.parametrize("n,E,block_m,bpc", [
    (1, 1, 128, 1), (9 * 8, 257, 128, 1), (9 * 256, 37, 128, 1), (1024, 8, 128, 1), (777, 8, 128, 2),
    (4096 * 2, 8, 128, 1), (64 * 8, 256, 128, 1), (8192 * 8, 128, 128, 1), (4096 * 8, 256, 128, 1),
    (5000, 1024, 128, 1), (3001, 513, 24, 3), (131072 * 4, 32, 128, 1), (63, 2, 16, 1), (65, 64, 128, 1),
])
def test_align_matches_oracle(n, E, block_m, bpc, device):
    rng = np.random.default_rng(n + E)
    ids = rng.integers(0, E, size=n)
    if n > 16:
        ids[rng.integers(0, n, size=n // 4)] = E - 1  # hot expert
    _run(ids, E, block_m, bpc, device)


def test_align_empty_and_single_expert(device):
    _run(np.zeros((0,), dtype=np.int64), 4, 128, 1, device)
    _run(np.zeros((300,), dtype=np.int64), 1, 128, 1, device)
    _run(np.full((130,), 6), 7, 128, 1, device)  # all on the last-but... one expert, others empty


def test_align_2d_input_and_zipf(device):
    rng = np.random.default_rng(0)
    pop = np.arange(1, 257, dtype=np.float64) ** -1.2
    pop /= pop.sum()
    ids = np.stack([rng.choice(256, size=8, replace=False, p=pop) for _ in range(64)])
    _run(ids, 256, 128, 1, device)


def test_align_deterministic(device):
    import prime_moe  # noqa: F401
    ids = torch.randint(0, 128, (65536,), device=device, dtype=torch.int32)
    a = torch.ops.prime_moe.moe_align(ids, 128, 128, 1)
    b = torch.ops.prime_moe.moe_align(ids, 128, 128, 1)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_align_errors(device):
    import prime_moe  # noqa: F401
    ids = torch.zeros((8,), device=device, dtype=torch.int32)
    with pytest.raises(RuntimeError):
        torch.ops.prime_moe.moe_align(ids.long(), 4, 128, 1)
    with pytest.raises(RuntimeError):
        torch.ops.prime_moe.moe_align(ids, 1025, 128, 1)
    with pytest.raises(RuntimeError):
        torch.ops.prime_moe.moe_align(ids, 4, 0, 1)
    with pytest.raises(RuntimeError):
        torch.ops.prime_moe.moe_align(torch.zeros((8, 2), device=device, dtype=torch.int32)[:, 0], 4, 128, 1)


@pytest.mark.parametrize("T,top_k,E", [
    (16385, 1, 8),        # one id past what a single workgroup takes: three slices, the last with one id
    (8192, 4, 37),        # whole slices only
    (20000, 3, 257),      # a hot last expert, odd sizes
    (30011, 2, 1024),     # the largest expert count, 8 waves per workgroup
    (40000, 1, 1),        # one expert
])
def test_many_ids_spread_over_workgroups(T, top_k, E, device):
    # above 16384 ids the op sorts with three launches over many workgroups; the result is the
    # single-workgroup one bit for bit (ascending pair ids inside an expert)
    rng = np.random.default_rng(T + E)
    ids = rng.integers(0, E, size=(T, top_k))
    if E == 257:
        ids[:, -1] = E - 1
    _run(ids, E, 128, 1, device)


def test_many_ids_with_ids_out_of_range_and_scratch_fallback(device):
    import prime_moe
    from prime_moe import _native
    rng = np.random.default_rng(3)
    ids = rng.integers(-2, 12, size=50000).astype(np.int32)
    # ids outside [0, E) are skipped: the expected result is the oracle's on the ids in range, with
    # its pair numbers mapped back and the arrays extended to the sizes of the full input
    keep = np.flatnonzero((ids >= 0) & (ids < 8))
    s_c, e_c, t_c = O.moe_align_fast(ids[keep], 8, 128, 1)
    _, max_padded, max_blocks = O.moe_align_sizes(50000, 8, 128, 1)
    s_w = np.full(max_padded, -1, dtype=np.int32)
    s_w[: s_c.size] = np.where(s_c >= 0, keep[np.maximum(s_c, 0)], -1)
    e_w = np.full(max_blocks, 7, dtype=np.int32)
    e_w[: e_c.size] = e_c
    want = (s_w, e_w, t_c)
    dev_ids = torch.from_numpy(ids).to(device)
    got = torch.ops.prime_moe.moe_align(dev_ids, 8, 128, 1)
    for a, b in zip(got, want):
        assert np.array_equal(a.cpu().numpy(), b)
    # the plain entry point (no scratch) sorts the same ids with its single workgroup
    lib = _native.load()
    assert lib.pmoe_moe_align_workspace_bytes(50000, 8) == 4 * (7 * 8 + 2 * 8 + 1)
    assert lib.pmoe_moe_align_workspace_bytes(16384, 8) == 0
    pad_to, max_padded, max_blocks = prime_moe.align_sizes(50000, 8, 128, 1)
    s = torch.empty((max_padded,), dtype=torch.int32, device=device)
    e = torch.empty((max_blocks,), dtype=torch.int32, device=device)
    t = torch.empty((1,), dtype=torch.int32, device=device)
    _native.check(lib.pmoe_moe_align(dev_ids.data_ptr(), s.data_ptr(), e.data_ptr(), t.data_ptr(), 50000, 8, 128,
                                     pad_to, max_padded, max_blocks, torch.cuda.current_stream(device).cuda_stream))
    torch.cuda.synchronize()
    for a, b in zip((s, e, t), want):
        assert np.array_equal(a.cpu().numpy(), b)
