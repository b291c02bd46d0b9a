"""pmoe_moe_align_static, the entry point that allocates nothing: its scratch is a device array built
into the library.  Called through the C ABI and compared bit for bit with pmoe_moe_align_ws (the
existing entry point with caller-provided scratch) and with the CPU oracle, on calls in a row that
share the built-in array, each smaller than the one before."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _call(lib, fn_name, ids, E, block_m, bpc, device, with_ws):
    import prime_moe
    from prime_moe import _native
    n = ids.numel()
    pad_to, max_padded, max_blocks = prime_moe.align_sizes(n, E, block_m, bpc)
    # poisoned outputs: every element must be written by the call
    s = torch.full((max_padded,), 0x5a5a5a5a, dtype=torch.int32, device=device)
    e = torch.full((max_blocks,), 0x5a5a5a5a, dtype=torch.int32, device=device)
    t = torch.full((1,), 0x5a5a5a5a, dtype=torch.int32, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    if with_ws:
        nbytes = lib.pmoe_moe_align_workspace_bytes(n, E)
        ws = torch.empty((max(nbytes, 4),), dtype=torch.uint8, device=device)
        _native.check(lib.pmoe_moe_align_ws(ids.data_ptr(), s.data_ptr(), e.data_ptr(), t.data_ptr(), n, E, block_m,
                                            pad_to, max_padded, max_blocks, ws.data_ptr(), nbytes, stream))
    else:
        _native.check(getattr(lib, fn_name)(ids.data_ptr(), s.data_ptr(), e.data_ptr(), t.data_ptr(), n, E, block_m,
                                            pad_to, max_padded, max_blocks, stream))
    torch.cuda.synchronize()
    return s, e, t


def test_static_scratch_align_matches_workspace_entry_point(device):
    from prime_moe import _native
    lib = _native.load()
    rng = np.random.default_rng(11)
    # every case is above the 16384 ids one workgroup takes, so all of them go through the built-in
    # scratch; sizes shrink from call to call (8 slices, 5, 3) and the expert count changes, so a call
    # that relied on what the call before left in the array would show
    cases = [(65536, 128, 128, 1), (40000, 257, 128, 1), (20000, 8, 128, 2)]
    for n, E, block_m, bpc in cases:
        ids_np = rng.integers(0, E, size=n).astype(np.int32)
        ids_np[rng.integers(0, n, size=n // 4)] = E - 1  # a hot expert
        ids = torch.from_numpy(ids_np).to(device)
        got = _call(lib, "pmoe_moe_align_static", ids, E, block_m, bpc, device, with_ws=False)
        want = _call(lib, None, ids, E, block_m, bpc, device, with_ws=True)
        ref = O.moe_align_fast(ids_np, E, block_m, bpc)
        for g, w, r, name in zip(got, want, ref, ("sorted_token_ids", "expert_ids", "num_tokens_post_padded")):
            assert torch.equal(g, w), f"{name}: differs from pmoe_moe_align_ws (n={n}, E={E})"
            np.testing.assert_array_equal(g.cpu().numpy(), r, err_msg=f"{name} vs oracle (n={n}, E={E})")


def test_static_scratch_align_small_input_and_size_limit(device):
    import prime_moe
    from prime_moe import _native
    lib = _native.load()
    ids_np = np.random.default_rng(5).integers(0, 16, size=777).astype(np.int32)
    ids = torch.from_numpy(ids_np).to(device)
    got = _call(lib, "pmoe_moe_align_static", ids, 16, 128, 1, device, with_ws=False)
    for g, r in zip(got, O.moe_align_fast(ids_np, 16, 128, 1)):
        np.testing.assert_array_equal(g.cpu().numpy(), r)
    # beyond the built-in scratch: rejected on the host, nothing is launched (the pointers are never read)
    n = (1 << 20) + 1
    pad_to, max_padded, max_blocks = prime_moe.align_sizes(n, 8, 128, 1)
    rc = lib.pmoe_moe_align_static(ids.data_ptr(), ids.data_ptr(), ids.data_ptr(), ids.data_ptr(), n, 8, 128, pad_to,
                                   max_padded, max_blocks, torch.cuda.current_stream(device).cuda_stream)
    assert rc == 1 and b"built-in scratch" in lib.pmoe_last_error()
