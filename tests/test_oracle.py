"""Pins of the CPU oracle (oracle/moe_oracle.py) against facts that do not depend on it:
invariants and brute force for moe_align, a closed form and an independent gather for the
scale packing, the exhaustive E4M3 code table and hand-derived MX known answers, and for the
forward pass a dense fp64 brute force, the SwiGLU-MLP special case and algebraic properties."""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O


# ----------------------------------------------------------------------------- moe_align

def _check_align_invariants(ids, E, block_m, bpc, out):
    sorted_ids, expert_ids, total = out
    ids = np.asarray(ids).reshape(-1)
    n = ids.size
    pad = block_m * bpc
    max_padded = (n + E * (pad - 1) + pad - 1) // pad * pad
    assert sorted_ids.dtype == np.int32 and expert_ids.dtype == np.int32 and total.dtype == np.int32
    assert sorted_ids.shape == (max_padded,) and expert_ids.shape == (max_padded // block_m,)
    counts = [int((ids == e).sum()) for e in range(E)]
    padded = [(c + pad - 1) // pad * pad for c in counts]
    assert int(total[0]) == sum(padded)
    pos = 0
    for e in range(E):
        seg = sorted_ids[pos:pos + padded[e]]
        live = seg[:counts[e]]
        assert list(live) == [i for i in range(n) if ids[i] == e]  # ascending pair ids of expert e
        assert (seg[counts[e]:] == -1).all()
        for j in range(pos // block_m, (pos + padded[e]) // block_m):
            assert expert_ids[j] == e
        pos += padded[e]
    assert (sorted_ids[pos:] == -1).all()
    assert (expert_ids[pos // block_m:] == E - 1).all()


@pytest.mark.parametrize("n,E,block_m,bpc", [
    (0, 4, 128, 1), (1, 1, 128, 1), (37, 8, 16, 1), (300, 5, 128, 1), (513, 37, 128, 2),
    (64, 257, 128, 1), (1000, 3, 24, 3), (2048, 128, 128, 1),
])
def test_align_invariants(n, E, block_m, bpc):
    rng = np.random.default_rng(n * 7 + E)
    ids = rng.integers(0, E, size=n)
    if n > 10:
        ids[: n // 3] = E - 1  # a hot expert, and (for large E) many empty ones
    out = O.moe_align(ids, E, block_m, bpc)
    _check_align_invariants(ids, E, block_m, bpc, out)
    fast = O.moe_align_fast(ids, E, block_m, bpc)
    for a, b in zip(out, fast):
        np.testing.assert_array_equal(a, b)


def test_align_hand_example():
    # 6 pairs, 3 experts, blocks of 4: expert0 <- pairs 1,4; expert1 <- none; expert2 <- 0,2,3,5
    ids = [2, 0, 2, 2, 0, 2]
    s, e, t = O.moe_align(ids, 3, 4, 1)
    # max_padded = ceil((6 + 3*3)/4)*4 = 16
    assert list(s) == [1, 4, -1, -1, 0, 2, 3, 5] + [-1] * 8
    assert list(e) == [0, 2, 2, 2]
    assert list(t) == [8]


def test_align_matches_sort_restatement():
    # the reference tests build the schedule with argsort + bincount (test/test.py:81-120);
    # a stable sort must give the same live prefix as the oracle, exact-size
    rng = np.random.default_rng(3)
    ids = rng.integers(0, 37, size=(32, 9))
    ids[:, -1] = 36
    flat = ids.reshape(-1)
    order = np.argsort(flat, kind="stable")
    counts = np.bincount(flat, minlength=37)
    padded = (counts + 127) // 128 * 128
    ref = np.full(padded.sum(), -1, dtype=np.int32)
    w = r = 0
    for e in range(37):
        ref[w:w + counts[e]] = order[r:r + counts[e]]
        w += padded[e]
        r += counts[e]
    s, eids, t = O.moe_align(ids, 37, 128, 1)
    np.testing.assert_array_equal(s[: int(t[0])], ref)
    np.testing.assert_array_equal(eids[: int(t[0]) // 128], np.repeat(np.arange(37), padded // 128))


def test_align_rejects_bad_ids():
    with pytest.raises(ValueError):
        O.moe_align([0, 5], 4, 128, 1)


# ----------------------------------------------------------------------------- scale packing

def test_pack_offset_closed_form_and_gather():
    rng = np.random.default_rng(0)
    E, MN, KB = 2, 256, 8
    s = rng.integers(0, 255, size=(E, MN, KB), dtype=np.uint8)
    packed = O.pack_scales_blocked(s)
    assert packed.shape == (E, MN * KB)
    # independent reading of the layout: walk tiles, then the 32x(4x4) interior
    for e in range(E):
        p = packed[e].reshape(MN // 128, KB // 4, 32, 4, 4)  # [row tile][k tile][r%32][r//32][b%4]
        for r in (0, 1, 31, 32, 127, 128, 200, 255):
            for b in range(KB):
                assert p[r // 128, b // 4, r % 32, (r % 128) // 32, b % 4] == s[e, r, b]
    # it is a permutation
    assert sorted(packed.reshape(-1).tolist()) == sorted(s.reshape(-1).tolist())
    # one row's four scales over 128 K are one aligned dword
    off = O.blocked_scale_offset(77, np.arange(4), KB)
    assert off[0] % 4 == 0 and list(off - off[0]) == [0, 1, 2, 3]


def test_pack_rejects_ragged():
    with pytest.raises(AssertionError):
        O.pack_scales_blocked(np.zeros((100, 4), dtype=np.uint8))
    with pytest.raises(AssertionError):
        O.pack_scales_blocked(np.zeros((128, 3), dtype=np.uint8))


# ----------------------------------------------------------------------------- e4m3 / MX

def test_e4m3_table_vs_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().numpy()
    got = O.e4m3_decode(np.arange(256, dtype=np.uint8))
    np.testing.assert_array_equal(np.isnan(ref), np.isnan(got))
    np.testing.assert_array_equal(ref[~np.isnan(ref)], got[~np.isnan(got)])
    assert got[0x7E] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9


def test_e4m3_encode_round_trip_and_rne():
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    vals = O.e4m3_decode(codes)
    back = O.e4m3_encode_sat(vals)
    np.testing.assert_array_equal(O.e4m3_decode(back), vals)  # (-0 and +0 both decode to 0)
    # ties go to even mantissa: 1.0625 lies between 1.0 (m=0) and 1.125 (m=1) -> 1.0;
    # 1.1875 between 1.125 (m=1) and 1.25 (m=2) -> 1.25
    np.testing.assert_array_equal(O.e4m3_decode(O.e4m3_encode_sat(np.float32([1.0625, 1.1875, 17.0, 19.0]))),
                                  np.float32([1.0, 1.25, 16.0, 20.0]))
    # saturation, and the subnormal grid 2^-9 with its tie rule
    np.testing.assert_array_equal(O.e4m3_decode(O.e4m3_encode_sat(np.float32([449, 1e9, -1e9, 464.1]))),
                                  np.float32([448, 448, -448, 448]))
    np.testing.assert_array_equal(O.e4m3_encode_sat(np.float32([2.0 ** -10, 3 * 2.0 ** -10, 2.0 ** -9])),
                                  np.uint8([0, 2, 1]))
    # against torch's cast on a dense random sample inside the finite range
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(20000) * rng.choice([1e-3, 0.1, 1, 30, 200], 20000)).astype(np.float32)
    x = np.clip(x, -448, 448)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = O.e4m3_encode_sat(x)
    np.testing.assert_array_equal(O.e4m3_decode(ref), O.e4m3_decode(got))


def test_mx_known_answers():
    # hand-derived: e = clamp(expfield(amax) - 8, 0, 254); q = rne_e4m3(v * 2^(127-e)), saturating
    def q1(v):
        block = np.zeros(32, dtype=np.float32)
        block[0] = v
        q, e = O.quantize_mx(block)
        return int(e[0]), float(O.e4m3_decode(q)[0]), float(O.dequantize_mx(q, e)[0])
    assert q1(0.0) == (0, 0.0, 0.0)
    assert q1(1.0) == (119, 256.0, 1.0)              # 1.0 = 2^0: field 127 -> e 119, 1.0 * 2^8
    assert q1(3.5) == (120, 448.0, 3.5)              # 3.5 = 1.75*2^1: e 120, 3.5 * 2^7 = 448
    assert q1(3.9) == (120, 448.0, 3.5)              # 3.9 * 128 = 499.2 saturates to 448
    assert q1(448.0) == (127, 448.0, 448.0)
    assert q1(449.0) == (127, 448.0, 448.0)
    assert q1(511.9) == (127, 448.0, 448.0)
    assert q1(512.0) == (128, 256.0, 512.0)
    assert q1(-3.5) == (120, -448.0, -3.5)
    # exponent field 7 -> e clamps to 0; 2^-120 * 2^127 = 128 is an E4M3 value, and 128 * 2^-127 = 2^-120
    assert q1(2.0 ** -120) == (0, 128.0, 2.0 ** -120)


def test_mx_tiny_block_exact():
    block = np.zeros(32, dtype=np.float32)
    block[0] = 2.0 ** -120
    q, e = O.quantize_mx(block)
    assert int(e[0]) == 0 and float(O.e4m3_decode(q)[0]) == 128.0


def test_mx_round_trip_on_grid_and_error_bound():
    rng = np.random.default_rng(5)
    # values already on an MX grid survive exactly
    e = rng.integers(100, 140, size=(7, 4)).astype(np.uint8)
    codes = rng.integers(0, 0x7F, size=(7, 128)).astype(np.uint8)
    codes[:, ::32] = 0x7E  # every block holds +-448 so the shared exponent is recovered
    x = O.dequantize_mx(codes, e)
    q2, e2 = O.quantize_mx(x)
    np.testing.assert_array_equal(e2, e)
    np.testing.assert_array_equal(O.dequantize_mx(q2, e2), x)
    # random data: rounding errs by at most half a step (<= amax/16); the block maximum itself may
    # saturate from just under 2^(k+1) down to 1.75 * 2^k, an error below amax/8
    x = rng.standard_normal((16, 256)).astype(np.float32)
    q, s = O.quantize_mx(x)
    d = O.dequantize_mx(q, s)
    amax = np.abs(x.reshape(16, 8, 32)).max(-1, keepdims=True)
    assert (np.abs(d - x).reshape(16, 8, 32) <= amax * 2.0 ** -3).all()


def test_mx_torch_twin():
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((33, 96)) * rng.choice([1e-4, 1, 500], (33, 1))).astype(np.float32)
    q, s = O.quantize_mx(x)
    qt, st = O.quantize_mx_torch(torch.from_numpy(x))
    np.testing.assert_array_equal(s, st.numpy())
    np.testing.assert_array_equal(O.e4m3_decode(q), qt.float().numpy())
    np.testing.assert_array_equal(O.dequantize_mx(q, s), O.dequantize_mx_torch(qt, st).numpy())


# ----------------------------------------------------------------------------- forward

def _tiny(seed=0, T=5, K=8, E=3, H=4, k=2, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, K), generator=g, dtype=dtype)
    w1 = torch.randn((E, 2 * H, K), generator=g, dtype=dtype) / K ** 0.5
    w2 = torch.randn((E, K, H), generator=g, dtype=dtype) / H ** 0.5
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    wts = torch.softmax(torch.randn((T, k), generator=g, dtype=dtype), -1)
    return x, w1, w2, ids, wts


def _brute(x, w1, w2, ids, wts):
    """out[t] = sum_r w[t,r] W2[e] (silu(G x) * (U x)), element by element in fp64."""
    T, K = x.shape
    H = w2.shape[2]
    out = torch.zeros((T, K), dtype=torch.float64)
    for t in range(T):
        for r in range(ids.shape[1]):
            e = int(ids[t, r])
            g = [sum(float(w1[e, h, c]) * float(x[t, c]) for c in range(K)) for h in range(H)]
            u = [sum(float(w1[e, H + h, c]) * float(x[t, c]) for c in range(K)) for h in range(H)]
            a = [u[h] * g[h] / (1.0 + np.exp(-g[h])) for h in range(H)]
            for c in range(K):
                out[t, c] += float(wts[t, r]) * sum(float(w2[e, c, h]) * a[h] for h in range(H))
    return out


def test_forward_vs_brute_force():
    x, w1, w2, ids, wts = _tiny()
    ref = _brute(x, w1, w2, ids, wts)
    got = O.fused_moe_dense(x, w1, w2, ids, wts, dtype=torch.float64)
    torch.testing.assert_close(got, ref, rtol=1e-12, atol=1e-12)
    s, e, t = O.moe_align(ids.numpy(), 3, 4, 1)
    got2 = O.fused_moe_sorted(x, w1, w2, s, e, t, wts, 2, block_m=4, dtype=torch.float64)
    torch.testing.assert_close(got2, ref, rtol=1e-12, atol=1e-12)


def test_forward_reduces_to_swiglu_mlp():
    x, w1, w2, _, _ = _tiny(seed=1, E=1, k=1)
    ids = torch.zeros((x.shape[0], 1), dtype=torch.int32)
    wts = torch.ones((x.shape[0], 1), dtype=torch.float64)
    H = w2.shape[2]
    mlp = (torch.nn.functional.silu(x @ w1[0, :H].t()) * (x @ w1[0, H:].t())) @ w2[0].t()
    got = O.fused_moe_dense(x, w1, w2, ids, wts, dtype=torch.float64)
    torch.testing.assert_close(got, mlp, rtol=1e-12, atol=1e-12)


def test_forward_properties():
    x, w1, w2, ids, wts = _tiny(seed=2, T=9, E=4, k=3)
    base = O.fused_moe_dense(x, w1, w2, ids, wts, dtype=torch.float64)
    perm = torch.randperm(9, generator=torch.Generator().manual_seed(0))
    torch.testing.assert_close(O.fused_moe_dense(x[perm], w1, w2, ids[perm], wts[perm], dtype=torch.float64), base[perm])
    # linear in the routing weights; zero gate rows give zero output; swapping gate/up changes it
    torch.testing.assert_close(O.fused_moe_dense(x, w1, w2, ids, 2 * wts, dtype=torch.float64), 2 * base)
    w1z = w1.clone()
    w1z[:, : w1.shape[1] // 2] = 0
    assert O.fused_moe_dense(x, w1z, w2, ids, wts, dtype=torch.float64).abs().max() == 0
    H = w2.shape[2]
    w1s = torch.cat([w1[:, H:], w1[:, :H]], 1)
    assert (O.fused_moe_dense(x, w1s, w2, ids, wts, dtype=torch.float64) - base).abs().max() > 1e-3
    # the same expert twice for a token adds both weights
    ids2 = ids.clone()
    ids2[:, 1] = ids2[:, 0]
    wsum = wts.clone()
    wsum[:, 0] += wsum[:, 1]
    wsum[:, 1] = 0
    a = O.fused_moe_dense(x, w1, w2, ids2, wts, dtype=torch.float64)
    ids3 = ids2.clone()
    ids3[:, 1] = (ids2[:, 0] + 1) % 4  # any other expert with zero weight
    b = O.fused_moe_dense(x, w1, w2, ids3, wsum, dtype=torch.float64)
    torch.testing.assert_close(a, b)


def test_forward_sorted_handles_schedule_edge_cases():
    x, w1, w2, ids, wts = _tiny(seed=4, T=6, E=5, k=2, dtype=torch.float32)
    s, e, t = O.moe_align(ids.numpy(), 5, 4, 1)
    full = O.fused_moe_sorted(x, w1, w2, s, e, t, wts, 2, block_m=4)
    dense = O.fused_moe_dense(x, w1, w2, ids, wts)
    torch.testing.assert_close(full, dense, rtol=1e-5, atol=1e-5)
    # exact-size schedule arrays (what the reference's Python restatement returns) are equivalent
    tot = int(t[0])
    torch.testing.assert_close(O.fused_moe_sorted(x, w1, w2, s[:tot], e[: tot // 4], t, wts, 2, block_m=4), full)
    # pair ids whose token is out of range are dropped (kernel: tok < M check)
    torch.testing.assert_close(O.fused_moe_sorted(x[:4], w1, w2, s, e, t, wts, 2, block_m=4), dense[:4], rtol=1e-5, atol=1e-5)


def test_forward_act_mx_matches_manual():
    x, w1, w2, ids, wts = _tiny(seed=6, T=4, K=16, E=2, H=32, k=1, dtype=torch.float32)
    got = O.fused_moe_dense(x, w1, w2, ids, wts, act_mx=True)
    out = torch.zeros_like(x)
    for t in range(4):
        e = int(ids[t, 0])
        h = w1[e] @ x[t]
        a = O.swiglu(h[:32], h[32:])
        q, s = O.quantize_mx(a.numpy()[None])
        a = torch.from_numpy(O.dequantize_mx(q, s))[0]
        out[t] = wts[t, 0] * (w2[e] @ a)
    torch.testing.assert_close(got, out, rtol=1e-5, atol=1e-6)


def test_flops_model():
    assert O.approx_flops(4096, 2, 4096, 28672) == 3.0 * 8192 * 4096 * 28672


# ----------------------------------------------------------------------------------- routing

def test_route_topk_hand_example_with_ties():
    # values: expert 1 and 3 tie at 2.0 (lower index first), then expert 0 and 4 tie at 1.0
    logits = np.array([[1.0, 2.0, -1.0, 2.0, 1.0, 0.5]], dtype=np.float32)
    ids, w = O.route_topk(logits, 3)
    assert ids.tolist() == [[1, 3, 0]]
    e = np.exp(np.array([0.0, 0.0, -1.0]))
    np.testing.assert_allclose(w[0], e / e.sum(), rtol=1e-6)
    ids, _ = O.route_topk(logits, 6)
    assert ids.tolist() == [[1, 3, 0, 4, 5, 2]]
    # -0 and +0 tie (lower index first); the bias is added before the selection
    ids, _ = O.route_topk(np.array([[0.0, -0.0, -1.0]], dtype=np.float32), 2)
    assert ids.tolist() == [[0, 1]]
    ids, w = O.route_topk(np.array([[0.0, 0.0, 0.0]], dtype=np.float32), 1, bias=np.array([0.0, 0.0, 1.0]))
    assert ids.tolist() == [[2]] and w.tolist() == [[1.0]]


@pytest.mark.parametrize("T,E,k", [(64, 8, 2), (33, 128, 8), (5, 1000, 32), (7, 1, 1)])
def test_route_topk_matches_torch_on_tie_free_inputs(T, E, k):
    g = torch.Generator().manual_seed(T + E)
    logits = torch.randn((T, E), generator=g)
    assert all(torch.unique(row).numel() == E for row in logits)  # no ties: torch.topk's order is then unique
    vals, idx = torch.topk(logits, k, dim=-1)
    ids, w = O.route_topk(logits.numpy(), k)
    np.testing.assert_array_equal(ids, idx.numpy().astype(np.int32))
    np.testing.assert_allclose(w, torch.softmax(vals.float(), -1).numpy(), rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(w.sum(1), 1.0, rtol=1e-6)


def test_forward_by_expert_equals_dense_and_subset_masks():
    x, w1, w2, ids, wts = _tiny(seed=9, T=12, K=16, E=5, H=32, k=3, dtype=torch.float32)
    fetch = lambda e: (w1[e], w2[e])
    for act_mx in (False, True):
        dense = O.fused_moe_dense(x, w1, w2, ids, wts, act_mx=act_mx)
        torch.testing.assert_close(O.fused_moe_by_expert(x, fetch, ids, wts, 5, act_mx=act_mx), dense, rtol=1e-6, atol=1e-6)
        # a subset of experts == the dense result with the other pairs' routing weights zeroed
        keep = (ids == 1) | (ids == 3)
        masked = O.fused_moe_dense(x, w1, w2, ids, wts * keep, act_mx=act_mx)
        torch.testing.assert_close(O.fused_moe_by_expert(x, fetch, ids, wts, 5, act_mx=act_mx, experts=[3, 1]),
                                   masked, rtol=1e-6, atol=1e-6)


def test_mx_flip_spacing_marks_what_can_flip_and_bounds_the_change():
    # hand-placed values in one block whose amax 3.0 gives the scale 2^-7 (scaled amax 384, spacing 32 there):
    # 0.40625 = 52 * 2^-7 is a code (spacing 4 in [32, 64)), 0.421875 = 54 * 2^-7 the midpoint to the next one
    # (56), 0.4296875 = 55 * 2^-7 lies a quarter spacing from it
    row = torch.zeros(32, dtype=torch.float64)
    row[0], row[1], row[2], row[3] = 3.0, 0.40625, 0.421875, 0.4296875
    row[4] = 0.421875 * (1 + 5e-5)   # within 1e-4 of the midpoint
    row[5] = 0.421875 * (1 + 3e-4)   # outside
    sp = O.mx_flip_spacing(row.view(1, 32), 1e-4)[0]
    assert sp[0] == 0 and sp[1] == 0 and sp[3] == 0 and sp[5] == 0
    assert sp[2] == 4 * 2.0 ** -7 and sp[4] == 4 * 2.0 ** -7
    # amax next to a power of two: the scale may come out either way, the whole block is marked with the spacing
    # of the coarser grid
    row2 = row.clone()
    row2[0] = 4.0 * (1 - 2e-5)
    sp2 = O.mx_flip_spacing(row2.view(1, 32), 1e-4)[0]
    assert (sp2 > 0).all() and sp2[1] == 2 * 4 * 2.0 ** -7
    # random activations moved by less than the margin: only marked elements change, by no more than the spacing
    g = torch.Generator().manual_seed(4)
    act = torch.randn((128, 256), generator=g, dtype=torch.float64) * 3
    sp = O.mx_flip_spacing(act, 1e-4)
    assert 0 < float((sp > 0).double().mean()) < 0.01
    changed = 0
    for _ in range(8):
        moved = act * (1 + (torch.rand(act.shape, generator=g, dtype=torch.float64) * 2 - 1) * 0.9e-4)
        d0 = O.dequantize_mx_torch(*O.quantize_mx_torch(act.float())).double()
        d1 = O.dequantize_mx_torch(*O.quantize_mx_torch(moved.float())).double()
        diff = (d0 - d1).abs()
        assert bool((diff <= sp + 1e-12).all())
        changed += int((diff > 0).sum())
    assert changed > 0


def test_flip_bound_of_the_forward_pass():
    # the bound is zero where no activation can flip, and covers the difference between two evaluations of the
    # forward pass whose activations differ by less than the margin
    g = torch.Generator().manual_seed(9)
    T, K, E, N, top_k = 24, 64, 3, 128, 2
    x = torch.randn((T, K), generator=g)
    w1 = torch.randn((E, N, K), generator=g) / K ** 0.5
    w2 = torch.randn((E, K, N // 2), generator=g) / (N // 2) ** 0.5
    ids = torch.stack([torch.randperm(E, generator=g)[:top_k] for _ in range(T)]).to(torch.int32)
    wts = torch.softmax(torch.randn((T, top_k), generator=g), -1)
    ref, bound = O.fused_moe_dense(x, w1, w2, ids, wts, act_mx=True, flip_delta=1e-4)
    assert bound.shape == ref.shape and float(bound.min()) >= 0
    other = O.fused_moe_dense(x * (1 + 2e-5), w1, w2, ids, wts, act_mx=True)  # every activation moves by ~4e-5
    rest = ((other.double() - ref.double()).abs() - bound).clamp_min(0)
    assert float(rest.max()) <= 2e-4 * float(ref.abs().max())
