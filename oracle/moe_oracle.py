"""CPU oracle for the fused-MoE forward path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, the algorithms the reference's fused MoE path
implements.  It exists to check the HIP kernels; nothing in the shipped package
may import it.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` use it, and only as the checker.

Every function cites the reference lines it follows (paths relative to the
reference checkout) and names the independent checks that pin it
(``tests/test_oracle.py``).  No function here is "parity unpinned".

  moe_align            prime_moe/csrc/torch_interface.cpp:85-91 (sizes),
                       prime_moe/csrc/kernels/fused_moe_bf16_kernel.cu:853-907
                       (histogram, padded prefix, -1 fill, tail expert ids),
                       test/test.py:81-120 (stable within-expert order).
                       Pinned by: set/size invariants + brute-force recount.
  pack_scales_blocked  prime_moe/__init__.py:106-115; the same layout as the
                       kernels address it: fused_moe_mxfp8_kernel.cu:78,:206,:396.
                       Pinned by: closed-form byte offset vs a gather/scatter.
  e4m3 codec           OCP FP8 E4M3 ("fn": no inf, 0x7f/0xff NaN, max 448).
                       Pinned by: exhaustive 256-code table vs torch casts,
                       round-to-nearest-even known answers.
  quantize_mx / dequantize_mx
                       test/test_mxfp8.py:21-47 == fused_moe_mxfp8_kernel.cu:4-20.
                       Pinned by: hand-derived known answers (amax 0, 1, 3.5,
                       3.9, 448, 449, 512, 2^-120), round trip on exact grids.
  swiglu               prime_moe/csrc/kernels/tcgen05_prelude.cuh:424-426.
  fused_moe_*          test/test.py:13-48, test/test_mxfp8.py:50-77 (dataflow);
                       fp32/fp64 math throughout (the kernels may be more
                       precise than the reference's bf16 roundings, never less).
                       Pinned by: dense per-token brute force in fp64, the
                       top_k=1/E=1 reduction to a plain SwiGLU MLP, token
                       permutation equivariance, duplicate-expert additivity.
  mx_flip_spacing      no counterpart in the reference: which elements of an activation sit so close
                       to a rounding boundary of its MX quantisation (test/test_mxfp8.py:21-38) that
                       two evaluations whose fp32 sums differ in order may quantise them to
                       neighbouring codes, and by how much the dequantised value then differs.
                       Pinned by: hand-placed values on, next to and away from midpoints and binade
                       edges; random activations perturbed by less than the margin change only
                       marked elements, and by no more than the spacing.
  route_topk           the routing the reference's callers do in front of moe_align
                       (README.md:147-149): top-k of the gate logits by value,
                       largest first, ties to the lower expert index, softmax over
                       the selected values.
                       Pinned by: torch.topk + torch.softmax on tie-free inputs, a
                       hand-worked example with ties, weights summing to one.
"""
from __future__ import annotations

import numpy as np
import torch

BLOCK = 32  # MX scale block (prime_moe/__init__.py:103)
E4M3_MAX = 448.0
E4M3_EMAX = 8


# --------------------------------------------------------------------------- moe_align

def moe_align_sizes(n: int, num_experts: int, block_m: int, bpc: int):
    """Output sizes the op allocates (torch_interface.cpp:88-91)."""
    pad_to = block_m * bpc
    max_padded = (n + num_experts * (pad_to - 1) + pad_to - 1) // pad_to * pad_to
    return pad_to, max_padded, max_padded // block_m


def moe_align(topk_ids, num_experts: int, block_m: int, bpc: int = 1):
    """Counting sort of pair ids by expert with per-expert padding.

    Follows fused_moe_bf16_kernel.cu:853-907.  The reference scatters with
    shared-memory atomics, so its within-expert order is a race outcome; this
    oracle fixes it to ascending pair id (what a stable sort gives and what
    test/test.py:94-96 produces), which is one of the legal outcomes.
    Returns numpy int32 arrays (sorted_token_ids[max_padded],
    expert_ids[max_blocks], num_tokens_post_padded[1]).
    """
    ids = np.asarray(topk_ids, dtype=np.int64).reshape(-1)
    n = ids.size
    pad_to, max_padded, max_blocks = moe_align_sizes(n, num_experts, block_m, bpc)
    if n and (ids.min() < 0 or ids.max() >= num_experts):
        raise ValueError("expert id out of range")
    counts = np.zeros(num_experts, dtype=np.int64)
    for e in ids:  # plain histogram (kernel line 873-874)
        counts[e] += 1
    offs = np.zeros(num_experts + 1, dtype=np.int64)
    for e in range(num_experts):  # serial padded prefix (kernel line 876-882)
        offs[e + 1] = offs[e] + (counts[e] + pad_to - 1) // pad_to * pad_to
    total = int(offs[num_experts])
    sorted_ids = np.full(max_padded, -1, dtype=np.int32)
    fill = np.zeros(num_experts, dtype=np.int64)
    for i in range(n):  # scatter in ascending pair id (kernel line 902-906)
        e = ids[i]
        sorted_ids[offs[e] + fill[e]] = i
        fill[e] += 1
    expert_ids = np.empty(max_blocks, dtype=np.int32)
    for j in range(max_blocks):  # kernel line 887-900
        row = j * block_m
        if row >= total:
            expert_ids[j] = num_experts - 1
            continue
        lo, hi = 0, num_experts - 1
        while lo < hi:
            mid = (lo + hi + 1) >> 1
            if offs[mid] <= row:
                lo = mid
            else:
                hi = mid - 1
        expert_ids[j] = lo
    return sorted_ids, expert_ids, np.array([total], dtype=np.int32)


def moe_align_fast(topk_ids, num_experts: int, block_m: int, bpc: int = 1):
    """Vectorised twin of :func:`moe_align` for large inputs (same outputs).

    Checked against the loop version in tests/test_oracle.py.
    """
    ids = np.asarray(topk_ids, dtype=np.int64).reshape(-1)
    n = ids.size
    pad_to, max_padded, max_blocks = moe_align_sizes(n, num_experts, block_m, bpc)
    counts = np.bincount(ids, minlength=num_experts).astype(np.int64)
    padded = (counts + pad_to - 1) // pad_to * pad_to
    offs = np.concatenate([[0], np.cumsum(padded)])
    total = int(offs[-1])
    order = np.argsort(ids, kind="stable")
    starts = np.concatenate([[0], np.cumsum(counts)])[:-1]
    rank = np.arange(n) - np.repeat(starts, counts)
    sorted_ids = np.full(max_padded, -1, dtype=np.int32)
    sorted_ids[offs[ids[order]] + rank] = order
    rows = np.arange(max_blocks, dtype=np.int64) * block_m
    eid = np.searchsorted(offs[1:], rows, side="right")
    # experts with zero rows never own a block: searchsorted(right) skips them
    eid = np.where(rows >= total, num_experts - 1, np.minimum(eid, num_experts - 1))
    return sorted_ids, eid.astype(np.int32), np.array([total], dtype=np.int32)


# --------------------------------------------------------------------------- routing

def route_topk(logits: np.ndarray, top_k: int, bias: np.ndarray = None):
    """Top-k routing in front of moe_align (what the reference's README.md:147-149 leaves to the gate).

    ids[t, r] = expert of the r-th largest value of logits[t] (+ bias), ties to the lower index;
    weights[t] = softmax over the selected values (float64 math, returned as float32).
    The addition of the bias is done in float32, as a gate would.
    """
    v = np.asarray(logits, dtype=np.float32)
    if bias is not None:
        v = (v + np.asarray(bias, dtype=np.float32)[None, :]).astype(np.float32)
    v = v + np.float32(0.0)  # -0 -> +0
    order = np.argsort(-v.astype(np.float64), axis=1, kind="stable")  # stable: equal values keep index order
    ids = order[:, :top_k]
    sel = np.take_along_axis(v, ids, axis=1).astype(np.float64)
    ex = np.exp(sel - sel[:, :1])
    w = ex / ex.sum(axis=1, keepdims=True)
    return ids.astype(np.int32), w.astype(np.float32)


# --------------------------------------------------------------------------- scale packing

def blocked_scale_offset(r, kb, n_kblocks: int):
    """Byte offset of the scale for (row r, 32-wide K block kb) in the blocked layout.

    One 512-byte tile covers 128 rows x 4 K-blocks; tiles are ordered
    [row tile][K tile]; inside a tile the byte sits at
    (r%32)*16 + ((r%128)//32)*4 + kb%4  (fused_moe_mxfp8_kernel.cu:78, :206, :396).
    """
    r = np.asarray(r, dtype=np.int64)
    kb = np.asarray(kb, dtype=np.int64)
    tile = (r // 128) * (n_kblocks // 4) + kb // 4
    return tile * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + kb % 4


def pack_scales_blocked(scales_u8: np.ndarray) -> np.ndarray:
    """Row-major (..., MN, K/32) e8m0 bytes -> blocked tiles (prime_moe/__init__.py:106-115).

    Written as an explicit scatter through :func:`blocked_scale_offset` rather
    than the reference's reshape/permute, so the two statements of the layout
    check each other.
    """
    u = np.ascontiguousarray(scales_u8, dtype=np.uint8)
    mn, kb = u.shape[-2:]
    if mn % 128 or kb % 4:
        raise AssertionError("MN must be a multiple of 128 and K a multiple of 128")
    lead = u.shape[:-2]
    flat = u.reshape(-1, mn, kb)
    out = np.empty((flat.shape[0], mn * kb), dtype=np.uint8)
    rr, kk = np.meshgrid(np.arange(mn), np.arange(kb), indexing="ij")
    off = blocked_scale_offset(rr, kk, kb)
    out[:, off.reshape(-1)] = flat.reshape(flat.shape[0], -1)
    return out.reshape(*lead, mn * kb)


# --------------------------------------------------------------------------- e4m3 / MX

def e4m3_decode_table() -> np.ndarray:
    """All 256 OCP E4M3 ("fn") code points as float32; NaN at 0x7f / 0xff."""
    t = np.empty(256, dtype=np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 7
        if e == 0xF and m == 7:
            t[c] = np.nan
        elif e == 0:
            t[c] = s * m * 2.0 ** -9  # subnormal: m/8 * 2^-6
        else:
            t[c] = s * (1 + m / 8.0) * 2.0 ** (e - 7)
    return t


_E4M3_TABLE = e4m3_decode_table()


def e4m3_decode(codes: np.ndarray) -> np.ndarray:
    return _E4M3_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3_encode_sat(v: np.ndarray) -> np.ndarray:
    """float32 -> E4M3 code, round-to-nearest-even, saturating at +-448.

    Bit-level: values below 2^-6 are rounded on the subnormal grid 2^-9,
    others keep 3 mantissa bits.  NaN encodes as 0x7f.
    """
    v = np.asarray(v, dtype=np.float32)
    sign = (np.signbit(v)).astype(np.uint8) << 7
    a = np.abs(v).astype(np.float64)
    nan = np.isnan(a)
    a = np.where(nan, 0.0, np.minimum(a, E4M3_MAX))
    # exponent of the grid step
    with np.errstate(divide="ignore"):
        ex = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    ex = np.maximum(ex, -6.0)
    step = 2.0 ** (ex - 3)
    q = np.rint(a / step)  # numpy rint = round half to even
    val = q * step  # may have carried into the next binade; still exact
    val = np.minimum(val, E4M3_MAX)
    # re-derive fields from the rounded value
    with np.errstate(divide="ignore"):
        ex2 = np.floor(np.log2(np.where(val > 0, val, 1.0)))
    sub = val < 2.0 ** -6
    ef = np.where(sub, 0, ex2 + 7).astype(np.int64)
    mf = np.where(sub, np.rint(val * 2.0 ** 9), np.rint((val / 2.0 ** ex2 - 1.0) * 8)).astype(np.int64)
    code = (ef << 3 | mf).astype(np.uint8) | sign
    return np.where(nan, np.uint8(0x7F), code).astype(np.uint8)


def shared_exponent(amax: np.ndarray) -> np.ndarray:
    """Biased e8m0 exponent of the MX shared scale (test_mxfp8.py:21-24,
    fused_moe_mxfp8_kernel.cu:4-9): clamp(expfield(amax) - 8, 0, 254)."""
    bits = np.asarray(amax, dtype=np.float32).view(np.uint32)
    e = ((bits >> 23) & 0xFF).astype(np.int64) - E4M3_EMAX
    return np.clip(e, 0, 254)


def quantize_mx(t: np.ndarray, block: int = BLOCK):
    """OCP-MX quantisation of the last axis (test_mxfp8.py:27-38).

    Returns (codes uint8 same shape, scales uint8 shape[:-1]+(K/block,)).
    """
    t = np.asarray(t, dtype=np.float32)
    k = t.shape[-1]
    assert k % block == 0
    g = t.reshape(*t.shape[:-1], k // block, block)
    e = shared_exponent(np.abs(g).max(-1))
    inv = np.ldexp(np.float32(1.0), (127 - e).astype(np.int32)).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        scaled = (g * inv[..., None]).astype(np.float32)
    q = e4m3_encode_sat(np.clip(scaled, -E4M3_MAX, E4M3_MAX))
    return q.reshape(t.shape), e.astype(np.uint8)


def dequantize_mx(q: np.ndarray, scales: np.ndarray, block: int = BLOCK) -> np.ndarray:
    """Inverse of :func:`quantize_mx` in float32 (test_mxfp8.py:41-47)."""
    q = np.asarray(q, dtype=np.uint8)
    k = q.shape[-1]
    e = np.asarray(scales, dtype=np.uint8).astype(np.int32)
    scale = np.ldexp(np.float32(1.0), e - 127).astype(np.float32)
    g = e4m3_decode(q).reshape(*q.shape[:-1], k // block, block) * scale[..., None]
    return g.reshape(q.shape).astype(np.float32)


# torch-side twins used on big tensors (bit-identical to the numpy versions; see
# tests/test_oracle.py::test_mx_torch_twin)

def quantize_mx_torch(t: torch.Tensor, block: int = BLOCK):
    k = t.shape[-1]
    g = t.float().reshape(*t.shape[:-1], k // block, block)
    bits = g.abs().amax(-1).contiguous().view(torch.int32)
    e = (((bits >> 23) & 0xFF) - E4M3_EMAX).clamp_(0, 254)
    inv = torch.exp2((127 - e).float())
    q = (g * inv.unsqueeze(-1)).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return q.reshape(*t.shape[:-1], k).contiguous(), e.to(torch.uint8)


def dequantize_mx_torch(q: torch.Tensor, scales_u8: torch.Tensor, block: int = BLOCK):
    k = q.shape[-1]
    scale = torch.exp2(scales_u8.to(torch.int32).float() - 127.0)
    g = q.float().reshape(*q.shape[:-1], k // block, block) * scale.unsqueeze(-1)
    return g.reshape(*q.shape[:-1], k)


# --------------------------------------------------------------------------- forward

def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """up * gate * sigmoid(gate) (tcgen05_prelude.cuh:424-426; test/test.py:36-37:
    gate = first H rows of w1, up = last H rows)."""
    return up * gate / (1.0 + torch.exp(-gate))


def mx_flip_spacing(act: torch.Tensor, delta: float, block: int = BLOCK) -> torch.Tensor:
    """Per element of ``act`` (rows x H, H % 32 == 0): 0 if the MX quantisation of the element
    (test/test_mxfp8.py:21-38: shared power-of-two scale per 32 elements from the block's amax, e4m3 values,
    round to nearest even, saturating) cannot change when every element moves by less than the relative
    distance ``delta``; otherwise the largest change of its dequantised value, which is the spacing of the
    e4m3 grid at that value times the block's scale:
      * the scaled value lies within ``delta`` (relative) of the midpoint of two neighbouring codes: one
        spacing;
      * the block's amax lies within ``delta`` of a power of two, so that the shared scale may come out one
        step larger or smaller: every element of the block, one spacing of the coarser of the two grids.
    Math in float64."""
    n, H = act.shape
    a = act.double().abs().view(n, H // block, block)
    amax = a.amax(-1)
    # the quantiser's scale: 2^(expfield(amax as fp32) - 8 - 127), expfield clamped as in shared_exponent
    bits = amax.float().view(torch.int32).to(torch.int64)
    e = (((bits >> 23) & 0xff) - E4M3_EMAX).clamp(0, 254)
    scale = torch.pow(torch.tensor(2.0, dtype=torch.float64, device=act.device), (e - 127).double()).unsqueeze(-1)
    s = a / scale
    # spacing of the e4m3 grid at |s|: 2^(floor(log2 s) - 3), binades from 2^-6 (below: subnormals, 2^-9) to 2^8
    _, ex = torch.frexp(s.clamp_min(2.0 ** -20))
    ex = (ex - 1).clamp(-6, 8)
    ulp = torch.pow(torch.tensor(2.0, dtype=torch.float64, device=act.device), (ex - 3).double())
    q = s / ulp
    near_mid = ((q - torch.floor(q) - 0.5).abs() <= delta * q) & (s < E4M3_MAX + 16.0)  # (beyond 464 everything saturates)
    m, _ = torch.frexp(amax.clamp_min(2.0 ** -140))  # amax = m * 2^k, m in [0.5, 1)
    near_pow2 = (((m - 0.5) <= delta * 0.5) | ((1.0 - m) <= delta)) & (amax > 0)
    spacing = torch.where(near_mid, ulp, torch.zeros_like(ulp))
    spacing = torch.where(near_pow2.unsqueeze(-1), 2.0 * ulp, spacing)
    return (spacing * scale).view(n, H)


def fused_moe_dense(x, w1, w2, topk_ids, topk_weights, act_mx: bool = False,
                    dtype=torch.float32, flip_delta: float = None):
    """out[t] = sum_r w[t,r] * W2[e] @ swiglu(W1[e] @ x[t]),  e = topk_ids[t,r].

    Dataflow of test/test.py:13-48 (grouped by expert), all math in ``dtype``
    (fp32 default, fp64 for the brute-force pins).  ``act_mx`` inserts the
    quantise->dequantise of the activation that the mxfp8 path performs before
    the down projection (test_mxfp8.py:70-72; kernel: fused_moe_mxfp8_kernel.cu:375-403,
    which requantises the fp32 SwiGLU value directly).
    x:(T,K) w1:(E,2H,K) w2:(E,K,H) topk_ids:(T,k) int, topk_weights:(T,k).
    ``flip_delta`` (with act_mx): also returns, per output element, how far another evaluation of the same
    dataflow may lie from this one because activations within that relative distance of a rounding boundary
    were quantised to the neighbouring code (see mx_flip_spacing): sum over the token's pairs of
    w * spacing . |W2[e]|; the activations that decide this are computed in float64.
    """
    T, K = x.shape
    E, N, _ = w1.shape
    H = N // 2
    xf = x.to(dtype)
    out = torch.zeros((T, K), dtype=dtype)
    bound = torch.zeros((T, K), dtype=torch.float64) if flip_delta is not None else None
    ids = topk_ids.to(torch.int64)
    wts = topk_weights.to(dtype)
    for e in range(E):
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        h = xf[tok] @ w1[e].to(dtype).t()
        act = swiglu(h[:, :H], h[:, H:])
        if act_mx:
            if bound is not None:
                h64 = x[tok].double() @ w1[e].double().t()
                sp = mx_flip_spacing(swiglu(h64[:, :H], h64[:, H:]), flip_delta)
                bound.index_add_(0, tok, (sp @ w2[e].double().abs().t()) * wts[tok, slot].double().abs()[:, None])
            q, s = quantize_mx_torch(act.float())
            act = dequantize_mx_torch(q, s).to(dtype)
        y = act @ w2[e].to(dtype).t()
        out.index_add_(0, tok, y * wts[tok, slot][:, None])
    return out if bound is None else (out, bound)


def fused_moe_by_expert(x, expert_weights, topk_ids, topk_weights, num_experts: int, act_mx: bool = False,
                        experts=None, dtype=torch.float32, flip_delta: float = None):
    """fused_moe_dense with the weights fetched one expert at a time: ``expert_weights(e)`` returns
    ``(w1_e (2H, K), w2_e (K, H))`` (already dequantised for mxfp8) on the device of ``x``.  Keeps the
    memory of a full-size configuration bounded, and runs wherever ``x`` lives.  ``experts``: only
    these experts contribute (the pairs routed elsewhere add nothing), for checks on a subset.
    Same dataflow and citations as fused_moe_dense; pinned against it in tests/test_oracle.py.
    ``flip_delta``: as in fused_moe_dense, except that the activations that decide the bound are the ``dtype``
    ones (a full-size configuration in float64 would take too long): choose a margin that covers their error.
    """
    T, K = x.shape
    xf = x.to(dtype)
    out = torch.zeros((T, K), dtype=dtype, device=x.device)
    bound = torch.zeros((T, K), dtype=torch.float64, device=x.device) if flip_delta is not None else None
    ids = topk_ids.to(torch.int64)
    wts = topk_weights.to(dtype)
    todo = range(num_experts) if experts is None else sorted(int(e) for e in experts)
    for e in todo:
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        if tok.numel() == 0:
            continue
        w1, w2 = expert_weights(e)
        H = w1.shape[0] // 2
        h = xf[tok] @ w1.to(dtype).t()
        act = swiglu(h[:, :H], h[:, H:])
        if act_mx:
            if bound is not None:
                sp = mx_flip_spacing(act, flip_delta)
                bound.index_add_(0, tok, (sp @ w2.double().abs().t()) * wts[tok, slot].double().abs()[:, None])
            q, s = quantize_mx_torch(act.float())
            act = dequantize_mx_torch(q, s).to(dtype)
        y = act @ w2.to(dtype).t()
        out.index_add_(0, tok, y * wts[tok, slot][:, None])
    return out if bound is None else (out, bound)


def fused_moe_sorted(x, w1, w2, sorted_token_ids, expert_ids, num_tokens_post_padded,
                     topk_weights, top_k: int, block_m: int = 128, act_mx: bool = False,
                     act_bf16: bool = False, dtype=torch.float32) -> torch.Tensor:
    """The op exactly as the kernels see it: driven by the aligned schedule.

    For each row s < total with p = sorted_token_ids[s] >= 0 and token p//top_k < T:
    expert = expert_ids[s // block_m]; contribution w_flat[p] * W2[e] @ act
    (fused_moe_bf16_kernel.cu:69-72, :92-98, :112, :287).  ``act_bf16`` rounds the
    activation to bf16 as the bf16 kernel does (:254).
    """
    T, K = x.shape
    H = w1.shape[1] // 2
    total = int(num_tokens_post_padded.reshape(-1)[0])
    sid = torch.as_tensor(sorted_token_ids).to(torch.int64)[:total]
    eid = torch.as_tensor(expert_ids).to(torch.int64)
    wflat = topk_weights.reshape(-1).to(dtype)
    out = torch.zeros((T, K), dtype=dtype)
    xf = x.to(dtype)
    nblk = (total + block_m - 1) // block_m
    for b in range(nblk):
        rows = sid[b * block_m:(b + 1) * block_m]
        rows = rows[rows >= 0]
        tok = rows // top_k
        keep = tok < T
        rows, tok = rows[keep], tok[keep]
        if rows.numel() == 0:
            continue
        e = int(eid[b])
        h = xf[tok] @ w1[e].to(dtype).t()
        act = swiglu(h[:, :H], h[:, H:])
        if act_bf16:
            act = act.to(torch.bfloat16).to(dtype)
        if act_mx:
            q, s = quantize_mx_torch(act.float())
            act = dequantize_mx_torch(q, s).to(dtype)
        y = act @ w2[e].to(dtype).t()
        out.index_add_(0, tok, y * wflat[rows][:, None])
    return out


def approx_flops(T: int, top_k: int, K: int, N: int) -> float:
    """3*P*K*N, P = T*top_k unpadded pairs (benchmark/benchmark.py:389-391)."""
    return 3.0 * T * top_k * K * N
