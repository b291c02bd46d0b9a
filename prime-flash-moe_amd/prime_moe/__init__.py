"""prime_moe for MI355X (gfx950): the fused-MoE forward behind the reference's op surface.

Drop-in for the reference package (prime_moe/__init__.py:1-122 and the op schemas of
prime_moe/csrc/torch_interface.cpp:271-324): the same three ``prime_moe::`` torch-library
ops with the same schemas, the same Python wrappers returning ``out``, ``BLOCK`` and
``pack_scales_blocked``.  The ops are registered from Python and call hand-written HIP
kernels through the C ABI of ``libprime_moe_hip.so`` (``include/prime_moe_hip.h``); the
PyTorch-ROCm device is dispatch key ``CUDA``.  Argument checks raise ``RuntimeError`` for
the conditions the reference's ``TORCH_CHECK``s reject (torch_interface.cpp:85-87,
:132-155, :208-241).

Extras that the reference leaves to its callers: a fake impl for ``moe_align`` (so all
three ops trace), :func:`quantize_mx`, the OCP-MX quantiser in front of the mxfp8 op, and
:func:`route`, the router front-end (top-k + softmax + ``moe_align``) in front of both.
"""
from __future__ import annotations

import torch

from . import _native

BLOCK = 32  # MX scale block size

_LIB = torch.library.Library("prime_moe", "FRAGMENT")
_LIB.define(
    "fused_moe_bf16(Tensor x, Tensor w, Tensor w2, Tensor sorted_token_ids, Tensor expert_ids, "
    "Tensor num_tokens_post_padded, Tensor topk_weights, Tensor(a!) out, int top_k, int block_m, "
    "int block_n, int warp_n, int stages, int bpc, int cpc, bool split=True) -> ()"
)
_LIB.define(
    "fused_moe_mxfp8(Tensor x, Tensor x_scales, Tensor w, Tensor w_scales, Tensor w2, "
    "Tensor w2_scales, Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, "
    "Tensor topk_weights, Tensor(a!) out, int top_k, int block_m, int block_n, int warp_n, "
    "int stages, int bpc, bool split=True) -> ()"
)
_LIB.define("moe_align(Tensor topk_ids, int num_experts, int block_m, int bpc) -> (Tensor, Tensor, Tensor)")


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)

def _require_same_device(what: str, named: dict, anchor: str = "x") -> None:
    """Every tensor must live on the GPU of `anchor`: the kernels take raw device pointers, so a CPU
    tensor (or one on another GPU) would be a memory fault on the device, not an exception."""
    dev = named[anchor].device
    _require(dev.type == "cuda", f"{what}: {anchor} must be a GPU tensor, got device {dev}")
    for name, t in named.items():
        _require(t.device == dev, f"{what}: {name} is on {t.device}, expected {dev} (the device of {anchor})")


def _require_aligned(what: str, named: dict, names, align: int) -> None:
    """The kernels read these with `align`-byte vector loads from the start of the tensor."""
    for name in names:
        _require(named[name].data_ptr() % align == 0,
                 f"{what}: {name} must start at a {align}-byte aligned address")


def _stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    # torch's caching allocator: stream ordered, no hipMalloc in steady state, graph-capture safe
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


# ------------------------------------------------------------------------------- moe_align

def align_sizes(n: int, num_experts: int, block_m: int, bpc: int):
    """(pad_to, max_padded, max_blocks) as torch_interface.cpp:88-91 computes them."""
    pad_to = block_m * bpc
    max_padded = (n + num_experts * (pad_to - 1) + pad_to - 1) // pad_to * pad_to
    return pad_to, max_padded, max_padded // block_m


def _validate_align(topk_ids: torch.Tensor, num_experts: int, block_m: int, bpc: int, placement: bool = True) -> None:
    _require(topk_ids.is_cuda or not placement, f"moe_align: topk_ids must be a GPU tensor, got device {topk_ids.device}")
    _require(topk_ids.is_contiguous(), "moe_align: topk_ids must be contiguous")
    _require(topk_ids.dtype == torch.int32, "moe_align: topk_ids must be int32")
    _require(block_m > 0 and bpc > 0 and num_experts > 0, "moe_align: block_m, bpc and num_experts must be positive")
    _require(num_experts <= 1024, f"moe_align supports at most 1024 experts, got {num_experts}")


def _moe_align_impl(topk_ids, num_experts, block_m, bpc):
    _validate_align(topk_ids, num_experts, block_m, bpc)
    n = topk_ids.numel()
    pad_to, max_padded, max_blocks = align_sizes(n, num_experts, block_m, bpc)
    dev = topk_ids.device
    sorted_token_ids = torch.empty((max_padded,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty((max_blocks,), dtype=torch.int32, device=dev)
    num_tokens_post_padded = torch.empty((1,), dtype=torch.int32, device=dev)
    lib = _native.load()
    # many ids: scratch for the multi-workgroup sort (0 bytes when one workgroup does it)
    ws_bytes = lib.pmoe_moe_align_workspace_bytes(n, num_experts)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev) if ws_bytes else None
    with torch.cuda.device(dev):
        _native.check(lib.pmoe_moe_align_ws(
            topk_ids.data_ptr(), sorted_token_ids.data_ptr(), expert_ids.data_ptr(),
            num_tokens_post_padded.data_ptr(), n, num_experts, block_m, pad_to, max_padded,
            max_blocks, ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(dev)))
    return sorted_token_ids, expert_ids, num_tokens_post_padded


def _moe_align_fake(topk_ids, num_experts, block_m, bpc):
    _, max_padded, max_blocks = align_sizes(topk_ids.numel(), num_experts, block_m, bpc)
    mk = lambda n: torch.empty((n,), dtype=torch.int32, device=topk_ids.device)
    return mk(max_padded), mk(max_blocks), mk(1)


# ------------------------------------------------------------------------------- fused_moe_bf16

def _check_tuning(block_m, block_n, warp_n, stages, max_stages, what):
    _require((block_n == 64 and warp_n == 4) or (block_n == 32 and warp_n == 8),
             f"{what}: (block_n, warp_n) must be (64, 4) or (32, 8), got ({block_n}, {warp_n})")
    _require(0 < stages <= max_stages, f"{what} supports stages in 1..{max_stages}, got {stages}")
    _require(block_m == 128, f"{what} requires block_m=128, got {block_m}")


def _validate_bf16(x, w, w2, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, out,
                   top_k, block_m, block_n, warp_n, stages, bpc, cpc, split, placement: bool = True) -> None:
    """Argument checks of the op.  `placement=False` skips the device and alignment checks (what is
    left can then be exercised with CPU tensors)."""
    _require(x.dim() == 2 and w.dim() == 3 and w2.dim() == 3, "fused_moe_bf16: x must be 2-D, w and w2 3-D")
    _require(x.size(0) > 0, "fused_moe_bf16: x has no rows")
    _require(x.size(1) == w.size(2), "fused_moe_bf16: x.size(1) must equal w.size(2)")
    _require(x.size(1) % 128 == 0, "K dimension must be a multiple of 128")
    _require(w.size(1) % 256 == 0, f"fused_moe_bf16: N must be a multiple of 256, got {w.size(1)}")
    _require(tuple(w2.shape) == (w.size(0), x.size(1), w.size(1) // 2),
             "fused_moe_bf16: w2 must have shape (E, K, N/2)")
    _check_tuning(block_m, block_n, warp_n, stages, 5, "fused_moe_bf16")
    _require(bpc == 1 and cpc == 1, "bpc=cpc=1 is the only supported configuration")
    _require((not split) or stages <= 4, f"split=True requires stages<=4, got stages={stages}")
    _require(top_k > 0, "fused_moe_bf16: top_k must be positive")
    named = dict(x=x, w=w, w2=w2, sorted_token_ids=sorted_token_ids, expert_ids=expert_ids,
                 num_tokens_post_padded=num_tokens_post_padded, topk_weights=topk_weights, out=out)
    if placement:
        _require_same_device("fused_moe_bf16", named)
        _require_aligned("fused_moe_bf16", named, ("x", "w", "w2", "out"), 16)
        _require_aligned("fused_moe_bf16", named, ("sorted_token_ids", "expert_ids", "num_tokens_post_padded",
                                                   "topk_weights"), 4)
    for name, t in named.items():
        _require(t.is_contiguous(), f"fused_moe_bf16: {name} must be contiguous")
    for name in ("x", "w", "w2", "out"):
        _require(named[name].dtype == torch.bfloat16, f"fused_moe_bf16: {name} must be bfloat16")
    _require(topk_weights.dtype == torch.float32, "fused_moe_bf16: topk_weights must be float32")
    for name in ("sorted_token_ids", "expert_ids", "num_tokens_post_padded"):
        _require(named[name].dtype == torch.int32, f"fused_moe_bf16: {name} must be int32")
    _require(tuple(out.shape) == tuple(x.shape), "fused_moe_bf16: out must have the shape of x")
    _require(num_tokens_post_padded.numel() >= 1, "fused_moe_bf16: num_tokens_post_padded is empty")
    _require(expert_ids.numel() * block_m >= sorted_token_ids.numel(),
             "fused_moe_bf16: expert_ids is shorter than sorted_token_ids / block_m")


def _fused_moe_bf16_impl(x, w, w2, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights,
                         out, top_k, block_m, block_n, warp_n, stages, bpc, cpc, split=True):
    _validate_bf16(x, w, w2, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, out,
                   top_k, block_m, block_n, warp_n, stages, bpc, cpc, split)
    lib = _native.load()
    M, K = x.shape
    E, N = w.size(0), w.size(1)
    S = sorted_token_ids.size(0)
    dev = x.device
    with torch.cuda.device(dev):
        nbytes = lib.pmoe_fused_moe_bf16_workspace_bytes(M, K, N, E, S, top_k, int(split))
        ws = _workspace(nbytes, dev)
        _native.check(lib.pmoe_fused_moe_bf16(
            x.data_ptr(), w.data_ptr(), w2.data_ptr(), out.data_ptr(), sorted_token_ids.data_ptr(),
            expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(), topk_weights.data_ptr(),
            top_k, M, K, N, E, S, block_m, block_n, warp_n, stages, bpc, cpc, int(split),
            ws.data_ptr(), ws.numel(), _stream_ptr(dev)))
    return None


def _fused_moe_bf16_fake(x, w, w2, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights,
                         out, top_k, block_m, block_n, warp_n, stages, bpc, cpc, split=True):
    return None


# ------------------------------------------------------------------------------- fused_moe_mxfp8

def _validate_mxfp8(x, x_scales, w, w_scales, w2, w2_scales, sorted_token_ids, expert_ids,
                    num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n, stages,
                    bpc, split, placement: bool = True) -> None:
    """Argument checks of the op.  `placement=False` skips the device and alignment checks."""
    _require(x.dim() == 2 and w.dim() == 3 and w2.dim() == 3, "fused_moe_mxfp8: x must be 2-D, w and w2 3-D")
    M, K = x.shape
    E, N = w.size(0), w.size(1)
    _require(M > 0, "fused_moe_mxfp8: x has no rows")
    _require(K == w.size(2), "fused_moe_mxfp8: x.size(1) must equal w.size(2)")
    _require(K % 256 == 0, "K dimension must be a multiple of 256 on the mxfp8 path")
    _require(N % 256 == 0, "N dimension must be a multiple of 256 on the mxfp8 path")
    _require(tuple(w2.shape) == (E, K, N // 2), "fused_moe_mxfp8: w2 must have shape (E, K, N/2)")
    _check_tuning(block_m, block_n, warp_n, stages, 4, "mxfp8")
    _require(bpc == 1, "mxfp8 supports bpc=1 only")
    _require(top_k > 0, "fused_moe_mxfp8: top_k must be positive")
    _require(x_scales.numel() == M * (K // 32), "x_scales must be a row major (M, K/32) e8m0 tensor")
    _require(w_scales.numel() == E * N * (K // 32), "w_scales must hold E*N*K/32 e8m0 values in the blocked layout")
    _require(w2_scales.numel() == E * K * ((N // 2) // 32),
             "w2_scales must hold E*K*(N/2)/32 e8m0 values in the blocked layout")
    named = dict(x=x, x_scales=x_scales, w=w, w_scales=w_scales, w2=w2, w2_scales=w2_scales,
                 sorted_token_ids=sorted_token_ids, expert_ids=expert_ids,
                 num_tokens_post_padded=num_tokens_post_padded, topk_weights=topk_weights, out=out)
    if placement:
        _require_same_device("fused_moe_mxfp8", named)
        _require_aligned("fused_moe_mxfp8", named, ("x", "w", "w2", "out"), 16)
        _require_aligned("fused_moe_mxfp8", named, ("x_scales", "w_scales", "w2_scales", "sorted_token_ids",
                                                    "expert_ids", "num_tokens_post_padded", "topk_weights"), 4)
    for name, t in named.items():
        _require(t.is_contiguous(), f"fused_moe_mxfp8: {name} must be contiguous")
    for name in ("x", "w", "w2"):
        _require(named[name].dtype == torch.float8_e4m3fn, f"fused_moe_mxfp8: {name} must be float8_e4m3fn")
    for name in ("x_scales", "w_scales", "w2_scales"):
        _require(named[name].dtype == torch.float8_e8m0fnu, f"fused_moe_mxfp8: {name} must be float8_e8m0fnu")
    _require(topk_weights.dtype == torch.float32, "fused_moe_mxfp8: topk_weights must be float32")
    for name in ("sorted_token_ids", "expert_ids", "num_tokens_post_padded"):
        _require(named[name].dtype == torch.int32, f"fused_moe_mxfp8: {name} must be int32")
    _require(out.dtype == torch.bfloat16, "fused_moe_mxfp8: out must be bfloat16")
    _require(tuple(out.shape) == (M, K), "fused_moe_mxfp8: out must have shape (M, K)")
    _require(num_tokens_post_padded.numel() >= 1, "fused_moe_mxfp8: num_tokens_post_padded is empty")
    _require(expert_ids.numel() * block_m >= sorted_token_ids.numel(),
             "fused_moe_mxfp8: expert_ids is shorter than sorted_token_ids / block_m")


def _fused_moe_mxfp8_impl(x, x_scales, w, w_scales, w2, w2_scales, sorted_token_ids, expert_ids,
                          num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n,
                          stages, bpc, split=True):
    _validate_mxfp8(x, x_scales, w, w_scales, w2, w2_scales, sorted_token_ids, expert_ids,
                    num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n, stages,
                    bpc, split)
    lib = _native.load()
    M, K = x.shape
    E, N = w.size(0), w.size(1)
    S = sorted_token_ids.size(0)
    dev = x.device
    with torch.cuda.device(dev):
        nbytes = lib.pmoe_fused_moe_mxfp8_workspace_bytes(M, K, N, E, S, top_k, int(split))
        ws = _workspace(nbytes, dev)
        _native.check(lib.pmoe_fused_moe_mxfp8(
            x.data_ptr(), x_scales.data_ptr(), w.data_ptr(), w_scales.data_ptr(), w2.data_ptr(),
            w2_scales.data_ptr(), out.data_ptr(), sorted_token_ids.data_ptr(), expert_ids.data_ptr(),
            num_tokens_post_padded.data_ptr(), topk_weights.data_ptr(), top_k, M, K, N, E, S,
            block_m, block_n, warp_n, stages, bpc, int(split), ws.data_ptr(), ws.numel(),
            _stream_ptr(dev)))
    return None


def _fused_moe_mxfp8_fake(x, x_scales, w, w_scales, w2, w2_scales, sorted_token_ids, expert_ids,
                          num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n,
                          stages, bpc, split=True):
    return None


_LIB.impl("moe_align", _moe_align_impl, "CUDA")
_LIB.impl("fused_moe_bf16", _fused_moe_bf16_impl, "CUDA")
_LIB.impl("fused_moe_mxfp8", _fused_moe_mxfp8_impl, "CUDA")
torch.library.register_fake("prime_moe::moe_align", _moe_align_fake, lib=_LIB)
torch.library.register_fake("prime_moe::fused_moe_bf16", _fused_moe_bf16_fake, lib=_LIB)
torch.library.register_fake("prime_moe::fused_moe_mxfp8", _fused_moe_mxfp8_fake, lib=_LIB)


# ------------------------------------------------------------------------------- public wrappers

def fused_moe_bf16(x, w, w2, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, out,
                   top_k: int, block_m: int, block_n: int, warp_n: int, stages: int, bpc: int = 1,
                   cpc: int = 1, split: bool = True) -> torch.Tensor:
    """Runs ``prime_moe::fused_moe_bf16`` and returns ``out`` (reference __init__.py:27-49)."""
    torch.ops.prime_moe.fused_moe_bf16(
        x, w, w2, sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, out,
        top_k, block_m, block_n, warp_n, stages, bpc, cpc, split)
    return out


def fused_moe_mxfp8(x, x_scales, w, w_scales, w2, w2_scales, sorted_token_ids, expert_ids,
                    num_tokens_post_padded, topk_weights, out, top_k: int, block_m: int, block_n: int,
                    warp_n: int, stages: int, bpc: int = 1, split: bool = True) -> torch.Tensor:
    """Runs ``prime_moe::fused_moe_mxfp8`` and returns ``out`` (reference __init__.py:75-100)."""
    torch.ops.prime_moe.fused_moe_mxfp8(
        x, x_scales, w, w_scales, w2, w2_scales, sorted_token_ids, expert_ids,
        num_tokens_post_padded, topk_weights, out, top_k, block_m, block_n, warp_n, stages, bpc, split)
    return out


def pack_scales_blocked(scales: torch.Tensor) -> torch.Tensor:
    """Row-major ``(..., MN, K/32)`` e8m0 scales -> the 128x4 blocked tiles the kernels read.

    Layout contract of the reference (__init__.py:106-115): tiles of 128 rows x 4 K-blocks, 512
    bytes each, ordered [row tile][K tile]; inside a tile the scale of (row r, block b) is byte
    ``(r % 32) * 16 + (r % 128 // 32) * 4 + b % 4``, so the four scales of one row over 128
    consecutive K form one aligned 32-bit word.  Load-time work, plain torch.
    """
    u = scales.view(torch.uint8)
    mn, kb = u.shape[-2], u.shape[-1]
    assert mn % 128 == 0, f"MN ({mn}) must be a multiple of 128"
    assert kb % 4 == 0, f"K ({kb * 32}) must be a multiple of 128"
    lead = u.shape[:-2]
    # axes: [lead, row tile, quarter (r%128//32), r%32, K tile, b%4] -> [lead, row tile, K tile, r%32, quarter, b%4]
    tiles = u.reshape(-1, mn // 128, 4, 32, kb // 4, 4).permute(0, 1, 4, 3, 2, 5)
    return tiles.contiguous().reshape(*lead, -1).view(torch.float8_e8m0fnu)


def quantize_mx(t: torch.Tensor):
    """OCP-MX quantisation of the last dimension of a bf16 tensor on the GPU.

    Returns ``(float8_e4m3fn values, float8_e8m0fnu scales)`` with scales of shape
    ``t.shape[:-1] + (K // 32,)`` row major -- the format ``fused_moe_mxfp8`` takes for ``x``
    and, after :func:`pack_scales_blocked`, for the weights (specification: the reference's
    test/test_mxfp8.py:21-38).
    """
    _require(t.is_cuda, "quantize_mx: a GPU tensor is required")
    _require(t.dtype == torch.bfloat16, "quantize_mx: bfloat16 input required")
    _require(t.is_contiguous(), "quantize_mx: input must be contiguous")
    cols = t.shape[-1]
    _require(cols % BLOCK == 0, f"quantize_mx: last dim {cols} must be a multiple of {BLOCK}")
    rows = t.numel() // cols
    q = torch.empty(t.shape, dtype=torch.float8_e4m3fn, device=t.device)
    s = torch.empty(t.shape[:-1] + (cols // BLOCK,), dtype=torch.uint8, device=t.device)
    lib = _native.load()
    with torch.cuda.device(t.device):
        _native.check(lib.pmoe_quantize_mx(t.data_ptr(), q.data_ptr(), s.data_ptr(), rows, cols,
                                           _stream_ptr(t.device)))
    return q, s.view(torch.float8_e8m0fnu)


def route(logits: torch.Tensor, top_k: int, block_m: int = 128, bpc: int = 1, bias: torch.Tensor = None):
    """Router front-end: gate logits ``(T, E)`` -> top-k, softmax weights and the ``moe_align`` schedule.

    The step the reference leaves to its callers (README.md:147-149): returns
    ``(topk_ids (T, top_k) int32, topk_weights (T, top_k) fp32, sorted_token_ids, expert_ids,
    num_tokens_post_padded)``; the last three are what ``torch.ops.prime_moe.moe_align(topk_ids, E,
    block_m, bpc)`` returns.  Selection: the ``top_k`` largest of ``logits[t] (+ bias)``, largest first,
    ties to the lower expert index; weights: softmax over the selected values in fp32.  One top-k kernel
    plus the align kernels on the current stream, no host synchronisation.
    """
    _require(logits.is_cuda, f"route: logits must be a GPU tensor, got device {logits.device}")
    _require(logits.dim() == 2 and logits.is_contiguous(), "route: logits must be a contiguous (T, E) tensor")
    _require(logits.dtype in (torch.float32, torch.bfloat16), "route: logits must be float32 or bfloat16")
    T, E = logits.shape
    _require(0 < E <= 1024, f"route supports 1..1024 experts, got {E}")
    _require(0 < top_k <= min(32, E), f"route: top_k must be in 1..min(32, E), got {top_k}")
    _require(block_m > 0 and bpc > 0, "route: block_m and bpc must be positive")
    if bias is not None:
        _require(bias.device == logits.device and bias.dtype == torch.float32 and bias.is_contiguous()
                 and bias.numel() == E, "route: bias must be a contiguous float32 (E,) tensor on the device of logits")
    dev = logits.device
    n = T * top_k
    pad_to, max_padded, max_blocks = align_sizes(n, E, block_m, bpc)
    topk_ids = torch.empty((T, top_k), dtype=torch.int32, device=dev)
    topk_weights = torch.empty((T, top_k), dtype=torch.float32, device=dev)
    sorted_token_ids = torch.empty((max_padded,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty((max_blocks,), dtype=torch.int32, device=dev)
    num_tokens_post_padded = torch.empty((1,), dtype=torch.int32, device=dev)
    lib = _native.load()
    ws_bytes = lib.pmoe_moe_align_workspace_bytes(n, E)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev) if ws_bytes else None
    with torch.cuda.device(dev):
        _native.check(lib.pmoe_route(
            logits.data_ptr(), 0 if logits.dtype == torch.float32 else 1,
            bias.data_ptr() if bias is not None else None, topk_ids.data_ptr(), topk_weights.data_ptr(),
            sorted_token_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(), T, E, top_k,
            block_m, pad_to, max_padded, max_blocks, ws.data_ptr() if ws is not None else None, ws_bytes,
            _stream_ptr(dev)))
    return topk_ids, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded


__all__ = [
    "route",
    "fused_moe_bf16",
    "fused_moe_mxfp8",
    "pack_scales_blocked",
    "quantize_mx",
    "BLOCK",
]
