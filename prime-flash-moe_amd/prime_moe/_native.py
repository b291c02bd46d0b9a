"""ctypes binding of libprime_moe_hip.so (the C ABI declared in include/prime_moe_hip.h).

The library is built in-tree by :mod:`prime_moe.build`.  There is no fallback: if it is
missing, every op raises with the build command instead of computing anything elsewhere.
"""
from __future__ import annotations

import ctypes
import os

LIB_NAME = "libprime_moe_hip.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

_c_int = ctypes.c_int
_c_void_p = ctypes.c_void_p
_c_size_t = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/prime_moe_hip.h one to one
SIGNATURES = {
    "pmoe_version": (_c_int, []),
    "pmoe_last_error": (ctypes.c_char_p, []),
    "pmoe_moe_align": (_c_int, [_c_void_p] * 4 + [_c_int] * 6 + [_c_void_p]),
    "pmoe_moe_align_workspace_bytes": (_c_size_t, [_c_int] * 2),
    "pmoe_moe_align_ws": (_c_int, [_c_void_p] * 4 + [_c_int] * 6 + [_c_void_p, _c_size_t, _c_void_p]),
    "pmoe_moe_align_static": (_c_int, [_c_void_p] * 4 + [_c_int] * 6 + [_c_void_p]),
    "pmoe_fused_moe_bf16_workspace_bytes": (_c_size_t, [_c_int] * 7),
    "pmoe_fused_moe_mxfp8_workspace_bytes": (_c_size_t, [_c_int] * 7),
    "pmoe_fused_moe_bf16": (_c_int, [_c_void_p] * 8 + [_c_int] * 13 + [_c_void_p, _c_size_t, _c_void_p]),
    "pmoe_fused_moe_mxfp8": (_c_int, [_c_void_p] * 11 + [_c_int] * 12 + [_c_void_p, _c_size_t, _c_void_p]),
    "pmoe_quantize_mx": (_c_int, [_c_void_p] * 3 + [ctypes.c_int64, _c_int, _c_void_p]),
    "pmoe_route": (_c_int, [_c_void_p, _c_int] + [_c_void_p] * 6 + [_c_int] * 7 + [_c_void_p, _c_size_t, _c_void_p]),
    "pmoe_set_phase_mask": (None, [_c_int]),
    "pmoe_set_tiles_per_workgroup": (None, [_c_int]),
    "pmoe_copy_calibration": (_c_int, [_c_void_p, _c_void_p, ctypes.c_int64, _c_void_p]),
    "pmoe_poison_lds": (_c_int, [_c_void_p, _c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Loads the library once; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"prime_moe: {LIB_PATH} is missing. Build the HIP library first: "
            "python prime-flash-moe_amd/prime_moe/build.py (there is no fallback path)."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the header and the library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    """Turns a non-zero C status into the RuntimeError the reference's TORCH_CHECKs raise."""
    if status != 0:
        msg = load().pmoe_last_error()
        raise RuntimeError(msg.decode("utf-8", "replace") if msg else f"prime_moe native error {status}")
