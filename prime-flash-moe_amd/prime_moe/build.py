"""Builds libprime_moe_hip.so (the C-ABI library) in-tree with hipcc for gfx950.

Usage: ``python -m prime_moe.build`` (with ``prime-flash-moe_amd`` on ``sys.path``) or
``python prime-flash-moe_amd/prime_moe/build.py``.  The library lands next to this file so that
``prime_moe._native`` finds it; nothing is installed outside the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_NAME = "libprime_moe_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["api.hip", "moe_align.hip", "route.hip", "quantize_mx.hip", "fused_moe.hip", "fused_moe_bf16.hip"]
ARCH = "gfx950"

# Packed-fp32 VALU forms are switched off for every device compile.
# Private arrays are never moved into LDS by the compiler: the kernels budget LDS themselves.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-mllvm", "-disable-promote-alloca-to-lds"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the prime_moe HIP library cannot be built")
    return exe


def _compile(src: str, verbose: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
           *DEVICE_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
    if verbose and res.stderr.strip():
        # the host pass reports the device-only target feature as unknown; harmless
        lines = [l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if lines:
            print("\n".join(lines), flush=True)
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=6) as pool:
        objs = list(pool.map(lambda s: _compile(s, verbose), SOURCES))
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
