"""Writes tests/golden/fixtures.npz from the CPU oracle (run from the repo root:
``python tests/golden/make_fixtures.py``).  The reference stores no vectors for this path (its
tests draw fresh random inputs), so these are the build's own: small inputs with the outputs the
pinned oracle gives, kept so that a later change of oracle or kernels is caught against fixed data."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import moe_oracle as O  # noqa: E402


def bf16_round(a: np.ndarray) -> np.ndarray:
    return torch.from_numpy(a.astype(np.float32)).to(torch.bfloat16).float().numpy()


def pattern_weights(E, N, K):
    """w1[e,n,k] = ((7n + 13k + 29e) % 31 - 15) / 64,  w2[e,k,h] = ((11k + 5h + 17e) % 29 - 14) / 64."""
    e, n, k = np.meshgrid(np.arange(E), np.arange(N), np.arange(K), indexing="ij")
    w1 = (((7 * n + 13 * k + 29 * e) % 31 - 15) / 64.0).astype(np.float32)
    e, k, h = np.meshgrid(np.arange(E), np.arange(K), np.arange(N // 2), indexing="ij")
    w2 = (((11 * k + 5 * h + 17 * e) % 29 - 14) / 64.0).astype(np.float32)
    return w1, w2


def main():
    rng = np.random.default_rng(20240607)
    fx = {}
    # --- moe_align: empty experts, duplicates inside a token, a hot last expert, bpc = 2 ---
    ids = rng.integers(0, 36, size=(40, 8))
    ids = np.concatenate([ids, np.full((40, 1), 36)], 1)
    ids[3, 0] = ids[3, 1]
    fx["align_ids"] = ids.astype(np.int32)
    for bpc in (1, 2):
        s, e, t = O.moe_align(ids, 37, 128, bpc)
        fx[f"align_sorted_bpc{bpc}"], fx[f"align_experts_bpc{bpc}"], fx[f"align_total_bpc{bpc}"] = s, e, t
    # --- scale packing: index map of a (256, 8) scale matrix ---
    sc = np.arange(256 * 8, dtype=np.int64).reshape(256, 8)
    fx["pack_offsets"] = O.blocked_scale_offset(np.arange(256)[:, None], np.arange(8)[None, :], 8).astype(np.int32)
    fx["pack_in"] = (sc % 251).astype(np.uint8)
    fx["pack_out"] = O.pack_scales_blocked(fx["pack_in"])
    # --- MX known answers: value alone in a block -> (scale byte, code) ---
    kat = np.float32([0.0, 1.0, 3.5, 3.9, 448.0, 449.0, 511.9, 512.0, -3.5, 2.0 ** -120, 1e-3, 57344.0, -0.3])
    blocks = np.zeros((kat.size, 32), dtype=np.float32)
    blocks[:, 0] = kat
    q, e = O.quantize_mx(blocks)
    fx["mx_kat_values"], fx["mx_kat_scale"], fx["mx_kat_code"] = kat, e[:, 0], q[:, 0]
    x = bf16_round(rng.standard_normal((8, 128)) * np.float32([1e-3, 1, 50, 1e4]).repeat(32)[None, :])
    fx["mx_in"] = x
    fx["mx_codes"], fx["mx_scales"] = O.quantize_mx(x)
    # --- tiny end-to-end cases.  Weights follow a closed-form pattern (pattern_weights) instead of
    # being stored: multiples of 1/64 that bf16 holds exactly.  x, routing and outputs are stored. ---
    T, K, E, N, k = 24, 128, 5, 256, 3
    xe = bf16_round(rng.standard_normal((T, K)))
    w1, w2 = pattern_weights(E, N, K)
    tid = np.stack([rng.choice(E, size=k, replace=False) for _ in range(T)]).astype(np.int32)
    lg = rng.standard_normal((T, k)).astype(np.float32)
    tw = (np.exp(lg) / np.exp(lg).sum(-1, keepdims=True)).astype(np.float32)
    tt = lambda a: torch.from_numpy(a)
    fx.update(e2e_x=xe, e2e_ids=tid, e2e_weights=tw)
    fx["e2e_out_bf16path"] = O.fused_moe_dense(tt(xe), tt(w1), tt(w2), tt(tid), tt(tw)).numpy()
    xq, xs = O.quantize_mx(xe)
    w1q, w1s = O.quantize_mx(w1)
    w2q, w2s = O.quantize_mx(w2)
    fx["e2e_out_mxfp8path"] = O.fused_moe_dense(
        tt(O.dequantize_mx(xq, xs)), tt(O.dequantize_mx(w1q, w1s)), tt(O.dequantize_mx(w2q, w2s)),
        tt(tid), tt(tw), act_mx=True).numpy()
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fixtures.npz")
    np.savez_compressed(out, **fx)
    print(out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
