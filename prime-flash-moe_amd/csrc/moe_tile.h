// Device-side tile engine shared by the fused-MoE kernels (gfx950, wave64).
//
// One workgroup = 256 threads = 4 waves and owns a (128 sorted rows) x (256 weight rows)
// tile of a grouped GEMM whose two operands are both contiguous along the contraction
// dimension:  token rows (x or the activation) and weight rows (W1 or W2 of one expert).
// The contraction is consumed in slabs of 128 bytes per row (64 bf16 or 128 e4m3), staged
// through LDS with a double buffer: while the MFMAs of slab k run out of one buffer, the
// global loads of slab k+1 are in flight into registers and are written to the other buffer.
//
// LDS layout of one stage: [384 rows][128 B]; rows 0..127 token rows, 128..383 weight rows.
// A row is 8 chunks of 16 B; chunk c of row r is stored in slot c ^ ((r >> 1) & 7), which
// makes the 16-byte MFMA operand reads of 16 consecutive rows hit all 64 banks once.
//
// MFMA shapes: v_mfma_f32_32x32x16_bf16 (4 per slab) and v_mfma_scale_f32_32x32x64_f8f6f4
// (2 per slab, e4m3 operands, e8m0 scales: lane l supplies the scale of (row l%32, K block l/32)).
// Lane l supplies row l%32; accumulator register i of lane l is element
// (m = 8*(i/4) + 4*(l/32) + i%4, n = l%32).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pmoe {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kTokRows = 128;   // sorted rows per block (= block_m)
constexpr int kWRows = 256;     // weight rows per tile
constexpr int kRowBytes = 128;  // contraction bytes per LDS row
constexpr int kTokRegion = kTokRows * kRowBytes;             // 16 KB
constexpr int kStageBytes = (kTokRows + kWRows) * kRowBytes;  // 48 KB
constexpr int kNumStages = 2;

enum : int { DT_BF16 = 0, DT_FP8 = 1 };

__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ float swiglu(float gate, float up) {
    return up * gate / (1.0f + __expf(-gate));
}

// OCP-MX shared scale of a 32-block with absolute maximum `amax`:
// e = clamp(expfield(amax) - 8, 0, 254); returns e and 2^(127-e) (0 when e == 254).
__device__ __forceinline__ void mx_block_scale(float amax, uint32_t &e8m0, float &inv) {
    int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 8;
    e = max(0, min(254, e));
    e8m0 = (uint32_t)e;
    inv = __uint_as_float((uint32_t)(254 - e) << 23);
}

// four fp32 -> four e4m3 bytes (round to nearest even, saturating at +-448), packed little endian
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d, float inv) {
    a = __builtin_amdgcn_fmed3f(a * inv, -448.0f, 448.0f);
    b = __builtin_amdgcn_fmed3f(b * inv, -448.0f, 448.0f);
    c = __builtin_amdgcn_fmed3f(c * inv, -448.0f, 448.0f);
    d = __builtin_amdgcn_fmed3f(d * inv, -448.0f, 448.0f);
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
    return (uint32_t)w;
}

// Byte offset of the 4-scale dword of weight row `row` for K tile `kt` (128 wide) in the blocked
// scale layout [row/128][kt][512 B]; inside a tile: (row%32)*16 + ((row%128)/32)*4.
__device__ __forceinline__ int64_t blocked_scale_off(int row, int kt, int n_ktiles) {
    return ((int64_t)(row >> 7) * n_ktiles + kt) * 512 + ((row & 31) << 4) + (((row >> 5) & 3) << 2);
}

// ------------------------------------------------------------------------------------------
// Per-thread description of the global -> LDS copy of one stage.
// Thread t moves chunk (t & 7) of rows (t >> 3) + 32*i : i < 4 token rows, i < 8 weight rows.
struct StageLoader {
    const char *tok_ptr[4];  // row start + chunk offset, per token row of this thread
    const char *w_ptr[2];    // first / second 128 weight rows: row (t>>3) start + chunk offset
    int64_t w_pitch32;       // bytes between weight rows 32 apart
    int lds_off;             // byte offset of this thread's chunk inside a 32-row group
    uint4 rt[4];
    uint4 rw[8];

    template <int NTF>
    __device__ __forceinline__ void load(int64_t koff) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i < NTF) rt[i] = *reinterpret_cast<const uint4 *>(tok_ptr[i] + koff);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            rw[i] = *reinterpret_cast<const uint4 *>(w_ptr[i >> 2] + (i & 3) * w_pitch32 + koff);
    }
    template <int NTF>
    __device__ __forceinline__ void load_tok(int64_t koff) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i < NTF) rt[i] = *reinterpret_cast<const uint4 *>(tok_ptr[i] + koff);
    }
    __device__ __forceinline__ void load_w(int64_t koff) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            rw[i] = *reinterpret_cast<const uint4 *>(w_ptr[i >> 2] + (i & 3) * w_pitch32 + koff);
    }
    template <int NTF>
    __device__ __forceinline__ void store_tok(char *stage) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i < NTF) *reinterpret_cast<uint4 *>(stage + lds_off + i * 32 * kRowBytes) = rt[i];
    }
    __device__ __forceinline__ void store_w(char *stage) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            *reinterpret_cast<uint4 *>(stage + kTokRegion + lds_off + i * 32 * kRowBytes) = rw[i];
    }
};

// ------------------------------------------------------------------------------------------
// MFMA over one 128-byte slab.  `tok` / `wgt` point at the token / weight regions of a stage.
// wrow[f] = first LDS weight row of this wave's fragment f.  TRANSPOSED: weight rows on the
// MFMA M side (accumulator registers run along weight rows, lanes along tokens); otherwise
// tokens on the M side (lanes run along weight rows).
template <int DT, int NTF, bool TRANSPOSED>
__device__ __forceinline__ void mfma_slab(f32x16 (&acc)[2][4], const char *tok, const char *wgt,
                                          const int (&wrow)[2], int lane, const uint32_t (&stok)[4],
                                          const uint32_t (&sw)[2]) {
    const int r = lane & 31;
    const int half = lane >> 5;
    const int sx = (lane >> 1) & 7;  // swz(row) for rows that are 32-aligned + r
    const int rowoff = r * kRowBytes;
    if constexpr (DT == DT_BF16) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int slot = ((2 * j + half) ^ sx) << 4;
            bf16x8 a[2], b[4];
#pragma unroll
            for (int f = 0; f < 2; ++f)
                a[f] = *reinterpret_cast<const bf16x8 *>(wgt + wrow[f] * kRowBytes + rowoff + slot);
#pragma unroll
            for (int t = 0; t < 4; ++t)
                if (t < NTF) b[t] = *reinterpret_cast<const bf16x8 *>(tok + t * 32 * kRowBytes + rowoff + slot);
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (t < NTF) {
                        if constexpr (TRANSPOSED)
                            acc[f][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[f], b[t], acc[f][t], 0, 0, 0);
                        else
                            acc[f][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[t], a[f], acc[f][t], 0, 0, 0);
                    }
        }
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            // Registers 0-3 of both lane halves form K block 2j (lanes < 32 its first 16 bytes, lanes >= 32
            // the last 16), registers 4-7 form K block 2j+1; the scale of block 2j is taken from lanes
            // < 32 and that of block 2j+1 from lanes >= 32 (measured on gfx950).
            const int slot = ((4 * j + half) ^ sx) << 4;
            const int sh = 8 * (2 * j + half);  // the scale byte this lane supplies
            i32x8 a[2], b[4];
            int sa[2], sb[4];
#pragma unroll
            for (int f = 0; f < 2; ++f) {
                const char *p = wgt + wrow[f] * kRowBytes + rowoff;
                i32x4 lo = *reinterpret_cast<const i32x4 *>(p + slot);
                i32x4 hi = *reinterpret_cast<const i32x4 *>(p + (slot ^ 32));
                a[f] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                sa[f] = (int)((sw[f] >> sh) & 0xffu);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
                if (t < NTF) {
                    const char *p = tok + t * 32 * kRowBytes + rowoff;
                    i32x4 lo = *reinterpret_cast<const i32x4 *>(p + slot);
                    i32x4 hi = *reinterpret_cast<const i32x4 *>(p + (slot ^ 32));
                    b[t] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                    sb[t] = (int)((stok[t] >> sh) & 0xffu);
                }
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (t < NTF) {
                        if constexpr (TRANSPOSED)
                            acc[f][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                                a[f], b[t], acc[f][t], 0, 0, 0, sa[f], 0, sb[t]);
                        else
                            acc[f][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                                b[t], a[f], acc[f][t], 0, 0, 0, sb[t], 0, sa[f]);
                    }
        }
    }
}

}  // namespace pmoe
