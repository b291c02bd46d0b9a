// Device-side helpers shared by the fused-MoE kernels (gfx950, wave64), and the register-staged
// tile engine of the single-group (256-thread) fused kernel; the two-group kernels of the split
// pipeline use the ring engine in moe_ring.h.
//
// A workgroup of 256 threads owns a tile of a grouped GEMM whose two operands are both contiguous
// along the contraction dimension:
//     128 token rows (one sorted block of x, or the activation tile)
//   x 256 weight rows (W1 or W2 of one expert).
// The contraction is consumed in slabs of 128 bytes per row (64 bf16 or 128 e4m3), staged
// through LDS with a double buffer: while the MFMAs of slab k run out of one buffer, the
// global loads of slab k+1 are in flight into registers and are then written to the other.
//
// LDS layout of one stage: [NG*128 token rows][128 B] then [256 weight rows][128 B].
// A row is 8 chunks of 16 B; chunk c of row r is stored in slot c ^ ((r >> 1) & 7), which
// makes the 16-byte MFMA operand reads of 16 consecutive rows hit all 64 banks once
// (measured: 242 of 256 B/clk/CU, against 43 B/clk unswizzled).
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

constexpr int kBlockRows = 128;  // sorted rows per block (= block_m)
constexpr int kWRows = 256;      // weight rows per tile
constexpr int kRowBytes = 128;   // contraction bytes per LDS row
constexpr int kGroupRegion = kBlockRows * kRowBytes;  // 16 KB: one group's token rows of a stage
constexpr int kNumStages = 2;

template <int NG>
struct Geo {
    static constexpr int kThreads = 256 * NG;
    static constexpr int kTokRows = kBlockRows * NG;
    static constexpr int kPassRows = 32 * NG;            // rows the workgroup moves per pass (8 threads a row)
    static constexpr int kTokPasses = kTokRows / kPassRows;  // 4
    static constexpr int kWPasses = kWRows / kPassRows;      // 8 or 4
    static constexpr int kWPassesPerHalf = 128 / kPassRows;  // passes per 128 weight rows
    static constexpr int kTokRegion = kTokRows * kRowBytes;
    static constexpr int kStageBytes = kTokRegion + kWRows * kRowBytes;  // 48 KB or 64 KB
};

enum : int { DT_BF16 = 0, DT_FP8 = 1 };

__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// round-to-nearest-even fp32 -> bf16 bits (NaN kept quiet)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// Two fp32 -> one dword of two bf16 (round to nearest even), the hardware conversion of gfx950.
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 v = __builtin_convertvector(f32x2{lo, hi}, bf16x2);
    return __builtin_bit_cast(uint32_t, v);
}

// silu(gate) * up with the hardware exponential and reciprocal (about 1 ulp each, far inside bf16).
__device__ __forceinline__ float swiglu(float gate, float up) {
    return up * gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate));
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
// Thread t moves chunk (t & 7) of rows (t >> 3) + kPassRows*i, for the token passes whose bit is
// set in tok_mask and for all weight passes.
template <int NG>
struct StageLoader {
    using G = Geo<NG>;
    // Addresses are a workgroup-uniform base (held in scalar registers) plus a 32-bit per-thread
    // byte offset: the token matrix and one expert's weight matrix are each below 4 GiB.
    const char *tok_base;
    const char *w_base[2];          // first / second 128 weight rows of the tile
    uint32_t tok_off[G::kTokPasses];  // row start + chunk offset of this thread's token rows
    uint32_t w_off;                  // row (t >> 3) start + chunk offset inside a 128-row half
    uint32_t w_pitch_pass;           // bytes between weight rows kPassRows apart
    int lds_off;                     // byte offset of this thread's chunk inside a pass
    int tok_mask;                    // token passes that hold live rows
    uint4 rt[G::kTokPasses];
    uint4 rw[G::kWPasses];

    __device__ __forceinline__ void load_tok(uint32_t koff) {
#pragma unroll
        for (int i = 0; i < G::kTokPasses; ++i)
            if (tok_mask & (1 << i)) rt[i] = *reinterpret_cast<const uint4 *>(tok_base + (tok_off[i] + koff));
    }
    __device__ __forceinline__ void load_w(uint32_t koff) {
#pragma unroll
        for (int i = 0; i < G::kWPasses; ++i)
            rw[i] = *reinterpret_cast<const uint4 *>(w_base[i / G::kWPassesPerHalf] +
                                                     (w_off + (i % G::kWPassesPerHalf) * w_pitch_pass + koff));
    }
    __device__ __forceinline__ void store_tok(char *stage) {
#pragma unroll
        for (int i = 0; i < G::kTokPasses; ++i)
            if (tok_mask & (1 << i))
                *reinterpret_cast<uint4 *>(stage + lds_off + i * G::kPassRows * kRowBytes) = rt[i];
    }
    __device__ __forceinline__ void store_w(char *stage) {
#pragma unroll
        for (int i = 0; i < G::kWPasses; ++i)
            *reinterpret_cast<uint4 *>(stage + G::kTokRegion + lds_off + i * G::kPassRows * kRowBytes) = rw[i];
    }
};

// ------------------------------------------------------------------------------------------
// MFMA over one 128-byte slab.  `tok` points at this wave's group of 128 token rows, `wgt` at the
// 256 weight rows of a stage.  wrow[f] = first LDS weight row of this wave's fragment f.
// TRANSPOSED: weight rows on the MFMA M side (accumulator registers run along weight rows, lanes
// along tokens); otherwise tokens on the M side (lanes run along weight rows).
template <int DT, int NTF, bool TRANSPOSED, bool PREFETCH>
__device__ __forceinline__ void mfma_slab(f32x16 (&acc)[2][4], const char *tok, const char *wgt,
                                          const int (&wrow)[2], int lane, const uint32_t (&stok)[4],
                                          const uint32_t (&sw)[2]) {
    const int r = lane & 31;
    const int half = lane >> 5;
    const int sx = (lane >> 1) & 7;  // swz(row) for rows that are 32-aligned + r
    const int rowoff = r * kRowBytes;
    if constexpr (DT == DT_BF16) {
        // PREFETCH: operand fragments are double-buffered in registers, the reads of sub-step j+1 are
        // issued before the MFMAs of sub-step j (one wave per SIMD has nobody else to cover its LDS
        // latency); without it one buffer is reused, which saves 24 registers.
        bf16x8 a[2][2], b[2][4];
        auto fetch = [&](int j, int buf) {
            const int slot = ((2 * j + half) ^ sx) << 4;
#pragma unroll
            for (int f = 0; f < 2; ++f)
                a[buf][f] = *reinterpret_cast<const bf16x8 *>(wgt + wrow[f] * kRowBytes + rowoff + slot);
#pragma unroll
            for (int t = 0; t < 4; ++t)
                if (t < NTF) b[buf][t] = *reinterpret_cast<const bf16x8 *>(tok + t * 32 * kRowBytes + rowoff + slot);
        };
        if constexpr (PREFETCH) fetch(0, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int cur = PREFETCH ? (j & 1) : 0;
            if constexpr (PREFETCH) {
                if (j + 1 < 4) fetch(j + 1, cur ^ 1);
            } else {
                fetch(j, 0);
            }
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (t < NTF) {
                        if constexpr (TRANSPOSED)
                            acc[f][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[cur][f], b[cur][t], acc[f][t], 0, 0, 0);
                        else
                            acc[f][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[cur][t], a[cur][f], acc[f][t], 0, 0, 0);
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
            // weight fragments of the sub-step stay in registers, token fragments stream through one
            // register set (8 VGPRs) to keep the kernel within 256 registers at two waves per SIMD
            i32x8 a[2];
            int sa[2];
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
                    const i32x8 b = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                    const int sb = (int)((stok[t] >> sh) & 0xffu);
#pragma unroll
                    for (int f = 0; f < 2; ++f) {
                        if constexpr (TRANSPOSED)
                            acc[f][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                                a[f], b, acc[f][t], 0, 0, 0, sa[f], 0, sb);
                        else
                            acc[f][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                                b, a[f], acc[f][t], 0, 0, 0, sb, 0, sa[f]);
                    }
                    if constexpr (!PREFETCH) __builtin_amdgcn_sched_barrier(0);  // keep the next fragment's reads behind these MFMAs
                }
        }
    }
}

}  // namespace pmoe
