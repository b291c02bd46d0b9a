// Ring engine of the two-group (512-thread) grouped-GEMM kernels, gfx950.
//
// Tile: 256 token rows (two sorted blocks, one per group of 4 waves) x 256 weight rows.
// The contraction is consumed in slabs of 64 bytes per row (32 bf16 / 64 e4m3).  Slabs are copied
// global -> LDS by the direct-to-LDS path (global_load_lds_*: no staging registers, no ds_write)
// into a ring of 4 stages; three slabs are in flight while one is consumed, which is what hides
// the ~1.5 us that a burst of copies needs to drain through the vector L1 and come back from
// L2/HBM.  One barrier per slab.
//
// Stage layout (32 KB, + 2 KB for mxfp8):
//   [256 token rows][64 B] [256 weight rows][64 B] [512 scale dwords]
// A row is 4 chunks of 16 B; chunk c of row r sits in slot c ^ ((r >> 2) & 3): the 16-byte MFMA
// operand reads of 16 consecutive rows then cover all 64 LDS banks exactly once.  The copy engine
// writes lane l of a wave instruction to bytes [16 l, 16 l + 16) behind a wave-uniform base, so the
// swizzle is applied on the global side (the lane landing in slot s of row r fetches chunk
// s ^ swz(r)).
//
// mxfp8 scales ride along: per stage, lane l of wave v copies the 4-scale dword of row 64 v + l
// (waves 0-3: token rows, from the row-major activation scales; waves 4-7: weight rows, from the
// blocked weight scales) that covers the 128-wide K tile the slab lies in.
//
// All copies are issued as inline assembly: the compiler cannot tell the stage being read from
// the stages being filled and would otherwise make every LDS read wait for all copies in
// flight.  The hardware load counter (vmcnt) still counts them, in issue order; wait_pending(n)
// lets the n most recent wave instructions stay in flight.
#pragma once
#include "moe_tile.h"

namespace pmoe {
namespace ring {

constexpr int kRB = 64;        // row bytes of a slab
constexpr int kStages = 4;
constexpr int kTokRows = 256;  // two groups of 128
constexpr int kTokRegion = kTokRows * kRB;           // 16 KB
constexpr int kGroupRegion = kBlockRows * kRB;       // 8 KB
constexpr int kWRegion = kWRows * kRB;               // 16 KB
constexpr int kScaleOff = kTokRegion + kWRegion;     // scale dwords of the 512 rows (mxfp8)
template <int DT>
constexpr int stage_bytes() { return kScaleOff + (DT == DT_FP8 ? 512 * 4 : 0); }
template <int DT>
constexpr int loads_per_stage() { return DT == DT_FP8 ? 5 : 4; }  // wave instructions per stage

__device__ __forceinline__ int swz64(int row) { return (row >> 2) & 3; }

__device__ __forceinline__ uint32_t lds_addr(const char *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}
__device__ __forceinline__ void copy16(const char *base, uint32_t voff, const char *lds_dst) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base), "s"(lds_addr(lds_dst)) : "memory");
}
__device__ __forceinline__ void copy4(const char *base, uint32_t voff, const char *lds_dst) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" : : "v"(voff), "s"(base), "s"(lds_addr(lds_dst)) : "memory");
}
// Waits until at most N of this wave's copies are in flight and its LDS reads have returned, then
// joins the workgroup barrier.
template <int N>
__device__ __forceinline__ void wait_and_barrier() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(N) : "memory");
}

// Per-thread description of the copies of one stage.  Thread t moves slot (t & 3) of row
// (t >> 2) of each 128-row pass: pass 0 / 1 of the token rows are the two groups, pass 0 / 1 of the
// weight rows are the two 128-row halves of the tile.
struct Loader {
    const char *tok_base;
    const char *w_base[2];
    uint32_t tok_off[2];
    uint32_t w_off;
    const char *sc_base;  // wave-uniform: activation scales (waves 0-3) or weight scales (4-7)
    uint32_t sc_off;      // this lane's row in them
    uint32_t sc_step;     // bytes between consecutive 128-wide K tiles: 4 (row major) or 512 (blocked)
    int wave_off;         // this wave's 16 rows inside a pass
    int wave_sc_off;      // this wave's 64 scale dwords inside a stage

    template <int DT>
    __device__ __forceinline__ void issue(char *stage, int slab) const {
        const uint32_t koff = (uint32_t)slab * kRB;
        copy16(tok_base, tok_off[0] + koff, stage + wave_off);
        copy16(tok_base, tok_off[1] + koff, stage + kGroupRegion + wave_off);
        copy16(w_base[0], w_off + koff, stage + kTokRegion + wave_off);
        copy16(w_base[1], w_off + koff, stage + kTokRegion + kWRegion / 2 + wave_off);
        if constexpr (DT == DT_FP8) copy4(sc_base, sc_off + (uint32_t)(slab >> 1) * sc_step, stage + kScaleOff + wave_sc_off);
    }
};

struct FragsBf16 {
    bf16x8 a[2];  // weight fragments
    bf16x8 b[4];  // token fragments
};

template <int NTF>
__device__ __forceinline__ void fetch_bf16(FragsBf16 &fr, const char *tok, const char *wgt, const int (&wrow)[2],
                                           int lane, int j) {
    const int r = lane & 31, half = lane >> 5, sx = (lane >> 2) & 3;
    const int off = r * kRB + (((2 * j + half) ^ sx) << 4);
#pragma unroll
    for (int f = 0; f < 2; ++f) fr.a[f] = *reinterpret_cast<const bf16x8 *>(wgt + wrow[f] * kRB + off);
#pragma unroll
    for (int t = 0; t < 4; ++t)
        if (t < NTF) fr.b[t] = *reinterpret_cast<const bf16x8 *>(tok + t * 32 * kRB + off);
}

template <int NTF, bool TRANSPOSED>
__device__ __forceinline__ void mma_bf16(f32x16 (&acc)[2][4], const FragsBf16 &fr) {
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if (t < NTF) {
                if constexpr (TRANSPOSED)
                    acc[f][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr.a[f], fr.b[t], acc[f][t], 0, 0, 0);
                else
                    acc[f][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr.b[t], fr.a[f], acc[f][t], 0, 0, 0);
            }
}

// One e4m3 slab = one v_mfma_scale_f32_32x32x64_f8f6f4 per (weight fragment, token fragment).
// Registers 0-3 of both lane halves form K block 0 of the slab (lanes < 32 its first 16 bytes,
// lanes >= 32 the last 16), registers 4-7 form K block 1; the scale of block 0 is taken from lanes
// < 32 and that of block 1 from lanes >= 32 (measured on gfx950).  `sel` = 8 * (2 * (slab & 1) +
// lane / 32) picks this lane's scale byte out of the row's 4-scale dword.
template <int NTF, bool TRANSPOSED>
__device__ __forceinline__ void mma_fp8_slab(f32x16 (&acc)[2][4], const char *tok, const char *wgt,
                                             const uint32_t *tok_sc, const uint32_t *w_sc,
                                             const int (&wrow)[2], int lane, int sel) {
    const int r = lane & 31, half = lane >> 5, sx = (lane >> 2) & 3;
    const int off = r * kRB + ((half ^ sx) << 4);
    i32x8 a[2];
    int sa[2];
#pragma unroll
    for (int f = 0; f < 2; ++f) {
        const char *p = wgt + wrow[f] * kRB;
        const i32x4 lo = *reinterpret_cast<const i32x4 *>(p + off);
        const i32x4 hi = *reinterpret_cast<const i32x4 *>(p + (off ^ 32));
        a[f] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        sa[f] = (int)((w_sc[wrow[f] + r] >> sel) & 0xffu);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
        if (t < NTF) {
            const char *p = tok + t * 32 * kRB;
            const i32x4 lo = *reinterpret_cast<const i32x4 *>(p + off);
            const i32x4 hi = *reinterpret_cast<const i32x4 *>(p + (off ^ 32));
            const i32x8 b = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            const int sb = (int)((tok_sc[32 * t + r] >> sel) & 0xffu);
#pragma unroll
            for (int f = 0; f < 2; ++f) {
                if constexpr (TRANSPOSED)
                    acc[f][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[f], b, acc[f][t], 0, 0, 0, sa[f], 0, sb);
                else
                    acc[f][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a[f], acc[f][t], 0, 0, 0, sb, 0, sa[f]);
            }
        }
}

// K loop.  COMPUTE = false is the loop of the waves of a group without live rows: they only
// issue their share of the copies and join the barriers.
//
// The slabs are visited in rotated order, starting at slab `start` (even): with row pitches that
// are multiples of 4 KB every row of a slab maps to the same memory channel, and workgroups that
// all walk K from 0 would queue on one channel at a time; giving concurrent workgroups different
// starting points spreads them over the channels.  The sum over K does not depend on the order.
template <int DT, int NTF, bool TRANSPOSED, bool COMPUTE>
__device__ __forceinline__ void main_loop(f32x16 (&acc)[2][4], const Loader &ld, char *lds, int n_slabs,
                                          const int (&wrow)[2], int lane, int grp, int start) {
    constexpr int SB = stage_bytes<DT>();
    constexpr int LPS = loads_per_stage<DT>();
    auto rot = [&](int s) {
        s += start;
        return s >= n_slabs ? s - n_slabs : s;
    };
#pragma unroll
    for (int s = 0; s < kStages - 1; ++s)
        if (s < n_slabs) ld.template issue<DT>(lds + s * SB, rot(s));
    FragsBf16 fx, fy;  // fy carries the held-back sub-step across the barrier
    if constexpr (DT == DT_BF16 && COMPUTE) {
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int i = 0; i < 8; ++i) fy.a[f][i] = (__bf16)0.0f;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 8; ++i) fy.b[t][i] = (__bf16)0.0f;
    }
    for (int kt = 0; kt < n_slabs; ++kt) {
        // slab kt has landed once at most the copies of the (up to two) later slabs are in flight
        if (kt + 2 < n_slabs) wait_and_barrier<2 * LPS>();
        else if (kt + 1 < n_slabs) wait_and_barrier<LPS>();
        else wait_and_barrier<0>();
        // the stage consumed in the previous iteration is free: everybody is past the barrier
        if (kt + kStages - 1 < n_slabs) ld.template issue<DT>(lds + ((kt + kStages - 1) & (kStages - 1)) * SB, rot(kt + kStages - 1));
        if constexpr (COMPUTE) {
            const char *cur = lds + (kt & (kStages - 1)) * SB;
            const char *tok = cur + grp * kGroupRegion;
            const char *wgt = cur + kTokRegion;
            if constexpr (DT == DT_BF16) {
                // software pipeline across the barrier: the second K sub-step of a slab is held back
                // and issued behind the first fragment reads of the next slab
                fetch_bf16<NTF>(fx, tok, wgt, wrow, lane, 0);
                mma_bf16<NTF, TRANSPOSED>(acc, fy);
                fetch_bf16<NTF>(fy, tok, wgt, wrow, lane, 1);
                mma_bf16<NTF, TRANSPOSED>(acc, fx);
                if constexpr (NTF == 4) {
                    // issue order: the 8 MFMAs of one fragment buffer alternate with the 6 LDS reads
                    // that refill the other
#pragma unroll
                    for (int p = 0; p < 2; ++p) {
#pragma unroll
                        for (int i = 0; i < 6; ++i) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                    }
                }
            } else {
                const uint32_t *sc = reinterpret_cast<const uint32_t *>(cur + kScaleOff);
                mma_fp8_slab<NTF, TRANSPOSED>(acc, tok, wgt, sc + grp * kBlockRows, sc + kTokRows, wrow, lane,
                                              8 * (2 * (kt & 1) + (lane >> 5)));  // start is even: parity of kt = parity of the slab
            }
        }
    }
    if constexpr (DT == DT_BF16 && COMPUTE) mma_bf16<NTF, TRANSPOSED>(acc, fy);
    __syncthreads();  // all reads of the last stages are done: the ring may be reused as scratch
}

}  // namespace ring
}  // namespace pmoe
