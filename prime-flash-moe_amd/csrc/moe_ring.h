// Stage-ring engine of the mxfp8 grouped-GEMM kernels (512 threads), gfx950, and the copy primitives that the
// bf16 engine (moe_tall.h) shares with it.
//
// Tile: token rows x 256 weight rows.  The contraction is consumed in slabs of RB = 64 or 128 bytes
// per row.  Slabs are copied global -> LDS by the direct-to-LDS path (global_load_lds_*: no staging
// registers, no ds_write) into a ring of stages; all but one stage are in flight while one is
// consumed.  One barrier per slab.  RB = 128 asks L2 for whole cache lines (half the requests, half
// the barriers; a plain stream from HBM runs 8 % faster); RB = 64 has twice the stages in the same LDS.
//
// The ring is sized per tile.  A stage holds only the 32-row token fragments that have live rows
// (group 0's first, then group 1's), the 256 weight rows and, for mxfp8, the scale dwords of both;
// as many stages as fit the LDS budget are used, at most 8.  The fewer token rows a tile has, the
// closer it is to a pure stream of weights from HBM, and what keeps HBM busy then is weight bytes in
// flight per CU.
//
// Stage layout: [live token rows][RB] [256 weight rows][RB] [scale dwords: token rows rounded up to a
// multiple of 64, then weight rows (mxfp8)].
// A row is RB/16 chunks of 16 B; chunk c of row r sits in slot c ^ swizzle(r) (64 B: (r >> 2) & 3,
// 128 B: (r >> 1) & 7): the 16-byte MFMA operand reads of 16 consecutive rows then cover all 64 LDS
// banks exactly once.  The copy engine writes lane l of a wave instruction to bytes [16 l, 16 l + 16)
// behind a wave-uniform base (one instruction = 1 KB = 1024 / RB rows), so the swizzle is applied on
// the global side (the lane landing in slot s of row r fetches chunk s ^ swizzle(r)).
//
// mxfp8 scales ride along: the 4-scale dword (128 K) of every row of the tile is copied with each
// slab into the stage's scale region, 4 bytes per lane.
//
// All copies are issued as inline assembly: the compiler cannot tell the stage being read from
// the stages being filled and would otherwise make every LDS read wait for all copies in
// flight.  The hardware load counter (vmcnt) still counts them, per wave and in issue order; a
// wave that issues `lps` copy instructions per stage has slab k when at most lps * (stages still
// behind it) of its copies are pending.
#pragma once
#include "moe_tile.h"

namespace pmoe {
namespace ring {

constexpr int kMaxStages = 8;

template <int RB>
__device__ __forceinline__ int swz(int row) {
    return RB == 64 ? (row >> 2) & 3 : (row >> 1) & 7;
}

// Geometry of a tile's ring; every member is wave-uniform.
struct Layout {
    int tok_rows;        // live token rows of both groups: 32 (ntf0 + ntf1)
    int group1_off;      // byte offset of group 1's token rows inside a stage
    int w_off;           // byte offset of the weight rows
    int scale_off;       // byte offset of the scale dwords (mxfp8)
    int scale_tok_rows;  // token scale dwords reserved: tok_rows rounded up to 64
    int stage_bytes;
    int stages;
};
template <int DT, int RB>
__device__ __forceinline__ Layout make_layout(int ntf0, int ntf1, int budget) {
    Layout l;
    l.tok_rows = 32 * (ntf0 + ntf1);
    l.group1_off = 32 * ntf0 * RB;
    l.w_off = l.tok_rows * RB;
    l.scale_off = l.w_off + kWRows * RB;
    l.scale_tok_rows = (l.tok_rows + 63) & ~63;
    const int bytes = l.scale_off + (DT == DT_FP8 ? (l.scale_tok_rows + kWRows) * 4 : 0);
    l.stage_bytes = (bytes + 255) & ~255;
    l.stages = min(kMaxStages, budget / l.stage_bytes);
    return l;
}
// LDS the ring may use, a multiple of 1 KB (the split kernels put their row table behind it).
template <int DT>
constexpr int ring_bytes() {
    static_assert(DT == DT_FP8, "the stage ring serves the mxfp8 kernels");
    return 156 * 1024;
}

__device__ __forceinline__ uint32_t lds_addr(const char *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}
// M0 holds the LDS address of a direct-to-LDS copy.  The statements below write it without declaring it: the
// compiler reserves the register and rejects it in a clobber list.  That is sound only while the compiler itself
// keeps no value in M0 across a statement, so the kernels that use these primitives stay clear of everything that
// makes it use M0 on gfx950: the LDS-DMA builtins (__builtin_amdgcn_global_load_lds, raw_buffer_load_lds), GWS
// and s_sendmsg builtins, register-indexed moves (accumulators and fragment arrays are indexed by constants after
// unrolling only), readlane / writelane with a lane number that is not a compile-time constant.  A host test
// compiles the two translation units that include this file to assembly and fails if a kernel that contains a
// copy touches M0 anywhere outside these statements (tests/test_host.py); a GPU test runs the tile paths with the
// most copies between two barriers on poisoned LDS (tests/test_gpu_lds_copies.py).
__device__ __forceinline__ void copy16(const char *base, uint32_t voff, const char *lds_dst) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base), "s"(lds_addr(lds_dst)) : "memory");
}
// The same copy with the non-temporal hint, for weight rows that no other workgroup reads (an expert with a
// single row tile): the lines leave the caches first.  The decode shape streams its weights 12 % faster
// with it; weight rows that several row tiles share lose up to 20 % with it.
__device__ __forceinline__ void copy16_once(const char *base, uint32_t voff, const char *lds_dst) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt" : : "v"(voff), "s"(base), "s"(lds_addr(lds_dst)) : "memory");
}
__device__ __forceinline__ void copy4(const char *base, uint32_t voff, const char *lds_dst) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" : : "v"(voff), "s"(base), "s"(lds_addr(lds_dst)) : "memory");
}
// A wave-uniform pointer, read through lane 0 so that the compiler keeps it in scalar registers.
__device__ __forceinline__ const char *uniform_ptr(const char *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const char *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
template <int N>
__device__ __forceinline__ void wait_and_barrier() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(N) : "memory");
}
// Waits until at most `n` (wave-uniform, <= 30) of this wave's copies are in flight and its LDS
// reads have returned, then joins the workgroup barrier.  The wait count is an immediate of the
// instruction, hence the switch (RB = 64: at most 5 copies per stage x 6 stages behind the current
// one; RB = 128: 9 x 2).
__device__ __forceinline__ void wait_and_barrier_dyn(int n) {
    switch (n) {
#define PMOE_WB(k) case k: wait_and_barrier<k>(); break;
        PMOE_WB(1) PMOE_WB(2) PMOE_WB(3) PMOE_WB(4) PMOE_WB(5) PMOE_WB(6) PMOE_WB(7) PMOE_WB(8) PMOE_WB(9)
        PMOE_WB(10) PMOE_WB(11) PMOE_WB(12) PMOE_WB(13) PMOE_WB(14) PMOE_WB(15) PMOE_WB(16) PMOE_WB(17)
        PMOE_WB(18) PMOE_WB(19) PMOE_WB(20) PMOE_WB(21) PMOE_WB(22) PMOE_WB(23) PMOE_WB(24) PMOE_WB(25)
        PMOE_WB(26) PMOE_WB(27) PMOE_WB(28) PMOE_WB(29) PMOE_WB(30)
#undef PMOE_WB
        default: wait_and_barrier<0>(); break;
    }
}

// Per-thread description of the copies of one stage.  A 128-row block of token rows or half of the
// weight tile takes N = RB / 64 instructions of every wave: instruction q of wave w moves rows
// q * 8 * rpc + rpc * w .. + rpc - 1 of it (rpc = 1024 / RB rows per instruction).  Token rows of
// fragments without live rows are not copied, nor are the rows without a token inside a live fragment
// (an instruction whose rows all lack one is dropped: the wait counts rely on every issued
// instruction having an active lane).  Scales: at most one 4-byte-per-lane instruction per
// wave.
template <int RB>
struct Loader {
    static constexpr int N = RB / 64;
    static constexpr int kRowsPerCopy = 1024 / RB;
    const char *tok_base;
    const char *w_base[2];
    uint32_t tok_off[2][N];
    uint32_t w_off[N];
    const char *sc_base;  // wave-uniform: activation scales or weight scales
    uint32_t sc_off;      // this lane's row in them
    uint32_t sc_step;     // bytes between consecutive 128-wide K tiles: 4 (row major) or 512 (blocked)
    int tok_dst[2][N];    // LDS offset inside a stage of this wave's token rows; -1: nothing to copy
    bool tok_live[2][N];  // this lane's row holds a token (rows without one are not fetched: what the
                          // stage holds for them only reaches their own, unused, output rows)
    int w_dst[2][N];      // LDS offsets of this wave's weight rows
    int sc_dst;           // LDS offset of this wave's scale dwords; -1: none
    int lps;              // copy instructions this wave issues per stage
    bool w_once;          // wave-uniform: the weight rows are read by this workgroup only (see copy16_once)

    // Row inside a 128-row block that lane `lane` of wave `wave` moves with instruction q.
    static __device__ __forceinline__ int row_of(int wave, int lane, int q) {
        return q * 8 * kRowsPerCopy + kRowsPerCopy * wave + lane / (RB / 16);
    }
    // The base pointers feed scalar operands of the copy instructions: pin them to scalar registers.
    __device__ __forceinline__ void make_uniform() {
        tok_base = uniform_ptr(tok_base);
        w_base[0] = uniform_ptr(w_base[0]);
        w_base[1] = uniform_ptr(w_base[1]);
        sc_base = uniform_ptr(sc_base);
    }
    __device__ __forceinline__ void issue(char *stage, int slab) const {
        const uint32_t koff = (uint32_t)slab * RB;
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int q = 0; q < N; ++q)
                if (tok_dst[b][q] >= 0) {
                    if (tok_live[b][q]) copy16(tok_base, tok_off[b][q] + koff, stage + tok_dst[b][q]);
                }
        if (w_once) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int q = 0; q < N; ++q) copy16_once(w_base[h], w_off[q] + koff, stage + w_dst[h][q]);
        } else {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int q = 0; q < N; ++q) copy16(w_base[h], w_off[q] + koff, stage + w_dst[h][q]);
        }
        if (sc_dst >= 0) copy4(sc_base, sc_off + (uint32_t)(RB == 64 ? slab >> 1 : slab) * sc_step, stage + sc_dst);
    }
};

// 64 e4m3 of K = one v_mfma_scale_f32_32x32x64_f8f6f4 per (weight fragment, token fragment); `j` is
// the 64-byte step inside the slab (0 for RB = 64).  Registers 0-3 of both lane halves form K block 0
// of the step (lanes < 32 its first 16 bytes, lanes >= 32 the last 16), registers 4-7 form K block 1;
// the scale of block 0 is taken from lanes < 32 and that of block 1 from lanes >= 32 (measured on
// gfx950).  `sel` = 8 * (2 * (64-byte step inside its 128-wide K tile) + lane / 32) picks this lane's
// scale byte out of the row's 4-scale dword.
template <int RB, int NTF, bool TRANSPOSED>
__device__ __forceinline__ void mma_fp8_step(f32x16 (&acc)[2][4], const char *tok, const char *wgt,
                                             const uint32_t *tok_sc, const uint32_t *w_sc,
                                             const int (&wrow)[2], int lane, int j, int sel) {
    const int r = lane & 31, half = lane >> 5, sx = swz<RB>(r);
    const int off = r * RB + (((4 * j + half) ^ sx) << 4);
    i32x8 a[2];
    int sa[2];
#pragma unroll
    for (int f = 0; f < 2; ++f) {
        const char *p = wgt + wrow[f] * RB;
        const i32x4 lo = *reinterpret_cast<const i32x4 *>(p + off);
        const i32x4 hi = *reinterpret_cast<const i32x4 *>(p + (off ^ 32));
        a[f] = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        sa[f] = (int)((w_sc[wrow[f] + r] >> sel) & 0xffu);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
        if (t < NTF) {
            const char *p = tok + t * 32 * RB;
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

// Issues slabs 0 .. n - 1 of a tile (at most stages - 1 of them, in rotated order from `start`) into
// stages stage0, stage0 + 1, ...
template <int DT, int RB>
__device__ __forceinline__ void pre_issue(const Loader<RB> &ld, const Layout &lay, char *lds, int n_slabs, int start,
                                          int stage0, int n) {
    const int SB = lay.stage_bytes, NS = lay.stages;
    for (int s = 0; s < n; ++s) {
        if (s >= n_slabs) break;
        int slab = s + start;
        if (slab >= n_slabs) slab -= n_slabs;
        int st = stage0 + s;
        if (st >= NS) st -= NS;
        ld.issue(lds + st * SB, slab);
    }
}
// K loop.  COMPUTE = false is the loop of the waves without matrix work (a group without live
// rows): they only issue their share of the copies and join the barriers.  `tok_region` = byte
// offset of this wave's group inside a stage's token rows.
//
// The slabs are visited in rotated order, starting at slab `start` (even for RB = 64): workgroups
// that run side by side and share rows then ask for different cache lines at any one time instead
// of queueing on the same ones.  The sum over K does not depend on the order.
//
// Geometry and wait counts are wave-uniform run-time values (the wait count goes through a switch).  A
// variant for tiles of two full blocks with compile-time geometry, 64-byte slabs and 4 stages measured 2 - 3 %
// slower on large mxfp8 batches than this loop with 128-byte slabs and 2 stages, and is gone.
//
// Slab 0 goes to stage `stage0`, the following ones to the stages behind it (wrapping).  `n_pre`: the
// caller has already issued slabs 0 .. n_pre - 1 (see pre_issue; a workgroup that runs one tile
// after another issues them under the previous tile's epilogue).
template <int DT, int RB, int NTF, bool TRANSPOSED, bool COMPUTE>
__device__ __forceinline__ void main_loop(f32x16 (&acc)[2][4], const Loader<RB> &ld, const Layout &lay, char *lds,
                                          int n_slabs, const int (&wrow)[2], int lane, int tok_region, int start,
                                          int stage0 = 0, int n_pre = 0) {
    const int SB = lay.stage_bytes, NS = lay.stages;
    const int w_off = lay.w_off, scale_off = lay.scale_off, scale_tok_rows = lay.scale_tok_rows;
    auto rot = [&](int s) {
        s += start;
        return s >= n_slabs ? s - n_slabs : s;
    };
    for (int s = n_pre; s < NS - 1; ++s) {
        int st = stage0 + s;
        if (st >= NS) st -= NS;
        if (s < n_slabs) ld.issue(lds + st * SB, rot(s));
    }
    const int lps = ld.lps;
    int cur_off = stage0 * SB;  // stage of slab kt
    // stage slab kt + NS - 1 goes to (the one slab kt - 1 used)
    int fill_off = (stage0 == 0 ? NS - 1 : stage0 - 1) * SB;
    for (int kt = 0; kt < n_slabs; ++kt) {
        // slab kt has landed once at most the copies of the later slabs (up to NS - 2) are pending
        wait_and_barrier_dyn(lps * min(NS - 2, n_slabs - 1 - kt));
        // the stage consumed in the previous iteration is free: everybody is past the barrier
        if (kt + NS - 1 < n_slabs) ld.issue(lds + fill_off, rot(kt + NS - 1));
        if constexpr (COMPUTE) {
            const char *cur = lds + cur_off;
            const char *tok = cur + tok_region;
            const char *wgt = cur + w_off;
            {
                const uint32_t *sc = reinterpret_cast<const uint32_t *>(cur + scale_off);
                const uint32_t *tok_sc = sc + tok_region / RB, *w_sc = sc + scale_tok_rows;
                if constexpr (RB == 64) {
                    // start is even: the parity of kt is the parity of the slab inside its 128-wide K tile
                    mma_fp8_step<RB, NTF, TRANSPOSED>(acc, tok, wgt, tok_sc, w_sc, wrow, lane, 0,
                                                      8 * (2 * (kt & 1) + (lane >> 5)));
                } else {
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        mma_fp8_step<RB, NTF, TRANSPOSED>(acc, tok, wgt, tok_sc, w_sc, wrow, lane, j,
                                                          8 * (2 * j + (lane >> 5)));
                }
            }
        }
        fill_off = cur_off;
        cur_off += SB;
        if (cur_off >= NS * SB) cur_off = 0;
    }
    __syncthreads();  // all reads of the last stages are done: the ring may be reused as scratch
}

}  // namespace ring
}  // namespace pmoe
