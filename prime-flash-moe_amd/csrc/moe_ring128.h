// Wide bf16 ring engine of the 512-thread grouped-GEMM kernels, gfx950: 128-byte row segments.
//
// Tile: 256 token rows (two sorted blocks, one per group of 4 waves) x 256 weight rows.  The
// contraction is consumed in slabs of 128 bytes per row (64 bf16): every global request is a whole
// 128-byte cache line, half as many requests to L2 as with 64-byte segments for the same bytes, and
// half as many workgroup barriers per tile.
//
// The whole LDS of a CU (160 KB) is a ring of five 32 KB units.  A unit holds 256 rows x 128 B of
// one operand of one slab; units are filled in the order W0 T0 W1 T1 W2 ... (W = weight rows, T =
// token rows), unit u into buffer u mod 5.  While slab k is consumed (units 2k, 2k+1), units 2k+2,
// 2k+3 and 2k+4 (96 KB) are in flight; the two buffers slab k-1 used are refilled right after the
// barrier that opens slab k.  Weight units are issued two slabs ahead of their use, token units one:
// weight rows are shared by fewer workgroups than token rows and miss L2 more often.
//
// A row is 8 chunks of 16 B; chunk c of row r sits in slot c ^ ((r >> 1) & 7), so the 16-byte MFMA
// operand reads of 16 consecutive rows cover all 64 banks once.  The copy engine writes lane l of a
// wave instruction to bytes [16 l, 16 l + 16) behind a wave-uniform base: one instruction moves 8
// rows, lane l fetching chunk (l & 7) ^ swizzle(row) of row l / 8.
//
// Wave w copies rows 32 w .. 32 w + 31 of every unit (4 instructions).  For a token unit these are
// one 32-row fragment of block w / 4; fragments without live rows are not copied.  A wave has slab
// k when at most the 4 copies of weight unit k + 1 are pending, whatever it copies of token rows.
#pragma once
#include "moe_ring.h"

namespace pmoe {
namespace ring128 {

constexpr int kRB = 128;                      // row bytes of a slab
constexpr int kUnitBytes = 256 * kRB;         // 32 KB
constexpr int kUnits = 5;
constexpr int kRingBytes = kUnits * kUnitBytes;  // 160 KB
constexpr int kGroupRegion = kBlockRows * kRB;   // one group's 128 token rows inside a token unit

__device__ __forceinline__ int swz128(int row) { return (row >> 1) & 7; }

struct Loader {
    const char *tok_base;
    const char *w_base;   // start of this wave's 128-row half of the weight tile
    uint32_t tok_off[4];  // byte offset of this lane's chunk in instruction i, slab 0
    uint32_t w_off[4];
    int dst;              // LDS offset of the wave's 32 rows inside a unit
    bool tok_live;        // this wave's token fragment has live rows

    // row_off(row) = byte offset of token tile row `row` (0..255) in tok_base; weight rows: the two
    // 128-row halves of the tile start at w_half[0/1], `w_pitch` bytes per row.
    template <typename TokOff>
    __device__ __forceinline__ void setup(int tid, const char *tok, const char *w_half0, const char *w_half1,
                                          uint32_t w_pitch, int ntf0, int ntf1, TokOff row_off) {
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        dst = wave * 32 * kRB;
        tok_live = (wave & 3) < (wave < 4 ? ntf0 : ntf1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = 32 * wave + 8 * i + (lane >> 3);
            const uint32_t chunk = (uint32_t)((lane & 7) ^ swz128(row)) * 16u;
            w_off[i] = (uint32_t)(row & 127) * w_pitch + chunk;
            tok_off[i] = tok_live ? row_off(row) + chunk : 0u;
        }
        tok_base = ring::uniform_ptr(tok);
        w_base = ring::uniform_ptr(wave < 4 ? w_half0 : w_half1);
    }
    // Copies i0 and i0 + 1 (of 4) of this wave's share of a weight / token unit.
    __device__ __forceinline__ void issue_w2(char *unit, int slab, int i0) const {
        const uint32_t koff = (uint32_t)slab * kRB;
#pragma unroll
        for (int i = i0; i < i0 + 2; ++i) ring::copy16(w_base, w_off[i] + koff, unit + dst + i * 8 * kRB);
    }
    __device__ __forceinline__ void issue_t2(char *unit, int slab, int i0) const {
        if (!tok_live) return;
        const uint32_t koff = (uint32_t)slab * kRB;
#pragma unroll
        for (int i = i0; i < i0 + 2; ++i) ring::copy16(tok_base, tok_off[i] + koff, unit + dst + i * 8 * kRB);
    }
    __device__ __forceinline__ void issue_w(char *unit, int slab) const {
        issue_w2(unit, slab, 0);
        issue_w2(unit, slab, 2);
    }
    __device__ __forceinline__ void issue_t(char *unit, int slab) const {
        issue_t2(unit, slab, 0);
        issue_t2(unit, slab, 2);
    }
};

// Operand fragments of K sub-step j (16 bf16) of the slab: lane l holds row l % 32, chunk 2 j + l / 32.
template <int NTF>
__device__ __forceinline__ void fetch(ring::FragsBf16 &fr, const char *tok, const char *wgt, const int (&wrow)[2],
                                      int lane, int j) {
    const int r = lane & 31, half = lane >> 5, sx = (lane >> 1) & 7;
    const int off = r * kRB + (((2 * j + half) ^ sx) << 4);
#pragma unroll
    for (int f = 0; f < 2; ++f) fr.a[f] = *reinterpret_cast<const bf16x8 *>(wgt + wrow[f] * kRB + off);
#pragma unroll
    for (int t = 0; t < 4; ++t)
        if (t < NTF) fr.b[t] = *reinterpret_cast<const bf16x8 *>(tok + t * 32 * kRB + off);
}

// Issue order of one (fetch, mma) pair of full tiles: the 8 MFMAs of one fragment buffer alternate
// with the 6 LDS reads that refill the other.
template <int NTF>
__device__ __forceinline__ void interleave_pair() {
    if constexpr (NTF == 4) {
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    }
}

// K loop.  COMPUTE = false is the loop of a group without live rows: its waves only copy their
// share of the weight rows and join the barriers.  `tok_region` = byte offset of the group's token
// rows inside a token unit.  Slabs are visited in rotated order starting at `start`.
template <int NTF, bool TRANSPOSED, bool COMPUTE>
__device__ __forceinline__ void main_loop(f32x16 (&acc)[2][4], const Loader &ld, char *lds, int n_slabs,
                                          const int (&wrow)[2], int lane, int tok_region, int start) {
    auto rot = [&](int s) {
        s += start;
        return s >= n_slabs ? s - n_slabs : s;
    };
    auto next = [](int b, int d) {
        b += d;
        return b >= kUnits ? b - kUnits : b;
    };
    ld.issue_w(lds, rot(0));
    ld.issue_t(lds + kUnitBytes, rot(0));
    if (n_slabs > 1) ld.issue_w(lds + 2 * kUnitBytes, rot(1));
    ring::FragsBf16 fx, fy;  // fy carries the held-back last sub-step across the barrier
    if constexpr (COMPUTE) {
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int i = 0; i < 8; ++i) fy.a[f][i] = (__bf16)0.0f;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 8; ++i) fy.b[t][i] = (__bf16)0.0f;
    }
    int bw = 0;  // buffer of weight unit kt; the token unit sits in the next buffer
    for (int kt = 0; kt < n_slabs; ++kt) {
        if (kt + 1 < n_slabs) ring::wait_and_barrier<4>();
        else ring::wait_and_barrier<0>();
        // Everybody is past the barrier: the buffers of slab kt - 1 (bw + 3, bw + 4) are free.  Their
        // refill (token unit kt + 1, then weight unit kt + 2) is spread over the slab, two copies per
        // quarter, so that the copy instructions of the eight waves reach the memory pipeline at the
        // rate it retires them instead of queueing in front of every wave's matrix instructions.
        char *t_unit = lds + next(bw, 3) * kUnitBytes;
        char *w_unit = lds + next(bw, 4) * kUnitBytes;
        const bool more_t = kt + 1 < n_slabs, more_w = kt + 2 < n_slabs;
        const int t_slab = rot(kt + 1), w_slab = rot(kt + 2);
        if constexpr (COMPUTE) {
            const char *wgt = lds + bw * kUnitBytes;
            const char *tok = lds + next(bw, 1) * kUnitBytes + tok_region;
            if (more_t) ld.issue_t2(t_unit, t_slab, 0);
            fetch<NTF>(fx, tok, wgt, wrow, lane, 0);
            ring::mma_bf16<NTF, TRANSPOSED>(acc, fy);
            interleave_pair<NTF>();
            if (more_t) ld.issue_t2(t_unit, t_slab, 2);
            fetch<NTF>(fy, tok, wgt, wrow, lane, 1);
            ring::mma_bf16<NTF, TRANSPOSED>(acc, fx);
            interleave_pair<NTF>();
            if (more_w) ld.issue_w2(w_unit, w_slab, 0);
            fetch<NTF>(fx, tok, wgt, wrow, lane, 2);
            ring::mma_bf16<NTF, TRANSPOSED>(acc, fy);
            interleave_pair<NTF>();
            if (more_w) ld.issue_w2(w_unit, w_slab, 2);
            fetch<NTF>(fy, tok, wgt, wrow, lane, 3);
            ring::mma_bf16<NTF, TRANSPOSED>(acc, fx);
            interleave_pair<NTF>();
        } else {
            if (more_t) ld.issue_t(t_unit, t_slab);
            if (more_w) ld.issue_w(w_unit, w_slab);
        }
        bw = next(bw, 2);
    }
    if constexpr (COMPUTE) ring::mma_bf16<NTF, TRANSPOSED>(acc, fy);
    __syncthreads();  // all reads of the last units are done: the ring may be reused as scratch
}

}  // namespace ring128
}  // namespace pmoe
