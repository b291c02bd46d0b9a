// Tall bf16 tiles of the grouped-GEMM kernels, gfx950: up to 384 token rows x 256 weight rows on eight
// waves (two per SIMD).
//
// Why: a 256 x 256 tile moves 64 KB from L2 to LDS per 2048 matrix-pipe cycles, and that copy path, not
// the matrix pipe, sets its pace.  A 384 x 256 tile moves 80 KB per 3072 cycles (-17 % bytes per flop).
// Tiles are cut by 32-row fragments, not by 128-row blocks: the tiles of an expert are of equal size (+-1
// pair of fragments), so no tile streams the expert's weight rows for a handful of rows.
//
// A tile has NTF = 2 FG token fragments (FG = 1 .. 6).  Wave (g, v) (g = wave / 4, v = wave % 4) owns
// token fragments g FG .. g FG + FG - 1 against two 32-row fragments of the weight tile (chosen by the
// caller: gate and matching up rows in the up kernel, so that both operands of one SwiGLU element land
// in the same lane and register): 2 x FG accumulators, at most 192 registers.
//
// LDS is a ring of stages, each [NTF token fragments of 4 KB][256 weight rows x 128 B]; as many stages
// as fit 160 KB, at most 4 (2 for NTF >= 6).  Rows are 8 chunks of 16 B, chunk c of row r in slot
// c ^ ((r >> 1) & 7), the layout of the other ring engines.  Wave w copies the 1 KB pieces (8 rows) w,
// w + 8, ... of a stage's weight rows (4 instructions) and of its token rows (FG instructions): the same
// count for every wave.
//
// Operand fragments are single-buffered: the registers of a fragment are refilled for the next 16-wide K
// sub-step right behind the last matrix instruction that reads them, FG or more matrix instructions
// before their next use.  The barrier that opens slab k + 1 sits in the middle of the last sub-step of
// slab k, where every fragment of slab k is in registers; the second half of that sub-step's matrix
// instructions covers the latency of the first reads of slab k + 1.
#pragma once
#include "moe_ring.h"

namespace pmoe {
namespace tall {

constexpr int kRB = 128;                    // row bytes of a slab
constexpr int kFragBytes = 32 * kRB;        // one 32-row token fragment of a slab
constexpr int kWUnitBytes = kWRows * kRB;   // the 256 weight rows of a slab
constexpr int kLdsBytes = 160 * 1024;
constexpr int kMaxFrags = 12;

template <int FG>
struct Geo {
    static constexpr int kNTF = 2 * FG;
    static constexpr int kTokBytes = kNTF * kFragBytes;
    static constexpr int kStageBytes = kTokBytes + kWUnitBytes;
    static constexpr int kFit = kLdsBytes / kStageBytes;
    static constexpr int kStages = kFit < 4 ? kFit : 4;
    static constexpr int kCopies = FG + 4;  // copy instructions per wave and stage
    static_assert(kStages >= 2, "a tall tile needs two stages");
};

// GATHER: the token rows of the tile are anywhere in `tok` (x rows picked by the schedule); otherwise they
// are consecutive rows of it (activation rows by sorted row), and one offset register serves all pieces.
template <int FG, bool GATHER>
struct Loader {
    static constexpr int NT = GATHER ? FG : 1;
    const char *tok_base;  // wave-uniform; gathered x rows (up kernel) or activation rows (down kernel)
    const char *w_base;    // wave-uniform: row 0 of the weight tile's first 128-row half
    const char *w_base2;   // the second half
    uint32_t tok_off[NT];  // byte offset of this lane's chunk of its token rows, slab 0
    uint32_t tok_step;     // !GATHER: bytes between the rows of consecutive pieces of this wave (64 rows)
    uint32_t w_off;        // the same for its weight rows, relative to row 0 of a half (first of the wave's two pieces)
    uint32_t w_step;       // bytes between the wave's two pieces of a half (64 rows)
    int lds_piece;         // LDS offset of the wave's first piece inside a 8 KB group of pieces

    // row_off(row) = byte offset of tile row `row` (0 .. 64 FG - 1) in `tok` (!GATHER: row * tok_pitch).
    template <typename TokOff>
    __device__ __forceinline__ void setup(int tid, const char *tok, const char *w_half0, const char *w_half1,
                                          uint32_t w_pitch, uint32_t tok_pitch, TokOff row_off) {
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
        lds_piece = wave * 1024;
        // piece p (8 rows) of a run of rows: rows 8 p .. 8 p + 7; this wave takes pieces wave + 8 q.  The
        // swizzle of row 8 (wave + 8 q) + lane / 8 does not depend on q.
        const int row = 8 * wave + (lane >> 3);
        const uint32_t chunk = (uint32_t)((lane & 7) ^ ((row >> 1) & 7)) * 16u;
#pragma unroll
        for (int q = 0; q < NT; ++q) tok_off[q] = row_off(row + 64 * q) + chunk;
        tok_step = 64u * tok_pitch;
        w_off = (uint32_t)row * w_pitch + chunk;
        w_step = 64u * w_pitch;
        tok_base = ring::uniform_ptr(tok);
        w_base = ring::uniform_ptr(w_half0);
        w_base2 = ring::uniform_ptr(w_half1);
    }
    // Copy c (of FG + 4; a constant once the caller's loop is unrolled) of this wave's share of a stage: the
    // weight rows first, then the token rows.
    __device__ __forceinline__ void issue(int c, char *stage, uint32_t koff) const {
        if (c < 4) {
            ring::copy16((c < 2 ? w_base : w_base2) + koff + (c & 1) * (size_t)w_step, w_off,
                         stage + Geo<FG>::kTokBytes + (c >> 1) * 128 * kRB + (c & 1) * 8192 + lds_piece);
        } else if constexpr (GATHER) {
            ring::copy16(tok_base + koff, tok_off[c - 4], stage + (c - 4) * 8192 + lds_piece);
        } else {
            ring::copy16(tok_base + koff + (c - 4) * (size_t)tok_step, tok_off[0], stage + (c - 4) * 8192 + lds_piece);
        }
    }
    __device__ __forceinline__ void issue_all(char *stage, uint32_t koff) const {
#pragma unroll
        for (int c = 0; c < Geo<FG>::kCopies; ++c) issue(c, stage, koff);
    }
};

__device__ __forceinline__ bf16x8 lds_frag(const char *p) { return *reinterpret_cast<const bf16x8 *>(p); }

// Nothing crosses this point in the instruction schedule: the order written is the order issued.
#define PMOE_TALL_FENCE() __builtin_amdgcn_sched_barrier(0)

// One slab of the K loop: four 16-wide sub-steps on the fragments held in a0, a1, b[] (sub-step 0 of `stage`
// on entry), which are replaced as they are used up by those of the next sub-step; the last sub-step's
// successors come from `nstage`, behind the barrier that certifies it has landed (LAST: there is none).  The
// copies of the stage being filled (`fill`: into `fstage`, slab offset `fkoff`) are spread over the first
// matrix instructions of sub-steps 0 and 1.
template <int FG, bool LAST, typename LD>
__device__ __forceinline__ void slab(f32x16 (&acc)[2][FG], bf16x8 &a0, bf16x8 &a1, bf16x8 (&b)[FG], const LD &ld,
                                     const char *stage, const char *nstage, bool fill, char *fstage, uint32_t fkoff,
                                     int off0, int w_at0, int w_at1, int t_at, int wait_later) {
    using G = Geo<FG>;
    constexpr int LPS = G::kCopies, SLOTS = 2 * FG;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const char *src = j < 3 ? stage : nstage;
        const int o = off0 ^ (((j + 1) & 3) << 5);  // chunk 2 j' + half of the lane's row, swizzled
#pragma unroll
        for (int t = 0; t < FG; ++t) {
            acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b[t], acc[0][t], 0, 0, 0);
            if (j < 2) {
                // copies [q LPS / SLOTS, (q + 1) LPS / SLOTS) behind matrix instruction q of the slab
                const int q = j * FG + t;
                const int c0 = q * LPS / SLOTS, c1 = (q + 1) * LPS / SLOTS;
                if (c1 > c0 && fill) {
#pragma unroll
                    for (int c = 0; c < LPS; ++c)
                        if (c >= c0 && c < c1) ld.issue(c, fstage, fkoff);
                }
            }
            PMOE_TALL_FENCE();
        }
        if (j == 3) {
            if constexpr (LAST) {
#pragma unroll
                for (int t = 0; t < FG; ++t)
                    acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b[t], acc[1][t], 0, 0, 0);
                return;
            } else {
                // the next slab has landed once at most the copies of the later slabs are pending
                if (wait_later <= 0) ring::wait_and_barrier<0>();
                else if (wait_later == 1) ring::wait_and_barrier<LPS>();
                else ring::wait_and_barrier<2 * LPS>();
            }
        }
        a0 = lds_frag(src + w_at0 + o);
        PMOE_TALL_FENCE();
#pragma unroll
        for (int t = 0; t < FG; ++t) {
            acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b[t], acc[1][t], 0, 0, 0);
            b[t] = lds_frag(src + t_at + t * kFragBytes + o);
            PMOE_TALL_FENCE();
        }
        a1 = lds_frag(src + w_at1 + o);
        PMOE_TALL_FENCE();
    }
}

// K loop of one tile.  acc[f][t]: weight fragment f (rows wrow[f] .. + 31 of the weight tile) against token
// fragment tok_frag0 + t (weight rows on the MFMA M side).  Slabs are visited in rotated order starting at
// `start`.  Ends with a barrier: the ring may be reused as scratch afterwards.
template <int FG, typename LD>
__device__ __forceinline__ void main_loop(f32x16 (&acc)[2][FG], const LD &ld, char *lds, int n_slabs,
                                          const int (&wrow)[2], int tok_frag0, int lane, int start) {
    using G = Geo<FG>;
    constexpr int S = G::kStages, LPS = G::kCopies, SB = G::kStageBytes;
    auto rot = [&](int s) {
        s += start;
        return s >= n_slabs ? s - n_slabs : s;
    };
    const int r = lane & 31, half = lane >> 5, sx = (lane >> 1) & 7;
    // sub-step j reads chunk (2 j + half) ^ sx of the lane's row: off0 ^ (j << 5)
    const int off0 = r * kRB + ((half ^ sx) << 4);
    const int w_at0 = G::kTokBytes + wrow[0] * kRB, w_at1 = G::kTokBytes + wrow[1] * kRB;
    const int t_at = tok_frag0 * kFragBytes;

#pragma unroll
    for (int s = 0; s < S - 1; ++s)
        if (s < n_slabs) ld.issue_all(lds + s * SB, (uint32_t)rot(s) * kRB);
    {
        // slab 0 has landed once at most the copies of the later slabs (up to S - 2) are pending
        const int later = min(S - 2, n_slabs - 1);
        if (later <= 0) ring::wait_and_barrier<0>();
        else if (later == 1) ring::wait_and_barrier<LPS>();
        else ring::wait_and_barrier<2 * LPS>();
    }
    bf16x8 a0, a1, b[FG];
    a0 = lds_frag(lds + w_at0 + off0);
    a1 = lds_frag(lds + w_at1 + off0);
#pragma unroll
    for (int t = 0; t < FG; ++t) b[t] = lds_frag(lds + t_at + t * kFragBytes + off0);

    int cur = 0;  // stage of slab kt
    for (int kt = 0; kt < n_slabs - 1; ++kt) {
        // the stage slab kt - 1 used is free: everybody is past the barrier that opened slab kt
        const bool fill = kt + S - 1 < n_slabs;
        int fs = cur - 1;
        if (fs < 0) fs += S;
        int nx = cur + 1;
        if (nx >= S) nx = 0;
        slab<FG, false>(acc, a0, a1, b, ld, lds + cur * SB, lds + nx * SB, fill, lds + fs * SB,
                        (uint32_t)rot(fill ? kt + S - 1 : 0) * kRB, off0, w_at0, w_at1, t_at,
                        S == 2 ? 0 : min(S - 2, n_slabs - 2 - kt));
        cur = nx;
    }
    slab<FG, true>(acc, a0, a1, b, ld, lds + cur * SB, lds, false, lds, 0u, off0, w_at0, w_at1, t_at, 0);
    __syncthreads();  // all reads of the last stage are done: the ring may be reused as scratch
}

}  // namespace tall
}  // namespace pmoe
