// Fused MoE forward for gfx950: the C entry points, the mxfp8 kernels (gate/up grouped GEMM + SwiGLU +
// on-chip MX requantisation, down GEMM) and the routing-weight reduction that ends both pipelines.  The
// bf16 kernels live in fused_moe_bf16.hip.
//
// Replaces the launchers and kernels of the reference's
// prime_moe/csrc/kernels/fused_moe_bf16_kernel.cu:930-964 (launcher) and fused_moe_mxfp8_kernel.cu:56-866.
//
// Pipeline of one call (all on the caller's stream):
//   prologue (row tiles and the schedule of the two kernels; inverts the sorted order: pair id -> sorted
//             row; mxfp8: re-tiles the scales of the gathered x rows)
//   -> up kernel (gate/up GEMM + SwiGLU, activation tile -> workspace)
//   -> down kernel (y[pair id, :K] = act . W2[e]^T, bf16, -> workspace)
//   -> finalize: out[t] = bf16(sum over the token's pairs p of w[p] * y[p]), fp32 sum in pair order;
//      split == 0: added to `out` (the reference's accumulate-into-out contract of its single-kernel
//      path), split != 0: `out` overwritten.
// Both values of `split` run the same kernels: on this hardware the two-kernel pipeline is the faster
// one at every shape, so `split` only selects what finalize does with `out`.  No value is accumulated with
// atomics and every sum has a fixed order: the result is a pure function of the inputs.
#include <algorithm>

#include "moe_pipeline.h"
#include "moe_ring.h"

namespace pmoe {

// Slab width (bytes per row and slab) of the stage-ring tiles.  128: every request is a whole cache line.
// 64 (twice the stages in the same LDS) stays selectable at build time for measurements: with the
// non-temporal weight copies it runs the decode shape 32 % and the DeepSeek-like prefill 40 % slower.
#ifndef PMOE_SKINNY_RB
#define PMOE_SKINNY_RB 128
#endif
#ifndef PMOE_PART_RB
#define PMOE_PART_RB 128
#endif
constexpr int kSkinnyRB = PMOE_SKINNY_RB;  // tiles with one live fragment
constexpr int kPartRB = PMOE_PART_RB;      // mxfp8 tiles with more

// What one workgroup of an mxfp8 kernel does: `n_sub` consecutive weight tiles from `wt` on for the row tile
// of `nb` blocks starting at block `first`, expert `e`.
struct Job {
    int first, nb, wt, e, n_sub;
    bool w_once;  // no other row tile of this expert: nobody else reads the weight rows of this job
};

// Workgroup id -> job: one load from the work list, which the prologue lays out by workgroup id (see
// emit_work); entries of workgroups without work are -1.
__device__ __forceinline__ bool resolve_job(const MoeArgs &a, Job &j) {
    const int4 w = a.work[blockIdx.x];
    if (w.x < 0) return false;
    j.first = w.x & 0x0fffffff;
    j.nb = w.x >> 28;
    j.wt = w.y & 0xffff;
    j.e = (w.y >> 16) & 0x3ff;
    j.n_sub = ((w.y >> 26) & 0xf) + 1;
    j.w_once = (w.w & 1) != 0;
    return true;
}

template <int NG>
struct RowInfo {
    int tok[kBlockRows * NG];   // token index of each sorted row, -1 for padding / dropped rows
    int pair[kBlockRows * NG];  // its pair id (the row of y it writes), -1 likewise
    int nvalid[NG];             // per group: 1 + index of the last live row
};

// Fills RowInfo for the `nb` blocks starting at `first`; returns the largest number of 32-row
// fragments holding live rows in any group.
template <int NG>
__device__ __forceinline__ int load_row_info(const MoeArgs &a, int first, int nb, RowInfo<NG> &ri) {
    const int tid = threadIdx.x;
    if (tid < NG) ri.nvalid[tid] = 0;
    __syncthreads();
    if (tid < kBlockRows * NG) {
        const int g = tid >> 7;
        int tok = -1, pair = -1;
        if (g < nb) {
            const int s = first * kBlockRows + tid;
            const int p = (s < a.sorted_num) ? a.sorted_ids[s] : -1;
            if (p >= 0 && p / a.top_k < a.M) {
                tok = p / a.top_k;
                pair = p;
            }
        }
        ri.tok[tid] = tok;
        ri.pair[tid] = pair;
        if (tok >= 0) atomicMax(&ri.nvalid[g], (tid & 127) + 1);
    }
    __syncthreads();
    int m = 0;
#pragma unroll
    for (int g = 0; g < NG; ++g) m = max(m, (ri.nvalid[g] + 31) >> 5);
    return m;
}

__device__ __forceinline__ void zero_acc(f32x16 (&acc)[2][4]) {
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[f][t][i] = 0.f;
}

// Epilogue of the down GEMM.  Weight rows (output columns) sit on the MFMA M side: register i of lane
// l = output column 64 w4 + 32 f + 8(i/4) + 4(l/32) + i%4 of sorted row 32 t + l%32.  The group's
// 128 x 256 tile is rounded to bf16 into `tile` (row pitch kYPitch) ...
template <int NTF>
__device__ __forceinline__ void y_epilogue(const f32x16 (&acc)[2][4], char *tile, int w4, int lane) {
    const int r = lane & 31, half = lane >> 5;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (t < NTF) {
            const int row = 32 * t + r;
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int col = 64 * w4 + 32 * f + 8 * g + 4 * half;
                    uint2 pk;
                    pk.x = pack2_bf16(acc[f][t][4 * g], acc[f][t][4 * g + 1]);
                    pk.y = pack2_bf16(acc[f][t][4 * g + 2], acc[f][t][4 * g + 3]);
                    *reinterpret_cast<uint2 *>(tile + row * kYPitch + col * 2) = pk;
                }
        }
    }
}
// Where a group's 128 x 256 output tile goes: the y rows of its pairs (y is indexed by pair id, row pitch
// K; the last tile of a K that is not a multiple of 256 has 128 columns).
struct YDst {
    char *base;     // first column of the group's tile in row 0 of y
    int64_t pitch;  // bytes per row
    int cols;       // columns to write
};
__device__ __forceinline__ YDst y_destination(const MoeArgs &a, int k0) {
    YDst d;
    d.base = a.y + (int64_t)k0 * 2;
    d.pitch = (int64_t)a.K * 2;
    d.cols = min(kWRows, a.K - k0);
    return d;
}
// Tiles with a single live fragment skip the detour through LDS: every lane stores its 8-byte runs
// straight to the destination (32 rows x 16 KB per tile at most; a barrier and an LDS round trip cost more).
// `pair_r` = pair id of this lane's row (lane % 32) of the group, < 0 if the row holds none.
__device__ __forceinline__ void store_y_direct(const YDst &d, const f32x16 (&acc)[2][4], int n_rows, int w4, int lane,
                                               int pair_r) {
    const int r = lane & 31, half = lane >> 5;
    if (r >= n_rows || pair_r < 0) return;
    char *dst = d.base + pair_r * d.pitch;
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int col = 64 * w4 + 32 * f + 8 * g + 4 * half;
            if (col < d.cols) {
                uint2 pk;
                pk.x = pack2_bf16(acc[f][0][4 * g], acc[f][0][4 * g + 1]);
                pk.y = pack2_bf16(acc[f][0][4 * g + 2], acc[f][0][4 * g + 3]);
                *reinterpret_cast<uint2 *>(dst + col * 2) = pk;
            }
        }
}
// ... and its first n_rows rows are copied to the destination; gt = thread index inside the group,
// `pair` = the pair ids of the group's 128 rows (rows without one are skipped).
__device__ __forceinline__ void store_y_tile(const YDst &d, const char *tile, int n_rows, int gt, const int *pair) {
    const int c = gt & 31;
    if (8 * c >= d.cols) return;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int row = (gt >> 5) + 8 * i;
        if (row < n_rows) {
            const int dst_row = pair[row];
            if (dst_row >= 0) {
                const uint4 v = *reinterpret_cast<const uint4 *>(tile + row * kYPitch + c * 16);
                store_once(d.base + dst_row * d.pitch + c * 16, v);
            }
        }
    }
}

// SwiGLU epilogue of the up GEMM, in registers: the 2H-wide gate/up tensor never leaves the chip.
// acc[0] holds gate rows, acc[1] the matching up rows (weight rows on the MFMA M side: register i
// of lane l = activation column 32 w4 + 8(i/4) + 4(l/32) + i%4 of token row 32 t + l%32).  The
// 128 x 128 activation tile of the group is written to `tile` with row pitch kActPitch*, for the
// coalesced copy to the workspace.
// mxfp8: per token row and 32 columns, amax -> e8m0 scale + e4m3 values; a lane holds 16 of the 32
// columns of one MX block, the partner lane (l ^ 32) the others.
template <int DT, int NTF>
__device__ __forceinline__ void swiglu_epilogue(const f32x16 (&acc)[2][4], char *tile, uint32_t *sc_tile,
                                                int w4, int lane) {
    const int r = lane & 31, half = lane >> 5;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (t < NTF) {
            float v[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = swiglu(acc[0][t][i], acc[1][t][i]);
            const int row = 32 * t + r;
            static_assert(DT == DT_FP8, "the bf16 epilogue lives in fused_moe_bf16.hip");
            float amax = 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[i]));
            amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
            uint32_t e8;
            float inv;
            mx_block_scale(amax, e8, inv);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int hl = 32 * w4 + 8 * g + 4 * half;
                const uint32_t q = pack4_e4m3(v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3], inv);
                *reinterpret_cast<uint32_t *>(tile + row * kActPitchFp8 + hl) = q;
            }
            if (half == 0) reinterpret_cast<uint8_t *>(sc_tile)[row * 4 + w4] = (uint8_t)e8;
        }
    }
}

// Coalesced copy of the first 32*ntf rows of a group's activation tile (pitch kActPitch*) to the
// workspace rows row0.., columns [h0, h0+128); gt = thread index inside the group (0..255).
template <int DT>
__device__ __forceinline__ void store_act_tile(const MoeArgs &a, const char *tile, const uint32_t *sc_tile,
                                               int64_t row0, int h0, int ntf, int gt) {
    const int H = a.H;
    static_assert(DT == DT_FP8, "the bf16 epilogue lives in fused_moe_bf16.hip");
    const int c = gt & 7;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = (gt >> 3) + 32 * i;
        if (i < ntf) {
            uint4 v = *reinterpret_cast<const uint4 *>(tile + row * kActPitchFp8 + c * 16);
            store_once(a.act + (row0 + row) * H + h0 + c * 16, v);
        }
    }
    if (gt < 32 * ntf)
        a.act_scales[((row0 >> 7) * (H >> 7) + (h0 >> 7)) * kBlockRows + gt] = sc_tile[gt];
}

// ==========================================================================================
// Two-group kernels on the ring engines
// ==========================================================================================

// Common set-up of the stage-ring loader.  Token rows: `tok_row_off(row)` gives the byte offset of
// tile row `row` (0..255: block 0, then block 1) in `tok_base`; weight rows: the tile's two 128-row
// halves start at w_base[0/1] with `w_pitch` bytes per row.  Scales (mxfp8): `tok_sc_off(row)` /
// `w_sc_off(row)` are the byte offsets of the row's first 4-scale dword; the dword of the next 128-wide
// K tile lies 512 bytes on in both (blocked weight scales, tiled token-side scales).  Only the live 32-row
// fragments of the two blocks (ntf0, ntf1 of them) are copied; they are packed one after the other in
// the stage (see ring::Layout).
template <int DT, int RB, typename TokOff, typename TokScOff, typename WScOff>
__device__ __forceinline__ void setup_ring_loader(ring::Loader<RB> &ld, const ring::Layout &lay, int tid,
                                                  uint32_t w_pitch, int ntf0, int ntf1, const RowInfo<2> &ri,
                                                  bool w_once, TokOff tok_row_off,
                                                  const uint8_t *tok_sc_base, TokScOff tok_sc_off,
                                                  const uint8_t *w_sc_base, WScOff w_sc_off) {
    using L = ring::Loader<RB>;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
#pragma unroll
    for (int q = 0; q < L::N; ++q) {
        const int row = L::row_of(wave, lane, q);          // row inside a 128-row block / half
        const int row0 = L::row_of(wave, 0, q);            // first row of the instruction
        const uint32_t gchunk = (uint32_t)((lane % (RB / 16)) ^ ring::swz<RB>(row)) * 16u;  // global chunk of this lane's slot
        ld.w_off[q] = (uint32_t)row * w_pitch + gchunk;
        ld.w_dst[0][q] = lay.w_off + row0 * RB;
        ld.w_dst[1][q] = ld.w_dst[0][q] + 128 * RB;
        const int frag = row0 >> 5;  // the instruction's rows lie in this 32-row fragment
        ld.tok_dst[0][q] = ld.tok_dst[1][q] = -1;
        ld.tok_off[0][q] = ld.tok_off[1][q] = 0;
        ld.tok_live[0][q] = frag < ntf0 && ri.tok[row] >= 0;
        ld.tok_live[1][q] = frag < ntf1 && ri.tok[kBlockRows + row] >= 0;
        if (__ballot(ld.tok_live[0][q]) != 0) {
            ld.tok_dst[0][q] = row0 * RB;
            ld.tok_off[0][q] = tok_row_off(row) + gchunk;
        }
        if (__ballot(ld.tok_live[1][q]) != 0) {
            ld.tok_dst[1][q] = lay.group1_off + row0 * RB;
            ld.tok_off[1][q] = tok_row_off(kBlockRows + row) + gchunk;
        }
    }
    ld.sc_base = nullptr;
    ld.sc_off = 0;
    ld.sc_step = 0;
    ld.sc_dst = -1;
    if constexpr (DT == DT_FP8) {
        if (wave >= 4) {  // weight rows 64 (wave - 4) + lane
            const int row = 64 * (wave - 4) + lane;
            ld.sc_base = reinterpret_cast<const char *>(w_sc_base);
            ld.sc_off = w_sc_off(row);
            ld.sc_step = 512u;
            ld.sc_dst = lay.scale_off + (lay.scale_tok_rows + 64 * (wave - 4)) * 4;
        } else if (64 * wave < lay.tok_rows) {
            // packed token rows 64 wave + lane (the lanes past the last live row repeat it)
            const int c = min(64 * wave + lane, lay.tok_rows - 1);
            const int row = c < 32 * ntf0 ? c : kBlockRows + c - 32 * ntf0;
            ld.sc_base = reinterpret_cast<const char *>(tok_sc_base);
            ld.sc_off = tok_sc_off(row);
            ld.sc_step = 512u;
            ld.sc_dst = lay.scale_off + 64 * wave * 4;
        }
    }
    int lps = 2 * L::N + (ld.sc_dst >= 0);
#pragma unroll
    for (int q = 0; q < L::N; ++q) lps += (ld.tok_dst[0][q] >= 0) + (ld.tok_dst[1][q] >= 0);
    ld.lps = lps;
    ld.w_once = w_once;
    ld.make_uniform();
}

// First slab of this workgroup's walk over K: workgroups that run side by side on an XCD (consecutive
// blockIdx / 8) start 128 bytes apart, 8 distinct phases over a 1 KB period.  The spread keeps the
// workgroups that share a weight tile off the same HBM channel at the same instant, and stays short
// enough that they still meet in L2 (a 16-phase, 4 KB spread read 30 % more from HBM for the same time).
// Even for 64-byte slabs: two of them share a scale dword.
template <int RB>
__device__ __forceinline__ int slab_rotation(int n_slabs) {
    const int phase = (int)((blockIdx.x >> 3) & 7) * (128 / RB);
    return RB == 64 ? phase % n_slabs & ~1 : phase % n_slabs;
}

// Up kernel tile on the stage ring: the live fragments of one or two row blocks x activation
// columns [128 ht, 128 ht + 128).  LDS weight rows 0..127 are gate rows, 128..255 the matching up rows;
// wave v of a group owns gate/up rows 32v..32v+31 so gate and up of one activation element sit in the
// same lane and register.
template <int DT, int RB, int NTF>
__device__ __forceinline__ void up_tile_ring(const MoeArgs &a, const Job &job, RowInfo<2> &ri, char *lds,
                                             uint32_t *act_sc_lds) {
    constexpr int ES = 1;  // bytes per element
    const int first = job.first, ht = job.wt, n_sub = job.n_sub, e = job.e;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, w4 = wave & 3, gt = tid & 255;
    const int K = a.K, H = a.H, N = a.N;
    const int ntf0 = __builtin_amdgcn_readfirstlane((ri.nvalid[0] + 31) >> 5);
    const int ntf1 = __builtin_amdgcn_readfirstlane((ri.nvalid[1] + 31) >> 5);
    const int my_ntf = grp ? ntf1 : ntf0;
    const bool active = my_ntf > 0;
    const ring::Layout lay = ring::make_layout<DT, RB>(ntf0, ntf1, ring::ring_bytes<DT>());

    int h0 = ht * 128;
    const int n_slabs = (K * ES) / RB;
    ring::Loader<RB> ld;
    ld.tok_base = a.x;
    ld.w_base[0] = a.w1 + ((int64_t)e * N + h0) * K * ES;
    ld.w_base[1] = ld.w_base[0] + (int64_t)H * K * ES;
    const uint32_t row_bytes = (uint32_t)(K * ES);
    const int kb = K >> 5, kt128 = K >> 7;
    setup_ring_loader<DT, RB>(
        ld, lay, tid, row_bytes, ntf0, ntf1, ri, job.w_once,
        [&](int row) { return (uint32_t)max(ri.tok[row], 0) * row_bytes; },
        reinterpret_cast<const uint8_t *>(a.xs_tiled + (int64_t)first * kt128 * kBlockRows),
        [&](int row) { return (uint32_t)(((row >> 7) * kt128 * kBlockRows + (row & 127)) * 4); },
        a.w1_scales + (int64_t)e * N * kb,
        [&](int row) { return (uint32_t)blocked_scale_off((row < 128 ? h0 : H + h0 - 128) + row, 0, K >> 7); });

    const int wrow[2] = {32 * w4, 128 + 32 * w4};
    const int start = slab_rotation<RB>(n_slabs);
    const int tok_region = grp ? lay.group1_off : 0;
    // the ring is free after main_loop (it ends with a barrier): its head holds the activation tiles
    constexpr int kPitch = kActPitchFp8;
    char *tile = lds + grp * (kBlockRows * kPitch);
    uint32_t *sc_tile = act_sc_lds + grp * kBlockRows;
    const int SB = lay.stage_bytes, NS = lay.stages;
    // first stage clear of the activation tiles: the next weight tile's copies start there, under
    // the epilogue of this one
    const int epi_bytes = (ntf1 > 0 ? 2 : 1) * kBlockRows * kPitch;
    const int free0 = (epi_bytes + SB - 1) / SB;
    int stage0 = 0, n_pre = 0;
    for (int sub = 0; sub < n_sub; ++sub) {
        f32x16 acc[2][4];
        zero_acc(acc);
        if (active)
            ring::main_loop<DT, RB, NTF, true, true>(acc, ld, lay, lds, n_slabs, wrow, lane, tok_region, start, stage0, n_pre);
        else
            ring::main_loop<DT, RB, NTF, true, false>(acc, ld, lay, lds, n_slabs, wrow, lane, tok_region, start, stage0, n_pre);
        const bool more = sub + 1 < n_sub;
        if (more) {
            // same token rows, the next 128 gate and 128 up rows of the expert
            ld.w_base[0] += (int64_t)128 * K * ES;
            ld.w_base[1] += (int64_t)128 * K * ES;
            if (DT == DT_FP8 && wave >= 4) ld.sc_off += (uint32_t)kt128 * 512u;
            ld.make_uniform();
            stage0 = free0 < NS ? free0 : 0;
            n_pre = free0 < NS ? min(NS - 1, NS - free0) : 0;
            ring::pre_issue<DT, RB>(ld, lay, lds, n_slabs, start, stage0, n_pre);
        }
        if (active) swiglu_epilogue<DT, NTF>(acc, tile, sc_tile, w4, lane);
        __syncthreads();
        if (active) store_act_tile<DT>(a, tile, sc_tile, (int64_t)(first + grp) * kBlockRows, h0, my_ntf, gt);
        if (more) __syncthreads();  // the tiles have been read: the head of the ring may be filled again
        h0 += 128;
    }
}

// LDS plan of the mxfp8 kernels: ring, row table, activation scales side by side.
template <int DT>
struct SplitLds {
    static constexpr int kRowInfoBytes = 2304;  // >= sizeof(RowInfo<2>)
    static constexpr int kRing = ring::ring_bytes<DT>();
    static constexpr int kRowInfoOff = kRing;
    static constexpr int kActScaleOff = kRowInfoOff + kRowInfoBytes;
    static constexpr int kTotal = kActScaleOff + kBlockRows * 2 * 4;
    static_assert(sizeof(RowInfo<2>) <= kRowInfoBytes, "row table does not fit its slot");
    // the epilogues reuse the head of the ring: two y tiles (down kernel) or two activation tiles (up kernel)
    static_assert(2 * kBlockRows * kYPitch <= kRing, "y tiles of the epilogue overrun their LDS");
    static_assert(2 * kBlockRows * kActPitchFp8 <= kRing, "activation tiles of the epilogue overrun the ring");
};

template <int DT>
__global__ __launch_bounds__(512) void moe_up_kernel(MoeArgs a) {
    using L = SplitLds<DT>;
    __shared__ __attribute__((aligned(1024))) char lds[L::kTotal];
    RowInfo<2> &ri = *reinterpret_cast<RowInfo<2> *>(lds + L::kRowInfoOff);
    Job j;
    if (!resolve_job(a, j)) return;
    const int ntf = load_row_info<2>(a, j.first, j.nb, ri);
    if (ntf == 0) return;
    uint32_t *act_sc_lds = reinterpret_cast<uint32_t *>(lds + L::kActScaleOff);
    if (ntf == 1) up_tile_ring<DT, kSkinnyRB, 1>(a, j, ri, lds, act_sc_lds);
    else if (ntf == 2) up_tile_ring<DT, kPartRB, 2>(a, j, ri, lds, act_sc_lds);
    else up_tile_ring<DT, kPartRB, 4>(a, j, ri, lds, act_sc_lds);
}

// Down kernel tile on the stage ring: y[rows, 256 cols of K] = act[rows, :H] . W2[e][cols, :H]^T, the
// whole reduction over H inside the workgroup; the
// routing weights are applied later, by finalize_kernel.
template <int DT, int RB, int NTF>
__device__ __forceinline__ void down_tile_ring(const MoeArgs &a, const Job &job, RowInfo<2> &ri, char *lds) {
    constexpr int ES = 1;  // bytes per element
    const int first = job.first, kt = job.wt, n_sub = job.n_sub, e = job.e;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, w4 = wave & 3, gt = tid & 255;
    const int K = a.K, H = a.H;
    const int64_t row0 = (int64_t)first * kBlockRows;
    const int ntf0 = __builtin_amdgcn_readfirstlane((ri.nvalid[0] + 31) >> 5);
    const int ntf1 = __builtin_amdgcn_readfirstlane((ri.nvalid[1] + 31) >> 5);
    const int my_ntf = grp ? ntf1 : ntf0;
    const int my_rows = ri.nvalid[grp];  // rows past the last live one are never read back
    const int my_pair = ri.pair[grp * kBlockRows + (lane & 31)];  // (tiles of one fragment store from registers)
    const bool active = my_ntf > 0;
    const ring::Layout lay = ring::make_layout<DT, RB>(ntf0, ntf1, ring::ring_bytes<DT>());

    int k0 = kt * kWRows;
    const uint32_t row_bytes = (uint32_t)(H * ES);
    const int hb = H >> 5, ht128 = H >> 7;
    const int n_slabs = (H * ES) / RB;
    ring::Loader<RB> ld;
    ld.tok_base = a.act + row0 * H * ES;
    // weight rows (output columns) k0 .. k0 + 255 of the expert; the last tile of a K that is not a
    // multiple of 256 has 128 of them and reads the first half twice
    auto set_weights = [&](int k) {
        ld.w_base[0] = a.w2 + ((int64_t)e * K + k) * H * ES;
        ld.w_base[1] = (k + 128 < K) ? ld.w_base[0] + (int64_t)128 * H * ES : ld.w_base[0];
        if (DT == DT_FP8 && wave >= 4)
            ld.sc_off = (uint32_t)blocked_scale_off(min(k + 64 * (wave - 4) + lane, K - 1), 0, ht128);
    };
    set_weights(k0);
    setup_ring_loader<DT, RB>(
        ld, lay, tid, row_bytes, ntf0, ntf1, ri, job.w_once, [&](int row) { return (uint32_t)row * row_bytes; },
        reinterpret_cast<const uint8_t *>(a.act_scales + (int64_t)first * ht128 * kBlockRows),
        [&](int row) { return (uint32_t)(((row >> 7) * ht128 * kBlockRows + (row & 127)) * 4); },
        a.w2_scales + (int64_t)e * K * hb,
        [&](int row) { return (uint32_t)blocked_scale_off(min(k0 + row, K - 1), 0, ht128); });

    const int wrow[2] = {64 * w4, 64 * w4 + 32};
    const int start = slab_rotation<RB>(n_slabs);
    const int tok_region = grp ? lay.group1_off : 0;
    const int SB = lay.stage_bytes, NS = lay.stages;
    // the ring is free after main_loop (it ends with a barrier): its head holds the 128 x 256 output
    // tiles of the live groups (none for tiles of one fragment, which store from registers); the
    // next weight tile's copies start in the first stage clear of them, under this tile's epilogue
    const int epi_bytes = NTF == 1 ? 0 : (ntf1 > 0 ? 2 : 1) * kBlockRows * kYPitch;
    const int free0 = (epi_bytes + SB - 1) / SB;
    int stage0 = 0, n_pre = 0;
    for (int sub = 0; sub < n_sub; ++sub) {
        f32x16 acc[2][4];
        zero_acc(acc);
        if (active)
            ring::main_loop<DT, RB, NTF, true, true>(acc, ld, lay, lds, n_slabs, wrow, lane, tok_region, start, stage0, n_pre);
        else
            ring::main_loop<DT, RB, NTF, true, false>(acc, ld, lay, lds, n_slabs, wrow, lane, tok_region, start, stage0, n_pre);
        const bool more = sub + 1 < n_sub;
        if (more) {
            set_weights(k0 + kWRows);
            ld.make_uniform();
            stage0 = free0 < NS ? free0 : 0;
            n_pre = free0 < NS ? min(NS - 1, NS - free0) : 0;
            ring::pre_issue<DT, RB>(ld, lay, lds, n_slabs, start, stage0, n_pre);
        }
        const YDst dst = y_destination(a, k0);
        if constexpr (NTF == 1) {
            if (active) store_y_direct(dst, acc, my_rows, w4, lane, my_pair);
        } else {
            char *tile = lds + grp * (kBlockRows * kYPitch);
            if (active) y_epilogue<NTF>(acc, tile, w4, lane);
            __syncthreads();
            if (active) store_y_tile(dst, tile, my_rows, gt, ri.pair + grp * kBlockRows);
            if (more) __syncthreads();  // the tiles have been read: the head of the ring may be filled again
        }
        k0 += kWRows;
    }
}

template <int DT>
__global__ __launch_bounds__(512) void moe_down_kernel(MoeArgs a) {
    using L = SplitLds<DT>;
    __shared__ __attribute__((aligned(1024))) char lds[L::kTotal];
    RowInfo<2> &ri = *reinterpret_cast<RowInfo<2> *>(lds + L::kRowInfoOff);
    Job j;
    if (!resolve_job(a, j)) return;
    const int ntf = load_row_info<2>(a, j.first, j.nb, ri);
    if (ntf == 0) return;
    if (ntf == 1) down_tile_ring<DT, kSkinnyRB, 1>(a, j, ri, lds);
    else if (ntf == 2) down_tile_ring<DT, kPartRB, 2>(a, j, ri, lds);
    else down_tile_ring<DT, kPartRB, 4>(a, j, ri, lds);
}

// Walk order of the tiles of one mxfp8 kernel: [group of 8 weight tiles][row tile][weight tile in group].
// The ~32 workgroups that run side by side on an XCD are then 4 consecutive row tiles (mostly of one
// expert) x 8 weight tiles: every token slab they fetch is shared by 8 weight tiles and every weight
// slab by the row tiles of its expert, inside that XCD's L2.
// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin, so position `l` of the walk
// is given to workgroup id 8 * (l mod per_xcd) + l / per_xcd: one XCD then runs a contiguous range of
// the walk.  The entry carries everything the workgroup needs to start: x = first block | blocks << 28,
// y = first weight tile | expert << 16 | (weight tiles - 1) << 26 (experts < 1024, up to 16 weight
// tiles), w = 1 if the row tile is the only one of its expert.
//
// Writes the work list entry of job `j` (of the (n_wt + per_job - 1) / per_job of the row tile; a workgroup
// takes `per_job` consecutive weight tiles).
__device__ __forceinline__ void emit_work(int4 *work, int n_wt, int per_job, int tile, int n_tiles, int first, int nb,
                                          int e, int j, int flags) {
    constexpr int GW = 8;
    const int n_jobs = (n_wt + per_job - 1) / per_job;
    const int per_xcd = (n_tiles * n_jobs + 7) >> 3;
    const int wg = j / GW;
    const int gw = min(GW, n_jobs - wg * GW);
    const int l = wg * GW * n_tiles + tile * gw + (j - wg * GW);
    const int wt = j * per_job, cnt = min(per_job, n_wt - wt);
    const int x = first | (nb << 28), y = wt | (e << 16) | ((cnt - 1) << 26);
    const int pos = l % per_xcd, xcd = l / per_xcd;
    work[8 * pos + xcd] = make_int4(x, y, 0, flags);
}

// Prologue of an mxfp8 call.  Workgroup 0 builds the row tiles and work lists of the two-group kernels:
// consecutive blocks of one expert are paired, an expert's odd last block stays single (one pass of
// block-wide scans per 256 blocks, then one pass over the tiles that writes the two walk orders).
// All workgroups invert the sorted order: inv[pair id] = sorted row.  Entries of pairs that are not
// in the schedule keep whatever the buffer held; the reader validates an entry against sorted_ids.
__global__ __launch_bounds__(256) void moe_prologue_kernel(const int32_t *expert_ids, const int32_t *ntpp,
                                                           int n_blocks, int2 *tiles, int *n_tiles,
                                                           int4 *work_up, int n_wt_up, int per_job_up, int grid_up,
                                                           int4 *work_down, int n_wt_down, int per_job_down,
                                                           int grid_down, int num_experts,
                                                           const int32_t *sorted_ids, int sorted_num, int32_t *inv,
                                                           int n_pairs, int do_invert, const uint8_t *x_scales,
                                                           uint32_t *xs_tiled, int nkt, int top_k, int M) {
    if (blockIdx.x == 0 && tiles != nullptr) {
        __shared__ int s_max[4], s_sum[4], s_carry[2];
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        for (int i = tid; i < grid_up; i += 256) work_up[i] = make_int4(-1, -1, 0, 0);
        for (int i = tid; i < grid_down; i += 256) work_down[i] = make_int4(-1, -1, 0, 0);
        const int n_live = min((ntpp[0] + kBlockRows - 1) / kBlockRows, n_blocks);
        if (tid == 0) { s_carry[0] = 0; s_carry[1] = 0; }
        __syncthreads();
        for (int base = 0; base < n_live; base += 256) {
            const int b = base + tid;
            const bool live = b < n_live;
            const int e = live ? expert_ids[b] : -2;
            const int prev = (live && b > 0) ? expert_ids[b - 1] : -1;
            int v = (live && e != prev) ? b : -1;  // start of a run of equal experts
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int t = __shfl_up(v, d, 64);
                if (lane >= d) v = max(v, t);
            }
            if (lane == 63) s_max[wave] = v;
            __syncthreads();
            int run_start = s_carry[0];
            for (int w = 0; w < wave; ++w) run_start = max(run_start, s_max[w]);
            run_start = max(run_start, v);
            const bool leader = live && (((b - run_start) & 1) == 0);
            const bool paired = leader && (b + 1 < n_live) && expert_ids[b + 1] == e;
            int incl = leader ? 1 : 0;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int t = __shfl_up(incl, d, 64);
                if (lane >= d) incl += t;
            }
            if (lane == 63) s_sum[wave] = incl;
            __syncthreads();
            int off = s_carry[1];
            for (int w = 0; w < wave; ++w) off += s_sum[w];
            if (leader) tiles[off + incl - 1] = make_int2(b, paired ? 2 : 1);
            __syncthreads();
            if (tid == 255) { s_carry[0] = run_start; s_carry[1] = off + incl; }
            __syncthreads();
        }
        const int nt = s_carry[1];
        if (tid == 0) n_tiles[0] = nt;
        __threadfence_block();
        __syncthreads();  // tiles written above are read below by other threads
        const int jobs_up = (n_wt_up + per_job_up - 1) / per_job_up, jobs_down = (n_wt_down + per_job_down - 1) / per_job_down;
        const int per_tile = jobs_up + jobs_down;
        // 1 if row tile t is the only one of its expert e (then nobody else reads that expert's weight rows)
        auto only_tile = [&](int t, int e) {
            const bool before = t > 0 && expert_ids[tiles[t - 1].x] == e;
            const bool after = t + 1 < nt && expert_ids[tiles[t + 1].x] == e;
            return (before || after) ? 0 : 1;
        };
        if (nt >= 64) {  // a row tile per thread and turn, its jobs one after the other
            for (int t = tid; t < nt; t += 256) {
                const int2 tl = tiles[t];
                const int e = expert_ids[tl.x];
                if (e < 0 || e >= num_experts) continue;  // nothing to compute for a block without an expert
                const int fl = only_tile(t, e);
                for (int j = 0; j < jobs_up; ++j) emit_work(work_up, n_wt_up, per_job_up, t, nt, tl.x, tl.y, e, j, fl);
                for (int j = 0; j < jobs_down; ++j) emit_work(work_down, n_wt_down, per_job_down, t, nt, tl.x, tl.y, e, j, fl);
            }
        } else {  // few row tiles for 256 threads: an entry per thread and turn
            for (int i = tid; i < nt * per_tile; i += 256) {
                const int t = i / per_tile, j = i - t * per_tile;
                const int2 tl = tiles[t];
                const int e = expert_ids[tl.x];
                if (e < 0 || e >= num_experts) continue;
                const int fl = only_tile(t, e);
                if (j < jobs_up) emit_work(work_up, n_wt_up, per_job_up, t, nt, tl.x, tl.y, e, j, fl);
                else emit_work(work_down, n_wt_down, per_job_down, t, nt, tl.x, tl.y, e, j - jobs_up, fl);
            }
        }
    }
    if (do_invert) {
        const int n_rows = min(ntpp[0], sorted_num);
        const int stride = (int)(gridDim.x * blockDim.x);
        for (int s = (int)(blockIdx.x * blockDim.x + threadIdx.x); s < n_rows; s += stride) {
            const int p = sorted_ids[s];
            const int e = expert_ids[s >> 7];  // rows of a block without an expert are not computed
            if (p >= 0 && p < n_pairs && e >= 0 && e < num_experts) inv[p] = s;
        }
    }
    if (do_invert && xs_tiled != nullptr) {
        // the e8m0 scales of the gathered x rows, re-tiled for the up kernel's loader (see
        // MoeArgs::xs_tiled); rows without a token get 2^0.  One sorted block per turn, through LDS so
        // that both the reads (a row's scales) and the writes (128 rows of one K tile) are contiguous.
        // Workgroup 0 builds the tiles above and takes no share unless it is alone.
        __shared__ int s_tok[kBlockRows];
        __shared__ uint32_t s_sc[kBlockRows][65];
        const int tid = threadIdx.x;
        const int n_live = min((ntpp[0] + kBlockRows - 1) / kBlockRows, n_blocks);
        const int workers = gridDim.x > 1 ? (int)gridDim.x - 1 : 1;
        const int me = gridDim.x > 1 ? (int)blockIdx.x - 1 : 0;
        const uint32_t *xs = reinterpret_cast<const uint32_t *>(x_scales);  // nkt dwords per token
        for (int b = me; b >= 0 && b < n_live; b += workers) {
            if (tid < kBlockRows) {
                const int srow = b * kBlockRows + tid;
                const int p = srow < sorted_num ? sorted_ids[srow] : -1;
                int tok = p >= 0 ? p / top_k : -1;
                if (tok >= M) tok = -1;
                s_tok[tid] = tok;
            }
            __syncthreads();
            for (int c0 = 0; c0 < nkt; c0 += 64) {
                const int cw = min(64, nkt - c0);
                for (int i = tid; i < kBlockRows * cw; i += 256) {
                    const int r = i / cw, c = i - r * cw;
                    const int tok = s_tok[r];
                    s_sc[r][c] = tok >= 0 ? xs[(int64_t)tok * nkt + c0 + c] : 0x7f7f7f7fu;
                }
                __syncthreads();
                for (int i = tid; i < kBlockRows * cw; i += 256) {
                    const int c = i >> 7, r = i & 127;
                    xs_tiled[((int64_t)b * nkt + c0 + c) * kBlockRows + r] = s_sc[r][c];
                }
                __syncthreads();
            }
        }
    }
}

// out[t] = bf16(sum over the token's top_k pairs p, in pair order, of w[p] * y[p]) (ACCUMULATE: added to
// what `out` holds).  A pair counts if inv[p] is a row of the schedule that really holds p in a block with
// an expert; otherwise the schedule dropped it, nobody wrote y[p], and it contributes nothing.  A pair id
// that the schedule lists more than once contributes once (if its rows lie in blocks of different experts,
// which of them is unspecified).
//
// One wave per (token, run of `chunks` pieces of 512 columns): lanes 0 .. top_k - 1 resolve the token's pairs
// once (inv, sorted_ids, expert_ids, routing weight), the result is broadcast, and then every lane streams its
// 8 columns of the top_k rows of y (contiguous: y is indexed by pair id), G loads in flight at a time.
template <bool ACCUMULATE, int G>
__global__ __launch_bounds__(256) void finalize_kernel(const char *y, const int32_t *inv, const int32_t *sorted_ids,
                                                       const int32_t *ntpp, int sorted_num, const float *topk_w,
                                                       int top_k, int M, int K, char *out,
                                                       const int32_t *expert_ids, int num_experts, int chunks,
                                                       int groups_per_token) {
    const int lane = threadIdx.x & 63;
    const int n_rows = min(ntpp[0], sorted_num);
    const int64_t n_items = (int64_t)M * groups_per_token;
    const int64_t wave_stride = (int64_t)gridDim.x * (blockDim.x >> 6);
    for (int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6); item < n_items; item += wave_stride) {
        const int t = (int)(item / groups_per_token), grp = (int)(item - (int64_t)t * groups_per_token);
        const int col_lo = grp * chunks * 512;
        for (int r0 = 0; r0 < top_k; r0 += 64) {
            // lane r resolves pair r0 + r: its weight, or 0 with `ok` unset
            float w_mine = 0.f;
            bool ok = false;
            if (r0 + lane < top_k) {
                const int p = t * top_k + r0 + lane;
                const int row = inv[p];
                ok = row >= 0 && row < n_rows;
                if (ok) ok = sorted_ids[row] == p;
                if (ok) {
                    const int e = expert_ids[row >> 7];
                    ok = e >= 0 && e < num_experts;
                }
                if (ok) w_mine = topk_w[p];
            }
            const uint64_t ok_mask = __ballot(ok);
            const int n_here = min(64, top_k - r0);
            for (int ch = 0; ch < chunks; ++ch) {
                const int col = col_lo + ch * 512 + lane * 8;
                if (col_lo + ch * 512 >= K) break;
                const bool in_range = col < K;
                float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                if (r0 > 0 || ACCUMULATE) {
                    if (in_range) {
                        const uint4 prev = *reinterpret_cast<const uint4 *>(out + ((int64_t)t * K + col) * 2);
                        const uint32_t u[4] = {prev.x, prev.y, prev.z, prev.w};
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            v[2 * j] = bf16_bits_to_f32(u[j] & 0xffffu);
                            v[2 * j + 1] = bf16_bits_to_f32(u[j] >> 16);
                        }
                    }
                }
                for (int g0 = 0; g0 < n_here; g0 += G) {
                    uint4 q[G];
                    float w[G];
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const int r = g0 + g;  // wave-uniform
                        const bool live = r < n_here && ((ok_mask >> r) & 1);
                        w[g] = __shfl(w_mine, r < 64 ? r : 0, 64);
                        q[g] = make_uint4(0, 0, 0, 0);
                        if (live && in_range) q[g] = load_once(y + ((int64_t)(t * top_k + r0 + r) * K + col) * 2);
                        if (!live) w[g] = 0.f;
                    }
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const uint32_t u[4] = {q[g].x, q[g].y, q[g].z, q[g].w};
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            v[2 * j] += w[g] * bf16_bits_to_f32(u[j] & 0xffffu);
                            v[2 * j + 1] += w[g] * bf16_bits_to_f32(u[j] >> 16);
                        }
                    }
                }
                if (in_range) {
                    uint32_t o[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) o[j] = pack2_bf16(v[2 * j], v[2 * j + 1]);
                    store_once(out + ((int64_t)t * K + col) * 2, make_uint4(o[0], o[1], o[2], o[3]));
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------ host

struct WorkspaceLayout {
    size_t n_tiles_off, tiles_off, work_up_off, work_down_off, inv_off, y_off, act_off, act_scales_off, xs_tiled_off, total;
};

// Workspace of an mxfp8 call.
static WorkspaceLayout workspace_layout(int M, int K, int N, int sorted_num, int top_k) {
    WorkspaceLayout l{};
    const size_t H = (size_t)N / 2;
    const size_t rows = align_up((size_t)sorted_num, kBlockRows);
    const size_t blocks = rows / kBlockRows;
    size_t off = 0;
    l.n_tiles_off = off;
    off += 256;
    l.tiles_off = off;
    off = align_up(off + blocks * sizeof(int2), 256);
    l.work_up_off = off;
    off = align_up(off + align_up(blocks * (H / 128), 8) * sizeof(int4), 256);
    l.work_down_off = off;
    const size_t n_wt_down = ((size_t)K + kWRows - 1) / kWRows;
    off = align_up(off + align_up(blocks * n_wt_down, 8) * sizeof(int4), 256);
    l.inv_off = off;
    const size_t pairs = (size_t)M * (size_t)std::max(top_k, 1);
    off = align_up(off + pairs * sizeof(int32_t), 256);
    l.y_off = off;  // one row per pair id
    off = align_up(off + pairs * K * 2, 256);
    l.act_off = off;
    off = align_up(off + rows * H, 256);
    l.act_scales_off = off;
    off = align_up(off + rows * (H / 32), 256);
    l.xs_tiled_off = off;
    off = align_up(off + rows * ((size_t)K / 32), 256);
    l.total = off;
    return l;
}

static int grid_for(int n_tiles) { return (n_tiles + 7) / 8 * 8; }

int resident_grid() {
    static thread_local int cached_dev = -1, cached = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev != cached_dev) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8) cus = 256;
        cached = cus / 8 * 8;
        cached_dev = dev;
    }
    return cached;
}

// Which phases of the pipeline the fused entry points enqueue (all by default); see
// pmoe_set_phase_mask in the header.
static thread_local int g_phase_mask = PMOE_PHASE_ALL;
int phase_mask() { return g_phase_mask; }
// Weight tiles a workgroup of the mxfp8 kernels takes in a row (0: chosen per launch); see
// pmoe_set_tiles_per_workgroup in the header.
static thread_local int g_tiles_per_wg = 0;

// A workgroup of the mxfp8 kernels can keep its token rows and take several weight tiles in a row: it
// saves the set-up of all but the first and starts each tile's copies under the epilogue of the one
// before, but the coarser work balances worse over the CUs.  Measured on the DeepSeek-V3-like prefill
// and decode shapes: two tiles gain 3 % on the down kernel (16 slabs per tile), nothing on the up kernel
// (56 slabs per tile), more than two lose on both.  So: two for the down kernel when that still leaves
// 8 rounds of workgroups per CU, one otherwise.
static int tiles_per_workgroup(bool down, int n_blocks, int n_wt) {
    if (g_tiles_per_wg > 0) return std::min(g_tiles_per_wg, n_wt);
    return (down && (int64_t)n_blocks * n_wt >= (int64_t)resident_grid() * 16) ? 2 : 1;
}

void launch_finalize(const MoeArgs &a, void *out, int split, int n_wt_down, hipStream_t s) {
    (void)n_wt_down;
    // a wave per (token, group of 512-column pieces); enough waves to fill the chip even for a few tokens
    const int pieces = (a.K + 511) / 512;
    int groups = std::min<int64_t>(pieces, std::max<int64_t>(1, 8192 / std::max(a.M, 1)));
    const int chunks = (pieces + groups - 1) / groups;
    groups = (pieces + chunks - 1) / chunks;
    const int64_t waves = (int64_t)a.M * groups;
    const int blocks = (int)std::min<int64_t>((waves + 3) / 4, 16384);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, s, a.y, a.inv, a.sorted_ids, a.ntpp, a.sorted_num,
                           a.topk_w, a.top_k, a.M, a.K, static_cast<char *>(out), a.expert_ids, a.E, chunks, groups);
    };
    if (split) {
        if (a.top_k <= 2) launch(finalize_kernel<false, 2>);
        else if (a.top_k <= 4) launch(finalize_kernel<false, 4>);
        else launch(finalize_kernel<false, 8>);
    } else {
        if (a.top_k <= 2) launch(finalize_kernel<true, 2>);
        else if (a.top_k <= 4) launch(finalize_kernel<true, 4>);
        else launch(finalize_kernel<true, 8>);
    }
}

struct SchedBuffers {
    int2 *tiles;
    int *n_tiles;
    int4 *work_up;
    int4 *work_down;
};

static int launch_mxfp8_pipeline(MoeArgs a, const SchedBuffers &sb, void *out, int split, hipStream_t s) {
    constexpr int DT = DT_FP8;
    const int mask = g_phase_mask;
    a.n_blocks = (a.sorted_num + kBlockRows - 1) / kBlockRows;
    a.n_wtiles = a.H / 128;
    const int n_wt_down = (a.K + kWRows - 1) / kWRows;
    const int per_up = tiles_per_workgroup(false, a.n_blocks, a.n_wtiles);
    const int per_down = tiles_per_workgroup(true, a.n_blocks, n_wt_down);
    const int grid_up = grid_for(a.n_blocks * ((a.n_wtiles + per_up - 1) / per_up));
    const int grid_down = grid_for(a.n_blocks * ((n_wt_down + per_down - 1) / per_down));
    {
        // the work lists are needed by the two kernels even when the rest of the prologue is masked off
        const int do_invert = (mask & PMOE_PHASE_PROLOGUE) ? 1 : 0;
        const int blocks = do_invert ? std::max(1, std::min((a.sorted_num + 255) / 256, 1024)) : 1;
        hipLaunchKernelGGL(moe_prologue_kernel, dim3(blocks), dim3(256), 0, s, a.expert_ids, a.ntpp, a.n_blocks,
                           sb.tiles, sb.n_tiles, sb.work_up, a.n_wtiles, per_up, grid_up,
                           sb.work_down, n_wt_down, per_down, grid_down, a.E,
                           a.sorted_ids, a.sorted_num, a.inv, a.M * a.top_k, do_invert, a.x_scales, a.xs_tiled,
                           a.K >> 7, a.top_k, a.M);
    }
    if (a.n_blocks > 0) {
        a.work = sb.work_up;
        if (mask & PMOE_PHASE_UP) hipLaunchKernelGGL((moe_up_kernel<DT>), dim3(grid_up), dim3(512), 0, s, a);
        MoeArgs d = a;
        d.n_wtiles = n_wt_down;
        d.work = sb.work_down;
        if (mask & PMOE_PHASE_DOWN) hipLaunchKernelGGL((moe_down_kernel<DT>), dim3(grid_down), dim3(512), 0, s, d);
    }
    if (mask & PMOE_PHASE_FINALIZE) launch_finalize(a, out, split, n_wt_down, s);
    return check_launch("fused_moe_mxfp8 launch");
}

}  // namespace pmoe

using namespace pmoe;

extern "C" void pmoe_set_phase_mask(int mask) { g_phase_mask = mask; }
extern "C" void pmoe_set_tiles_per_workgroup(int n) { g_tiles_per_wg = n < 0 ? 0 : (n > 16 ? 16 : n); }

extern "C" size_t pmoe_fused_moe_bf16_workspace_bytes(int M, int K, int N, int num_experts,
                                                      int sorted_num, int top_k, int split) {
    (void)num_experts;
    (void)split;
    if (M <= 0 || K <= 0 || N <= 0 || sorted_num < 0) return 0;
    MoeArgs a{};
    a.M = M; a.K = K; a.N = N; a.H = N / 2; a.sorted_num = sorted_num; a.top_k = top_k;
    return bf16_workspace(a, nullptr);
}

extern "C" size_t pmoe_fused_moe_mxfp8_workspace_bytes(int M, int K, int N, int num_experts,
                                                       int sorted_num, int top_k, int split) {
    (void)num_experts;
    (void)split;
    if (M <= 0 || K <= 0 || N <= 0 || sorted_num < 0) return 0;
    return workspace_layout(M, K, N, sorted_num, top_k).total;
}

static int check_tuning(const char *op, int block_m, int block_n, int warp_n, int stages,
                        int max_stages) {
    PMOE_REQUIRE((block_n == 64 && warp_n == 4) || (block_n == 32 && warp_n == 8),
                 "%s: (block_n, warp_n) must be (64, 4) or (32, 8), got (%d, %d)", op, block_n, warp_n);
    PMOE_REQUIRE(stages > 0 && stages <= max_stages, "%s supports stages in 1..%d, got %d", op, max_stages, stages);
    PMOE_REQUIRE(block_m == 128, "%s requires block_m=128, got %d", op, block_m);
    return PMOE_OK;
}

extern "C" int pmoe_fused_moe_bf16(const void *x, const void *w, const void *w2, void *out,
                                   const int32_t *sorted_token_ids, const int32_t *expert_idxs,
                                   const int32_t *num_tokens_post_padded, const float *topk_weights,
                                   int top_k, int M, int K, int N, int num_experts, int sorted_num,
                                   int block_m, int block_n, int warp_n, int stages, int bpc, int cpc,
                                   int split, void *workspace, size_t workspace_bytes, void *stream) {
    PMOE_REQUIRE(M > 0, "fused_moe_bf16: x has no rows");
    PMOE_REQUIRE(K > 0 && (K & 127) == 0, "K dimension must be a multiple of 128");
    PMOE_REQUIRE(N > 0 && (N & 255) == 0, "fused_moe_bf16: N must be a multiple of 256, got %d", N);
    if (int rc = check_tuning("fused_moe_bf16", block_m, block_n, warp_n, stages, 5)) return rc;
    PMOE_REQUIRE(bpc == 1 && cpc == 1, "bpc=cpc=1 is the only supported configuration");
    PMOE_REQUIRE(!split || stages <= 4, "split=True requires stages<=4, got stages=%d", stages);
    PMOE_REQUIRE(top_k > 0 && num_experts > 0 && sorted_num >= 0, "fused_moe_bf16: bad top_k / num_experts / sorted_num");
    PMOE_REQUIRE(num_experts <= 1024, "fused_moe_bf16: at most 1024 experts, got %d", num_experts);
    // the gather addresses a token row by a 32-bit byte offset from x
    PMOE_REQUIRE((uint64_t)M * (uint64_t)K * 2u < (1ull << 32), "fused_moe_bf16: x must be smaller than 4 GiB, got %d x %d", M, K);
    PMOE_REQUIRE(x && w && w2 && out && sorted_token_ids && expert_idxs && num_tokens_post_padded && topk_weights,
                 "fused_moe_bf16: null pointer");
    MoeArgs a{};
    a.x = static_cast<const char *>(x);
    a.w1 = static_cast<const char *>(w);
    a.w2 = static_cast<const char *>(w2);
    a.sorted_ids = sorted_token_ids;
    a.expert_ids = expert_idxs;
    a.ntpp = num_tokens_post_padded;
    a.topk_w = topk_weights;
    a.top_k = top_k; a.M = M; a.K = K; a.N = N; a.H = N / 2; a.E = num_experts; a.sorted_num = sorted_num;
    const size_t need = bf16_workspace(a, nullptr);
    PMOE_REQUIRE(workspace && workspace_bytes >= need, "fused_moe_bf16: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    PMOE_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "fused_moe_bf16: workspace must be 256-byte aligned");
    bf16_workspace(a, static_cast<char *>(workspace));
    return launch_bf16_pipeline(a, out, split, static_cast<hipStream_t>(stream));
}

extern "C" int pmoe_fused_moe_mxfp8(const void *x, const void *x_scales, const void *w,
                                    const void *w_scales, const void *w2, const void *w2_scales,
                                    void *out, const int32_t *sorted_token_ids,
                                    const int32_t *expert_idxs, const int32_t *num_tokens_post_padded,
                                    const float *topk_weights, int top_k, int M, int K, int N,
                                    int num_experts, int sorted_num, int block_m, int block_n,
                                    int warp_n, int stages, int bpc, int split, void *workspace,
                                    size_t workspace_bytes, void *stream) {
    PMOE_REQUIRE(M > 0, "fused_moe_mxfp8: x has no rows");
    PMOE_REQUIRE(K > 0 && (K & 255) == 0, "K dimension must be a multiple of 256 on the mxfp8 path");
    PMOE_REQUIRE(N > 0 && (N & 255) == 0, "N dimension must be a multiple of 256 on the mxfp8 path");
    if (int rc = check_tuning("fused_moe_mxfp8", block_m, block_n, warp_n, stages, 4)) return rc;
    PMOE_REQUIRE(bpc == 1, "mxfp8 supports bpc=1 only");
    PMOE_REQUIRE(top_k > 0 && num_experts > 0 && sorted_num >= 0, "fused_moe_mxfp8: bad top_k / num_experts / sorted_num");
    PMOE_REQUIRE(num_experts <= 1024, "fused_moe_mxfp8: at most 1024 experts, got %d", num_experts);
    // the gather addresses a token row by a 32-bit byte offset from x
    PMOE_REQUIRE((uint64_t)M * (uint64_t)K < (1ull << 32), "fused_moe_mxfp8: x must be smaller than 4 GiB, got %d x %d", M, K);
    PMOE_REQUIRE(x && x_scales && w && w_scales && w2 && w2_scales && out && sorted_token_ids && expert_idxs &&
                     num_tokens_post_padded && topk_weights,
                 "fused_moe_mxfp8: null pointer");
    const WorkspaceLayout l = workspace_layout(M, K, N, sorted_num, top_k);
    PMOE_REQUIRE(workspace && workspace_bytes >= l.total, "fused_moe_mxfp8: workspace of %zu bytes needed, got %zu", l.total, workspace_bytes);
    PMOE_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "fused_moe_mxfp8: workspace must be 256-byte aligned");
    MoeArgs a{};
    a.x = static_cast<const char *>(x);
    a.x_scales = static_cast<const uint8_t *>(x_scales);
    a.w1 = static_cast<const char *>(w);
    a.w1_scales = static_cast<const uint8_t *>(w_scales);
    a.w2 = static_cast<const char *>(w2);
    a.w2_scales = static_cast<const uint8_t *>(w2_scales);
    a.sorted_ids = sorted_token_ids;
    a.expert_ids = expert_idxs;
    a.ntpp = num_tokens_post_padded;
    a.topk_w = topk_weights;
    char *ws = static_cast<char *>(workspace);
    a.y = ws + l.y_off;
    a.inv = reinterpret_cast<int32_t *>(ws + l.inv_off);
    a.act = ws + l.act_off;
    a.act_scales = reinterpret_cast<uint32_t *>(ws + l.act_scales_off);
    a.xs_tiled = reinterpret_cast<uint32_t *>(ws + l.xs_tiled_off);
    a.top_k = top_k; a.M = M; a.K = K; a.N = N; a.H = N / 2; a.E = num_experts; a.sorted_num = sorted_num;
    SchedBuffers sb;
    sb.n_tiles = reinterpret_cast<int *>(ws + l.n_tiles_off);
    sb.tiles = reinterpret_cast<int2 *>(ws + l.tiles_off);
    sb.work_up = reinterpret_cast<int4 *>(ws + l.work_up_off);
    sb.work_down = reinterpret_cast<int4 *>(ws + l.work_down_off);
    return launch_mxfp8_pipeline(a, sb, out, split, static_cast<hipStream_t>(stream));
}
