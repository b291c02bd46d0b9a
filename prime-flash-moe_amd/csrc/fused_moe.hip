// Fused MoE forward for gfx950: gate/up grouped GEMM + SwiGLU (+ on-chip MX requantisation),
// down GEMM with the routing-weight reduction, for bf16 and mxfp8 operands.
//
// Replaces the launchers and kernels of the reference's
// prime_moe/csrc/kernels/fused_moe_bf16_kernel.cu:21-733 and fused_moe_mxfp8_kernel.cu:56-866.
//
// Pipeline of one call (all on the caller's stream):
//   prologue (pair blocks into row tiles, build the two work lists, invert the sorted order:
//             pair id -> sorted row; mxfp8: re-tile the scales of the gathered x rows)
//   -> up kernel (gate/up GEMM + SwiGLU, activation tile -> workspace)
//   -> down kernel (y[sorted row, :K] = act . W2[e]^T, bf16, -> workspace)
//   -> finalize: out[t] = bf16(sum over the token's pairs p of w[p] * y[row(p)]), fp32 sum in pair
//      order; split == 0: added to `out` (the reference's accumulate-into-out contract of its
//      single-kernel path), split != 0: `out` overwritten.
// Both values of `split` run the same kernels: on this hardware the two-kernel pipeline is the faster
// one at every shape, so `split` only selects what finalize does with `out`.  The jobs of a bf16 kernel
// that start last share their tile's contraction among several workgroups (see TailSplit).  No value
// is accumulated with atomics and every sum has a fixed order: the result is a pure function of the
// inputs.
#include <algorithm>

#include "moe_ring.h"
#include "moe_ring128.h"
#include "moe_tile.h"
#include "pmoe_common.h"

namespace pmoe {

struct MoeArgs {
    const char *x;
    const uint8_t *x_scales;
    const char *w1;
    const uint8_t *w1_scales;
    const char *w2;
    const uint8_t *w2_scales;
    const int32_t *sorted_ids;
    const int32_t *expert_ids;
    const int32_t *ntpp;
    const float *topk_w;
    char *act;            // (sorted_num, H) activation workspace, bf16 or e4m3
    // e8m0 scales of the token-side operands of the two mxfp8 GEMMs, as the loaders want them: one
    // dword (4 scales = 128 contraction elements) per row, [sorted block][128-wide K tile][row in block],
    // so that the 64 lanes of a copy instruction read 256 contiguous bytes.
    uint32_t *xs_tiled;   // scales of the gathered x rows (written by the prologue from x_scales)
    uint32_t *act_scales; // scales of the activation (written by the up kernel's epilogue)
    char *y;              // (sorted_num, K) bf16: down-projected rows, before the routing weights
    int32_t *inv;         // (M * top_k): sorted row of each pair id (validated against sorted_ids when read)
    const int4 *work;     // this kernel's work list, one entry per workgroup (see emit_work)
    char *y_tail;         // partial tiles of down jobs whose contraction is split (see plan_tail_split)
    float *up_partials;   // fp32 partial accumulators of up jobs whose contraction is split
    int *up_counters;     // per such job: parts that have stored theirs (zeroed by the prologue)
    int4 *join_tab;       // per such job, when a separate kernel joins the parts: its tile (see moe_up_join_kernel)
    int up_part_stride;   // partial accumulators reserved per job (the largest number of parts)
    int deep_join;        // the parts of split up jobs only store; moe_up_join_kernel adds them and finishes the tiles
    int top_k, M, K, N, H, E, sorted_num;
    int n_blocks;  // sorted_num / 128 (rounded up)
    int n_wtiles;  // weight tiles along the free dimension: H/128 (up) or ceil(K/256) (down)
};

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

// 16 bytes that this kernel writes or reads once (activation and y tiles, out): non-temporal, so that they
// do not displace what the L2s could serve again (finalize: C3 -14 us, C4 -12 us; the two GEMM kernels gain
// a few microseconds).
__device__ __forceinline__ uint4 load_once(const void *p) {
    const i32x4 v = __builtin_nontemporal_load(reinterpret_cast<const i32x4 *>(p));
    return make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
}
__device__ __forceinline__ void store_once(void *p, uint4 q) {
    i32x4 v;
    v[0] = (int)q.x; v[1] = (int)q.y; v[2] = (int)q.z; v[3] = (int)q.w;
    __builtin_nontemporal_store(v, reinterpret_cast<i32x4 *>(p));
}
constexpr int kActPitchBf16 = 272;  // 128 bf16 + 16 B pad: 16-byte aligned rows, 2-way conflicts at most
constexpr int kActPitchFp8 = 144;   // 128 e4m3 + 16 B pad

// What one workgroup does: `n_sub` consecutive weight tiles from `wt` on for the row tile of `nb` blocks
// starting at block `first`, expert `e`.  A job of a bf16 kernel can be one of `parts` workgroups that
// split the contraction of one tile (tail job number `slot`): this one sums slabs
// [part n / parts, (part + 1) n / parts) of the n.  Down kernel: part 0 writes y, part p > 0 tile
// slot (parts - 1) + p - 1 of y_tail, and the finalize kernel adds them up.  Up kernel: every part
// stores its fp32 accumulators, and the one that finishes last adds them in part order and goes on to
// the epilogue (see join_parts).
struct Job {
    int first, nb, wt, e, n_sub;
    int part, parts, slot;
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
    j.part = w.z & 0xf;
    j.parts = (w.z >> 4) & 0xf;
    j.slot = w.z >> 8;
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
constexpr int kYPitch = 528;  // 256 bf16 + 16 B pad
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
// K; the last tile of a K that is not a multiple of 256 has 128 columns) or a tile of y_tail (256 x 256,
// pitch 512 bytes).
struct YDst {
    char *base;     // first column of the group's tile: in row 0 of y (by_pair) or in the tile's first row
    int64_t pitch;  // bytes per row
    int cols;       // columns to write
    bool by_pair;   // row r of the tile goes to y row pair[r] (else to row r of a y_tail tile)
};
__device__ __forceinline__ YDst y_destination(const MoeArgs &a, const Job &j, int grp, int k0) {
    YDst d;
    d.by_pair = j.part == 0;
    if (j.part == 0) {
        d.base = a.y + (int64_t)k0 * 2;
        d.pitch = (int64_t)a.K * 2;
        d.cols = min(kWRows, a.K - k0);
    } else {
        d.base = a.y_tail + ((int64_t)(j.slot * (j.parts - 1) + j.part - 1) * 2 + grp) * (kBlockRows * kWRows * 2);
        d.pitch = kWRows * 2;
        d.cols = kWRows;
    }
    return d;
}
// Tiles with a single live fragment skip the detour through LDS: every lane stores its 8-byte runs
// straight to the destination (32 rows x 16 KB per tile at most; a barrier and an LDS round trip cost more).
// `pair_r` = pair id of this lane's row (lane % 32) of the group, < 0 if the row holds none.
__device__ __forceinline__ void store_y_direct(const YDst &d, const f32x16 (&acc)[2][4], int n_rows, int w4, int lane,
                                               int pair_r) {
    const int r = lane & 31, half = lane >> 5;
    if (r >= n_rows || (d.by_pair && pair_r < 0)) return;
    char *dst = d.base + (d.by_pair ? pair_r : r) * d.pitch;
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
            const int dst_row = d.by_pair ? pair[row] : row;
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
            if constexpr (DT == DT_BF16) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int hl = 32 * w4 + 8 * g + 4 * half;  // tile-local activation column
                    uint2 pk;
                    pk.x = pack2_bf16(v[4 * g], v[4 * g + 1]);
                    pk.y = pack2_bf16(v[4 * g + 2], v[4 * g + 3]);
                    *reinterpret_cast<uint2 *>(tile + row * kActPitchBf16 + hl * 2) = pk;
                }
            } else {
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
}

// Coalesced copy of the first 32*ntf rows of a group's activation tile (pitch kActPitch*) to the
// workspace rows row0.., columns [h0, h0+128); gt = thread index inside the group (0..255).
template <int DT>
__device__ __forceinline__ void store_act_tile(const MoeArgs &a, const char *tile, const uint32_t *sc_tile,
                                               int64_t row0, int h0, int ntf, int gt) {
    const int H = a.H;
    if constexpr (DT == DT_BF16) {
        const int c = gt & 15;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = (gt >> 4) + 16 * i;
            if (row < 32 * ntf) {
                uint4 v = *reinterpret_cast<const uint4 *>(tile + row * kActPitchBf16 + c * 16);
                store_once(a.act + ((row0 + row) * H + h0) * 2 + c * 16, v);
            }
        }
    } else {
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
}

// Contraction split of an up tile: every part stores its accumulators (32 float4 per thread, thread
// index fastest; only the NTF live fragments of the groups that have rows), makes them visible to the
// device and counts itself in; the part that counts last adds all parts in part order (its own too,
// from memory: the same bits whichever part is last) and returns true.  Nobody waits for anybody.
// `lds_flag` is a word of LDS no copy is in flight to.
constexpr int kUpTailJobs = 64;
// Few jobs on many CUs (a.deep_join): the contraction is split further (up to kDeepParts parts) and nobody
// joins here; every part stores and leaves (returns false), and moe_up_join_kernel, with one workgroup per
// 32 x 128 piece of every tile, adds the parts and runs the epilogue: the join then costs a few microseconds
// whatever the number of parts, where the last part alone would read parts x 256 KB.
constexpr int kDeepParts = 8;  // (6 to 8 measure alike on the README shape, 12 and 16 slower: shorter walks, more to join)
template <int NTF>
__device__ __forceinline__ bool join_parts(const MoeArgs &a, const Job &j, f32x16 (&acc)[2][4], bool active,
                                           int *lds_flag) {
    const int tid = threadIdx.x;
    float4 *mine = reinterpret_cast<float4 *>(a.up_partials) + ((int64_t)(j.slot * a.up_part_stride + j.part) * 32) * 512;
    if (active) {
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int t = 0; t < NTF; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    mine[((f * 4 + t) * 4 + q) * 512 + tid] =
                        make_float4(acc[f][t][4 * q], acc[f][t][4 * q + 1], acc[f][t][4 * q + 2], acc[f][t][4 * q + 3]);
    }
    if (a.deep_join) return false;  // (the kernel boundary orders the stores before the join kernel's loads)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");  // the stores above are visible device-wide before the count below
    __syncthreads();
    if (tid == 0) *lds_flag = atomicAdd(&a.up_counters[j.slot], 1);
    __syncthreads();
    const bool last = *lds_flag == j.parts - 1;
    if (!last) return false;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // the other parts' stores are visible to the loads below
    if (active) {
        zero_acc(acc);
        for (int p = 0; p < j.parts; ++p) {
            const float4 *src = reinterpret_cast<const float4 *>(a.up_partials) + ((int64_t)(j.slot * a.up_part_stride + p) * 32) * 512;
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int t = 0; t < NTF; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float4 v = src[((f * 4 + t) * 4 + q) * 512 + tid];
                        acc[f][t][4 * q] += v.x;
                        acc[f][t][4 * q + 1] += v.y;
                        acc[f][t][4 * q + 2] += v.z;
                        acc[f][t][4 * q + 3] += v.w;
                    }
        }
    }
    return true;
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
    constexpr int ES = DT == DT_BF16 ? 2 : 1;
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
    // this workgroup's share of the contraction (all of it unless the tile is split, which only
    // happens to bf16 tiles: the scales of a slab are addressed from the start of the row)
    const int n_slabs_all = (K * ES) / RB;
    const int slab0 = job.part * n_slabs_all / job.parts;
    const int n_slabs = (job.part + 1) * n_slabs_all / job.parts - slab0;
    ring::Loader<RB> ld;
    ld.tok_base = a.x + slab0 * RB;
    ld.w_base[0] = a.w1 + ((int64_t)e * N + h0) * K * ES + slab0 * RB;
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
    constexpr int kPitch = DT == DT_BF16 ? kActPitchBf16 : kActPitchFp8;
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
        if constexpr (DT == DT_BF16) {
            if (job.parts > 1 && !join_parts<NTF>(a, job, acc, active, reinterpret_cast<int *>(lds + 128 * 1024))) return;
        }
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

// LDS plan of the split kernels.  bf16: the 160 KB ring of the wide engine is all the LDS there is;
// the row table sits in the tail of its last unit, which the ring first fills after the barrier
// that opens slab 0, when the loaders hold everything they need of it in registers (the skinny
// ring is shorter and never reaches it).  mxfp8: ring, row table, activation scales side by side.
template <int DT>
struct SplitLds {
    static constexpr int kRowInfoBytes = 2304;  // >= sizeof(RowInfo<2>)
    // bf16: the pair ids of the tile's rows, fetched again for the down kernel's epilogue (the ring has run
    // over the row table by then); behind the two output tiles of the epilogue
    static constexpr int kPairOff = 140 * 1024;
    static constexpr int kRing = DT == DT_BF16 ? ring128::kRingBytes : ring::ring_bytes<DT>();
    static constexpr int kRowInfoOff = DT == DT_BF16 ? kRing - kRowInfoBytes : kRing;
    static constexpr int kActScaleOff = kRowInfoOff + kRowInfoBytes;  // mxfp8 only
    static constexpr int kTotal = DT == DT_BF16 ? kRing : kActScaleOff + kBlockRows * 2 * 4;
    static_assert(sizeof(RowInfo<2>) <= kRowInfoBytes, "row table does not fit its slot");
    // the epilogues reuse the head of the ring: two y tiles (down kernel) or two activation tiles (up kernel)
    static_assert(2 * kBlockRows * kYPitch <= (DT == DT_BF16 ? kPairOff : kRing), "y tiles of the epilogue overrun their LDS");
    static_assert(2 * kBlockRows * kActPitchBf16 <= kRing, "activation tiles of the epilogue overrun the ring");
    static_assert(DT != DT_BF16 || ring::ring_bytes<DT_BF16>() <= kRowInfoOff, "64-byte ring reaches the row table");
};

// First slab of a wide bf16 tile's walk over K: 8 phases, one 128-byte slab apart.
__device__ __forceinline__ int slab_rotation128(int n_slabs) { return (int)((blockIdx.x >> 3) & 7) % n_slabs; }

// Up kernel tile on the 128-byte ring (bf16, two blocks or one block with more than 32 live rows).
template <int NTF, bool SPLIT>
__device__ __forceinline__ void up_tile_wide_bf16(const MoeArgs &a, const Job &job, RowInfo<2> &ri, char *lds) {
    const int first = job.first, ht = job.wt, e = job.e;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int grp = wave >> 2, w4 = wave & 3, gt = tid & 255;
    const int K = a.K, H = a.H, N = a.N;
    const int h0 = ht * 128;
    const int ntf0 = __builtin_amdgcn_readfirstlane((ri.nvalid[0] + 31) >> 5);
    const int ntf1 = __builtin_amdgcn_readfirstlane((ri.nvalid[1] + 31) >> 5);
    const int my_ntf = grp ? ntf1 : ntf0;
    const bool active = my_ntf > 0;

    const uint32_t row_bytes = (uint32_t)K * 2u;
    // this workgroup's share of the contraction (all of it unless the tile is SPLIT)
    const int n_slabs_all = (int)(row_bytes / ring128::kRB);
    const int slab0 = SPLIT ? job.part * n_slabs_all / job.parts : 0;
    const int n_slabs = SPLIT ? (job.part + 1) * n_slabs_all / job.parts - slab0 : n_slabs_all;
    const char *w_gate = a.w1 + ((int64_t)e * N + h0) * K * 2 + slab0 * ring128::kRB;
    ring128::Loader ld;
    ld.setup(tid, a.x + slab0 * ring128::kRB, w_gate, w_gate + (int64_t)H * K * 2, row_bytes, ntf0, ntf1,
             [&](int row) { return (uint32_t)max(ri.tok[row], 0) * row_bytes; });  // dead rows read token 0

    const int wrow[2] = {32 * w4, 128 + 32 * w4};
    f32x16 acc[2][4];
    zero_acc(acc);
    const int start = slab_rotation128(n_slabs);
    const int tok_region = grp * ring128::kGroupRegion;
    if (active) ring128::main_loop<NTF, true, true>(acc, ld, lds, n_slabs, wrow, lane, tok_region, start);
    else ring128::main_loop<NTF, true, false>(acc, ld, lds, n_slabs, wrow, lane, tok_region, start);
    if constexpr (SPLIT) {
        if (!join_parts<NTF>(a, job, acc, active, reinterpret_cast<int *>(lds + 4 * ring128::kUnitBytes))) return;
    }

    char *tile = lds + grp * (kBlockRows * kActPitchBf16);
    if (active) swiglu_epilogue<DT_BF16, NTF>(acc, tile, nullptr, w4, lane);
    __syncthreads();
    if (active) store_act_tile<DT_BF16>(a, tile, nullptr, (int64_t)(first + grp) * kBlockRows, h0, my_ntf, gt);
}

template <int DT>
__global__ __launch_bounds__(512) void moe_up_kernel(MoeArgs a) {
    using L = SplitLds<DT>;
    __shared__ __attribute__((aligned(1024))) char lds[L::kTotal];
    RowInfo<2> &ri = *reinterpret_cast<RowInfo<2> *>(lds + L::kRowInfoOff);
    Job j;
    if (!resolve_job(a, j)) return;
    const int ntf = load_row_info<2>(a, j.first, j.nb, ri);
    if (ntf == 0) return;
    const bool skinny = ntf == 1 && ri.nvalid[1] == 0;
    if constexpr (DT == DT_BF16) {  // one weight tile per workgroup on this path (see launch_pipeline)
        j.n_sub = 1;
        if (skinny) {
            // (an expert's last few rows: whatever its other row tiles fetched of these weight rows has left the
            // caches by the time this tile runs, so its copies are non-temporal too; C2 -0.6 %, no loss elsewhere)
            j.w_once = true;
            up_tile_ring<DT, kSkinnyRB, 1>(a, j, ri, lds, nullptr);
        }
        else if (j.parts > 1) {  // one of the workgroups that share a tile of the kernel's tail
            if (ntf == 1) up_tile_wide_bf16<1, true>(a, j, ri, lds);
            else if (ntf == 2) up_tile_wide_bf16<2, true>(a, j, ri, lds);
            else up_tile_wide_bf16<4, true>(a, j, ri, lds);
        } else if (ntf == 1) up_tile_wide_bf16<1, false>(a, j, ri, lds);
        else if (ntf == 2) up_tile_wide_bf16<2, false>(a, j, ri, lds);
        else up_tile_wide_bf16<4, false>(a, j, ri, lds);
    } else {
        uint32_t *act_sc_lds = reinterpret_cast<uint32_t *>(lds + L::kActScaleOff);
        if (ntf == 1) up_tile_ring<DT, kSkinnyRB, 1>(a, j, ri, lds, act_sc_lds);
        else if (ntf == 2) up_tile_ring<DT, kPartRB, 2>(a, j, ri, lds, act_sc_lds);
        else up_tile_ring<DT, kPartRB, 4>(a, j, ri, lds, act_sc_lds);
    }
}

// Down kernel tile on the stage ring: y[rows, 256 cols of K] = act[rows, :H] . W2[e][cols, :H]^T, the
// whole reduction over H inside the workgroup unless the job is one part of a split tail tile; the
// routing weights are applied later, by finalize_kernel.
template <int DT, int RB, int NTF>
__device__ __forceinline__ void down_tile_ring(const MoeArgs &a, const Job &job, RowInfo<2> &ri, char *lds) {
    constexpr int ES = DT == DT_BF16 ? 2 : 1;
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
    // this workgroup's share of the contraction (all of it unless the tile is split, which only
    // happens to bf16 tiles: the scales of a slab are addressed from the start of the row)
    const int n_slabs_all = (H * ES) / RB;
    const int slab0 = job.part * n_slabs_all / job.parts;
    const int n_slabs = (job.part + 1) * n_slabs_all / job.parts - slab0;
    ring::Loader<RB> ld;
    ld.tok_base = a.act + row0 * H * ES + slab0 * RB;
    // weight rows (output columns) k0 .. k0 + 255 of the expert; the last tile of a K that is not a
    // multiple of 256 has 128 of them and reads the first half twice
    auto set_weights = [&](int k) {
        ld.w_base[0] = a.w2 + ((int64_t)e * K + k) * H * ES + slab0 * RB;
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
        const YDst dst = y_destination(a, job, grp, k0);
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

// Down kernel tile on the 128-byte unit ring (bf16).
template <int NTF>
__device__ __forceinline__ void down_tile_wide_bf16(const MoeArgs &a, const Job &job, RowInfo<2> &ri, char *lds) {
    const int first = job.first, kt = job.wt, e = job.e;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int grp = wave >> 2, w4 = wave & 3, gt = tid & 255;
    const int K = a.K, H = a.H;
    const int k0 = kt * kWRows;
    const int64_t row0 = (int64_t)first * kBlockRows;
    const int ntf0 = __builtin_amdgcn_readfirstlane((ri.nvalid[0] + 31) >> 5);
    const int ntf1 = __builtin_amdgcn_readfirstlane((ri.nvalid[1] + 31) >> 5);
    const int my_ntf = grp ? ntf1 : ntf0;
    const int my_rows = ri.nvalid[grp];  // read before the ring overwrites the row table
    const int my_pair = ri.pair[grp * kBlockRows + (lane & 31)];
    const bool active = my_ntf > 0;

    const uint32_t row_bytes = (uint32_t)H * 2u;
    // this workgroup's share of the contraction (all of it unless the tile is split)
    const int n_slabs_all = (int)(row_bytes / ring128::kRB);
    const int slab0 = job.part * n_slabs_all / job.parts;
    const int n_slabs = (job.part + 1) * n_slabs_all / job.parts - slab0;
    const char *w_lo = a.w2 + ((int64_t)e * K + k0) * H * 2 + slab0 * ring128::kRB;
    const char *w_hi = (k0 + 128 < K) ? w_lo + (int64_t)128 * H * 2 : w_lo;
    ring128::Loader ld;
    ld.setup(tid, a.act + row0 * H * 2 + slab0 * ring128::kRB, w_lo, w_hi, row_bytes, ntf0, ntf1,
             [&](int row) { return (uint32_t)row * row_bytes; });

    const int wrow[2] = {64 * w4, 64 * w4 + 32};
    f32x16 acc[2][4];
    zero_acc(acc);
    const int start = slab_rotation128(n_slabs);
    const int tok_region = grp * ring128::kGroupRegion;
    if (active) ring128::main_loop<NTF, true, true>(acc, ld, lds, n_slabs, wrow, lane, tok_region, start);
    else ring128::main_loop<NTF, true, false>(acc, ld, lds, n_slabs, wrow, lane, tok_region, start);
    const YDst dst = y_destination(a, job, grp, k0);
    if constexpr (NTF == 1) {
        if (active) store_y_direct(dst, acc, my_rows, w4, lane, my_pair);
    } else {
        char *tile = lds + grp * (kBlockRows * kYPitch);
        int *pair = reinterpret_cast<int *>(lds + SplitLds<DT_BF16>::kPairOff);
        if (tid < 2 * kBlockRows) {  // the same test as load_row_info's: a pair id whose token is out of range is none
            const int64_t srow = row0 + tid;
            const int p = (tid < job.nb * kBlockRows && srow < a.sorted_num) ? a.sorted_ids[srow] : -1;
            pair[tid] = (p >= 0 && p / a.top_k < a.M) ? p : -1;
        }
        if (active) y_epilogue<NTF>(acc, tile, w4, lane);
        __syncthreads();
        if (active) store_y_tile(dst, tile, my_rows, gt, pair + grp * kBlockRows);
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
    const bool skinny = ntf == 1 && ri.nvalid[1] == 0;
    if constexpr (DT == DT_BF16) {  // one weight tile per workgroup on this path (see launch_pipeline)
        j.n_sub = 1;
        if (skinny) {
            j.w_once = true;  // (see moe_up_kernel)
            down_tile_ring<DT, kSkinnyRB, 1>(a, j, ri, lds);
        }
        else if (ntf == 1) down_tile_wide_bf16<1>(a, j, ri, lds);
        else if (ntf == 2) down_tile_wide_bf16<2>(a, j, ri, lds);
        else down_tile_wide_bf16<4>(a, j, ri, lds);
    } else {
        if (ntf == 1) down_tile_ring<DT, kSkinnyRB, 1>(a, j, ri, lds);
        else if (ntf == 2) down_tile_ring<DT, kPartRB, 2>(a, j, ri, lds);
        else down_tile_ring<DT, kPartRB, 4>(a, j, ri, lds);
    }
}

// Joins the parts of split up tiles when the up kernel left them in memory (a.deep_join).  One workgroup of
// 4 waves per (job, row block of the tile, 32-row fragment, quarter of the accumulator registers): thread
// (w4, lane) takes over registers 4q .. 4q + 3 of what thread (block, w4, lane) of an up workgroup holds for
// that fragment, gate and up sums, adds the parts in part order, applies SwiGLU and writes its 4 activation
// values.  Same sums in the same order as join_parts, so the same bits.  All loads of a thread (the row's
// sorted id, which only decides whether anything is written, and the 2 x parts partial sums) are in flight
// together: the kernel is one memory latency long.
__global__ __launch_bounds__(256) void moe_up_join_kernel(MoeArgs a) {
    const int slot = blockIdx.x >> 5, grp = (blockIdx.x >> 4) & 1, t = (blockIdx.x >> 2) & 3, q = blockIdx.x & 3;
    const int4 jt = a.join_tab[slot];
    const int parts = jt.z;
    if (parts < 2) return;
    const int first = jt.x & 0x0fffffff, nb = jt.x >> 28, ht = jt.y & 0xffff;
    if (grp >= nb) return;
    const int tid = threadIdx.x, lane = tid & 63, w4 = tid >> 6;
    const int r = lane & 31, half = lane >> 5;
    const int64_t srow0 = (int64_t)(first + grp) * kBlockRows + 32 * t;
    const int64_t s = srow0 + r;
    const int p_row = s < a.sorted_num ? a.sorted_ids[s] : -1;
    const int src_tid = grp * 256 + tid;
    const float4 *base = reinterpret_cast<const float4 *>(a.up_partials);
    float4 vg[kDeepParts], vu[kDeepParts];
#pragma unroll
    for (int p = 0; p < kDeepParts; ++p)
        if (p < parts) {
            const float4 *src = base + ((int64_t)(slot * a.up_part_stride + p) * 32) * 512;
            vg[p] = src[((0 * 4 + t) * 4 + q) * 512 + src_tid];
            vu[p] = src[((1 * 4 + t) * 4 + q) * 512 + src_tid];
        }
    // a fragment without a live row has nothing to write (every wave looks at the same 32 rows)
    if (__ballot(p_row >= 0 && p_row / a.top_k < a.M) == 0) return;
    float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < kDeepParts; ++p)
        if (p < parts) {
            g[0] += vg[p].x; g[1] += vg[p].y; g[2] += vg[p].z; g[3] += vg[p].w;
            u[0] += vu[p].x; u[1] += vu[p].y; u[2] += vu[p].z; u[3] += vu[p].w;
        }
    const int hl = 32 * w4 + 8 * q + 4 * half;  // tile-local activation column, as in swiglu_epilogue
    uint2 pk;
    pk.x = pack2_bf16(swiglu(g[0], u[0]), swiglu(g[1], u[1]));
    pk.y = pack2_bf16(swiglu(g[2], u[2]), swiglu(g[3], u[3]));
    *reinterpret_cast<uint2 *>(a.act + ((srow0 + r) * a.H + ht * 128 + hl) * 2) = pk;
}

// Walk order of the tiles of one kernel: [group of 8 weight tiles][row tile][weight tile in group].
// The ~32 workgroups that run side by side on an XCD are then 4 consecutive row tiles (mostly of one
// expert) x 8 weight tiles: every token slab they fetch is shared by 8 weight tiles and every weight
// slab by the row tiles of its expert, inside that XCD's L2.  (Walking expert by expert instead,
// so that all row tiles of an expert always meet, measured 5 % slower on the Mixtral-like shape:
// more workgroups then ask for the same lines at the same moment.)
// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin, so position `l` of the walk
// is given to workgroup id 8 * (l mod per_xcd) + l / per_xcd: one XCD then runs a contiguous range of
// the walk.  The entry carries everything the workgroup needs to start: x = first block | blocks << 28,
// y = first weight tile | expert << 16 | (weight tiles - 1) << 26 (experts < 1024, up to 16 weight
// tiles), z = part | parts << 4 | tail slot << 8 (see TailSplit), w = 1 if the row tile is the only one of
// its expert.
//
// Workgroups start in the order of their ids, so the last `per_xcd_tail` positions of every XCD's range
// are the jobs that would run while most CUs have nothing left to do.  The bf16 kernels split the
// contraction of each of them over `parts` workgroups: part 0 stays in place, the others go behind the
// list proper (from entry `extra_base` on).  Down kernel: they write partial tiles to y_tail, which the
// finalize kernel adds (tail_tab tells it which tiles have parts and where).  Up kernel: see join_parts.
constexpr int kTailSlots = 192;  // work list entries behind the list proper = partial tiles y_tail holds
struct TailSplit {
    int parts;         // 1: no split
    int per_xcd_tail;  // jobs split at the end of each XCD's range
    int extra_base;    // first work list entry of the parts > 0
    int *tail_tab;     // down kernel: per (block, weight tile) 0, or first y_tail tile << 8 | block inside its tile << 4 | parts
    int4 *join_tab;    // up kernel with a separate join: per tail job its tile (first block | blocks << 28, weight tile, parts)
};

// How the tail of `n_jobs` jobs on `n_cus` CUs is split: at most `max_jobs` of them, every part gets at
// least one slab, and the parts > 0 fit `extra_cap` (<= kTailSlots) entries behind the list.
__device__ __forceinline__ void plan_tail_split(TailSplit &ts, int n_jobs, int n_cus, int n_slabs, int max_jobs,
                                                int extra_cap, int max_parts = 4) {
    ts.parts = 1;
    ts.per_xcd_tail = 0;
    if (n_cus <= 0 || n_jobs <= 0) return;
    const int rounds = n_jobs / n_cus, rest = n_jobs % n_cus;
    if (rest == 0 || rounds >= 16) return;  // nothing left over, or too little to matter
    int parts = min(min(max_parts, n_slabs), n_cus / rest);
    const int per_xcd_tail = (rest + 7) >> 3;
    if (per_xcd_tail * 8 > max_jobs) return;
    while (parts > 1 && per_xcd_tail * 8 * (parts - 1) > extra_cap) --parts;
    if (parts < 2) return;
    ts.parts = parts;
    ts.per_xcd_tail = per_xcd_tail;
}

// Writes the work list entry of job `j` (of the (n_wt + per_job - 1) / per_job of the row tile; a workgroup
// takes `per_job` consecutive weight tiles).
__device__ __forceinline__ void emit_work(int4 *work, int n_wt, int per_job, int tile, int n_tiles, int first, int nb,
                                          int e, const TailSplit *ts, int j, int flags) {
    constexpr int GW = 8;
    const int n_jobs = (n_wt + per_job - 1) / per_job;
    const int per_xcd = (n_tiles * n_jobs + 7) >> 3;
    {
        const int wg = j / GW;
        const int gw = min(GW, n_jobs - wg * GW);
        const int l = wg * GW * n_tiles + tile * gw + (j - wg * GW);
        const int wt = j * per_job, cnt = min(per_job, n_wt - wt);
        const int x = first | (nb << 28), y = wt | (e << 16) | ((cnt - 1) << 26);
        const int pos = l % per_xcd, xcd = l / per_xcd;
        if (ts != nullptr && ts->parts > 1 && pos >= per_xcd - ts->per_xcd_tail) {
            const int slot = (pos - (per_xcd - ts->per_xcd_tail)) * 8 + xcd;  // number of the tail job
            const int z = (ts->parts << 4) | (slot << 8);
            const int extra = slot * (ts->parts - 1);
            work[8 * pos + xcd] = make_int4(x, y, z, flags);
            for (int p = 1; p < ts->parts; ++p) work[ts->extra_base + extra + p - 1] = make_int4(x, y, z | p, flags);
            if (ts->join_tab != nullptr) ts->join_tab[slot] = make_int4(x, wt, ts->parts, 0);
            if (ts->tail_tab != nullptr)
                for (int b = 0; b < nb; ++b) ts->tail_tab[(first + b) * n_wt + wt] = (extra << 8) | (b << 4) | ts->parts;
        } else {
            work[8 * pos + xcd] = make_int4(x, y, 1 << 4, flags);
        }
    }
}

// Prologue of every call.  Workgroup 0 builds the row tiles and work lists of the two-group kernels:
// consecutive blocks of one expert are paired, an expert's odd last block stays single (one pass of
// block-wide scans per 256 blocks, then one pass over the tiles that writes the two walk orders).
// All workgroups invert the sorted order: inv[pair id] = sorted row.  Entries of pairs that are not
// in the schedule keep whatever the buffer held; the reader validates an entry against sorted_ids.
__global__ __launch_bounds__(256) void moe_prologue_kernel(const int32_t *expert_ids, const int32_t *ntpp,
                                                           int n_blocks, int2 *tiles, int *n_tiles,
                                                           int4 *work_up, int n_wt_up, int per_job_up, int grid_up,
                                                           int4 *work_down, int n_wt_down, int per_job_down,
                                                           int grid_down, int split_cus, int up_slabs, int down_slabs,
                                                           int *tail_tab, int *up_counters, int down_tail_tiles,
                                                           int up_tail_jobs, int4 *join_tab, int up_max_parts,
                                                           int num_experts,
                                                           const int32_t *sorted_ids, int sorted_num, int32_t *inv,
                                                           int n_pairs, int do_invert, const uint8_t *x_scales,
                                                           uint32_t *xs_tiled, int nkt, int top_k, int M) {
    if (blockIdx.x == 0 && tiles != nullptr) {
        __shared__ int s_max[4], s_sum[4], s_carry[2];
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        for (int i = tid; i < grid_up; i += 256) work_up[i] = make_int4(-1, -1, 0, 0);
        for (int i = tid; i < grid_down; i += 256) work_down[i] = make_int4(-1, -1, 0, 0);
        if (tail_tab != nullptr)
            for (int i = tid; i < n_blocks * n_wt_down; i += 256) tail_tab[i] = 0;
        if (up_counters != nullptr && tid < kUpTailJobs) up_counters[tid] = 0;
        if (join_tab != nullptr && tid < kUpTailJobs) join_tab[tid] = make_int4(0, 0, 0, 0);
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
        // contraction splits of the two kernels' tails (bf16 only: tail_tab and up_counters are null else)
        TailSplit ts, ts_up;
        ts.extra_base = grid_down - kTailSlots;
        ts.tail_tab = tail_tab;
        ts.join_tab = nullptr;
        plan_tail_split(ts, tail_tab != nullptr ? nt * ((n_wt_down + per_job_down - 1) / per_job_down) : 0, split_cus,
                        down_slabs, down_tail_tiles, down_tail_tiles);
        ts_up.extra_base = grid_up - kTailSlots;
        ts_up.tail_tab = nullptr;
        ts_up.join_tab = join_tab;
        plan_tail_split(ts_up, up_counters != nullptr ? nt * ((n_wt_up + per_job_up - 1) / per_job_up) : 0, split_cus,
                        up_slabs, up_tail_jobs, kTailSlots, up_max_parts);
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
                for (int j = 0; j < jobs_up; ++j) emit_work(work_up, n_wt_up, per_job_up, t, nt, tl.x, tl.y, e, &ts_up, j, fl);
                for (int j = 0; j < jobs_down; ++j) emit_work(work_down, n_wt_down, per_job_down, t, nt, tl.x, tl.y, e, &ts, j, fl);
            }
        } else {  // few row tiles for 256 threads: an entry per thread and turn (README shape: whole op 60 -> 56 us)
            for (int i = tid; i < nt * per_tile; i += 256) {
                const int t = i / per_tile, j = i - t * per_tile;
                const int2 tl = tiles[t];
                const int e = expert_ids[tl.x];
                if (e < 0 || e >= num_experts) continue;
                const int fl = only_tile(t, e);
                if (j < jobs_up) emit_work(work_up, n_wt_up, per_job_up, t, nt, tl.x, tl.y, e, &ts_up, j, fl);
                else emit_work(work_down, n_wt_down, per_job_down, t, nt, tl.x, tl.y, e, &ts, j - jobs_up, fl);
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
        // mxfp8: the e8m0 scales of the gathered x rows, re-tiled for the up kernel's loader (see
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

// out[t, 8 columns] = bf16(sum over the token's top_k pairs p, in pair order, of w[p] * y[p])
// (y[p] = part 0 of the pair's down projection plus, for tiles the down kernel split, the partial rows in
// y_tail, found through the pair's sorted row) (ACCUMULATE: added to what `out` holds).  A pair counts if
// inv[p] is a row of the schedule that really holds p in a block with an expert; otherwise the schedule
// dropped it, nobody wrote y[p], and it contributes nothing.  A pair id that the schedule lists more than
// once contributes once.  One thread per (token, 8 columns).
template <bool ACCUMULATE, int G>
__global__ __launch_bounds__(256) void finalize_kernel(const char *y, const int32_t *inv, const int32_t *sorted_ids,
                                                       const int32_t *ntpp, int sorted_num, const float *topk_w,
                                                       int top_k, int M, int K, uint4 *out, const int *tail_tab,
                                                       const char *y_tail, int n_wt, const int32_t *expert_ids,
                                                       int num_experts) {
    // G pairs are resolved and fetched together: their loads are in flight at the same time
    const int k8 = K >> 3;
    const int64_t total = (int64_t)M * k8;
    const int n_rows = min(ntpp[0], sorted_num);
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int t = (int)(i / k8), c = (int)(i - (int64_t)t * k8);
        float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        auto add = [&](const uint4 q, float w) {
            const uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[2 * j] += w * bf16_bits_to_f32(u[j] & 0xffffu);
                v[2 * j + 1] += w * bf16_bits_to_f32(u[j] >> 16);
            }
        };
        for (int r0 = 0; r0 < top_k; r0 += G) {
            int row[G];
            float w[G];
            uint4 q[G];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int p = t * top_k + r0 + g;
                row[g] = r0 + g < top_k ? inv[p] : -1;
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int p = t * top_k + r0 + g;
                bool ok = row[g] >= 0 && row[g] < n_rows;
                if (ok) ok = sorted_ids[row[g]] == p;
                if (ok) {
                    const int e = expert_ids[row[g] >> 7];
                    ok = e >= 0 && e < num_experts;
                }
                if (!ok) row[g] = -1;
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int p = t * top_k + r0 + g;
                if (row[g] >= 0) {
                    w[g] = topk_w[p];
                    q[g] = load_once(y + ((int64_t)p * K + 8 * c) * 2);
                }
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (row[g] < 0) continue;
                add(q[g], w[g]);
                // a tile whose contraction was split: the other parts' partial rows, in part order
                const int tt = tail_tab != nullptr ? tail_tab[(row[g] >> 7) * n_wt + (c >> 5)] : 0;
                if (tt != 0) {
                    const int parts = tt & 15, rr = ((tt >> 4) & 15) * kBlockRows + (row[g] & 127), slot = tt >> 8;
                    for (int part = 1; part < parts; ++part)
                        add(*reinterpret_cast<const uint4 *>(y_tail + (((int64_t)(slot + part - 1) * 256 + rr) * 256 + 8 * (c & 31)) * 2), w[g]);
                }
            }
        }
        uint32_t o[4];
        if constexpr (ACCUMULATE) {
            const uint4 prev = out[i];
            o[0] = prev.x; o[1] = prev.y; o[2] = prev.z; o[3] = prev.w;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[2 * j] += bf16_bits_to_f32(o[j] & 0xffffu);
                v[2 * j + 1] += bf16_bits_to_f32(o[j] >> 16);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = pack2_bf16(v[2 * j], v[2 * j + 1]);
        store_once(out + i, make_uint4(o[0], o[1], o[2], o[3]));
    }
}

// ------------------------------------------------------------------------------------------ host

struct WorkspaceLayout {
    size_t n_tiles_off, up_counters_off, join_tab_off, tiles_off, work_up_off, work_down_off, tail_tab_off, y_tail_off,
        up_partials_off, inv_off, y_off, act_off,
        act_scales_off, xs_tiled_off, total;
    int down_tail_tiles, up_tail_jobs;  // partial tiles y_tail holds / jobs up_partials holds (0: no split tails)
    int up_part_stride;                 // partial accumulators per up job: 4, or kDeepParts with the separate join
    bool deep_join;
};

static WorkspaceLayout workspace_layout(int dt, int M, int K, int N, int sorted_num, int top_k) {
    WorkspaceLayout l{};
    const size_t H = (size_t)N / 2;
    const size_t rows = align_up((size_t)sorted_num, kBlockRows);
    const size_t blocks = rows / kBlockRows;
    size_t off = 0;
    l.n_tiles_off = off;
    off += 256;
    l.up_counters_off = off;
    off += kUpTailJobs * sizeof(int32_t);
    l.join_tab_off = off;
    off += kUpTailJobs * sizeof(int4);
    l.tiles_off = off;
    off = align_up(off + blocks * sizeof(int2), 256);
    l.work_up_off = off;
    off = align_up(off + (align_up(blocks * (H / 128), 8) + kTailSlots) * sizeof(int4), 256);
    l.work_down_off = off;
    const size_t n_wt_down = ((size_t)K + kWRows - 1) / kWRows;
    off = align_up(off + (align_up(blocks * n_wt_down, 8) + kTailSlots) * sizeof(int4), 256);
    l.tail_tab_off = off;
    if (dt == DT_BF16) off = align_up(off + blocks * n_wt_down * sizeof(int32_t), 256);
    // split tail jobs: no more of them than there are jobs; up to 3 partial tiles per down job
    l.down_tail_tiles = dt == DT_BF16 ? (int)std::min<size_t>(kTailSlots, 3 * align_up(blocks * n_wt_down, 8)) : 0;
    l.up_tail_jobs = dt == DT_BF16 ? (int)std::min<size_t>(kUpTailJobs, align_up(blocks * (H / 128), 8)) : 0;
    l.y_tail_off = off;
    off = align_up(off + (size_t)l.down_tail_tiles * kWRows * kWRows * 2, 256);
    // few up jobs for the chip (no more than the split can hold) and a contraction long enough to share among
    // more workgroups: deeper split, joined by a kernel of its own (see moe_up_join_kernel)
    // (at most kUpTailJobs / 2 jobs, so that the partial sums stay within what the shallow split reserves)
    l.deep_join = dt == DT_BF16 && blocks * (H / 128) <= (size_t)kUpTailJobs / 2 && K >= 2048;
    l.up_part_stride = l.deep_join ? kDeepParts : 4;
    l.up_partials_off = off;  // parts x 512 threads x 128 floats per job
    off = align_up(off + (size_t)l.up_tail_jobs * l.up_part_stride * 512 * 128 * sizeof(float), 256);
    l.inv_off = off;
    const size_t pairs = (size_t)M * (size_t)std::max(top_k, 1);
    off = align_up(off + pairs * sizeof(int32_t), 256);
    l.y_off = off;  // one row per pair id
    off = align_up(off + pairs * K * 2, 256);
    l.act_off = off;
    off = align_up(off + rows * H * (dt == DT_BF16 ? 2 : 1), 256);
    l.act_scales_off = off;
    if (dt == DT_FP8) off = align_up(off + rows * (H / 32), 256);
    l.xs_tiled_off = off;
    if (dt == DT_FP8) off = align_up(off + rows * ((size_t)K / 32), 256);
    l.total = off;
    return l;
}

static int grid_for(int n_tiles) { return (n_tiles + 7) / 8 * 8; }

// CU count of the current device, rounded down to a multiple of the 8 XCDs.
static int resident_grid() {
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
// Weight tiles a workgroup of the mxfp8 kernels takes in a row (0: chosen per launch); see
// pmoe_set_tiles_per_workgroup in the header.
static thread_local int g_tiles_per_wg = 0;

// A workgroup of the mxfp8 kernels can keep its token rows and take several weight tiles in a row: it
// saves the set-up of all but the first and starts each tile's copies under the epilogue of the one
// before, but the coarser work balances worse over the CUs.  Measured on the DeepSeek-V3-like prefill
// and decode shapes: two tiles gain 3 % on the down kernel (16 slabs per tile), nothing on the up kernel
// (56 slabs per tile), more than two lose on both.  So: two for the down kernel when that still leaves
// 8 rounds of workgroups per CU, one otherwise.  The bf16 kernels take one (their wide tiles run on the
// unit ring, which has no such hand-over).
static int tiles_per_workgroup(int dt, bool down, int n_blocks, int n_wt) {
    if (dt != DT_FP8) return 1;
    if (g_tiles_per_wg > 0) return std::min(g_tiles_per_wg, n_wt);
    return (down && (int64_t)n_blocks * n_wt >= (int64_t)resident_grid() * 16) ? 2 : 1;
}

struct SchedBuffers {
    int2 *tiles;
    int *n_tiles;
    int4 *work_up;
    int4 *work_down;
    int *tail_tab;     // null: the down kernel's tail is not split (mxfp8)
    int *up_counters;  // null: the up kernel's tail is not split (mxfp8)
    int down_tail_tiles, up_tail_jobs;  // capacities of y_tail and up_partials
    int4 *join_tab;    // null unless the split up jobs are joined by moe_up_join_kernel
};

template <int DT>
static int launch_pipeline(MoeArgs a, const SchedBuffers &sb, void *out, int split, hipStream_t s) {
    const int64_t n_out = (int64_t)a.M * a.K;  // K % 128 == 0, so n_out % 8 == 0
    const int mask = g_phase_mask;
    a.n_blocks = (a.sorted_num + kBlockRows - 1) / kBlockRows;
    a.n_wtiles = a.H / 128;
    const int n_wt_down = (a.K + kWRows - 1) / kWRows;
    const int per_up = tiles_per_workgroup(DT, false, a.n_blocks, a.n_wtiles);
    const int per_down = tiles_per_workgroup(DT, true, a.n_blocks, n_wt_down);
    const int grid_up = grid_for(a.n_blocks * ((a.n_wtiles + per_up - 1) / per_up)) + kTailSlots;
    // (the parts > 0 of split tail jobs sit behind the lists proper)
    const int grid_down = grid_for(a.n_blocks * ((n_wt_down + per_down - 1) / per_down)) + kTailSlots;
    {
        // the work lists are needed by the two kernels even when the rest of the prologue is masked off
        const int do_invert = (mask & PMOE_PHASE_PROLOGUE) ? 1 : 0;
        const int blocks = do_invert ? std::max(1, std::min((a.sorted_num + 255) / 256, 1024)) : 1;
        hipLaunchKernelGGL(moe_prologue_kernel, dim3(blocks), dim3(256), 0, s, a.expert_ids, a.ntpp, a.n_blocks,
                           sb.tiles, sb.n_tiles, sb.work_up, a.n_wtiles, per_up, grid_up,
                           sb.work_down, n_wt_down, per_down, grid_down, resident_grid(), a.K * 2 / 128, a.H * 2 / 128,
                           sb.tail_tab, sb.up_counters, sb.down_tail_tiles, sb.up_tail_jobs, sb.join_tab,
                           sb.join_tab != nullptr ? std::min(kDeepParts, std::max(1, a.K * 2 / 128 / 4)) : 4, a.E,
                           a.sorted_ids, a.sorted_num, a.inv, a.M * a.top_k, do_invert, a.x_scales, a.xs_tiled,
                           a.K >> 7, a.top_k, a.M);
    }
    if (a.n_blocks > 0) {
        a.work = sb.work_up;
        if (mask & PMOE_PHASE_UP) {
            hipLaunchKernelGGL((moe_up_kernel<DT>), dim3(grid_up), dim3(512), 0, s, a);
            if (a.deep_join) hipLaunchKernelGGL(moe_up_join_kernel, dim3(sb.up_tail_jobs * 32), dim3(256), 0, s, a);
        }
        MoeArgs d = a;
        d.n_wtiles = n_wt_down;
        d.work = sb.work_down;
        if (mask & PMOE_PHASE_DOWN)
            hipLaunchKernelGGL((moe_down_kernel<DT>), dim3(grid_down), dim3(512), 0, s, d);
    }
    if (mask & PMOE_PHASE_FINALIZE) {
        const int64_t n8 = n_out / 8;
        const int blocks = (int)std::min<int64_t>((n8 + 255) / 256, 8192);
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, s, a.y, a.inv, a.sorted_ids, a.ntpp, a.sorted_num,
                               a.topk_w, a.top_k, a.M, a.K, reinterpret_cast<uint4 *>(out), sb.tail_tab, a.y_tail,
                               n_wt_down, a.expert_ids, a.E);
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
    return check_launch("fused_moe launch");
}

static SchedBuffers sched_buffers(char *ws, const WorkspaceLayout &l) {
    SchedBuffers sb;
    sb.n_tiles = reinterpret_cast<int *>(ws + l.n_tiles_off);
    sb.tiles = reinterpret_cast<int2 *>(ws + l.tiles_off);
    sb.work_up = reinterpret_cast<int4 *>(ws + l.work_up_off);
    sb.work_down = reinterpret_cast<int4 *>(ws + l.work_down_off);
    sb.tail_tab = l.down_tail_tiles > 0 ? reinterpret_cast<int *>(ws + l.tail_tab_off) : nullptr;
    sb.up_counters = l.up_tail_jobs > 0 ? reinterpret_cast<int *>(ws + l.up_counters_off) : nullptr;
    sb.down_tail_tiles = l.down_tail_tiles;
    sb.up_tail_jobs = l.up_tail_jobs;
    sb.join_tab = l.deep_join ? reinterpret_cast<int4 *>(ws + l.join_tab_off) : nullptr;
    return sb;
}

}  // namespace pmoe

using namespace pmoe;

extern "C" void pmoe_set_phase_mask(int mask) { g_phase_mask = mask; }
extern "C" void pmoe_set_tiles_per_workgroup(int n) { g_tiles_per_wg = n < 0 ? 0 : (n > 16 ? 16 : n); }

extern "C" size_t pmoe_fused_moe_bf16_workspace_bytes(int M, int K, int N, int num_experts,
                                                      int sorted_num, int top_k, int split) {
    (void)num_experts;
    if (M <= 0 || K <= 0 || N <= 0 || sorted_num < 0) return 0;
    return workspace_layout(DT_BF16, M, K, N, sorted_num, top_k).total;
}

extern "C" size_t pmoe_fused_moe_mxfp8_workspace_bytes(int M, int K, int N, int num_experts,
                                                       int sorted_num, int top_k, int split) {
    (void)num_experts;
    if (M <= 0 || K <= 0 || N <= 0 || sorted_num < 0) return 0;
    return workspace_layout(DT_FP8, M, K, N, sorted_num, top_k).total;
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
    const WorkspaceLayout l = workspace_layout(DT_BF16, M, K, N, sorted_num, top_k);
    PMOE_REQUIRE(workspace && workspace_bytes >= l.total, "fused_moe_bf16: workspace of %zu bytes needed, got %zu", l.total, workspace_bytes);
    PMOE_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "fused_moe_bf16: workspace must be 256-byte aligned");
    MoeArgs a{};
    a.x = static_cast<const char *>(x);
    a.w1 = static_cast<const char *>(w);
    a.w2 = static_cast<const char *>(w2);
    a.sorted_ids = sorted_token_ids;
    a.expert_ids = expert_idxs;
    a.ntpp = num_tokens_post_padded;
    a.topk_w = topk_weights;
    char *ws = static_cast<char *>(workspace);
    a.y = ws + l.y_off;
    a.y_tail = ws + l.y_tail_off;
    a.up_partials = reinterpret_cast<float *>(ws + l.up_partials_off);
    a.up_counters = reinterpret_cast<int *>(ws + l.up_counters_off);
    a.join_tab = reinterpret_cast<int4 *>(ws + l.join_tab_off);
    a.up_part_stride = l.up_part_stride;
    a.deep_join = l.deep_join ? 1 : 0;
    a.inv = reinterpret_cast<int32_t *>(ws + l.inv_off);
    a.act = ws + l.act_off;
    a.top_k = top_k; a.M = M; a.K = K; a.N = N; a.H = N / 2; a.E = num_experts; a.sorted_num = sorted_num;
    return launch_pipeline<DT_BF16>(a, sched_buffers(ws, l), out, split, static_cast<hipStream_t>(stream));
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
    const WorkspaceLayout l = workspace_layout(DT_FP8, M, K, N, sorted_num, top_k);
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
    return launch_pipeline<DT_FP8>(a, sched_buffers(ws, l), out, split, static_cast<hipStream_t>(stream));
}
