// bf16 kernels of the fused MoE forward for gfx950, on tall tiles (moe_tall.h): prologue (row tiles cut by
// 32-row fragments, plan of the two kernels), gate/up GEMM + SwiGLU, down GEMM.
//
// Replaces the bf16 launcher and kernels of the reference's
// prime_moe/csrc/kernels/fused_moe_bf16_kernel.cu:21-733 (gather :21-47, gate/up GEMM + SwiGLU :196-229,
// down GEMM :496-542).
//
// No work list: a workgroup derives its job from its id and a 48-byte plan that workgroup 0 of the
// prologue writes (see TallPlan), so the prologue only builds the table of row tiles.  No value is
// accumulated with atomics and every sum has a fixed order: the result is a pure function of the inputs.
#include <algorithm>

#include "moe_pipeline.h"
#include "moe_tall.h"

namespace pmoe {

constexpr int kPrologueThreads = 1024;
// Inclusive scan of one int per thread over the workgroup of the prologue; `s_part` holds an int per wave.
__device__ __forceinline__ int block_scan(int v, int *s_part) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int t = __shfl_up(v, d, 64);
        if (lane >= d) v += t;
    }
    __syncthreads();  // s_part may still be read from the previous call
    if (lane == 63) s_part[wave] = v;
    __syncthreads();
    for (int w = 0; w < wave; ++w) v += s_part[w];
    return v;
}

// Estimated time of a kernel (in units of a third of a microsecond) whose `f2` pairs of fragments are cut into
// `n_tiles` row tiles: whole rounds of the chip's CUs at the cost of a mean tile, plus a last round whose jobs
// are shared by rows.  A tile of g pairs costs (0.6 + g) per slab of its K loop (measured on operands that stay in
// L2: 0.18 + 0.34 g us on tiles of 2 to 6 pairs; inside a full kernel the fixed part is larger, which only
// strengthens the preference for few, tall tiles) and 3 + 2.5 g for set-up and epilogue; a round of nothing but shared jobs costs 1.3
// times what its small tiles would among large ones (measured on the Mixtral-like down kernel: every weight row
// is then read twice as often).
__device__ __forceinline__ float estimate_kernel(int n_tiles, int f2, int n_wt, int n_slabs, int n_cus, int &parts,
                                                 int &tail) {
    parts = 1;
    tail = 0;
    if (n_tiles <= 0) return 0.f;
    const float g = (float)f2 / (float)n_tiles;
    auto cost = [&](float pairs) { return (float)n_slabs * (0.6f + pairs) + 3.f + 2.5f * pairs; };
    const int jobs = n_tiles * n_wt, rounds = jobs / n_cus, rest = jobs % n_cus;
    float t = (float)rounds * cost(g);
    if (rest > 0) {
        const int p = rounds >= 16 ? 1 : min(min(4, n_cus / rest), max(1, (int)g));
        t += p > 1 ? 1.3f * cost(g / (float)p) : cost(g);
        if (p > 1) {
            parts = p;
            tail = rest;
        }
    }
    return t;
}
// Number of row tiles for a kernel with n_wt weight tiles: the fewest there can be (t_min, tiles of up to 6
// pairs), or, if the estimate likes it better, the next number that fills whole rounds of the CUs (smaller
// tiles, nothing left over), as long as that is at most half as many again and fits the tables (t_cap).
__device__ __forceinline__ int choose_tiles(int t_min, int t_cap, int f2, int n_wt, int n_slabs, int n_cus) {
    if (t_min <= 0) return 0;
    int g = n_cus, r = n_wt;  // gcd
    while (r) {
        const int x = g % r;
        g = r;
        r = x;
    }
    const int step = n_cus / g;  // tiles x n_wt is a multiple of n_cus for every multiple of step
    const int t_full = (t_min + step - 1) / step * step;
    if (t_full == t_min || t_full > t_cap || 2 * t_full > 3 * t_min || t_full > f2) return t_min;
    int parts, tail;
    const float e_min = estimate_kernel(t_min, f2, n_wt, n_slabs, n_cus, parts, tail);
    const float e_full = estimate_kernel(t_full, f2, n_wt, n_slabs, n_cus, parts, tail);
    return e_full < 0.98f * e_min ? t_full : t_min;
}

// Prologue of a bf16 call.  Workgroup 0 builds the row tiles and the plan:
//  1. runs of blocks with one expert (a thread per block, block-wide scans per 1024 blocks); the thread of a run's
//     last block reads that block's 128 ids for the last row that holds a pair: the run has f2 pairs of fragments;
//  2. per kernel the number of row tiles (see choose_tiles);
//  3. the runs in the order of falling f2 (a counting sort; runs of one size in the order their threads arrive,
//     which only moves equal tiles in the schedule): the walk of a kernel then ends with the small tiles, and
//     what is left over when the CUs run out of jobs is short;
//  4. the tiles of the two cuts (a run gets the tiles it needs at 6 pairs a tile, and the largest runs one more
//     each until the chosen number is reached), then the plans with the split of the tails.
// The list of runs lives in LDS (in the workspace when there are more than kLdsRuns blocks).
// All workgroups invert the sorted order: inv[pair id] = sorted row.  Entries of pairs that are not in the
// schedule keep whatever the buffer held; the reader validates an entry against sorted_ids.
constexpr int kLdsRuns = 2048;
constexpr int kSizeKeys = 128;  // runs are ordered by min(f2, kSizeKeys - 1)
__global__ __launch_bounds__(kPrologueThreads) void moe_prologue_kernel_bf16(MoeArgs a, int n_wt_up, int n_wt_down, int n_cus,
                                                                int do_invert) {
    const int n_pairs = a.M * a.top_k;
    if (blockIdx.x == 0) {
        __shared__ int4 s_runs[kLdsRuns];  // {first block, f2, expert, 0}
        __shared__ int s_order[kLdsRuns];
        __shared__ int s_part[kPrologueThreads / 64], s_carry[2], s_want[2], s_tiles[2];
        __shared__ int s_sum[8];            // [0]: tiles of up to 6 pairs the runs need; [4]: pairs of fragments
        __shared__ int s_hist[kSizeKeys];   // runs per size key, then the first place of each key in the order
        const int tid = threadIdx.x;
        const int n_live = min((a.ntpp[0] + kBlockRows - 1) / kBlockRows, a.n_blocks);
        int4 *runs = n_live <= kLdsRuns ? s_runs : a.runs;
        int *order = n_live <= kLdsRuns ? s_order : reinterpret_cast<int *>(a.runs + n_live);
        if (tid < 2) s_carry[tid] = tid == 0 ? -1 : 0;
        if (tid < 8) s_sum[tid] = 0;
        if (tid < kSizeKeys) s_hist[tid] = 0;
        if (tid < 16) a.plan->counters[tid] = n_cus / 8;  // the first slots are taken without asking (see ask_slot)
        __syncthreads();
        // 1. runs
        for (int base = 0; base < n_live; base += kPrologueThreads) {
            const int b = base + tid;
            const bool live = b < n_live;
            const int e = live ? a.expert_ids[b] : -1;
            const bool is_start = live && (b == 0 || a.expert_ids[b - 1] != e);
            const bool is_last = live && (b + 1 == n_live || a.expert_ids[b + 1] != e);
            // start of this block's run: the largest start at or before it
            int v = is_start ? b : -1;
            {
                const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
                for (int d = 1; d < 64; d <<= 1) {
                    const int t = __shfl_up(v, d, 64);
                    if (lane >= d) v = max(v, t);
                }
                __syncthreads();
                if (lane == 63) s_part[wave] = v;
                __syncthreads();
                for (int w = 0; w < wave; ++w) v = max(v, s_part[w]);
                v = max(v, s_carry[0]);
            }
            const int run_start = v;
            int f2 = 0;
            if (is_last && e >= 0 && e < a.E) {
                const int s0 = b * kBlockRows;
                int last = -1;
                if (s0 + kBlockRows <= a.sorted_num && (reinterpret_cast<uintptr_t>(a.sorted_ids) & 15) == 0) {
                    // all 32 loads in flight together
                    const int4 *src = reinterpret_cast<const int4 *>(a.sorted_ids + s0);
                    int4 v[kBlockRows / 4];
#pragma unroll
                    for (int r = 0; r < kBlockRows / 4; ++r) v[r] = src[r];
#pragma unroll
                    for (int r = 0; r < kBlockRows / 4; ++r) {
                        if ((unsigned)v[r].x < (unsigned)n_pairs) last = 4 * r;
                        if ((unsigned)v[r].y < (unsigned)n_pairs) last = 4 * r + 1;
                        if ((unsigned)v[r].z < (unsigned)n_pairs) last = 4 * r + 2;
                        if ((unsigned)v[r].w < (unsigned)n_pairs) last = 4 * r + 3;
                    }
                } else {
                    for (int r = 0; r < kBlockRows; ++r) {
                        const int p = s0 + r < a.sorted_num ? a.sorted_ids[s0 + r] : -1;
                        if ((unsigned)p < (unsigned)n_pairs) last = r;
                    }
                }
                f2 = ((b - run_start) * kBlockRows + last + 1 + 63) >> 6;
            }
            const int incl = block_scan(f2 > 0 ? 1 : 0, s_part);
            const int carry = s_carry[1];
            if (f2 > 0) {
                runs[carry + incl - 1] = make_int4(run_start, f2, e, 0);
                atomicAdd(&s_hist[min(f2, kSizeKeys - 1)], 1);
                atomicAdd(&s_sum[4], f2);
                atomicAdd(&s_sum[0], (f2 + 5) / 6);
            }
            __syncthreads();
            if (tid == kPrologueThreads - 1) {
                s_carry[0] = run_start;
                s_carry[1] = carry + incl;
            }
            __syncthreads();
        }
        const int n_runs = s_carry[1];
        __threadfence_block();
        // 2. the number of row tiles of each kernel: tid 0 the up kernel's, tid 1 the down kernel's
        if (tid < 2) {
            const int n_wt = tid ? n_wt_down : n_wt_up, n_slabs = (tid ? a.H : a.K) * 2 / tall::kRB;
            s_want[tid] = choose_tiles(s_sum[0], a.n_blocks, s_sum[4], n_wt, n_slabs, n_cus);
        }
        // 3. order of the runs: by falling size key, runs of one key in their own order.  First place of each key ...
        if (tid < 64) {
            // (one wave: key k's place = runs with a larger key; two keys per lane, largest keys first)
            const int k_hi = kSizeKeys - 1 - 2 * tid, k_lo = k_hi - 1;
            const int c_hi = s_hist[k_hi], c_lo = s_hist[k_lo];
            int incl = c_hi + c_lo;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int t = __shfl_up(incl, d, 64);
                if (tid >= d) incl += t;
            }
            s_hist[k_hi] = incl - c_hi - c_lo;
            s_hist[k_lo] = incl - c_lo;
        }
        __syncthreads();
        // ... then every run takes the next place of its key
        for (int i = tid; i < n_runs; i += kPrologueThreads) order[atomicAdd(&s_hist[min(runs[i].y, kSizeKeys - 1)], 1)] = i;
        __syncthreads();
        __threadfence_block();
        // 4. the tiles of the two cuts (one pass when both kernels use the same cut), and the plans
        const int t_min = s_sum[0];
        const bool same = s_want[0] == s_want[1];
        for (int k = 0; k < (same ? 1 : 2); ++k) {
            const int extra = max(s_want[k] - t_min, 0);
            if (tid == 0) s_carry[0] = 0;
            __syncthreads();
            for (int base = 0; base < n_runs; base += kPrologueThreads) {
                const int i = base + tid;  // place in the order: the largest runs come first
                int4 r = make_int4(0, 0, 0, 0);
                if (i < n_runs) r = runs[order[i]];
                const int f2 = r.y;
                int n = (f2 + 5) / 6;
                if (i < n_runs) n = min(f2, n + extra / n_runs + (i < extra % n_runs ? 1 : 0));
                const int incl = block_scan(n, s_part);
                const int carry = s_carry[0];
                int t = carry + incl - n, frag = 4 * r.x;
                for (int q = 0; q < n; ++q) {
                    const int fg = f2 / n + (q < f2 % n ? 1 : 0);
                    const int4 tl = make_int4(frag, fg, r.z, 0);
                    if (k == 0) a.tiles[t + q] = tl;
                    if (k == 1 || same) a.tiles_down[t + q] = tl;
                    frag += 2 * fg;
                }
                __syncthreads();
                if (tid == kPrologueThreads - 1) s_carry[0] = carry + incl;
                __syncthreads();
            }
            if (tid == 0) s_tiles[k] = s_carry[0];
            if (tid == 0 && same) s_tiles[1] = s_carry[0];
            __syncthreads();
        }
        if (tid < 2) {
            const int n_wt = tid ? n_wt_down : n_wt_up, n_slabs = (tid ? a.H : a.K) * 2 / tall::kRB;
            KernelPlan kp{};
            kp.n_tiles = s_tiles[tid];
            estimate_kernel(kp.n_tiles, s_sum[4], n_wt, n_slabs, n_cus, kp.parts, kp.tail);
            if (tid == 0) {
                const int jobs_up = kp.n_tiles * n_wt_up;
                int deep_parts = 1;
                if (a.deep_ok && jobs_up > 0) deep_parts = min(min(kDeepParts, n_slabs / 4), n_cus / jobs_up);
                if (deep_parts >= 2) {
                    kp.deep = 1;
                    kp.parts = deep_parts;
                    kp.tail = 0;
                }
                a.plan->up = kp;
            } else {
                a.plan->down = kp;
            }
        }
    }
    if (do_invert) {
        const int n_rows = min(a.ntpp[0], a.sorted_num);
        const int stride = (int)(gridDim.x * blockDim.x);
        for (int s = (int)(blockIdx.x * blockDim.x + threadIdx.x); s < n_rows; s += stride) {
            const int p = a.sorted_ids[s];
            const int e = a.expert_ids[s >> 7];  // rows of a block without an expert are not computed
            if (p >= 0 && p < n_pairs && e >= 0 && e < a.E) a.inv[p] = s;
        }
    }
}

template <int FG>
__device__ __forceinline__ void zero_acc(f32x16 (&acc)[2][FG]) {
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int t = 0; t < FG; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[f][t][i] = 0.f;
}

// The part of a tile (first fragment f0, FG pairs of fragments) that part `part` of `parts` takes when a
// tail job is shared by rows: pairs [part FG / parts, (part + 1) FG / parts).  Returns its number of pairs.
__device__ __forceinline__ int row_split(int &f0, int fg, int part, int parts) {
    const int lo = part * fg / parts, hi = (part + 1) * fg / parts;
    f0 += 2 * lo;
    return hi - lo;
}

// Where deep-mode partial sums of (part, fragment, weight tile) live: 2048 float4 = the two accumulators
// (gate, up) of the four waves that own the fragment, [f][q][wave % 4][lane].
__device__ __forceinline__ float4 *partial_block(const MoeArgs &a, int part, int frag, int wt) {
    return reinterpret_cast<float4 *>(a.up_partials) +
           (((int64_t)part * (4 * a.n_blocks) + frag) * a.n_wtiles + wt) * 2048;
}

// The queue of an XCD: its workgroups (workgroup w is number w / 8 of XCD w mod 8) start with the slot of their own
// number and take further slots from the XCD's counter, which the prologue sets to the number of workgroups
// per XCD.  Thread 0 asks for the next slot when the K loop of a tile ends (`ask`), so that the answer arrives
// under the epilogue (asked earlier, a busy workgroup would hold a job that an idle one could run); `pass`
// hands it to every thread through `word`, a word of LDS that nothing else uses at that moment.
__device__ __forceinline__ int ask_slot(int *counter) { return threadIdx.x == 0 ? atomicAdd(counter, 1) : 0; }
__device__ __forceinline__ int pass_slot(int asked, int *word) {
    __syncthreads();  // whatever used the LDS before is done
    if (threadIdx.x == 0) *word = asked;
    __syncthreads();
    const int pos = *word;
    __syncthreads();  // everybody has read the word: the LDS is free again
    return __builtin_amdgcn_readfirstlane(pos);
}

// Up kernel tile: token fragments f0 .. f0 + 2 FG - 1 x activation columns [128 wt, 128 wt + 128) of expert e,
// contraction slabs [slab0, slab0 + n_slabs).  LDS weight rows 0..127 are gate rows, 128..255 the matching up
// rows; wave v of a group owns gate/up rows 32v..32v+31, so gate and up of one activation element sit in the
// same lane and register: SwiGLU in registers, the 2H-wide tensor never leaves the chip.
// deep_part >= 0: the contraction is shared (deep mode); the fp32 sums go to up_partials instead.
template <int FG>
__device__ __forceinline__ int up_tile_tall(const MoeArgs &a, int e, int f0, int wt, int slab0, int n_slabs,
                                            int deep_part, int pos, int *counter, char *lds) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, w4 = wave & 3;
    const int K = a.K, H = a.H, N = a.N;
    const int h0 = wt * 128;
    const int64_t row0 = (int64_t)f0 * 32;
    const uint32_t row_bytes = (uint32_t)K * 2u;
    const uint32_t n_pairs = (uint32_t)(a.M * a.top_k);
    const char *w_gate = a.w1 + ((int64_t)e * N + h0) * K * 2 + slab0 * tall::kRB;
    tall::Loader<FG, true> ld;
    ld.setup(tid, a.x + slab0 * tall::kRB, w_gate, w_gate + (int64_t)H * K * 2, row_bytes, row_bytes, [&](int row) {
        const int64_t s = row0 + row;
        const int p = s < a.sorted_num ? a.sorted_ids[s] : -1;
        const uint32_t tok = (uint32_t)p < n_pairs ? (uint32_t)p / (uint32_t)a.top_k : 0u;  // dead rows read token 0
        return tok * row_bytes;
    });
    const int wrow[2] = {32 * w4, 128 + 32 * w4};
    f32x16 acc[2][FG];
    zero_acc<FG>(acc);
    const int start = (pos & 7) % n_slabs;  // workgroups that run side by side start their K walks at different slabs
    tall::main_loop<FG>(acc, ld, lds, n_slabs, wrow, grp * FG, lane, start);
    const int asked = ask_slot(counter);

    const int r = lane & 31, half = lane >> 5;
    if (deep_part >= 0) {
#pragma unroll
        for (int t = 0; t < FG; ++t) {
            float4 *dst = partial_block(a, deep_part, f0 + grp * FG + t, wt);
#pragma unroll
            for (int f = 0; f < 2; ++f)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    dst[((f * 4 + q) * 4 + w4) * 64 + lane] =
                        make_float4(acc[f][t][4 * q], acc[f][t][4 * q + 1], acc[f][t][4 * q + 2], acc[f][t][4 * q + 3]);
        }
        return asked;
    }
    // register i of lane l = activation column 32 w4 + 8(i/4) + 4(l/32) + i%4 of token row 32 t + l%32
    char *tile = lds + grp * (32 * FG * kActPitchBf16);
#pragma unroll
    for (int t = 0; t < FG; ++t) {
        const int row = 32 * t + r;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int hl = 32 * w4 + 8 * g + 4 * half;  // tile-local activation column
            uint2 pk;
            pk.x = pack2_bf16(swiglu(acc[0][t][4 * g], acc[1][t][4 * g]), swiglu(acc[0][t][4 * g + 1], acc[1][t][4 * g + 1]));
            pk.y = pack2_bf16(swiglu(acc[0][t][4 * g + 2], acc[1][t][4 * g + 2]),
                              swiglu(acc[0][t][4 * g + 3], acc[1][t][4 * g + 3]));
            *reinterpret_cast<uint2 *>(tile + row * kActPitchBf16 + hl * 2) = pk;
        }
    }
    __syncthreads();
    // coalesced copy of the group's 32 FG x 128 tile to the activation rows (by sorted row)
    const int gt = tid & 255, c = gt & 15;
    const int64_t grow0 = row0 + grp * 32 * FG;
#pragma unroll
    for (int i = 0; i < 2 * FG; ++i) {
        const int row = (gt >> 4) + 16 * i;
        const uint4 v = *reinterpret_cast<const uint4 *>(tile + row * kActPitchBf16 + c * 16);
        store_once(a.act + ((grow0 + row) * H + h0) * 2 + c * 16, v);
    }
    return asked;
}

__global__ __launch_bounds__(512) void moe_up_kernel_bf16(MoeArgs a) {
    __shared__ __attribute__((aligned(1024))) char lds[tall::kLdsBytes];
    const KernelPlan kp = a.plan->up;
    const int xcd = (int)(blockIdx.x & 7);
    const int n_slabs_all = a.K * 2 / tall::kRB;
    int *counter = &a.plan->counters[xcd];
    for (int pos = (int)(blockIdx.x >> 3);;) {
        TallJob j;
        const int st = resolve_tall_job(8 * pos + xcd, a.n_wtiles, kp, j);
        if (st < 0) break;
        if (st == 0) {
            pos = pass_slot(ask_slot(counter), reinterpret_cast<int *>(lds));
            continue;
        }
        int asked = 0;
        const int4 tl = a.tiles[j.tile];
        int f0 = tl.x, fg = tl.y;
        const int e = tl.z;
        int slab0 = 0, n_slabs = n_slabs_all, deep_part = -1;
        if (kp.deep) {
            slab0 = j.part * n_slabs_all / j.parts;
            n_slabs = (j.part + 1) * n_slabs_all / j.parts - slab0;
            deep_part = j.part;
        } else if (j.parts > 1) {
            fg = row_split(f0, fg, j.part, j.parts);
        }
        fg = __builtin_amdgcn_readfirstlane(fg);
        switch (fg) {
            case 1: asked = up_tile_tall<1>(a, e, f0, j.wt, slab0, n_slabs, deep_part, pos, counter, lds); break;
            case 2: asked = up_tile_tall<2>(a, e, f0, j.wt, slab0, n_slabs, deep_part, pos, counter, lds); break;
            case 3: asked = up_tile_tall<3>(a, e, f0, j.wt, slab0, n_slabs, deep_part, pos, counter, lds); break;
            case 4: asked = up_tile_tall<4>(a, e, f0, j.wt, slab0, n_slabs, deep_part, pos, counter, lds); break;
            case 5: asked = up_tile_tall<5>(a, e, f0, j.wt, slab0, n_slabs, deep_part, pos, counter, lds); break;
            case 6: asked = up_tile_tall<6>(a, e, f0, j.wt, slab0, n_slabs, deep_part, pos, counter, lds); break;
            default: asked = ask_slot(counter); break;
        }
        pos = pass_slot(asked, reinterpret_cast<int *>(lds));
    }
}

// Deep mode: adds the partial sums the parts of every up job left in memory and finishes the tiles.  One
// workgroup of 4 waves per (row tile, fragment of it, weight tile, quarter of the accumulator registers):
// thread (v, lane) takes over registers 4q .. 4q + 3 of what thread (v, lane) of the fragment's group held, gate
// and up sums, adds the parts in part order, applies SwiGLU and writes its 4 activation values.  All loads of
// a thread are in flight together: the kernel is one memory latency long.
__global__ __launch_bounds__(256) void moe_up_join_kernel(MoeArgs a) {
    const KernelPlan kp = a.plan->up;
    if (!kp.deep) return;
    int b = blockIdx.x;
    const int q = b & 3;
    b >>= 2;
    const int wt = b % a.n_wtiles;
    b /= a.n_wtiles;
    const int t = b % tall::kMaxFrags, tile = b / tall::kMaxFrags;
    if (tile >= kp.n_tiles) return;
    const int4 tl = a.tiles[tile];
    if (t >= 2 * tl.y) return;
    const int frag = tl.x + t, parts = kp.parts;
    const int tid = threadIdx.x, lane = tid & 63, v = tid >> 6;
    float4 vg[kDeepParts], vu[kDeepParts];
#pragma unroll
    for (int p = 0; p < kDeepParts; ++p)
        if (p < parts) {
            const float4 *src = partial_block(a, p, frag, wt);
            vg[p] = src[((0 * 4 + q) * 4 + v) * 64 + lane];
            vu[p] = src[((1 * 4 + q) * 4 + v) * 64 + lane];
        }
    float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < kDeepParts; ++p)
        if (p < parts) {
            g[0] += vg[p].x; g[1] += vg[p].y; g[2] += vg[p].z; g[3] += vg[p].w;
            u[0] += vu[p].x; u[1] += vu[p].y; u[2] += vu[p].z; u[3] += vu[p].w;
        }
    const int hl = 32 * v + 8 * q + 4 * (lane >> 5);  // tile-local activation column, as in up_tile_tall
    uint2 pk;
    pk.x = pack2_bf16(swiglu(g[0], u[0]), swiglu(g[1], u[1]));
    pk.y = pack2_bf16(swiglu(g[2], u[2]), swiglu(g[3], u[3]));
    *reinterpret_cast<uint2 *>(a.act + (((int64_t)frag * 32 + (lane & 31)) * a.H + wt * 128 + hl) * 2) = pk;
}

// Down kernel tile: y[pairs of the tile's rows, 256 columns of K from 256 wt] = act[rows, :H] . W2[e][cols, :H]^T,
// the whole reduction over H inside the workgroup; the routing weights are applied later, by finalize_kernel.
// Weight rows (output columns) sit on the MFMA M side: register i of lane l = output column
// 64 w4 + 32 f + 8(i/4) + 4(l/32) + i%4 of tile row 32 t + l%32.  A group's 32 FG x 256 tile is rounded to
// bf16 and transposed through LDS (one group after the other: both do not fit), then all 512 threads store
// its rows, 512 contiguous bytes each, to y[pair id]; rows without a pair are skipped.
template <int FG>
__device__ __forceinline__ int down_tile_tall(const MoeArgs &a, int e, int f0, int wt, int pos, int *counter, char *lds) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, w4 = wave & 3;
    const int K = a.K, H = a.H;
    const int k0 = wt * kWRows;
    const int64_t row0 = (int64_t)f0 * 32;
    const uint32_t row_bytes = (uint32_t)H * 2u;
    const int n_slabs = (int)(row_bytes / tall::kRB);
    // weight rows (output columns) k0 .. k0 + 255 of the expert; the last tile of a K that is not a multiple
    // of 256 has 128 of them and reads the first half twice
    const char *w_lo = a.w2 + ((int64_t)e * K + k0) * H * 2;
    const char *w_hi = (k0 + 128 < K) ? w_lo + (int64_t)128 * H * 2 : w_lo;
    tall::Loader<FG, false> ld;
    ld.setup(tid, a.act + row0 * H * 2, w_lo, w_hi, row_bytes, row_bytes, [&](int row) { return (uint32_t)row * row_bytes; });
    const int wrow[2] = {64 * w4, 64 * w4 + 32};
    f32x16 acc[2][FG];
    zero_acc<FG>(acc);
    const int start = (pos & 7) % n_slabs;  // workgroups that run side by side start their K walks at different slabs
    tall::main_loop<FG>(acc, ld, lds, n_slabs, wrow, grp * FG, lane, start);
    const int asked = ask_slot(counter);

    const int r = lane & 31, half = lane >> 5;
    const int cols = min(kWRows, K - k0);
    const uint32_t n_pairs = (uint32_t)(a.M * a.top_k);
    const int c = tid & 31;
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        // 32 threads per row (16 bytes each), 16 rows per turn; the pair ids of this thread's rows are fetched
        // first, so that they are in flight during the LDS round trip
        int pr[2 * FG];
#pragma unroll
        for (int i = 0; i < 2 * FG; ++i) {
            const int64_t s = row0 + g * 32 * FG + (tid >> 5) + 16 * i;
            pr[i] = s < a.sorted_num ? a.sorted_ids[s] : -1;
        }
        if (grp == g) {
#pragma unroll
            for (int t = 0; t < FG; ++t) {
                const int row = 32 * t + r;
#pragma unroll
                for (int f = 0; f < 2; ++f)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int col = 64 * w4 + 32 * f + 8 * q + 4 * half;
                        uint2 pk;
                        pk.x = pack2_bf16(acc[f][t][4 * q], acc[f][t][4 * q + 1]);
                        pk.y = pack2_bf16(acc[f][t][4 * q + 2], acc[f][t][4 * q + 3]);
                        *reinterpret_cast<uint2 *>(lds + row * kYPitch + col * 2) = pk;
                    }
            }
        }
        __syncthreads();
        if (8 * c < cols) {
#pragma unroll
            for (int i = 0; i < 2 * FG; ++i) {
                const int row = (tid >> 5) + 16 * i;
                if ((uint32_t)pr[i] < n_pairs) {
                    const uint4 v = *reinterpret_cast<const uint4 *>(lds + row * kYPitch + c * 16);
                    store_once(a.y + (int64_t)pr[i] * K * 2 + (int64_t)k0 * 2 + c * 16, v);
                }
            }
        }
        if (g == 0) __syncthreads();
    }
    return asked;
}

__global__ __launch_bounds__(512) void moe_down_kernel_bf16(MoeArgs a) {
    __shared__ __attribute__((aligned(1024))) char lds[tall::kLdsBytes];
    const KernelPlan kp = a.plan->down;
    const int xcd = (int)(blockIdx.x & 7);
    int *counter = &a.plan->counters[8 + xcd];
    for (int pos = (int)(blockIdx.x >> 3);;) {
        TallJob j;
        const int st = resolve_tall_job(8 * pos + xcd, a.n_wtiles, kp, j);
        if (st < 0) break;
        if (st == 0) {
            pos = pass_slot(ask_slot(counter), reinterpret_cast<int *>(lds));
            continue;
        }
        int asked = 0;
        const int4 tl = a.tiles_down[j.tile];
        int f0 = tl.x, fg = tl.y;
        const int e = tl.z;
        if (j.parts > 1) fg = row_split(f0, fg, j.part, j.parts);
        fg = __builtin_amdgcn_readfirstlane(fg);
        switch (fg) {
            case 1: asked = down_tile_tall<1>(a, e, f0, j.wt, pos, counter, lds); break;
            case 2: asked = down_tile_tall<2>(a, e, f0, j.wt, pos, counter, lds); break;
            case 3: asked = down_tile_tall<3>(a, e, f0, j.wt, pos, counter, lds); break;
            case 4: asked = down_tile_tall<4>(a, e, f0, j.wt, pos, counter, lds); break;
            case 5: asked = down_tile_tall<5>(a, e, f0, j.wt, pos, counter, lds); break;
            case 6: asked = down_tile_tall<6>(a, e, f0, j.wt, pos, counter, lds); break;
            default: asked = ask_slot(counter); break;
        }
        pos = pass_slot(asked, reinterpret_cast<int *>(lds));
    }
}

// ------------------------------------------------------------------------------------------ host

size_t bf16_workspace(MoeArgs &a, char *ws) {
    const size_t H = (size_t)a.H;
    const size_t rows = align_up((size_t)a.sorted_num, kBlockRows);
    const size_t blocks = rows / kBlockRows;
    const size_t n_wt_up = H / 128;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off = align_up(off + bytes, 256);
        return ws != nullptr ? ws + at : nullptr;
    };
    a.plan = reinterpret_cast<TallPlan *>(take(sizeof(TallPlan)));
    // (run list and its order, used when they do not fit the LDS of the prologue)
    a.runs = reinterpret_cast<int4 *>(take((blocks + 1) * (sizeof(int4) + sizeof(int))));
    // (a cut has at most one tile per block: choose_tiles)
    a.tiles = reinterpret_cast<int4 *>(take((blocks + 1) * sizeof(int4)));
    a.tiles_down = reinterpret_cast<int4 *>(take((blocks + 1) * sizeof(int4)));
    // few up jobs for the chip and a contraction long enough to share: deep mode may be planned
    a.deep_ok = (blocks * n_wt_up <= (size_t)kDeepJobs && a.K >= 2048) ? 1 : 0;
    a.up_partials = reinterpret_cast<float *>(
        take(a.deep_ok ? (size_t)kDeepParts * 4 * blocks * n_wt_up * 2048 * sizeof(float4) : 0));
    const size_t pairs = (size_t)a.M * (size_t)std::max(a.top_k, 1);
    a.inv = reinterpret_cast<int32_t *>(take(pairs * sizeof(int32_t)));
    a.y = take(pairs * a.K * 2);  // one row per pair id
    a.act = take(rows * H * 2);
    return off;
}

int launch_bf16_pipeline(MoeArgs a, void *out, int split, hipStream_t s) {
    const int mask = phase_mask();
    a.n_blocks = (a.sorted_num + kBlockRows - 1) / kBlockRows;
    const int n_wt_up = a.H / 128, n_wt_down = (a.K + kWRows - 1) / kWRows;
    const int n_cus = resident_grid();
    {
        // the plan is needed by the two kernels even when the rest of the prologue is masked off
        const int do_invert = (mask & PMOE_PHASE_PROLOGUE) ? 1 : 0;
        const int blocks = do_invert ? std::max(1, std::min((a.sorted_num + kPrologueThreads - 1) / kPrologueThreads, 512)) : 1;
        hipLaunchKernelGGL(moe_prologue_kernel_bf16, dim3(blocks), dim3(kPrologueThreads), 0, s, a, n_wt_up, n_wt_down, n_cus,
                           do_invert);
    }
    if (a.n_blocks > 0) {
        // resident kernels: a workgroup per CU (their 160 KB of LDS leave room for one)
        a.n_wtiles = n_wt_up;
        if (mask & PMOE_PHASE_UP) {
            hipLaunchKernelGGL(moe_up_kernel_bf16, dim3(n_cus), dim3(512), 0, s, a);
            if (a.deep_ok)
                hipLaunchKernelGGL(moe_up_join_kernel, dim3(a.n_blocks * tall::kMaxFrags * n_wt_up * 4), dim3(256), 0, s, a);
        }
        MoeArgs d = a;
        d.n_wtiles = n_wt_down;
        if (mask & PMOE_PHASE_DOWN) hipLaunchKernelGGL(moe_down_kernel_bf16, dim3(n_cus), dim3(512), 0, s, d);
    }
    if (mask & PMOE_PHASE_FINALIZE) launch_finalize(a, out, split, n_wt_down, s);
    return check_launch("fused_moe_bf16 launch");
}

}  // namespace pmoe
