// What the two translation units of the fused-MoE pipeline share (fused_moe.hip: entry points, mxfp8
// kernels, finalize; fused_moe_bf16.hip: the bf16 kernels on tall tiles): the argument block of the
// kernels, the schedule of the bf16 path (tiles cut by 32-row fragments, workgroup -> job by
// arithmetic on a small plan), cache-policy helpers.
#pragma once
#include "moe_tile.h"
#include "pmoe_common.h"

namespace pmoe {

// Schedule of the bf16 kernels, written by workgroup 0 of their prologue.
//
// Row tiles: an expert's live rows are F2 pairs of fragments of 32 sorted rows (the rows of its blocks up to
// the last one that holds a pair, rounded up inside the expert's own padding); they are cut into
// tiles of FG pairs each (FG = 1 .. 6, the tiles of one expert differ by at most one pair).
// tiles[i] = {first fragment, FG, expert, 0}.  Each of the two kernels has its own cut: the fewest tiles there
// can be, or as many more as make its jobs fill whole rounds of the chip's CUs when a cost model prefers that
// (the largest experts are then cut into one more tile each): the activation is indexed by sorted row, so the
// kernels need not agree on the tiles.
//
// Jobs of a kernel: (row tile, weight tile), n_tiles x n_wt of them, walked in the order
// [group of 8 weight tiles][row tile][weight tile in group].  The kernels are resident: one workgroup per CU,
// and the workgroups of an XCD (workgroup id mod 8: consecutive ids go round-robin to the XCDs) take the
// slots of that XCD's queue one after the other from a counter.  Slot `pos` of XCD `xcd` has the number
// b = 8 pos + xcd:
//  * b < main_end = jobs rounded up to whole rounds of 256: whole rounds are dealt to the XCDs in chunks of 32
//    positions of the walk (4 row tiles x 8 weight tiles: what runs side by side on the 32 CUs of an XCD
//    shares token slabs 8 ways and weight slabs 4 ways inside that XCD's L2), chunk c to XCD c mod 8; every
//    XCD then holds the same share of every part of the walk, whatever the sizes of the tiles.  The last,
//    partial round is dealt position by position, so that it loads all XCDs alike.
//  * The jobs of that last round (`tail` of them, if the plan splits them) would run while most CUs have
//    nothing left to do: each is shared among `parts` workgroups, which take `FG / parts` pairs of fragments
//    each (no sums to join: a part is a smaller tile).  The parts > 0 follow the main list on the XCD of their
//    part 0 (they read the same weight rows): b = main_end + 8 m + xcd is the m-th (job, part) pair of that XCD.
//
// Deep mode (up kernel only, up.deep != 0): so few jobs that even all of them together leave most CUs
// idle (the README shape: 16 jobs).  Then every job's contraction is shared among up.parts workgroups,
// b = job * parts + part; each stores its fp32 partial sums and moe_up_join_kernel adds them in part order and
// finishes the tiles.
struct KernelPlan {
    int n_tiles;
    int parts;  // 1: no split
    int tail;   // split jobs: the last, partial round of the walk
    int deep;   // up kernel: contraction split of every job (see above)
};
struct TallPlan {
    KernelPlan up, down;
    int counters[16];  // next slot of every XCD's queue: up kernel [0, 8), down kernel [8, 16)
};
struct TallJob {
    int tile, wt;
    int part, parts;
};
constexpr int kDeepParts = 8;    // most parts of an up job in deep mode
constexpr int kDeepJobs = 32;    // deep mode is considered up to this many (row block, weight tile) pairs

// Position l of a kernel's walk -> job.
__device__ __forceinline__ void walk_to_job(int l, int nt, int n_wt, int &tile, int &wt) {
    const int wg = l / (8 * nt), rem = l - wg * 8 * nt;
    const int gw = min(8, n_wt - wg * 8);
    tile = rem / gw;
    wt = wg * 8 + rem - tile * gw;
}
// Slot number b -> job.  Returns 1 with the job, 0 if the slot is empty, -1 if the queue of this slot's XCD has
// ended (every later slot is empty).
__device__ __forceinline__ int resolve_tall_job(int b, int n_wt, const KernelPlan &kp, TallJob &j) {
    const int nt = kp.n_tiles, n_jobs = nt * n_wt;
    j.part = 0;
    j.parts = 1;
    int l;
    if (kp.deep) {
        l = b / kp.parts;
        if (l >= n_jobs) return -1;
        j.part = b - l * kp.parts;
        j.parts = kp.parts;
    } else {
        const int full = n_jobs & ~255, main_end = (n_jobs + 255) & ~255;
        if (b < full) {
            const int xcd = b & 7, pos = b >> 3;
            l = (((pos >> 5) * 8 + xcd) << 5) + (pos & 31);
        } else if (b < main_end) {
            l = b;
            if (l >= n_jobs) return kp.parts > 1 ? 0 : -1;
            if (kp.parts > 1) j.parts = kp.parts;
        } else {
            if (kp.parts < 2) return -1;
            const int i = b - main_end, xcd = i & 7, m = i >> 3;
            const int q = m / (kp.parts - 1);
            const int k = q * 8 + xcd;  // the q-th tail job of this XCD
            if (k >= kp.tail) return -1;
            l = full + k;
            j.part = 1 + m - q * (kp.parts - 1);
            j.parts = kp.parts;
        }
    }
    walk_to_job(l, nt, n_wt, j.tile, j.wt);
    return 1;
}

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
    char *y;              // (M * top_k, K) bf16, by pair id: down-projected rows, before the routing weights
    int32_t *inv;         // (M * top_k): sorted row of each pair id (validated against sorted_ids when read)
    const int4 *work;     // mxfp8: this kernel's work list, one entry per workgroup
    // bf16 (tall tiles): the schedule, see TallPlan
    TallPlan *plan;
    int4 *tiles;          // row tiles of this kernel (the up kernel's or the down kernel's cut)
    int4 *tiles_down;     // the down kernel's cut
    int4 *runs;           // prologue scratch: the runs of blocks with one expert
    float *up_partials;   // deep mode: fp32 partial sums, [part][fragment][weight tile][32 KB]
    int deep_ok;          // deep mode may be planned (the workspace holds up_partials)
    int top_k, M, K, N, H, E, sorted_num;
    int n_blocks;  // sorted_num / 128 (rounded up)
    int n_wtiles;  // weight tiles along the free dimension: H/128 (up) or ceil(K/256) (down)
};

// 16 bytes that a kernel writes or reads once (activation and y tiles, out): non-temporal, so that they
// do not displace what the L2s could serve again.
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
constexpr int kYPitch = 528;        // 256 bf16 + 16 B pad

// CU count of the current device, rounded down to a multiple of the 8 XCDs.
int resident_grid();
// Which phases of the pipeline the fused entry points enqueue (see pmoe_set_phase_mask).
int phase_mask();
// Enqueues the routing-weight reduction: out[t] (+)= sum over the token's pairs of w * y (see finalize_kernel).
void launch_finalize(const MoeArgs &a, void *out, int split, int n_wt_down, hipStream_t s);

// The bf16 pipeline (fused_moe_bf16.hip): prologue, up kernel (+ join), down kernel; finalize through
// launch_finalize.  Returns a PMOE_* status.
int launch_bf16_pipeline(MoeArgs a, void *out, int split, hipStream_t s);
// Workspace of the bf16 pipeline: fills the pointers of `a` from `ws` (null: only sizes) and returns the bytes.
size_t bf16_workspace(MoeArgs &a, char *ws);

}  // namespace pmoe
