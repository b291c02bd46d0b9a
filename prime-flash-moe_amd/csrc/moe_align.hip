// moe_align for gfx950: stable counting sort of pair ids by expert, padded per expert.
//
// Semantics follow the reference kernel (prime_moe/csrc/kernels/fused_moe_bf16_kernel.cu:853-907)
// except that the within-expert order is made unique (ascending pair id) instead of being
// left to an atomic race.  One workgroup, wave64:
//   1. each wave histograms a contiguous slice of the ids into its own LDS row,
//   2. per expert, the per-wave counts become exclusive per-wave bases; the padded
//      per-expert totals are prefix-summed by one wave with a shuffle scan,
//   3. each wave walks its slice again 64 ids at a time; lanes holding the same
//      expert find each other with one ballot per id bit, the lane's rank inside
//      that group is a popcount of the lower lanes, and the destination is
//      offs[e] + base[wave][e] + rank.
// All arithmetic is int32 and the output is a pure function of the input.
#include <mutex>

#include "pmoe_common.h"

namespace {

constexpr int kMaxExperts = 1024;

template <int NW>
__global__ __launch_bounds__(NW * 64) void moe_align_kernel(
    const int32_t *__restrict__ topk_ids, int32_t *__restrict__ sorted_token_ids,
    int32_t *__restrict__ expert_ids, int32_t *__restrict__ num_tokens_post_padded, int n,
    int num_experts, int block_m, int pad_to, int max_padded, int max_blocks, int id_bits) {
    extern __shared__ int32_t smem[];
    int32_t *offs = smem;                          // [E+1] exclusive prefix of padded counts
    int32_t *padc = smem + (num_experts + 1);      // [E]   padded count per expert
    int32_t *wbase = smem + (2 * num_experts + 1);  // [NW][E] per-wave counts, then running bases
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    constexpr int NT = NW * 64;
    const int E = num_experts;

    for (int i = tid; i < NW * E; i += NT) wbase[i] = 0;
    __syncthreads();

    // contiguous slice per wave, a multiple of 64 ids so groups never straddle waves
    const int per_wave = (n + NT - 1) / NT * 64;
    const int beg = wave * per_wave;
    const int end = min(n, beg + per_wave);
    int32_t *mine = wbase + wave * E;
    for (int i = beg + lane; i < end; i += 64) {
        int e = topk_ids[i];
        if (e >= 0 && e < E) atomicAdd(mine + e, 1);
    }
    __syncthreads();

    // per expert: counts of the waves -> exclusive bases; padded total of the expert
    for (int e = tid; e < E; e += NT) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            int c = wbase[w * E + e];
            wbase[w * E + e] = run;
            run += c;
        }
        padc[e] = (run + pad_to - 1) / pad_to * pad_to;
    }
    __syncthreads();

    // exclusive prefix over experts by wave 0: serial inside a lane's chunk, shuffle scan across
    if (wave == 0) {
        const int chunk = (E + 63) >> 6;
        const int b = lane * chunk;
        int local = 0;
        for (int j = 0; j < chunk; ++j)
            if (b + j < E) local += padc[b + j];
        int incl = local;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int v = __shfl_up(incl, d, 64);
            if (lane >= d) incl += v;
        }
        int run = incl - local;
        for (int j = 0; j < chunk; ++j)
            if (b + j < E) {
                offs[b + j] = run;
                run += padc[b + j];
            }
        if (lane == 63) offs[E] = incl;  // lane 63's inclusive sum is the grand total
    }
    __syncthreads();
    const int total = offs[E];
    if (tid == 0) num_tokens_post_padded[0] = total;

    for (int i = tid; i < max_padded; i += NT) sorted_token_ids[i] = -1;
    for (int j = tid; j < max_blocks; j += NT) {
        const int row = j * block_m;
        int owner = E - 1;
        if (row < total) {
            int lo = 0, hi = E - 1;
            while (lo < hi) {
                int mid = (lo + hi + 1) >> 1;
                if (offs[mid] <= row) lo = mid;
                else hi = mid - 1;
            }
            owner = lo;
        }
        expert_ids[j] = owner;
    }
    __syncthreads();  // the -1 fill is complete before any pair id lands on top of it

    for (int i0 = beg; i0 < end; i0 += 64) {
        const int i = i0 + lane;
        int e = (i < end) ? topk_ids[i] : -1;
        const bool valid = e >= 0 && e < E;
        unsigned long long peers = __ballot(valid);
        for (int b = 0; b < id_bits; ++b) {
            const bool bit = (e >> b) & 1;
            const unsigned long long set = __ballot(bit);
            peers &= bit ? set : ~set;
        }
        if (valid) {
            const int rank = __popcll(peers & ((1ull << lane) - 1ull));
            const int cnt = __popcll(peers);
            const int base = mine[e];
            sorted_token_ids[offs[e] + base + rank] = i;
            if (rank == cnt - 1) mine[e] = base + cnt;  // one writer per group, after all reads
        }
    }
}

// ---- many ids: the same sort spread over workgroups, three launches.
//   count:   workgroup g histograms ids [g S, (g+1) S) -> counts[g][e]
//   scan:    one workgroup turns counts[.][e] into exclusive bases over the workgroups, writes the
//            per-expert totals cnt[e], the padded exclusive prefix offs[0..E], the total and expert_ids
//   scatter: workgroup g sorts its slice as the single-workgroup kernel does (per-wave histogram,
//            ballot ranks) and writes pair id i to offs[e] + counts[g][e] + base of its wave + rank;
//            it also writes -1 to the padding slots of its share of the output (a slot is padding if
//            it lies at or behind cnt[e] inside its expert's padded range, or behind the total), so
//            no slot is written twice and no order between workgroups is needed.
// Slices are contiguous and ascending in g, waves inside a slice likewise: the order inside an expert is
// ascending pair id, bit for bit what the single workgroup produces.
constexpr int kSliceIds = 8192;       // ids per workgroup
constexpr int kSingleMaxIds = 16384;  // up to here one workgroup is faster than three launches

struct AlignScratch {
    int32_t *counts;  // [G][E]
    int32_t *offs;    // [E + 1]
    int32_t *cnt;     // [E]
};

__global__ __launch_bounds__(1024) void align_count_kernel(const int32_t *__restrict__ topk_ids, int n, int E,
                                                           int32_t *__restrict__ counts) {
    extern __shared__ int32_t smem[];
    const int tid = threadIdx.x, g = blockIdx.x;
    for (int e = tid; e < E; e += 1024) smem[e] = 0;
    __syncthreads();
    const int beg = g * kSliceIds, end = min(n, beg + kSliceIds);
    for (int i = beg + tid; i < end; i += 1024) {
        const int e = topk_ids[i];
        if (e >= 0 && e < E) atomicAdd(smem + e, 1);
    }
    __syncthreads();
    for (int e = tid; e < E; e += 1024) counts[g * E + e] = smem[e];
}

__global__ __launch_bounds__(1024) void align_scan_kernel(AlignScratch sc, int G, int E, int block_m, int pad_to,
                                                          int max_blocks, int32_t *__restrict__ expert_ids,
                                                          int32_t *__restrict__ num_tokens_post_padded) {
    extern __shared__ int32_t smem[];
    int32_t *offs = smem;            // [E + 1]
    int32_t *padc = smem + (E + 1);  // [E]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int e = tid; e < E; e += 1024) {
        int run = 0;
        for (int g = 0; g < G; ++g) {
            const int c = sc.counts[g * E + e];
            sc.counts[g * E + e] = run;
            run += c;
        }
        sc.cnt[e] = run;
        padc[e] = (run + pad_to - 1) / pad_to * pad_to;
    }
    __syncthreads();
    if (wave == 0) {  // exclusive prefix over experts, as in the single-workgroup kernel
        const int chunk = (E + 63) >> 6;
        const int b = lane * chunk;
        int local = 0;
        for (int j = 0; j < chunk; ++j)
            if (b + j < E) local += padc[b + j];
        int incl = local;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int v = __shfl_up(incl, d, 64);
            if (lane >= d) incl += v;
        }
        int run = incl - local;
        for (int j = 0; j < chunk; ++j)
            if (b + j < E) {
                offs[b + j] = run;
                run += padc[b + j];
            }
        if (lane == 63) offs[E] = incl;
    }
    __syncthreads();
    const int total = offs[E];
    if (tid == 0) num_tokens_post_padded[0] = total;
    for (int e = tid; e <= E; e += 1024) sc.offs[e] = offs[e];
    for (int j = tid; j < max_blocks; j += 1024) {
        const int row = j * block_m;
        int owner = E - 1;
        if (row < total) {
            int lo = 0, hi = E - 1;
            while (lo < hi) {
                int mid = (lo + hi + 1) >> 1;
                if (offs[mid] <= row) lo = mid;
                else hi = mid - 1;
            }
            owner = lo;
        }
        expert_ids[j] = owner;
    }
}

template <int NW>
__global__ __launch_bounds__(NW * 64) void align_scatter_kernel(const int32_t *__restrict__ topk_ids,
                                                                int32_t *__restrict__ sorted_token_ids,
                                                                AlignScratch sc, int n, int E, int max_padded,
                                                                int id_bits) {
    extern __shared__ int32_t smem[];
    int32_t *offs = smem;                  // [E + 1]
    int32_t *cnt = smem + (E + 1);         // [E]
    int32_t *wbase = smem + (2 * E + 1);   // [NW][E] per-wave counts, then running bases
    constexpr int NT = NW * 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = blockIdx.x, G = gridDim.x;
    for (int e = tid; e <= E; e += NT) offs[e] = sc.offs[e];
    for (int e = tid; e < E; e += NT) cnt[e] = sc.cnt[e];
    for (int i = tid; i < NW * E; i += NT) wbase[i] = 0;
    __syncthreads();

    // this workgroup's share of the -1 fill
    {
        const int total = offs[E];
        const int per = (max_padded + G - 1) / G;
        const int pend = min(max_padded, (g + 1) * per);
        for (int pos = g * per + tid; pos < pend; pos += NT) {
            bool pad = pos >= total;
            if (!pad) {
                int lo = 0, hi = E - 1;
                while (lo < hi) {
                    int mid = (lo + hi + 1) >> 1;
                    if (offs[mid] <= pos) lo = mid;
                    else hi = mid - 1;
                }
                pad = pos - offs[lo] >= cnt[lo];
            }
            if (pad) sorted_token_ids[pos] = -1;
        }
    }

    // the slice, one contiguous run of a multiple of 64 ids per wave
    const int sbeg = g * kSliceIds, send = min(n, sbeg + kSliceIds);
    constexpr int per_wave = kSliceIds / NW;
    const int beg = sbeg + wave * per_wave;
    const int end = min(send, beg + per_wave);
    int32_t *mine = wbase + wave * E;
    for (int i = beg + lane; i < end; i += 64) {
        const int e = topk_ids[i];
        if (e >= 0 && e < E) atomicAdd(mine + e, 1);
    }
    __syncthreads();
    for (int e = tid; e < E; e += NT) {
        int run = offs[e] + sc.counts[g * E + e];  // first slot of this workgroup's ids of expert e
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const int c = wbase[w * E + e];
            wbase[w * E + e] = run;
            run += c;
        }
    }
    __syncthreads();
    for (int i0 = beg; i0 < end; i0 += 64) {
        const int i = i0 + lane;
        const int e = (i < end) ? topk_ids[i] : -1;
        const bool valid = e >= 0 && e < E;
        unsigned long long peers = __ballot(valid);
        for (int b = 0; b < id_bits; ++b) {
            const bool bit = (e >> b) & 1;
            const unsigned long long set = __ballot(bit);
            peers &= bit ? set : ~set;
        }
        if (valid) {
            const int rank = __popcll(peers & ((1ull << lane) - 1ull));
            const int c = __popcll(peers);
            const int base = mine[e];
            sorted_token_ids[base + rank] = i;
            if (rank == c - 1) mine[e] = base + c;  // one writer per group, after all reads
        }
    }
}


// Scratch of the entry point that allocates nothing (pmoe_moe_align_static): counts[G][E], offs[E + 1],
// cnt[E] of the multi-workgroup sort for up to kStaticMaxIds ids and kMaxExperts experts, 520 KB held by
// every device the library runs on until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress; kernels get the address that call returns.
constexpr int kStaticMaxIds = PMOE_ALIGN_STATIC_MAX_IDS;
constexpr size_t kStaticWords = (size_t)(kStaticMaxIds / kSliceIds) * kMaxExperts + 2 * kMaxExperts + 1;
static __device__ __align__(256) int32_t scratch[kStaticWords];

int id_bits_for(int num_experts) {
    int id_bits = 1;
    while ((1 << id_bits) < num_experts) ++id_bits;
    return id_bits;
}

int validate(const int32_t *topk_ids, const int32_t *sorted_token_ids, const int32_t *expert_ids,
             const int32_t *num_tokens_post_padded, int n, int num_experts, int block_m, int pad_to, int max_padded,
             int max_blocks) {
    PMOE_REQUIRE(num_experts > 0 && block_m > 0 && pad_to > 0, "moe_align: block_m, bpc and num_experts must be positive");
    PMOE_REQUIRE(num_experts <= kMaxExperts, "moe_align supports at most 1024 experts, got %d", num_experts);
    PMOE_REQUIRE(n >= 0 && max_padded >= 0 && max_blocks >= 0, "moe_align: negative size");
    PMOE_REQUIRE(pad_to % block_m == 0, "moe_align: pad_to must be a multiple of block_m");
    const long long need = ((long long)n + (long long)num_experts * (pad_to - 1) + pad_to - 1) / pad_to * pad_to;
    PMOE_REQUIRE(max_padded >= need, "moe_align: max_padded %d is smaller than the worst case %lld", max_padded, need);
    PMOE_REQUIRE((long long)max_blocks * block_m <= (long long)max_padded + block_m - 1,
                 "moe_align: max_blocks %d does not match max_padded %d", max_blocks, max_padded);
    PMOE_REQUIRE(sorted_token_ids && expert_ids && num_tokens_post_padded && (topk_ids || n == 0), "moe_align: null pointer");
    return PMOE_OK;
}

// One workgroup sorts everything.
int launch_single(const int32_t *topk_ids, int32_t *sorted_token_ids, int32_t *expert_ids,
                  int32_t *num_tokens_post_padded, int n, int num_experts, int block_m, int pad_to, int max_padded,
                  int max_blocks, hipStream_t s) {
    const int id_bits = id_bits_for(num_experts);
    if (num_experts <= 512) {
        constexpr int NW = 16;
        const size_t smem = sizeof(int32_t) * (size_t)(2 * num_experts + 1 + NW * num_experts);
        hipLaunchKernelGGL(moe_align_kernel<NW>, dim3(1), dim3(NW * 64), smem, s, topk_ids, sorted_token_ids,
                           expert_ids, num_tokens_post_padded, n, num_experts, block_m, pad_to, max_padded,
                           max_blocks, id_bits);
    } else {
        constexpr int NW = 8;
        const size_t smem = sizeof(int32_t) * (size_t)(2 * num_experts + 1 + NW * num_experts);
        hipLaunchKernelGGL(moe_align_kernel<NW>, dim3(1), dim3(NW * 64), smem, s, topk_ids, sorted_token_ids,
                           expert_ids, num_tokens_post_padded, n, num_experts, block_m, pad_to, max_padded,
                           max_blocks, id_bits);
    }
    return pmoe::check_launch("moe_align launch");
}

// The three launches of the multi-workgroup sort; `words` holds G * E + 2 E + 1 int32 of device scratch,
// every one of which is written before it is read.
int launch_multi(const int32_t *topk_ids, int32_t *sorted_token_ids, int32_t *expert_ids,
                 int32_t *num_tokens_post_padded, int n, int num_experts, int block_m, int pad_to, int max_padded,
                 int max_blocks, int32_t *words, hipStream_t s) {
    const int id_bits = id_bits_for(num_experts);
    const int G = (n + kSliceIds - 1) / kSliceIds;
    AlignScratch sc;
    sc.counts = words;
    sc.offs = sc.counts + (size_t)G * num_experts;
    sc.cnt = sc.offs + num_experts + 1;
    hipLaunchKernelGGL(align_count_kernel, dim3(G), dim3(1024), sizeof(int32_t) * num_experts, s, topk_ids, n,
                       num_experts, sc.counts);
    hipLaunchKernelGGL(align_scan_kernel, dim3(1), dim3(1024), sizeof(int32_t) * (2 * num_experts + 1), s, sc, G,
                       num_experts, block_m, pad_to, max_blocks, expert_ids, num_tokens_post_padded);
    if (num_experts <= 512) {
        constexpr int NW = 16;
        hipLaunchKernelGGL(align_scatter_kernel<NW>, dim3(G), dim3(NW * 64),
                           sizeof(int32_t) * (size_t)(2 * num_experts + 1 + NW * num_experts), s, topk_ids,
                           sorted_token_ids, sc, n, num_experts, max_padded, id_bits);
    } else {
        constexpr int NW = 8;
        hipLaunchKernelGGL(align_scatter_kernel<NW>, dim3(G), dim3(NW * 64),
                           sizeof(int32_t) * (size_t)(2 * num_experts + 1 + NW * num_experts), s, topk_ids,
                           sorted_token_ids, sc, n, num_experts, max_padded, id_bits);
    }
    return pmoe::check_launch("moe_align launch");
}

// Device address of `scratch` on the current device: every device holds its own copy of the array at
// its own address, looked up once per device (with that device current) and kept.  `data` is one of the
// call's device pointers: the current device must be the one that holds it (the kernels run where the data
// is, and another device's copy of the array has another address), otherwise the call is rejected.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
int32_t *g_scratch_ptr[kMaxDevices] = {nullptr};

int static_scratch(const void *data, int32_t **out) {
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return pmoe::fail(PMOE_ERR_HIP, "moe_align_static: hipGetDevice: %s", hipGetErrorString(err));
    PMOE_REQUIRE(dev >= 0 && dev < kMaxDevices, "moe_align_static: device index %d out of range", dev);
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, data) == hipSuccess)
        PMOE_REQUIRE(attr.device == dev, "moe_align_static: the data lives on device %d but device %d is current", attr.device, dev);
    else
        (void)hipGetLastError();  // (a pointer the runtime does not know: nothing to compare)
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || p == nullptr)
            return pmoe::fail(PMOE_ERR_HIP, "moe_align_static: hipGetSymbolAddress: %s", hipGetErrorString(err));
        g_scratch_ptr[dev] = static_cast<int32_t *>(p);
    }
    *out = g_scratch_ptr[dev];
    return PMOE_OK;
}

}  // namespace

extern "C" size_t pmoe_moe_align_workspace_bytes(int n, int num_experts) {
    if (n <= kSingleMaxIds || num_experts <= 0 || num_experts > kMaxExperts) return 0;
    const size_t G = ((size_t)n + kSliceIds - 1) / kSliceIds;
    return sizeof(int32_t) * (G * (size_t)num_experts + 2 * (size_t)num_experts + 1);
}

extern "C" int pmoe_moe_align(const int32_t *topk_ids, int32_t *sorted_token_ids,
                              int32_t *expert_ids, int32_t *num_tokens_post_padded, int n,
                              int num_experts, int block_m, int pad_to, int max_padded,
                              int max_blocks, void *stream) {
    return pmoe_moe_align_ws(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded, n, num_experts, block_m,
                             pad_to, max_padded, max_blocks, nullptr, 0, stream);
}

extern "C" int pmoe_moe_align_ws(const int32_t *topk_ids, int32_t *sorted_token_ids, int32_t *expert_ids,
                                 int32_t *num_tokens_post_padded, int n, int num_experts, int block_m, int pad_to,
                                 int max_padded, int max_blocks, void *workspace, size_t workspace_bytes,
                                 void *stream) {
    if (int rc = validate(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded, n, num_experts, block_m,
                          pad_to, max_padded, max_blocks))
        return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t ws_need = pmoe_moe_align_workspace_bytes(n, num_experts);
    if (ws_need > 0 && workspace != nullptr && workspace_bytes >= ws_need) {
        PMOE_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 3) == 0, "moe_align: workspace must be 4-byte aligned");
        return launch_multi(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded, n, num_experts, block_m,
                            pad_to, max_padded, max_blocks, static_cast<int32_t *>(workspace), s);
    }
    return launch_single(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded, n, num_experts, block_m,
                         pad_to, max_padded, max_blocks, s);
}

extern "C" int pmoe_moe_align_static(const int32_t *topk_ids, int32_t *sorted_token_ids, int32_t *expert_ids,
                                     int32_t *num_tokens_post_padded, int n, int num_experts, int block_m,
                                     int pad_to, int max_padded, int max_blocks, void *stream) {
    if (int rc = validate(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded, n, num_experts, block_m,
                          pad_to, max_padded, max_blocks))
        return rc;
    PMOE_REQUIRE(n <= kStaticMaxIds, "moe_align_static: at most %d ids fit the built-in scratch, got %d", kStaticMaxIds, n);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n <= kSingleMaxIds)  // one workgroup sorts these in its LDS: no device scratch involved
        return launch_single(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded, n, num_experts, block_m,
                             pad_to, max_padded, max_blocks, s);
    int32_t *words = nullptr;
    if (int rc = static_scratch(topk_ids, &words)) return rc;
    return launch_multi(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded, n, num_experts, block_m,
                        pad_to, max_padded, max_blocks, words, s);
}
