// Router front-end for gfx950: gate logits -> top-k expert ids + softmax weights, followed by moe_align.
//
// The reference leaves routing to the caller ("routing comes from your gate", README.md:147-149; its
// benchmark draws ids directly, benchmark/benchmark.py:124-166) and starts at moe_align.  This is the
// step in front of it, on the same stream, without a host synchronisation:
//   topk_ids[t, r]     = index of the r-th largest of logits[t, :] (+ bias), ties to the lower index,
//                        NaN above every number (the order torch.topk documents);
//   topk_weights[t, :] = softmax over the top_k selected values, fp32
//   then the moe_align sort of the T * top_k ids (same kernels, same bits as pmoe_moe_align_ws).
//
// One wave per token.  Lane l holds experts l, l + 64, l + 128, ... (EPL of them) as order-preserving
// 32-bit keys; every round each lane offers its best (key, index) as one 64-bit word
// key << 32 | ~index, a six-step xor butterfly leaves the maximum in all lanes (largest key, and
// among equal keys the smallest index), and the owner retires that element.  The softmax of the
// top_k winners is computed redundantly by every lane from the winners' values.
#include "pmoe_common.h"

extern "C" int pmoe_moe_align_ws(const int32_t *, int32_t *, int32_t *, int32_t *, int, int, int, int, int, int, void *,
                                 size_t, void *);

namespace {

constexpr int kMaxTopK = 32;

__device__ __forceinline__ float load_logit(const float *p, int64_t i) { return p[i]; }
__device__ __forceinline__ float load_logit(const uint16_t *p, int64_t i) { return __uint_as_float((uint32_t)p[i] << 16); }

// Monotone map float -> uint32 (a < b <=> key(a) < key(b)); -0 counts as +0, NaN lands above +inf.
__device__ __forceinline__ uint32_t order_key(float v) {
    v += 0.0f;  // -0 -> +0
    uint32_t u = __float_as_uint(v);
    if (v != v) u = 0x7fffffffu;  // every NaN: the largest positive pattern
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    const uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

template <int EPL, typename T>
__global__ __launch_bounds__(256) void route_topk_kernel(const T *__restrict__ logits, const float *__restrict__ bias,
                                                         int32_t *__restrict__ topk_ids,
                                                         float *__restrict__ topk_weights, int n_tokens, int E,
                                                         int top_k) {
    const int lane = threadIdx.x & 63;
    const int t = (int)((blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6);
    if (t >= n_tokens) return;
    uint32_t key[EPL];
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
        const int e = lane + 64 * j;
        key[j] = 0u;  // below every real key: never selected before a real element
        if (e < E) {
            float v = load_logit(logits, (int64_t)t * E + e);
            if (bias != nullptr) v += bias[e];
            key[j] = order_key(v);
        }
    }
    float my_val = 0.f;  // lane r keeps the value of winner r
    int my_id = 0;
    for (int r = 0; r < top_k; ++r) {
        uint64_t best = 0;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            const uint32_t e = (uint32_t)(lane + 64 * j);
            const uint64_t c = ((uint64_t)key[j] << 32) | (uint32_t)~e;
            best = c > best ? c : best;
        }
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t lo = __shfl_xor((uint32_t)best, d, 64), hi = __shfl_xor((uint32_t)(best >> 32), d, 64);
            const uint64_t o = ((uint64_t)hi << 32) | lo;
            best = o > best ? o : best;
        }
        const int win = (int)~(uint32_t)best;
#pragma unroll
        for (int j = 0; j < EPL; ++j)
            if (lane + 64 * j == win) key[j] = 0u;
        if (lane == r) {
            my_val = key_value((uint32_t)(best >> 32));
            my_id = win;
        }
    }
    // softmax over the winners: lanes 0 .. top_k - 1 hold them, winner 0 is the maximum
    const float vmax = __shfl(my_val, 0, 64);
    float ex = lane < top_k ? expf(my_val - vmax) : 0.f;
    float sum = ex;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) sum += __shfl_xor(sum, d, 64);
    if (lane < top_k) {
        topk_ids[(int64_t)t * top_k + lane] = my_id;
        topk_weights[(int64_t)t * top_k + lane] = ex / sum;
    }
}

template <typename T>
int launch_topk(const T *logits, const float *bias, int32_t *topk_ids, float *topk_weights, int n_tokens, int E,
                int top_k, hipStream_t s) {
    const dim3 grid((unsigned)((n_tokens + 3) / 4)), block(256);  // four tokens (waves) per workgroup
    const int epl = (E + 63) / 64;
#define PMOE_ROUTE_CASE(N)                                                                                        \
    hipLaunchKernelGGL((route_topk_kernel<N, T>), grid, block, 0, s, logits, bias, topk_ids, topk_weights, n_tokens, \
                       E, top_k)
    if (epl <= 1) PMOE_ROUTE_CASE(1);
    else if (epl <= 2) PMOE_ROUTE_CASE(2);
    else if (epl <= 4) PMOE_ROUTE_CASE(4);
    else if (epl <= 8) PMOE_ROUTE_CASE(8);
    else PMOE_ROUTE_CASE(16);
#undef PMOE_ROUTE_CASE
    return pmoe::check_launch("route_topk launch");
}

}  // namespace

extern "C" int pmoe_route(const void *logits, int logits_dtype, const float *bias, int32_t *topk_ids,
                          float *topk_weights, int32_t *sorted_token_ids, int32_t *expert_ids,
                          int32_t *num_tokens_post_padded, int n_tokens, int num_experts, int top_k, int block_m,
                          int pad_to, int max_padded, int max_blocks, void *workspace, size_t workspace_bytes,
                          void *stream) {
    PMOE_REQUIRE(n_tokens >= 0, "route: negative token count");
    PMOE_REQUIRE(num_experts > 0 && num_experts <= 1024, "route supports 1..1024 experts, got %d", num_experts);
    PMOE_REQUIRE(top_k > 0 && top_k <= kMaxTopK && top_k <= num_experts,
                 "route: top_k must be in 1..min(%d, num_experts), got %d", kMaxTopK, top_k);
    PMOE_REQUIRE(logits_dtype == PMOE_DTYPE_F32 || logits_dtype == PMOE_DTYPE_BF16, "route: logits must be fp32 or bf16");
    PMOE_REQUIRE((int64_t)n_tokens * top_k < (1ll << 31), "route: too many (token, slot) pairs");
    PMOE_REQUIRE(topk_ids && topk_weights && (logits || n_tokens == 0), "route: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n_tokens > 0) {
        const int rc = logits_dtype == PMOE_DTYPE_F32
                           ? launch_topk(static_cast<const float *>(logits), bias, topk_ids, topk_weights, n_tokens,
                                         num_experts, top_k, s)
                           : launch_topk(static_cast<const uint16_t *>(logits), bias, topk_ids, topk_weights, n_tokens,
                                         num_experts, top_k, s);
        if (rc != PMOE_OK) return rc;
    }
    if (sorted_token_ids == nullptr) return PMOE_OK;  // top-k and weights only
    return pmoe_moe_align_ws(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_padded, n_tokens * top_k,
                             num_experts, block_m, pad_to, max_padded, max_blocks, workspace, workspace_bytes, stream);
}
