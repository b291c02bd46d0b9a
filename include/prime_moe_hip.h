/*
 * prime_moe_hip.h -- C ABI of the gfx950 (MI355X) fused-MoE forward library.
 *
 * libprime_moe_hip.so exports exactly the native seam that the reference's torch
 * extension binds: the three `namespace pi` functions declared in
 * prime_moe/csrc/torch_interface.cpp:11-75 of the reference.  Differences are
 * mechanical: plain C linkage, `void*` in place of typed fp8/bf16 pointers and of
 * the stream handle (a hipStream_t), an int status in place of C++ exceptions
 * (0 = ok; on failure pmoe_last_error() holds the message), and a caller-provided
 * workspace in place of the per-call cudaMallocAsync/cudaFreeAsync of the reference
 * (fused_moe_bf16_kernel.cu:607,:730; fused_moe_mxfp8_kernel.cu:751,:863) so the
 * entry points allocate nothing and stay capturable in a HIP graph.
 *
 * All pointers are device pointers to contiguous, caller-owned memory.  Nothing
 * here synchronises the host: work is enqueued on `stream` and the grids are sized
 * from `sorted_num`; kernels read `num_tokens_post_padded` on the device.
 */
#ifndef PRIME_MOE_HIP_H
#define PRIME_MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PMOE_OK 0
#define PMOE_ERR_INVALID 1 /* argument rejected; nothing was launched */
#define PMOE_ERR_HIP 2     /* a HIP runtime call failed */

/* Library ABI version (bumped when a signature changes). */
int pmoe_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char *pmoe_last_error(void);

/*
 * moe_align -- replaces pi::moe_align (torch_interface.cpp:63-75; kernel
 * fused_moe_bf16_kernel.cu:853-928).
 * Counting sort of the n pair ids 0..n-1 by expert, each expert padded to a
 * multiple of pad_to (= block_m * bpc):
 *   sorted_token_ids[max_padded]  pair ids, -1 in padding and past the total
 *   expert_ids[max_blocks]        owner of each block_m rows, num_experts-1 past the total
 *   num_tokens_post_padded[1]     sum of padded counts
 * Within an expert the pair ids are ascending (the reference leaves the order to
 * an atomic race; ascending is one of its outcomes and makes the result unique).
 * Ids outside [0, num_experts) are skipped.  num_experts <= 1024 as in the
 * reference (fused_moe_bf16_kernel.cu:922-923).
 */
int pmoe_moe_align(const int32_t *topk_ids, int32_t *sorted_token_ids, int32_t *expert_ids,
                   int32_t *num_tokens_post_padded, int n, int num_experts, int block_m,
                   int pad_to, int max_padded, int max_blocks, void *stream);

/*
 * The same sort with scratch memory from the caller, which lets it spread over many
 * workgroups (three launches) when n is large; no counterpart in the reference, whose
 * kernel is one thread block for any n.  The query returns 0 for sizes the single
 * workgroup of pmoe_moe_align handles (then `workspace` may be null); with a null or too
 * small workspace the call falls back to that single workgroup.  Same output, bit for bit.
 */
size_t pmoe_moe_align_workspace_bytes(int n, int num_experts);
int pmoe_moe_align_ws(const int32_t *topk_ids, int32_t *sorted_token_ids, int32_t *expert_ids,
                      int32_t *num_tokens_post_padded, int n, int num_experts, int block_m,
                      int pad_to, int max_padded, int max_blocks, void *workspace,
                      size_t workspace_bytes, void *stream);

/*
 * The same sort for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc); no counterpart in the reference.
 * Takes what pmoe_moe_align takes and gives the same output, bit for bit, but the scratch of
 * the multi-workgroup sort lives in a device array built into the library (520 KB on every
 * device the library runs on, held until the process ends), so large inputs still spread
 * over many workgroups.  n > PMOE_ALIGN_STATIC_MAX_IDS is rejected (PMOE_ERR_INVALID).
 * Calls no hipMalloc / hipFree or any allocating routine; the first call on a device looks
 * up the array's address (hipGetSymbolAddress), so make that one outside a capture.
 * All calls on one device share the array: calls that overlap on one device (two streams,
 * two threads) race and must be serialised by the caller.
 */
#define PMOE_ALIGN_STATIC_MAX_IDS (1 << 20)
int pmoe_moe_align_static(const int32_t *topk_ids, int32_t *sorted_token_ids, int32_t *expert_ids,
                          int32_t *num_tokens_post_padded, int n, int num_experts, int block_m,
                          int pad_to, int max_padded, int max_blocks, void *stream);

/*
 * Workspace (bytes) the fused calls below need for a problem of this size.  The
 * caller allocates it on the device (any 256-byte aligned buffer) and passes it in.
 * The size does not depend on `split` (both values run the same kernels); the argument
 * is kept so that the query takes what the call takes.
 */
size_t pmoe_fused_moe_bf16_workspace_bytes(int M, int K, int N, int num_experts, int sorted_num,
                                           int top_k, int split);
size_t pmoe_fused_moe_mxfp8_workspace_bytes(int M, int K, int N, int num_experts,
                                            int sorted_num, int top_k, int split);

/*
 * fused_moe_bf16 -- replaces pi::fused_moe_bf16 (torch_interface.cpp:11-34; launcher
 * fused_moe_bf16_kernel.cu:930-964).
 *   x (M,K) bf16; w (E,N,K) bf16 with gate rows [0,N/2) and up rows [N/2,N);
 *   w2 (E,K,N/2) bf16; topk_weights flat fp32 indexed by pair id; out (M,K) bf16.
 *   out[t] (+)= sum over rows s of the schedule with sorted_token_ids[s]/top_k == t of
 *               topk_weights[p] * W2[e] . swiglu(W1[e] . x[t]),  e = expert_idxs[s/block_m].
 * split != 0: `out` is overwritten (the reference zeroes it itself and adds).
 * split == 0: the result is added to `out`; the caller pre-zeroes it.
 * Either way the work is done by the same up and down kernels with the activation in the
 * workspace; `split` selects only how the last kernel treats `out`.
 * block_n / warp_n / stages are validated exactly as the reference does and then
 * ignored (they size Blackwell thread blocks and smem rings); block_m must be 128,
 * bpc == cpc == 1, K % 128 == 0, N % 256 == 0.  Limits of this implementation, checked:
 * num_experts <= 1024 (as moe_align) and x smaller than 4 GiB.
 * The workspace is scratch of this one call: calls that may run at the same time need
 * their own.
 * A schedule that lists a pair id twice: inside one block the pair contributes once; in blocks
 * of different experts one of the two rows stands for the pair, which one is unspecified
 * (nothing faults, the rest of the output is unaffected).
 */
int pmoe_fused_moe_bf16(const void *x, const void *w, const void *w2, void *out,
                        const int32_t *sorted_token_ids, const int32_t *expert_idxs,
                        const int32_t *num_tokens_post_padded, const float *topk_weights,
                        int top_k, int M, int K, int N, int num_experts, int sorted_num,
                        int block_m, int block_n, int warp_n, int stages, int bpc, int cpc,
                        int split, void *workspace, size_t workspace_bytes, void *stream);

/*
 * fused_moe_mxfp8 -- replaces pi::fused_moe_mxfp8 (torch_interface.cpp:36-61; launcher
 * fused_moe_mxfp8_kernel.cu:944-1009).
 *   x (M,K) e4m3 + x_scales (M,K/32) e8m0 row major; w (E,N,K) e4m3 + w_scales in the
 *   128x4 blocked tiles [E][N/128][K/128][512]; w2 (E,K,N/2) e4m3 + w2_scales blocked
 *   [E][K/128][(N/2)/128][512].  The SwiGLU activation is requantised on chip to e4m3
 *   with one e8m0 scale per 32 elements along N/2 before the down projection.
 *   K % 256 == 0, N % 256 == 0, bpc == 1, block_m == 128; num_experts <= 1024 and x
 *   smaller than 4 GiB as for fused_moe_bf16.
 */
int pmoe_fused_moe_mxfp8(const void *x, const void *x_scales, const void *w, const void *w_scales,
                         const void *w2, const void *w2_scales, void *out,
                         const int32_t *sorted_token_ids, const int32_t *expert_idxs,
                         const int32_t *num_tokens_post_padded, const float *topk_weights,
                         int top_k, int M, int K, int N, int num_experts, int sorted_num,
                         int block_m, int block_n, int warp_n, int stages, int bpc, int split,
                         void *workspace, size_t workspace_bytes, void *stream);

/*
 * quantize_mx -- the step in front of fused_moe_mxfp8 (the reference leaves it to
 * the caller and specifies it in test/test_mxfp8.py:21-38): OCP-MX quantisation of a
 * row-major (rows, cols) bf16 matrix along cols, cols % 32 == 0.
 *   q (rows, cols) e4m3;  scales (rows, cols/32) e8m0 row major.
 * Uses the same device routine as the on-chip activation requantisation.
 */
int pmoe_quantize_mx(const void *src_bf16, void *q, void *scales, int64_t rows, int cols,
                     void *stream);

/*
 * route -- the step in front of moe_align, which the reference leaves to the caller ("routing
 * comes from your gate", README.md:147-149; its benchmark draws expert ids directly,
 * benchmark/benchmark.py:124-166): gate logits -> top-k + softmax -> moe_align, enqueued
 * back to back on `stream` with no host synchronisation.
 *   logits (n_tokens, num_experts) fp32 or bf16 (logits_dtype), row major; bias (num_experts)
 *   fp32 added to every row before the selection, or null.
 *   topk_ids (n_tokens, top_k) int32: experts of the top_k largest values, largest first, ties
 *   to the lower index, NaN above every number; topk_weights (n_tokens, top_k) fp32: softmax
 *   over the selected values.  top_k <= min(32, num_experts), num_experts <= 1024.
 *   sorted_token_ids / expert_ids / num_tokens_post_padded and the sizes that follow are those
 *   of pmoe_moe_align_ws for n = n_tokens * top_k (workspace from
 *   pmoe_moe_align_workspace_bytes(n, num_experts)); with sorted_token_ids == NULL only the
 *   top-k and the weights are computed.
 */
#define PMOE_DTYPE_F32 0
#define PMOE_DTYPE_BF16 1
int pmoe_route(const void *logits, int logits_dtype, const float *bias, int32_t *topk_ids,
               float *topk_weights, int32_t *sorted_token_ids, int32_t *expert_ids,
               int32_t *num_tokens_post_padded, int n_tokens, int num_experts, int top_k,
               int block_m, int pad_to, int max_padded, int max_blocks, void *workspace,
               size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PRIME_MOE_HIP_H */
