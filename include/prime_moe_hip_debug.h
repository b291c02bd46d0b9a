/*
 * prime_moe_hip_debug.h -- profiling, tuning and test hooks of libprime_moe_hip.so.
 *
 * None of these has a counterpart in the reference and none belongs to the seam a maintainer binds
 * (that is prime_moe_hip.h).  They exist for this repository's benchmark and tests.  The settings
 * are per calling thread and change what the fused entry points enqueue: with a phase mask other
 * than PMOE_PHASE_ALL the output of pmoe_fused_moe_* is not the result of the op.
 */
#ifndef PRIME_MOE_HIP_DEBUG_H
#define PRIME_MOE_HIP_DEBUG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Profiling aid with no counterpart in the reference: restricts, for the calling thread, which
 * kernels the two fused entry points enqueue, so a harness can time one kernel of the pipeline
 * with events around the call.  Results are only meaningful with PMOE_PHASE_ALL (the default).
 */
#define PMOE_PHASE_PROLOGUE 1 /* inversion of the sorted order (the work lists are always built) */
#define PMOE_PHASE_UP 2       /* gate/up GEMM + SwiGLU */
#define PMOE_PHASE_DOWN 4     /* down GEMM */
#define PMOE_PHASE_FINALIZE 8 /* routing-weight reduction into bf16 `out` */
#define PMOE_PHASE_ALL 15
void pmoe_set_phase_mask(int mask);

/*
 * Tuning and test aid with no counterpart in the reference: the number of consecutive weight tiles
 * (1..16) one workgroup of the mxfp8 up and down kernels takes for its row tile, for the calling
 * thread; 0 (the default) lets every launch choose from its sizes.  The result does not depend on it.
 */
void pmoe_set_tiles_per_workgroup(int n);

/*
 * Second profiling aid without a counterpart in the reference: a plain device copy of `bytes`
 * bytes (multiple of 16) done by a kernel named copy_calibration_kernel.  Its known traffic
 * (bytes read, bytes written) scales the FETCH_SIZE / WRITE_SIZE hardware counters of a
 * counter-collection run that also contains the fused kernels.
 */
int pmoe_copy_calibration(const void *src, void *dst, int64_t bytes, void *stream);

/*
 * Test aid without a counterpart in the reference: fills the LDS of every CU with 0xff bytes (NaN as bf16, e4m3
 * and e8m0), so that a kernel launched next which reads LDS that its own copies did not fill (a direct-to-LDS copy
 * that landed in the wrong place) produces NaNs instead of whatever an earlier kernel left behind.
 * `scratch_word`: one int of device memory (written only if the fill itself misbehaves).
 */
int pmoe_poison_lds(int *scratch_word, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PRIME_MOE_HIP_DEBUG_H */
