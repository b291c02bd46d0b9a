// Library-wide C-ABI entry points: version and the thread-local error message.
#include "pmoe_common.h"

namespace pmoe {
char *error_buffer() {
    static thread_local char buf[kErrorBufferBytes] = {0};
    return buf;
}
}  // namespace pmoe

extern "C" int pmoe_version(void) { return 1; }

extern "C" const char *pmoe_last_error(void) { return pmoe::error_buffer(); }

// Plain device copy of `bytes` bytes (a multiple of 16): a kernel of known traffic, used to scale the
// FETCH_SIZE / WRITE_SIZE counters of a counter-collection run of the fused kernels.
namespace {
__global__ __launch_bounds__(256) void copy_calibration_kernel(const uint4 *src, uint4 *dst, int64_t n16) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}
}  // namespace

// Fills the LDS of every CU with 0xff bytes (a NaN as bf16, as e4m3 and as e8m0): what a kernel that runs next
// reads from LDS it has not written itself.  A test aid: a copy into LDS that lands in the wrong place, or not at
// all, then shows as NaNs in the result instead of depending on what an earlier kernel left there.
namespace {
__global__ __launch_bounds__(1024) void poison_lds_kernel(int *sink) {
    __shared__ uint4 lds[160 * 1024 / 16];
    for (int i = threadIdx.x; i < 160 * 1024 / 16; i += 1024) lds[i] = make_uint4(~0u, ~0u, ~0u, ~0u);
    __syncthreads();
    if (lds[(threadIdx.x * 37) % (160 * 1024 / 16)].x != ~0u) sink[0] = 1;  // (keeps the stores alive)
}
}  // namespace

extern "C" int pmoe_poison_lds(int *scratch_word, void *stream) {
    PMOE_REQUIRE(scratch_word != nullptr, "poison_lds: a device word is needed");
    // one workgroup holds a CU's whole LDS, so the grid lands one on every CU; a few rounds for good measure
    hipLaunchKernelGGL(poison_lds_kernel, dim3(4 * 256), dim3(1024), 0, static_cast<hipStream_t>(stream), scratch_word);
    return pmoe::check_launch("poison_lds launch");
}

extern "C" int pmoe_copy_calibration(const void *src, void *dst, int64_t bytes, void *stream) {
    PMOE_REQUIRE(src && dst && bytes >= 0 && bytes % 16 == 0, "copy_calibration: bytes must be a multiple of 16");
    if (bytes == 0) return PMOE_OK;
    hipLaunchKernelGGL(copy_calibration_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), bytes / 16);
    return pmoe::check_launch("copy_calibration launch");
}
