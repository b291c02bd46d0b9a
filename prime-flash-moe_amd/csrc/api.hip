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

extern "C" int pmoe_copy_calibration(const void *src, void *dst, int64_t bytes, void *stream) {
    PMOE_REQUIRE(src && dst && bytes >= 0 && bytes % 16 == 0, "copy_calibration: bytes must be a multiple of 16");
    if (bytes == 0) return PMOE_OK;
    hipLaunchKernelGGL(copy_calibration_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), bytes / 16);
    return pmoe::check_launch("copy_calibration launch");
}
