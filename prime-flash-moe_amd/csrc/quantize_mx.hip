// OCP-MX quantiser for row-major bf16 matrices: e4m3 values + one e8m0 scale per 32 columns.
// Specification: test/test_mxfp8.py:21-38 of the reference (the caller-side step in front of
// fused_moe_mxfp8).  Shares mx_block_scale / pack4_e4m3 with the on-chip activation requantiser.
#include <algorithm>

#include "moe_tile.h"
#include "pmoe_common.h"

namespace {

using namespace pmoe;

// One lane quantises 8 consecutive columns (16 bytes in, 8 bytes out); the 4 lanes of a 32-block
// combine their maxima with two DPP-class shuffles.
__global__ __launch_bounds__(256) void quantize_mx_kernel(const uint4 *__restrict__ src,
                                                          uint2 *__restrict__ q,
                                                          uint8_t *__restrict__ scales,
                                                          int64_t n_groups8) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t rounds = (n_groups8 + stride - 1) / stride;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (int64_t it = 0; it < rounds; ++it, i += stride) {
        const bool live = i < n_groups8;  // n_groups8 % 4 == 0, so a block's 4 lanes agree
        uint4 raw = live ? src[i] : make_uint4(0, 0, 0, 0);
        const uint32_t wv[4] = {raw.x, raw.y, raw.z, raw.w};
        float v[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = bf16_bits_to_f32(wv[j] & 0xffffu);
            v[2 * j + 1] = bf16_bits_to_f32(wv[j] >> 16);
        }
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
        amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
        uint32_t e8;
        float inv;
        mx_block_scale(amax, e8, inv);
        if (live) {
            uint2 o;
            o.x = pack4_e4m3(v[0], v[1], v[2], v[3], inv);
            o.y = pack4_e4m3(v[4], v[5], v[6], v[7], inv);
            q[i] = o;
            if ((i & 3) == 0) scales[i >> 2] = (uint8_t)e8;
        }
    }
}

}  // namespace

extern "C" int pmoe_quantize_mx(const void *src_bf16, void *q, void *scales, int64_t rows, int cols,
                                void *stream) {
    PMOE_REQUIRE(rows >= 0 && cols > 0 && cols % 32 == 0, "quantize_mx: cols (%d) must be a positive multiple of 32", cols);
    if (rows == 0) return PMOE_OK;
    PMOE_REQUIRE(src_bf16 && q && scales, "quantize_mx: null pointer");
    const int64_t n8 = rows * cols / 8;
    const int blocks = (int)std::min<int64_t>((n8 + 255) / 256, 8192);
    hipLaunchKernelGGL(quantize_mx_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4 *>(src_bf16), static_cast<uint2 *>(q),
                       static_cast<uint8_t *>(scales), n8);
    return pmoe::check_launch("quantize_mx launch");
}
