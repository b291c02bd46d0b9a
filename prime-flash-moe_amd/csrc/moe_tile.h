// Device-side helpers shared by the fused-MoE kernels (gfx950, wave64): vector types, tile
// constants, bf16 / e4m3 / e8m0 conversions, SwiGLU, the blocked scale layout.
//
// MFMA shapes used by the kernels: v_mfma_f32_32x32x16_bf16 and v_mfma_scale_f32_32x32x64_f8f6f4
// (e4m3 operands, e8m0 scales).  Lane l supplies row l%32; accumulator register i of lane l is
// element (m = 8*(i/4) + 4*(l/32) + i%4, n = l%32).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pmoe {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kBlockRows = 128;  // sorted rows per block (= block_m)
constexpr int kWRows = 256;      // weight rows per tile

enum : int { DT_BF16 = 0, DT_FP8 = 1 };

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// Two fp32 -> one dword of two bf16 (round to nearest even), the hardware conversion of gfx950.
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 v = __builtin_convertvector(f32x2{lo, hi}, bf16x2);
    return __builtin_bit_cast(uint32_t, v);
}

// silu(gate) * up with the hardware exponential and reciprocal (about 1 ulp each, far inside bf16).
__device__ __forceinline__ float swiglu(float gate, float up) {
    return up * gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate));
}

// OCP-MX shared scale of a 32-block with absolute maximum `amax`:
// e = clamp(expfield(amax) - 8, 0, 254); returns e and 2^(127-e) (0 when e == 254).
__device__ __forceinline__ void mx_block_scale(float amax, uint32_t &e8m0, float &inv) {
    int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 8;
    e = max(0, min(254, e));
    e8m0 = (uint32_t)e;
    inv = __uint_as_float((uint32_t)(254 - e) << 23);
}

// four fp32 -> four e4m3 bytes (round to nearest even, saturating at +-448), packed little endian
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d, float inv) {
    a = __builtin_amdgcn_fmed3f(a * inv, -448.0f, 448.0f);
    b = __builtin_amdgcn_fmed3f(b * inv, -448.0f, 448.0f);
    c = __builtin_amdgcn_fmed3f(c * inv, -448.0f, 448.0f);
    d = __builtin_amdgcn_fmed3f(d * inv, -448.0f, 448.0f);
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
    return (uint32_t)w;
}

// Byte offset of the 4-scale dword of weight row `row` for K tile `kt` (128 wide) in the blocked
// scale layout [row/128][kt][512 B]; inside a tile: (row%32)*16 + ((row%128)/32)*4.
__device__ __forceinline__ int64_t blocked_scale_off(int row, int kt, int n_ktiles) {
    return ((int64_t)(row >> 7) * n_ktiles + kt) * 512 + ((row & 31) << 4) + (((row >> 5) & 3) << 2);
}

}  // namespace pmoe
