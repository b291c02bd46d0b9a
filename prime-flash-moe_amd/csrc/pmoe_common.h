// Shared host-side helpers for the C-ABI entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/prime_moe_hip.h"
#include "../../include/prime_moe_hip_debug.h"

namespace pmoe {

// Thread-local message of the last failing call; read through pmoe_last_error().
char *error_buffer();
constexpr int kErrorBufferBytes = 512;

inline int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), kErrorBufferBytes, fmt, ap);
    va_end(ap);
    return code;
}

inline int check_launch(const char *what) {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(PMOE_ERR_HIP, "%s: %s", what, hipGetErrorString(err));
    return PMOE_OK;
}

#define PMOE_REQUIRE(cond, ...)                                   \
    do {                                                          \
        if (!(cond)) return ::pmoe::fail(PMOE_ERR_INVALID, __VA_ARGS__); \
    } while (0)

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace pmoe
