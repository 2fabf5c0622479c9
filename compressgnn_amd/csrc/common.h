// Shared host-side helpers of the device library: error reporting and launch checks.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "compressgnn_abi.h"

namespace cgnn {

void set_error(const char *fmt, ...);

inline int fail(int code, const char *what) {
    set_error("%s", what);
    return code;
}

// Called after every launch: hipGetLastError is cheap and does not synchronise.
inline int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(e));
        return CGNN_ELAUNCH;
    }
    return CGNN_OK;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

inline int pow2_ceil(int64_t x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}

constexpr int kBlock = 256;  // threads per workgroup: four wave64
constexpr int kWave = 64;

}  // namespace cgnn

#define CGNN_REQUIRE(cond, msg)                         \
    do {                                                \
        if (!(cond)) return ::cgnn::fail(CGNN_EINVAL, msg); \
    } while (0)
