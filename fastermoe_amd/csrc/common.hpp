// Shared host-side helpers of libfmoe_hip.so: error reporting, argument
// checks, launch checks.  gfx950 (wave64) only.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/fmoe_hip.h"

namespace fmoe {

constexpr int kWave = 64;

char *error_buffer();  // thread-local, 512 bytes

inline int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

#define FMOE_REQUIRE(cond, ...)                                   \
    do {                                                          \
        if (!(cond)) return ::fmoe::fail(FMOE_EINVAL, __VA_ARGS__); \
    } while (0)

#define FMOE_HIP_CHECK(expr)                                                   \
    do {                                                                       \
        hipError_t err__ = (expr);                                             \
        if (err__ != hipSuccess)                                               \
            return ::fmoe::fail(FMOE_EHIP, "%s failed: %s (%s:%d)", #expr,     \
                                hipGetErrorString(err__), __FILE__, __LINE__); \
    } while (0)

// after a kernel launch
#define FMOE_LAUNCH_CHECK() FMOE_HIP_CHECK(hipGetLastError())

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline int dtype_bytes(int dtype) {
    switch (dtype) {
        case FMOE_F32: return 4;
        case FMOE_BF16: return 2;
        case FMOE_F16: return 2;
        case FMOE_F64: return 8;
        default: return 0;
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace fmoe
