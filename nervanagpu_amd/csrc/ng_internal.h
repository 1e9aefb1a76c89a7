// Internal declarations shared by the translation units of libnervana_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "../../include/nervana_hip.h"

namespace ng {

// records a message for ng_last_error() and returns a non-zero code
int fail(int code, const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);
int device_cu_count();

inline size_t dtype_size(int dtype)
{
    switch (dtype) {
    case NG_F16: return 2;
    case NG_F32: return 4;
    default: return 1;
    }
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace ng

#define NG_HIP(expr)                                                   \
    do {                                                               \
        hipError_t ng_e_ = (expr);                                     \
        if (ng_e_ != hipSuccess) return ::ng::hip_fail(ng_e_, #expr);  \
    } while (0)

#define NG_CHECK_LAUNCH(what)                                          \
    do {                                                               \
        hipError_t ng_e_ = hipGetLastError();                          \
        if (ng_e_ != hipSuccess) return ::ng::hip_fail(ng_e_, what);   \
    } while (0)
