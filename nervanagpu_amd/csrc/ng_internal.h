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
// looks up this device's copy of the GEMM static scratch array (gemm.hip)
int gemm_static_scratch_setup(int device);

inline size_t dtype_size(int dtype)
{
    switch (dtype) {
    case NG_F16: return 2;
    case NG_F32: return 4;
    default: return 1;
    }
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// n / d for 0 <= n < 2^31 as a multiply and a shift.  With s = ceil(log2 d),
// mul = floor(2^(31+s) / d) + 1 fits 32 bits and the quotient is exact because
// the rounding excess n * (mul*d - 2^(31+s)) stays below 2^(31+s).
struct FastDiv {
    unsigned mul, shift;
    __host__ __device__ __forceinline__ unsigned div(unsigned n) const
    {
        return (unsigned)(((unsigned long long)n * mul) >> shift);
    }
    static FastDiv make(unsigned d)
    {
        unsigned s = 0;
        while ((1ull << s) < d) s++;
        FastDiv f;
        f.mul = (unsigned)((1ull << (31 + s)) / d + 1);
        f.shift = 31 + s;
        return f;
    }
};

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
