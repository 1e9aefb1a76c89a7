// Stand-in for <hip/hip_runtime.h> that lets the kernel sources of nervanagpu_amd/csrc be compiled
// for the HOST and run lane by lane on the CPU (tests/emu/emu_runtime.cpp): every thread of a
// workgroup is a fiber, workgroup barriers and wavefront-wide instructions (MFMA, transposing LDS
// reads, readlane, shuffles) are rendezvous points between fibers, buffer descriptors are plain
// pointers with the hardware's out-of-range rule, and loads that write LDS directly are queued and
// land either at once or only when the issuing wavefront's s_waitcnt covers them.
//
// Test infrastructure only: nothing in the product includes this file.  It checks index
// arithmetic, tile layouts, barriers and wait counts of the kernels without a GPU; it says
// nothing about speed.
#pragma once
#define NG_HOST_EMULATION 1

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <math.h>
using std::isfinite;
using std::isinf;
using std::isnan;

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __shared__ static
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) x

struct dim3 {
    unsigned x, y, z;
    constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint2 { unsigned x, y; };
struct uint4 { unsigned x, y, z, w; };
static inline uint2 make_uint2(unsigned x, unsigned y) { return uint2{x, y}; }

typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
typedef struct emu_stream_t* hipStream_t;
typedef struct emu_event_t* hipEvent_t;
enum { hipEventDisableTiming = 2, hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2 };
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emulated runtime"; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
template <class T> inline hipError_t hipGetSymbolAddress(void** p, T& sym) { *p = (void*)&sym; return hipSuccess; }
inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) { *e = nullptr; return hipSuccess; }
inline hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) { return hipSuccess; }
inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
void* emu_alloc(size_t bytes);     // 256-byte aligned, known to the access check
void emu_free(void* p);
template <class T> inline hipError_t hipMalloc(T** p, size_t n) { *p = (T*)emu_alloc(n); return hipSuccess; }
inline hipError_t hipFree(void* p) { emu_free(p); return hipSuccess; }
inline hipError_t hipMemcpy(void* d, const void* s, size_t n, int) { std::memcpy(d, s, n); return hipSuccess; }

namespace emu {

struct Lane {
    dim3 tid;
    int lane, wave;
};
extern Lane* cur;                 // the fiber that is running
extern dim3 g_grid, g_block, g_bidx;

void wg_sync();                   // __syncthreads
// rendezvous of the live lanes of the current wavefront; returns the 64 exchange slots
// (64 bytes each) of this rendezvous: write your own before, read any after
char* wave_exchange_begin();      // slots to deposit into
void wave_exchange_sync();        // all lanes have deposited
void launch(dim3 grid, dim3 block, const std::function<void()>& body, const char* name = nullptr);

// vector-memory operations of the current wavefront that s_waitcnt vmcnt counts
void vmem_issue(char* lds_dst, const void* src16);   // 16 bytes to LDS (src16 == nullptr: zeros)
void vmem_issue_plain();                             // a load into registers or a store
void vmem_wait(int outstanding);

}  // namespace emu

#define threadIdx (emu::cur->tid)
#define blockIdx (emu::g_bidx)
#define gridDim (emu::g_grid)
#define blockDim (emu::g_block)
#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
    emu::launch((grid), (block), [=]() { kernel(__VA_ARGS__); }, __PRETTY_FUNCTION__)

inline void __syncthreads() { emu::wg_sync(); }

#define NG_EMU_MINMAX(T)                                   \
    inline T min(T a, T b) { return b < a ? b : a; }       \
    inline T max(T a, T b) { return a < b ? b : a; }
NG_EMU_MINMAX(int) NG_EMU_MINMAX(unsigned) NG_EMU_MINMAX(long) NG_EMU_MINMAX(unsigned long)
NG_EMU_MINMAX(long long) NG_EMU_MINMAX(unsigned long long) NG_EMU_MINMAX(float) NG_EMU_MINMAX(double)
#undef NG_EMU_MINMAX

inline unsigned __float_as_uint(float f) { unsigned u; std::memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(unsigned u) { float f; std::memcpy(&f, &u, 4); return f; }
inline float __uint2float_rn(unsigned u) { return (float)u; }
inline float __builtin_amdgcn_rcpf(float x) { return 1.0f / x; }
inline float __builtin_amdgcn_sqrtf(float x) { return std::sqrt(x); }
inline int __shfl_xor(int v, int mask, int width);
inline float __shfl_xor(float v, int mask, int width);

// ---- scheduling hints and counters that need no emulation -------------------------------
inline void __builtin_amdgcn_sched_barrier(int) {}
inline void __builtin_amdgcn_sched_group_barrier(int, int, int) {}
// The lanes of a wavefront run in lockstep on the hardware; here they are separate fibers, so
// the one place the kernels lean on lockstep (a wavefront's private LDS staging: write, fence +
// wave barrier, read what the other lanes wrote) must be a real rendezvous.
inline void __builtin_amdgcn_wave_barrier() { emu::wave_exchange_begin(); emu::wave_exchange_sync(); }
inline void __builtin_amdgcn_fence(int, const char*) {}
// imm: vmcnt in bits 3:0 and 15:14 (the LDS / scalar counter needs no emulation: LDS accesses
// of a fiber are immediate)
inline void __builtin_amdgcn_s_waitcnt(int imm) { emu::vmem_wait((imm & 15) | (((imm >> 14) & 3) << 4)); }

// the kernels only read values that are uniform over the wavefront through readfirstlane
inline int __builtin_amdgcn_readfirstlane(int v) { return v; }
inline int __builtin_amdgcn_readlane(int v, int src_lane)
{
    char* slots = emu::wave_exchange_begin();
    std::memcpy(slots + 64 * emu::cur->lane, &v, 4);
    emu::wave_exchange_sync();
    int r;
    std::memcpy(&r, slots + 64 * (src_lane & 63), 4);
    return r;
}
inline int __shfl_xor(int v, int mask, int /*width*/)
{
    char* slots = emu::wave_exchange_begin();
    std::memcpy(slots + 64 * emu::cur->lane, &v, 4);
    emu::wave_exchange_sync();
    int r;
    std::memcpy(&r, slots + 64 * ((emu::cur->lane ^ mask) & 63), 4);
    return r;
}
inline float __shfl_xor(float v, int mask, int /*width*/)
{
    char* slots = emu::wave_exchange_begin();
    std::memcpy(slots + 64 * emu::cur->lane, &v, 4);
    emu::wave_exchange_sync();
    float r;
    std::memcpy(&r, slots + 64 * ((emu::cur->lane ^ mask) & 63), 4);
    return r;
}

// ---- conversions --------------------------------------------------------------------------
typedef _Float16 emu_half2_t __attribute__((ext_vector_type(2)));
// fp32 -> fp16 toward zero: overflow saturates at the largest finite value, infinities and NaN stay
inline _Float16 emu_f32_to_f16_rz(float f)
{
    const unsigned u = __float_as_uint(f);
    const unsigned sign = (u >> 16) & 0x8000u, mag = u & 0x7FFFFFFFu;
    unsigned short h;
    if (mag >= 0x7F800000u) h = (unsigned short)(sign | 0x7C00u | (mag > 0x7F800000u ? 0x200u | ((mag >> 13) & 0x3FFu) : 0u));
    else if (mag >= 0x47800000u) h = (unsigned short)(sign | 0x7BFFu);                 // >= 65536: largest finite
    else if (mag >= 0x38800000u) h = (unsigned short)(sign | ((mag - 0x38000000u) >> 13));   // normal: drop 13 bits
    else if (mag < 0x33000000u) h = (unsigned short)sign;                                // below half the smallest subnormal... truncates to 0
    else {
        const int e = (int)(mag >> 23);                      // 102 .. 112: subnormal result
        const unsigned man = (mag & 0x7FFFFFu) | 0x800000u;
        h = (unsigned short)(sign | (man >> (126 - e)));     // value / 2^-24, truncated
    }
    _Float16 r;
    std::memcpy(&r, &h, 2);
    return r;
}
inline emu_half2_t __builtin_amdgcn_cvt_pkrtz(float a, float b)
{
    emu_half2_t r = {emu_f32_to_f16_rz(a), emu_f32_to_f16_rz(b)};
    return r;
}

// ---- buffer descriptors ----------------------------------------------------------------------
struct emu_rsrc_t { const char* base; unsigned num_records; };
typedef emu_rsrc_t __amdgpu_buffer_rsrc_t;
typedef unsigned emu_uint4_t __attribute__((ext_vector_type(4)));
typedef unsigned emu_uint2_t __attribute__((ext_vector_type(2)));
inline emu_rsrc_t __builtin_amdgcn_make_buffer_rsrc(void* base, short, int num_records, int)
{
    return emu_rsrc_t{(const char*)base, (unsigned)num_records};
}
// raw buffer access: a byte range that does not fit below num_records reads as zero / is dropped
inline bool emu_in_range(const emu_rsrc_t& r, int voffset, int soffset, unsigned bytes)
{
    const unsigned long off = (unsigned long)(unsigned)voffset + (unsigned long)(unsigned)soffset;
    return off + bytes <= (unsigned long)r.num_records;
}
void emu_check_access(const void* p, size_t bytes, const char* what);   // aborts on an address outside every registered buffer
inline emu_uint4_t __builtin_amdgcn_raw_buffer_load_b128(emu_rsrc_t r, int voffset, int soffset, int)
{
    emu::vmem_issue_plain();
    emu_uint4_t v = {0, 0, 0, 0};
    if (emu_in_range(r, voffset, soffset, 16)) {
        const char* p = r.base + (unsigned)voffset + (unsigned)soffset;
        emu_check_access(p, 16, "buffer load (16 bytes)");
        std::memcpy(&v, p, 16);
    }
    return v;
}
inline emu_uint2_t __builtin_amdgcn_raw_buffer_load_b64(emu_rsrc_t r, int voffset, int soffset, int)
{
    emu::vmem_issue_plain();
    emu_uint2_t v = {0, 0};
    if (emu_in_range(r, voffset, soffset, 8)) {
        const char* p = r.base + (unsigned)voffset + (unsigned)soffset;
        emu_check_access(p, 8, "buffer load (8 bytes)");
        std::memcpy(&v, p, 8);
    }
    return v;
}
inline void __builtin_amdgcn_raw_buffer_store_b128(emu_uint4_t v, emu_rsrc_t r, int voffset, int soffset, int)
{
    emu::vmem_issue_plain();
    if (emu_in_range(r, voffset, soffset, 16)) {
        char* p = const_cast<char*>(r.base) + (unsigned)voffset + (unsigned)soffset;
        emu_check_access(p, 16, "buffer store (16 bytes)");
        std::memcpy(p, &v, 16);
    }
}

namespace ng {
// the load that writes LDS directly (inline assembly in the product): lane l of the wavefront
// writes lds_base + 16 l; an out-of-range offset stores zeros
inline void buffer_load_chunk_to_lds(emu_rsrc_t rsrc, char* lds_base, unsigned byte_offset)
{
    const char* src = nullptr;
    if (emu_in_range(rsrc, (int)byte_offset, 0, 16)) {
        src = rsrc.base + byte_offset;
        emu_check_access(src, 16, "buffer load to LDS");
    }
    emu::vmem_issue(lds_base + 16 * emu::cur->lane, src);
}
}  // namespace ng

// ---- wavefront-wide LDS read and matrix instructions ----------------------------------------
typedef short emu_short4_t __attribute__((ext_vector_type(4)));
// Within each group of 16 lanes the 16 x 8-byte pieces the lanes point at form a 4 (k) x 16 (row)
// matrix of 16-bit values, lanes 4j..4j+3 supplying line k = j; lane i gets the four k values of row i.
inline emu_short4_t __builtin_amdgcn_ds_read_tr16_b64_v4i16(__attribute__((address_space(3))) emu_short4_t* lds_p)
{
    const char* p = (const char*)(lds_p);
    char* slots = emu::wave_exchange_begin();
    std::memcpy(slots + 64 * emu::cur->lane, &p, sizeof(p));
    emu::wave_exchange_sync();
    const int lane = emu::cur->lane, group = lane & ~15, i = lane & 15;
    emu_short4_t r;
    for (int k = 0; k < 4; k++) {
        const char* src;
        std::memcpy(&src, slots + 64 * (group + 4 * k + i / 4), sizeof(src));
        short v;
        std::memcpy(&v, src + 2 * (i % 4), 2);
        r[k] = v;
    }
    return r;
}

typedef _Float16 emu_half8_t __attribute__((ext_vector_type(8)));
typedef float emu_float16_t __attribute__((ext_vector_type(16)));
// D = A (32 x 16) . B (16 x 32) + C: lane l holds row / column l & 31 and contraction values
// 8 (l >> 5) .. + 7 of A / B, and column l & 31, rows 8 (v / 4) + 4 (l >> 5) + (v & 3) of C / D
inline emu_float16_t __builtin_amdgcn_mfma_f32_32x32x16_f16(emu_half8_t a, emu_half8_t b, emu_float16_t c, int, int, int)
{
    char* slots = emu::wave_exchange_begin();
    std::memcpy(slots + 64 * emu::cur->lane, &a, 16);
    std::memcpy(slots + 64 * emu::cur->lane + 16, &b, 16);
    emu::wave_exchange_sync();
    const int lane = emu::cur->lane, col = lane & 31;
    for (int v = 0; v < 16; v++) {
        const int row = 8 * (v / 4) + 4 * (lane >> 5) + (v & 3);
        float sum = 0.0f;
        for (int k = 0; k < 16; k++) {
            _Float16 av, bv;
            std::memcpy(&av, slots + 64 * (row + 32 * (k / 8)) + 2 * (k % 8), 2);
            std::memcpy(&bv, slots + 64 * (col + 32 * (k / 8)) + 16 + 2 * (k % 8), 2);
            sum += (float)av * (float)bv;
        }
        c[v] += sum;
    }
    return c;
}
// D = A (32 x 2) . B (2 x 32) + C with one fp32 value per lane and operand: contraction index l >> 5
inline emu_float16_t __builtin_amdgcn_mfma_f32_32x32x2f32(float a, float b, emu_float16_t c, int, int, int)
{
    char* slots = emu::wave_exchange_begin();
    std::memcpy(slots + 64 * emu::cur->lane, &a, 4);
    std::memcpy(slots + 64 * emu::cur->lane + 4, &b, 4);
    emu::wave_exchange_sync();
    const int lane = emu::cur->lane, col = lane & 31;
    for (int v = 0; v < 16; v++) {
        const int row = 8 * (v / 4) + 4 * (lane >> 5) + (v & 3);
        float sum = 0.0f;
        for (int k = 0; k < 2; k++) {
            float av, bv;
            std::memcpy(&av, slots + 64 * (row + 32 * k), 4);
            std::memcpy(&bv, slots + 64 * (col + 32 * k) + 4, 4);
            sum += av * bv;
        }
        c[v] += sum;
    }
    return c;
}
