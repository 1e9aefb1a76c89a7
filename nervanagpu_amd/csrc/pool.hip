// Pooling over a (J,T,R,S) window of a CHWN tensor: max and average, forward
// and backward.  Replaces {h,s}pool_max launched by NervanaGPU._execute_pool
// (nervanagpu/nervanagpu.py:789-818) and adds the average mode the reference
// only names (nervanagpu/nervanagpu.py:746, numpy definition
// benchmarks/pool_test.py:142-144).
//
// These are pure streaming kernels: every thread owns VEC consecutive images
// (16 bytes of the innermost N dimension) of one output or input element, so
// each wavefront instruction moves whole contiguous runs of the tensor.
//
// Backward is a gather, not a scatter: for each input element the kernel sums
// the errors of the windows that cover it (for max: those whose first maximum,
// in (j,t,r,s) scan order with strict '>', is this element, following
// kernels/sass/hpool_max.sass:264-282).  The result does not depend on
// execution order and every element of grad_I is written exactly once, so no
// zero fill and no atomics are needed.
#include "ng_internal.h"
#include "ng_device_common.h"

#include <algorithm>

namespace ng {

template <typename T, int VEC> struct Pack;
template <> struct Pack<_Float16, 8> { typedef uint4 raw_t; };
template <> struct Pack<float, 4>    { typedef uint4 raw_t; };
template <> struct Pack<_Float16, 1> { typedef unsigned short raw_t; };
template <> struct Pack<float, 1>    { typedef unsigned raw_t; };

template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const T* p, float (&v)[VEC])
{
    typedef typename Pack<T, VEC>::raw_t raw_t;
    raw_t raw = *reinterpret_cast<const raw_t*>(p);
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int i = 0; i < VEC; i++) v[i] = (float)e[i];
}

template <typename T, int VEC>
__device__ __forceinline__ void store_vec(T* p, const float (&v)[VEC])
{
    typedef typename Pack<T, VEC>::raw_t raw_t;
    raw_t raw;
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int i = 0; i < VEC; i++) e[i] = (T)v[i];   // nearest-even for fp16
    *reinterpret_cast<raw_t*>(p) = raw;
}

struct PoolGeom {
    int N, C, D, H, W;
    int J, T, R, S;
    int K, M, P, Q;
    int pad_j, pad_d, pad_h, pad_w;
    int str_j, str_d, str_h, str_w;
    int nvec;           // N / VEC
};

enum { OP_MAX = 0, OP_AVG = 1 };

#define NG_FLT_MAX 3.402823466e+38f

// one thread: VEC images of one output element
template <typename T, int VEC, int OP, bool WRITE_ARG>
__global__ __launch_bounds__(256)
void pool_fprop_kernel(const T* __restrict__ I, T* __restrict__ O, unsigned char* __restrict__ arg, PoolGeom g)
{
    const long total = (long)g.K * g.M * g.P * g.Q * g.nvec;
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int nv = (int)(e % g.nvec);
    long r = e / g.nvec;
    const int q = (int)(r % g.Q); r /= g.Q;
    const int p = (int)(r % g.P); r /= g.P;
    const int m = (int)(r % g.M);
    const int k = (int)(r / g.M);
    const int c0 = k * g.str_j - g.pad_j, z0 = m * g.str_d - g.pad_d;
    const int y0 = p * g.str_h - g.pad_h, x0 = q * g.str_w - g.pad_w;

    float best[VEC];
    int   slot_of[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) { best[i] = (OP == OP_MAX) ? -NG_FLT_MAX : 0.0f; slot_of[i] = 0; }

    int slot = 0;
    for (int j = 0; j < g.J; j++) {
        const int c = c0 + j;
        for (int t = 0; t < g.T; t++) {
            const int z = z0 + t;
            for (int rr = 0; rr < g.R; rr++) {
                const int y = y0 + rr;
                for (int s = 0; s < g.S; s++, slot++) {
                    const int x = x0 + s;
                    if ((unsigned)c < (unsigned)g.C && (unsigned)z < (unsigned)g.D &&
                        (unsigned)y < (unsigned)g.H && (unsigned)x < (unsigned)g.W) {
                        float v[VEC];
                        load_vec<T, VEC>(I + ((((long)c * g.D + z) * g.H + y) * g.W + x) * g.N + (long)nv * VEC, v);
#pragma unroll
                        for (int i = 0; i < VEC; i++) {
                            if (OP == OP_MAX) {
                                if (v[i] > best[i]) { best[i] = v[i]; slot_of[i] = slot; }
                            } else {
                                best[i] += v[i];
                            }
                        }
                    }
                }
            }
        }
    }
    const long o = e * VEC;
    if (WRITE_ARG) {
#pragma unroll
        for (int i = 0; i < VEC; i++) arg[o + i] = (unsigned char)slot_of[i];
    } else {
        if (OP == OP_AVG) {
            const float inv = 1.0f / (float)(g.J * g.T * g.R * g.S);
#pragma unroll
            for (int i = 0; i < VEC; i++) best[i] *= inv;
        }
        store_vec<T, VEC>(O + o, best);
    }
}

__device__ __forceinline__ void window_range(int coord, int pad, int win, int str, int count, int& lo, int& hi)
{
    // outputs o with o*str - pad <= coord <= o*str - pad + win - 1
    const int a = coord + pad - win + 1;
    lo = a <= 0 ? 0 : (a + str - 1) / str;
    hi = (coord + pad) / str;
    if (hi > count - 1) hi = count - 1;
}

// one thread: VEC images of one input element; sums the errors of the covering
// windows in a fixed (k,m,p,q) order
template <typename T, int VEC, int OP>
__global__ __launch_bounds__(256)
void pool_bprop_kernel(const T* __restrict__ E, const unsigned char* __restrict__ arg, T* __restrict__ B, PoolGeom g)
{
    const long total = (long)g.C * g.D * g.H * g.W * g.nvec;
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int nv = (int)(e % g.nvec);
    long r = e / g.nvec;
    const int x = (int)(r % g.W); r /= g.W;
    const int y = (int)(r % g.H); r /= g.H;
    const int z = (int)(r % g.D);
    const int c = (int)(r / g.D);

    int k0, k1, m0, m1, p0, p1, q0, q1;
    window_range(c, g.pad_j, g.J, g.str_j, g.K, k0, k1);
    window_range(z, g.pad_d, g.T, g.str_d, g.M, m0, m1);
    window_range(y, g.pad_h, g.R, g.str_h, g.P, p0, p1);
    window_range(x, g.pad_w, g.S, g.str_w, g.Q, q0, q1);

    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) acc[i] = 0.0f;

    for (int k = k0; k <= k1; k++)
        for (int m = m0; m <= m1; m++)
            for (int p = p0; p <= p1; p++)
                for (int q = q0; q <= q1; q++) {
                    const long o = (((((long)k * g.M + m) * g.P + p) * g.Q + q) * g.nvec + nv) * VEC;
                    float ev[VEC];
                    load_vec<T, VEC>(E + o, ev);
                    if (OP == OP_MAX) {
                        const int slot = (((c - (k * g.str_j - g.pad_j)) * g.T + (z - (m * g.str_d - g.pad_d))) * g.R +
                                          (y - (p * g.str_h - g.pad_h))) * g.S + (x - (q * g.str_w - g.pad_w));
                        if (VEC == 8) {
                            const uint2 a = *reinterpret_cast<const uint2*>(arg + o);
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                if ((int)((a.x >> (8 * i)) & 0xFF) == slot) acc[i] += ev[i];
                                if ((int)((a.y >> (8 * i)) & 0xFF) == slot) acc[(i + 4) % VEC] += ev[(i + 4) % VEC];
                            }
                        } else {
#pragma unroll
                            for (int i = 0; i < VEC; i++)
                                if ((int)arg[o + i] == slot) acc[i] += ev[i];
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < VEC; i++) acc[i] += ev[i];
                    }
                }
    if (OP == OP_AVG) {
        const float inv = 1.0f / (float)(g.J * g.T * g.R * g.S);
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] *= inv;
    }
    store_vec<T, VEC>(B + e * VEC, acc);
}

// windows that tile the input exactly (stride == window, no padding, extents
// divisible): one thread owns a whole window and writes all of its grad_I
// elements, so max bprop needs a single pass and no argmax scratch.
template <typename T, int VEC>
__global__ __launch_bounds__(256)
void pool_bprop_max_tiled_kernel(const T* __restrict__ I, const T* __restrict__ E, T* __restrict__ B, PoolGeom g)
{
    const long total = (long)g.K * g.M * g.P * g.Q * g.nvec;
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int nv = (int)(e % g.nvec);
    long r = e / g.nvec;
    const int q = (int)(r % g.Q); r /= g.Q;
    const int p = (int)(r % g.P); r /= g.P;
    const int m = (int)(r % g.M);
    const int k = (int)(r / g.M);
    const int c0 = k * g.J, z0 = m * g.T, y0 = p * g.R, x0 = q * g.S;

    float best[VEC];
    int   slot_of[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) { best[i] = -NG_FLT_MAX; slot_of[i] = 0; }
    int slot = 0;
    for (int j = 0; j < g.J; j++)
        for (int t = 0; t < g.T; t++)
            for (int rr = 0; rr < g.R; rr++)
                for (int s = 0; s < g.S; s++, slot++) {
                    float v[VEC];
                    load_vec<T, VEC>(I + ((((long)(c0 + j) * g.D + z0 + t) * g.H + y0 + rr) * g.W + x0 + s) * g.N +
                                         (long)nv * VEC, v);
#pragma unroll
                    for (int i = 0; i < VEC; i++)
                        if (v[i] > best[i]) { best[i] = v[i]; slot_of[i] = slot; }
                }
    float ev[VEC];
    load_vec<T, VEC>(E + e * VEC, ev);
    slot = 0;
    for (int j = 0; j < g.J; j++)
        for (int t = 0; t < g.T; t++)
            for (int rr = 0; rr < g.R; rr++)
                for (int s = 0; s < g.S; s++, slot++) {
                    float out[VEC];
#pragma unroll
                    for (int i = 0; i < VEC; i++) out[i] = (slot_of[i] == slot) ? ev[i] : 0.0f;
                    store_vec<T, VEC>(B + ((((long)(c0 + j) * g.D + z0 + t) * g.H + y0 + rr) * g.W + x0 + s) * g.N +
                                          (long)nv * VEC, out);
                }
}

static PoolGeom make_geom(const ng_pool_params& p, int vec)
{
    PoolGeom g{p.N, p.C, p.D, p.H, p.W, p.J, p.T, p.R, p.S, p.K, p.M, p.P, p.Q,
               p.pad_j, p.pad_d, p.pad_h, p.pad_w, p.str_j, p.str_d, p.str_h, p.str_w, p.N / vec};
    return g;
}

static bool tiles_exactly(const ng_pool_params& p)
{
    return p.pad_j == 0 && p.pad_d == 0 && p.pad_h == 0 && p.pad_w == 0 &&
           p.str_j == p.J && p.str_d == p.T && p.str_h == p.R && p.str_w == p.S &&
           p.K * p.J == p.C && p.M * p.T == p.D && p.P * p.R == p.H && p.Q * p.S == p.W;
}

static int check_params(const ng_pool_params& p, int dtype, int op)
{
    if (dtype != NG_F16 && dtype != NG_F32) return fail(-60, "pool: dtype must be fp16 or fp32");
    if (op != OP_MAX && op != OP_AVG) return fail(-61, "pool: op must be 0 (max) or 1 (avg)");
    if (p.N <= 0 || p.C <= 0 || p.K <= 0 || p.M <= 0 || p.P <= 0 || p.Q <= 0) return fail(-62, "pool: empty geometry");
    if (p.str_j < 1 || p.str_d < 1 || p.str_h < 1 || p.str_w < 1) return fail(-63, "pool: strides must be >= 1");
    return 0;
}

static unsigned blocks_for(long total) { return (unsigned)((total + 255) / 256); }

template <typename T, int VEC>
static int run_fprop(const ng_pool_params& p, int op, const void* I, void* O, hipStream_t st)
{
    PoolGeom g = make_geom(p, VEC);
    const long total = (long)g.K * g.M * g.P * g.Q * g.nvec;
    if (op == OP_MAX)
        hipLaunchKernelGGL((pool_fprop_kernel<T, VEC, OP_MAX, false>), dim3(blocks_for(total)), dim3(256), 0, st,
                           (const T*)I, (T*)O, (unsigned char*)nullptr, g);
    else
        hipLaunchKernelGGL((pool_fprop_kernel<T, VEC, OP_AVG, false>), dim3(blocks_for(total)), dim3(256), 0, st,
                           (const T*)I, (T*)O, (unsigned char*)nullptr, g);
    NG_CHECK_LAUNCH("pool fprop");
    return 0;
}

template <typename T, int VEC>
static int run_bprop(const ng_pool_params& p, int op, const void* I, const void* E, void* B,
                     void* ws, size_t ws_bytes, hipStream_t st)
{
    PoolGeom g = make_geom(p, VEC);
    const long out_total = (long)g.K * g.M * g.P * g.Q * g.nvec;
    const long in_total = (long)g.C * g.D * g.H * g.W * g.nvec;
    if (op == OP_AVG) {
        hipLaunchKernelGGL((pool_bprop_kernel<T, VEC, OP_AVG>), dim3(blocks_for(in_total)), dim3(256), 0, st,
                           (const T*)E, (const unsigned char*)nullptr, (T*)B, g);
        NG_CHECK_LAUNCH("pool avg bprop");
        return 0;
    }
    if (tiles_exactly(p)) {
        hipLaunchKernelGGL((pool_bprop_max_tiled_kernel<T, VEC>), dim3(blocks_for(out_total)), dim3(256), 0, st,
                           (const T*)I, (const T*)E, (T*)B, g);
        NG_CHECK_LAUNCH("pool max bprop (tiled)");
        return 0;
    }
    const size_t need = (size_t)out_total * VEC;
    if (!ws || ws_bytes < need) return fail(-64, "pool max bprop: workspace too small (%zu < %zu)", ws_bytes, need);
    if (p.J * p.T * p.R * p.S > 256) return fail(-65, "pool max bprop: windows of more than 256 elements are not supported");
    hipLaunchKernelGGL((pool_fprop_kernel<T, VEC, OP_MAX, true>), dim3(blocks_for(out_total)), dim3(256), 0, st,
                       (const T*)I, (T*)nullptr, (unsigned char*)ws, g);
    NG_CHECK_LAUNCH("pool argmax");
    hipLaunchKernelGGL((pool_bprop_kernel<T, VEC, OP_MAX>), dim3(blocks_for(in_total)), dim3(256), 0, st,
                       (const T*)E, (const unsigned char*)ws, (T*)B, g);
    NG_CHECK_LAUNCH("pool max bprop");
    return 0;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace ng

using namespace ng;

extern "C" {

size_t ng_pool_workspace_bytes(const ng_pool_params* p, int /*dtype*/, int op)
{
    if (op != OP_MAX || tiles_exactly(*p)) return 0;
    return align_up((size_t)p->K * p->M * p->P * p->Q * p->N, 256);
}

int ng_pool_fprop(const ng_pool_params* p, int dtype, int op, const void* I, void* O, void* stream)
{
    int rc = check_params(*p, dtype, op);
    if (rc) return rc;
    if (!I || !O) return fail(-66, "pool: null tensor");
    hipStream_t st = (hipStream_t)stream;
    const bool al = aligned16(I) && aligned16(O);
    if (dtype == NG_F16)
        return (al && p->N % 8 == 0) ? run_fprop<_Float16, 8>(*p, op, I, O, st) : run_fprop<_Float16, 1>(*p, op, I, O, st);
    return (al && p->N % 4 == 0) ? run_fprop<float, 4>(*p, op, I, O, st) : run_fprop<float, 1>(*p, op, I, O, st);
}

int ng_pool_bprop(const ng_pool_params* p, int dtype, int op, const void* I, const void* E, void* gradI,
                  void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_params(*p, dtype, op);
    if (rc) return rc;
    if (!E || !gradI || (op == OP_MAX && !I)) return fail(-66, "pool: null tensor");
    hipStream_t st = (hipStream_t)stream;
    const bool al = aligned16(E) && aligned16(gradI) && (op != OP_MAX || aligned16(I)) &&
                    (!workspace || aligned16(workspace));
    if (dtype == NG_F16)
        return (al && p->N % 8 == 0) ? run_bprop<_Float16, 8>(*p, op, I, E, gradI, workspace, workspace_bytes, st)
                                     : run_bprop<_Float16, 1>(*p, op, I, E, gradI, workspace, workspace_bytes, st);
    return (al && p->N % 4 == 0) ? run_bprop<float, 4>(*p, op, I, E, gradI, workspace, workspace_bytes, st)
                                 : run_bprop<float, 1>(*p, op, I, E, gradI, workspace, workspace_bytes, st);
}

}  // extern "C"
