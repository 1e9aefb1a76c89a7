// Pooling over a (J,T,R,S) window of a CHWN tensor: max and average, forward
// and backward.  Replaces {h,s}pool_max launched by NervanaGPU._execute_pool
// (nervanagpu/nervanagpu.py:789-818) and adds the average and l2 modes the
// reference only names (nervanagpu/nervanagpu.py:746, numpy definitions
// benchmarks/pool_test.py:142-146; l2 = square root of the sum of squares,
// forward only: the reference defines no derivative for it).
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
#include <cstdlib>

namespace ng {

template <typename T, int VEC> struct Pack;
template <> struct Pack<_Float16, 8> { typedef uint4 raw_t; };
template <> struct Pack<float, 4>    { typedef uint4 raw_t; };
template <> struct Pack<_Float16, 1> { typedef unsigned short raw_t; };
template <> struct Pack<float, 1>    { typedef unsigned raw_t; };

// non-temporal load of a 2-, 4- or 16-byte packet
template <typename R>
__device__ __forceinline__ R load_streaming(const R* p)
{
    if constexpr (sizeof(R) == 16) {
        typedef unsigned v4u __attribute__((ext_vector_type(4)));
        const v4u v = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p));
        return __builtin_bit_cast(R, v);
    } else if constexpr (sizeof(R) == 4) {
        return __builtin_bit_cast(R, __builtin_nontemporal_load(reinterpret_cast<const unsigned*>(p)));
    } else {
        return __builtin_bit_cast(R, __builtin_nontemporal_load(reinterpret_cast<const unsigned short*>(p)));
    }
}

// One 16-byte (or scalar) load.  The empty asm pins the four words in
// registers: without it the optimiser may follow the element-wise uses back to
// the load and split it into 2- and 4-byte pieces of lower alignment.
template <typename R>
__device__ __forceinline__ R load_packet(const R* p)
{
    R v = *p;
    if constexpr (sizeof(R) == 16) asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
    return v;
}

template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const T* p, float (&v)[VEC])
{
    typedef typename Pack<T, VEC>::raw_t raw_t;
    raw_t raw = load_packet(reinterpret_cast<const raw_t*>(p));
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
    // index decomposition without integer division: a thread's position inside
    // one feature map is split by nvec, then by the two inner spatial extents
    // (fprop kernels: Q, P; bprop gather: W, H); window ranges divide by strides
    FastDiv div_nvec, div_q, div_p, div_w, div_h;
    FastDiv div_sj, div_sd, div_sh, div_sw;
    // input read exactly once (windows do not overlap) and larger than the
    // last-level cache: streamed with non-temporal loads
    int stream_in;
    // forward kernels with overlapping windows and many workgroups per feature
    // map: XCD-contiguous workgroup numbering (gridDim.x padded to a multiple of 8)
    int xcd_remap;
    // backward by cells (pool_bprop_cell_kernel): which compiled (window, stride)
    // shape applies (0: none) and the number of stride-sized cells along h and w
    // that hold at least one input element
    int use_cells, cells_h, cells_w, cell_remap;
    FastDiv div_ch, div_cw;
    // backward by cells on maps of fewer workgroups: whole feature maps per XCD
    // (see xcd_map_block); div_cell_blocks divides by the workgroups of one map
    int cell_map_xcd;
    FastDiv div_cell_blocks;
    // the same numbering for the forward kernels (instead of xcd_remap)
    int fwd_map_xcd;
    FastDiv div_fwd_blocks;
    // max pooling backward with the rectifier derivative of the layer below
    // folded in: a window whose maximum is not positive passes nothing on
    int relu_mask;
};

enum { OP_MAX = 0, OP_AVG = 1, OP_L2 = 2 };
// argmax value no element of a window of at most 255 elements carries
enum { NO_SLOT = 255 };

#define NG_FLT_MAX 3.402823466e+38f

// Launch geometry shared by the kernels: blockIdx.y is the outermost index
// (output or input feature map), blockIdx.x * 256 + threadIdx.x the position
// inside that map: ((d * H + h) * W + w) * nvec + nv, below 2^31.
// Workgroups are dealt to the 8 XCDs round robin by linear id.  With gridDim.x a
// multiple of 8, the XCD of a workgroup is blockIdx.x % 8; renumbering gives
// each XCD one contiguous eighth of every feature map, and rows shared by
// overlapping windows are fetched into one L2 instead of several.
__device__ __forceinline__ unsigned xcd_block_index(int remap)
{
    return remap ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3) : blockIdx.x;
}

// Whole feature maps per XCD, for maps too small to cut into eighths: workgroups
// are handed to the 8 XCDs in turn in launch order (x fastest), so workgroup
// L = y * gridDim.x + x runs on XCD L % 8.  That XCD works through the maps
// xcd, xcd + 8, xcd + 16, ... one after the other: the windows two neighbouring
// rows of cells share are then fetched into one L2 once instead of into two.
// Needs gridDim.y (the feature maps) to be a multiple of 8.
__device__ __forceinline__ void xcd_map_block(const FastDiv& blocks_per_map, unsigned& block, unsigned& map)
{
    const unsigned linear = blockIdx.y * gridDim.x + blockIdx.x;
    const unsigned turn = linear >> 3;
    const unsigned round = blocks_per_map.div(turn);
    block = turn - round * gridDim.x;
    map = round * 8u + (linear & 7u);
}

__device__ __forceinline__ bool split_inner(unsigned inner, unsigned limit, const FastDiv& dn, const FastDiv& d1,
                                            const FastDiv& d2, int nvec, int e1, int e2, int& nv, int& i1, int& i2,
                                            int& i3)
{
    if (inner >= limit) return false;
    unsigned r = dn.div(inner);
    nv = (int)(inner - r * (unsigned)nvec);
    unsigned r1 = d1.div(r);
    i1 = (int)(r - r1 * (unsigned)e1);
    unsigned r2 = d2.div(r1);
    i2 = (int)(r1 - r2 * (unsigned)e2);
    i3 = (int)r2;
    return true;
}

// VEC elements of T as one register vector
template <typename T, int VEC> struct Lanes {
    typedef T type __attribute__((ext_vector_type(VEC)));
    static __device__ __forceinline__ type splat(T v) { return (type)(v); }
    static __device__ __forceinline__ type max(type a, type b) { return __builtin_elementwise_max(a, b); }
    static __device__ __forceinline__ T get(const type& a, int i) { return a[i]; }
};
template <typename T> struct Lanes<T, 1> {
    typedef T type;
    static __device__ __forceinline__ type splat(T v) { return v; }
    static __device__ __forceinline__ type max(type a, type b) { return a < b ? b : a; }
    static __device__ __forceinline__ T get(const type& a, int) { return a; }
};

// argmax slots of VEC elements, one byte each
template <int VEC>
__device__ __forceinline__ void store_slots(unsigned char* dst, const int (&slot_of)[VEC])
{
    if constexpr (VEC == 8) {
        uint2 packed;
        packed.x = (unsigned)slot_of[0] | ((unsigned)slot_of[1] << 8) | ((unsigned)slot_of[2] << 16) | ((unsigned)slot_of[3] << 24);
        packed.y = (unsigned)slot_of[4] | ((unsigned)slot_of[5] << 8) | ((unsigned)slot_of[6] << 16) | ((unsigned)slot_of[7] << 24);
        *reinterpret_cast<uint2*>(dst) = packed;
    } else {
#pragma unroll
        for (int i = 0; i < VEC; i++) dst[i] = (unsigned char)slot_of[i];
    }
}

// one thread: VEC images of one output element.  RS > 0: the window is a 2-D
// RS x RS square (J == T == 1), known at compile time, so all its loads are
// issued together; taps outside the image are redirected to a valid address and
// replaced by the identity of the reduction.
template <typename T, int VEC, int OP, bool WRITE_ARG, int RS>
__global__ __launch_bounds__(256)
void pool_fprop_kernel(const T* __restrict__ I, T* __restrict__ O, unsigned char* __restrict__ arg, PoolGeom g)
{
    const unsigned per_map = (unsigned)(g.M * g.P * g.Q * g.nvec);
    unsigned block = xcd_block_index(g.xcd_remap), map = blockIdx.y;
    if (g.fwd_map_xcd) xcd_map_block(g.div_fwd_blocks, block, map);
    const unsigned inner = block * 256u + threadIdx.x;
    const int k = (int)map;
    int nv, q, p, m;
    if (!split_inner(inner, per_map, g.div_nvec, g.div_q, g.div_p, g.nvec, g.Q, g.P, nv, q, p, m)) return;
    const int c0 = k * g.str_j - g.pad_j, z0 = m * g.str_d - g.pad_d;
    const int y0 = p * g.str_h - g.pad_h, x0 = q * g.str_w - g.pad_w;

    float best[VEC];
    int   slot_of[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) { best[i] = (OP == OP_MAX) ? -NG_FLT_MAX : 0.0f; slot_of[i] = 0; }

    const T* Inv = I + (long)nv * VEC;
    if (RS > 0) {
        constexpr int NTAP = RS > 0 ? RS * RS : 1;
        const bool plane_ok = (unsigned)c0 < (unsigned)g.C && (unsigned)z0 < (unsigned)g.D;
        const T* plane = Inv + ((long)c0 * g.D + z0) * g.H * g.W * g.N;
        typedef typename Pack<T, VEC>::raw_t raw_t;
        raw_t raw[NTAP];
        bool ok[NTAP];
#pragma unroll
        for (int tap = 0; tap < NTAP; tap++) {
            const int y = y0 + tap / (RS > 0 ? RS : 1), x = x0 + tap % (RS > 0 ? RS : 1);
            ok[tap] = plane_ok && (unsigned)y < (unsigned)g.H && (unsigned)x < (unsigned)g.W;
            const T* src = ok[tap] ? plane + ((long)y * g.W + x) * g.N : Inv;
            raw[tap] = g.stream_in ? load_streaming(reinterpret_cast<const raw_t*>(src))
                                   : *reinterpret_cast<const raw_t*>(src);
        }
        if constexpr (OP == OP_MAX) {
            // Branch-free, in the element type: the running maximum over all taps
            // (two fp16 elements per instruction), then a scan from the last tap
            // to the first for the first one that holds it: the element the
            // reference's strict '>' scan keeps.  That scan starts from -FLT_MAX at
            // slot 0 (kernels/sass/hpool_max.sass:218-219), so taps outside the image
            // count as -FLT_MAX (-inf once narrowed to fp16), a window without any
            // tap inside the image yields that value, and a window in which nothing
            // exceeds it keeps slot 0: the same results as the generic loop below.
            typedef typename Lanes<T, VEC>::type lanes_t;
            const T lowest = (T)(-NG_FLT_MAX);
            lanes_t taps[NTAP];
            bool all_ok = true;
#pragma unroll
            for (int tap = 0; tap < NTAP; tap++) {
                taps[tap] = __builtin_bit_cast(lanes_t, raw[tap]);
                all_ok = all_ok && ok[tap];
            }
            if (!all_ok) {
#pragma unroll
                for (int tap = 0; tap < NTAP; tap++)
                    if (!ok[tap]) taps[tap] = Lanes<T, VEC>::splat(lowest);
            }
            lanes_t top = Lanes<T, VEC>::max(Lanes<T, VEC>::splat(lowest), taps[0]);
#pragma unroll
            for (int tap = 1; tap < NTAP; tap++) top = Lanes<T, VEC>::max(top, taps[tap]);
            const long o = ((long)k * per_map + inner) * VEC;
            if constexpr (!WRITE_ARG) {
                *reinterpret_cast<raw_t*>(O + o) = __builtin_bit_cast(raw_t, top);
            } else {
#pragma unroll
                for (int tap = NTAP - 1; tap >= 0; tap--) {
#pragma unroll
                    for (int i = 0; i < VEC; i++)
                        slot_of[i] = (Lanes<T, VEC>::get(taps[tap], i) == Lanes<T, VEC>::get(top, i)) ? tap : slot_of[i];
                }
                if (!all_ok) {
#pragma unroll
                    for (int i = 0; i < VEC; i++) slot_of[i] = (Lanes<T, VEC>::get(top, i) > lowest) ? slot_of[i] : 0;
                }
                if (g.relu_mask) {
#pragma unroll
                    for (int i = 0; i < VEC; i++) slot_of[i] = ((float)Lanes<T, VEC>::get(top, i) > 0.0f) ? slot_of[i] : NO_SLOT;
                }
                store_slots<VEC>(arg + o, slot_of);
            }
            return;
        } else {
#pragma unroll
            for (int tap = 0; tap < NTAP; tap++) {
                const T* e = reinterpret_cast<const T*>(&raw[tap]);
#pragma unroll
                for (int i = 0; i < VEC; i++) {
                    const float v = ok[tap] ? (float)e[i] : 0.0f;
                    best[i] += (OP == OP_L2) ? v * v : v;
                }
            }
        }
    } else {
        int slot = 0;
        for (int j = 0; j < g.J; j++) {
            const int c = c0 + j;
            for (int t = 0; t < g.T; t++) {
                const int z = z0 + t;
                const bool plane_ok = (unsigned)c < (unsigned)g.C && (unsigned)z < (unsigned)g.D;
                const long plane = ((long)c * g.D + z) * g.H;
                for (int rr = 0; rr < g.R; rr++) {
                    const int y = y0 + rr;
                    const bool row_ok = plane_ok && (unsigned)y < (unsigned)g.H;
                    const T* row = Inv + (plane + y) * g.W * g.N;
                    for (int s = 0; s < g.S; s++, slot++) {
                        const int x = x0 + s;
                        if (row_ok && (unsigned)x < (unsigned)g.W) {
                            float v[VEC];
                            load_vec<T, VEC>(row + (long)x * g.N, v);
#pragma unroll
                            for (int i = 0; i < VEC; i++) {
                                if (OP == OP_MAX) {
                                    if (v[i] > best[i]) { best[i] = v[i]; slot_of[i] = slot; }
                                } else {
                                    best[i] += (OP == OP_L2) ? v[i] * v[i] : v[i];
                                }
                            }
                        }
                    }
                }
            }
        }
    }
    const long o = ((long)k * per_map + inner) * VEC;
    if (WRITE_ARG) {
        if (g.relu_mask) {
#pragma unroll
            for (int i = 0; i < VEC; i++) slot_of[i] = (best[i] > 0.0f) ? slot_of[i] : NO_SLOT;
        }
        store_slots<VEC>(arg + o, slot_of);
    } else {
        if (OP == OP_AVG) {
            const float inv = 1.0f / (float)(g.J * g.T * g.R * g.S);
#pragma unroll
            for (int i = 0; i < VEC; i++) best[i] *= inv;
        }
        if (OP == OP_L2) {
#pragma unroll
            for (int i = 0; i < VEC; i++) best[i] = sqrtf(best[i]);
        }
        store_vec<T, VEC>(O + o, best);
    }
}

__device__ __forceinline__ void window_range(int coord, int pad, int win, int str, const FastDiv& dstr, int count,
                                             int& lo, int& hi)
{
    // outputs o with o*str - pad <= coord <= o*str - pad + win - 1
    const int a = coord + pad - win + 1;
    lo = a <= 0 ? 0 : (int)dstr.div((unsigned)(a + str - 1));
    hi = (int)dstr.div((unsigned)(coord + pad));
    if (hi > count - 1) hi = count - 1;
}

// accumulate the error of one covering window into acc
template <typename T, int VEC, int OP>
__device__ __forceinline__ void add_window(float (&acc)[VEC], const typename Pack<T, VEC>::raw_t& eraw, uint2 a, int slot,
                                           bool valid)
{
    const T* ev = reinterpret_cast<const T*>(&eraw);
    if (OP == OP_MAX) {
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            const unsigned word = (i < 4) ? a.x : a.y;
            const int s = (int)((word >> (8 * (i & 3))) & 0xFF);
            acc[i] += (valid && s == slot) ? (float)ev[i] : 0.0f;
        }
    } else {
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] += valid ? (float)ev[i] : 0.0f;
    }
}

// one thread: VEC images of one input element; sums the errors of the covering
// windows in a fixed (k,m,p,q) order.  WIN2: at most two windows cover an
// element along h and along w, and one along c and d; the (up to) four loads
// are then issued together instead of inside data-dependent loops.
template <typename T, int VEC, int OP, bool WIN2>
__global__ __launch_bounds__(256)
void pool_bprop_kernel(const T* __restrict__ E, const unsigned char* __restrict__ arg, T* __restrict__ B, PoolGeom g)
{
    const unsigned per_map = (unsigned)(g.D * g.H * g.W * g.nvec);
    const unsigned inner = blockIdx.x * 256u + threadIdx.x;
    const int c = blockIdx.y;
    int nv, x, y, z;
    if (!split_inner(inner, per_map, g.div_nvec, g.div_w, g.div_h, g.nvec, g.W, g.H, nv, x, y, z)) return;

    int k0, k1, m0, m1, p0, p1, q0, q1;
    window_range(c, g.pad_j, g.J, g.str_j, g.div_sj, g.K, k0, k1);
    window_range(z, g.pad_d, g.T, g.str_d, g.div_sd, g.M, m0, m1);
    window_range(y, g.pad_h, g.R, g.str_h, g.div_sh, g.P, p0, p1);
    window_range(x, g.pad_w, g.S, g.str_w, g.div_sw, g.Q, q0, q1);

    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) acc[i] = 0.0f;

    if (WIN2 && VEC == 8) {
        typedef typename Pack<T, VEC>::raw_t raw_t;
        const bool km_ok = k0 <= k1 && m0 <= m1;
        const int k = k0, m = m0;
        const int slot_km = ((c - (k * g.str_j - g.pad_j)) * g.T + (z - (m * g.str_d - g.pad_d))) * g.R;
        raw_t eraw[4];
        uint2 a[4];
        bool ok[4];
        int slot[4];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const int p = p0 + (w >> 1), q = q0 + (w & 1);
            ok[w] = km_ok && p <= p1 && q <= q1;
            const long o = ok[w] ? (((((long)k * g.M + m) * g.P + p) * g.Q + q) * g.nvec + nv) * VEC : (long)nv * VEC;
            eraw[w] = *reinterpret_cast<const raw_t*>(E + o);
            a[w] = (OP == OP_MAX) ? *reinterpret_cast<const uint2*>(arg + o) : make_uint2(0, 0);
            slot[w] = (slot_km + (y - (p * g.str_h - g.pad_h))) * g.S + (x - (q * g.str_w - g.pad_w));
        }
#pragma unroll
        for (int w = 0; w < 4; w++) add_window<T, VEC, OP>(acc, eraw[w], a[w], slot[w], ok[w]);
    } else {
        for (int k = k0; k <= k1; k++)
            for (int m = m0; m <= m1; m++) {
                const int slot_km = ((c - (k * g.str_j - g.pad_j)) * g.T + (z - (m * g.str_d - g.pad_d))) * g.R;
                for (int p = p0; p <= p1; p++) {
                    const int slot_p = (slot_km + (y - (p * g.str_h - g.pad_h))) * g.S + x + g.pad_w;
                    const long row = ((((long)k * g.M + m) * g.P + p) * g.Q * g.nvec + nv) * VEC;
                    for (int q = q0; q <= q1; q++) {
                        const long o = row + (long)q * g.nvec * VEC;
                        float ev[VEC];
                        load_vec<T, VEC>(E + o, ev);
                        if (OP == OP_MAX) {
                            const int slot = slot_p - q * g.str_w;
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
                }
            }
    }
    if (OP == OP_AVG) {
        const float inv = 1.0f / (float)(g.J * g.T * g.R * g.S);
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[i] *= inv;
    }
    store_vec<T, VEC>(B + ((long)c * per_map + inner) * VEC, acc);
}

// Backward for 2-D RS x RS windows of stride STR <= RS, known at compile time.
// Shift the input by the padding and cut it into STR x STR cells: with
// NW = ceil(RS / STR), every element of cell (cy,cx) is covered by windows out
// of the same NW x NW, (cy-NW+1..cy) x (cx-NW+1..cx), and its tap inside each
// of them is a compile-time constant.  One thread loads those errors (and
// argmax bytes) once and produces the whole cell (3x3 /2: four windows for four
// elements; 3x3 /1: nine for one; 2x2 /2: one for four), instead of every
// element finding and decoding the windows of its own.  Accumulation order per
// element is (p,q) ascending, as in pool_bprop_kernel.
template <typename T, int VEC, int OP, int RS, int STR>
__global__ __launch_bounds__(256)
void pool_bprop_cell_kernel(const T* __restrict__ E, const unsigned char* __restrict__ arg, T* __restrict__ B, PoolGeom g)
{
    static_assert(VEC == 4 || VEC == 8, "one or two argmax words per packet");
    static_assert(STR <= RS, "every element inside a window row / column range");
    constexpr int NW = (RS + STR - 1) / STR;
    typedef typename Pack<T, VEC>::raw_t raw_t;
    const unsigned per_map = (unsigned)(g.D * g.cells_h * g.cells_w * g.nvec);
    unsigned block = xcd_block_index(g.cell_remap), map = blockIdx.y;
    if (g.cell_map_xcd) xcd_map_block(g.div_cell_blocks, block, map);
    const unsigned inner = block * 256u + threadIdx.x;
    int nv, cx, cy, z;
    if (!split_inner(inner, per_map, g.div_nvec, g.div_cw, g.div_ch, g.nvec, g.cells_w, g.cells_h, nv, cx, cy, z)) return;
    // one feature map holds fewer than 2^31 elements: 32-bit offsets inside it
    const long out_map = (long)map * g.M * g.P * g.Q * g.N;
    const T* Em = E + out_map;
    const unsigned char* am = arg + (OP == OP_MAX ? out_map : 0);
    T* Bm = B + (long)map * g.D * g.H * g.W * g.N;

    raw_t eraw[NW * NW];
    unsigned words[NW * NW][2];
#pragma unroll
    for (int w = 0; w < NW * NW; w++) {
        const int p = cy - (NW - 1) + w / NW, q = cx - (NW - 1) + w % NW;
        const bool ok = (unsigned)p < (unsigned)g.P && (unsigned)q < (unsigned)g.Q;
        const unsigned o = ok ? (unsigned)((((z * g.P + p) * g.Q + q) * g.nvec + nv) * VEC) : (unsigned)(nv * VEC);
        eraw[w] = load_packet(reinterpret_cast<const raw_t*>(Em + o));
        if (OP == OP_MAX) {
            // a window outside the output matches no tap
            if (VEC == 8) {
                const uint2 a = *reinterpret_cast<const uint2*>(am + o);
                words[w][0] = ok ? a.x : 0xFFFFFFFFu;
                words[w][1] = ok ? a.y : 0xFFFFFFFFu;
            } else {
                const unsigned a = *reinterpret_cast<const unsigned*>(am + o);
                words[w][0] = words[w][1] = ok ? a : 0xFFFFFFFFu;
            }
        } else if (!ok) {
            eraw[w] = raw_t{};
        }
    }

    float acc[STR * STR][VEC];
#pragma unroll
    for (int px = 0; px < STR * STR; px++)
#pragma unroll
        for (int i = 0; i < VEC; i++) acc[px][i] = 0.0f;
#pragma unroll
    for (int w = 0; w < NW * NW; w++) {
        const T* e = reinterpret_cast<const T*>(&eraw[w]);
        float ev[VEC];
        int   tap[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) {
            ev[i] = (float)e[i];
            tap[i] = (int)((words[w][i >> 2] >> (8 * (i & 3))) & 0xFF);
        }
#pragma unroll
        for (int px = 0; px < STR * STR; px++) {
            // row / column of cell element px inside window w
            const int ty = px / STR + (NW - 1 - w / NW) * STR, tx = px % STR + (NW - 1 - w % NW) * STR;
            if (ty >= RS || tx >= RS) continue;
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                if (OP == OP_MAX) acc[px][i] += (tap[i] == ty * RS + tx) ? ev[i] : 0.0f;
                else              acc[px][i] += ev[i];
            }
        }
    }

    const float inv = 1.0f / (float)(RS * RS);
#pragma unroll
    for (int px = 0; px < STR * STR; px++) {
        const int y = cy * STR + px / STR - g.pad_h, x = cx * STR + px % STR - g.pad_w;
        if ((unsigned)y >= (unsigned)g.H || (unsigned)x >= (unsigned)g.W) continue;
        if (OP == OP_AVG) {
#pragma unroll
            for (int i = 0; i < VEC; i++) acc[px][i] *= inv;
        }
        store_vec<T, VEC>(Bm + (unsigned)((((z * g.H + y) * g.W + x) * g.nvec + nv) * VEC), acc[px]);
    }
}

// windows that tile the input exactly (stride == window, no padding, extents
// divisible): one thread owns a whole window and writes all of its grad_I
// elements, so max bprop needs a single pass and no argmax scratch.
template <typename T, int VEC, int RS>
__global__ __launch_bounds__(256)
void pool_bprop_max_tiled_kernel(const T* __restrict__ I, const T* __restrict__ E, T* __restrict__ B, PoolGeom g)
{
    const unsigned per_map = (unsigned)(g.M * g.P * g.Q * g.nvec);
    const unsigned inner = blockIdx.x * 256u + threadIdx.x;
    const int k = blockIdx.y;
    int nv, q, p, m;
    if (!split_inner(inner, per_map, g.div_nvec, g.div_q, g.div_p, g.nvec, g.Q, g.P, nv, q, p, m)) return;
    const int c0 = k * g.J, z0 = m * g.T, y0 = p * g.R, x0 = q * g.S;
    const long in_base = ((((long)c0 * g.D + z0) * g.H + y0) * g.W + x0) * g.N + (long)nv * VEC;
    const long sx = g.N, sy = (long)g.W * g.N, sz = (long)g.H * g.W * g.N, sc = (long)g.D * g.H * g.W * g.N;

    if (RS > 0) {
        // 2-D RS x RS window known at compile time: all loads, then all stores
        constexpr int NTAP = RS > 0 ? RS * RS : 1;
        typedef typename Pack<T, VEC>::raw_t raw_t;
        raw_t raw[NTAP];
#pragma unroll
        for (int tap = 0; tap < NTAP; tap++) {
            const raw_t* src = reinterpret_cast<const raw_t*>(I + in_base + (tap / (RS > 0 ? RS : 1)) * sy + (tap % (RS > 0 ? RS : 1)) * sx);
            raw[tap] = g.stream_in ? load_streaming(src) : *src;
        }
        float ev[VEC];
        load_vec<T, VEC>(E + ((long)k * per_map + inner) * VEC, ev);
        float best[VEC];
        int   slot_of[VEC];
#pragma unroll
        for (int i = 0; i < VEC; i++) { best[i] = -NG_FLT_MAX; slot_of[i] = 0; }
#pragma unroll
        for (int tap = 0; tap < NTAP; tap++) {
            const T* e = reinterpret_cast<const T*>(&raw[tap]);
#pragma unroll
            for (int i = 0; i < VEC; i++) {
                const float v = (float)e[i];
                if (v > best[i]) { best[i] = v; slot_of[i] = tap; }
            }
        }
        if (g.relu_mask) {
#pragma unroll
            for (int i = 0; i < VEC; i++) slot_of[i] = (best[i] > 0.0f) ? slot_of[i] : NO_SLOT;
        }
#pragma unroll
        for (int tap = 0; tap < NTAP; tap++) {
            float out[VEC];
#pragma unroll
            for (int i = 0; i < VEC; i++) out[i] = (slot_of[i] == tap) ? ev[i] : 0.0f;
            store_vec<T, VEC>(B + in_base + (tap / (RS > 0 ? RS : 1)) * sy + (tap % (RS > 0 ? RS : 1)) * sx, out);
        }
        return;
    }
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
                    load_vec<T, VEC>(I + in_base + j * sc + t * sz + rr * sy + s * sx, v);
#pragma unroll
                    for (int i = 0; i < VEC; i++)
                        if (v[i] > best[i]) { best[i] = v[i]; slot_of[i] = slot; }
                }
    if (g.relu_mask) {
#pragma unroll
        for (int i = 0; i < VEC; i++) slot_of[i] = (best[i] > 0.0f) ? slot_of[i] : NO_SLOT;
    }
    float ev[VEC];
    load_vec<T, VEC>(E + ((long)k * per_map + inner) * VEC, ev);
    slot = 0;
    for (int j = 0; j < g.J; j++)
        for (int t = 0; t < g.T; t++)
            for (int rr = 0; rr < g.R; rr++)
                for (int s = 0; s < g.S; s++, slot++) {
                    float out[VEC];
#pragma unroll
                    for (int i = 0; i < VEC; i++) out[i] = (slot_of[i] == slot) ? ev[i] : 0.0f;
                    store_vec<T, VEC>(B + in_base + j * sc + t * sz + rr * sy + s * sx, out);
                }
}

static PoolGeom make_geom(const ng_pool_params& p, int vec, size_t elem_bytes)
{
    PoolGeom g{p.N, p.C, p.D, p.H, p.W, p.J, p.T, p.R, p.S, p.K, p.M, p.P, p.Q,
               p.pad_j, p.pad_d, p.pad_h, p.pad_w, p.str_j, p.str_d, p.str_h, p.str_w, p.N / vec};
    g.div_nvec = FastDiv::make((unsigned)g.nvec);
    g.div_q = FastDiv::make((unsigned)p.Q);
    g.div_p = FastDiv::make((unsigned)p.P);
    g.div_w = FastDiv::make((unsigned)p.W);
    g.div_h = FastDiv::make((unsigned)p.H);
    g.div_sj = FastDiv::make((unsigned)p.str_j);
    g.div_sd = FastDiv::make((unsigned)p.str_d);
    g.div_sh = FastDiv::make((unsigned)p.str_h);
    g.div_sw = FastDiv::make((unsigned)p.str_w);
    const bool disjoint = p.str_j >= p.J && p.str_d >= p.T && p.str_h >= p.R && p.str_w >= p.S;
    const size_t in_bytes = (size_t)p.C * p.D * p.H * p.W * p.N * elem_bytes;
    g.stream_in = (disjoint && in_bytes > (256u << 20)) ? 1 : 0;
    g.xcd_remap = (!disjoint && (long)p.M * p.P * p.Q * g.nvec >= 16 * 256) ? 1 : 0;
    g.use_cells = 0;
    g.cells_h = (p.H - 1 + p.pad_h) / p.str_h + 1;
    g.cells_w = (p.W - 1 + p.pad_w) / p.str_w + 1;
    // neighbouring cells read the same windows: XCD-contiguous numbering as in the
    // forward kernels, for overlapping windows and maps of 64 workgroups or more
    // (rounding a smaller grid up to a multiple of 8 idles too many of them)
    g.cell_remap = (!disjoint && (long)p.D * g.cells_h * g.cells_w * g.nvec >= 64 * 256) ? 1 : 0;
    g.div_ch = FastDiv::make((unsigned)g.cells_h);
    g.div_cw = FastDiv::make((unsigned)g.cells_w);
    // smaller maps: whole maps per XCD when the maps divide over the 8 XCDs (the
    // 56x56 maps of 128 images are 49 workgroups: without it consecutive
    // workgroups, i.e. neighbouring rows of cells, sit on different XCDs and the
    // errors and argmax bytes are fetched twice: 152 MB for 72 MB)
    const long cell_blocks = ((long)p.D * g.cells_h * g.cells_w * g.nvec + 255) / 256;
    // NG_POOL_MAP_XCD (read once): 0 = launch-order numbering as before; 2 = also the forward kernels of
    // such maps (16 to 63 workgroups per map are cut into eighths today: a candidate, not measured yet)
    static const int map_xcd = getenv("NG_POOL_MAP_XCD") ? atoi(getenv("NG_POOL_MAP_XCD")) : 1;
    g.cell_map_xcd = (!disjoint && !g.cell_remap && p.C % 8 == 0 && cell_blocks >= 2 && map_xcd != 0) ? 1 : 0;
    g.div_cell_blocks = FastDiv::make((unsigned)cell_blocks);
    const long fwd_blocks = ((long)p.M * p.P * p.Q * g.nvec + 255) / 256;
    g.fwd_map_xcd = (map_xcd == 2 && !disjoint && p.K % 8 == 0 && fwd_blocks >= 2 && fwd_blocks < 64) ? 1 : 0;
    if (g.fwd_map_xcd) g.xcd_remap = 0;
    g.div_fwd_blocks = FastDiv::make((unsigned)fwd_blocks);
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
    if (op != OP_MAX && op != OP_AVG && op != OP_L2) return fail(-61, "pool: op must be 0 (max), 1 (avg) or 2 (l2)");
    if (p.N <= 0 || p.C <= 0 || p.K <= 0 || p.M <= 0 || p.P <= 0 || p.Q <= 0) return fail(-62, "pool: empty geometry");
    if (p.str_j < 1 || p.str_d < 1 || p.str_h < 1 || p.str_w < 1) return fail(-63, "pool: strides must be >= 1");
    if (p.D <= 0 || p.H <= 0 || p.W <= 0) return fail(-62, "pool: empty geometry");
    // one feature map is indexed with 31 bits, feature maps with gridDim.y
    if ((long)p.D * p.H * p.W * p.N >= (1L << 31) || (long)p.M * p.P * p.Q * p.N >= (1L << 31))
        return fail(-67, "pool: a single feature map must hold fewer than 2^31 elements");
    if (p.C > 65535 || p.K > 65535) return fail(-68, "pool: more than 65535 feature maps are not supported");
    return 0;
}

// grid over (positions of one feature map) x (feature maps)
static dim3 grid_for(long per_map, int maps, int pad8 = 0)
{
    unsigned blocks = (unsigned)((per_map + 255) / 256);
    if (pad8) blocks = (blocks + 7u) / 8u * 8u;   // see xcd_block_index()
    return dim3(blocks, (unsigned)maps, 1);
}

// compile-time window size of the unrolled forward kernels (0: generic loops)
static int square_window(const ng_pool_params& p)
{
    if (p.J != 1 || p.T != 1 || p.R != p.S) return 0;
    return (p.R == 2 || p.R == 3) ? p.R : 0;
}

template <typename T, int VEC, int OP, bool WRITE_ARG>
static void launch_fprop(const PoolGeom& g, int rs, dim3 grid, const T* I, T* O, unsigned char* arg, hipStream_t st)
{
    if (rs == 2 && VEC > 1)
        hipLaunchKernelGGL((pool_fprop_kernel<T, VEC, OP, WRITE_ARG, 2>), grid, dim3(256), 0, st, I, O, arg, g);
    else if (rs == 3 && VEC > 1)
        hipLaunchKernelGGL((pool_fprop_kernel<T, VEC, OP, WRITE_ARG, 3>), grid, dim3(256), 0, st, I, O, arg, g);
    else
        hipLaunchKernelGGL((pool_fprop_kernel<T, VEC, OP, WRITE_ARG, 0>), grid, dim3(256), 0, st, I, O, arg, g);
}

template <typename T, int VEC>
static int run_fprop(const ng_pool_params& p, int op, const void* I, void* O, hipStream_t st)
{
    PoolGeom g = make_geom(p, VEC, sizeof(T));
    const dim3 grid = grid_for((long)g.M * g.P * g.Q * g.nvec, g.K, g.xcd_remap);
    const int rs = square_window(p);
    if (op == OP_MAX)      launch_fprop<T, VEC, OP_MAX, false>(g, rs, grid, (const T*)I, (T*)O, nullptr, st);
    else if (op == OP_AVG) launch_fprop<T, VEC, OP_AVG, false>(g, rs, grid, (const T*)I, (T*)O, nullptr, st);
    else                   launch_fprop<T, VEC, OP_L2, false>(g, rs, grid, (const T*)I, (T*)O, nullptr, st);
    NG_CHECK_LAUNCH("pool fprop");
    return 0;
}

// at most two covering windows along h and w and one along c and d
static bool two_window_cover(const ng_pool_params& p)
{
    return p.J == 1 && p.T == 1 && (p.R + p.str_h - 1) / p.str_h <= 2 && (p.S + p.str_w - 1) / p.str_w <= 2;
}

// 2-D square windows over whole feature maps with a (window, stride) pair the
// cell kernel is compiled for: 0 = none, else RS * 16 + STR
static int cell_shape(const ng_pool_params& p)
{
    const bool plane = p.J == 1 && p.T == 1 && p.str_j == 1 && p.str_d == 1 && p.pad_j == 0 && p.pad_d == 0 &&
                       p.K == p.C && p.M == p.D && p.R == p.S && p.str_h == p.str_w && p.pad_h >= 0 && p.pad_w >= 0;
    if (!plane) return 0;
    const int shape = p.R * 16 + p.str_h;
    return (shape == 0x32 || shape == 0x31 || shape == 0x22) ? shape : 0;
}

template <typename T, int VEC, int OP>
static void launch_gather(const PoolGeom& g, bool win2, dim3 grid, const T* E, const unsigned char* arg, T* B,
                          hipStream_t st)
{
    if constexpr (VEC > 1) {
        const dim3 cgrid = grid_for((long)g.D * g.cells_h * g.cells_w * g.nvec, g.C, g.cell_remap);
        switch (g.use_cells) {
        case 0x32:
            hipLaunchKernelGGL((pool_bprop_cell_kernel<T, VEC, OP, 3, 2>), cgrid, dim3(256), 0, st, E, arg, B, g);
            return;
        case 0x31:
            hipLaunchKernelGGL((pool_bprop_cell_kernel<T, VEC, OP, 3, 1>), cgrid, dim3(256), 0, st, E, arg, B, g);
            return;
        case 0x22:
            hipLaunchKernelGGL((pool_bprop_cell_kernel<T, VEC, OP, 2, 2>), cgrid, dim3(256), 0, st, E, arg, B, g);
            return;
        default: break;
        }
    }
    if (win2 && VEC == 8)
        hipLaunchKernelGGL((pool_bprop_kernel<T, VEC, OP, true>), grid, dim3(256), 0, st, E, arg, B, g);
    else
        hipLaunchKernelGGL((pool_bprop_kernel<T, VEC, OP, false>), grid, dim3(256), 0, st, E, arg, B, g);
}

template <typename T, int VEC>
static int run_bprop(const ng_pool_params& p, int op, const void* I, const void* E, void* B, unsigned flags,
                     void* ws, size_t ws_bytes, hipStream_t st)
{
    PoolGeom g = make_geom(p, VEC, sizeof(T));
    g.relu_mask = (flags & NG_FLAG_RELU) ? 1 : 0;
    const long out_total = (long)g.K * g.M * g.P * g.Q * g.nvec;
    const dim3 out_grid = grid_for((long)g.M * g.P * g.Q * g.nvec, g.K, g.xcd_remap);
    const dim3 in_grid = grid_for((long)g.D * g.H * g.W * g.nvec, g.C);
    const bool win2 = two_window_cover(p);
    g.use_cells = cell_shape(p);
    if (op == OP_AVG) {
        launch_gather<T, VEC, OP_AVG>(g, win2, in_grid, (const T*)E, nullptr, (T*)B, st);
        NG_CHECK_LAUNCH("pool avg bprop");
        return 0;
    }
    if (tiles_exactly(p)) {
        const int rs = (VEC > 1) ? square_window(p) : 0;
        if (rs == 2)
            hipLaunchKernelGGL((pool_bprop_max_tiled_kernel<T, VEC, 2>), out_grid, dim3(256), 0, st,
                               (const T*)I, (const T*)E, (T*)B, g);
        else if (rs == 3)
            hipLaunchKernelGGL((pool_bprop_max_tiled_kernel<T, VEC, 3>), out_grid, dim3(256), 0, st,
                               (const T*)I, (const T*)E, (T*)B, g);
        else
            hipLaunchKernelGGL((pool_bprop_max_tiled_kernel<T, VEC, 0>), out_grid, dim3(256), 0, st,
                               (const T*)I, (const T*)E, (T*)B, g);
        NG_CHECK_LAUNCH("pool max bprop (tiled)");
        return 0;
    }
    const size_t need = (size_t)out_total * VEC;
    if (!ws || ws_bytes < need) return fail(-64, "pool max bprop: workspace too small (%zu < %zu)", ws_bytes, need);
    if (p.J * p.T * p.R * p.S > 256) return fail(-65, "pool max bprop: windows of more than 256 elements are not supported");
    launch_fprop<T, VEC, OP_MAX, true>(g, square_window(p), out_grid, (const T*)I, (T*)nullptr, (unsigned char*)ws, st);
    NG_CHECK_LAUNCH("pool argmax");
    launch_gather<T, VEC, OP_MAX>(g, win2, in_grid, (const T*)E, (const unsigned char*)ws, (T*)B, st);
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
                  unsigned flags, void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_params(*p, dtype, op);
    if (rc) return rc;
    if (op == OP_L2) return fail(-61, "pool bprop: l2 pooling has no backward pass (the reference defines none)");
    if (!E || !gradI || (op == OP_MAX && !I)) return fail(-66, "pool: null tensor");
    if (flags & ~(unsigned)NG_FLAG_RELU) return fail(-69, "pool bprop: unknown flag bits 0x%x", flags);
    if ((flags & NG_FLAG_RELU) && (op != OP_MAX || p->J * p->T * p->R * p->S > 255))
        return fail(-69, "pool bprop: the rectifier mask needs max pooling over windows of at most 255 elements");
    hipStream_t st = (hipStream_t)stream;
    const bool al = aligned16(E) && aligned16(gradI) && (op != OP_MAX || aligned16(I)) &&
                    (!workspace || aligned16(workspace));
    if (dtype == NG_F16)
        return (al && p->N % 8 == 0) ? run_bprop<_Float16, 8>(*p, op, I, E, gradI, flags, workspace, workspace_bytes, st)
                                     : run_bprop<_Float16, 1>(*p, op, I, E, gradI, flags, workspace, workspace_bytes, st);
    return (al && p->N % 4 == 0) ? run_bprop<float, 4>(*p, op, I, E, gradI, flags, workspace, workspace_bytes, st)
                                 : run_bprop<float, 1>(*p, op, I, E, gradI, flags, workspace, workspace_bytes, st);
}

}  // extern "C"
