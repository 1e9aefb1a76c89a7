// Operand loaders and epilogues that turn the MFMA contraction core into the
// three convolution operations on CHWN tensors (N innermost):
//
//   fprop   O[k, pix, n]  = sum_j  F[j, k]       * I[gather(j, pix), n]   j = (c,t,r,s)
//   bprop   gI[c, pix, n] = sum_j  Fs[j, c]      * E[gather(j, pix), n]   j = (tap, k)
//   update  gF[j, k]      = sum_(pix,n) I[gather(j, pix), n] * E[k, pix, n]
//
// In all three the row of the activation tensor selected by (j, pix) is one
// contiguous run of N elements, so a 16-byte chunk never straddles a pixel
// (N is a multiple of 8) and gathers stay fully vectorised.  Which rows exist
// is described by a small device table with one entry per contraction row j.
//
// Semantics follow the reference's numpy statement of the operation
// (benchmarks/conv_test.py:99-167) and the index formulas of
// kernels/sass/hconv_fprop_K64_N64.sass:188-240.
#pragma once

#include "gemm_core.h"

namespace ng {

// one contraction row: element offset of the tap relative to the pixel origin,
// and the tap's coordinate deltas for the bounds test
struct TapEntry { int off, dz, dy, dx; };

typedef unsigned char u8_t;
typedef signed char   s8_t;

// 16-byte chunk of compute type T from a run of storage type TIN
template <typename T, typename TIN> struct ChunkFetch;

template <typename T> struct ChunkFetch<T, T> {
    static __device__ __forceinline__ uint4_t get(const T* p) { return *reinterpret_cast<const uint4_t*>(p); }
};

// bytes -> fp16, exact for every 8-bit value (I2F on load in the reference,
// kernels/sass/hconv_updat_C64_K64.sass:324-345)
template <> struct ChunkFetch<_Float16, u8_t> {
    static __device__ __forceinline__ uint4_t get(const u8_t* p)
    {
        const uint2 raw = *reinterpret_cast<const uint2*>(p);
        _Float16 h[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e]     = (_Float16)(float)((raw.x >> (8 * e)) & 0xFFu);
            h[e + 4] = (_Float16)(float)((raw.y >> (8 * e)) & 0xFFu);
        }
        return *reinterpret_cast<const uint4_t*>(h);
    }
};

template <> struct ChunkFetch<_Float16, s8_t> {
    static __device__ __forceinline__ uint4_t get(const s8_t* p)
    {
        const uint2 raw = *reinterpret_cast<const uint2*>(p);
        _Float16 h[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e]     = (_Float16)(float)(int)(signed char)((raw.x >> (8 * e)) & 0xFFu);
            h[e + 4] = (_Float16)(float)(int)(signed char)((raw.y >> (8 * e)) & 0xFFu);
        }
        return *reinterpret_cast<const uint4_t*>(h);
    }
};

// how output/activation columns enumerate pixels: column = pixel * N + n, and
// pixel = (iz * ny + iy) * nx + ix over an (nz, ny, nx) lattice
struct PixelLattice {
    int N;
    int ncols;      // nz*ny*nx*N
    int nx, nxy;    // nx, nx*ny
};

// B operand of fprop / bprop (row-contiguous tile: lines are contraction rows,
// columns are (pixel, n)).  Gathered coordinate of tap j at lattice point
// (iz,iy,ix) is (iz*gs_d + dz_j, iy*gs_h + dy_j, ix*gs_w + dx_j) inside a
// (lim_d, lim_h, lim_w) volume; taps outside contribute zero.
template <typename T, typename TIN>
struct GatherColsLoader {
    const TIN*      X;
    const TapEntry* tab;
    int             J;          // contraction rows
    PixelLattice    lat;
    int             gs_d, gs_h, gs_w;
    int             lim_d, lim_h, lim_w;

    struct Ctx { int base, z0, y0, x0; };

    __device__ __forceinline__ Ctx prepare(int col) const
    {
        Ctx c;
        if (col >= lat.ncols) { c.base = 0; c.z0 = c.y0 = c.x0 = -0x40000000; return c; }
        const int pix = col / lat.N, nn = col - pix * lat.N;
        const int iz = pix / lat.nxy, rem = pix - iz * lat.nxy;
        const int iy = rem / lat.nx, ix = rem - iy * lat.nx;
        c.z0 = iz * gs_d; c.y0 = iy * gs_h; c.x0 = ix * gs_w;
        c.base = ((c.z0 * lim_h + c.y0) * lim_w + c.x0) * lat.N + nn;
        return c;
    }

    __device__ __forceinline__ uint4_t load(const Ctx& c, int k, int /*zb*/) const
    {
        uint4_t out = {0u, 0u, 0u, 0u};
        if (k < J) {
            const TapEntry e = tab[k];
            if ((unsigned)(c.z0 + e.dz) < (unsigned)lim_d && (unsigned)(c.y0 + e.dy) < (unsigned)lim_h &&
                (unsigned)(c.x0 + e.dx) < (unsigned)lim_w)
                out = ChunkFetch<T, TIN>::get(X + (c.base + e.off));
        }
        return out;
    }
};

// A operand of update (contraction-contiguous tile: rows are filter rows
// j = (c,t,r,s), the contraction index is (output pixel, n)).
template <typename T, typename TIN>
struct GatherRowsLoader {
    const TIN*      X;
    const TapEntry* tab;
    int             J;          // filter rows C*T*R*S
    int             N, kdim;    // kdim = M*P*Q*N
    int             Q, PQ;
    int             str_d, str_h, str_w;
    int             D, H, W;

    typedef TapEntry Ctx;

    __device__ __forceinline__ Ctx prepare(int r) const
    {
        if (r < J) return tab[r];
        Ctx c = {0, -0x40000000, -0x40000000, -0x40000000};
        return c;
    }

    __device__ __forceinline__ uint4_t load(const Ctx& c, int kk, int /*zb*/) const
    {
        uint4_t out = {0u, 0u, 0u, 0u};
        if (kk < kdim) {
            const int pix = kk / N, nn = kk - pix * N;
            const int m = pix / PQ, rem = pix - m * PQ;
            const int p = rem / Q, q = rem - p * Q;
            const int z0 = m * str_d, y0 = p * str_h, x0 = q * str_w;
            if ((unsigned)(z0 + c.dz) < (unsigned)D && (unsigned)(y0 + c.dy) < (unsigned)H &&
                (unsigned)(x0 + c.dx) < (unsigned)W)
                out = ChunkFetch<T, TIN>::get(X + (((z0 * H + y0) * W + x0) * N + nn + c.off));
        }
        return out;
    }
};

// Epilogue of the strided data-gradient classes: column (lattice point, n) of
// class (oz,oy,ox) lands on input pixel (oz + sz*iz, oy + sy*iy, ox + sx*ix).
template <typename T>
struct LatticeStoreEpilogue {
    typedef typename StoreBits<T>::bits_t bits_t;
    T*           out;
    int          rows;         // C
    long         row_stride;   // D*H*W*N
    PixelLattice lat;
    int          oz, oy, ox, sz, sy, sx;
    int          H, W;
    float        alpha;

    __device__ __forceinline__ void store8(int i, int j0, int /*z*/, int /*split*/, const float (&acc)[8]) const
    {
        if (i >= rows || j0 >= lat.ncols) return;
        const int pix = j0 / lat.N, nn = j0 - pix * lat.N;
        const int iz = pix / lat.nxy, rem = pix - iz * lat.nxy;
        const int iy = rem / lat.nx, ix = rem - iy * lat.nx;
        bits_t* p = reinterpret_cast<bits_t*>(
            out + i * row_stride + (long)(((oz + sz * iz) * H + (oy + sy * iy)) * W + (ox + sx * ix)) * lat.N + nn);
        bits_t b[8];
#pragma unroll
        for (int e = 0; e < 8; e++) b[e] = StoreBits<T>::round(acc[e] * alpha, 0, 0, 0, 0);
        constexpr int NV = (int)sizeof(bits_t) * 8 / 16;
#pragma unroll
        for (int q = 0; q < NV; q++) reinterpret_cast<uint4_t*>(p)[q] = reinterpret_cast<const uint4_t*>(b)[q];
    }
};

}  // namespace ng
