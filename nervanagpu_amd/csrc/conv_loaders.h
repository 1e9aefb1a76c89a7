// Operand loaders and epilogues that turn the MFMA contraction core into the
// three convolution operations on CHWN tensors (N innermost):
//
//   fprop   O[k, pix, n]  = sum_j  F[j, k]       * I[gather(j, pix), n]   j = (tap, c)
//   bprop   gI[c, pix, n] = sum_j  Fs[j, c]      * E[gather(j, pix), n]   j = (tap, k)
//   update  gF[j, k]      = sum_(pix,n) I[gather(j, pix), n] * E[k, pix, n]
//
// In all three the row of the activation tensor selected by (j, pix) is one
// contiguous run of N elements, so a 16-byte chunk never straddles a pixel
// (N is a multiple of 8) and gathers stay fully vectorised.  Taps that fall
// outside the image read as zero through the out-of-range offset of the raw
// buffer load, so the loaders are branch free.
//
// "Blocked" loaders order the contraction tap-major with a whole block of BK
// channels (fprop: input channels, bprop: output channels) per tile: the tap,
// and with it the validity of a pixel, is uniform for a tile and the BK rows
// differ by a constant stride.  "Flat" loaders take any row order from a table
// with one entry per contraction row (used when the channel count is not a
// multiple of BK, e.g. the C=3 first layers).
//
// Semantics follow the reference's numpy statement of the operation
// (benchmarks/conv_test.py:99-167) and the index formulas of
// kernels/sass/hconv_fprop_K64_N64.sass:188-240.
#pragma once

#include "gemm_core.h"

#include <type_traits>

namespace ng {

// a tap (or, in flat tables, one contraction row): element offset relative to
// the pixel origin and the coordinate deltas for the bounds test
struct TapEntry { int off, dz, dy, dx; };

typedef unsigned char u8_t;
typedef signed char   s8_t;

// 16-byte chunk of compute type T from storage type TIN via a raw buffer load
template <typename T, typename TIN> struct ChunkFetch;

template <typename T> struct ChunkFetch<T, T> {
    static constexpr int ES = (int)sizeof(T);
    static __device__ __forceinline__ uint4_t get(BufferRsrc r, unsigned byte_off) { return buffer_load_chunk(r, byte_off); }
};

// bytes -> fp16, exact for every 8-bit value (I2F on load in the reference,
// kernels/sass/hconv_updat_C64_K64.sass:324-345)
template <> struct ChunkFetch<_Float16, u8_t> {
    static constexpr int ES = 1;
    static __device__ __forceinline__ uint4_t get(BufferRsrc r, unsigned byte_off)
    {
        typedef unsigned uint2_t __attribute__((ext_vector_type(2)));
        const uint2_t raw = __builtin_amdgcn_raw_buffer_load_b64(r, (int)byte_off, 0, 0);
        _Float16 h[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e]     = (_Float16)(float)((raw[0] >> (8 * e)) & 0xFFu);
            h[e + 4] = (_Float16)(float)((raw[1] >> (8 * e)) & 0xFFu);
        }
        return *reinterpret_cast<const uint4_t*>(h);
    }
};

template <> struct ChunkFetch<_Float16, s8_t> {
    static constexpr int ES = 1;
    static __device__ __forceinline__ uint4_t get(BufferRsrc r, unsigned byte_off)
    {
        typedef unsigned uint2_t __attribute__((ext_vector_type(2)));
        const uint2_t raw = __builtin_amdgcn_raw_buffer_load_b64(r, (int)byte_off, 0, 0);
        _Float16 h[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e]     = (_Float16)(float)(int)(signed char)((raw[0] >> (8 * e)) & 0xFFu);
            h[e + 4] = (_Float16)(float)(int)(signed char)((raw[1] >> (8 * e)) & 0xFFu);
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
    FastDiv div_n, div_nxy, div_nx;

    static PixelLattice make(int N, int ncols, int nx, int nxy)
    {
        return PixelLattice{N, ncols, nx, nxy, FastDiv::make((unsigned)N), FastDiv::make((unsigned)nxy),
                            FastDiv::make((unsigned)nx)};
    }
    // column -> (iz, iy, ix, n)
    __device__ __forceinline__ void split(int col, int& iz, int& iy, int& ix, int& nn) const
    {
        const int pix = (int)div_n.div((unsigned)col);
        nn = col - pix * N;
        iz = (int)div_nxy.div((unsigned)pix);
        const int rem = pix - iz * nxy;
        iy = (int)div_nx.div((unsigned)rem);
        ix = rem - iy * nx;
    }
};

#define NG_FAR (-0x40000000)

// contraction tile index -> (tap, channel block); div divides by nblk when
// block_major_taps == 0 and by block_major_taps otherwise
__device__ __forceinline__ void decode_tile(int kt, const FastDiv& div, int nblk, int block_major_taps, int& tap, int& blk)
{
    const int hi = (int)div.div((unsigned)kt);
    if (block_major_taps) { blk = hi; tap = kt - hi * block_major_taps; }
    else                  { tap = hi; blk = kt - hi * nblk; }
}

// B operand of fprop / bprop (row-contiguous tile: lines are contraction rows,
// columns are (pixel, n)).  Gathered coordinate of a tap at lattice point
// (iz,iy,ix) is (iz*gs_d + dz, iy*gs_h + dy, ix*gs_w + dx) inside a
// (lim_d, lim_h, lim_w) volume.
template <typename T, typename TIN, bool BLOCKED, int BK>
struct GatherColsLoader {
    const TIN*      X;
    const TapEntry* tab;        // BLOCKED: one entry per tap; flat: one per contraction row
    int             J;          // contraction rows
    PixelLattice    lat;
    int             gs_d, gs_h, gs_w;
    int             lim_d, lim_h, lim_w;
    int             row_stride; // BLOCKED: elements between consecutive rows of a block
    FastDiv         blk_div;    // BLOCKED: tile index / nblk (blocks per tap) or / ntaps, see block_major
    int             nblk;
    int             chan;       // BLOCKED: rows per tap; the last block of a tap may be partly empty
    // BLOCKED tile order.  0: tap-major (all channel blocks of a tap, then the next
    // tap).  ntaps > 0: block-major (all taps of a channel block, then the next
    // block): the taps of one block re-read the same activations shifted by a
    // pixel or a row, so the share an XCD works on stays in its L2 across the
    // taps (tap-major re-fetched the data gradient's E of a 5x5 layer 8.7 times
    // from HBM).  The A operand's loader must use the same order.
    int             block_major_taps;
    // BLOCKED: entries of `tab`.  A table of at most 64 taps is kept in registers,
    // lane l holding entry l, and a tile fetches its tap with v_readlane: no memory
    // access (and no wait for one) between the barrier of a tile step and its
    // requests.  0 = not stated: tile() reads the table from memory.
    int             ntaps = 0;

    // same-type inputs are plain 16-byte buffer loads (see DenseLoader::DIRECT)
    static constexpr bool DIRECT = std::is_same<T, TIN>::value;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { int base, z0, y0, x0, kr; };
    // k0: flat: first contraction row of the tile; BLOCKED: rows of the block that exist
    struct Tile { BufferRsrc rsrc; int toff, dz, dy, dx, k0; };
    struct Wave { int off, dz, dy, dx; };

    __device__ __forceinline__ bool lane_table() const { return ntaps > 0 && ntaps <= 64; }
    __device__ __forceinline__ Wave wave_init(int lane) const
    {
        Wave w{0, 0, 0, 0};
        if (BLOCKED && lane_table()) {
            const TapEntry e = tab[min(lane, ntaps - 1)];
            w.off = e.off; w.dz = e.dz; w.dy = e.dy; w.dx = e.dx;
        }
        return w;
    }

    __device__ __forceinline__ Ctx prepare(int col, int kr) const
    {
        Ctx c;
        c.kr = kr;
        if (col >= lat.ncols) { c.base = 0; c.z0 = c.y0 = c.x0 = NG_FAR; return c; }
        int iz, iy, ix, nn;
        lat.split(col, iz, iy, ix, nn);
        c.z0 = iz * gs_d; c.y0 = iy * gs_h; c.x0 = ix * gs_w;
        c.base = ((c.z0 * lim_h + c.y0) * lim_w + c.x0) * lat.N + nn;
        if (BLOCKED) c.base += kr * row_stride;
        return c;
    }

    __device__ __forceinline__ Tile tile(int kt, int k0, int /*zb*/, const Wave& w) const
    {
        Tile t;
        t.rsrc = make_rsrc(X);
        t.k0 = k0;
        if (BLOCKED) {
            int tap, blk;
            decode_tile(kt, blk_div, nblk, block_major_taps, tap, blk);
            TapEntry e;
            if (lane_table()) {
                e.off = __builtin_amdgcn_readlane(w.off, tap); e.dz = __builtin_amdgcn_readlane(w.dz, tap);
                e.dy = __builtin_amdgcn_readlane(w.dy, tap);   e.dx = __builtin_amdgcn_readlane(w.dx, tap);
            } else {
                e = tab[tap];
            }
            t.toff = e.off + blk * BK * row_stride;
            t.dz = e.dz; t.dy = e.dy; t.dx = e.dx;
            t.k0 = chan - blk * BK;
        } else {
            t.toff = 0; t.dz = t.dy = t.dx = 0;
        }
        return t;
    }

    // byte offset of the chunk, out of range for taps outside the image
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        constexpr int ES = ChunkFetch<T, TIN>::ES;
        if (BLOCKED) {
            // bitwise, not short-circuit: the four tests and the offset are computed
            // unconditionally, so no execution-mask branches surround the request
            const bool ok = ((unsigned)(c.z0 + t.dz) < (unsigned)lim_d) & ((unsigned)(c.y0 + t.dy) < (unsigned)lim_h) &
                            ((unsigned)(c.x0 + t.dx) < (unsigned)lim_w) & (c.kr < t.k0);
            const unsigned off = (unsigned)(c.base + t.toff) * ES;
            return ok ? off : NG_OOB_OFFSET;
        } else {
            const int k = t.k0 + c.kr;
            const TapEntry e = tab[min(k, J - 1)];
            const bool ok = k < J && (unsigned)(c.z0 + e.dz) < (unsigned)lim_d &&
                            (unsigned)(c.y0 + e.dy) < (unsigned)lim_h && (unsigned)(c.x0 + e.dx) < (unsigned)lim_w;
            return ok ? (unsigned)(c.base + e.off) * ES : NG_OOB_OFFSET;
        }
    }

    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const
    {
        return ChunkFetch<T, TIN>::get(t.rsrc, offset(t, c));
    }
};

// A operand of blocked fprop: filter F[c][tap][k] read as rows j = (tap, c):
// tile (tap, block) holds channels block*BK .. +BK-1, consecutive rows are
// RST*K elements apart.  The last block of a tap may reach past channel C-1:
// those rows are not read (zero operands).
template <typename T, int BK>
struct FilterBlockLoader {
    const T* F;
    int      K;          // row length (output feature maps)
    int      RSTK;       // elements between consecutive channels
    FastDiv  tap_div;    // tile index -> channel block (block-major order, ntaps tiles per block)
    int      ntaps;
    int      C;          // channels

    static constexpr bool DIRECT = true;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { unsigned off; int kr; };
    struct Tile { BufferRsrc rsrc; int rows; };
    typedef NoWaveState Wave;
    __device__ __forceinline__ Wave wave_init(int /*lane*/) const { return Wave{}; }

    __device__ __forceinline__ Ctx prepare(int m, int kr) const
    {
        Ctx c;
        c.off = (m < K) ? (unsigned)(kr * RSTK + m) * (unsigned)sizeof(T) : NG_OOB_OFFSET;
        c.kr = kr;
        return c;
    }
    __device__ __forceinline__ Tile tile(int kt, int /*k0*/, int /*zb*/, const Wave&) const
    {
        const int blk = (int)tap_div.div((unsigned)kt);
        const int tap = kt - blk * ntaps;
        Tile t;
        t.rsrc = make_rsrc(F + (long)blk * BK * RSTK + (long)tap * K);
        t.rows = C - blk * BK;
        return t;
    }
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        return c.kr < t.rows ? c.off : NG_OOB_OFFSET;
    }
    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const { return buffer_load_chunk(t.rsrc, offset(t, c)); }
};

// ---- forward convolution with the horizontal taps of a filter row sharing one
// ---- activation tile (unit strides) ------------------------------------------------
// A contraction tile is (channel block, t, r): its B tile holds, for BK channels,
// the input row segment under the tile's PIX = BN / N consecutive output pixels,
// PIX + S - 1 pixels wide, and tap s multiplies the window that starts s pixels
// (N columns) into it.  The S taps of a filter row thus move the activations
// from L2 to LDS once instead of S times; the A tile stacks the S filter slices
// (tap-major, BK channels each).
//
// B operand.  Output pixels of a tile must lie in one image row (the host checks
// Q % PIX == 0).  Column r of the tile is input pixel x = q0 - pad_w + r / N of
// image n = r % N; x outside the image reads zero, whatever the tap.
template <typename T, int BK, int TAPS_, int TAP_COLS_>
struct GatherRowSegLoader {
    static constexpr int TAPS = TAPS_, TAP_COLS = TAP_COLS_;
    const T*     X;
    PixelLattice lat;          // output pixels (M, P, Q) x N
    int          D, H, W;
    int          pad_d, pad_h, pad_w;
    int          row_stride;   // elements between consecutive channels (D*H*W*N)
    FastDiv      tr_div, r_div;
    int          TR, R;        // filter rows (t, r) per channel block; R
    int          chan;         // channels

    static constexpr bool DIRECT = true;
    static constexpr bool TILE_READS_TABLE = false;

    // The image row (z, y) of a tile is the same for all its chunks and the filter
    // row of a contraction tile is uniform anyway, so the row test runs on the
    // scalar unit; per lane remain one add and one select.  The channel count is a
    // multiple of BK (the host checks), so no chunk lies past the last channel.
    struct Ctx { unsigned base; int z0, y0; bool xok; };
    struct Tile { BufferRsrc rsrc; int toff, dz, dy; int blk, ft, fr; };
    typedef NoWaveState Wave;
    __device__ __forceinline__ Wave wave_init(int /*lane*/) const { return Wave{}; }

    __device__ __forceinline__ Ctx prepare_seg(int n0, int r, int kr) const
    {
        Ctx c;
        int iz, iy, ix0, nn0;
        lat.split(min(n0, lat.ncols - 1), iz, iy, ix0, nn0);
        const int pix = r / TAP_COLS, nn = r - pix * TAP_COLS;
        const int ix = ix0 + pix - pad_w;
        c.xok = (n0 < lat.ncols) & ((unsigned)ix < (unsigned)W);
        c.z0 = __builtin_amdgcn_readfirstlane(iz);
        c.y0 = __builtin_amdgcn_readfirstlane(iy);
        c.base = (unsigned)(((iz * H + iy) * W + ix) * lat.N + nn + kr * row_stride) * (unsigned)sizeof(T);
        return c;
    }
    __device__ __forceinline__ void place(Tile& t) const
    {
        t.dz = t.ft - pad_d; t.dy = t.fr - pad_h;
        t.toff = ((t.dz * H + t.dy) * W * lat.N + t.blk * BK * row_stride) * (int)sizeof(T);
    }
    __device__ __forceinline__ Tile tile(int kt, int /*k0*/, int /*zb*/, const Wave&) const
    {
        Tile t;
        t.rsrc = make_rsrc(X);
        t.blk = (int)tr_div.div((unsigned)kt);
        const int tr = kt - t.blk * TR;
        t.ft = (int)r_div.div((unsigned)tr);
        t.fr = tr - t.ft * R;
        place(t);
        return t;
    }
    // next contraction tile: filter rows (t, r) are the fast index, channel blocks the slow one
    static constexpr bool INCREMENTAL = true;
    __device__ __forceinline__ void advance(Tile& t, int /*bk*/) const
    {
        if (++t.fr == R) {
            t.fr = 0;
            if (++t.ft * R == TR) { t.ft = 0; t.blk++; }
        }
        place(t);
    }
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        const bool rowok = ((unsigned)(c.z0 + t.dz) < (unsigned)D) & ((unsigned)(c.y0 + t.dy) < (unsigned)H);
        return (rowok & c.xok) ? c.base + (unsigned)t.toff : NG_OOB_OFFSET;
    }
    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const { return buffer_load_chunk(t.rsrc, offset(t, c)); }
};

// A operand of the same kernel: line s * BK + c of tile (block, t, r) is filter
// row (channel block*BK + c, t, r, s), K contiguous output maps each.
template <typename T, int BK, int TAPS>
struct FilterTapRowLoader {
    const T* F;
    int      K;
    int      RSTK;       // elements between consecutive channels
    FastDiv  tr_div;
    int      TR;         // filter rows (t, r)
    int      C;

    static constexpr bool DIRECT = true;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { unsigned off; int c; };
    struct Tile { BufferRsrc rsrc; const T* p; int rows, tr; };
    typedef NoWaveState Wave;
    __device__ __forceinline__ Wave wave_init(int /*lane*/) const { return Wave{}; }

    __device__ __forceinline__ Ctx prepare(int m, int kr) const
    {
        Ctx c;
        const int tap = kr / BK;
        c.c = kr - tap * BK;
        c.off = (m < K) ? (unsigned)(c.c * RSTK + tap * K + m) * (unsigned)sizeof(T) : NG_OOB_OFFSET;
        return c;
    }
    __device__ __forceinline__ Tile tile(int kt, int /*k0*/, int /*zb*/, const Wave&) const
    {
        const int blk = (int)tr_div.div((unsigned)kt);
        Tile t;
        t.tr = kt - blk * TR;
        t.p = F + (long)blk * BK * RSTK + (long)t.tr * TAPS * K;
        t.rsrc = make_rsrc(t.p);
        t.rows = C - blk * BK;
        return t;
    }
    // next contraction tile: the next filter row, or the first one of the next channel block
    static constexpr bool INCREMENTAL = true;
    __device__ __forceinline__ void advance(Tile& t, int /*bk*/) const
    {
        t.p += TAPS * K;
        if (++t.tr == TR) {
            t.tr = 0;
            t.p += (long)BK * RSTK - (long)TR * TAPS * K;
            t.rows -= BK;
        }
        t.rsrc = make_rsrc(t.p);
    }
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        return c.c < t.rows ? c.off : NG_OOB_OFFSET;
    }
    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const { return buffer_load_chunk(t.rsrc, offset(t, c)); }
};

// A operand of the data gradient with shared taps: rows are channels c, the
// contraction is (mirrored tap s', output map k) over BK output maps, k contiguous.
// Tile (block, t', r') reads filter row (T-1-t', R-1-r'): the data gradient at
// pixel x sums E at x + pad - s, so with mirrored taps it is a forward gather
// over E with padding (T-1-pad_d, R-1-pad_h, S-1-pad_w), served by
// GatherRowSegLoader.  The TAPS filter columns are one row of the filter (S = TAPS).
template <typename T, int BK, int TAPS>
struct FilterTapColsLoader {
    const T* F;
    int      C;          // rows
    int      K;          // output maps
    int      RSTK;       // elements between consecutive channels
    FastDiv  tr_div, r_div;
    int      TR, R;      // filter rows (t, r); R

    static constexpr bool DIRECT = true;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { unsigned off; int kc; };
    struct Tile { BufferRsrc rsrc; const T* p; int kvalid, tr; };
    typedef NoWaveState Wave;
    __device__ __forceinline__ Wave wave_init(int /*lane*/) const { return Wave{}; }

    __device__ __forceinline__ Ctx prepare(int m, int kr) const
    {
        Ctx c;
        const int tap = kr / BK;
        c.kc = kr - tap * BK;
        c.off = (m < C) ? (unsigned)(m * RSTK + (TAPS - 1 - tap) * K + c.kc) * (unsigned)sizeof(T) : NG_OOB_OFFSET;
        return c;
    }
    // tile (block, t', r') reads filter row TR-1 - (t'*R + r') (both coordinates mirrored)
    __device__ __forceinline__ Tile tile(int kt, int /*k0*/, int /*zb*/, const Wave&) const
    {
        const int blk = (int)tr_div.div((unsigned)kt);
        Tile t;
        t.tr = kt - blk * TR;
        t.p = F + (long)(TR - 1 - t.tr) * TAPS * K + (long)blk * BK;
        t.rsrc = make_rsrc(t.p);
        t.kvalid = K - blk * BK;
        return t;
    }
    // next contraction tile: the filter row before, or the last one for the next block of output maps
    static constexpr bool INCREMENTAL = true;
    __device__ __forceinline__ void advance(Tile& t, int /*bk*/) const
    {
        t.p -= TAPS * K;
        if (++t.tr == TR) {
            t.tr = 0;
            t.p += (long)TR * TAPS * K + BK;
            t.kvalid -= BK;
        }
        t.rsrc = make_rsrc(t.p);
    }
    // K is a multiple of the chunk length, so a chunk is inside or outside as a whole
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        return c.kc < t.kvalid ? c.off : NG_OOB_OFFSET;
    }
    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const { return buffer_load_chunk(t.rsrc, offset(t, c)); }
};

// Data gradient of a layer with very few channels (3 * C <= 32, filter rows of
// three taps, unit strides, N = 64).  Rows are (c, s): G[(c,s)][z,y,x'] = sum over
// (t, r, k) of F[c,t,r,s,k] * E[k, z+pad_d-t, y+pad_h-r, x'], so the horizontal
// tap never enters the contraction (192 deep for 64 output maps instead of 576)
// and the 32 rows of a matrix instruction hold three taps of every channel
// instead of the channels alone.  The epilogue adds the three taps of a channel at
// columns shifted by one pixel each: gradI[c,z,y,x] = sum_s G[(c,s)][z,y,x+pad_w-s].
//
// A workgroup's tile is one strip of an image row: HALO_PIX = OUT_PIX + 2 pixels
// of E (x' from x0 + pad_w - 2) give OUT_PIX pixels of the gradient from x0 =
// OUT_PIX * (strip index).  Column tiles are numbered (z*H + y) * strips + strip.
//
// The tiles are numbered down the image: tile = strip * (D*H) + (z*H + y), so that
// consecutive tiles of a workgroup's run are vertically adjacent and share two of
// the three rows of E they read (numbered along the rows, every load missed the
// L2: FETCH_SIZE showed 3.9 x |E| for a 3x3 filter).
//
// A operand: line kc of tile (t, r, block) for row (c, s) is F[c][t][r][s][block*BK + kc].
// tile -> (image row zy, strip): `rows_div` divides by the number of image rows D*H
__device__ __forceinline__ void strip_of_tile(int tile, const FastDiv& rows_div, int img_rows, int& zy, int& strip)
{
    strip = (int)rows_div.div((unsigned)tile);
    zy = tile - strip * img_rows;
}

template <typename T, int BK>
struct FilterChannelTapLoader {
    const T* F;
    int      rows;       // 3 * C
    int      K;
    int      RSTK;       // elements between consecutive channels
    FastDiv  blk_div;    // tile index -> filter row (t, r); blocks of output maps are the fast index
    int      nblk;

    static constexpr bool DIRECT = true;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { unsigned off; int kc; };
    struct Tile { BufferRsrc rsrc; int kvalid; };
    typedef NoWaveState Wave;
    __device__ __forceinline__ Wave wave_init(int /*lane*/) const { return Wave{}; }

    __device__ __forceinline__ Ctx prepare(int m, int kc) const
    {
        Ctx c;
        const int ch = m / 3, tap = m - ch * 3;
        c.kc = kc;
        c.off = (m < rows) ? (unsigned)(ch * RSTK + tap * K + kc) * (unsigned)sizeof(T) : NG_OOB_OFFSET;
        return c;
    }
    __device__ __forceinline__ Tile tile(int kt, int /*k0*/, int /*zb*/, const Wave&) const
    {
        const int tr = (int)blk_div.div((unsigned)kt);
        const int blk = kt - tr * nblk;
        Tile t;
        t.rsrc = make_rsrc(F + (long)tr * 3 * K + (long)blk * BK);
        t.kvalid = K - blk * BK;
        return t;
    }
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        return c.kc < t.kvalid ? c.off : NG_OOB_OFFSET;
    }
    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const { return buffer_load_chunk(t.rsrc, offset(t, c)); }
};

// B operand of the same kernel: column r of tile (z, y, strip) is pixel
// x' = strip*OUT_PIX + pad_w - 2 + r / N of E row (z + pad_d - t, y + pad_h - r_f),
// image r % N; everything outside E reads zero.
template <typename T, int BK, int BN, int OUT_PIX>
struct HaloStripLoader {
    const T* E;
    int      M, P, Q;        // extents of E
    int      N;
    int      row_stride;     // elements between consecutive output maps (M*P*Q*N)
    int      ncols;          // tiles * BN
    FastDiv  imgrow_div, h_div;
    int      img_rows, H;    // image rows D*H; image rows per depth slice
    int      pad_d, pad_h, pad_w;
    FastDiv  blk_div, r_div;
    int      nblk, R, K;

    static constexpr bool DIRECT = true;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { int base, z0, y0, kr; };
    struct Tile { BufferRsrc rsrc; int toff, dz, dy, k0; };
    typedef NoWaveState Wave;
    __device__ __forceinline__ Wave wave_init(int /*lane*/) const { return Wave{}; }

    __device__ __forceinline__ Ctx prepare(int col, int kr) const
    {
        Ctx c;
        c.kr = kr;
        c.base = 0; c.z0 = c.y0 = NG_FAR;
        if (col >= ncols) return c;
        const int tile = col / BN, r = col - tile * BN;
        int zy, strip;
        strip_of_tile(tile, imgrow_div, img_rows, zy, strip);
        const int z = (int)h_div.div((unsigned)zy);
        const int y = zy - z * H;
        const int pix = r / N, nn = r - pix * N;
        const int x = strip * OUT_PIX + pad_w - 2 + pix;
        if ((unsigned)x >= (unsigned)Q) return c;
        c.z0 = z + pad_d; c.y0 = y + pad_h;
        c.base = ((c.z0 * P + c.y0) * Q + x) * N + nn + kr * row_stride;
        return c;
    }
    __device__ __forceinline__ Tile tile(int kt, int /*k0*/, int /*zb*/, const Wave&) const
    {
        Tile t;
        t.rsrc = make_rsrc(E);
        const int tr = (int)blk_div.div((unsigned)kt);
        const int blk = kt - tr * nblk;
        const int ft = (int)r_div.div((unsigned)tr);
        const int fr = tr - ft * R;
        t.dz = -ft; t.dy = -fr;
        t.toff = (t.dz * P + t.dy) * Q * N + blk * BK * row_stride;
        t.k0 = K - blk * BK;
        return t;
    }
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        const bool ok = ((unsigned)(c.z0 + t.dz) < (unsigned)M) & ((unsigned)(c.y0 + t.dy) < (unsigned)P) & (c.kr < t.k0);
        const unsigned off = (unsigned)(c.base + t.toff) * (unsigned)sizeof(T);
        return ok ? off : NG_OOB_OFFSET;
    }
    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const { return buffer_load_chunk(t.rsrc, offset(t, c)); }
};

// Epilogue of the same kernel: g holds the fp32 tile, rows (c, s), BN columns
// (HALO_PIX pixels x N images).  Output pixel i of the strip adds column block
// i + 2 - s of row (c, s) over the three taps, in that order; one rounding.
template <typename T, int BN, int OUT_PIX, int MAX_ROWS_ = 32>
struct ShiftSumStoreEpilogue {
    static constexpr bool WHOLE_TILE = true;
    static constexpr int MAX_ROWS = MAX_ROWS_;   // rows the streaming kernel parks (3 * C at most)
    typedef typename StoreBits<T>::bits_t bits_t;
    T*      out;
    int     rows;          // 3 * C
    long    chan_stride;   // D*H*W*N
    int     W, N;
    FastDiv imgrow_div;
    int     img_rows;      // image rows D*H
    float   alpha;

    __device__ __forceinline__ const void* base() const { return out; }
    // the same for the streaming kernel: exactly one descriptor store per thread
    // (3 * C <= MAX_ROWS <= 16 keeps the 8-element pieces of a strip within 256
    // threads); threads without a piece store out of range
    static constexpr int STORES_PER_THREAD = 1;
    __device__ __forceinline__ void tile_buffer(BufferRsrc rsrc, const float* g, int tid, int n0) const
    {
        int zy, strip;
        strip_of_tile(n0 / BN, imgrow_div, img_rows, zy, strip);
        const int x0 = strip * OUT_PIX;
        const int per_chan = OUT_PIX * (N / 8);
        const int chans = rows / 3;
        const int c = tid / per_chan, rem = tid - c * per_chan;
        const int i = rem / (N / 8), n8 = (rem - i * (N / 8)) * 8;
        const int x = x0 + i;
        const int cr = min(c, chans - 1);   // keeps the LDS reads of idle threads inside the parked rows
        float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int s = 0; s < 3; s++) {
            const float* p = g + (cr * 3 + s) * BN + (i + 2 - s) * N + n8;
            const float4_t lo = *reinterpret_cast<const float4_t*>(p);
            const float4_t hi = *reinterpret_cast<const float4_t*>(p + 4);
#pragma unroll
            for (int q = 0; q < 4; q++) { sum[q] += lo[q]; sum[4 + q] += hi[q]; }
        }
        bits_t r[8];
#pragma unroll
        for (int q = 0; q < 8; q++) r[q] = StoreBits<T>::round(sum[q] * alpha, 0, 0, 0, 0);
        const long e = (long)c * chan_stride + ((long)zy * W + x) * N + n8;
        const unsigned off = (c < chans && x < W) ? (unsigned)e * 2u : NG_OOB_OFFSET;
        buffer_store_chunk(rsrc, off, *reinterpret_cast<const uint4_t*>(r));
    }

    __device__ __forceinline__ void tile(const float* g, int tid, int nthreads, int n0) const
    {
        int zy, strip;
        strip_of_tile(n0 / BN, imgrow_div, img_rows, zy, strip);
        const int x0 = strip * OUT_PIX;
        const int per_chan = OUT_PIX * (N / 8);
        const int total = (rows / 3) * per_chan;
        for (int e = tid; e < total; e += nthreads) {
            const int c = e / per_chan, rem = e - c * per_chan;
            const int i = rem / (N / 8), n8 = (rem - i * (N / 8)) * 8;
            const int x = x0 + i;
            if (x >= W) continue;
            float sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int s = 0; s < 3; s++) {
                const float* p = g + (c * 3 + s) * BN + (i + 2 - s) * N + n8;
                const float4_t lo = *reinterpret_cast<const float4_t*>(p);
                const float4_t hi = *reinterpret_cast<const float4_t*>(p + 4);
#pragma unroll
                for (int q = 0; q < 4; q++) { sum[q] += lo[q]; sum[4 + q] += hi[q]; }
            }
            bits_t r[8];
#pragma unroll
            for (int q = 0; q < 8; q++) r[q] = StoreBits<T>::round(sum[q] * alpha, 0, 0, 0, 0);
            bits_t* dst = reinterpret_cast<bits_t*>(out) + (long)c * chan_stride + ((long)zy * W + x) * N + n8;
            *reinterpret_cast<uint4_t*>(dst) = *reinterpret_cast<const uint4_t*>(r);
        }
    }
};

// ---- gather functors of the streaming kernel (stream_core.h) --------------------
// Both describe a chunk as base(column) + off(contraction row), valid when the
// column's pixel shifted by the row's (dz, dy, dx) lies inside the tensor.
struct StreamFixed { int off, dz, dy, dx; };
struct StreamCol { int base, z0, y0, x0; };

template <typename T>
__device__ __forceinline__ unsigned stream_offset(const StreamFixed& f, const StreamCol& c, int lim_d, int lim_h, int lim_w)
{
    const bool ok = ((unsigned)(c.z0 + f.dz) < (unsigned)lim_d) & ((unsigned)(c.y0 + f.dy) < (unsigned)lim_h) &
                    ((unsigned)(c.x0 + f.dx) < (unsigned)lim_w);
    const unsigned off = (unsigned)(c.base + f.off) * (unsigned)sizeof(T);
    return ok ? off : NG_OOB_OFFSET;
}

// forward convolution, contraction rows (c, t, r, s) from the flat tap table
template <typename T>
struct FlatTapGather {
    const T*        X;
    const TapEntry* tab;
    int             J;
    PixelLattice    lat;
    int             gs_d, gs_h, gs_w;
    int             lim_d, lim_h, lim_w;
    typedef StreamFixed Fixed;
    typedef StreamCol Col;

    __device__ __forceinline__ Fixed fixed(int j) const
    {
        if (j >= J) return Fixed{0, NG_FAR, NG_FAR, NG_FAR};
        const TapEntry e = tab[j];
        return Fixed{e.off, e.dz, e.dy, e.dx};
    }
    __device__ __forceinline__ Col col(int c) const
    {
        if (c >= lat.ncols) return Col{0, NG_FAR, NG_FAR, NG_FAR};
        int iz, iy, ix, nn;
        lat.split(c, iz, iy, ix, nn);
        Col o;
        o.z0 = iz * gs_d; o.y0 = iy * gs_h; o.x0 = ix * gs_w;
        o.base = ((o.z0 * lim_h + o.y0) * lim_w + o.x0) * lat.N + nn;
        return o;
    }
    __device__ __forceinline__ unsigned offset(const Fixed& f, const Col& c) const
    {
        return stream_offset<T>(f, c, lim_d, lim_h, lim_w);
    }
};

// Forward convolution of a first layer with a large filter (few channels, 7x7 or 11x11 taps: more
// contraction rows than the flat gather above can keep a table entry for in registers).  What
// contraction row j = ((c * T + t) * R + r) * S + s contributes is decoded from j itself: tile lines
// are whole wavefront requests, so j is uniform and the three divisions run on the scalar unit; a lane
// keeps one column descriptor per column tile, and a request costs three compares and an add.
template <typename T>
struct TapDecodeGather {
    const T*     X;
    int          J;                   // contraction rows C * T * R * S
    PixelLattice lat;                 // output pixels (m, p, q) x n
    int          str_d, str_h, str_w;
    int          pad_d, pad_h, pad_w;
    int          D, H, W;
    int          T_, R, S;
    FastDiv      s_div, r_div, t_div;
    static constexpr bool FIXED_ON_DEMAND = true;
    typedef StreamFixed Fixed;
    typedef StreamCol Col;

    __device__ __forceinline__ Fixed fixed(int j) const
    {
        if (j >= J) return Fixed{0, NG_FAR, NG_FAR, NG_FAR};
        const int crt = (int)s_div.div((unsigned)j), s = j - crt * S;
        const int ct = (int)r_div.div((unsigned)crt), r = crt - ct * R;
        const int c = (int)t_div.div((unsigned)ct), t = ct - c * T_;
        Fixed f;
        f.off = __builtin_amdgcn_readfirstlane((((c * D + t) * H + r) * W + s) * lat.N);
        f.dz = __builtin_amdgcn_readfirstlane(t);
        f.dy = __builtin_amdgcn_readfirstlane(r);
        f.dx = __builtin_amdgcn_readfirstlane(s);
        return f;
    }
    // the origin of the column's receptive field (its first tap may lie in the padding)
    __device__ __forceinline__ Col col(int c) const
    {
        if (c >= lat.ncols) return Col{0, NG_FAR, NG_FAR, NG_FAR};
        int m, p, q, nn;
        lat.split(c, m, p, q, nn);
        Col o;
        o.z0 = m * str_d - pad_d; o.y0 = p * str_h - pad_h; o.x0 = q * str_w - pad_w;
        o.base = ((o.z0 * H + o.y0) * W + o.x0) * lat.N + nn;
        return o;
    }
    __device__ __forceinline__ unsigned offset(const Fixed& f, const Col& c) const
    {
        return stream_offset<T>(f, c, D, H, W);
    }
};

// data gradient with rows (channel, horizontal tap): contraction rows
// ((t, r), output map), columns the halo strips of HaloStripLoader.
// A line of the tile (BN = 512 columns) is exactly one wavefront request, so what
// a contraction row contributes is uniform over the wavefront, and so is the image
// row of a column tile: those parts are kept in scalar registers and the row test
// runs on the scalar unit; per lane remain one add and one select per request.
template <typename T, int BK, int BN, int OUT_PIX>
struct HaloStripGather {
    static_assert(BN * sizeof(T) == 64 * 16, "one line of the tile per wavefront request");
    const T* X;              // E
    int      M, P, Q, N;
    int      row_stride;     // M*P*Q*N
    int      ncols;
    FastDiv  imgrow_div, h_div;
    int      img_rows, H;
    int      pad_d, pad_h, pad_w;
    FastDiv  blk_div, r_div;
    int      nblk, R, K;
    static constexpr bool FIXED_PER_TILE = true;
    struct Fixed { int off, dz, dy, kleft; };            // uniform: byte offset of the tile's first row, row shifts, rows that exist
    struct Col { unsigned base; int z0, y0; bool xok; }; // z0, y0 uniform; base, xok per lane

    // j: first contraction row of a tile
    __device__ __forceinline__ Fixed fixed(int j) const
    {
        const int kt = j / BK;
        const int tr = (int)blk_div.div((unsigned)kt);
        const int k0 = (kt - tr * nblk) * BK;
        const int ft = (int)r_div.div((unsigned)tr);
        const int fr = tr - ft * R;
        Fixed f;
        f.off = __builtin_amdgcn_readfirstlane(((-ft * P - fr) * Q * N + k0 * row_stride) * (int)sizeof(T));
        f.dz = __builtin_amdgcn_readfirstlane(-ft);
        f.dy = __builtin_amdgcn_readfirstlane(-fr);
        f.kleft = __builtin_amdgcn_readfirstlane(K - k0);
        return f;
    }
    __device__ __forceinline__ Col col(int c) const
    {
        const int cc = min(c, ncols - 1);
        const int tile = cc / BN, r = cc - tile * BN;
        int zy, strip;
        strip_of_tile(tile, imgrow_div, img_rows, zy, strip);
        zy = __builtin_amdgcn_readfirstlane(zy);
        const int z = (int)h_div.div((unsigned)zy);
        const int y = zy - z * H;
        const int pix = r / N, nn = r - pix * N;
        const int x = strip * OUT_PIX + pad_w - 2 + pix;
        Col o;
        o.z0 = z + pad_d; o.y0 = y + pad_h;
        o.xok = (c < ncols) & ((unsigned)x < (unsigned)Q);
        o.base = (unsigned)(((o.z0 * P + o.y0) * Q + x) * N + nn) * (unsigned)sizeof(T);
        return o;
    }
    // kr: row inside the tile (uniform over the wavefront)
    __device__ __forceinline__ unsigned offset(const Fixed& f, int kr, const Col& c) const
    {
        const bool rowok = ((unsigned)(c.z0 + f.dz) < (unsigned)M) & ((unsigned)(c.y0 + f.dy) < (unsigned)P) & (kr < f.kleft);
        return (rowok & c.xok) ? c.base + (unsigned)(f.off + kr * row_stride * (int)sizeof(T)) : NG_OOB_OFFSET;
    }
};

// A operand of the blocked data gradient: the filter F[c][trs][k] in place,
// read as rows c with the contraction (tap, k): for one tap the k values of a
// row are contiguous, so tile (tap, block) is a contraction-contiguous tile of
// rows RST*K elements apart starting at trs(tap)*K + block*BK.  The taps of a
// residue class come from a small table (filter position of each class tap);
// the last block of a tap may reach past k = K-1: those chunks are not read.
template <typename T, int BK>
struct FilterRowsLoader {
    const T*   F;
    const int* tap_trs;   // filter position (t*R + r)*S + s of each tap of the class
    int        C;         // rows
    int        K;         // contraction extent per tap
    int        RSTK;      // elements between consecutive rows
    FastDiv    tap_div;   // tile index -> block of output maps (block-major order, ntaps tiles per block)
    int        ntaps;

    static constexpr bool DIRECT = true;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { unsigned off; int kc; };
    struct Tile { BufferRsrc rsrc; int kvalid; };
    // the filter positions of up to 64 class taps, one per lane (see GatherColsLoader::ntaps)
    struct Wave { int trs; };
    __device__ __forceinline__ Wave wave_init(int lane) const
    {
        Wave w{0};
        if (ntaps <= 64) w.trs = tap_trs[min(lane, max(ntaps, 1) - 1)];
        return w;
    }

    __device__ __forceinline__ Ctx prepare(int row, int kc) const
    {
        Ctx c;
        c.kc = kc;
        c.off = (row < C) ? ((unsigned)row * (unsigned)RSTK + (unsigned)kc) * (unsigned)sizeof(T) : NG_OOB_OFFSET;
        return c;
    }
    __device__ __forceinline__ Tile tile(int kt, int /*k0*/, int /*zb*/, const Wave& w) const
    {
        const int blk = (int)tap_div.div((unsigned)kt);
        const int tap = kt - blk * ntaps;
        Tile t;
        // the table entry is wavefront-uniform; the descriptor must live in scalar registers
        const int trs = (ntaps <= 64) ? __builtin_amdgcn_readlane(w.trs, tap)
                                      : __builtin_amdgcn_readfirstlane(tap_trs[tap]);
        t.rsrc = make_rsrc(F + (long)trs * K + (long)blk * BK);
        t.kvalid = K - blk * BK;
        return t;
    }
    // K is a multiple of the chunk length, so a chunk is inside or outside as a whole
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        return c.kc < t.kvalid ? c.off : NG_OOB_OFFSET;
    }
    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const { return buffer_load_chunk(t.rsrc, offset(t, c)); }
};

// A operand of update (contraction-contiguous tile: rows are filter rows
// j = (c,t,r,s), the contraction index is (output pixel, n)).  BLOCKED: N is a
// multiple of BK, so a tile lies inside one output pixel.
template <typename T, typename TIN, bool BLOCKED, int BK>
struct GatherRowsLoader {
    const TIN*      X;
    const TapEntry* tab;        // one entry per filter row
    int             J;          // filter rows C*T*R*S
    int             N, kdim;    // kdim = M*P*Q*N
    int             Q, PQ;
    int             str_d, str_h, str_w;
    int             D, H, W;
    FastDiv         npt_div, pq_div, q_div;   // tiles per pixel, P*Q, Q
    int             npt;

    static constexpr bool DIRECT = std::is_same<T, TIN>::value;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { int off, dz, dy, dx, kc; };
    // BLOCKED: (m, p, q, nb) = output pixel and block inside it, kept so that the
    // next tile is a counter step instead of three divisions
    struct Tile { BufferRsrc rsrc; int pixbase, z0, y0, x0, k0; int m, p, q, nb; };
    typedef NoWaveState Wave;
    __device__ __forceinline__ Wave wave_init(int /*lane*/) const { return Wave{}; }

    static constexpr bool INCREMENTAL = true;
    __device__ __forceinline__ void place(Tile& t) const
    {
        t.z0 = t.m * str_d; t.y0 = t.p * str_h; t.x0 = t.q * str_w;
        t.pixbase = ((t.z0 * H + t.y0) * W + t.x0) * N + t.nb * BK;
    }
    __device__ __forceinline__ void advance(Tile& t, int bk) const
    {
        t.k0 += bk;
        if (BLOCKED) {
            if (++t.nb == npt) {
                t.nb = 0;
                if (++t.q == Q) {
                    t.q = 0;
                    if (++t.p * Q == PQ) { t.p = 0; t.m++; }   // p reached P
                }
            }
            place(t);
        }
    }

    __device__ __forceinline__ Ctx prepare(int r, int kc) const
    {
        Ctx c;
        c.kc = kc;
        if (r < J) {
            const TapEntry e = tab[r];
            c.off = e.off + (BLOCKED ? kc : 0); c.dz = e.dz; c.dy = e.dy; c.dx = e.dx;
        } else {
            c.off = 0; c.dz = c.dy = c.dx = NG_FAR;
        }
        return c;
    }

    __device__ __forceinline__ Tile tile(int kt, int k0, int /*zb*/, const Wave&) const
    {
        Tile t;
        t.rsrc = make_rsrc(X);
        t.k0 = k0;
        if (BLOCKED) {
            const unsigned pix = npt_div.div((unsigned)kt);
            t.nb = kt - (int)pix * npt;
            const unsigned m = pq_div.div(pix);
            const unsigned rem = pix - m * PQ;
            const unsigned p = q_div.div(rem);
            t.m = (int)m; t.p = (int)p; t.q = (int)(rem - p * Q);
            place(t);
        } else {
            t.z0 = t.y0 = t.x0 = t.pixbase = 0;
            t.m = t.p = t.q = t.nb = 0;
        }
        return t;
    }

    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        constexpr int ES = ChunkFetch<T, TIN>::ES;
        if (BLOCKED) {
            const bool ok = ((unsigned)(t.z0 + c.dz) < (unsigned)D) & ((unsigned)(t.y0 + c.dy) < (unsigned)H) &
                            ((unsigned)(t.x0 + c.dx) < (unsigned)W);
            const unsigned off = (unsigned)(t.pixbase + c.off) * ES;
            return ok ? off : NG_OOB_OFFSET;
        } else {
            const int kk = t.k0 + c.kc;
            const int kc2 = min(kk, kdim - 1);
            const int pix = kc2 / N, nn = kc2 - pix * N;
            const int m = pix / PQ, rem = pix - m * PQ;
            const int p = rem / Q, q = rem - p * Q;
            const int z0 = m * str_d, y0 = p * str_h, x0 = q * str_w;
            const bool ok = kk < kdim && (unsigned)(z0 + c.dz) < (unsigned)D && (unsigned)(y0 + c.dy) < (unsigned)H &&
                            (unsigned)(x0 + c.dx) < (unsigned)W;
            return ok ? (unsigned)(((z0 * H + y0) * W + x0) * N + nn + c.off) * ES : NG_OOB_OFFSET;
        }
    }

    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const
    {
        return ChunkFetch<T, TIN>::get(t.rsrc, offset(t, c));
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
        int iz, iy, ix, nn;
        lat.split(j0, iz, iy, ix, nn);
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

// Epilogue of the merged strided data gradient: row (class, c), column
// (lattice point, n) lands on input pixel residue(class) + stride * lattice
// point, if that pixel exists.
template <typename T>
struct MergedLatticeStoreEpilogue {
    typedef typename StoreBits<T>::bits_t bits_t;
    T*           out;
    int          rows;         // classes * C
    int          C;
    FastDiv      div_c, div_hw, div_w;   // C, str_h*str_w, str_w
    long         chan_stride;  // D*H*W*N
    PixelLattice lat;
    int          sz, sy, sx;
    int          D, H, W;
    float        alpha;

    __device__ __forceinline__ void store8(int i, int j0, int /*z*/, int /*split*/, const float (&acc)[8]) const
    {
        if (i >= rows || j0 >= lat.ncols) return;
        const int cls = (int)div_c.div((unsigned)i), c = i - cls * C;
        const int rz = (int)div_hw.div((unsigned)cls), rem = cls - rz * (sy * sx);
        const int ry = (int)div_w.div((unsigned)rem), rx = rem - ry * sx;
        int iz, iy, ix, nn;
        lat.split(j0, iz, iy, ix, nn);
        const int z = rz + sz * iz, y = ry + sy * iy, x = rx + sx * ix;
        if (z >= D || y >= H || x >= W) return;
        bits_t* p = reinterpret_cast<bits_t*>(out + c * chan_stride + (long)((z * H + y) * W + x) * lat.N + nn);
        bits_t b[8];
#pragma unroll
        for (int e = 0; e < 8; e++) b[e] = StoreBits<T>::round(acc[e] * alpha, 0, 0, 0, 0);
        constexpr int NV = (int)sizeof(bits_t) * 8 / 16;
#pragma unroll
        for (int q = 0; q < NV; q++) reinterpret_cast<uint4_t*>(p)[q] = reinterpret_cast<const uint4_t*>(b)[q];
    }
};

}  // namespace ng
