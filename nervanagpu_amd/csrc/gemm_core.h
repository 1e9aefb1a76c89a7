// LDS-tiled MFMA contraction core for gfx950, shared by the GEMM and the
// convolution kernels.
//
//   D[m][n] = sum_k A[m][k] * B[k][n]       fp32 accumulate
//
// One workgroup computes a BM x BN tile; WM x WN wavefronts (64 lanes each) own
// (BM/WM) x (BN/WN) sub-tiles built from 32x32 MFMA blocks:
//   fp16 operands : v_mfma_f32_32x32x16_f16, 8 contraction values per lane
//   fp32 operands : 4 x v_mfma_f32_32x32x2_f32, 4 contraction values per lane
// Operand tiles are staged through LDS in 16-byte chunks, keeping the global
// layout of the source:
//   KC  contraction-contiguous  lds[row][k]   (A not transposed, B transposed)
//   MC  row-contiguous          lds[k][row]   (A transposed, B not transposed,
//                                              CHWN activations, CTRSK filters)
// KC fragments are one ds_read_b128 per lane; MC fp16 fragments use the
// transposing LDS read (ds_read_b64_tr_b16), which hands each lane four
// contraction values of one row from a row-contiguous tile, so no register or
// LDS-write transposes are needed for any operand layout.
//
// Where the operand bytes come from is decided by loader functors (dense
// matrices here, gathered receptive fields in conv.hip); what happens to the
// accumulators is decided by an epilogue functor.
#pragma once

#include "ng_internal.h"
#include "ng_device_common.h"

#include <type_traits>

namespace ng {

typedef _Float16 half8_t   __attribute__((ext_vector_type(8)));
typedef short    short4_t  __attribute__((ext_vector_type(4)));
typedef short    short8_t  __attribute__((ext_vector_type(8)));
typedef float    float4_t  __attribute__((ext_vector_type(4)));
typedef float    float16_t __attribute__((ext_vector_type(16)));
typedef unsigned uint4_t   __attribute__((ext_vector_type(4)));  // one 16-byte chunk

#define NG_LDS __attribute__((address_space(3)))

enum { KC = 0, MC = 1 };

template <typename T> struct Elem;
template <> struct Elem<_Float16> { static constexpr int EPC = 8, KSTEP = 16; };
template <> struct Elem<float>    { static constexpr int EPC = 4, KSTEP = 8;  };

// geometry of one operand tile in LDS
template <typename T, int LAYOUT, int ROWS, int BK>
struct LdsTile {
    static constexpr int EPC    = Elem<T>::EPC;
    static constexpr int ES     = (int)sizeof(T);
    static constexpr int PAD    = (LAYOUT == KC) ? 16 : 64;
    static constexpr int PITCH  = (LAYOUT == KC) ? BK * ES + PAD : ROWS * ES + PAD;
    static constexpr int LINES  = (LAYOUT == KC) ? ROWS : BK;
    static constexpr int BYTES  = PITCH * LINES;
    static constexpr int CHUNKS = ROWS * BK / EPC;
    static constexpr int CPR    = (LAYOUT == KC) ? BK / EPC : ROWS / EPC;  // chunks per LDS line

    // chunk id -> first element (row r, contraction index k) and LDS byte offset
    static __device__ __forceinline__ void chunk_pos(int id, int& r, int& k, int& off)
    {
        const int line = id / CPR, c = (id % CPR) * EPC;
        if (LAYOUT == KC) { r = line; k = c; } else { k = line; r = c; }
        off = line * PITCH + c * ES;
    }
};

template <typename T> struct Frag;
template <> struct Frag<_Float16> { half8_t v; };
template <> struct Frag<float>    { float4_t v; };

// rows rbase..rbase+31, contraction k0..k0+KSTEP-1 of an LDS tile -> MFMA operand
template <typename T, int LAYOUT, int PITCH>
struct FragLoader;

template <int PITCH>
struct FragLoader<_Float16, KC, PITCH> {
    static __device__ __forceinline__ Frag<_Float16> load(const char* lds, int rbase, int k0, int lane)
    {
        Frag<_Float16> f;
        f.v = *reinterpret_cast<const half8_t*>(lds + (rbase + (lane & 31)) * PITCH + (k0 + (lane >> 5) * 8) * 2);
        return f;
    }
};

template <int PITCH>
struct FragLoader<_Float16, MC, PITCH> {
    static __device__ __forceinline__ Frag<_Float16> load(const char* lds, int rbase, int k0, int lane)
    {
        // Within each group of 16 lanes the transposing read treats the 16 x 8-byte
        // pieces the lanes point at as a 4 (k) x 16 (row) matrix, lanes 4j..4j+3
        // supplying line k=j, and returns to lane i the four k values of row i.
        const int l16 = lane & 15, blk = (lane >> 4) & 1, kg = lane >> 5;
        const char* p = lds + (k0 + kg * 8 + (l16 >> 2)) * PITCH + (rbase + blk * 16 + (l16 & 3) * 4) * 2;
        short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NG_LDS short4_t*)(p));
        short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NG_LDS short4_t*)(p + 4 * PITCH));
        short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        Frag<_Float16> f;
        f.v = __builtin_bit_cast(half8_t, both);
        return f;
    }
};

template <int PITCH>
struct FragLoader<float, KC, PITCH> {
    static __device__ __forceinline__ Frag<float> load(const char* lds, int rbase, int k0, int lane)
    {
        Frag<float> f;
        f.v = *reinterpret_cast<const float4_t*>(lds + (rbase + (lane & 31)) * PITCH + (k0 + (lane >> 5) * 4) * 4);
        return f;
    }
};

template <int PITCH>
struct FragLoader<float, MC, PITCH> {
    static __device__ __forceinline__ Frag<float> load(const char* lds, int rbase, int k0, int lane)
    {
        Frag<float> f;
        const char* p = lds + (k0 + (lane >> 5) * 4) * PITCH + (rbase + (lane & 31)) * 4;
#pragma unroll
        for (int j = 0; j < 4; j++) f.v[j] = *reinterpret_cast<const float*>(p + j * PITCH);
        return f;
    }
};

__device__ __forceinline__ void mfma_step(const Frag<_Float16>& a, const Frag<_Float16>& b, float16_t& acc)
{
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.v, b.v, acc, 0, 0, 0);
}

__device__ __forceinline__ void mfma_step(const Frag<float>& a, const Frag<float>& b, float16_t& acc)
{
#pragma unroll
    for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[j], b.v[j], acc, 0, 0, 0);
}

// problem extents seen by the core
struct CoreShape {
    int m, n;          // output extents (rows of A-operand, rows of B-operand)
    int k_tiles;       // BK-sized contraction tiles per pass
    int passes;        // contraction passes accumulated into one output (batch_loops)
    int splits;        // the (passes * k_tiles) tile range is cut into this many slices
    int tiles_m, tiles_n;
    int n_base = 0;    // first column of this launch's tile 0 (a launch may cover a column range of the problem)
};

// gridDim.y of a launch over `tiles` output tiles (gridDim.x) and `splits`
// slices: with more than one slice the (tile, slice) pairs are dealt to the XCDs
// in eight equal contiguous shares (see block_work), which needs 8 * ceil(pairs / 8)
// workgroups
// gridDim.x: the output tiles; a launch with one slice rounds them up to a
// multiple of 8 so that every XCD can be given one contiguous share
inline unsigned grid_tiles(int tiles, int splits) { return splits > 1 ? (unsigned)tiles : (unsigned)((tiles + 7) / 8 * 8); }
inline unsigned grid_slices(int tiles, int splits)
{
    if (splits <= 1) return 1u;
    const long per = ((long)tiles * splits + 7) / 8;
    return (unsigned)((8 * per + tiles - 1) / tiles);
}

// Global operand chunks are fetched with raw buffer loads: an offset at or
// beyond the 2 GiB range of the descriptor returns zeros in hardware, which is
// how invalid rows, contraction tails and out-of-image convolution taps become
// zero operands without a branch or a select after the load.
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
#define NG_OOB_OFFSET 0x80000000u

__device__ __forceinline__ BufferRsrc make_rsrc(const void* base)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x80000000, 0x00020000);
}

__device__ __forceinline__ uint4_t buffer_load_chunk(BufferRsrc rsrc, unsigned byte_offset)
{
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_offset, 0, 0);
}

// 16-byte store through a descriptor: an offset at or beyond its range is dropped
// by the hardware, so a lane with nothing to store still takes part and every
// wavefront issues the same number of store instructions
__device__ __forceinline__ void buffer_store_chunk(BufferRsrc rsrc, unsigned byte_offset, uint4_t v)
{
    __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, (int)byte_offset, 0, 0);
}

// Loader protocol used by the core (all three calls are inlined):
//   Ctx  prepare(r, kc)      once per 16-byte chunk a thread owns: r = absolute
//                            row of the operand, kc = contraction offset of the
//                            chunk inside a tile
//   Tile tile(kt, k0, zb)    once per contraction tile, wavefront-uniform values
//                            (kt = tile index inside the pass, k0 = kt*BK,
//                            zb = batch / pass index)
//   load(tile, ctx)          the chunk; must be branch free so that the loads of
//                            the next tile can be scheduled between the MFMAs of
//                            the current one
//
//   Wave wave_init(lane)     once per thread: per-lane state a loader wants to keep
//                            in registers for tile() (e.g. a small table held one
//                            entry per lane and fetched with v_readlane); passed
//                            back as the last argument of tile()
//
// Dense row-major operand.  KC: element (r,k) at base[r*ld + k]; MC: at base[k*ld + r].
// VEC: the host guarantees 16-byte alignment of every chunk, that chunks do not
// straddle the matrix edge and that the matrix spans less than 4 GiB; otherwise
// elements are fetched one by one.
struct NoWaveState {};

// A B-operand loader may serve several horizontally adjacent filter taps from
// ONE LDS tile: it then declares TAPS (> 1) and TAP_COLS, loads BN + (TAPS-1) *
// TAP_COLS columns per tile through prepare_seg(), and tap s of the tile reads
// its fragments TAP_COLS * s columns to the right.  The A tile of such a
// kernel is TAPS * BK deep (tap-major).
template <class L, class = void> struct LoaderTaps { static constexpr int taps = 1, cols = 0; };
template <class L> struct LoaderTaps<L, std::enable_if_t<(L::TAPS > 1)>> { static constexpr int taps = L::TAPS, cols = L::TAP_COLS; };

// An epilogue that combines values across the columns of a workgroup's tile
// declares `static constexpr bool WHOLE_TILE = true` and tile(g, tid, nthreads,
// n0): the kernel (one row block of 32 rows) parks the fp32 tile in LDS, row-major
// with BN columns, before calling it.
template <class E, class = void> struct EpilogueWholeTile { static constexpr bool value = false; };
template <class E> struct EpilogueWholeTile<E, std::enable_if_t<E::WHOLE_TILE>> { static constexpr bool value = true; };

// loaders that can step a tile descriptor to the next contraction tile declare
// `static constexpr bool INCREMENTAL = true` and advance(Tile&, bk)
template <class L, class = void> struct LoaderIncremental { static constexpr bool value = false; };
template <class L> struct LoaderIncremental<L, std::enable_if_t<L::INCREMENTAL>> { static constexpr bool value = true; };

template <typename T, int LAYOUT, bool VEC>
struct DenseLoader {
    const T* base;
    long     ldz;    // batch / pass stride in elements
    int      ld;
    int      rows;   // extent along r
    int      kdim;   // extent along k (per pass)

    // a chunk is one 16-byte buffer load whose offset offset() returns, so the
    // core may send it straight to LDS
    static constexpr bool DIRECT = VEC;
    static constexpr bool TILE_READS_TABLE = false;

    struct Ctx { unsigned off; int k; int r; };
    struct Tile { BufferRsrc rsrc; const T* p; int krem; };
    typedef NoWaveState Wave;
    __device__ __forceinline__ Wave wave_init(int /*lane*/) const { return Wave{}; }

    __device__ __forceinline__ Ctx prepare(int r, int kc) const
    {
        Ctx c;
        c.k = kc;
        c.r = r;
        const unsigned e = (LAYOUT == KC) ? (unsigned)r * (unsigned)ld + (unsigned)kc
                                          : (unsigned)kc * (unsigned)ld + (unsigned)r;
        c.off = (r < rows) ? e * (unsigned)sizeof(T) : NG_OOB_OFFSET;
        return c;
    }

    __device__ __forceinline__ Tile tile(int /*kt*/, int k0, int zb, const Wave& = Wave{}) const
    {
        Tile t;
        t.p = base + (long)zb * ldz + (long)k0 * (LAYOUT == KC ? 1 : ld);
        t.rsrc = make_rsrc(t.p);
        t.krem = kdim - k0;
        return t;
    }

    // the descriptor of the next contraction tile of the same pass: a pointer
    // bump instead of the 64-bit products of tile()
    static constexpr bool INCREMENTAL = true;
    __device__ __forceinline__ void advance(Tile& t, int bk) const
    {
        t.p += (LAYOUT == KC) ? (long)bk : (long)bk * ld;
        t.rsrc = make_rsrc(t.p);
        t.krem -= bk;
    }

    // rows past the matrix edge and contraction indices past kdim read as zero
    __device__ __forceinline__ unsigned offset(const Tile& t, const Ctx& c) const
    {
        return (c.k < t.krem) ? c.off : NG_OOB_OFFSET;
    }

    __device__ __forceinline__ uint4_t load(const Tile& t, const Ctx& c) const
    {
        constexpr int EPC = Elem<T>::EPC;
        if (VEC) {
            return buffer_load_chunk(t.rsrc, offset(t, c));
        } else {
            const T* p = t.p;
            T tmp[EPC];
#pragma unroll
            for (int e = 0; e < EPC; e++) {
                const int rr = (LAYOUT == KC) ? c.r : c.r + e;
                const int kk = (LAYOUT == KC) ? c.k + e : c.k;
                tmp[e] = (rr < rows && kk < t.krem)
                             ? ((LAYOUT == KC) ? p[(long)rr * ld + kk] : p[(long)kk * ld + rr])
                             : (T)0;
            }
            return *reinterpret_cast<const uint4_t*>(tmp);
        }
    }
};

// blockIdx.x -> (tile_m, tile_n).  Workgroups are handed to the 8 XCDs round
// robin; renumbering them gives each XCD a contiguous range of tile numbers,
// and numbering the tiles in bands of 8 rows (column-major inside a band) makes
// such a range a compact block of the output (e.g. 8 x 4 tiles for 32 CUs
// instead of 16 x 2), so fewer distinct operand tiles pass through its L2.
__device__ __forceinline__ void tile_of_block(const CoreShape& s, int pid, int& tm, int& tn)
{
    constexpr int BAND = 8;
    const int per_band = BAND * s.tiles_n;
    const int band = pid / per_band;
    const int first_m = band * BAND;
    const int rows = min(BAND, s.tiles_m - first_m);
    const int in_band = pid - band * per_band;
    tn = in_band / rows;
    tm = first_m + (in_band - tn * rows);
}

// Output tile and contraction slice of this workgroup; false: nothing to do.
// Workgroups are dealt to the 8 XCDs round robin in dispatch order (x fastest,
// then y).  One slice: an XCD gets a contiguous eighth of the tile numbers
// (gridDim.x is grid_tiles(); surplus workgroups leave).  Several slices: the workgroups of one slice
// read the same contraction range of both operands, so the (slice, tile) pairs,
// numbered slice-major, are cut into eight equal contiguous shares, one per
// XCD: an XCD then works on one or two slices at a time and its L2 fetches
// their operand ranges once, instead of every XCD fetching every slice
// (measured on a weight gradient: 3.3 GB from HBM where 0.8 GB are needed).
// gridDim.y is grid_slices().
__device__ __forceinline__ bool block_work(const CoreShape& s, int& tm, int& tn, int& split)
{
    int pid;
    const int total = s.tiles_m * s.tiles_n;
    if (s.splits > 1) {
        const unsigned linear = blockIdx.x + gridDim.x * blockIdx.y;
        const unsigned xcd = linear & 7u, slot = linear >> 3;
        const unsigned pairs = (unsigned)total * (unsigned)s.splits;
        const unsigned per = (pairs + 7u) >> 3;
        const unsigned pair = xcd * per + slot;
        if (slot >= per || pair >= pairs) return false;
        split = (int)(pair / (unsigned)total);
        pid = (int)(pair - (unsigned)split * (unsigned)total);
    } else {
        split = 0;
        const int per = (total + 7) >> 3;
        const int slot = (int)(blockIdx.x >> 3);
        pid = (int)(blockIdx.x & 7u) * per + slot;
        if (pid >= total) return false;
    }
    tile_of_block(s, pid, tm, tn);
    return true;
}

// Scheduling directive for one k-step.  After each MFMA: two LDS reads of the
// next step's fragments until they are used up; one global load after every
// other MFMA until the step's share of the next tile is issued.
template <int I, int N_MFMA, int N_READS, int N_LOADS>
struct InterleaveStep {
    static __device__ __forceinline__ void emit()
    {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
        if constexpr (2 * I < N_READS)
            __builtin_amdgcn_sched_group_barrier(0x100, (N_READS - 2 * I) >= 2 ? 2 : 1, 0);   // LDS reads
        if constexpr ((I & 1) == 1 && (I / 2) < N_LOADS)
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // one global load
        if constexpr (I + 1 < N_MFMA) InterleaveStep<I + 1, N_MFMA, N_READS, N_LOADS>::emit();
    }
};

// One 32-row band of a wavefront's accumulators: registers -> private LDS
// staging -> 8-column chunks handed to the epilogue functor.  The band index is
// a template parameter so that every accumulator access is a static register
// reference.
// The staging region of the epilogue is private to a wavefront and LDS
// operations of one wavefront execute in order, so write -> read -> rewrite only
// needs the compiler kept from reordering them; no workgroup barrier.
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// epilogues with a descriptor-store form of their plain case declare BUFFER_STORE
template <class E, class = void> struct EpilogueBufferStore { static constexpr bool value = false; };
template <class E> struct EpilogueBufferStore<E, std::enable_if_t<E::BUFFER_STORE>> { static constexpr bool value = true; };

// ROW_TAPS > 1: the TM bands of a wavefront are ROW_TAPS interleaved row sets (band
// I holds rows (mbase + ((I / ROW_TAPS) * 32 + r) * ROW_STRIDE) * ROW_TAPS + I % ROW_TAPS:
// the horizontal taps of 32 filter rows of the weight gradient's ring kernel; with
// ROW_STRIDE 3 those rows are one vertical tap of 32 channels of a 3x3 filter)
template <int TM, int TN, int WTN, int EPITCH, int I, int ROW_TAPS = 1, int ROW_STRIDE = 1>
struct EpilogueBands {
    static __device__ __forceinline__ int row_of(int mbase, int r)
    {
        return ROW_TAPS == 1 ? mbase + I * 32 + r
                             : (mbase + ((I / ROW_TAPS) * 32 + r) * ROW_STRIDE) * ROW_TAPS + I % ROW_TAPS;
    }
    template <class Epi>
    static __device__ __forceinline__ void run(float16_t (&acc)[TM][TN], char* stage, int lane,
                                               int mbase, int nbase, int z, int split, const Epi& epi)
    {
        constexpr int CPW = 32 * WTN / 8;   // 8-column chunks per band
        const int col = lane & 31;
        const int rsub = (lane >> 5) * 4;
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                *reinterpret_cast<float*>(stage + ((v >> 2) * 8 + rsub + (v & 3)) * EPITCH + (j * 32 + col) * 4) =
                    acc[I][j][v];
        wave_lds_fence();
        // The common store (16-bit output, aligned rows, no beta, nearest rounding,
        // no mask) goes through a buffer descriptor: edges are dropped by the
        // hardware and the address is a 32-bit offset, a third of the instructions
        // of the general store8 with its run-time choices.
        bool plain = false;
        if constexpr (EpilogueBufferStore<Epi>::value) plain = epi.plain_store();
        if (plain) {
            if constexpr (EpilogueBufferStore<Epi>::value) {
                const BufferRsrc rsrc = epi.store_rsrc(z);
#pragma unroll
                for (int c = 0; c < CPW / 64; c++) {
                    const int id = lane + c * 64;
                    const int r = id / (WTN / 8);
                    const int cc = (id % (WTN / 8)) * 8;
                    const float4_t lo = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4);
                    const float4_t hi = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4 + 16);
                    const float vals[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                    epi.store8_buffer(rsrc, row_of(mbase, r), nbase + cc, vals);
                }
            }
        } else {
#pragma unroll
            for (int c = 0; c < CPW / 64; c++) {
                const int id = lane + c * 64;
                const int r = id / (WTN / 8);
                const int cc = (id % (WTN / 8)) * 8;
                const float4_t lo = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4);
                const float4_t hi = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4 + 16);
                const float vals[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                epi.store8(row_of(mbase, r), nbase + cc, z, split, vals);
            }
        }
        wave_lds_fence();
        if constexpr (I + 1 < TM)
            EpilogueBands<TM, TN, WTN, EPITCH, I + 1, ROW_TAPS, ROW_STRIDE>::run(acc, stage, lane, mbase, nbase, z, split, epi);
    }
};

template <typename T, int BM, int BN, int BK, int WM, int WN, int LA, int LB,
          class ALoad, class BLoad, class Epi>
__global__ __launch_bounds__(WM * WN * 64)
void mfma_gemm_kernel(ALoad aload, BLoad bload, Epi epi, CoreShape s)
{
    constexpr int NT = WM * WN * 64;
    constexpr int KSTEP = Elem<T>::KSTEP;
    using TA = LdsTile<T, LA, BM, BK>;
    using TB = LdsTile<T, LB, BN, BK>;
    constexpr int CPT_A = TA::CHUNKS / NT;
    constexpr int CPT_B = TB::CHUNKS / NT;
    static_assert(TA::CHUNKS % NT == 0 && TB::CHUNKS % NT == 0, "tile chunks must divide evenly over threads");
    constexpr int TM = BM / WM / 32;
    constexpr int TN = BN / WN / 32;
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % (2 * KSTEP) == 0, "bad tile shape");

    constexpr int STAGE = TA::BYTES + TB::BYTES;
    constexpr int WTN = BN / WN;                 // columns of a wavefront's sub-tile
    constexpr int EPITCH = WTN * 4 + 16;         // bytes per staged epilogue row
    constexpr int EPI_BYTES = 32 * EPITCH;       // epilogue staging per wavefront
    constexpr int SMEM_BYTES = (2 * STAGE > EPI_BYTES * WM * WN) ? 2 * STAGE : EPI_BYTES * WM * WN;
    __shared__ __attribute__((aligned(16))) char smem[SMEM_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;

    int tm, tn, split;
    if (!block_work(s, tm, tn, split)) return;
    const int m0 = tm * BM, n0 = s.n_base + tn * BN;
    const int z = blockIdx.z;

    // contraction tile range of this split
    const int total_tiles = s.passes * s.k_tiles;
    const int per = (total_tiles + s.splits - 1) / s.splits;
    const int t_begin = split * per;
    const int t_end = min(t_begin + per, total_tiles);

    int ra_r[CPT_A], ra_k[CPT_A], ra_off[CPT_A];
    int rb_r[CPT_B], rb_k[CPT_B], rb_off[CPT_B];
#pragma unroll
    for (int i = 0; i < CPT_A; i++) TA::chunk_pos(tid + i * NT, ra_r[i], ra_k[i], ra_off[i]);
#pragma unroll
    for (int i = 0; i < CPT_B; i++) TB::chunk_pos(tid + i * NT, rb_r[i], rb_k[i], rb_off[i]);

    // loaders may precompute per-row state (e.g. the pixel a column belongs to)
    typename ALoad::Ctx actx[CPT_A];
    typename BLoad::Ctx bctx[CPT_B];
#pragma unroll
    for (int i = 0; i < CPT_A; i++) actx[i] = aload.prepare(m0 + ra_r[i], ra_k[i]);
#pragma unroll
    for (int i = 0; i < CPT_B; i++) bctx[i] = bload.prepare(n0 + rb_r[i], rb_k[i]);

    uint4_t ra[CPT_A], rb[CPT_B];
    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    // position of the next tile to fetch: (pass, tile inside the pass), kept
    // incrementally so that no division runs inside the loop
    int g_pass = t_begin / s.k_tiles;
    int g_kt = t_begin - g_pass * s.k_tiles;
    // Global loads of the next tile are issued in NSTEP-1 parts, one inside each
    // of the first k-steps, so that the address pipeline is fed at its own pace
    // instead of blocking instruction issue with a burst at the top of the tile.
    constexpr int N_CHUNKS = CPT_A + CPT_B;
    constexpr int G_PARTS = (BK / KSTEP > 1) ? BK / KSTEP - 1 : 1;
    constexpr int G_PER = (N_CHUNKS + G_PARTS - 1) / G_PARTS;
    typename ALoad::Tile g_ta;
    typename BLoad::Tile g_tb;
    const typename ALoad::Wave a_wave = aload.wave_init(lane);
    const typename BLoad::Wave b_wave = bload.wave_init(lane);
    auto gtile = [&]() {
        g_ta = aload.tile(g_kt, g_kt * BK, z + g_pass, a_wave);
        g_tb = bload.tile(g_kt, g_kt * BK, z + g_pass, b_wave);
        if (++g_kt == s.k_tiles) { g_kt = 0; g_pass++; }
    };
    auto gload_part = [&](int part) {
#pragma unroll
        for (int c = 0; c < N_CHUNKS; c++) {
            if (c / G_PER != part) continue;
            if (c < CPT_A) ra[c < CPT_A ? c : 0] = aload.load(g_ta, actx[c < CPT_A ? c : 0]);
            else           rb[c >= CPT_A ? c - CPT_A : 0] = bload.load(g_tb, bctx[c >= CPT_A ? c - CPT_A : 0]);
        }
    };
    auto gload = [&]() {
        gtile();
#pragma unroll
        for (int part = 0; part < G_PARTS; part++) gload_part(part);
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < CPT_A; i++) *reinterpret_cast<uint4_t*>(smem + buf * STAGE + ra_off[i]) = ra[i];
#pragma unroll
        for (int i = 0; i < CPT_B; i++) *reinterpret_cast<uint4_t*>(smem + buf * STAGE + TA::BYTES + rb_off[i]) = rb[i];
    };

    // Main loop, software pipelined for one wavefront per SIMD:
    //  * global loads of tile t+1 are issued at the top of tile t and land in
    //    registers while tile t is multiplied;
    //  * MFMA fragments are double buffered: the LDS reads of k-step s+1 are
    //    issued before the MFMAs of step s;
    //  * the registers of tile t+1 are written to the other LDS stage and the
    //    single barrier of the iteration is taken BEFORE the last k-step, so the
    //    first fragments of tile t+1 are already in flight while the last MFMAs
    //    of tile t execute.
    constexpr int NSTEP = BK / KSTEP;
    Frag<T> fa[2][TM], fb[2][TN];

    auto load_frags = [&](int stage_buf, int step, Frag<T> (&a)[TM], Frag<T> (&b)[TN]) {
        const char* a_lds = smem + stage_buf * STAGE;
        const char* b_lds = a_lds + TA::BYTES;
#pragma unroll
        for (int i = 0; i < TM; i++)
            a[i] = FragLoader<T, LA, TA::PITCH>::load(a_lds, wm * (BM / WM) + i * 32, step * KSTEP, lane);
#pragma unroll
        for (int j = 0; j < TN; j++)
            b[j] = FragLoader<T, LB, TB::PITCH>::load(b_lds, wn * (BN / WN) + j * 32, step * KSTEP, lane);
    };
    auto multiply = [&](const Frag<T> (&a)[TM], const Frag<T> (&b)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) mfma_step(a[i], b[j], acc[i][j]);
    };

    if (t_begin < t_end) {
        gload();
        sstore(0);
    }
    __syncthreads();
    if (t_begin < t_end) load_frags(0, 0, fa[0], fb[0]);

    // LDS read instructions one k-step issues for the next step's fragments
    constexpr bool IS_HALF = (sizeof(T) == 2);
    constexpr int RD_A = (LA == KC) ? 1 : (IS_HALF ? 2 : 4);
    constexpr int RD_B = (LB == KC) ? 1 : (IS_HALF ? 2 : 4);
    constexpr int N_READS = TM * RD_A + TN * RD_B;
    constexpr int N_MFMA = TM * TN * (IS_HALF ? 1 : 4);

    // One k-step: prefetch the next fragments, multiply the current ones, and
    // tell the scheduler to issue the prefetch reads at the head of the step,
    // two after each MFMA, instead of sinking them next to their first use.
    auto step = [&](int rd_buf, int rd_step, Frag<T> (&na)[TM], Frag<T> (&nb)[TN],
                    const Frag<T> (&ca)[TM], const Frag<T> (&cb)[TN], int load_part) {
        if (load_part >= 0) gload_part(load_part);
        load_frags(rd_buf, rd_step, na, nb);
        multiply(ca, cb);
        if (load_part >= 0) InterleaveStep<0, N_MFMA, N_READS, G_PER>::emit();
        else                InterleaveStep<0, N_MFMA, N_READS, 0>::emit();
        __builtin_amdgcn_sched_barrier(0);
    };

    // every tile but the last: one straight-line block per iteration
    for (int t = t_begin; t + 1 < t_end; t++) {
        const int buf = (t - t_begin) & 1;
        gtile();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NSTEP - 1; s++)
            step(buf, s + 1, fa[(s + 1) & 1], fb[(s + 1) & 1], fa[s & 1], fb[s & 1], s);
        sstore(buf ^ 1);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        step(buf ^ 1, 0, fa[NSTEP & 1], fb[NSTEP & 1], fa[(NSTEP - 1) & 1], fb[(NSTEP - 1) & 1], -1);
    }
    // last tile: nothing left to fetch
    if (t_begin < t_end) {
        const int buf = (t_end - 1 - t_begin) & 1;
#pragma unroll
        for (int s = 0; s < NSTEP - 1; s++)
            step(buf, s + 1, fa[(s + 1) & 1], fb[(s + 1) & 1], fa[s & 1], fb[s & 1], -1);
        multiply(fa[(NSTEP - 1) & 1], fb[(NSTEP - 1) & 1]);
    }

    // Epilogue.  The 32x32 MFMA block leaves lane l with column (l & 31) and rows
    // (v/4)*8 + (l>>5)*4 + (v&3) of the block.  Each wavefront passes one 32-row
    // band of its sub-tile at a time through a private LDS region so that a lane
    // ends up with 8 consecutive columns of one row: the global stores (and the
    // beta*C loads) are then 16-byte accesses covering whole rows.
    char* stage = smem + wave * EPI_BYTES;
    __syncthreads();
    EpilogueBands<TM, TN, WTN, EPITCH, 0>::run(acc, stage, lane, m0 + wm * (BM / WM), n0 + wn * WTN, z, split, epi);
}

// ---------------------------------------------------------------------------
// Direct-to-LDS variant (fp16).  Operand chunks go from global memory straight
// into LDS (buffer_load ... lds: a wavefront instruction fills 1 KiB of LDS, lane
// l writing bytes [16 l, 16 l + 16) after the wave-uniform base), so the tile
// never passes through registers and NSTAGE >= 2 tiles can be in flight.
//
// The hardware fixes where a lane's chunk lands, so LDS tiles are unpadded and
// bank conflicts are avoided by permuting WHICH chunk a lane fetches: the chunk
// at position pc of line `line` holds logical chunk pc ^ swizzle(line).
// ---------------------------------------------------------------------------
template <typename T, int LAYOUT, int ROWS, int BK>
struct SwizzledTile {
    static constexpr int EPC    = Elem<T>::EPC;
    static constexpr int CPR    = (LAYOUT == KC) ? BK / EPC : ROWS / EPC;   // chunks per line
    static constexpr int PITCH  = CPR * 16;
    static constexpr int LINES  = (LAYOUT == KC) ? ROWS : BK;
    static constexpr int BYTES  = PITCH * LINES;
    static constexpr int CHUNKS = ROWS * BK / EPC;
    static constexpr int LP     = (CPR >= 16) ? 1 : 16 / CPR;               // lines per 256 bytes
    // MC: 64-byte groups permuted among themselves; the permuted span (GROUPS * 64
    // bytes) must divide the line, so lines of 24 chunks permute pairs of groups
    static constexpr int GROUPS = (CPR % 16 == 0) ? 4 : (CPR % 8 == 0) ? 2 : 1;
    static_assert(sizeof(T) == 2, "direct LDS tiles are implemented for 16-bit elements");
    static_assert(LAYOUT == MC || CPR <= 16, "contraction-contiguous lines longer than 256 bytes are not swizzled");
    static_assert(LAYOUT == KC || CPR >= 8, "row-contiguous tiles need at least 64 rows");
    static_assert(LAYOUT == KC || CPR % (GROUPS * 4) == 0, "the group permutation must stay inside a line");

    // KC: 16 consecutive rows read the same logical chunk -> spread them over the
    //     16 chunk slots of a 256-byte bank period.
    // MC: a transposing read touches 64 contiguous bytes in each of 4 consecutive
    //     lines -> send the 4 lines to 4 different 64-byte groups.
    static __device__ __forceinline__ int swizzle(int line)
    {
        return (LAYOUT == KC) ? (line / LP) % CPR : ((line / LP) % GROUPS) * 4;
    }
    // LDS chunk position id (byte offset 16*id) -> first element it must hold
    static __device__ __forceinline__ void chunk_pos(int id, int& r, int& k)
    {
        const int line = id / CPR, c = ((id % CPR) ^ swizzle(line)) * EPC;
        if (LAYOUT == KC) { r = line; k = c; } else { k = line; r = c; }
    }
};

// Fragment addressing in a swizzled tile.  base() is the lane-constant part for
// the 32-row block `blk32` (block index inside the tile); load() adds the k-step.
template <int LAYOUT, class Tile> struct SwizzledFrag;

template <class Tile>
struct SwizzledFrag<KC, Tile> {
    static __device__ __forceinline__ int base(int blk32, int lane)
    {
        // the swizzle of row 32*b + r only depends on r
        const int r = lane & 31;
        return (blk32 * 32 + r) * Tile::PITCH + (((lane >> 5) ^ Tile::swizzle(r)) * 16);
    }
    static __device__ __forceinline__ Frag<_Float16> load(const char* tile, int base, int step)
    {
        // chunk index of step s is (2 s | lane>>5): the xor with the swizzle distributes
        Frag<_Float16> f;
        f.v = *reinterpret_cast<const half8_t*>(tile + (base ^ (step * 32)));
        return f;
    }
    // the base from which load(.., step) reads k-step first + step; `first` must be a
    // multiple of a power of two that every later `step` stays below
    static __device__ __forceinline__ int skip(int base, int first) { return base ^ (first * 32); }
};

template <class Tile>
struct SwizzledFrag<MC, Tile> {
    static __device__ __forceinline__ int base(int blk32, int lane)
    {
        // lines step*16 + kg*8 + (l16>>2) (+4 for the second read) all share the
        // swizzle of line kg*8 + (l16>>2)
        const int l16 = lane & 15, blk = (lane >> 4) & 1, kg = lane >> 5;
        const int line = kg * 8 + (l16 >> 2);
        const int c = blk32 * 4 + blk * 2 + ((l16 >> 1) & 1);
        return line * Tile::PITCH + ((c ^ Tile::swizzle(line)) * 16) + (l16 & 1) * 8;
    }
    static __device__ __forceinline__ Frag<_Float16> load(const char* tile, int base, int step)
    {
        const char* p = tile + base + step * 16 * Tile::PITCH;
        short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NG_LDS short4_t*)(p));
        short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((NG_LDS short4_t*)(p + 4 * Tile::PITCH));
        short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        Frag<_Float16> f;
        f.v = __builtin_bit_cast(half8_t, both);
        return f;
    }
    static __device__ __forceinline__ int skip(int base, int first) { return base + first * 16 * Tile::PITCH; }
};

// A operand of a kernel whose B tile serves TAPS filter taps.  A row-contiguous
// tile simply gets TAPS * BK lines.  A contraction-contiguous one would get lines
// of TAPS * BK elements, which the power-of-two swizzle cannot permute, so it is
// kept as TAPS tiles of BK elements per line, one behind the other.
template <typename T, int LAYOUT, int ROWS, int BK, int TAPS>
struct TapTile {
    static constexpr bool STACKED = (LAYOUT == KC && TAPS > 1);
    using Sub = SwizzledTile<T, LAYOUT, ROWS, STACKED ? BK : BK * TAPS>;
    static constexpr int BYTES  = Sub::BYTES * (STACKED ? TAPS : 1);
    static constexpr int CHUNKS = Sub::CHUNKS * (STACKED ? TAPS : 1);
    static __device__ __forceinline__ void chunk_pos(int id, int& r, int& k)
    {
        if (STACKED) {
            const int tap = id / Sub::CHUNKS;
            Sub::chunk_pos(id - tap * Sub::CHUNKS, r, k);
            k += tap * BK;
        } else {
            Sub::chunk_pos(id, r, k);
        }
    }
    // byte offset of the sub-tile and the k-step inside it for k-step `step` of the whole tile
    static constexpr int tile_of(int step, int ks) { return STACKED ? (step / ks) * Sub::BYTES : 0; }
    static constexpr int step_of(int step, int ks) { return STACKED ? step % ks : step; }
};

// s_waitcnt immediate: at most `vm` vector-memory operations outstanding, all
// LDS operations complete
// 16 bytes per lane from a buffer straight into LDS: lane l of the wavefront
// writes lds_base + 16 l (lds_base is wave-uniform and travels in M0); an
// out-of-range offset stores zeros.
//
// Written as inline assembly on purpose.  The compiler's wait-count insertion
// orders every LDS access it regards as a store (the transposing LDS reads are
// among them) behind all outstanding LDS-bound loads, i.e. it would wait for the
// tile just requested before reading the current one.  Hidden from it, these
// loads are ordered by hand: an explicit s_waitcnt vmcnt(..) precedes the
// barrier that publishes a stage.
// (The lane-level CPU emulation of tests/emu, which checks the index arithmetic of these
// kernels without a GPU, supplies this one function itself: host compilers cannot take
// the assembly.)
#ifndef NG_HOST_EMULATION
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void buffer_load_chunk_to_lds(BufferRsrc rsrc, char* lds_base, unsigned byte_offset)
{
    const unsigned lds_addr = (unsigned)(unsigned long)(NG_LDS char*)lds_base;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(lds_addr), "v"(byte_offset), "s"(rsrc) : "memory", "m0");
}
#pragma clang diagnostic pop
#endif

template <int VM> struct WaitVmLgkm0 { static constexpr int IMM = (VM & 15) | ((VM >> 4) << 14) | (7 << 4); };

// WK > 1: WK groups of WM x WN wavefronts share one output tile and split the
// k-steps of every contraction tile among themselves (group g takes steps
// g * KS / WK onwards), so a workgroup of WM * WN * WK wavefronts keeps a tile of
// BK in flight per stage while each wavefront still owns a whole BM/WM x BN/WN
// sub-tile.  The groups' accumulators are added through LDS, group by group in
// a fixed order, before the epilogue, which group 0 runs.
template <typename T, int BM, int BN, int BK, int WM, int WN, int LA, int LB, int NSTAGE,
          class ALoad, class BLoad, class Epi, int WK = 1>
__global__ __launch_bounds__(WM * WN * WK * 64)
void mfma_gemm_direct_kernel(ALoad aload, BLoad bload, Epi epi, CoreShape s)
{
    static_assert(ALoad::DIRECT && BLoad::DIRECT, "operands must be plain 16-byte buffer loads");
    static_assert(NSTAGE >= 2, "need at least two LDS stages");
    constexpr int NT = WM * WN * WK * 64;
    constexpr int KSTEP = Elem<T>::KSTEP;
    constexpr int TAPS = LoaderTaps<BLoad>::taps;          // filter taps served by one B tile
    constexpr int TAP_COLS = LoaderTaps<BLoad>::cols;      // columns by which a tap shifts its window
    static_assert(TAPS == 1 || (LB == MC && TAP_COLS % 32 == 0), "shared taps need a row-contiguous B tile");
    using TA = TapTile<T, LA, BM, BK, TAPS>;
    using TB = SwizzledTile<T, LB, BN + (TAPS - 1) * TAP_COLS, BK>;
    using FA = SwizzledFrag<LA, typename TA::Sub>;
    using FB = SwizzledFrag<LB, TB>;
    constexpr int CPT_A = TA::CHUNKS / NT;
    constexpr int CPT_B = TB::CHUNKS / NT;
    static_assert(TA::CHUNKS % NT == 0 && TB::CHUNKS % NT == 0, "tile chunks must divide evenly over threads");
    constexpr int TM = BM / WM / 32;
    constexpr int TN = BN / WN / 32;
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % (2 * KSTEP * WK) == 0, "bad tile shape");
    static_assert(WK == 1 || (TAPS == 1 && (WK & (WK - 1)) == 0), "the k-steps of a plain tile are split over a power of two of groups");

    constexpr int STAGE = TA::BYTES + TB::BYTES;
    constexpr int WTN = BN / WN;
    constexpr int EPITCH = WTN * 4 + 16;
    constexpr int EPI_BYTES = 32 * EPITCH;
    // accumulators of one group of wavefronts on their way to group 0
    constexpr int RED_BYTES = (WK > 1) ? WM * WN * TM * TN * 16 * 64 * 4 : 0;
    constexpr int SMEM_TILES = (NSTAGE * STAGE > EPI_BYTES * WM * WN) ? NSTAGE * STAGE : EPI_BYTES * WM * WN;
    constexpr int SMEM_BYTES = (SMEM_TILES > RED_BYTES) ? SMEM_TILES : RED_BYTES;
    static_assert(SMEM_BYTES <= 160 * 1024, "tile stages exceed the LDS of a compute unit");
    __shared__ __attribute__((aligned(16))) char smem[SMEM_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wtile = (WK > 1) ? wave % (WM * WN) : wave;     // which sub-tile of the output
    const int wk = (WK > 1) ? wave / (WM * WN) : 0;           // which share of the k-steps
    const int wm = wtile % WM, wn = wtile / WM;

    int tm, tn, split;
    if (!block_work(s, tm, tn, split)) return;
    const int m0 = tm * BM, n0 = s.n_base + tn * BN;
    const int z = blockIdx.z;

    const int total_tiles = s.passes * s.k_tiles;
    const int per = (total_tiles + s.splits - 1) / s.splits;
    const int t_begin = split * per;
    const int t_end = min(t_begin + per, total_tiles);
    const int ntiles = t_end - t_begin;

    // the chunk a lane fetches with its i-th load instruction of a tile
    typename ALoad::Ctx actx[CPT_A];
    typename BLoad::Ctx bctx[CPT_B];
#pragma unroll
    for (int i = 0; i < CPT_A; i++) { int r, k; TA::chunk_pos(tid + i * NT, r, k); actx[i] = aload.prepare(m0 + r, k); }
#pragma unroll
    for (int i = 0; i < CPT_B; i++) {
        int r, k;
        TB::chunk_pos(tid + i * NT, r, k);
        if constexpr (TAPS > 1) bctx[i] = bload.prepare_seg(n0, r, k);
        else                    bctx[i] = bload.prepare(n0 + r, k);
    }

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    int g_pass = t_begin / s.k_tiles;
    int g_kt = t_begin - g_pass * s.k_tiles;
    constexpr int KS = BK / KSTEP;              // k-steps per tap
    constexpr int NSTEP = TAPS * KS / WK;       // k-steps of a tile this wavefront multiplies
    constexpr int N_CHUNKS = CPT_A + CPT_B;
    typename ALoad::Tile g_ta;
    typename BLoad::Tile g_tb;
    // Tile descriptors (they may involve scalar table loads) are prepared one
    // request ahead when that is free.  Not for the 8-wavefront shapes, which
    // have no registers to spare, and not when a descriptor reads a table: a
    // scalar load in flight makes every later LDS wait a full wait
    // (scalar and LDS operations share one counter and return out of order).
    constexpr bool PREP_AHEAD = NT <= 256 && !ALoad::TILE_READS_TABLE && !BLoad::TILE_READS_TABLE;
    int g_left = ntiles;
    const typename ALoad::Wave a_wave = aload.wave_init(lane);
    const typename BLoad::Wave b_wave = bload.wave_init(lane);
    bool g_fresh = true;    // the next descriptor starts a pass (or is the first of this workgroup)
    auto gprep = [&]() {
        if (g_left > 0) {
            if constexpr (LoaderIncremental<ALoad>::value) {
                if (g_fresh) g_ta = aload.tile(g_kt, g_kt * BK, z + g_pass, a_wave); else aload.advance(g_ta, BK);
            } else {
                g_ta = aload.tile(g_kt, g_kt * BK, z + g_pass, a_wave);
            }
            if constexpr (LoaderIncremental<BLoad>::value) {
                if (g_fresh) g_tb = bload.tile(g_kt, g_kt * BK, z + g_pass, b_wave); else bload.advance(g_tb, BK);
            } else {
                g_tb = bload.tile(g_kt, g_kt * BK, z + g_pass, b_wave);
            }
            g_fresh = false;
            if (++g_kt == s.k_tiles) { g_kt = 0; g_pass++; g_fresh = true; }
            g_left--;
        }
    };
    if (PREP_AHEAD) gprep();
    // fetch the next global tile into the LDS stage at byte offset `stage_off`
    auto gissue = [&](int stage_off) {
        if (!PREP_AHEAD) gprep();
#pragma unroll
        for (int i = 0; i < CPT_A; i++)
            buffer_load_chunk_to_lds(g_ta.rsrc, smem + stage_off + (i * NT + wave * 64) * 16, aload.offset(g_ta, actx[i]));
#pragma unroll
        for (int i = 0; i < CPT_B; i++)
            buffer_load_chunk_to_lds(g_tb.rsrc, smem + stage_off + TA::BYTES + (i * NT + wave * 64) * 16,
                                     bload.offset(g_tb, bctx[i]));
        if (PREP_AHEAD) gprep();
    };

    // lane-constant fragment addresses (of the first k-step this wavefront multiplies)
    int fa_base[TM], fb_base[TAPS][TN];
#pragma unroll
    for (int i = 0; i < TM; i++) fa_base[i] = FA::skip(FA::base(wm * TM + i, lane), wk * NSTEP);
#pragma unroll
    for (int tap = 0; tap < TAPS; tap++)
#pragma unroll
        for (int j = 0; j < TN; j++)
            fb_base[tap][j] = TA::BYTES + FB::skip(FB::base(wn * TN + j + tap * (TAP_COLS / 32), lane), wk * NSTEP);

    Frag<T> fa[2][TM], fb[2][TN];
    // k-step `step` of a tile: A lines 16*step .. +15; B lines 16*(step % KS) .. +15
    // of the window of tap step / KS
    auto load_frags = [&](int stage_off, int step, Frag<T> (&a)[TM], Frag<T> (&b)[TN]) {
        const char* tile = smem + stage_off;
#pragma unroll
        for (int i = 0; i < TM; i++) a[i] = FA::load(tile + TA::tile_of(step, KS), fa_base[i], TA::step_of(step, KS));
#pragma unroll
        for (int j = 0; j < TN; j++) b[j] = FB::load(tile, fb_base[step / KS][j], step % KS);
    };
    auto multiply = [&](const Frag<T> (&a)[TM], const Frag<T> (&b)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) mfma_step(a[i], b[j], acc[i][j]);
    };

    constexpr int RD_A = (LA == KC) ? 1 : 2;
    constexpr int RD_B = (LB == KC) ? 1 : 2;
    constexpr int N_READS = TM * RD_A + TN * RD_B;
    constexpr int N_MFMA = TM * TN;
    auto step = [&](int rd_stage, int rd_step, Frag<T> (&na)[TM], Frag<T> (&nb)[TN],
                    const Frag<T> (&ca)[TM], const Frag<T> (&cb)[TN]) {
        load_frags(rd_stage, rd_step, na, nb);
        multiply(ca, cb);
        InterleaveStep<0, N_MFMA, N_READS, 0>::emit();
        __builtin_amdgcn_sched_barrier(0);
    };
    // all k-steps of a tile but the last, fragments of the next step prefetched
    auto head_steps = [&](int rd_stage) {
#pragma unroll
        for (int st = 0; st < NSTEP - 1; st++)
            step(rd_stage, st + 1, fa[(st + 1) & 1], fb[(st + 1) & 1], fa[st & 1], fb[st & 1]);
    };

    // Pipeline.  Up to NSTAGE tiles are resident or in flight.  The iteration of
    // tile t runs its first k-steps, waits until tile t+1 has landed, and takes
    // the one barrier of the iteration: behind it no wavefront reads stage
    // t % NSTAGE any more (the fragments of the last k-step are already in
    // registers), so tile t+NSTAGE is requested into it right away and has the
    // time of NSTAGE-1 whole tiles to arrive.  The last k-step of tile t then
    // overlaps the first fragment reads of tile t+1.
    auto next_stage = [&](int off) { return (off + STAGE == NSTAGE * STAGE) ? 0 : off + STAGE; };

#pragma unroll
    for (int p = 0; p < NSTAGE; p++)
        if (p < ntiles) gissue(p * STAGE);
    // tile 0 must have landed; the other prologue tiles may still be in flight
    if (ntiles >= NSTAGE) __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(NSTAGE - 1) * N_CHUNKS>::IMM);
    else                  __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
    __syncthreads();
    int rd_off = 0;
    if (ntiles > 0) load_frags(0, 0, fa[0], fb[0]);

    int t = 0;
    // steady state: every tile consumed frees a stage for tile t + NSTAGE
    for (; t + NSTAGE < ntiles; t++) {
        head_steps(rd_off);
        __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(NSTAGE - 2) * N_CHUNKS>::IMM);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (N_MFMA >= 8) {
            // Last k-step of tile t with the requests for tile t+NSTAGE and the
            // first fragment reads of tile t+1 placed between its MFMAs by hand,
            // one request per MFMA: the matrix pipe keeps running behind the
            // barrier instead of waiting out a burst of requests.  (With fewer
            // MFMAs per step the requests would outnumber them; those shapes
            // issue the burst first.)
            const int wr_off = rd_off;
            rd_off = next_stage(rd_off);
            if (!PREP_AHEAD) gprep();
            const char* tile = smem + rd_off;
            Frag<T> (&na)[TM] = fa[NSTEP & 1];
            Frag<T> (&nb)[TN] = fb[NSTEP & 1];
            const Frag<T> (&ca)[TM] = fa[(NSTEP - 1) & 1];
            const Frag<T> (&cb)[TN] = fb[(NSTEP - 1) & 1];
            constexpr int PER = (N_CHUNKS + N_MFMA - 1) / N_MFMA;
            constexpr int FPM = (TM + TN + N_MFMA - 1) / N_MFMA;   // fragment reads per MFMA
#pragma unroll
            for (int m = 0; m < N_MFMA; m++) {
                mfma_step(ca[m / TN], cb[m % TN], acc[m / TN][m % TN]);
#pragma unroll
                for (int q = 0; q < FPM; q++) {
                    const int f = m * FPM + q;   // fragment of tile t+1 read behind this MFMA
                    if (f < TM) na[f < TM ? f : 0] = FA::load(tile, fa_base[f < TM ? f : 0], 0);
                    else if (f < TM + TN) nb[f >= TM && f < TM + TN ? f - TM : 0] = FB::load(tile, fb_base[0][f >= TM && f < TM + TN ? f - TM : 0], 0);
                }
#pragma unroll
                for (int q = 0; q < PER; q++) {
                    const int c = m * PER + q;
                    if (c < CPT_A) {
                        const int i = c < CPT_A ? c : 0;
                        buffer_load_chunk_to_lds(g_ta.rsrc, smem + wr_off + (i * NT + wave * 64) * 16, aload.offset(g_ta, actx[i]));
                    } else if (c < N_CHUNKS) {
                        const int i = (c >= CPT_A && c < N_CHUNKS) ? c - CPT_A : 0;
                        buffer_load_chunk_to_lds(g_tb.rsrc, smem + wr_off + TA::BYTES + (i * NT + wave * 64) * 16,
                                                 bload.offset(g_tb, bctx[i]));
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (PREP_AHEAD) gprep();
        } else {
            gissue(rd_off);
            __builtin_amdgcn_sched_barrier(0);
            rd_off = next_stage(rd_off);
            step(rd_off, 0, fa[NSTEP & 1], fb[NSTEP & 1], fa[(NSTEP - 1) & 1], fb[(NSTEP - 1) & 1]);
        }
    }
    // drain: nothing left to request
    for (; t + 1 < ntiles; t++) {
        head_steps(rd_off);
        __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        rd_off = next_stage(rd_off);
        step(rd_off, 0, fa[NSTEP & 1], fb[NSTEP & 1], fa[(NSTEP - 1) & 1], fb[(NSTEP - 1) & 1]);
    }
    if (ntiles > 0) {
        head_steps(rd_off);
        multiply(fa[(NSTEP - 1) & 1], fb[(NSTEP - 1) & 1]);
    }

    __syncthreads();
    if constexpr (WK > 1) {
        // add the groups' accumulators into group 0, one group at a time in group
        // order (the order of the additions is fixed); value v of block (i, j) of a
        // sub-tile sits at float ((sub-tile * TM * TN + i * TN + j) * 16 + v) * 64 + lane
        float* red = reinterpret_cast<float*>(smem) + (size_t)wtile * (TM * TN * 16 * 64) + lane;
#pragma unroll 1
        for (int g = 1; g < WK; g++) {
            if (wk == g) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int v = 0; v < 16; v++) red[((i * TN + j) * 16 + v) * 64] = acc[i][j][v];
            }
            __syncthreads();
            if (wk == 0) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int v = 0; v < 16; v++) acc[i][j][v] += red[((i * TN + j) * 16 + v) * 64];
            }
            __syncthreads();
        }
        if (wk != 0) return;    // no barrier follows: the epilogue staging is private to a wavefront
    }
    if constexpr (EpilogueWholeTile<Epi>::value) {
        static_assert(WK == 1, "whole-tile epilogues run on every wavefront");
        static_assert(BM == 32 && WM == 1, "whole-tile epilogues take one block of 32 rows");
        static_assert(32 * BN * 4 <= SMEM_BYTES, "the fp32 tile must fit the LDS of the stages");
        float* g = reinterpret_cast<float*>(smem);
        const int nrows = epi.rows;
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if (row < nrows) g[row * BN + wn * WTN + j * 32 + (lane & 31)] = acc[0][j][v];
            }
        __syncthreads();
        epi.tile(g, tid, NT, n0);
    } else {
        char* stage = smem + wtile * EPI_BYTES;
        EpilogueBands<TM, TN, WTN, EPITCH, 0>::run(acc, stage, lane, m0 + wm * (BM / WM), n0 + wn * WTN, z, split, epi);
    }
}

// ---------------------------------------------------------------------------
// epilogues
// ---------------------------------------------------------------------------

// final rounding: fp32 register -> storage bits, nearest or stochastic
template <typename T> struct StoreBits;
template <> struct StoreBits<_Float16> {
    typedef unsigned short bits_t;
    static __device__ __forceinline__ bits_t round(float v, unsigned sr_bits, unsigned seed, unsigned stream, unsigned idx)
    {
        return sr_bits ? ng_sr_f16(v, sr_bits, ng_rand_sr16(seed, stream, idx)) : ng_f32_to_f16_rn(v);
    }
    // random words of 8 consecutive elements starting at an even index: one
    // draw per pair of elements
    static __device__ __forceinline__ void words8(unsigned seed, unsigned stream, unsigned idx0, unsigned (&w)[8])
    {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const unsigned h = ng_rand32(seed, stream, (idx0 >> 1) + k);
            w[2 * k] = h;
            w[2 * k + 1] = h << 16;
        }
    }
    static __device__ __forceinline__ bits_t round_word(float v, unsigned sr_bits, unsigned r)
    {
        return ng_sr_f16(v, sr_bits, r);
    }
    static __device__ __forceinline__ float widen(bits_t b) { return ng_f16_to_f32(b); }
};
template <> struct StoreBits<float> {
    typedef unsigned bits_t;
    static __device__ __forceinline__ bits_t round(float v, unsigned sr_bits, unsigned seed, unsigned stream, unsigned idx)
    {
        return __float_as_uint(sr_bits ? ng_sr_f32(v, sr_bits, ng_rand32(seed, stream, idx)) : v);
    }
    static __device__ __forceinline__ void words8(unsigned seed, unsigned stream, unsigned idx0, unsigned (&w)[8])
    {
#pragma unroll
        for (int e = 0; e < 8; e++) w[e] = ng_rand32(seed, stream, idx0 + e);
    }
    static __device__ __forceinline__ bits_t round_word(float v, unsigned sr_bits, unsigned r)
    {
        return __float_as_uint(ng_sr_f32(v, sr_bits, r));
    }
    static __device__ __forceinline__ float widen(bits_t b) { return __uint_as_float(b); }
};

// alpha -> relu -> + beta*C -> round -> store
// (order of kernels/sass/hgemm_common_128x128.sass:183-264 in the reference)
template <typename T>
struct ScaleStoreEpilogue {
    typedef typename StoreBits<T>::bits_t bits_t;
    T*       C;
    long     ldcz;
    int      ldc;
    int      m, n;
    float    alpha, beta;
    unsigned relu;
    unsigned sr_bits, seed, stream;
    unsigned vec;   // rows of C are 16-byte aligned and n is a multiple of 8
    // optional tensor laid out like C (16-byte aligned): outputs whose mask
    // element is not positive are stored as zero (the rectifier derivative of
    // the layer whose activations the mask holds)
    const T* mask = nullptr;
    // Optional column fold.  The kernel's columns are rows of fold_from columns of
    // which only the first fold_to exist in C (image rows padded to a whole number
    // of tiles): column q*fold_from + r goes to q*fold_to + r, r >= fold_to to nowhere.
    // n stays the column count of C.  Groups of 8 columns never straddle a fold.
    int      fold_from = 0, fold_to = 0;
    FastDiv  fold_div = FastDiv{0, 0};

    __device__ __forceinline__ const void* base() const { return C; }
    static constexpr bool BUFFER_STORE = sizeof(bits_t) == 2;
    // the case store8_buffer covers (uniform over the launch)
    __device__ __forceinline__ bool plain_store() const
    {
        return vec && beta == 0.0f && sr_bits == 0u && mask == nullptr && fold_from == 0 && (long)m * ldc < (1L << 30);
    }
    __device__ __forceinline__ BufferRsrc store_rsrc(int z) const { return make_rsrc(C + (long)z * ldcz); }
    __device__ __forceinline__ bool masked_out(long offset) const
    {
        return !(StoreBits<T>::widen(reinterpret_cast<const bits_t*>(mask)[offset]) > 0.0f);
    }
    // zero those of 8 consecutive outputs at element offset `offset` whose mask is not positive
    __device__ __forceinline__ void mask8(bits_t (&out)[8], long offset) const
    {
        constexpr int NV = (int)sizeof(bits_t) * 8 / 16;
        bits_t mk[8];
#pragma unroll
        for (int q = 0; q < NV; q++)
            reinterpret_cast<uint4_t*>(mk)[q] = reinterpret_cast<const uint4_t*>(reinterpret_cast<const bits_t*>(mask) + offset)[q];
#pragma unroll
        for (int e = 0; e < 8; e++) out[e] = (StoreBits<T>::widen(mk[e]) > 0.0f) ? out[e] : (bits_t)0;
    }

    __device__ __forceinline__ float scale(float acc) const
    {
        float v = acc * alpha;
        return relu ? fmaxf(v, 0.0f) : v;
    }
    __device__ __forceinline__ unsigned rng_index(int i, int j, int z) const
    {
        return ((unsigned)z * (unsigned)m + (unsigned)i) * (unsigned)n + (unsigned)j;
    }
    __device__ __forceinline__ void apply(int i, int j, int z, float acc) const
    {
        float v = scale(acc);
        const long offset = (long)z * ldcz + (long)i * ldc + j;
        bits_t* p = reinterpret_cast<bits_t*>(C + offset);
        if (beta != 0.0f) v += beta * StoreBits<T>::widen(*p);
        const bits_t r = StoreBits<T>::round(v, sr_bits, seed, stream, rng_index(i, j, z));
        *p = (mask && masked_out(offset)) ? (bits_t)0 : r;
    }
    // The plain case of store8 (16-bit elements, rows of C 16-byte aligned, no beta,
    // nearest rounding, no mask, one matrix) as a descriptor store on C: positions
    // outside the matrix are dropped by the hardware instead of branched around.
    __device__ __forceinline__ void store8_buffer(BufferRsrc rsrc, int i, int j0, const float (&acc)[8]) const
    {
        bits_t out[8];
        if (relu) {
#pragma unroll
            for (int e = 0; e < 8; e++) out[e] = StoreBits<T>::round(fmaxf(acc[e] * alpha, 0.0f), 0, 0, 0, 0);
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) out[e] = StoreBits<T>::round(acc[e] * alpha, 0, 0, 0, 0);
        }
        if constexpr (sizeof(bits_t) == 2) {
            const unsigned off = (i < m && j0 < n) ? ((unsigned)i * (unsigned)ldc + (unsigned)j0) * 2u : NG_OOB_OFFSET;
            buffer_store_chunk(rsrc, off, *reinterpret_cast<const uint4_t*>(out));
        }
    }
    // the same store with an optional stochastic rounding at the full 10 bits (pairs of
    // outputs share a draw): for kernels that must issue the same number of stores from
    // every wavefront whatever the rounding mode; z is the batch index of the descriptor
    __device__ __forceinline__ bool buffer_storable() const
    {
        return sizeof(bits_t) == 2 && vec && beta == 0.0f && (sr_bits == 0u || sr_bits == 10u) && mask == nullptr &&
               fold_from == 0 && (long)m * ldc < (1L << 30);
    }
    __device__ __forceinline__ void store8_buffer_sr(BufferRsrc rsrc, int i, int j0, int z, const float (&acc)[8]) const
    {
        if constexpr (sizeof(bits_t) == 2) {
            if (sr_bits == 0u) {
                store8_buffer(rsrc, i, j0, acc);
            } else {
                const unsigned pair0 = rng_index(i, j0, z) >> 1;
                unsigned packed[4];
#pragma unroll
                for (int q = 0; q < 4; q++)
                    packed[q] = ng_sr10_f16x2(scale(acc[2 * q]), scale(acc[2 * q + 1]), ng_rand32(seed, stream, pair0 + q));
                const unsigned off = (i < m && j0 < n) ? ((unsigned)i * (unsigned)ldc + (unsigned)j0) * 2u : NG_OOB_OFFSET;
                buffer_store_chunk(rsrc, off, *reinterpret_cast<const uint4_t*>(packed));
            }
        }
    }
    __device__ __forceinline__ void store8(int i, int j0, int z, int /*split*/, const float (&acc)[8]) const
    {
        if (fold_from) {
            const int q = (int)fold_div.div((unsigned)j0), r = j0 - q * fold_from;
            if (r >= fold_to) return;
            j0 = q * fold_to + r;
        }
        if (i >= m || j0 >= n) return;
        constexpr int NV = (int)sizeof(bits_t) * 8 / 16;   // 16-byte pieces per 8 elements
        const long offset = (long)z * ldcz + (long)i * ldc + j0;
        bits_t* p = reinterpret_cast<bits_t*>(C + offset);
        if (vec && beta == 0.0f && sr_bits == 0) {
            // common case, kept free of the rounding-stream arithmetic:
            // scale, optional relu, nearest rounding, 16-byte stores
            // (the clamp only exists with relu: NaN and infinities of an
            // unrectified product must reach the output)
            bits_t out[8];
            if (relu) {
#pragma unroll
                for (int e = 0; e < 8; e++) out[e] = StoreBits<T>::round(fmaxf(acc[e] * alpha, 0.0f), 0, 0, 0, 0);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) out[e] = StoreBits<T>::round(acc[e] * alpha, 0, 0, 0, 0);
            }
            if (mask) mask8(out, offset);
#pragma unroll
            for (int q = 0; q < NV; q++)
                reinterpret_cast<uint4_t*>(p)[q] = reinterpret_cast<const uint4_t*>(out)[q];
        } else if (vec && sizeof(bits_t) == 2 && sr_bits == 10u) {
            // fp16 at the full 10 bits: pairs share a draw and a packed convert
            bits_t cur[8];
            if (beta != 0.0f) *reinterpret_cast<uint4_t*>(cur) = *reinterpret_cast<const uint4_t*>(p);
            const unsigned pair0 = rng_index(i, j0, z) >> 1;
            unsigned packed[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                float v0 = scale(acc[2 * q]), v1 = scale(acc[2 * q + 1]);
                if (beta != 0.0f) {
                    v0 += beta * StoreBits<T>::widen(cur[2 * q]);
                    v1 += beta * StoreBits<T>::widen(cur[2 * q + 1]);
                }
                packed[q] = ng_sr10_f16x2(v0, v1, ng_rand32(seed, stream, pair0 + q));
            }
            if (mask) {
                bits_t out[8];
                *reinterpret_cast<uint4_t*>(out) = *reinterpret_cast<const uint4_t*>(packed);
                mask8(out, offset);
                *reinterpret_cast<uint4_t*>(packed) = *reinterpret_cast<const uint4_t*>(out);
            }
            *reinterpret_cast<uint4_t*>(p) = *reinterpret_cast<const uint4_t*>(packed);
        } else if (vec) {
            bits_t out[8];
            if (beta != 0.0f) {
#pragma unroll
                for (int q = 0; q < NV; q++)
                    reinterpret_cast<uint4_t*>(out)[q] = reinterpret_cast<const uint4_t*>(p)[q];
            }
            // n and j0 are multiples of 8 here, so the stream index of the first
            // element is even
            unsigned words[8];
            if (sr_bits) StoreBits<T>::words8(seed, stream, rng_index(i, j0, z), words);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                float v = scale(acc[e]);
                if (beta != 0.0f) v += beta * StoreBits<T>::widen(out[e]);
                out[e] = sr_bits ? StoreBits<T>::round_word(v, sr_bits, words[e]) : StoreBits<T>::round(v, 0, 0, 0, 0);
            }
            if (mask) mask8(out, offset);
#pragma unroll
            for (int q = 0; q < NV; q++)
                reinterpret_cast<uint4_t*>(p)[q] = reinterpret_cast<const uint4_t*>(out)[q];
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (j0 + e < n) apply(i, j0 + e, z, acc[e]);
        }
    }
};

// raw fp32 partial sums for split contraction: ws[split][z][m][n]
struct PartialEpilogue {
    float* ws;
    int    m, n;
    int    zcount;
    unsigned vec;   // n is a multiple of 8

    __device__ __forceinline__ void store8(int i, int j0, int z, int split, const float (&acc)[8]) const
    {
        if (i >= m || j0 >= n) return;
        float* p = ws + (((long)split * zcount + z) * m + i) * (long)n + j0;
        if (vec) {
            float4_t lo = {acc[0], acc[1], acc[2], acc[3]}, hi = {acc[4], acc[5], acc[6], acc[7]};
            reinterpret_cast<float4_t*>(p)[0] = lo;
            reinterpret_cast<float4_t*>(p)[1] = hi;
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (j0 + e < n) p[e] = acc[e];
        }
    }
};

// fixed-order sum of the partial slices followed by the final epilogue.
// vec8: n is a multiple of 8; a thread then owns 8 consecutive columns of a row
// (32-byte loads from every slice, one 16-byte store).
template <typename T, class Epi>
__global__ __launch_bounds__(256)
void splitk_reduce_kernel(const float* __restrict__ ws, int splits, int zcount, int m, int n, Epi epi, unsigned vec8)
{
    const long total = (long)zcount * m * n;
    if (vec8) {
        const long groups = total >> 3;
        const int per_row = n >> 3;
        for (long g = (long)blockIdx.x * 256 + threadIdx.x; g < groups; g += (long)gridDim.x * 256) {
            float acc[8];
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] = 0.0f;
            const float* p = ws + g * 8;
#pragma unroll 4
            for (int sidx = 0; sidx < splits; sidx++) {
                const float4_t lo = *reinterpret_cast<const float4_t*>(p + sidx * total);
                const float4_t hi = *reinterpret_cast<const float4_t*>(p + sidx * total + 4);
#pragma unroll
                for (int e = 0; e < 4; e++) { acc[e] += lo[e]; acc[e + 4] += hi[e]; }
            }
            const long r = g / per_row;
            const int j0 = (int)(g - r * per_row) * 8;
            const int i = (int)(r % m);
            const int z = (int)(r / m);
            epi.store8(i, j0, z, 0, acc);
        }
        return;
    }
    for (long e = (long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long)gridDim.x * 256) {
        float acc = 0.0f;
        for (int sidx = 0; sidx < splits; sidx++) acc += ws[sidx * total + e];
        const int j = (int)(e % n);
        const long r = e / n;
        const int i = (int)(r % m);
        const int z = (int)(r / m);
        epi.apply(i, j, z, acc);
    }
}

// The same reduction for outputs too small to fill the chip with one thread
// per 8 columns (weight gradients of small filters cut into a hundred or more
// slices): 2^lanes_log2 lanes share a group of 8 columns, lane l adds slices
// l, l + L, ... in order, and an exchange tree over the lanes of the group adds
// the lane sums.  The order of the additions depends only on (splits, L), so
// results are reproducible.  n must be a multiple of 8.
template <typename T, class Epi>
__global__ __launch_bounds__(256)
void splitk_reduce_lanes_kernel(const float* __restrict__ ws, int splits, int zcount, int m, int n, Epi epi,
                                int lanes_log2)
{
    const long total = (long)zcount * m * n;
    const long groups = total >> 3;
    const int per_row = n >> 3;
    const int L = 1 << lanes_log2;
    const int gpw = 64 >> lanes_log2;            // groups per wavefront
    const int lane = threadIdx.x & 63;
    const int gi = lane & (gpw - 1);             // consecutive lanes read consecutive groups
    const int l = lane >> (6 - lanes_log2);
    const long wave = ((long)blockIdx.x * 256 + threadIdx.x) >> 6;
    const long nwaves = (long)gridDim.x * 4;
    for (long gb = wave * gpw; gb < groups; gb += nwaves * gpw) {
        const long g = gb + gi;
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = 0.0f;
        if (g < groups) {
            const float* p = ws + g * 8;
#pragma unroll 2
            for (int sidx = l; sidx < splits; sidx += L) {
                const float4_t lo = *reinterpret_cast<const float4_t*>(p + sidx * total);
                const float4_t hi = *reinterpret_cast<const float4_t*>(p + sidx * total + 4);
#pragma unroll
                for (int e = 0; e < 4; e++) { acc[e] += lo[e]; acc[e + 4] += hi[e]; }
            }
        }
        for (int mask = gpw; mask < 64; mask <<= 1) {
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] += __shfl_xor(acc[e], mask, 64);
        }
        if (l == 0 && g < groups) {
            const long r = g / per_row;
            const int j0 = (int)(g - r * per_row) * 8;
            epi.store8((int)(r % m), j0, (int)(r / m), 0, acc);
        }
    }
}

// sum the `splits` partial slices in the scratch arena and run the epilogue
template <typename T, class Epi>
inline void launch_splitk_reduce(const float* ws, int splits, int zcount, int m, int n, const Epi& epi,
                                 hipStream_t stream)
{
    const long total = (long)zcount * m * n;
    const unsigned vec8 = (n % 8 == 0) ? 1u : 0u;
    const long items = vec8 ? total / 8 : total;
    // lanes per group: until the launch has about two wavefronts per SIMD, every
    // lane keeping at least two slices
    int lanes_log2 = 0;
    const long want = (long)device_cu_count() * 512;
    while (vec8 && lanes_log2 < 6 && (items << (lanes_log2 + 1)) <= want && (4 << lanes_log2) <= splits) lanes_log2++;
    if (lanes_log2 > 0) {
        const long threads = items << lanes_log2;
        const int blocks = (int)std::min<long>((threads + 255) / 256, 16384);
        hipLaunchKernelGGL((splitk_reduce_lanes_kernel<T, Epi>), dim3(blocks), dim3(256), 0, stream,
                           ws, splits, zcount, m, n, epi, lanes_log2);
    } else {
        const int blocks = (int)std::min<long>((items + 255) / 256, 16384);
        hipLaunchKernelGGL((splitk_reduce_kernel<T, Epi>), dim3(blocks), dim3(256), 0, stream,
                           ws, splits, zcount, m, n, epi, vec8);
    }
}

// Launch the contraction core: the direct-to-LDS pipeline when both operands
// are plain 16-byte buffer loads of 16-bit elements, the register-staged one
// otherwise (fp32, element-wise edge handling, 8-bit inputs converted on load).
template <typename T, int BM, int BN, int BK, int WM, int WN, int LA, int LB, int NSTAGE = 2, int WK = 1, class ALoad,
          class BLoad, class Epi>
inline void launch_mfma_core(dim3 grid, hipStream_t stream, const ALoad& al, const BLoad& bl, const Epi& epi,
                             const CoreShape& s)
{
    if constexpr (sizeof(T) == 2 && ALoad::DIRECT && BLoad::DIRECT) {
        hipLaunchKernelGGL((mfma_gemm_direct_kernel<T, BM, BN, BK, WM, WN, LA, LB, NSTAGE, ALoad, BLoad, Epi, WK>), grid,
                           dim3(WM * WN * WK * 64), 0, stream, al, bl, epi, s);
    } else {
        static_assert(WK == 1, "the register-staged kernel does not split its k-steps over wavefront groups");
        hipLaunchKernelGGL((mfma_gemm_kernel<T, BM, BN, BK, WM, WN, LA, LB, ALoad, BLoad, Epi>), grid,
                           dim3(WM * WN * 64), 0, stream, al, bl, epi, s);
    }
}

}  // namespace ng
