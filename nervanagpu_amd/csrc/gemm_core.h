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
    int splits;        // the (passes * k_tiles) tile range is cut into this many slices (gridDim.y)
    int tiles_m, tiles_n;
};

// Dense row-major operand.  KC: element (r,k) at base[r*ld + k]; MC: at base[k*ld + r].
// VEC: the host guarantees 16-byte alignment of every chunk and that chunks do
// not straddle the matrix edge; otherwise elements are fetched one by one.
template <typename T, int LAYOUT, bool VEC>
struct DenseLoader {
    const T* base;
    long     ldz;    // batch / pass stride in elements
    int      ld;
    int      rows;   // extent along r
    int      kdim;   // extent along k (per pass)

    typedef int Ctx;   // per-chunk row context: the row index itself
    __device__ __forceinline__ Ctx prepare(int r) const { return r; }

    __device__ __forceinline__ uint4_t load(const Ctx& r, int k, int zb) const
    {
        constexpr int EPC = Elem<T>::EPC;
        const T* p = base + (long)zb * ldz;
        uint4_t out = {0u, 0u, 0u, 0u};
        if (VEC) {
            if (r < rows && k < kdim) {
                const T* q = (LAYOUT == KC) ? p + (long)r * ld + k : p + (long)k * ld + r;
                out = *reinterpret_cast<const uint4_t*>(q);
            }
        } else {
            T tmp[EPC];
#pragma unroll
            for (int e = 0; e < EPC; e++) {
                const int rr = (LAYOUT == KC) ? r : r + e;
                const int kk = (LAYOUT == KC) ? k + e : k;
                tmp[e] = (rr < rows && kk < kdim)
                             ? ((LAYOUT == KC) ? p[(long)rr * ld + kk] : p[(long)kk * ld + rr])
                             : (T)0;
            }
            out = *reinterpret_cast<const uint4_t*>(tmp);
        }
        return out;
    }
};

// blockIdx.x -> (tile_m, tile_n).  Workgroups are handed to the 8 XCDs round
// robin; renumbering them so that each XCD works on a contiguous range of tiles
// keeps the operand tiles it re-reads in its own L2.
__device__ __forceinline__ void tile_of_block(const CoreShape& s, int& tm, int& tn)
{
    int pid = blockIdx.x;
    const int total = gridDim.x;
    if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    tm = pid % s.tiles_m;
    tn = pid / s.tiles_m;
}

// One 32-row band of a wavefront's accumulators: registers -> private LDS
// staging -> 8-column chunks handed to the epilogue functor.  The band index is
// a template parameter so that every accumulator access is a static register
// reference.
template <int TM, int TN, int WTN, int EPITCH, int I>
struct EpilogueBands {
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
        __syncthreads();
#pragma unroll
        for (int c = 0; c < CPW / 64; c++) {
            const int id = lane + c * 64;
            const int r = id / (WTN / 8);
            const int cc = (id % (WTN / 8)) * 8;
            const float4_t lo = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4);
            const float4_t hi = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4 + 16);
            const float vals[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            epi.store8(mbase + I * 32 + r, nbase + cc, z, split, vals);
        }
        __syncthreads();
        if constexpr (I + 1 < TM)
            EpilogueBands<TM, TN, WTN, EPITCH, I + 1>::run(acc, stage, lane, mbase, nbase, z, split, epi);
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
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % KSTEP == 0, "bad tile shape");

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

    int tm, tn;
    tile_of_block(s, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int z = blockIdx.z;
    const int split = blockIdx.y;

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
    for (int i = 0; i < CPT_A; i++) actx[i] = aload.prepare(m0 + ra_r[i]);
#pragma unroll
    for (int i = 0; i < CPT_B; i++) bctx[i] = bload.prepare(n0 + rb_r[i]);

    uint4_t ra[CPT_A], rb[CPT_B];
    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    auto gload = [&](int t) {
        const int pass = t / s.k_tiles;
        const int k0 = (t - pass * s.k_tiles) * BK;
#pragma unroll
        for (int i = 0; i < CPT_A; i++) ra[i] = aload.load(actx[i], k0 + ra_k[i], z + pass);
#pragma unroll
        for (int i = 0; i < CPT_B; i++) rb[i] = bload.load(bctx[i], k0 + rb_k[i], z + pass);
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < CPT_A; i++) *reinterpret_cast<uint4_t*>(smem + buf * STAGE + ra_off[i]) = ra[i];
#pragma unroll
        for (int i = 0; i < CPT_B; i++) *reinterpret_cast<uint4_t*>(smem + buf * STAGE + TA::BYTES + rb_off[i]) = rb[i];
    };

    if (t_begin < t_end) {
        gload(t_begin);
        sstore(0);
    }
    __syncthreads();

    for (int t = t_begin; t < t_end; t++) {
        const int buf = (t - t_begin) & 1;
        const bool more = (t + 1 < t_end);
        if (more) gload(t + 1);

        const char* a_lds = smem + buf * STAGE;
        const char* b_lds = a_lds + TA::BYTES;
#pragma unroll
        for (int kk = 0; kk < BK; kk += KSTEP) {
            Frag<T> fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++)
                fa[i] = FragLoader<T, LA, TA::PITCH>::load(a_lds, wm * (BM / WM) + i * 32, kk, lane);
#pragma unroll
            for (int j = 0; j < TN; j++)
                fb[j] = FragLoader<T, LB, TB::PITCH>::load(b_lds, wn * (BN / WN) + j * 32, kk, lane);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) mfma_step(fa[i], fb[j], acc[i][j]);
        }

        if (more) sstore(buf ^ 1);
        __syncthreads();
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
// epilogues
// ---------------------------------------------------------------------------

// final rounding: fp32 register -> storage bits, nearest or stochastic
template <typename T> struct StoreBits;
template <> struct StoreBits<_Float16> {
    typedef unsigned short bits_t;
    static __device__ __forceinline__ bits_t round(float v, unsigned sr_bits, unsigned seed, unsigned stream, unsigned idx)
    {
        return sr_bits ? ng_sr_f16(v, sr_bits, ng_rand32(seed, stream, idx)) : ng_f32_to_f16_rn(v);
    }
    static __device__ __forceinline__ float widen(bits_t b) { return ng_f16_to_f32(b); }
};
template <> struct StoreBits<float> {
    typedef unsigned bits_t;
    static __device__ __forceinline__ bits_t round(float v, unsigned sr_bits, unsigned seed, unsigned stream, unsigned idx)
    {
        return __float_as_uint(sr_bits ? ng_sr_f32(v, sr_bits, ng_rand32(seed, stream, idx)) : v);
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
        bits_t* p = reinterpret_cast<bits_t*>(C + (long)z * ldcz + (long)i * ldc + j);
        if (beta != 0.0f) v += beta * StoreBits<T>::widen(*p);
        *p = StoreBits<T>::round(v, sr_bits, seed, stream, rng_index(i, j, z));
    }
    __device__ __forceinline__ void store8(int i, int j0, int z, int /*split*/, const float (&acc)[8]) const
    {
        if (i >= m || j0 >= n) return;
        if (vec) {
            constexpr int NV = (int)sizeof(bits_t) * 8 / 16;   // 16-byte pieces per 8 elements
            bits_t* p = reinterpret_cast<bits_t*>(C + (long)z * ldcz + (long)i * ldc + j0);
            bits_t out[8];
            if (beta != 0.0f) {
#pragma unroll
                for (int q = 0; q < NV; q++)
                    reinterpret_cast<uint4_t*>(out)[q] = reinterpret_cast<const uint4_t*>(p)[q];
            }
            const unsigned idx0 = rng_index(i, j0, z);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                float v = scale(acc[e]);
                if (beta != 0.0f) v += beta * StoreBits<T>::widen(out[e]);
                out[e] = StoreBits<T>::round(v, sr_bits, seed, stream, idx0 + e);
            }
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

// fixed-order sum of the partial slices followed by the final epilogue
template <typename T, class Epi>
__global__ void splitk_reduce_kernel(const float* ws, int splits, int zcount, int m, int n, Epi epi)
{
    const long total = (long)zcount * m * n;
    const long slice = total;
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
        float acc = 0.0f;
        for (int sidx = 0; sidx < splits; sidx++) acc += ws[sidx * slice + e];
        const int j = (int)(e % n);
        const long r = e / n;
        const int i = (int)(r % m);
        const int z = (int)(r / m);
        epi.apply(i, j, z, acc);
    }
}

}  // namespace ng
