// GEMM entry points: C = round(beta*C + relu(alpha * op(A).op(B))).
// Replaces the {h,s}gemm_{nn,nt,tn}[_vec]_{tile} kernel family selected in
// NervanaGPU.dot / batched_dot (nervanagpu/nervanagpu.py:820-1105) and the
// GEMM-only C interface (kernels/C_interface/nervana_c_api.h:31-128).
#include "gemm_core.h"
#include "stream_core.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <mutex>

namespace ng {

struct GemmArgs {
    int trans_a, trans_b;
    int m, n, k;
    const void* A; int lda;
    const void* B; int ldb;
    void* C; int ldc;
    float alpha, beta;
    unsigned flags, seed, rng_stream;
    int batch_grid; long ldaz, ldbz, ldcz; int batch_loops;
    void* ws; size_t ws_bytes;
    hipStream_t stream;
};

struct TileChoice { int bm, bn, bk, threads; };

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

// how many slices to cut the contraction into so that the grid fills the chip
static int choose_splits(int out_tiles, int total_k_tiles, size_t slice_bytes, size_t ws_bytes)
{
    const int cus = device_cu_count();
    if (out_tiles >= cus || total_k_tiles < 8) return 1;
    // about one and a half workgroups per CU: more slices only add fp32 partials
    int splits = ceil_div(3 * cus / 2, out_tiles);
    splits = std::min(splits, total_k_tiles / 4);
    if (slice_bytes) splits = (int)std::min<size_t>((size_t)splits, ws_bytes / slice_bytes);
    // every slice must own at least one tile
    while (splits > 1 && (splits - 1) * ceil_div(total_k_tiles, splits) >= total_k_tiles) splits--;
    return std::max(splits, 1);
}

// Slices for the minibatch-wide shapes (one column tile, long contraction), whose
// workgroups hold a whole CU each: as many as give every CU at most one workgroup,
// each slice at least four contraction tiles deep.  A grid of one and a half
// workgroups per CU would take as long as one of two per CU.
static int one_per_cu_splits(int out_tiles, int total_k_tiles, size_t slice_bytes, size_t ws_bytes)
{
    int splits = std::max(1, device_cu_count() / std::max(out_tiles, 1));
    splits = std::min(splits, std::max(1, total_k_tiles / 4));
    if (slice_bytes) splits = (int)std::min<size_t>((size_t)splits, ws_bytes / slice_bytes);
    while (splits > 1 && (splits - 1) * ceil_div(total_k_tiles, splits) >= total_k_tiles) splits--;
    return std::max(splits, 1);
}

template <typename T, int BM, int BN, int BK, int WM, int WN, int LA, int LB, bool VEC, int NSTAGE = 2, int WK = 1,
          bool ONE_PER_CU = (WK > 1)>
static int launch_gemm(const GemmArgs& g, unsigned sr_bits)
{
    CoreShape s;
    s.m = g.m; s.n = g.n;
    s.k_tiles = ceil_div(g.k, BK);
    s.passes = g.batch_loops;
    s.tiles_m = ceil_div(g.m, BM);
    s.tiles_n = ceil_div(g.n, BN);
    const int zcount = g.batch_grid;
    const int out_tiles = s.tiles_m * s.tiles_n * zcount;
    const size_t slice_bytes = (size_t)zcount * g.m * g.n * sizeof(float);
    if (ONE_PER_CU) s.splits = g.ws ? one_per_cu_splits(out_tiles, s.passes * s.k_tiles, slice_bytes, g.ws_bytes) : 1;
    else        s.splits = g.ws ? choose_splits(out_tiles, s.passes * s.k_tiles, slice_bytes, g.ws_bytes) : 1;

    DenseLoader<T, LA, VEC> al{(const T*)g.A, g.ldaz, g.lda, g.m, g.k};
    DenseLoader<T, LB, VEC> bl{(const T*)g.B, g.ldbz, g.ldb, g.n, g.k};
    ScaleStoreEpilogue<T> epi{(T*)g.C, g.ldcz, g.ldc, g.m, g.n, g.alpha, g.beta,
                              (g.flags & NG_FLAG_RELU) ? 1u : 0u, sr_bits, g.seed, g.rng_stream,
                              (((uintptr_t)g.C & 15) == 0 && g.ldc % 8 == 0 && g.ldcz % 8 == 0 && g.n % 8 == 0) ? 1u : 0u};

    dim3 grid(grid_tiles(s.tiles_m * s.tiles_n, s.splits), grid_slices(s.tiles_m * s.tiles_n, s.splits), zcount);
    if (s.splits == 1) {
        launch_mfma_core<T, BM, BN, BK, WM, WN, LA, LB, NSTAGE, WK>(grid, g.stream, al, bl, epi, s);
        NG_CHECK_LAUNCH("gemm kernel");
    } else {
        PartialEpilogue pe{(float*)g.ws, g.m, g.n, zcount, (g.n % 8 == 0) ? 1u : 0u};
        launch_mfma_core<T, BM, BN, BK, WM, WN, LA, LB, NSTAGE, WK>(grid, g.stream, al, bl, pe, s);
        NG_CHECK_LAUNCH("gemm split kernel");
        launch_splitk_reduce<T, ScaleStoreEpilogue<T>>((const float*)g.ws, s.splits, zcount, g.m, g.n, epi, g.stream);
        NG_CHECK_LAUNCH("gemm split reduce");
    }
    return 0;
}

template <typename T, int BM, int BN, int BK, int WM, int WN, bool VEC, int NSTAGE = 2, int WK = 1, bool ONE_PER_CU = (WK > 1)>
static int launch_layout(const GemmArgs& g, unsigned sr_bits)
{
    if (!g.trans_a && !g.trans_b) return launch_gemm<T, BM, BN, BK, WM, WN, KC, MC, VEC, NSTAGE, WK, ONE_PER_CU>(g, sr_bits);
    if (!g.trans_a && g.trans_b)  return launch_gemm<T, BM, BN, BK, WM, WN, KC, KC, VEC, NSTAGE, WK, ONE_PER_CU>(g, sr_bits);
    return launch_gemm<T, BM, BN, BK, WM, WN, MC, MC, VEC, NSTAGE, WK, ONE_PER_CU>(g, sr_bits);
}

// B operand of the streaming kernel for a dense "nt" product: column c of the
// product is row c of B (n x k, contraction contiguous)
struct DenseRowsGather {
    const _Float16* X;
    int ld, n, kdim;
    struct Fixed { unsigned off; };
    struct Col { unsigned off; };
    __device__ __forceinline__ Fixed fixed(int k) const { return Fixed{k < kdim ? (unsigned)k * 2u : NG_OOB_OFFSET}; }
    __device__ __forceinline__ Col col(int c) const { return Col{c < n ? (unsigned)c * (unsigned)ld * 2u : NG_OOB_OFFSET}; }
    // both parts are below 2^31 when valid, so bit 31 of the sum flags an invalid part
    __device__ __forceinline__ unsigned offset(const Fixed& f, const Col& c) const
    {
        return ((f.off | c.off) & NG_OOB_OFFSET) ? NG_OOB_OFFSET : f.off + c.off;
    }
};

// "nt" products with a contraction of at most 128 (the weight gradient of a fully
// connected layer at a minibatch of 128: m x n outputs from 128-deep rows) are
// bound by the output stream.  64 rows of A stay in registers as MFMA fragments
// while the rows of B run through the LDS ring of the streaming kernel, 256 output
// columns per tile, and the stores of one tile overlap the requests of the next.
template <int KT, bool SR, int NSTAGE = 4, int PER_CU = 1>
static int launch_nt_stream(const GemmArgs& g, unsigned sr_bits)
{
    typedef _Float16 T;
    constexpr int BM = 64, BN = 256, BK = 32, WN = 4;
    DenseLoader<T, KC, true> al{(const T*)g.A, 0, g.lda, g.m, g.k};
    DenseRowsGather bg{(const T*)g.B, g.ldb, g.n, g.k};
    ScaleStoreEpilogue<T> epi{(T*)g.C, 0, g.ldc, g.m, g.n, g.alpha, 0.0f, (g.flags & NG_FLAG_RELU) ? 1u : 0u,
                              sr_bits, g.seed, g.rng_stream, 1u};
    const int tiles = ceil_div(g.n, BN), row_blocks = ceil_div(g.m, BM);
    // PER_CU workgroups fit the LDS of a CU (a ring of four stages: one; of two stages: two, whose
    // stores and stochastic rounding overlap each other's products): as many column groups as fill those slots
    const int col_groups = std::max(1, std::min(tiles, PER_CU * device_cu_count() / row_blocks));
    launch_stream_rows<T, BM, BN, BK, WN, KT, KC, KC, NSTAGE, SR>(al, bg, epi, tiles, row_blocks, col_groups, g.stream);
    NG_CHECK_LAUNCH("gemm nt (streamed columns)");
    return 0;
}

static bool nt_streams(const GemmArgs& g, unsigned sr_bits)
{
    return !g.trans_a && g.trans_b && g.k <= 128 && g.k > 32 && g.m >= 64 && g.n >= 1024 && g.batch_grid == 1 &&
           g.batch_loops == 1 && g.beta == 0.0f && (sr_bits == 0u || sr_bits == 10u) &&
           ((uintptr_t)g.C & 15) == 0 && g.ldc % 8 == 0 && g.n % 8 == 0 && (long)g.m * g.ldc < (1L << 30) &&
           (long)g.n * g.ldb < (1L << 30) && ceil_div(g.m, 64) <= 65535;
}

template <typename T>
static bool operands_vectorizable(const GemmArgs& g)
{
    constexpr int EPC = Elem<T>::EPC;
    // 16-byte chunks must be aligned and whole, and one matrix must fit the
    // 2 GiB window of a buffer descriptor
    auto ok = [&](const void* p, int ld, long ldz, int contiguous_extent, int other_extent) {
        return ((uintptr_t)p & 15) == 0 && ld % EPC == 0 && ldz % EPC == 0 && contiguous_extent % EPC == 0 &&
               (long)other_extent * ld * (long)sizeof(T) < (1L << 31);
    };
    const bool a = ok(g.A, g.lda, g.ldaz, g.trans_a ? g.m : g.k, g.trans_a ? g.k : g.m);
    const bool b = ok(g.B, g.ldb, g.ldbz, g.trans_b ? g.k : g.n, g.trans_b ? g.n : g.k);
    return a && b;
}

template <typename T> static int dispatch(const GemmArgs& g, unsigned sr_bits);

template <>
int dispatch<_Float16>(const GemmArgs& g, unsigned sr_bits)
{
    if (!operands_vectorizable<_Float16>(g)) return launch_layout<_Float16, 128, 128, 64, 2, 2, false>(g, sr_bits);
    const int cus = device_cu_count();
    const int k_tiles = ceil_div(g.k, 64) * g.batch_loops;
    {
        // A candidate that has passed the CPU emulation but has not been measured on a device yet: off unless
        // NG_NT_STREAM is set (1: four ring stages, one workgroup per CU; 2: two stages, two per CU)
        static const int nt_stream = getenv("NG_NT_STREAM") ? atoi(getenv("NG_NT_STREAM")) : 0;
        if (nt_stream && nt_streams(g, sr_bits)) {
            if (g.k <= 64) return sr_bits ? launch_nt_stream<2, true>(g, sr_bits) : launch_nt_stream<2, false>(g, sr_bits);
            if (nt_stream == 2) return sr_bits ? launch_nt_stream<4, true, 2, 2>(g, sr_bits) : launch_nt_stream<4, false, 2, 2>(g, sr_bits);
            return sr_bits ? launch_nt_stream<4, true>(g, sr_bits) : launch_nt_stream<4, false>(g, sr_bits);
        }
    }
    // 256x256 tiles when they cover more than half the chip and the contraction
    // is long enough to amortise their prologue and epilogue (exactly half the
    // chip is one full round of 128x128 tiles at two workgroups per CU, which is
    // a third faster)
    const long big_tiles = (long)ceil_div(g.m, 256) * ceil_div(g.n, 256) * g.batch_grid;
    if (g.m >= 256 && g.n >= 256 && big_tiles > cus / 2 && k_tiles >= 8)
        return launch_layout<_Float16, 256, 256, 64, 2, 4, true>(g, sr_bits);
    // minibatch-wide outputs (n <= 128) stream the weight matrix: halve the row
    // tile so that fewer contraction slices, i.e. fewer fp32 partials, fill the chip
    const long tiles128 = (long)ceil_div(g.m, 128) * ceil_div(g.n, 128) * g.batch_grid;
    if (tiles128 >= cus) {
        // short contractions are all prologue and epilogue: half-depth tiles halve
        // the LDS footprint, so more workgroups overlap their loads and stores
        if (k_tiles <= 4) return launch_layout<_Float16, 128, 128, 32, 2, 2, true>(g, sr_bits);
        // about one workgroup per CU: no second workgroup overlaps the wait for a
        // tile, a third stage does (2048^3: 29.5 -> 25.4 us)
        if (4 * tiles128 <= 5 * cus && k_tiles >= 16) return launch_layout<_Float16, 128, 128, 64, 2, 2, true, 3>(g, sr_bits);
        return launch_layout<_Float16, 128, 128, 64, 2, 2, true>(g, sr_bits);
    }
    if (g.n <= 128) {
        // Candidates that have passed the CPU emulation but have not been measured on a device yet: NG_FC_CFG
        // (read once per process) picks one; unset, the measured 64x128x64 tile on 2x2 wavefronts runs
        static const int fc_cfg = getenv("NG_FC_CFG") ? atoi(getenv("NG_FC_CFG")) : 0;
        if (g.n > 64 && g.batch_grid == 1 && k_tiles >= 8) {
            int cfg = fc_cfg;
            if (cfg < 0) {
                // the rule the candidates would be used by, from what their designs predict (to be
                // replaced by what the first measurement says): few rows of a row-major A on 32-row
                // tiles; rows that 64-row tiles spread over at most a chip on those (half the partial
                // sums of 128-row tiles); more rows on 128-row tiles
                const int tiles64 = ceil_div(g.m, 64);
                if (!g.trans_a && g.m <= 2048) cfg = 10;
                else if (tiles64 <= cus / 2) cfg = 11;
                else cfg = 9;
            }
            switch (cfg) {
            case 1: return launch_layout<_Float16, 128, 128, 64, 4, 1, true, 4, 2>(g, sr_bits);
            case 2: return launch_layout<_Float16, 64, 128, 128, 2, 1, true, 3, 4>(g, sr_bits);
            case 3: return launch_layout<_Float16, 128, 128, 128, 2, 1, true, 2, 4>(g, sr_bits);
            case 4: return launch_layout<_Float16, 64, 128, 64, 2, 1, true, 4, 2>(g, sr_bits);
            case 6: return launch_layout<_Float16, 128, 128, 64, 2, 2, true, 4, 2>(g, sr_bits);
            case 7:   // few rows (m <= 2048): 32-row tiles, four wavefronts splitting a 128-deep tile
                if (!g.trans_a && !g.trans_b) return launch_gemm<_Float16, 32, 128, 128, 1, 1, KC, MC, true, 3, 4>(g, sr_bits);
                return launch_layout<_Float16, 64, 128, 64, 2, 1, true, 4, 2>(g, sr_bits);
            case 10:  // as 7 with a fourth stage: the four tiles of a 512-deep slice are all requested at once
                if (!g.trans_a && !g.trans_b) return launch_gemm<_Float16, 32, 128, 128, 1, 1, KC, MC, true, 4, 4>(g, sr_bits);
                return launch_layout<_Float16, 64, 128, 64, 2, 1, true, 4, 2>(g, sr_bits);
            // the same rows without the in-workgroup split: a whole CU of LDS as stages of the weight stream
            case 8: return launch_layout<_Float16, 128, 128, 32, 2, 2, true, 8, 1, true>(g, sr_bits);
            case 9: return launch_layout<_Float16, 128, 128, 64, 2, 2, true, 4, 1, true>(g, sr_bits);
            // 64 rows (half the slices, i.e. half the partial sums, of 128) with six stages: 40 KB of weights in flight
            case 11: return launch_layout<_Float16, 64, 128, 64, 2, 2, true, 6, 1, true>(g, sr_bits);
            case 12: return launch_layout<_Float16, 64, 128, 64, 2, 1, true, 6, 2>(g, sr_bits);
            // the measured kernel and its slicing (one and a half workgroups per CU; two fit) with a third stage only
            case 13: return launch_layout<_Float16, 64, 128, 64, 2, 2, true, 3>(g, sr_bits);
            default: break;
            }
        }
        return launch_layout<_Float16, 64, 128, 64, 2, 2, true>(g, sr_bits);
    }
    // long contractions over half a chip or more of 128x128 tiles: two slices of
    // those beat the small tiles (1792x1792x4096 55 -> 42 us, 1536x1536x8192 88 -> 53 us)
    if (2 * tiles128 >= cus && k_tiles >= 48) return launch_layout<_Float16, 128, 128, 64, 2, 2, true>(g, sr_bits);
    // mid-sized outputs: small tiles fill the chip without (or with fewer)
    // contraction slices, which cost fp32 partials and a second launch
    return launch_layout<_Float16, 64, 64, 64, 2, 2, true>(g, sr_bits);
}

template <>
int dispatch<float>(const GemmArgs& g, unsigned sr_bits)
{
    if (!operands_vectorizable<float>(g)) return launch_layout<float, 128, 128, 16, 2, 2, false>(g, sr_bits);
    const long tiles128 = (long)ceil_div(g.m, 128) * ceil_div(g.n, 128) * g.batch_grid;
    if (tiles128 >= device_cu_count() || g.n <= 128) return launch_layout<float, 128, 128, 16, 2, 2, true>(g, sr_bits);
    return launch_layout<float, 64, 64, 32, 2, 2, true>(g, sr_bits);
}

static int check_args(const GemmArgs& g, int dtype)
{
    if (dtype != NG_F16 && dtype != NG_F32) return fail(-20, "ng_gemm: only floating point dot is supported");
    if (g.trans_a && g.trans_b) return fail(-21, "ng_gemm: op \"tt\" is not supported");
    if (g.m < 0 || g.n < 0 || g.k < 0) return fail(-22, "ng_gemm: negative extent");
    if (g.batch_grid < 1 || g.batch_loops < 1) return fail(-23, "ng_gemm: batch_grid and batch_loops must be >= 1");
    if (g.batch_grid > 1 && g.batch_loops > 1) return fail(-24, "ng_gemm: batch_grid and batch_loops are exclusive");
    if (g.m && g.n && (!g.C || (g.k && (!g.A || !g.B)))) return fail(-25, "ng_gemm: null operand");
    const int a_cols = g.trans_a ? g.m : g.k, b_cols = g.trans_b ? g.k : g.n;
    if (g.lda < a_cols || g.ldb < b_cols || g.ldc < g.n) return fail(-26, "ng_gemm: leading dimension smaller than row length");
    if ((long)g.batch_grid * g.m * g.n >= (1L << 32)) return fail(-27, "ng_gemm: output larger than 2^32 elements");
    return 0;
}

static unsigned sr_bits_of(unsigned flags, int dtype)
{
    if (!(flags & NG_FLAG_SR)) return 0;
    unsigned bits = flags >> 16;
    if (bits == 0) bits = 10;
    const unsigned cap = (dtype == NG_F16) ? 10u : 15u;
    return std::max(1u, std::min(bits, cap));
}

}  // namespace ng

using namespace ng;

extern "C" {

size_t ng_gemm_workspace_bytes(int dtype, int trans_a, int trans_b, int m, int n, int k,
                               int batch_grid, int batch_loops)
{
    (void)trans_a; (void)trans_b;
    const int bk = (dtype == NG_F16) ? 64 : 16;
    const int total_k = ceil_div(k, bk) * batch_loops;
    // the largest slice count any tile shape the dispatcher may pick would use
    int splits = 1;
    for (int bm : {64, 128})
        for (int bn : {64, 128})
            splits = std::max(splits, choose_splits(ceil_div(m, bm) * ceil_div(n, bn) * batch_grid, total_k, 0, 0));
    // the minibatch-wide kernels (64-deep tiles or deeper) run one workgroup per CU
    if (dtype == NG_F16 && n <= 128)
        for (int bm : {32, 64, 128}) splits = std::max(splits, one_per_cu_splits(ceil_div(m, bm) * batch_grid, total_k, 0, 0));
    if (splits <= 1) return 0;
    return (size_t)splits * batch_grid * m * n * sizeof(float);
}

int ng_gemm(int dtype, int trans_a, int trans_b, int m, int n, int k,
            const void* A, int lda, const void* B, int ldb, void* C, int ldc,
            float alpha, float beta, unsigned flags,
            unsigned seed, unsigned rng_stream,
            int batch_grid, long ldaz, long ldbz, long ldcz, int batch_loops,
            void* workspace, size_t workspace_bytes, void* stream)
{
    GemmArgs g{trans_a, trans_b, m, n, k, A, lda, B, ldb, C, ldc, alpha, beta, flags, seed, rng_stream,
               batch_grid, ldaz, ldbz, ldcz, batch_loops, workspace, workspace_bytes, (hipStream_t)stream};
    int rc = check_args(g, dtype);
    if (rc) return rc;
    if (m == 0 || n == 0) return 0;
    const unsigned sr_bits = sr_bits_of(flags, dtype);
    return dtype == NG_F16 ? dispatch<_Float16>(g, sr_bits) : dispatch<float>(g, sr_bits);
}

// ---- GEMM without allocation ------------------------------------------------
// Split-contraction partial sums live in a device array that is part of the
// loaded code object, so a caller that cannot allocate (stream capture, serving
// loops) still gets the sliced schedule of the minibatch-wide shapes.  Every
// device holds its own copy of the array; its address on a device is looked up
// once, with that device current, and only that address is handed to kernels.
}  // extern "C"

static __device__ __align__(256) unsigned char scratch[NG_GEMM_STATIC_SCRATCH_BYTES];

static constexpr int MAX_DEVICES = 64;
// written once per device under the mutex, read by every call without it
static std::atomic<void*> g_scratch_ptr[MAX_DEVICES];
static std::mutex g_scratch_mutex;
// The nervana_* entry points also put their partial sums into the array.  Their
// callers may use several streams, so the last call that used it leaves an event
// behind, and a call on another stream waits for that event first.
struct ScratchOrder { hipEvent_t done; hipStream_t last; bool used; };
static ScratchOrder g_scratch_order[MAX_DEVICES];

namespace ng {

// called by ng_init with `device` current; idempotent
int gemm_static_scratch_setup(int device)
{
    if (device < 0 || device >= MAX_DEVICES) return fail(-30, "device index %d out of range", device);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device].load(std::memory_order_acquire)) return 0;
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (!ptr) return fail(-31, "static scratch has no device address");
    e = hipEventCreateWithFlags(&g_scratch_order[device].done, hipEventDisableTiming);
    if (e != hipSuccess) return hip_fail(e, "hipEventCreateWithFlags(scratch order)");
    g_scratch_order[device].used = false;
    g_scratch_ptr[device].store(ptr, std::memory_order_release);
    return 0;
}

}  // namespace ng

extern "C" {

size_t ng_gemm_static_scratch_bytes(void) { return NG_GEMM_STATIC_SCRATCH_BYTES; }

int ng_gemm_noalloc(int dtype, int trans_a, int trans_b, int m, int n, int k,
                    const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                    float alpha, float beta, unsigned flags,
                    unsigned seed, unsigned rng_stream,
                    int batch_grid, long ldaz, long ldbz, long ldcz, int batch_loops,
                    void* stream)
{
    int dev = -1;
    NG_HIP(hipGetDevice(&dev));
    void* const arena = (dev >= 0 && dev < MAX_DEVICES) ? g_scratch_ptr[dev].load(std::memory_order_acquire) : nullptr;
    if (!arena) return fail(-32, "ng_gemm_noalloc: ng_init has not been called for device %d", dev);
    if (m < 0 || n < 0 || k < 0 || batch_grid < 1 || batch_loops < 1)
        return fail(-22, "ng_gemm_noalloc: bad extent");
    const size_t need = ng_gemm_workspace_bytes(dtype, trans_a, trans_b, m, n, k, batch_grid, batch_loops);
    if (need > (size_t)NG_GEMM_STATIC_SCRATCH_BYTES)
        return fail(-33, "ng_gemm_noalloc: this problem wants %zu bytes of partial sums, the static scratch holds %zu; "
                         "use ng_gemm with a caller workspace", need, (size_t)NG_GEMM_STATIC_SCRATCH_BYTES);
    // partial slices are written in full by the split kernel before the reduce
    // reads them, so nothing in the array has to start at zero
    return ng_gemm(dtype, trans_a, trans_b, m, n, k, A, lda, B, ldb, C, ldc, alpha, beta, flags, seed, rng_stream,
                   batch_grid, ldaz, ldbz, ldcz, batch_loops,
                   need ? arena : nullptr, need, stream);
}

// ---- GEMM-only C interface (kernels/C_interface/nervana_c_api.h) -----------

bool nervana_loadKernels(const char* /*base_path*/)
{
    // kernels are linked into this library; select the current device
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    return ng_init(dev) == 0;
}

bool nervana_unloadKernels(void) { return true; }

size_t nervana_randStateSizeBytes(void) { return 2048 * 32 * sizeof(unsigned); }

static bool c_gemm(int dtype, void* A, void* B, void* C, bool a_t, bool b_t, int m, int n, int k,
                   int lda, int ldb, int ldc, float alpha, float beta, bool sr, bool relu, void* stream)
{
    unsigned flags = (sr ? (NG_FLAG_SR | (10u << 16)) : 0u) | (relu ? NG_FLAG_RELU : 0u);
    // stochastic rounding: seed 0, one stream of random words per call, numbered
    // from 1 in call order (the reference's per-thread state in rand_state,
    // kernels/C_interface/nervana_c_api.h:59-61, is not reproducible)
    static std::atomic<unsigned> call_counter{0};
    const unsigned rng_stream = sr ? call_counter.fetch_add(1u) + 1u : 0u;
    // Shapes that fill the chip only when their contraction is cut into slices
    // (fully connected layers at a minibatch of 128) keep the partial sums in the
    // static array, so this entry runs the same schedule as NervanaGPU.dot.
    int dev = -1;
    const size_t need = (m > 0 && n > 0 && k > 0) ? ng_gemm_workspace_bytes(dtype, a_t, b_t, m, n, k, 1, 1) : 0;
    void* arena = nullptr;
    if (need > 0 && need <= (size_t)NG_GEMM_STATIC_SCRATCH_BYTES && hipGetDevice(&dev) == hipSuccess && dev >= 0 &&
        dev < MAX_DEVICES)
        arena = g_scratch_ptr[dev].load(std::memory_order_acquire);
    const bool sliced = arena != nullptr;
    int rc;
    if (sliced) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        ScratchOrder& ord = g_scratch_order[dev];
        hipError_t e = hipSuccess;
        if (ord.used && ord.last != (hipStream_t)stream) e = hipStreamWaitEvent((hipStream_t)stream, ord.done, 0);
        rc = (e != hipSuccess) ? hip_fail(e, "hipStreamWaitEvent(scratch order)")
                               : ng_gemm(dtype, a_t, b_t, m, n, k, A, lda, B, ldb, C, ldc, alpha, beta, flags,
                                         0u, rng_stream, 1, 0, 0, 0, 1, arena, need, stream);
        if (rc == 0) {
            e = hipEventRecord(ord.done, (hipStream_t)stream);
            if (e != hipSuccess) rc = hip_fail(e, "hipEventRecord(scratch order)");
            ord.last = (hipStream_t)stream;
            ord.used = true;
        }
    } else {
        rc = ng_gemm(dtype, a_t, b_t, m, n, k, A, lda, B, ldb, C, ldc, alpha, beta, flags,
                     0u, rng_stream, 1, 0, 0, 0, 1, nullptr, 0, stream);
    }
    if (rc) fprintf(stderr, "nervana gemm: %s\n", ng_last_error());
    return rc == 0;
}

bool nervana_sgemm(float* A, float* B, float* C, bool a_t, bool b_t, int m, int n, int k,
                   int lda, int ldb, int ldc, float alpha, float beta, unsigned int* /*rand_state*/,
                   bool stochastic_round, bool apply_relu, void* stream, int /*grid*/)
{
    return c_gemm(NG_F32, A, B, C, a_t, b_t, m, n, k, lda, ldb, ldc, alpha, beta, stochastic_round, apply_relu, stream);
}

bool nervana_hgemm(short* A, short* B, short* C, bool a_t, bool b_t, int m, int n, int k,
                   int lda, int ldb, int ldc, float alpha, float beta, unsigned int* /*rand_state*/,
                   bool stochastic_round, bool apply_relu, void* stream, int /*grid*/)
{
    return c_gemm(NG_F16, A, B, C, a_t, b_t, m, n, k, lda, ldb, ldc, alpha, beta, stochastic_round, apply_relu, stream);
}

// column-major C(m,n) = op(A).op(B) is the row-major product C^T(n,m) = op(B)^T.op(A)^T
bool nervana_sgemm_colmajor(float* A, float* B, float* C, bool a_t, bool b_t, int m, int n, int k,
                            int lda, int ldb, int ldc, float alpha, float beta, unsigned int* rand_state,
                            bool stochastic_round, bool apply_relu, void* stream, int grid)
{
    return nervana_sgemm(B, A, C, b_t, a_t, n, m, k, ldb, lda, ldc, alpha, beta, rand_state,
                         stochastic_round, apply_relu, stream, grid);
}

bool nervana_hgemm_colmajor(short* A, short* B, short* C, bool a_t, bool b_t, int m, int n, int k,
                            int lda, int ldb, int ldc, float alpha, float beta, unsigned int* rand_state,
                            bool stochastic_round, bool apply_relu, void* stream, int grid)
{
    return nervana_hgemm(B, A, C, b_t, a_t, n, m, k, ldb, lda, ldc, alpha, beta, rand_state,
                         stochastic_round, apply_relu, stream, grid);
}

}  // extern "C"
