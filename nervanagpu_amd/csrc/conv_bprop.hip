// Convolution data gradient: gradI = round(alpha * conv_transpose(E, F)).
// Replaces {h,s}conv_bprop_{C64_N64,C32_N64} and the dimShuffle / transpose /
// memset launches around them (nervanagpu/nervanagpu.py:652-659, 685-719).
//
// Always the gather form, for every C and stride.  The filter operand is read
// in place (rows c, contraction (tap, k), k contiguous per tap) whenever the
// contraction runs in blocks of output maps; the row-by-row form for few output
// maps first re-lays the filter out into [(tap,k)][C].  Strided layers are decomposed
// into str_d*str_h*str_w stride-1 sub-problems (one per residue class of the
// input pixel), each with only the taps that can reach that class.  When all
// classes together have at most 256 rows (few channels, e.g. a first layer)
// they are stacked into ONE problem: the output-pixel offsets a lattice point
// reads are the same for every class, so the gathered operand is shared and E
// is read once instead of once per class.  No atomics, no zero fill, fp32
// accumulation, one rounding.
#include "conv_plan.h"
#include <cstdlib>
#include "conv_stream_taps.h"

namespace ng {

// filter (C,TRS,K) -> per-class matrices [(tap,k)][Cpad], zero padded in c and
// in k (Kpad rows per tap)
template <typename T>
__global__ void filter_relayout_kernel(const T* F, T* out, const int* tap_dest, int C, int RST, int K, int Kpad, int Cpad)
{
    const long total = (long)RST * Kpad * Cpad;
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
        const int c = (int)(e % Cpad);
        const long r = e / Cpad;
        const int k = (int)(r % Kpad);
        const int trs = (int)(r / Kpad);
        const T v = (c < C && k < K) ? F[((long)c * RST + trs) * K + k] : (T)0;
        out[((long)tap_dest[trs] + k) * Cpad + c] = v;
    }
}

// filter (C,TRS,K) -> merged matrix [(offset,k)][rpad], rows (class, c): the
// tap of class (rz,ry,rx) that reads output offset (dz,dy,dx) is
// (rz + pad_d - dz*str_d, ...); rows whose tap falls outside the filter are zero
template <typename T>
__global__ void filter_merge_kernel(const T* F, T* out, const TapEntry* mtaps, ng_conv_params p, int m_taps,
                                    int m_rows, int m_rpad)
{
    const long total = (long)m_taps * p.K * m_rpad;
    const int RST = p.T * p.R * p.S;
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
        const int row = (int)(e % m_rpad);
        const long r = e / m_rpad;
        const int k = (int)(r % p.K);
        const int mt = (int)(r / p.K);
        T v = (T)0;
        if (row < m_rows) {
            const int cls = row / p.C, c = row - cls * p.C;
            const int rz = cls / (p.str_h * p.str_w), rem = cls - rz * (p.str_h * p.str_w);
            const int ry = rem / p.str_w, rx = rem - ry * p.str_w;
            const TapEntry d = mtaps[mt];
            const int t = rz + p.pad_d - d.dz * p.str_d, rr = ry + p.pad_h - d.dy * p.str_h,
                      ss = rx + p.pad_w - d.dx * p.str_w;
            if ((unsigned)t < (unsigned)p.T && (unsigned)rr < (unsigned)p.R && (unsigned)ss < (unsigned)p.S)
                v = F[((long)c * RST + (t * p.R + rr) * p.S + ss) * p.K + k];
        }
        out[e] = v;
    }
}

template <typename T, bool BLOCKED, int BM, int BN, int BK, int WM, int WN>
static int bprop_merged(const ConvPlan& pl, const T* Fm, const void* E, void* gradI, float alpha, hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    const int ncols = pl.m_nz * pl.m_ny * pl.m_nx * p.N;
    const int MPQN = p.M * p.P * p.Q * p.N;
    const int J = pl.m_taps * p.K;
    const PixelLattice lat = PixelLattice::make(p.N, ncols, pl.m_nx, pl.m_nx * pl.m_ny);
    DenseLoader<T, MC, true> al{Fm, 0, pl.m_rpad, pl.m_rpad, J};
    const int nblk = BLOCKED ? p.K / BK : 1;
    GatherColsLoader<T, T, BLOCKED, BK> bl{(const T*)E, BLOCKED ? pl.d_merged_taps : pl.d_merged_flat, J, lat,
                                           1, 1, 1, p.M, p.P, p.Q, MPQN, FastDiv::make((unsigned)nblk), nblk, p.K, 0,
                                           BLOCKED ? pl.m_taps : 0};
    MergedLatticeStoreEpilogue<T> epi{(T*)gradI, pl.m_rows, p.C, FastDiv::make((unsigned)p.C),
                                      FastDiv::make((unsigned)(p.str_h * p.str_w)), FastDiv::make((unsigned)p.str_w),
                                      (long)p.D * p.H * p.W * p.N, lat, p.str_d, p.str_h, p.str_w, p.D, p.H, p.W, alpha};
    return launch_core<T, BM, BN, BK, WM, WN, MC, MC>(al, bl, epi, pl.m_rows, ncols, cdiv(J, BK), 1, stream,
                                                      "conv bprop (merged)");
}

template <typename T, bool BLOCKED>
static int run_bprop_merged(const ConvPlan& pl, const void* F, const void* E, void* gradI, float alpha, void* ws,
                            hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    T* Fm = (T*)ws;
    const long total = (long)pl.m_taps * p.K * pl.m_rpad;
    const int blocks = (int)std::min<long>((total + 255) / 256, 4096);
    hipLaunchKernelGGL(filter_merge_kernel<T>, dim3(blocks), dim3(256), 0, stream, (const T*)F, Fm,
                       pl.d_merged_taps, p, pl.m_taps, pl.m_rows, pl.m_rpad);
    NG_CHECK_LAUNCH("filter merge");
    if constexpr (sizeof(T) == 2) {
        switch (pick_row_tile(pl.m_rows, pl.m_nz * pl.m_ny * pl.m_nx * p.N, 256)) {
        case 256: return bprop_merged<T, BLOCKED, 256, 256, 64, 2, 4>(pl, Fm, E, gradI, alpha, stream);
        case 128: return bprop_merged<T, BLOCKED, 128, 256, 64, 2, 4>(pl, Fm, E, gradI, alpha, stream);
        default:  return bprop_merged<T, BLOCKED, 64, 256, 64, 1, 4>(pl, Fm, E, gradI, alpha, stream);
        }
    } else {
        return bprop_merged<T, BLOCKED, 128, 128, 16, 2, 2>(pl, Fm, E, gradI, alpha, stream);
    }
}

template <typename T, bool BLOCKED, int BM, int BN, int BK, int WM, int WN, int NSTAGE = 2>
static int bprop_class(const ConvPlan& pl, const BpropClass& c, const void* F, const T* Fs, const void* E, void* gradI,
                       float alpha, const void* mask, hipStream_t stream, int col_begin = 0, int col_end = -1,
                       void* ws = nullptr, size_t ws_bytes = 0)
{
    const ng_conv_params& p = pl.p;
    const int ncols = c.nz * c.ny * c.nx * p.N;
    const int MPQN = p.M * p.P * p.Q * p.N;
    const PixelLattice lat = PixelLattice::make(p.N, ncols, c.nx, c.nx * c.ny);
    const int nblk = BLOCKED ? pl.Kpad / BK : 1;
    GatherColsLoader<T, T, BLOCKED, BK> bl{(const T*)E,
                                           BLOCKED ? pl.d_bprop_taps + c.tap_offset : pl.d_bprop_flat + c.flat_offset,
                                           c.J, lat, 1, 1, 1, p.M, p.P, p.Q,
                                           MPQN, FastDiv::make((unsigned)(BLOCKED ? std::max(c.taps, 1) : nblk)), nblk, p.K,
                                           BLOCKED ? c.taps : 0, BLOCKED ? c.taps : 0};
    const int k_tiles = cdiv(c.J, BK);
    const bool dense = (p.str_d == 1 && p.str_h == 1 && p.str_w == 1);
    ScaleStoreEpilogue<T> depi{(T*)gradI, 0, ncols, p.C, ncols, alpha, 0.0f, 0u, 0u, 0u, 0u, 1u, (const T*)mask};
    LatticeStoreEpilogue<T> lepi{(T*)gradI, p.C, (long)p.D * p.H * p.W * p.N, lat, c.rz, c.ry, c.rx,
                                 p.str_d, p.str_h, p.str_w, p.H, p.W, alpha};
    if constexpr (BLOCKED) {
        // the filter is read in place: rows c, contraction (tap, k)
        FilterRowsLoader<T, BK> al{(const T*)F, pl.d_bprop_trs + c.tap_offset, p.C, p.K, pl.RST * p.K,
                                   FastDiv::make((unsigned)std::max(c.taps, 1)), c.taps};
        // the filter is read in place, so the scratch is free for contraction slices of a small grid
        if (dense && col_begin == 0 && col_end < 0)
            return launch_core_sliced<T, BM, BN, BK, WM, WN, KC, MC, NSTAGE>(al, bl, depi, p.C, ncols, k_tiles, ws, ws_bytes, stream, "conv bprop");
        if (dense) return launch_core<T, BM, BN, BK, WM, WN, KC, MC, NSTAGE>(al, bl, depi, p.C, ncols, k_tiles, 1, stream, "conv bprop", col_begin, col_end);
        return launch_core<T, BM, BN, BK, WM, WN, KC, MC, NSTAGE>(al, bl, lepi, p.C, ncols, k_tiles, 1, stream, "conv bprop", col_begin, col_end);
    } else {
        DenseLoader<T, MC, true> al{Fs + c.w_row * pl.Cpad, 0, pl.Cpad, pl.Cpad, c.J};
        if (dense) return launch_core<T, BM, BN, BK, WM, WN, MC, MC>(al, bl, depi, p.C, ncols, k_tiles, 1, stream, "conv bprop", col_begin, col_end);
        return launch_core<T, BM, BN, BK, WM, WN, MC, MC>(al, bl, lepi, p.C, ncols, k_tiles, 1, stream, "conv bprop", col_begin, col_end);
    }
}

// Unit strides, filter rows of three taps, N = 64 or 128: the taps of a filter row
// share one tile of E (see FilterTapColsLoader); a 256-column tile is four pixels
// (N = 64) or two (N = 128) of one row of the input image.
static bool shares_taps(const ConvPlan& pl)
{
    const ng_conv_params& p = pl.p;
    // 128 images: image rows of an odd number of pixels are padded by one if that wastes
    // at most a twelfth of the columns (the epilogue folds the padding away)
    const bool rows_fit = p.N == 128 ? 12 * (p.W % 2) <= p.W + p.W % 2 : p.W % 4 == 0;
    return p.S == 3 && (p.N == 64 || p.N == 128) && rows_fit && p.K % 32 == 0 &&
           p.str_d == 1 && p.str_h == 1 && p.str_w == 1 && !pl.merged;
}

template <int BM, int WM, int WN, int BN = 256, int COLS = 64, int PX = 4>
static int bprop_shared_taps(const ConvPlan& pl, const void* F, const void* E, void* gradI, float alpha,
                             const void* mask, hipStream_t stream, int col_begin = 0, int col_end = -1)
{
    typedef _Float16 T;
    constexpr int BK = 32, TAPS = 3;
    static_assert(BN == PX * COLS || BN == COLS, "PX pixels per tile, or one (tail launch)");
    const ng_conv_params& p = pl.p;
    const int wpad = cdiv(p.W, PX) * PX;
    const int ncols = p.D * p.H * wpad * p.N;           // the kernel's columns: padded image rows
    const int out_cols = p.D * p.H * p.W * p.N;
    const int TR = p.T * p.R, nblk = cdiv(p.K, BK);
    ScaleStoreEpilogue<T> epi{(T*)gradI, 0, out_cols, p.C, out_cols, alpha, 0.0f, 0u, 0u, 0u, 0u, 1u, (const T*)mask};
    if (wpad != p.W) {
        epi.fold_from = wpad * p.N; epi.fold_to = p.W * p.N;
        epi.fold_div = FastDiv::make((unsigned)epi.fold_from);
    }
    FilterTapColsLoader<T, BK, TAPS> al{(const T*)F, p.C, p.K, pl.RST * p.K, FastDiv::make((unsigned)TR),
                                        FastDiv::make((unsigned)p.R), TR, p.R};
    GatherRowSegLoader<T, BK, TAPS, COLS> bl{(const T*)E, PixelLattice::make(p.N, ncols, wpad, p.H * wpad), p.M, p.P, p.Q,
                                             p.T - 1 - p.pad_d, p.R - 1 - p.pad_h, p.S - 1 - p.pad_w,
                                             p.M * p.P * p.Q * p.N,
                                             FastDiv::make((unsigned)TR), FastDiv::make((unsigned)p.R), TR, p.R, p.K};
    return launch_core<T, BM, BN, BK, WM, WN, KC, MC>(al, bl, epi, p.C, ncols, TR * nblk, 1, stream, "conv bprop (shared taps)",
                                                      col_begin, col_end);
}

// The same layer shape with at most 64 channels and at most 64 output maps, one
// image plane, no rectifier mask: the (mirrored) filter stays in registers and E
// streams (conv_stream_taps.h).  KT = 3 contraction tiles per block of 32 output maps.
template <int KT, int BM = 64, int WM = 2>
static int bprop_stream_taps(const ConvPlan& pl, const void* F, const void* E, void* gradI, float alpha, hipStream_t stream)
{
    typedef _Float16 T;
    constexpr int BK = 32, TAPS = 3, PX = 4;
    const ng_conv_params& p = pl.p;
    const int ncols = p.H * p.W * p.N;
    ScaleStoreEpilogue<T> epi{(T*)gradI, 0, ncols, p.C, ncols, alpha, 0.0f, 0u, 0u, 0u, 0u, 1u};
    FilterTapColsLoader<T, BK, TAPS> al{(const T*)F, p.C, p.K, pl.RST * p.K, FastDiv::make((unsigned)p.R),
                                        FastDiv::make((unsigned)p.R), p.R, p.R};
    RowSegStream<T> bg{(const T*)E, p.P, p.Q, p.R - 1 - p.pad_h, p.S - 1 - p.pad_w, p.P * p.Q * p.N, p.H, p.W,
                       FastDiv::make((unsigned)p.H)};
    launch_stream_taps<T, BM, PX, BK, WM, 4, KT, KC>(al, bg, epi, p.H * (p.W / PX), stream);
    NG_CHECK_LAUNCH("conv bprop (resident filter, shared taps)");
    return 0;
}

static bool streams_shared_taps(const ConvPlan& pl, const void* mask)
{
    const ng_conv_params& p = pl.p;
    return !mask && shares_taps(pl) && p.N == 64 && p.C <= 64 && p.K <= 64 && p.T == 1 && p.R == 3 &&
           p.D == 1 && p.M == 1 && p.W % 4 == 0 && p.H * (p.W / 4) >= 4 * device_cu_count() &&
           (long)p.P * p.Q < (1L << 19) && (long)p.C * p.H * p.W * p.N < (1L << 30);
}

// Very few channels (a first layer): rows (channel, horizontal tap), see
// FilterChannelTapLoader.  Strips of six output pixels from eight pixels of E.
static bool thin_channels(const ConvPlan& pl, const void* mask)
{
    const ng_conv_params& p = pl.p;
    return !mask && 3 * p.C <= 32 && p.S == 3 && p.N == 64 && p.K % 8 == 0 &&
           p.str_d == 1 && p.str_h == 1 && p.str_w == 1;
}

// the same problem on the streaming kernel (stream_core.h): the filter, KT tiles of
// 32 contraction rows, stays in registers; at most five channels (15 parked rows)
template <int KT>
static int bprop_thin_stream(const ConvPlan& pl, const void* F, const void* E, void* gradI, float alpha, hipStream_t stream)
{
    typedef _Float16 T;
    constexpr int BN = 512, BK = 32, OUT_PIX = 6;
    const ng_conv_params& p = pl.p;
    const int strips = cdiv(p.W, OUT_PIX);
    const int tiles = p.D * p.H * strips;
    const int nblk = cdiv(p.K, BK);
    FilterChannelTapLoader<T, BK> al{(const T*)F, 3 * p.C, p.K, pl.RST * p.K, FastDiv::make((unsigned)nblk), nblk};
    HaloStripGather<T, BK, BN, OUT_PIX> bg{(const T*)E, p.M, p.P, p.Q, p.N, p.M * p.P * p.Q * p.N, tiles * BN,
                                           FastDiv::make((unsigned)(p.D * p.H)), FastDiv::make((unsigned)p.H), p.D * p.H, p.H,
                                           p.pad_d, p.pad_h, p.pad_w,
                                           FastDiv::make((unsigned)nblk), FastDiv::make((unsigned)p.R), nblk, p.R, p.K};
    ShiftSumStoreEpilogue<T, BN, OUT_PIX, 16> epi{(T*)gradI, 3 * p.C, (long)p.D * p.H * p.W * p.N, p.W, p.N,
                                                  FastDiv::make((unsigned)(p.D * p.H)), p.D * p.H, alpha};
    launch_stream<T, 32, BN, BK, 4, KT, KC, 2>(al, bg, epi, tiles, 2, stream);
    NG_CHECK_LAUNCH("conv bprop (channel-tap rows, streamed)");
    return 0;
}

static int bprop_thin(const ConvPlan& pl, const void* F, const void* E, void* gradI, float alpha, hipStream_t stream)
{
    typedef _Float16 T;
    constexpr int BN = 512, BK = 32, OUT_PIX = 6;
    const ng_conv_params& p = pl.p;
    const int strips = cdiv(p.W, OUT_PIX);
    const int tiles = p.D * p.H * strips;
    const int TR = p.T * p.R, nblk = cdiv(p.K, BK);
    if (p.C <= 5 && tiles >= device_cu_count()) {
        if (TR * nblk == 3) return bprop_thin_stream<3>(pl, F, E, gradI, alpha, stream);
        if (TR * nblk == 6) return bprop_thin_stream<6>(pl, F, E, gradI, alpha, stream);
    }
    FilterChannelTapLoader<T, BK> al{(const T*)F, 3 * p.C, p.K, pl.RST * p.K, FastDiv::make((unsigned)nblk), nblk};
    HaloStripLoader<T, BK, BN, OUT_PIX> bl{(const T*)E, p.M, p.P, p.Q, p.N, p.M * p.P * p.Q * p.N, tiles * BN,
                                           FastDiv::make((unsigned)(p.D * p.H)), FastDiv::make((unsigned)p.H), p.D * p.H, p.H,
                                           p.pad_d, p.pad_h, p.pad_w,
                                           FastDiv::make((unsigned)nblk), FastDiv::make((unsigned)p.R), nblk, p.R, p.K};
    ShiftSumStoreEpilogue<T, BN, OUT_PIX> epi{(T*)gradI, 3 * p.C, (long)p.D * p.H * p.W * p.N, p.W, p.N,
                                              FastDiv::make((unsigned)(p.D * p.H)), p.D * p.H, alpha};
    return launch_core<T, 32, BN, BK, 1, 2, KC, MC>(al, bl, epi, 3 * p.C, tiles * BN, TR * nblk, 1, stream,
                                                    "conv bprop (channel-tap rows)");
}

template <bool BLOCKED>
static int bprop_class_h(const ConvPlan& pl, const BpropClass& c, const void* F, const _Float16* Fs, const void* E,
                         void* gradI, float alpha, const void* mask, hipStream_t st, void* ws, size_t ws_bytes)
{
    const int ncols = c.nz * c.ny * c.nx * pl.p.N;
    const int row_tile = pick_row_tile(pl.p.C, ncols, 256);
    if constexpr (BLOCKED) {
        // 128 rows and more 256-column tiles than CUs: 512-column tiles, 64 x 128 per wavefront (the
        // fragment traffic of the 256 x 256 tile; Overfeat conv2, 96 channels from 256 maps, 5x5: 0.191 -> 0.154 ms)
        if (row_tile == 128 && (long)cdiv(pl.p.C, 128) * cdiv(ncols, 256) > device_cu_count())
            return bprop_class<_Float16, BLOCKED, 128, 512, 64, 2, 4>(pl, c, F, Fs, E, gradI, alpha, mask, st, 0, -1, ws, ws_bytes);
    }
    if constexpr (BLOCKED) {
        // trailing column tiles beyond whole rounds: 64x64 tiles behind the main launch
        const int tail = row_tile >= 128 ? tail_column_tiles(cdiv(pl.p.C, row_tile), cdiv(ncols, 256)) : 0;
        if (tail) {
            const int cut = (cdiv(ncols, 256) - tail) * 256;
            const int rc = row_tile == 256 ? bprop_class<_Float16, BLOCKED, 256, 256, 64, 2, 4>(pl, c, F, Fs, E, gradI, alpha, mask, st, 0, cut)
                                           : bprop_class<_Float16, BLOCKED, 128, 256, 64, 2, 4>(pl, c, F, Fs, E, gradI, alpha, mask, st, 0, cut);
            return rc ? rc : bprop_class<_Float16, BLOCKED, 64, 64, 64, 2, 2>(pl, c, F, Fs, E, gradI, alpha, mask, st, cut, -1);
        }
    }
    if constexpr (BLOCKED) {
        // A candidate that has not been measured on a device yet (conv_stage_switch): a grid of at most one
        // workgroup per CU has nobody to cover the wait for a tile requested one tile step ahead; a third
        // stage (144 KB) gives the request two steps
        if (conv_stage_switch() >= 3 && row_tile == 128 && (long)cdiv(pl.p.C, 128) * cdiv(ncols, 256) <= device_cu_count())
            return bprop_class<_Float16, BLOCKED, 128, 256, 64, 2, 4, 3>(pl, c, F, Fs, E, gradI, alpha, mask, st, 0, -1, ws, ws_bytes);
    }
    switch (row_tile) {
    case 256: return bprop_class<_Float16, BLOCKED, 256, 256, 64, 2, 4>(pl, c, F, Fs, E, gradI, alpha, mask, st, 0, -1, ws, ws_bytes);
    case 128: return bprop_class<_Float16, BLOCKED, 128, 256, 64, 2, 4>(pl, c, F, Fs, E, gradI, alpha, mask, st, 0, -1, ws, ws_bytes);
    default:  return bprop_class<_Float16, BLOCKED, 64, 256, 64, 1, 4>(pl, c, F, Fs, E, gradI, alpha, mask, st, 0, -1, ws, ws_bytes);
    }
}

template <typename T>
static int run_bprop(const ConvPlan& pl, const void* F, const void* E, void* gradI, float alpha, const void* mask,
                     void* ws, size_t ws_bytes, hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    // the mask shares the plain store epilogue's indexing: unit strides only
    if (mask && (pl.merged || p.str_d != 1 || p.str_h != 1 || p.str_w != 1))
        return fail(-51, "ng_conv_bprop: the rectifier mask needs unit strides");
    // A misaligned workspace is never used.  The re-laid-out filter needs one (merged classes, and the
    // row-by-row kernels of layers with few output maps); the kernels that read the filter in place
    // do not, and run without: the requirement is checked where the filter is re-laid out.
    if ((uintptr_t)ws & 15) { ws = nullptr; ws_bytes = 0; }
    auto require_filter_scratch = [&]() -> int {
        if (pl.ws_bprop && (ws_bytes < pl.ws_bprop || !ws))
            return fail(-40, "ng_conv_bprop: workspace too small (%zu < %zu)", ws_bytes, pl.ws_bprop);
        return 0;
    };
    if (pl.merged) {
        if (int rc = require_filter_scratch()) return rc;
        return (p.K % pl.bk == 0) ? run_bprop_merged<T, true>(pl, F, E, gradI, alpha, ws, stream)
                                  : run_bprop_merged<T, false>(pl, F, E, gradI, alpha, ws, stream);
    }
    const bool blocked = pl.bprop_blocked;
    if constexpr (sizeof(T) == 2) {
        // at most 32 channels (a first layer among them): one block of 32 rows on four wavefronts
        // (VGG conv1.1: 0.141 ms against 0.226 with rows (channel, tap) on halo strips)
        if (streams_shared_taps(pl, mask) && p.C <= 32)
            return p.K == 64 ? bprop_stream_taps<6, 32, 1>(pl, F, E, gradI, alpha, stream) : bprop_stream_taps<3, 32, 1>(pl, F, E, gradI, alpha, stream);
        if (thin_channels(pl, mask)) return bprop_thin(pl, F, E, gradI, alpha, stream);
        if (shares_taps(pl) && p.N == 128) {
            // padded image rows can cost a round over the chip more than the separate taps need
            double cost, cost_plain;
            const int row_tile = pick_row_tile(p.C, p.D * p.H * cdiv(p.W, 2) * 2 * p.N, 256, &cost);
            const int plain_tile = pick_row_tile(p.C, p.D * p.H * p.W * p.N, 256, &cost_plain);
            const bool three_stages = conv_stage_switch() == 4 && plain_tile == 128 && blocked &&
                                      (long)cdiv(p.C, 128) * cdiv(p.D * p.H * p.W * p.N, 256) <= device_cu_count();
            if (cost <= cost_plain && row_tile >= 128 && !three_stages) {
                const int ncols = p.D * p.H * cdiv(p.W, 2) * 2 * p.N;
                const int tail = tail_column_tiles(cdiv(p.C, row_tile), cdiv(ncols, 256));
                const int cut = tail ? (cdiv(ncols, 256) - tail) * 256 : -1;
                const int rc = row_tile == 256 ? bprop_shared_taps<256, 2, 4, 256, 128, 2>(pl, F, E, gradI, alpha, mask, stream, 0, cut)
                                               : bprop_shared_taps<128, 2, 4, 256, 128, 2>(pl, F, E, gradI, alpha, mask, stream, 0, cut);
                if (rc || !tail) return rc;
                return bprop_shared_taps<64, 2, 2, 128, 128, 2>(pl, F, E, gradI, alpha, mask, stream, cut, -1);
            }
        } else if (streams_shared_taps(pl, mask)) {
            return p.K == 64 ? bprop_stream_taps<6>(pl, F, E, gradI, alpha, stream) : bprop_stream_taps<3>(pl, F, E, gradI, alpha, stream);
        } else if (shares_taps(pl)) {
            const int ncols = p.D * p.H * p.W * p.N;
            const int row_tile = pick_row_tile(p.C, ncols, 256);
            // trailing column tiles beyond whole rounds: 64x64 tiles behind the main launch
            // 128 rows over a round and a half or more of 512-column tiles: eight pixels per tile
            if (row_tile == 128 && p.W % 8 == 0 && 2 * cdiv(ncols, 512) >= 3 * device_cu_count()) {
                const int t512 = cdiv(ncols, 512);
                const int wtail = tail_column_tiles(cdiv(p.C, 128), t512);
                const int wcut = wtail ? (t512 - wtail) * 512 : -1;
                const int rc = bprop_shared_taps<128, 2, 4, 512, 64, 8>(pl, F, E, gradI, alpha, mask, stream, 0, wcut);
                if (rc || !wtail) return rc;
                return bprop_shared_taps<64, 2, 2, 64>(pl, F, E, gradI, alpha, mask, stream, wcut, -1);
            }
            const int tail = row_tile >= 128 ? tail_column_tiles(cdiv(p.C, row_tile), cdiv(ncols, 256)) : 0;
            if (tail) {
                const int cut = (cdiv(ncols, 256) - tail) * 256;
                const int rc = row_tile == 256 ? bprop_shared_taps<256, 2, 4>(pl, F, E, gradI, alpha, mask, stream, 0, cut)
                                               : bprop_shared_taps<128, 2, 4>(pl, F, E, gradI, alpha, mask, stream, 0, cut);
                return rc ? rc : bprop_shared_taps<64, 2, 2, 64>(pl, F, E, gradI, alpha, mask, stream, cut, -1);
            }
            switch (row_tile) {
            case 256: return bprop_shared_taps<256, 2, 4>(pl, F, E, gradI, alpha, mask, stream);
            case 128: return bprop_shared_taps<128, 2, 4>(pl, F, E, gradI, alpha, mask, stream);
            default:  return bprop_shared_taps<64, 1, 4>(pl, F, E, gradI, alpha, mask, stream);
            }
        }
    }
    // the row-by-row kernels of a layer whose output maps do not fill contraction blocks read the
    // filter as [(tap, k)][C] from scratch
    T* Fs = (T*)ws;
    if (!blocked) {
        if (int rc = require_filter_scratch()) return rc;
        const long total = (long)pl.RST * pl.Kpad * pl.Cpad;
        const int blocks = (int)std::min<long>((total + 255) / 256, 4096);
        hipLaunchKernelGGL(filter_relayout_kernel<T>, dim3(blocks), dim3(256), 0, stream,
                           (const T*)F, Fs, pl.d_tap_dest, p.C, pl.RST, p.K, pl.Kpad, pl.Cpad);
        NG_CHECK_LAUNCH("filter relayout");
    }
    for (const BpropClass& c : pl.classes) {
        if (c.nz * c.ny * c.nx == 0) continue;
        int rc;
        if (sizeof(T) == 2)
            rc = blocked ? bprop_class_h<true>(pl, c, F, (const _Float16*)Fs, E, gradI, alpha, mask, stream, ws, ws_bytes)
                         : bprop_class_h<false>(pl, c, F, (const _Float16*)Fs, E, gradI, alpha, mask, stream, nullptr, 0);
        else
            rc = blocked ? bprop_class<float, true, 128, 128, 16, 2, 2>(pl, c, F, (const float*)Fs, E, gradI, alpha, mask, stream, 0, -1, ws, ws_bytes)
                         : bprop_class<float, false, 128, 128, 16, 2, 2>(pl, c, F, (const float*)Fs, E, gradI, alpha, mask, stream);
        if (rc) return rc;
    }
    return 0;
}

}  // namespace ng

using namespace ng;

extern "C" int ng_conv_bprop(const void* plan, const void* F, const void* E, void* gradI, float alpha,
                             const void* relu_mask, void* workspace, size_t workspace_bytes, void* stream)
{
    const ConvPlan* pl = (const ConvPlan*)plan;
    if (!pl) return fail(-48, "conv: null plan");
    int rc;
    if ((rc = check_ptr16(F, "F")) || (rc = check_ptr16(E, "E")) || (rc = check_ptr16(gradI, "grad_I")) ||
        (relu_mask && (rc = check_ptr16(relu_mask, "relu_mask"))))
        return rc;
    hipStream_t st = (hipStream_t)stream;
    if (pl->pointwise && !relu_mask) {
        // gradI (C x columns) = F (C x K) * E (K x columns)
        const ng_conv_params& p = pl->p;
        const int cols = p.M * p.P * p.Q * p.N;
        const bool ws_ok = ((uintptr_t)workspace & 15) == 0;
        return ng_gemm(pl->dtype, 0, 0, p.C, cols, p.K, F, p.K, E, cols, gradI, cols, alpha, 0.0f, 0u, 0u, 0u,
                       1, 0, 0, 0, 1, ws_ok ? workspace : nullptr, ws_ok ? workspace_bytes : 0, stream);
    }
    if (pl->dtype == NG_F16) return run_bprop<_Float16>(*pl, F, E, gradI, alpha, relu_mask, workspace, workspace_bytes, st);
    return run_bprop<float>(*pl, F, E, gradI, alpha, relu_mask, workspace, workspace_bytes, st);
}
