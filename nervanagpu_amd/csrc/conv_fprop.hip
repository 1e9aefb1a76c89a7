// Convolution forward: O = round(relu?(alpha * conv(I, F))).  Replaces
// {h,s}conv_fprop_K64_N64 (nervanagpu/nervanagpu.py:642-650, 671-734).
#include "conv_plan.h"
#include "conv_stream_taps.h"

#include <cstdlib>

namespace ng {

template <typename T, typename TIN, bool BLOCKED, int BM, int BN, int BK, int WM, int WN, int NSTAGE = 2>
static int fprop_tile(const ConvPlan& pl, const void* I, const void* F, void* O, float alpha, unsigned flags,
                      hipStream_t stream, int col_begin = 0, int col_end = -1, void* ws = nullptr, size_t ws_bytes = 0)
{
    const bool whole = col_begin == 0 && col_end < 0;     // a launch over all columns may slice its contraction
    const ng_conv_params& p = pl.p;
    const int ncols = p.M * p.P * p.Q * p.N;
    const int DHWN = p.D * p.H * p.W * p.N;
    ScaleStoreEpilogue<T> epi{(T*)O, 0, ncols, p.K, ncols, alpha, 0.0f,
                              (flags & NG_FLAG_RELU) ? 1u : 0u, 0u, 0u, 0u, 1u};
    const PixelLattice lat = PixelLattice::make(p.N, ncols, p.Q, p.P * p.Q);
    if (BLOCKED) {
        const int nblk = cdiv(p.C, BK);
        FilterBlockLoader<T, BK> al{(const T*)F, p.K, pl.RST * p.K, FastDiv::make((unsigned)pl.RST), pl.RST, p.C};
        GatherColsLoader<T, TIN, true, BK> bl{(const TIN*)I, pl.d_fprop_taps, pl.CRST, lat,
                                              p.str_d, p.str_h, p.str_w, p.D, p.H, p.W,
                                              DHWN, FastDiv::make((unsigned)pl.RST), nblk, p.C, pl.RST, pl.RST};
        if (whole) return launch_core_sliced<T, BM, BN, BK, WM, WN, MC, MC, NSTAGE>(al, bl, epi, p.K, ncols, pl.RST * nblk, ws, ws_bytes, stream, "conv fprop");
        return launch_core<T, BM, BN, BK, WM, WN, MC, MC, NSTAGE>(al, bl, epi, p.K, ncols, pl.RST * nblk, 1, stream, "conv fprop",
                                                                  col_begin, col_end);
    } else {
        DenseLoader<T, MC, true> al{(const T*)F, 0, p.K, p.K, pl.CRST};
        GatherColsLoader<T, TIN, false, BK> bl{(const TIN*)I, pl.d_fprop_flat, pl.CRST, lat,
                                               p.str_d, p.str_h, p.str_w, p.D, p.H, p.W,
                                               0, FastDiv{0, 0}, 1, 0, 0};
        if (whole) return launch_core_sliced<T, BM, BN, BK, WM, WN, MC, MC, NSTAGE>(al, bl, epi, p.K, ncols, cdiv(pl.CRST, BK), ws, ws_bytes, stream, "conv fprop");
        return launch_core<T, BM, BN, BK, WM, WN, MC, MC, NSTAGE>(al, bl, epi, p.K, ncols, cdiv(pl.CRST, BK), 1, stream, "conv fprop",
                                                                  col_begin, col_end);
    }
}

// Filter rows of three taps on unit strides share their activation tile (see
// GatherRowSegLoader): a 256-column tile is four output pixels of one image row
// for N = 64 images (two for N = 128; N = 32 runs 128-column tiles of four), and
// the shared tile is two input pixels wider.
static int tap_share_pixels(int N) { return N == 128 ? 2 : 4; }

static bool shares_taps(const ConvPlan& pl)
{
    const ng_conv_params& p = pl.p;
    // image rows that are not a whole number of tiles are padded to one if that
    // wastes at most a twelfth of the columns (the epilogue folds them away)
    const int px = tap_share_pixels(p.N);
    const int qpad = cdiv(p.Q, px) * px;
    return p.S == 3 && (p.N == 64 || p.N == 32 || p.N == 128) && 12 * (qpad - p.Q) <= qpad && p.C % 32 == 0 &&
           p.str_d == 1 && p.str_h == 1 && p.str_w == 1;
}

// COLS = N images per pixel; a tile of BN columns is BN / COLS output pixels of one
// image row (PX of them, or one for the narrow tiles of a tail launch); the image
// rows are padded to a multiple of PX pixels
template <int BM, int WM, int WN, int BN = 256, int COLS = 64, int PX = 4>
static int fprop_shared_taps(const ConvPlan& pl, const void* I, const void* F, void* O, float alpha, unsigned flags,
                             hipStream_t stream, int col_begin = 0, int col_end = -1)
{
    typedef _Float16 T;
    constexpr int BK = 32, TAPS = 3;
    static_assert(BN == PX * COLS || BN == COLS, "PX output pixels per tile, or one");
    const ng_conv_params& p = pl.p;
    const int qpad = cdiv(p.Q, PX) * PX;
    const int ncols = p.M * p.P * qpad * p.N;           // the kernel's columns: padded image rows
    const int out_cols = p.M * p.P * p.Q * p.N;
    const int TR = p.T * p.R, nblk = cdiv(p.C, BK);
    ScaleStoreEpilogue<T> epi{(T*)O, 0, out_cols, p.K, out_cols, alpha, 0.0f, (flags & NG_FLAG_RELU) ? 1u : 0u, 0u, 0u, 0u, 1u};
    if (qpad != p.Q) {
        epi.fold_from = qpad * p.N; epi.fold_to = p.Q * p.N;
        epi.fold_div = FastDiv::make((unsigned)epi.fold_from);
    }
    FilterTapRowLoader<T, BK, TAPS> al{(const T*)F, p.K, pl.RST * p.K, FastDiv::make((unsigned)TR), TR, p.C};
    GatherRowSegLoader<T, BK, TAPS, COLS> bl{(const T*)I, PixelLattice::make(p.N, ncols, qpad, p.P * qpad), p.D, p.H, p.W,
                                             p.pad_d, p.pad_h, p.pad_w, p.D * p.H * p.W * p.N,
                                             FastDiv::make((unsigned)TR), FastDiv::make((unsigned)p.R), TR, p.R, p.C};
    return launch_core<T, BM, BN, BK, WM, WN, MC, MC>(al, bl, epi, p.K, ncols, TR * nblk, 1, stream, "conv fprop (shared taps)",
                                                      col_begin, col_end);
}

// A filter of at most 64 output maps and 128 contraction rows (a first layer on
// fp16 images) stays in registers while the output columns stream past (see
// stream_core.h): KT contraction tiles of 32 rows.
template <int KT>
static int fprop_stream(const ConvPlan& pl, const void* I, const void* F, void* O, float alpha, unsigned flags,
                        hipStream_t stream)
{
    typedef _Float16 T;
    constexpr int BN = 256, BK = 32;
    const ng_conv_params& p = pl.p;
    const int ncols = p.M * p.P * p.Q * p.N;
    ScaleStoreEpilogue<T> epi{(T*)O, 0, ncols, p.K, ncols, alpha, 0.0f, (flags & NG_FLAG_RELU) ? 1u : 0u, 0u, 0u, 0u, 1u};
    DenseLoader<T, MC, true> al{(const T*)F, 0, p.K, p.K, pl.CRST};
    FlatTapGather<T> bg{(const T*)I, pl.d_fprop_flat, pl.CRST, PixelLattice::make(p.N, ncols, p.Q, p.P * p.Q),
                        p.str_d, p.str_h, p.str_w, p.D, p.H, p.W};
    // two stages and two workgroups per CU (67 KB of LDS each) beat one workgroup
    // with a deeper ring: 0.097 against 0.115 ms on VGG conv1.1
    launch_stream<T, 64, BN, BK, 4, KT, MC, 2>(al, bg, epi, cdiv(ncols, BN), 2, stream);
    NG_CHECK_LAUNCH("conv fprop (streamed columns)");
    return 0;
}

// First layers with large filters (7x7, 11x11 on a few channels): KT contraction tiles of 16 rows,
// all held in registers as MFMA fragments while tiles of 512 output columns stream (see
// TapDecodeGather).  16-deep tiles keep the padding of the last tile small (363 rows: 23 tiles).
template <int KT>
static int fprop_stream_rows(const ConvPlan& pl, const void* I, const void* F, void* O, float alpha, unsigned flags,
                             hipStream_t stream)
{
    typedef _Float16 T;
    constexpr int BN = 512, BK = 16;
    const ng_conv_params& p = pl.p;
    const int ncols = p.M * p.P * p.Q * p.N;
    ScaleStoreEpilogue<T> epi{(T*)O, 0, ncols, p.K, ncols, alpha, 0.0f, (flags & NG_FLAG_RELU) ? 1u : 0u, 0u, 0u, 0u, 1u};
    DenseLoader<T, MC, true> al{(const T*)F, 0, p.K, p.K, pl.CRST};
    TapDecodeGather<T> bg{(const T*)I, pl.CRST, PixelLattice::make(p.N, ncols, p.Q, p.P * p.Q), p.str_d, p.str_h, p.str_w,
                          p.pad_d, p.pad_h, p.pad_w, p.D, p.H, p.W, p.T, p.R, p.S,
                          FastDiv::make((unsigned)p.S), FastDiv::make((unsigned)p.R), FastDiv::make((unsigned)p.T)};
    // a ring of four stages of 16 KB and the epilogue staging of four wavefronts: one workgroup per CU
    launch_stream<T, 64, BN, BK, 4, KT, MC, 4>(al, bg, epi, cdiv(ncols, BN), 1, stream);
    NG_CHECK_LAUNCH("conv fprop (streamed columns, decoded taps)");
    return 0;
}

// contraction tiles of the kernel above for this layer (0: it does not apply): 129 to 384
// contraction rows (fewer run with a table entry per row), at most 64 output maps
static int streams_decoded_taps(const ConvPlan& pl)
{
    const ng_conv_params& p = pl.p;
    if (pl.fprop_blocked || p.K > 64 || p.K % 8 || p.N % 8 || pl.CRST <= 128 || pl.CRST > 384) return 0;
    if ((long)p.M * p.P * p.Q * p.N < 512L * device_cu_count()) return 0;     // a column tile per CU or more
    if ((long)p.C * p.D * p.H * p.W * p.N >= (1L << 30) || (long)p.K * p.M * p.P * p.Q * p.N >= (1L << 30)) return 0;
    return cdiv(pl.CRST, 16);
}

// Three filter rows of three taps over at most 64 channels, at most 64 output maps,
// 64 images, one image plane: the filter stays in registers and the taps of a
// filter row share the streamed activation tile (conv_stream_taps.h).  KT = 3
// contraction tiles (filter rows) per block of 32 channels.
template <int KT>
static int fprop_stream_taps(const ConvPlan& pl, const void* I, const void* F, void* O, float alpha, unsigned flags,
                             hipStream_t stream)
{
    typedef _Float16 T;
    constexpr int BK = 32, TAPS = 3, PX = 4;
    const ng_conv_params& p = pl.p;
    const int ncols = p.P * p.Q * p.N;
    ScaleStoreEpilogue<T> epi{(T*)O, 0, ncols, p.K, ncols, alpha, 0.0f, (flags & NG_FLAG_RELU) ? 1u : 0u, 0u, 0u, 0u, 1u};
    FilterTapRowLoader<T, BK, TAPS> al{(const T*)F, p.K, pl.RST * p.K, FastDiv::make((unsigned)p.R), p.R, p.C};
    RowSegStream<T> bg{(const T*)I, p.H, p.W, p.pad_h, p.pad_w, p.H * p.W * p.N, p.P, p.Q, FastDiv::make((unsigned)p.P)};
    launch_stream_taps<T, 64, PX, BK, 2, 4, KT, MC>(al, bg, epi, p.P * (p.Q / PX), stream);
    NG_CHECK_LAUNCH("conv fprop (resident filter, shared taps)");
    return 0;
}

static bool streams_shared_taps(const ConvPlan& pl)
{
    const ng_conv_params& p = pl.p;
    return shares_taps(pl) && p.N == 64 && p.K <= 64 && p.K % 8 == 0 && p.C <= 64 && p.T == 1 && p.R == 3 &&
           p.D == 1 && p.M == 1 && p.Q % 4 == 0 && p.P * (p.Q / 4) >= 4 * device_cu_count() &&
           (long)p.H * p.W < (1L << 19) && (long)p.K * p.P * p.Q * p.N < (1L << 30);
}

static bool streams_columns(const ConvPlan& pl)
{
    const ng_conv_params& p = pl.p;
    return !pl.fprop_blocked && p.K <= 64 && p.K % 8 == 0 && pl.CRST <= 128 && p.N % 8 == 0 &&
           (long)p.M * p.P * p.Q * p.N >= 64L * 1024;   // a column tile per CU or more
}

template <typename TIN, bool BLOCKED>
static int fprop_h(const ConvPlan& pl, const void* I, const void* F, void* O, float alpha, unsigned flags, hipStream_t st,
                   void* ws, size_t ws_bytes)
{
    if constexpr (std::is_same<TIN, _Float16>::value) {
        // whichever way the plan would read the filter otherwise
        if (streams_shared_taps(pl))
            return pl.p.C == 64 ? fprop_stream_taps<6>(pl, I, F, O, alpha, flags, st) : fprop_stream_taps<3>(pl, I, F, O, alpha, flags, st);
    }
    if constexpr (BLOCKED && std::is_same<TIN, _Float16>::value) {
        if (shares_taps(pl) && pl.p.N == 32) {
            // 32 images: 128-column tiles; 128 rows on four wavefronts
            if (pl.p.K >= 128) return fprop_shared_taps<128, 2, 2, 128, 32>(pl, I, F, O, alpha, flags, st);
        } else if (shares_taps(pl) && pl.p.N == 128) {
            // 128 images: two output pixels per tile, the shared tile is four wide
            const int ncols = pl.p.M * pl.p.P * cdiv(pl.p.Q, 2) * 2 * pl.p.N;
            // padded image rows can push the grid into one more round over the chip
            // than the unpadded columns of the separate taps need: not worth it then
            double cost, cost_plain;
            const int row_tile = pick_row_tile(pl.p.K, ncols, 256, &cost);
            const int plain_cols = pl.p.M * pl.p.P * pl.p.Q * pl.p.N;
            const int plain_tile = pick_row_tile(pl.p.K, plain_cols, 256, &cost_plain);
            const bool three_stages = conv_stage_switch() == 4 && plain_tile == 128 &&
                                      (long)cdiv(pl.p.K, 128) * cdiv(plain_cols, 256) <= device_cu_count();
            if (cost <= cost_plain && row_tile >= 128 && !three_stages) {
                // trailing column tiles beyond whole rounds: 64-row tiles of one pixel behind the main launch
                const int tail = tail_column_tiles(cdiv(pl.p.K, row_tile), cdiv(ncols, 256));
                const int cut = tail ? (cdiv(ncols, 256) - tail) * 256 : -1;
                const int rc = row_tile == 256 ? fprop_shared_taps<256, 2, 4, 256, 128, 2>(pl, I, F, O, alpha, flags, st, 0, cut)
                                               : fprop_shared_taps<128, 2, 4, 256, 128, 2>(pl, I, F, O, alpha, flags, st, 0, cut);
                if (rc || !tail) return rc;
                return fprop_shared_taps<64, 2, 2, 128, 128, 2>(pl, I, F, O, alpha, flags, st, cut, -1);
            }
        } else if (shares_taps(pl)) {
            const int ncols = pl.p.M * pl.p.P * cdiv(pl.p.Q, 4) * 4 * pl.p.N;
            const int row_tile = pick_row_tile(pl.p.K, ncols, 256);
            // the few column tiles beyond whole rounds of one-per-CU workgroups run
            // behind the main launch as 64x64 tiles, which cover the chip at once
            // 128 rows over a round and a half or more of 512-column tiles: eight pixels per tile (the
            // shared segment is ten wide instead of twice six) and 64 x 128 per wavefront, the
            // fragment traffic of the 256 x 256 tile (VGG conv2.2 forward 0.271 -> 0.232 ms)
            if (row_tile == 128 && pl.p.Q % 8 == 0 && 2 * cdiv(ncols, 512) >= 3 * device_cu_count()) {
                const int t512 = cdiv(ncols, 512);
                const int wtail = tail_column_tiles(cdiv(pl.p.K, 128), t512);
                const int wcut = wtail ? (t512 - wtail) * 512 : -1;
                const int rc = fprop_shared_taps<128, 2, 4, 512, 64, 8>(pl, I, F, O, alpha, flags, st, 0, wcut);
                if (rc || !wtail) return rc;
                return fprop_shared_taps<64, 2, 2, 64, 64>(pl, I, F, O, alpha, flags, st, wcut, -1);
            }
            const int tail = row_tile >= 128 ? tail_column_tiles(cdiv(pl.p.K, row_tile), cdiv(ncols, 256)) : 0;
            if (tail) {
                const int cut = (cdiv(ncols, 256) - tail) * 256;
                const int rc = row_tile == 256 ? fprop_shared_taps<256, 2, 4>(pl, I, F, O, alpha, flags, st, 0, cut)
                                               : fprop_shared_taps<128, 2, 4>(pl, I, F, O, alpha, flags, st, 0, cut);
                return rc ? rc : fprop_shared_taps<64, 2, 2, 64, 64>(pl, I, F, O, alpha, flags, st, cut, -1);
            }
            switch (row_tile) {
            case 256: return fprop_shared_taps<256, 2, 4>(pl, I, F, O, alpha, flags, st);
            case 128: return fprop_shared_taps<128, 2, 4>(pl, I, F, O, alpha, flags, st);
            default:  return fprop_shared_taps<64, 1, 4>(pl, I, F, O, alpha, flags, st);
            }
        }
    }
    if constexpr (!BLOCKED && std::is_same<TIN, _Float16>::value) {
        // A candidate that has passed the CPU emulation but has not been measured on a device yet: off unless
        // NG_CONV_ROWS=1 (read once per process); it becomes the default, or goes, with its first measurement
        static const int tap_rows_on = getenv("NG_CONV_ROWS") ? atoi(getenv("NG_CONV_ROWS")) : 0;
        if (tap_rows_on) {
            // the kernel is compiled for the tile counts of the usual first layers: 7x7 on three
            // channels (147 rows: 10 tiles), 11x11 on three channels (363 rows: 23 tiles); other
            // counts run the next larger one with empty tiles
            const int kt = streams_decoded_taps(pl);
            if (kt > 0 && kt <= 10) return fprop_stream_rows<10>(pl, I, F, O, alpha, flags, st);
            if (kt > 10 && kt <= 16) return fprop_stream_rows<16>(pl, I, F, O, alpha, flags, st);
            if (kt > 16 && kt <= 24) return fprop_stream_rows<24>(pl, I, F, O, alpha, flags, st);
        }
        if (streams_columns(pl)) {
            switch (cdiv(pl.CRST, 32)) {
            case 1: return fprop_stream<1>(pl, I, F, O, alpha, flags, st);
            case 2: return fprop_stream<2>(pl, I, F, O, alpha, flags, st);
            case 3: return fprop_stream<3>(pl, I, F, O, alpha, flags, st);
            default: return fprop_stream<4>(pl, I, F, O, alpha, flags, st);
            }
        }
    }
    const int ncols = pl.p.M * pl.p.P * pl.p.Q * pl.p.N;
    double row_cost;
    const int row_tile = pick_row_tile(pl.p.K, ncols, 256, &row_cost);
    if constexpr (BLOCKED && std::is_same<TIN, _Float16>::value) {
        // output maps in multiples of 192 (AlexNet conv2): 192-row tiles, three row blocks per
        // wavefront, leave no padding rows; the step is priced between the 128- and 256-row ones
        // (64 -> 192 maps, 5x5 on 27x27, N = 128: 0.086 -> 0.074 ms)
        if (pl.p.K % 192 == 0) {
            const long blocks = (long)(pl.p.K / 192) * cdiv(ncols, 256);
            const int cus = device_cu_count();
            if ((double)((blocks + cus - 1) / cus) * 1.5 < row_cost * 0.95)
                return fprop_tile<_Float16, TIN, BLOCKED, 192, 256, 64, 2, 4>(pl, I, F, O, alpha, flags, st, 0, -1, ws, ws_bytes);
        }
    }
    if constexpr (BLOCKED && std::is_same<TIN, _Float16>::value) {
        // 128 rows and more 256-column tiles than CUs: 512-column tiles, 64 x 128 per wavefront
        if (row_tile == 128 && (long)cdiv(pl.p.K, 128) * cdiv(ncols, 256) > device_cu_count())
            return fprop_tile<_Float16, TIN, BLOCKED, 128, 512, 64, 2, 4>(pl, I, F, O, alpha, flags, st, 0, -1, ws, ws_bytes);
    }
    if constexpr (BLOCKED && std::is_same<TIN, _Float16>::value) {
        // as with the shared taps: the few column tiles beyond whole rounds of one-per-CU
        // workgroups run behind the main launch as 64x64 tiles
        const int tail = row_tile >= 128 ? tail_column_tiles(cdiv(pl.p.K, row_tile), cdiv(ncols, 256)) : 0;
        if (tail) {
            const int cut = (cdiv(ncols, 256) - tail) * 256;
            const int rc = row_tile == 256 ? fprop_tile<_Float16, TIN, BLOCKED, 256, 256, 64, 2, 4>(pl, I, F, O, alpha, flags, st, 0, cut)
                                           : fprop_tile<_Float16, TIN, BLOCKED, 128, 256, 64, 2, 4>(pl, I, F, O, alpha, flags, st, 0, cut);
            return rc ? rc : fprop_tile<_Float16, TIN, BLOCKED, 64, 64, 64, 2, 2>(pl, I, F, O, alpha, flags, st, cut, -1);
        }
    }
    if constexpr (BLOCKED && std::is_same<TIN, _Float16>::value) {
        // A candidate that has not been measured on a device yet (conv_stage_switch): a grid of at most one
        // workgroup per CU has nobody to cover the wait for a tile requested one tile step ahead; a third
        // stage (144 KB) gives the request two steps
        if (conv_stage_switch() >= 3 && row_tile == 128 && (long)cdiv(pl.p.K, 128) * cdiv(ncols, 256) <= device_cu_count())
            return fprop_tile<_Float16, TIN, BLOCKED, 128, 256, 64, 2, 4, 3>(pl, I, F, O, alpha, flags, st, 0, -1, ws, ws_bytes);
    }
    switch (row_tile) {
    case 256: return fprop_tile<_Float16, TIN, BLOCKED, 256, 256, 64, 2, 4>(pl, I, F, O, alpha, flags, st, 0, -1, ws, ws_bytes);
    // 128 rows on eight wavefronts: mid-sized layers run about one workgroup per
    // CU, and twice the wavefronts hide the LDS and request latency of a tile
    case 128: return fprop_tile<_Float16, TIN, BLOCKED, 128, 256, 64, 2, 4>(pl, I, F, O, alpha, flags, st, 0, -1, ws, ws_bytes);
    default:
        // Row-by-row gathered contractions (first layers, few channels) are bound
        // by request latency, not by the matrix pipe: half-depth tiles halve the
        // LDS footprint, so twice as many workgroups per CU keep requests in flight
        if (!BLOCKED) return fprop_tile<_Float16, TIN, BLOCKED, 64, 256, 32, 1, 4>(pl, I, F, O, alpha, flags, st, 0, -1, ws, ws_bytes);
        return fprop_tile<_Float16, TIN, BLOCKED, 64, 256, 64, 1, 4>(pl, I, F, O, alpha, flags, st, 0, -1, ws, ws_bytes);
    }
}

}  // namespace ng

using namespace ng;

extern "C" int ng_conv_fprop(const void* plan, int in_dtype, const void* I, const void* F, void* O,
                             float alpha, unsigned flags, void* workspace, size_t workspace_bytes,
                             void* stream)
{
    const ConvPlan* pl = (const ConvPlan*)plan;
    if (!pl) return fail(-48, "conv: null plan");
    int rc;
    if ((rc = check_ptr16(I, "I")) || (rc = check_ptr16(F, "F")) || (rc = check_ptr16(O, "O"))) return rc;
    hipStream_t st = (hipStream_t)stream;
    if ((uintptr_t)workspace & 15) { workspace = nullptr; workspace_bytes = 0; }   // optional here: only small grids slice
    if (pl->pointwise && in_dtype == pl->dtype) {
        // O (K x columns) = F^T (F is C x K) * I (C x columns): the GEMM dispatcher has the tile rules for
        // short contractions and small outputs (832 -> 256 maps on 7x7, N = 128: 17.5 -> 8.5 us)
        const ng_conv_params& p = pl->p;
        const int cols = p.M * p.P * p.Q * p.N;
        return ng_gemm(pl->dtype, 1, 0, p.K, cols, p.C, F, p.K, I, cols, O, cols, alpha, 0.0f, flags & NG_FLAG_RELU, 0u, 0u,
                       1, 0, 0, 0, 1, workspace, workspace_bytes, stream);
    }
    const bool blocked = pl->fprop_blocked;
    if (pl->dtype == NG_F16) {
        if (in_dtype == NG_F16)
            return blocked ? fprop_h<_Float16, true>(*pl, I, F, O, alpha, flags, st, workspace, workspace_bytes)
                           : fprop_h<_Float16, false>(*pl, I, F, O, alpha, flags, st, workspace, workspace_bytes);
        // byte inputs: first layers, few channels
        if (in_dtype == NG_U8) return fprop_h<u8_t, false>(*pl, I, F, O, alpha, flags, st, workspace, workspace_bytes);
        if (in_dtype == NG_I8) return fprop_h<s8_t, false>(*pl, I, F, O, alpha, flags, st, workspace, workspace_bytes);
    } else if (in_dtype == NG_F32) {
        return blocked ? fprop_tile<float, float, true, 128, 128, 16, 2, 2>(*pl, I, F, O, alpha, flags, st, 0, -1, workspace, workspace_bytes)
                       : fprop_tile<float, float, false, 128, 128, 16, 2, 2>(*pl, I, F, O, alpha, flags, st, 0, -1, workspace, workspace_bytes);
    }
    return fail(-49, "conv fprop: unsupported input dtype %d for filter dtype %d", in_dtype, pl->dtype);
}
