// Host-side description of one convolution geometry, shared by the three
// convolution translation units.
#pragma once
#include <cstdlib>

#include "conv_loaders.h"
#include "stream_core.h"

#include <algorithm>
#include <vector>

namespace ng {

struct BpropClass {
    int rz, ry, rx;         // residues of the input pixel coordinates
    int nz, ny, nx;         // lattice extents of the class
    int taps;               // filter taps that reach the class
    int J;                  // contraction rows: taps * K
    long flat_offset;       // first flat TapEntry (one per (tap,k)) in d_bprop_flat
    long tap_offset;        // first per-tap TapEntry in d_bprop_taps
    long w_row;             // first row of the class in the re-laid filter
};

struct ConvPlan {
    ng_conv_params p;
    int dtype;
    int bk;                 // contraction tile depth of the kernels for this dtype
    int CRST, RST, Cpad;
    // Blocked contraction tiles (one filter tap x bk channels) are used when the
    // channel count is a multiple of bk or padding it to one wastes little;
    // Kpad is K rounded up to bk when the data gradient runs blocked, else K.
    bool fprop_blocked = false, bprop_blocked = false;
    int Kpad = 0;
    TapEntry* d_fprop_flat = nullptr;   // CRST entries, rows (c,t,r,s)
    TapEntry* d_fprop_taps = nullptr;   // RST entries
    TapEntry* d_bprop_flat = nullptr;   // K*RST entries grouped by class, rows (tap,k)
    TapEntry* d_bprop_taps = nullptr;   // RST entries grouped by class
    int* d_bprop_trs = nullptr;         // RST ints grouped by class: filter position of each class tap
    int* d_tap_dest = nullptr;          // RST ints: first re-laid filter row of each tap
    std::vector<BpropClass> classes;
    // Merged form of the strided data gradient (used when all classes together
    // have at most 256 rows): one problem whose rows are (class, c) and whose
    // contraction runs over the union of the classes' output-pixel offsets.
    bool merged = false;
    int m_rows = 0, m_rpad = 0;         // classes * C and its multiple of 8
    int m_taps = 0;                     // distinct (dz,dy,dx) offsets
    int m_nz = 0, m_ny = 0, m_nx = 0;   // lattice of class 0 (the largest)
    TapEntry* d_merged_taps = nullptr;  // m_taps entries
    TapEntry* d_merged_flat = nullptr;  // m_taps * K entries, rows (offset, k)
    size_t ws_bprop = 0, ws_update = 0;
    size_t ws_small = 0;                // contraction slices of small forward / data-gradient grids
    // 1x1x1 filter, unit strides, no padding: forward and data gradient are plain matrix products
    // (O = F^T I, gradI = F E over the (pixel, n) columns) and go to the GEMM dispatcher
    bool pointwise = false;
};

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// channel blocks of depth bk: exact, or padded by at most one half
inline bool blocks_pay(int channels, int bk) { return channels % bk == 0 || 2 * cdiv(channels, bk) * bk <= 3 * channels; }

// how many slices to cut a contraction into: as many as fill every workgroup
// slot of the chip exactly once (`per_cu` workgroups of this tile shape fit the
// LDS of a CU), rounded down.  Workgroups that share a CU share its matrix
// pipes, so a grid is as slow as its fullest CU: one and a half workgroups per
// CU cost what two cost, and a grid a few workgroups over a whole round costs a
// round more (VGG weight gradients 7-22 % faster than with a rounded-up one and
// a half per CU).  Contractions too short to leave 15 tiles per slice get one
// workgroup per CU: the fp32 partials then cost more than the overlap gains.
// NG_CONV_STAGES (read once per process), candidates that have not been measured on a device yet:
// 3 = forward / data gradient grids of at most one workgroup per CU of 128x256x64 tiles run three
// LDS stages; 4 = also, layers of 128 images on such grids leave the shared taps (whose 56 KB stages
// only fit twice) for those tiles.  Unset: two stages everywhere, as measured.
inline int conv_stage_switch()
{
    static const int v = std::getenv("NG_CONV_STAGES") ? std::atoi(std::getenv("NG_CONV_STAGES")) : 2;
    return v;
}

inline int conv_splits(int out_tiles, int total_k_tiles, size_t slice_bytes, size_t ws_bytes, int per_cu = 2)
{
    const int cus = device_cu_count();
    if (total_k_tiles < 8) return 1;
    const int slots = cus * per_cu;
    int splits = std::max(1, slots / out_tiles);
    if (splits == 1 && out_tiles < slots && slice_bytes) {
        // More than half a round of tiles but less than a whole one (144 tiles of 256x256 on 256 CUs): a
        // few slices can still pay.  Cost in tile steps: rounds over the chip times steps per slice, plus
        // the fp32 partial sums written and read again (at about 5 TB/s, a tile step being about 1.4 us).
        const double step_bytes = 1.4e-6 * 5e12 / 2;
        double best = (double)total_k_tiles;
        for (int s = 2; s <= 6 && s * 8 <= total_k_tiles; s++) {
            const double cost = (double)cdiv(out_tiles * s, slots) * cdiv(total_k_tiles, s) + s * (double)slice_bytes / step_bytes;
            if (cost < best * 0.95) { best = cost; splits = s; }
        }
    }
    if (total_k_tiles / splits < 15) splits = std::max(1, cus / out_tiles);
    splits = std::min(splits, std::max(1, total_k_tiles / 4));
    if (slice_bytes) splits = (int)std::min<size_t>((size_t)splits, ws_bytes / slice_bytes);
    while (splits > 1 && (splits - 1) * cdiv(total_k_tiles, splits) >= total_k_tiles) splits--;
    return std::max(splits, 1);
}

// workgroups of a weight-gradient tile shape (64-deep, two stages) that fit
// the LDS of a CU: three of the 64x64 tile (measured better than four: VGG
// conv1 119 -> 86 us against two), one of 256x256, two of the shapes between
inline int update_tiles_per_cu(int bm, int bn)
{
    if (bm == 64 && bn == 64) return 3;
    return bm >= 256 ? 1 : 2;
}

inline int check_ptr16(const void* p, const char* what)
{
    if (!p) return fail(-41, "conv: null %s", what);
    if ((uintptr_t)p & 15) return fail(-42, "conv: %s must be 16-byte aligned", what);
    return 0;
}

// Row tile (output feature maps or input channels) for BN-column tiles: the
// candidate with the least estimated time per contraction tile, rounds of
// workgroups over the chip times the duration of one tile step of that shape.
// The steps are measured ones (microseconds per 64-deep tile with the CU to
// itself: 256 rows and 128 rows on eight wavefronts, 64 rows on four); two
// 64-row workgroups fit the LDS of a CU and overlap, the larger shapes run one
// per CU.  Padding rows count as work through the number of row tiles, so a
// 64-row problem with many column tiles picks the 64-row tile, while a grid of
// at most one workgroup per CU prefers the 128-row tile, whose eight wavefronts
// hide the latency of a tile step better.
inline int pick_row_tile(int rows, int ncols, int bn, double* cost_out = nullptr)
{
    static const int tiles[3] = {256, 128, 64};
    static const int resident[3] = {1, 1, 2};
    static const double step_us[3] = {1.75, 1.2, 1.39};
    const int cus = device_cu_count();
    int best = tiles[0];
    double best_cost = 0.0;
    for (int i = 0; i < 3; i++) {
        const long blocks = (long)cdiv(rows, tiles[i]) * cdiv(ncols, bn);
        const long slots = (long)cus * resident[i];
        const double cost = (double)((blocks + slots - 1) / slots) * step_us[i];
        if (i == 0 || cost < best_cost * 0.999) { best = tiles[i]; best_cost = cost; }
    }
    if (cost_out) *cost_out = best_cost;
    return best;
}

// A grid of one-per-CU workgroups that is a few tiles more than a whole number
// of rounds over the chip spends a full round on those few (784 tiles on 256 CUs:
// four rounds for 3.06; 4 x 72 = 288 tiles: two for 1.125).  Returns how many trailing
// column tiles (all their row tiles) to take out of the main launch and run behind it as
// many small tiles that cover the chip at once: enough to bring the main launch down to
// whole rounds, when there is at least one full round and the remainder is at most a
// quarter of the chip; else 0.
inline int tail_column_tiles(int tiles_m, int tiles_n)
{
    const int cus = device_cu_count();
    const long total = (long)tiles_m * tiles_n;
    if (total <= cus) return 0;
    const int rem = (int)(total % cus);
    if (rem == 0 || 4 * rem > cus) return 0;
    const int cols = cdiv(rem, tiles_m);
    return cols < tiles_n ? cols : 0;
}

// Contraction slices for a forward / data-gradient grid that covers less than half of the
// chip (7x7 maps: 25-75 workgroups on 256 CUs): as many as fill the chip once, each
// keeping at least 8 contraction tiles; 1 = no slicing.
inline int small_grid_splits(int tiles, int k_tiles, size_t slice_bytes, const void* ws, size_t ws_bytes)
{
    const int cus = device_cu_count();
    if (!ws || 2 * tiles > cus || k_tiles < 16 || slice_bytes == 0) return 1;
    int splits = std::min(cus / tiles, k_tiles / 8);
    splits = (int)std::min<size_t>((size_t)splits, ws_bytes / slice_bytes);
    while (splits > 1 && (splits - 1) * cdiv(k_tiles, splits) >= k_tiles) splits--;
    return std::max(splits, 1);
}

// col_begin / col_end: the column range this launch covers (multiples of BN; default: all)
template <typename T, int BM, int BN, int BK, int WM, int WN, int LA, int LB, int NSTAGE = 2, class AL, class BL, class Epi>
inline int launch_core(const AL& al, const BL& bl, const Epi& epi, int rows, int ncols, int k_tiles, int splits,
                       hipStream_t stream, const char* what, int col_begin = 0, int col_end = -1)
{
    if (col_end < 0) col_end = ncols;
    CoreShape s;
    s.m = rows; s.n = ncols;
    s.k_tiles = k_tiles;
    s.passes = 1; s.splits = splits;
    s.tiles_m = cdiv(rows, BM);
    s.tiles_n = cdiv(col_end - col_begin, BN);
    s.n_base = col_begin;
    launch_mfma_core<T, BM, BN, BK, WM, WN, LA, LB, NSTAGE>(dim3(grid_tiles(s.tiles_m * s.tiles_n, splits), grid_slices(s.tiles_m * s.tiles_n, splits), 1), stream, al, bl, epi, s);
    NG_CHECK_LAUNCH(what);
    return 0;
}

// launch_core over the whole problem, with the contraction sliced (fp32 partial sums in `ws`,
// added in slice order by the reduce kernel, which then runs `epi`) when the grid is small
template <typename T, int BM, int BN, int BK, int WM, int WN, int LA, int LB, int NSTAGE = 2, class AL, class BL, class Epi>
inline int launch_core_sliced(const AL& al, const BL& bl, const Epi& epi, int rows, int ncols, int k_tiles,
                              void* ws, size_t ws_bytes, hipStream_t stream, const char* what)
{
    const size_t slice = (size_t)rows * ncols * sizeof(float);
    const int splits = small_grid_splits(cdiv(rows, BM) * cdiv(ncols, BN), k_tiles, slice, ws, ws_bytes);
    if (splits == 1) return launch_core<T, BM, BN, BK, WM, WN, LA, LB, NSTAGE>(al, bl, epi, rows, ncols, k_tiles, 1, stream, what);
    PartialEpilogue pe{(float*)ws, rows, ncols, 1, (ncols % 8 == 0) ? 1u : 0u};
    const int rc = launch_core<T, BM, BN, BK, WM, WN, LA, LB, NSTAGE>(al, bl, pe, rows, ncols, k_tiles, splits, stream, what);
    if (rc) return rc;
    launch_splitk_reduce<T, Epi>((const float*)ws, splits, 1, rows, ncols, epi, stream);
    NG_CHECK_LAUNCH(what);
    return 0;
}

}  // namespace ng
