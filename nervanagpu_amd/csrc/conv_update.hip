// Convolution weight gradient: gradF = round(alpha * sum_{pixels,n} I x E).
// Replaces {h,s}conv_updat_C128_{K64,K128}, the zero fill and the fp32 convert
// launch (nervanagpu/nervanagpu.py:661-669, 695-724).  fp32 partial sums over
// slices of the (pixel, n) range are added in a fixed order instead of with
// fp32 atomics, so the result does not depend on execution order.
#include "conv_plan.h"
#include <cstdlib>
#include "conv_update_ring.h"
#include "conv_update_strip.h"

namespace ng {

template <typename T, typename TIN, typename TOUT, bool BLOCKED, int BM, int BN, int BK, int WM, int WN>
static int launch_update(const ConvPlan& pl, const void* I, const void* E, void* gradF, float alpha,
                         void* ws, size_t ws_bytes, hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    const int kdim = p.M * p.P * p.Q * p.N;
    const int rows = pl.CRST, cols = p.K;
    const int k_tiles = cdiv(kdim, BK);
    const int tiles = cdiv(rows, BM) * cdiv(cols, BN);
    const size_t slice = (size_t)rows * cols * sizeof(float);
    const int splits = ws ? conv_splits(tiles, k_tiles, slice, ws_bytes, update_tiles_per_cu(BM, BN)) : 1;
    const int npt = BLOCKED ? p.N / BK : 1;

    GatherRowsLoader<T, TIN, BLOCKED, BK> al{(const TIN*)I, pl.d_fprop_flat, pl.CRST, p.N, kdim, p.Q, p.P * p.Q,
                                             p.str_d, p.str_h, p.str_w, p.D, p.H, p.W,
                                             FastDiv::make((unsigned)npt), FastDiv::make((unsigned)(p.P * p.Q)),
                                             FastDiv::make((unsigned)p.Q), npt};
    DenseLoader<T, KC, true> bl{(const T*)E, 0, kdim, p.K, kdim};
    ScaleStoreEpilogue<TOUT> epi{(TOUT*)gradF, 0, p.K, rows, cols, alpha, 0.0f, 0u, 0u, 0u, 0u,
                                 (((uintptr_t)gradF & 15) == 0) ? 1u : 0u};
    if (splits == 1)
        return launch_core<T, BM, BN, BK, WM, WN, KC, KC>(al, bl, epi, rows, cols, k_tiles, 1, stream, "conv update");
    PartialEpilogue pe{(float*)ws, rows, cols, 1, 1u};
    int rc = launch_core<T, BM, BN, BK, WM, WN, KC, KC>(al, bl, pe, rows, cols, k_tiles, splits, stream, "conv update");
    if (rc) return rc;
    launch_splitk_reduce<TOUT, ScaleStoreEpilogue<TOUT>>((const float*)ws, splits, 1, rows, cols, epi, stream);
    NG_CHECK_LAUNCH("conv update reduce");
    return 0;
}

// Three horizontal taps, unit strides, 64 images, at most 64 output maps and at least 64
// rows (c,t,r): the ring kernel (conv_update_ring.h).  With more output maps the tiles of
// gemm_core.h are less bound by their requests (64 -> 128 maps on 112x112: 0.143 against
// 0.160 ms with 64-row workgroups).
static bool update_shares_taps(const ConvPlan& pl)
{
    const ng_conv_params& p = pl.p;
    const int CR = p.C * p.T * p.R;
    // 65 .. 128 output maps: only with whole 128-row workgroups on large maps (3-6 % faster than the
    // general tiles on 96x96 and 112x112 maps; on 56x56 and with padded rows it is a draw or worse)
    const bool fits = p.K <= 64 ? CR >= 64 : (p.K <= 128 && CR % 128 == 0 && (long)p.M * p.P * p.Q >= 8192);
    return p.S == 3 && p.pad_w == 1 && p.N == 64 && fits && p.K % 8 == 0 &&
           p.str_d == 1 && p.str_h == 1 && p.str_w == 1 &&
           (long)p.C * p.D * p.H * p.W * p.N * 2 < (1L << 31) && (long)p.K * p.M * p.P * p.Q * p.N * 2 < (1L << 31);
}

template <typename TOUT, int CRB, int BN, int LEAD, int PER_CU>
static int launch_update_ring(const ConvPlan& pl, const void* I, const void* E, void* gradF, float alpha,
                              void* ws, size_t ws_bytes, hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    const int CR = p.C * p.T * p.R, rows = pl.CRST, cols = p.K;
    CoreShape s;
    s.m = rows; s.n = cols;
    s.tiles_m = cdiv(CR, CRB); s.tiles_n = cdiv(cols, BN);
    s.passes = 1;
    const int tiles = s.tiles_m * s.tiles_n;
    const int steps = p.M * p.P * (p.W + 2);
    s.k_tiles = steps;
    const size_t slice = (size_t)rows * cols * sizeof(float);
    s.splits = ws ? conv_splits(tiles, steps, slice, ws_bytes, PER_CU) : 1;
    UpdateRingGeom g{(const _Float16*)I, (const _Float16*)E, CR, p.T * p.R, p.R, p.D, p.H, p.W, p.M * p.P, p.P,
                     p.pad_d, p.pad_h, p.K, p.D * p.H * p.W * p.N, p.M * p.P * p.Q * p.N, steps,
                     FastDiv::make((unsigned)(p.T * p.R)), FastDiv::make((unsigned)p.R), FastDiv::make((unsigned)(p.W + 2)),
                     FastDiv::make((unsigned)p.P)};
    ScaleStoreEpilogue<TOUT> epi{(TOUT*)gradF, 0, p.K, rows, cols, alpha, 0.0f, 0u, 0u, 0u, 0u,
                                 (((uintptr_t)gradF & 15) == 0) ? 1u : 0u};
    const dim3 grid(grid_tiles(tiles, s.splits), grid_slices(tiles, s.splits), 1);
    const dim3 block(CRB / 32 * 2 * 64);
    if (s.splits == 1) {
        hipLaunchKernelGGL((conv_update_ring_kernel<CRB, BN, LEAD, ScaleStoreEpilogue<TOUT>>), grid, block, 0, stream, g, epi, s);
        NG_CHECK_LAUNCH("conv update (ring)");
        return 0;
    }
    PartialEpilogue pe{(float*)ws, rows, cols, 1, 1u};
    hipLaunchKernelGGL((conv_update_ring_kernel<CRB, BN, LEAD, PartialEpilogue>), grid, block, 0, stream, g, pe, s);
    NG_CHECK_LAUNCH("conv update (ring)");
    launch_splitk_reduce<TOUT, ScaleStoreEpilogue<TOUT>>((const float*)ws, s.splits, 1, rows, cols, epi, stream);
    NG_CHECK_LAUNCH("conv update reduce");
    return 0;
}

// 3x3 filters, padding 1, unit strides, one image plane, 64 images, 33 to 64 channels and at most
// 64 output maps: the strip kernel (conv_update_strip.h), all nine taps on one ring
static bool update_walks_strips(const ConvPlan& pl)
{
    const ng_conv_params& p = pl.p;
    return p.R == 3 && p.S == 3 && p.T == 1 && p.D == 1 && p.pad_d == 0 && p.pad_h == 1 && p.pad_w == 1 &&
           p.str_d == 1 && p.str_h == 1 && p.str_w == 1 && p.N == 64 && p.C > 32 && p.C <= 64 && p.K <= 64 && p.K % 8 == 0 &&
           p.P == p.H && p.Q == p.W && p.W >= 8 &&
           (long)p.C * p.H * p.W * p.N * 2 < (1L << 31) && (long)p.K * p.P * p.Q * p.N * 2 < (1L << 31);
}

template <typename TOUT>
static int launch_update_strip(const ConvPlan& pl, const void* I, const void* E, void* gradF, float alpha,
                               void* ws, size_t ws_bytes, hipStream_t stream)
{
    constexpr int WT = 4, LEAD = 2;
    const ng_conv_params& p = pl.p;
    const int rows = pl.CRST, cols = p.K;
    CoreShape s;
    s.m = rows; s.n = cols;
    s.tiles_m = 1; s.tiles_n = 1;
    s.passes = 1;
    const int strips = cdiv(p.W, WT);
    const int strip_rows = strips * (p.H + 2);      // the unit of a contraction slice: WT + 2 steps each
    s.k_tiles = strip_rows;
    const size_t slice = (size_t)rows * cols * sizeof(float);
    s.splits = ws ? conv_splits(1, strip_rows, slice, ws_bytes, 1) : 1;
    UpdateStripGeom g{(const _Float16*)I, (const _Float16*)E, p.C, p.K, p.H, p.W, strips, p.H * p.W * p.N,
                      p.P * p.Q * p.N, strip_rows, FastDiv::make((unsigned)(p.H + 2))};
    ScaleStoreEpilogue<TOUT> epi{(TOUT*)gradF, 0, p.K, rows, cols, alpha, 0.0f, 0u, 0u, 0u, 0u,
                                 (((uintptr_t)gradF & 15) == 0) ? 1u : 0u};
    const dim3 grid(grid_tiles(1, s.splits), grid_slices(1, s.splits), 1);
    const dim3 block(768);
    if (s.splits == 1) {
        hipLaunchKernelGGL((conv_update_strip_kernel<WT, LEAD, ScaleStoreEpilogue<TOUT>>), grid, block, 0, stream, g, epi, s);
        NG_CHECK_LAUNCH("conv update (strips)");
        return 0;
    }
    PartialEpilogue pe{(float*)ws, rows, cols, 1, 1u};
    hipLaunchKernelGGL((conv_update_strip_kernel<WT, LEAD, PartialEpilogue>), grid, block, 0, stream, g, pe, s);
    NG_CHECK_LAUNCH("conv update (strips)");
    launch_splitk_reduce<TOUT, ScaleStoreEpilogue<TOUT>>((const float*)ws, s.splits, 1, rows, cols, epi, stream);
    NG_CHECK_LAUNCH("conv update reduce");
    return 0;
}

template <typename TIN, typename TOUT>
static int update_h(const ConvPlan& pl, const void* I, const void* E, void* gradF, float alpha,
                    void* ws, size_t ws_bytes, hipStream_t st)
{
    if (pl.p.N % 64 == 0) {
        // fp16 activations: tile shaped after the filter matrix (CRST x K)
        if constexpr (std::is_same<TIN, _Float16>::value) {
            {
                // A candidate that has passed the CPU emulation but has not been measured on a device yet:
                // off unless NG_UPDATE_STRIPS=1 (read once per process)
                static const int strips_on = getenv("NG_UPDATE_STRIPS") ? atoi(getenv("NG_UPDATE_STRIPS")) : 0;
                if (strips_on && update_walks_strips(pl)) return launch_update_strip<TOUT>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
            }
            if (update_shares_taps(pl)) {
                // all rows of a 64-channel 3x3 filter in one workgroup of twelve wavefronts (E is
                // then requested once instead of once per 64 rows; VGG conv1.2 0.47 -> 0.38 ms),
                // when 192-row tiles pad the rows no more than 64-row tiles do
                const int CR = pl.p.C * pl.p.T * pl.p.R;
                if (pl.p.K > 64) return launch_update_ring<TOUT, 128, 128, 1, 1>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
                if (cdiv(CR, 192) * 192 <= cdiv(CR, 64) * 64)
                    return launch_update_ring<TOUT, 192, 64, 2, 1>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
                return launch_update_ring<TOUT, 64, 64, 1, 3>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
            }
            // 256x256 tiles leave few output tiles, i.e. many contraction slices
            // and fp32 partials: worth it for long pixel ranges, or when the filter
            // is so large that the 128x128 tiles take more than one round of the
            // chip without any slicing (512 -> 1024 maps on 12x12 pixels, N = 128:
            // 0.259 -> 0.200 ms)
            const long kdim = (long)pl.p.M * pl.p.P * pl.p.Q * pl.p.N;
            const long tiles128 = (long)cdiv(pl.CRST, 128) * cdiv(pl.p.K, 128);
            if (pl.p.K >= 256 && pl.CRST >= 256 && (kdim >= 512 * 64 || tiles128 > device_cu_count()))
                return launch_update<_Float16, TIN, TOUT, true, 256, 256, 64, 2, 4>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
            if (pl.p.K <= 64 && pl.CRST <= 64)
                return launch_update<_Float16, TIN, TOUT, true, 64, 64, 64, 2, 2>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
            // 192-row tiles when they pad the filter rows no more than 128-row tiles do
            // (C * 9 rows of 3x3 filters over 64 k channels divide evenly) and the
            // pixel range is long: a wavefront then multiplies three row blocks with
            // each fragment of E it reads (VGG conv1.2 0.63 -> 0.51 ms, conv2.1
            // 0.190 -> 0.166 ms; at 28x28 and 55x55 pixels the 128-row tiles,
            // which cut the contraction into fewer slices, are 7-10 % faster)
            const bool rows192 = cdiv(pl.CRST, 192) * 192 <= cdiv(pl.CRST, 128) * 128 && kdim >= 4096 * 64;
            // output maps that fill their last 128-column tile only half (192, 320): 64-column tiles
            // output maps in odd multiples of 192 would leave a 128-column tile half empty: 192-column
            // tiles (three column blocks per wavefront) on contractions long enough to pay for the
            // extra slices (64 -> 192 maps, 5x5 on 27x27, N = 128: 0.083 -> 0.073 ms)
            if (pl.p.K % 192 == 0 && pl.p.K % 128 != 0 && kdim >= 256 * 64)
                return launch_update<_Float16, TIN, TOUT, true, 128, 192, 64, 2, 2>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
            if (pl.p.K <= 64) {
                if (rows192) return launch_update<_Float16, TIN, TOUT, true, 192, 64, 64, 2, 2>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
                return launch_update<_Float16, TIN, TOUT, true, 128, 64, 64, 2, 2>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
            }
            if (rows192) return launch_update<_Float16, TIN, TOUT, true, 192, 128, 64, 2, 2>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
        }
        return launch_update<_Float16, TIN, TOUT, true, 128, 128, 64, 2, 2>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
    }
    return launch_update<_Float16, TIN, TOUT, false, 128, 128, 64, 2, 2>(pl, I, E, gradF, alpha, ws, ws_bytes, st);
}

}  // namespace ng

using namespace ng;

extern "C" int ng_conv_update(const void* plan, int in_dtype, int out_dtype, const void* I, const void* E,
                              void* gradF, float alpha, void* workspace, size_t workspace_bytes, void* stream)
{
    const ConvPlan* pl = (const ConvPlan*)plan;
    if (!pl) return fail(-48, "conv: null plan");
    int rc;
    if ((rc = check_ptr16(I, "I")) || (rc = check_ptr16(E, "E")) || (rc = check_ptr16(gradF, "grad_F"))) return rc;
    if (workspace && ((uintptr_t)workspace & 15)) return fail(-42, "conv: workspace must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    if (pl->dtype == NG_F16) {
        if (in_dtype == NG_F16 && out_dtype == NG_F32) return update_h<_Float16, float>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        if (in_dtype == NG_F16 && out_dtype == NG_F16) return update_h<_Float16, _Float16>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        if (in_dtype == NG_U8 && out_dtype == NG_F32)  return update_h<u8_t, float>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        if (in_dtype == NG_U8 && out_dtype == NG_F16)  return update_h<u8_t, _Float16>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        if (in_dtype == NG_I8 && out_dtype == NG_F32)  return update_h<s8_t, float>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        if (in_dtype == NG_I8 && out_dtype == NG_F16)  return update_h<s8_t, _Float16>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
    } else if (in_dtype == NG_F32 && out_dtype == NG_F32) {
        if (pl->p.N % 16 == 0)
            return launch_update<float, float, float, true, 128, 128, 16, 2, 2>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        return launch_update<float, float, float, false, 128, 128, 16, 2, 2>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
    }
    return fail(-50, "conv update: unsupported dtype combination (in %d, out %d, filter %d)", in_dtype, out_dtype, pl->dtype);
}
