// Convolution entry points (fprop / bprop / update) on the MFMA contraction
// core.  Replaces the {h,s}conv_{fprop,bprop,updat}_* kernels and the helper
// launches around them in NervanaGPU._execute_conv
// (nervanagpu/nervanagpu.py:642-734).
//
// Differences from the reference kernels, all of which bring the results closer
// to its numpy statement (benchmarks/conv_test.py:138-167):
//  * bprop is always the gather form, for every C and stride: strided layers
//    are decomposed into str_d*str_h*str_w stride-1 sub-problems (one per
//    residue class of the input pixel), each with only the taps that can reach
//    that class.  No atomics, no zero fill, fp32 accumulation, one rounding.
//  * update accumulates fp32 partial sums over slices of the (pixel, n) range
//    and adds them in a fixed order instead of using fp32 atomics.
#include "conv_loaders.h"

#include <algorithm>
#include <vector>

namespace ng {

struct BpropClass {
    int rz, ry, rx;         // residues of the input pixel coordinates
    int nz, ny, nx;         // lattice extents of the class
    int J;                  // contraction rows: taps_in_class * K
    long tab_offset;        // first TapEntry of the class in d_bprop_tab
    long w_row;             // first row of the class in the re-laid filter
};

struct ConvPlan {
    ng_conv_params p;
    int dtype;
    int CRST, RST, Cpad;
    TapEntry* d_fprop_tab = nullptr;   // CRST entries
    TapEntry* d_bprop_tab = nullptr;   // K*RST entries, grouped by class
    int* d_tap_dest = nullptr;         // RST ints: first re-laid filter row of each tap
    std::vector<BpropClass> classes;
    size_t ws_bprop = 0, ws_update = 0;
};

static int cdiv(int a, int b) { return (a + b - 1) / b; }

static int splits_for(int out_tiles, int total_k_tiles, size_t slice_bytes, size_t ws_bytes)
{
    const int cus = device_cu_count();
    if (out_tiles >= cus || total_k_tiles < 8) return 1;
    int splits = cdiv(cus, out_tiles);
    splits = std::min(splits, total_k_tiles / 4);
    if (slice_bytes) splits = (int)std::min<size_t>((size_t)splits, ws_bytes / slice_bytes);
    while (splits > 1 && (splits - 1) * cdiv(total_k_tiles, splits) >= total_k_tiles) splits--;
    return std::max(splits, 1);
}

// filter (C,TRS,K) -> per-class matrices [(tap,k)][Cpad], zero padded in c
template <typename T>
__global__ void filter_relayout_kernel(const T* F, T* out, const int* tap_dest, int C, int RST, int K, int Cpad)
{
    const long total = (long)RST * K * Cpad;
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (long)gridDim.x * blockDim.x) {
        const int c = (int)(e % Cpad);
        const long r = e / Cpad;
        const int k = (int)(r % K);
        const int trs = (int)(r / K);
        const T v = (c < C) ? F[((long)c * RST + trs) * K + k] : (T)0;
        out[((long)tap_dest[trs] + k) * Cpad + c] = v;
    }
}

// ---------------------------------------------------------------------------
// launches
// ---------------------------------------------------------------------------

template <typename T, typename TIN, int BM, int BN, int BK, int WM, int WN, class Epi>
static int launch_gather_cols(const DenseLoader<T, MC, true>& al, const GatherColsLoader<T, TIN>& bl,
                              const Epi& epi, int rows, int ncols, int J, hipStream_t stream)
{
    CoreShape s;
    s.m = rows; s.n = ncols;
    s.k_tiles = cdiv(J, BK);
    s.passes = 1; s.splits = 1;
    s.tiles_m = cdiv(rows, BM);
    s.tiles_n = cdiv(ncols, BN);
    hipLaunchKernelGGL((mfma_gemm_kernel<T, BM, BN, BK, WM, WN, MC, MC, DenseLoader<T, MC, true>,
                                         GatherColsLoader<T, TIN>, Epi>),
                       dim3(s.tiles_m * s.tiles_n, 1, 1), dim3(WM * WN * 64), 0, stream, al, bl, epi, s);
    NG_CHECK_LAUNCH("conv kernel");
    return 0;
}

// pick the row tile with the least padding (ties -> larger tile)
template <typename T> struct RowTiles;
template <> struct RowTiles<_Float16> { static constexpr int n = 3; static constexpr int bm[3] = {256, 128, 64}; };
template <> struct RowTiles<float>    { static constexpr int n = 1; static constexpr int bm[1] = {128}; };

template <typename T>
static int pick_row_tile(int rows)
{
    int best = RowTiles<T>::bm[0], best_pad = cdiv(rows, best) * best;
    for (int i = 1; i < RowTiles<T>::n; i++) {
        const int b = RowTiles<T>::bm[i], pad = cdiv(rows, b) * b;
        if (pad < best_pad) { best = b; best_pad = pad; }
    }
    return best;
}

template <typename TIN, class Epi>
static int dispatch_gather_cols(const DenseLoader<_Float16, MC, true>& al, const GatherColsLoader<_Float16, TIN>& bl,
                                const Epi& epi, int rows, int ncols, int J, hipStream_t stream)
{
    switch (pick_row_tile<_Float16>(rows)) {
    case 256: return launch_gather_cols<_Float16, TIN, 256, 256, 32, 2, 2>(al, bl, epi, rows, ncols, J, stream);
    case 128: return launch_gather_cols<_Float16, TIN, 128, 256, 32, 2, 2>(al, bl, epi, rows, ncols, J, stream);
    default:  return launch_gather_cols<_Float16, TIN, 64, 512, 32, 1, 4>(al, bl, epi, rows, ncols, J, stream);
    }
}

template <class Epi>
static int dispatch_gather_cols(const DenseLoader<float, MC, true>& al, const GatherColsLoader<float, float>& bl,
                                const Epi& epi, int rows, int ncols, int J, hipStream_t stream)
{
    return launch_gather_cols<float, float, 128, 128, 16, 2, 2>(al, bl, epi, rows, ncols, J, stream);
}

template <typename T, typename TIN>
static int run_fprop(const ConvPlan& pl, const void* I, const void* F, void* O, float alpha, unsigned flags,
                     hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    const int ncols = p.M * p.P * p.Q * p.N;
    DenseLoader<T, MC, true> al{(const T*)F, 0, p.K, p.K, pl.CRST};
    GatherColsLoader<T, TIN> bl{(const TIN*)I, pl.d_fprop_tab, pl.CRST,
                                PixelLattice{p.N, ncols, p.Q, p.P * p.Q},
                                p.str_d, p.str_h, p.str_w, p.D, p.H, p.W};
    ScaleStoreEpilogue<T> epi{(T*)O, 0, ncols, p.K, ncols, alpha, 0.0f,
                              (flags & NG_FLAG_RELU) ? 1u : 0u, 0u, 0u, 0u, 1u};
    return dispatch_gather_cols(al, bl, epi, p.K, ncols, pl.CRST, stream);
}

template <typename T>
static int run_bprop(const ConvPlan& pl, const void* F, const void* E, void* gradI, float alpha,
                     void* ws, size_t ws_bytes, hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    if (ws_bytes < pl.ws_bprop || !ws) return fail(-40, "ng_conv_bprop: workspace too small (%zu < %zu)", ws_bytes, pl.ws_bprop);
    T* Fs = (T*)ws;
    {
        const long total = (long)pl.RST * p.K * pl.Cpad;
        const int blocks = (int)std::min<long>((total + 255) / 256, 4096);
        hipLaunchKernelGGL(filter_relayout_kernel<T>, dim3(blocks), dim3(256), 0, stream,
                           (const T*)F, Fs, pl.d_tap_dest, p.C, pl.RST, p.K, pl.Cpad);
        NG_CHECK_LAUNCH("filter relayout");
    }
    const long chan = (long)p.D * p.H * p.W * p.N;
    const bool dense = (p.str_d == 1 && p.str_h == 1 && p.str_w == 1);
    for (const BpropClass& c : pl.classes) {
        const int ncols = c.nz * c.ny * c.nx * p.N;
        if (ncols == 0) continue;
        PixelLattice lat{p.N, ncols, c.nx, c.nx * c.ny};
        DenseLoader<T, MC, true> al{Fs + c.w_row * pl.Cpad, 0, pl.Cpad, pl.Cpad, c.J};
        GatherColsLoader<T, T> bl{(const T*)E, pl.d_bprop_tab + c.tab_offset, c.J, lat,
                                  1, 1, 1, p.M, p.P, p.Q};
        int rc;
        if (dense) {
            ScaleStoreEpilogue<T> epi{(T*)gradI, 0, ncols, p.C, ncols, alpha, 0.0f, 0u, 0u, 0u, 0u, 1u};
            rc = dispatch_gather_cols(al, bl, epi, p.C, ncols, c.J, stream);
        } else {
            LatticeStoreEpilogue<T> epi{(T*)gradI, p.C, chan, lat, c.rz, c.ry, c.rx,
                                        p.str_d, p.str_h, p.str_w, p.H, p.W, alpha};
            rc = dispatch_gather_cols(al, bl, epi, p.C, ncols, c.J, stream);
        }
        if (rc) return rc;
    }
    return 0;
}

template <typename T, typename TIN, typename TOUT, int BM, int BN, int BK, int WM, int WN>
static int launch_update(const ConvPlan& pl, const void* I, const void* E, void* gradF, float alpha,
                         void* ws, size_t ws_bytes, hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    const int kdim = p.M * p.P * p.Q * p.N;
    CoreShape s;
    s.m = pl.CRST; s.n = p.K;
    s.k_tiles = cdiv(kdim, BK);
    s.passes = 1;
    s.tiles_m = cdiv(s.m, BM);
    s.tiles_n = cdiv(s.n, BN);
    const size_t slice = (size_t)s.m * s.n * sizeof(float);
    s.splits = ws ? splits_for(s.tiles_m * s.tiles_n, s.k_tiles, slice, ws_bytes) : 1;

    GatherRowsLoader<T, TIN> al{(const TIN*)I, pl.d_fprop_tab, pl.CRST, p.N, kdim, p.Q, p.P * p.Q,
                                p.str_d, p.str_h, p.str_w, p.D, p.H, p.W};
    DenseLoader<T, KC, true> bl{(const T*)E, 0, kdim, p.K, kdim};
    ScaleStoreEpilogue<TOUT> epi{(TOUT*)gradF, 0, p.K, s.m, s.n, alpha, 0.0f, 0u, 0u, 0u, 0u,
                                 (((uintptr_t)gradF & 15) == 0) ? 1u : 0u};
    dim3 grid(s.tiles_m * s.tiles_n, s.splits, 1), block(WM * WN * 64);
    if (s.splits == 1) {
        hipLaunchKernelGGL((mfma_gemm_kernel<T, BM, BN, BK, WM, WN, KC, KC, GatherRowsLoader<T, TIN>,
                                             DenseLoader<T, KC, true>, ScaleStoreEpilogue<TOUT>>),
                           grid, block, 0, stream, al, bl, epi, s);
        NG_CHECK_LAUNCH("conv update kernel");
    } else {
        PartialEpilogue pe{(float*)ws, s.m, s.n, 1, 1u};
        hipLaunchKernelGGL((mfma_gemm_kernel<T, BM, BN, BK, WM, WN, KC, KC, GatherRowsLoader<T, TIN>,
                                             DenseLoader<T, KC, true>, PartialEpilogue>),
                           grid, block, 0, stream, al, bl, pe, s);
        NG_CHECK_LAUNCH("conv update split kernel");
        const long total = (long)s.m * s.n;
        const int blocks = (int)std::min<long>((total + 255) / 256, 8192);
        hipLaunchKernelGGL((splitk_reduce_kernel<TOUT, ScaleStoreEpilogue<TOUT>>), dim3(blocks), dim3(256), 0,
                           stream, (const float*)ws, s.splits, 1, s.m, s.n, epi);
        NG_CHECK_LAUNCH("conv update reduce");
    }
    return 0;
}

template <typename TIN, typename TOUT>
static int run_update_h(const ConvPlan& pl, const void* I, const void* E, void* gradF, float alpha,
                        void* ws, size_t ws_bytes, hipStream_t stream)
{
    return launch_update<_Float16, TIN, TOUT, 128, 128, 32, 2, 2>(pl, I, E, gradF, alpha, ws, ws_bytes, stream);
}

static int check_ptr16(const void* p, const char* what)
{
    if (!p) return fail(-41, "conv: null %s", what);
    if ((uintptr_t)p & 15) return fail(-42, "conv: %s must be 16-byte aligned", what);
    return 0;
}

}  // namespace ng

using namespace ng;

extern "C" {

int ng_conv_plan_create(const ng_conv_params* pp, int dtype, void** plan_out)
{
    *plan_out = nullptr;
    const ng_conv_params& p = *pp;
    if (dtype != NG_F16 && dtype != NG_F32) return fail(-43, "conv: dtype must be fp16 or fp32");
    if (p.N % 8 || p.K % 8) return fail(-44, "conv: N and K must be multiples of 8");
    if (p.N <= 0 || p.C <= 0 || p.K <= 0 || p.M <= 0 || p.P <= 0 || p.Q <= 0) return fail(-45, "conv: empty geometry");
    if (p.str_d < 1 || p.str_h < 1 || p.str_w < 1) return fail(-46, "conv: strides must be >= 1");
    const long sizeI = (long)p.C * p.D * p.H * p.W * p.N, sizeO = (long)p.K * p.M * p.P * p.Q * p.N;
    if (sizeI >= (1L << 31) || sizeO >= (1L << 31)) return fail(-47, "conv: tensors of 2^31 elements or more are not supported");

    ConvPlan* pl = new ConvPlan();
    pl->p = p;
    pl->dtype = dtype;
    pl->RST = p.T * p.R * p.S;
    pl->CRST = p.C * pl->RST;
    pl->Cpad = cdiv(p.C, 8) * 8;
    const int HW = p.H * p.W, DHW = p.D * HW;

    // forward taps, rows j = (c,t,r,s)
    std::vector<TapEntry> ft((size_t)pl->CRST);
    for (int c = 0; c < p.C; c++)
        for (int t = 0; t < p.T; t++)
            for (int r = 0; r < p.R; r++)
                for (int s = 0; s < p.S; s++) {
                    const int dz = t - p.pad_d, dy = r - p.pad_h, dx = s - p.pad_w;
                    TapEntry e{(int)(((long)c * DHW + (long)dz * HW + dy * p.W + dx) * p.N), dz, dy, dx};
                    ft[(((size_t)c * p.T + t) * p.R + r) * p.S + s] = e;
                }

    // data-gradient classes: input pixel (z,y,x) with z % str_d == rz ... receives
    // tap t iff (rz + pad_d - t) % str_d == 0, from output m = iz + (rz + pad_d - t)/str_d
    std::vector<TapEntry> bt;
    std::vector<int> tap_dest((size_t)pl->RST, 0);
    const int PQ = p.P * p.Q;
    long w_row = 0;
    for (int rz = 0; rz < p.str_d; rz++)
        for (int ry = 0; ry < p.str_h; ry++)
            for (int rx = 0; rx < p.str_w; rx++) {
                BpropClass c;
                c.rz = rz; c.ry = ry; c.rx = rx;
                c.nz = (p.D > rz) ? (p.D - rz + p.str_d - 1) / p.str_d : 0;
                c.ny = (p.H > ry) ? (p.H - ry + p.str_h - 1) / p.str_h : 0;
                c.nx = (p.W > rx) ? (p.W - rx + p.str_w - 1) / p.str_w : 0;
                c.tab_offset = (long)bt.size();
                c.w_row = w_row;
                int taps = 0;
                for (int t = 0; t < p.T; t++) {
                    if ((rz + p.pad_d - t) % p.str_d) continue;
                    for (int r = 0; r < p.R; r++) {
                        if ((ry + p.pad_h - r) % p.str_h) continue;
                        for (int s = 0; s < p.S; s++) {
                            if ((rx + p.pad_w - s) % p.str_w) continue;
                            const int dz = (rz + p.pad_d - t) / p.str_d, dy = (ry + p.pad_h - r) / p.str_h,
                                      dx = (rx + p.pad_w - s) / p.str_w;
                            tap_dest[(size_t)(t * p.R + r) * p.S + s] = (int)(w_row + (long)taps * p.K);
                            for (int k = 0; k < p.K; k++)
                                bt.push_back(TapEntry{(int)(((long)k * p.M * PQ + (long)dz * PQ + dy * p.Q + dx) * p.N),
                                                      dz, dy, dx});
                            taps++;
                        }
                    }
                }
                c.J = taps * p.K;
                w_row += c.J;
                pl->classes.push_back(c);
            }

    auto upload = [&](const void* src, size_t bytes, void** dst) -> int {
        if (bytes == 0) { *dst = nullptr; return 0; }
        NG_HIP(hipMalloc(dst, bytes));
        NG_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return 0;
    };
    int rc = upload(ft.data(), ft.size() * sizeof(TapEntry), (void**)&pl->d_fprop_tab);
    if (!rc) rc = upload(bt.data(), bt.size() * sizeof(TapEntry), (void**)&pl->d_bprop_tab);
    if (!rc) rc = upload(tap_dest.data(), tap_dest.size() * sizeof(int), (void**)&pl->d_tap_dest);
    if (rc) { ng_conv_plan_destroy(pl); return rc; }

    pl->ws_bprop = align_up((size_t)pl->RST * p.K * pl->Cpad * dtype_size(dtype), 256);
    {
        const int kt = cdiv(p.M * p.P * p.Q * p.N, dtype == NG_F16 ? 32 : 16);
        const int tiles = cdiv(pl->CRST, 128) * cdiv(p.K, 128);
        const int splits = splits_for(tiles, kt, 0, 0);
        pl->ws_update = splits > 1 ? align_up((size_t)splits * pl->CRST * p.K * sizeof(float), 256) : 0;
    }
    *plan_out = pl;
    return 0;
}

int ng_conv_plan_destroy(void* plan)
{
    ConvPlan* pl = (ConvPlan*)plan;
    if (!pl) return 0;
    if (pl->d_fprop_tab) (void)hipFree(pl->d_fprop_tab);
    if (pl->d_bprop_tab) (void)hipFree(pl->d_bprop_tab);
    if (pl->d_tap_dest) (void)hipFree(pl->d_tap_dest);
    delete pl;
    return 0;
}

size_t ng_conv_plan_workspace_bytes(const void* plan)
{
    const ConvPlan* pl = (const ConvPlan*)plan;
    return pl ? std::max(pl->ws_bprop, pl->ws_update) : 0;
}

int ng_conv_fprop(const void* plan, int in_dtype, const void* I, const void* F, void* O,
                  float alpha, unsigned flags, void* /*workspace*/, size_t /*workspace_bytes*/, void* stream)
{
    const ConvPlan* pl = (const ConvPlan*)plan;
    if (!pl) return fail(-48, "conv: null plan");
    int rc;
    if ((rc = check_ptr16(I, "I")) || (rc = check_ptr16(F, "F")) || (rc = check_ptr16(O, "O"))) return rc;
    hipStream_t st = (hipStream_t)stream;
    if (pl->dtype == NG_F16) {
        if (in_dtype == NG_F16) return run_fprop<_Float16, _Float16>(*pl, I, F, O, alpha, flags, st);
        if (in_dtype == NG_U8)  return run_fprop<_Float16, u8_t>(*pl, I, F, O, alpha, flags, st);
        if (in_dtype == NG_I8)  return run_fprop<_Float16, s8_t>(*pl, I, F, O, alpha, flags, st);
    } else if (in_dtype == NG_F32) {
        return run_fprop<float, float>(*pl, I, F, O, alpha, flags, st);
    }
    return fail(-49, "conv fprop: unsupported input dtype %d for filter dtype %d", in_dtype, pl->dtype);
}

int ng_conv_bprop(const void* plan, const void* F, const void* E, void* gradI, float alpha,
                  void* workspace, size_t workspace_bytes, void* stream)
{
    const ConvPlan* pl = (const ConvPlan*)plan;
    if (!pl) return fail(-48, "conv: null plan");
    int rc;
    if ((rc = check_ptr16(F, "F")) || (rc = check_ptr16(E, "E")) || (rc = check_ptr16(gradI, "grad_I")) ||
        (rc = check_ptr16(workspace, "workspace")))
        return rc;
    hipStream_t st = (hipStream_t)stream;
    if (pl->dtype == NG_F16) return run_bprop<_Float16>(*pl, F, E, gradI, alpha, workspace, workspace_bytes, st);
    return run_bprop<float>(*pl, F, E, gradI, alpha, workspace, workspace_bytes, st);
}

int ng_conv_update(const void* plan, int in_dtype, int out_dtype, const void* I, const void* E, void* gradF,
                   float alpha, void* workspace, size_t workspace_bytes, void* stream)
{
    const ConvPlan* pl = (const ConvPlan*)plan;
    if (!pl) return fail(-48, "conv: null plan");
    int rc;
    if ((rc = check_ptr16(I, "I")) || (rc = check_ptr16(E, "E")) || (rc = check_ptr16(gradF, "grad_F"))) return rc;
    if (workspace && ((uintptr_t)workspace & 15)) return fail(-42, "conv: workspace must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    if (pl->dtype == NG_F16) {
        if (in_dtype == NG_F16 && out_dtype == NG_F32) return run_update_h<_Float16, float>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        if (in_dtype == NG_F16 && out_dtype == NG_F16) return run_update_h<_Float16, _Float16>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        if (in_dtype == NG_U8 && out_dtype == NG_F32)  return run_update_h<u8_t, float>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
        if (in_dtype == NG_U8 && out_dtype == NG_F16)  return run_update_h<u8_t, _Float16>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
    } else if (in_dtype == NG_F32 && out_dtype == NG_F32) {
        return launch_update<float, float, float, 128, 128, 16, 2, 2>(*pl, I, E, gradF, alpha, workspace, workspace_bytes, st);
    }
    return fail(-50, "conv update: unsupported dtype combination (in %d, out %d, filter %d)", in_dtype, out_dtype, pl->dtype);
}

}  // extern "C"
