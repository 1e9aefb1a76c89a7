// Convolution data gradient: gradI = round(alpha * conv_transpose(E, F)).
// Replaces {h,s}conv_bprop_{C64_N64,C32_N64} and the dimShuffle / transpose /
// memset launches around them (nervanagpu/nervanagpu.py:652-659, 685-719).
//
// Always the gather form, for every C and stride: strided layers are decomposed
// into str_d*str_h*str_w stride-1 sub-problems (one per residue class of the
// input pixel), each with only the taps that can reach that class.  No atomics,
// no zero fill, fp32 accumulation, one rounding.
#include "conv_plan.h"

namespace ng {

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

template <typename T, bool BLOCKED, int BM, int BN, int BK, int WM, int WN>
static int bprop_class(const ConvPlan& pl, const BpropClass& c, const T* Fs, const void* E, void* gradI,
                       float alpha, hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    const int ncols = c.nz * c.ny * c.nx * p.N;
    const int MPQN = p.M * p.P * p.Q * p.N;
    const PixelLattice lat = PixelLattice::make(p.N, ncols, c.nx, c.nx * c.ny);
    DenseLoader<T, MC, true> al{Fs + c.w_row * pl.Cpad, 0, pl.Cpad, pl.Cpad, c.J};
    const int nblk = BLOCKED ? p.K / BK : 1;
    GatherColsLoader<T, T, BLOCKED, BK> bl{(const T*)E,
                                           BLOCKED ? pl.d_bprop_taps + c.tap_offset : pl.d_bprop_flat + c.flat_offset,
                                           c.J, lat, 1, 1, 1, p.M, p.P, p.Q,
                                           MPQN, FastDiv::make((unsigned)nblk), nblk};
    const int k_tiles = cdiv(c.J, BK);
    const bool dense = (p.str_d == 1 && p.str_h == 1 && p.str_w == 1);
    if (dense) {
        ScaleStoreEpilogue<T> epi{(T*)gradI, 0, ncols, p.C, ncols, alpha, 0.0f, 0u, 0u, 0u, 0u, 1u};
        return launch_core<T, BM, BN, BK, WM, WN, MC, MC>(al, bl, epi, p.C, ncols, k_tiles, 1, stream, "conv bprop");
    }
    LatticeStoreEpilogue<T> epi{(T*)gradI, p.C, (long)p.D * p.H * p.W * p.N, lat, c.rz, c.ry, c.rx,
                                p.str_d, p.str_h, p.str_w, p.H, p.W, alpha};
    return launch_core<T, BM, BN, BK, WM, WN, MC, MC>(al, bl, epi, p.C, ncols, k_tiles, 1, stream, "conv bprop");
}

template <bool BLOCKED>
static int bprop_class_h(const ConvPlan& pl, const BpropClass& c, const _Float16* Fs, const void* E, void* gradI,
                         float alpha, hipStream_t st)
{
    switch (pick_row_tile(pl.p.C, c.nz * c.ny * c.nx * pl.p.N, 256)) {
    case 256: return bprop_class<_Float16, BLOCKED, 256, 256, 64, 2, 4>(pl, c, Fs, E, gradI, alpha, st);
    case 128: return bprop_class<_Float16, BLOCKED, 128, 256, 64, 1, 4>(pl, c, Fs, E, gradI, alpha, st);
    default:  return bprop_class<_Float16, BLOCKED, 64, 256, 64, 1, 4>(pl, c, Fs, E, gradI, alpha, st);
    }
}

template <typename T>
static int run_bprop(const ConvPlan& pl, const void* F, const void* E, void* gradI, float alpha,
                     void* ws, size_t ws_bytes, hipStream_t stream)
{
    const ng_conv_params& p = pl.p;
    if (ws_bytes < pl.ws_bprop || !ws)
        return fail(-40, "ng_conv_bprop: workspace too small (%zu < %zu)", ws_bytes, pl.ws_bprop);
    T* Fs = (T*)ws;
    {
        const long total = (long)pl.RST * p.K * pl.Cpad;
        const int blocks = (int)std::min<long>((total + 255) / 256, 4096);
        hipLaunchKernelGGL(filter_relayout_kernel<T>, dim3(blocks), dim3(256), 0, stream,
                           (const T*)F, Fs, pl.d_tap_dest, p.C, pl.RST, p.K, pl.Cpad);
        NG_CHECK_LAUNCH("filter relayout");
    }
    const bool blocked = p.K % pl.bk == 0;
    for (const BpropClass& c : pl.classes) {
        if (c.nz * c.ny * c.nx == 0) continue;
        int rc;
        if (sizeof(T) == 2)
            rc = blocked ? bprop_class_h<true>(pl, c, (const _Float16*)Fs, E, gradI, alpha, stream)
                         : bprop_class_h<false>(pl, c, (const _Float16*)Fs, E, gradI, alpha, stream);
        else
            rc = blocked ? bprop_class<float, true, 128, 128, 16, 2, 2>(pl, c, (const float*)Fs, E, gradI, alpha, stream)
                         : bprop_class<float, false, 128, 128, 16, 2, 2>(pl, c, (const float*)Fs, E, gradI, alpha, stream);
        if (rc) return rc;
    }
    return 0;
}

}  // namespace ng

using namespace ng;

extern "C" int ng_conv_bprop(const void* plan, const void* F, const void* E, void* gradI, float alpha,
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
