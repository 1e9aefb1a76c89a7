// Convolution plans: the per-geometry tap tables of the gather loaders
// (counterpart of ConvLayer.__init__ precomputing its kernel arguments,
// nervanagpu/layers.py:281-481).
#include "conv_plan.h"

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
    const long es = (long)dtype_size(dtype);
    if (sizeI * es >= (1L << 31) || sizeO * es >= (1L << 31))
        return fail(-47, "conv: tensors of 2 GiB or more are not supported");

    ConvPlan* pl = new ConvPlan();
    pl->p = p;
    pl->dtype = dtype;
    pl->bk = (dtype == NG_F16) ? 64 : 16;
    pl->RST = p.T * p.R * p.S;
    pl->CRST = p.C * pl->RST;
    pl->Cpad = cdiv(p.C, 8) * 8;
    pl->fprop_blocked = blocks_pay(p.C, pl->bk);
    pl->bprop_blocked = blocks_pay(p.K, pl->bk);
    pl->Kpad = pl->bprop_blocked ? cdiv(p.K, pl->bk) * pl->bk : p.K;
    const int HW = p.H * p.W, DHW = p.D * HW;

    // forward taps
    std::vector<TapEntry> ftaps((size_t)pl->RST), fflat((size_t)pl->CRST);
    for (int t = 0; t < p.T; t++)
        for (int r = 0; r < p.R; r++)
            for (int s = 0; s < p.S; s++) {
                const int dz = t - p.pad_d, dy = r - p.pad_h, dx = s - p.pad_w;
                const int trs = (t * p.R + r) * p.S + s;
                ftaps[(size_t)trs] = TapEntry{(int)(((long)dz * HW + dy * p.W + dx) * p.N), dz, dy, dx};
                for (int c = 0; c < p.C; c++)
                    fflat[(size_t)c * pl->RST + trs] =
                        TapEntry{(int)(((long)c * DHW + (long)dz * HW + dy * p.W + dx) * p.N), dz, dy, dx};
            }

    // data-gradient classes: input pixel (z,y,x) with z % str_d == rz ... receives
    // tap t iff (rz + pad_d - t) % str_d == 0, from output m = iz + (rz + pad_d - t)/str_d
    std::vector<TapEntry> bflat, btaps;
    std::vector<int> btrs;
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
                c.flat_offset = (long)bflat.size();
                c.tap_offset = (long)btaps.size();
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
                            tap_dest[(size_t)(t * p.R + r) * p.S + s] = (int)(w_row + (long)taps * pl->Kpad);
                            btaps.push_back(TapEntry{(int)(((long)dz * PQ + dy * p.Q + dx) * p.N), dz, dy, dx});
                            btrs.push_back((t * p.R + r) * p.S + s);
                            for (int k = 0; k < p.K; k++)
                                bflat.push_back(TapEntry{(int)(((long)k * p.M * PQ + (long)dz * PQ + dy * p.Q + dx) * p.N),
                                                         dz, dy, dx});
                            taps++;
                        }
                    }
                }
                c.taps = taps;
                c.J = taps * pl->Kpad;
                w_row += c.J;
                pl->classes.push_back(c);
            }

    // merged strided data gradient: offsets d = (residue + pad - tap) / stride over
    // all classes span a small box; every (dz,dy,dx) of the box is one merged tap
    std::vector<TapEntry> mtaps, mflat;
    const int nclasses = p.str_d * p.str_h * p.str_w;
    if (nclasses > 1 && (long)nclasses * p.C <= 256) {
        auto lo = [](int pad, int win, int str) {       // floor((pad - (win-1)) / str)
            const int a = pad - (win - 1);
            return a >= 0 ? a / str : -((-a + str - 1) / str);
        };
        auto hi = [](int pad, int str) { return (str - 1 + pad) / str; };
        const int z0 = lo(p.pad_d, p.T, p.str_d), z1 = hi(p.pad_d, p.str_d);
        const int y0 = lo(p.pad_h, p.R, p.str_h), y1 = hi(p.pad_h, p.str_h);
        const int x0 = lo(p.pad_w, p.S, p.str_w), x1 = hi(p.pad_w, p.str_w);
        for (int dz = z0; dz <= z1; dz++)
            for (int dy = y0; dy <= y1; dy++)
                for (int dx = x0; dx <= x1; dx++) {
                    mtaps.push_back(TapEntry{(int)(((long)dz * PQ + dy * p.Q + dx) * p.N), dz, dy, dx});
                    for (int k = 0; k < p.K; k++)
                        mflat.push_back(TapEntry{(int)(((long)k * p.M * PQ + (long)dz * PQ + dy * p.Q + dx) * p.N),
                                                 dz, dy, dx});
                }
        pl->merged = true;
        pl->m_rows = nclasses * p.C;
        pl->m_rpad = cdiv(pl->m_rows, 8) * 8;
        pl->m_taps = (int)mtaps.size();
        pl->m_nz = cdiv(p.D, p.str_d); pl->m_ny = cdiv(p.H, p.str_h); pl->m_nx = cdiv(p.W, p.str_w);
    }

    auto upload = [&](const void* src, size_t bytes, void** dst) -> int {
        if (bytes == 0) { *dst = nullptr; return 0; }
        NG_HIP(hipMalloc(dst, bytes));
        NG_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return 0;
    };
    int rc = upload(fflat.data(), fflat.size() * sizeof(TapEntry), (void**)&pl->d_fprop_flat);
    if (!rc) rc = upload(ftaps.data(), ftaps.size() * sizeof(TapEntry), (void**)&pl->d_fprop_taps);
    if (!rc) rc = upload(bflat.data(), bflat.size() * sizeof(TapEntry), (void**)&pl->d_bprop_flat);
    if (!rc) rc = upload(btaps.data(), btaps.size() * sizeof(TapEntry), (void**)&pl->d_bprop_taps);
    if (!rc) rc = upload(btrs.data(), btrs.size() * sizeof(int), (void**)&pl->d_bprop_trs);
    if (!rc) rc = upload(tap_dest.data(), tap_dest.size() * sizeof(int), (void**)&pl->d_tap_dest);
    if (!rc) rc = upload(mtaps.data(), mtaps.size() * sizeof(TapEntry), (void**)&pl->d_merged_taps);
    if (!rc) rc = upload(mflat.data(), mflat.size() * sizeof(TapEntry), (void**)&pl->d_merged_flat);
    if (rc) { ng_conv_plan_destroy(pl); return rc; }

    // data gradient scratch: the merged filter, or the re-laid filter of the
    // row-by-row form; the blocked form reads the filter in place
    if (pl->merged)
        pl->ws_bprop = align_up((size_t)pl->m_taps * p.K * pl->m_rpad * dtype_size(dtype), 256);
    else if (!pl->bprop_blocked)
        pl->ws_bprop = align_up((size_t)pl->RST * pl->Kpad * pl->Cpad * dtype_size(dtype), 256);
    else
        pl->ws_bprop = 0;
    {
        const int kt = cdiv(p.M * p.P * p.Q * p.N, pl->bk);
        const size_t upd_slice = (size_t)pl->CRST * p.K * sizeof(float);
        // the most slices any tile shape of the update dispatcher would ask for
        static const int shapes[7][2] = {{128, 128}, {256, 256}, {64, 64}, {192, 64}, {192, 128}, {128, 64}, {128, 192}};
        int splits = 1;
        for (const auto& t : shapes)
            splits = std::max(splits, conv_splits(cdiv(pl->CRST, t[0]) * cdiv(p.K, t[1]), kt, upd_slice, ~(size_t)0, update_tiles_per_cu(t[0], t[1])));
        // the ring kernel of filters with three horizontal taps: 64 or 192 rows (c,t,r) per tile, W + 2 positions per image row
        if (p.S == 3 && p.K <= 128) {
            const int ring_steps = p.M * p.P * (p.W + 2), CR = p.C * p.T * p.R;
            splits = std::max(splits, conv_splits(cdiv(CR, 64), ring_steps, upd_slice, ~(size_t)0, 3));
            splits = std::max(splits, conv_splits(cdiv(CR, 192), ring_steps, upd_slice, ~(size_t)0, 1));
            splits = std::max(splits, conv_splits(cdiv(CR, 128), ring_steps, upd_slice, ~(size_t)0, 1));
        }
        pl->ws_update = splits > 1 ? align_up((size_t)splits * pl->CRST * p.K * sizeof(float), 256) : 0;
    }
    {
        // forward and (with the filter read in place) data gradient may slice the contraction of a
        // grid that covers less than half of the chip: room for the most slices any tile shape asks for
        auto room = [&](int rows, long ncols_l, int kt) {
            if (ncols_l * rows >= (1L << 30)) return (size_t)0;
            const int ncols = (int)ncols_l;
            const size_t slice = (size_t)rows * ncols * sizeof(float);
            size_t bytes = 0;
            static const int shapes[4][2] = {{256, 256}, {128, 256}, {64, 256}, {128, 128}};
            for (const auto& t : shapes) {
                const int sp = small_grid_splits(cdiv(rows, t[0]) * cdiv(ncols, t[1]), kt, slice, pl, ~(size_t)0);
                if (sp > 1) bytes = std::max(bytes, (size_t)sp * slice);
            }
            return bytes;
        };
        const int kt_f = std::max(pl->RST * cdiv(p.C, pl->bk), cdiv(pl->CRST, 16));
        pl->ws_small = room(p.K, (long)p.M * p.P * p.Q * p.N, kt_f);
        const bool unit = p.str_d == 1 && p.str_h == 1 && p.str_w == 1;
        if (pl->bprop_blocked && !pl->merged && unit)
            pl->ws_small = std::max(pl->ws_small, room(p.C, (long)p.D * p.H * p.W * p.N, pl->RST * cdiv(p.K, pl->bk)));
        pl->pointwise = pl->RST == 1 && unit && p.pad_d == 0 && p.pad_h == 0 && p.pad_w == 0 &&
                        (long)p.M * p.P * p.Q * p.N < (1L << 31);
        if (pl->pointwise) {
            const int cols = p.M * p.P * p.Q * p.N;
            pl->ws_small = std::max(pl->ws_small, ng_gemm_workspace_bytes(dtype, 1, 0, p.K, cols, p.C, 1, 1));
            pl->ws_small = std::max(pl->ws_small, ng_gemm_workspace_bytes(dtype, 0, 0, p.C, cols, p.K, 1, 1));
        }
        pl->ws_small = align_up(pl->ws_small, 256);
    }
    *plan_out = pl;
    return 0;
}

int ng_conv_plan_destroy(void* plan)
{
    ConvPlan* pl = (ConvPlan*)plan;
    if (!pl) return 0;
    if (pl->d_fprop_flat) (void)hipFree(pl->d_fprop_flat);
    if (pl->d_fprop_taps) (void)hipFree(pl->d_fprop_taps);
    if (pl->d_bprop_flat) (void)hipFree(pl->d_bprop_flat);
    if (pl->d_bprop_taps) (void)hipFree(pl->d_bprop_taps);
    if (pl->d_bprop_trs) (void)hipFree(pl->d_bprop_trs);
    if (pl->d_tap_dest) (void)hipFree(pl->d_tap_dest);
    if (pl->d_merged_taps) (void)hipFree(pl->d_merged_taps);
    if (pl->d_merged_flat) (void)hipFree(pl->d_merged_flat);
    delete pl;
    return 0;
}

size_t ng_conv_plan_workspace_bytes(const void* plan)
{
    const ConvPlan* pl = (const ConvPlan*)plan;
    return pl ? std::max(std::max(pl->ws_bprop, pl->ws_update), pl->ws_small) : 0;
}

}  // extern "C"
