// 3x3 convolution (unit strides, 64 images) whose filter has at most 64 rows and
// at most 64 contraction channels: the filter stays in registers, the activations
// stream, and every activation row is fetched once.
//
// The tiled kernel gives such a layer one workgroup per 64 x 256 output tile.  With
// six contraction tiles that workgroup is mostly set-up and epilogue (VGG conv1.2:
// 6 vector and 5 scalar instructions per MFMA where the 256-row tiles spend 2 and
// 2), and every input row travels to the CUs three times, once per filter row
// (1.18 GB from the memory side for the 411 MB of that layer: the L2 of an XCD
// is smaller than what its workgroups touch between two uses of a row).
//
// Here a workgroup owns a contiguous run of column tiles counted down the image: it
// walks down a strip of PX output pixels.  The whole filter, per block of BK
// channels three contraction tiles (filter rows) of 3 taps x BK rows, is read once
// into registers as MFMA fragments.  The activations of the strip (PX + 2 pixels
// wide, shared by the three taps of a filter row as in GatherRowSegLoader) live in
// LDS as a ring of three image rows: output row y multiplies rows y-1, y, y+1, and
// as soon as the tiles of row y-1 are done its slots take row y+2 for the next
// output row, whose request so has the other two thirds of the tile to arrive.
// The stores of a column tile overlap the multiplications of the next.
//
// What a lane adds to a request is fixed for the whole run (its pixel, images and
// channel inside the tile); where the tile lies travels in the buffer descriptor,
// computed on the scalar unit, and a descriptor of zero length stands for a row in
// the padding.
#pragma once

#include "stream_core.h"

namespace ng {

// StreamBands with a quarter of the staging: the eight rows a lane group holds in
// accumulator registers 4g .. 4g+3 of a 32-row band go through LDS at a time, so a
// lane leaves each pass with 8 consecutive columns of one row (one 16-byte store).
template <int TM, int TN, int WTN, int EPITCH, int I>
struct StreamBandsNarrow {
    template <class Epi>
    static __device__ __forceinline__ void run(float16_t (&acc)[TM][TN], char* stage, int lane, int mbase, int nbase,
                                               BufferRsrc rsrc, const Epi& epi)
    {
        static_assert(8 * WTN / 8 == 64, "a pass is one store instruction per lane");
        const int col = lane & 31;
        const int rsub = (lane >> 5) * 4;
#pragma unroll
        for (int g = 0; g < 4; g++) {
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int v = 0; v < 4; v++)
                    *reinterpret_cast<float*>(stage + (rsub + v) * EPITCH + (j * 32 + col) * 4) = acc[I][j][g * 4 + v];
            wave_lds_fence();
            const int r = lane / (WTN / 8);
            const int cc = (lane % (WTN / 8)) * 8;
            const float4_t lo = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4);
            const float4_t hi = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4 + 16);
            const float vals[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            epi.store8_buffer(rsrc, mbase + I * 32 + g * 8 + r, nbase + cc, vals);
            wave_lds_fence();
        }
        if constexpr (I + 1 < TM) StreamBandsNarrow<TM, TN, WTN, EPITCH, I + 1>::run(acc, stage, lane, mbase, nbase, rsrc, epi);
    }
};

// geometry of the activation stream (2-D: one image plane per channel)
template <typename T>
struct RowSegStream {
    const T* X;            // activations (forward) or output gradients (data gradient), C x H x W x 64
    int      H, W;         // rows and pixels per row of X
    int      pad_h, pad_w; // first filter row / tap lies this far above / left of the output pixel
    int      plane;        // elements between consecutive channels (H * W * 64)
    int      out_rows;     // output rows
    int      out_width;    // output pixels per row (a multiple of PX)
    FastDiv  rows_div;
};

template <typename T, int BM, int PX, int BK, int WM, int WN, int KT, int LA, class ALoad, class Epi>
__global__ __launch_bounds__(WM * WN * 64)
void conv_stream_taps_kernel(ALoad aload, RowSegStream<T> bg, Epi epi, int tiles)
{
    static_assert(sizeof(T) == 2 && ALoad::DIRECT, "16-bit operands through direct LDS loads");
    constexpr int NIMG = 64, TAPS = 3, FR = 3;   // images, taps per filter row, filter rows
    static_assert(KT % FR == 0, "whole channel blocks");
    constexpr int BN = PX * NIMG, SEG = BN + (TAPS - 1) * NIMG;
    constexpr int NT = WM * WN * 64;
    constexpr int KSTEP = Elem<T>::KSTEP;
    constexpr int KS = BK / KSTEP, NSTEP = TAPS * KS;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32, WTN = BN / WN;
    using TA = TapTile<T, LA, BM, BK, TAPS>;
    using TB = SwizzledTile<T, MC, SEG, BK>;
    using FA = SwizzledFrag<LA, typename TA::Sub>;
    using FB = SwizzledFrag<MC, TB>;
    constexpr int CPT_B = TB::CHUNKS / NT;
    static_assert(TB::CHUNKS % NT == 0, "B tile chunks must divide evenly over threads");
    static_assert(TA::CHUNKS % 64 == 0 && TA::BYTES <= FR * (KT / FR) * TB::BYTES, "A tile is staged through the ring, wavefront by wavefront");
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % KSTEP == 0, "bad tile shape");
    constexpr int NB = KT / FR;                  // channel blocks
    constexpr int EPITCH = WTN * 4;              // unpadded: the ring leaves 16 KB
    constexpr int EPI_BYTES = 8 * EPITCH;        // epilogue staging per wavefront: eight rows at a time
    constexpr int RING = FR * NB * TB::BYTES;    // three image rows
    static_assert(RING + EPI_BYTES * WM * WN <= 160 * 1024, "ring and epilogue staging exceed the LDS of a compute unit");
    __shared__ __attribute__((aligned(16))) char smem[RING + EPI_BYTES * WM * WN];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    // contiguous share of the column tiles, counted down the image (strip-major)
    const int nwg = (int)gridDim.x;
    const int per = (tiles + nwg - 1) / nwg;
    const int first = (int)blockIdx.x * per;
    const int count = min(per, tiles - first);
    if (count <= 0) return;

    // ---- A: every contraction tile once through LDS into fragments ----
    // contraction tiles are counted (channel block, filter row), block-major, as the A loaders count them
    Frag<T> fa[KT][NSTEP][TM];
    int fa_base[TM];
#pragma unroll
    for (int i = 0; i < TM; i++) fa_base[i] = FA::base(wm * TM + i, lane);
    const typename ALoad::Wave a_wave = aload.wave_init(lane);
#pragma unroll
    for (int kt = 0; kt < KT; kt++) {
        const typename ALoad::Tile ta = aload.tile(kt, kt * BK, 0, a_wave);
#pragma unroll
        for (int i = 0; i * NT < TA::CHUNKS; i++) {
            if (i * NT + wave * 64 < TA::CHUNKS) {   // uniform over the wavefront
                int r, k;
                TA::chunk_pos(tid + i * NT, r, k);
                buffer_load_chunk_to_lds(ta.rsrc, smem + (i * NT + wave * 64) * 16, aload.offset(ta, aload.prepare(r, k)));
            }
        }
        __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
        __syncthreads();
#pragma unroll
        for (int st = 0; st < NSTEP; st++)
#pragma unroll
            for (int i = 0; i < TM; i++) fa[kt][st][i] = FA::load(smem + TA::tile_of(st, KS), fa_base[i], TA::step_of(st, KS));
        __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
        __syncthreads();
    }

    // ---- B: ring of three image rows ----
    // the part of a request's offset that belongs to the lane, and its pixel in the segment
    unsigned voff[CPT_B], xoff[CPT_B];
    int pix[CPT_B];
#pragma unroll
    for (int c = 0; c < CPT_B; c++) {
        int r, k;
        TB::chunk_pos(tid + c * NT, r, k);
        pix[c] = r / NIMG;
        voff[c] = (unsigned)(r + k * bg.plane) * (unsigned)sizeof(T);
    }
    // output row, first output pixel and ring phase (y mod 3) of the current column tile
    int y, x0, ph;
    {
        const int strip = (int)bg.rows_div.div((unsigned)first);
        y = first - strip * bg.out_rows;
        x0 = strip * PX;
        ph = y - (y / 3) * 3;
    }
    auto set_strip = [&]() {
#pragma unroll
        for (int c = 0; c < CPT_B; c++)
            xoff[c] = ((unsigned)(x0 - bg.pad_w + pix[c]) < (unsigned)bg.W) ? voff[c] : NG_OOB_OFFSET;
    };
    // request the input row under filter row `fr` of output row `yy` (all channel blocks) into ring slot `slot`
    auto issue_row = [&](int yy, int fr, int slot) {
        const int iy = yy + fr - bg.pad_h;
        const unsigned len = ((unsigned)iy < (unsigned)bg.H) ? 0x80000000u : 0u;
#pragma unroll
        for (int blk = 0; blk < NB; blk++) {
            const long at = ((long)iy * bg.W + (x0 - bg.pad_w)) * NIMG + (long)blk * BK * bg.plane;
            const BufferRsrc rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(bg.X + at), 0, len, 0x00020000);
#pragma unroll
            for (int c = 0; c < CPT_B; c++)
                buffer_load_chunk_to_lds(rsrc, smem + (slot * NB + blk) * TB::BYTES + (c * NT + wave * 64) * 16, xoff[c]);
        }
    };
    auto next_phase = [](int p) { return p == 2 ? 0 : p + 1; };

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
    int fb_base[TAPS][TN];
#pragma unroll
    for (int tap = 0; tap < TAPS; tap++)
#pragma unroll
        for (int j = 0; j < TN; j++) fb_base[tap][j] = FB::base(wn * TN + j + tap * (NIMG / 32), lane);
    // k-steps G0 .. G1-1 of a column tile; step g is k-step g % NSTEP of contraction
    // tile (block (g / NSTEP) % NB, filter row g / (NB * NSTEP)).  One wavefront per
    // SIMD has nobody to hide an LDS round trip behind: fragments are read two
    // k-steps (eight MFMAs) ahead.
    Frag<T> fb[3][TN];
    auto load_step = [&](auto g_c, const int (&slot)[FR]) {
        constexpr int g = decltype(g_c)::value;
        constexpr int fr = g / (NB * NSTEP), blk = (g / NSTEP) % NB, st = g % NSTEP;
        const char* tile = smem + (slot[fr] * NB + blk) * TB::BYTES;
#pragma unroll
        for (int j = 0; j < TN; j++) fb[g % 3][j] = FB::load(tile, fb_base[st / KS][j], st % KS);
    };
    auto run_steps = [&](auto g0_c, auto g1_c, const int (&slot)[FR]) {
        constexpr int G0 = decltype(g0_c)::value, G1 = decltype(g1_c)::value;
        load_step(std::integral_constant<int, G0>{}, slot);
        if constexpr (G0 + 1 < G1) load_step(std::integral_constant<int, G0 + 1>{}, slot);
        static_for<G0, G1>([&](auto g_c) {
            constexpr int g = decltype(g_c)::value;
            constexpr int fr = g / (NB * NSTEP), blk = (g / NSTEP) % NB, st = g % NSTEP;
            if constexpr (g + 2 < G1) load_step(std::integral_constant<int, g + 2>{}, slot);
#pragma unroll
            for (int m = 0; m < TM; m++)
#pragma unroll
                for (int j = 0; j < TN; j++) mfma_step(fa[blk * FR + fr][st][m], fb[g % 3][j], acc[m][j]);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    constexpr int ROW_STEPS = NB * NSTEP;        // k-steps per filter row
    constexpr int ROW_LOADS = NB * CPT_B;        // requests per image row and thread

    // store instructions every wavefront issues per epilogue
    constexpr int NS = TM * (32 * WTN / 8 / 64);
    static_assert(NS + FR * NB * CPT_B < 64, "the vector-memory counter holds 63 operations");
    static_assert(NS + NB * CPT_B < 64, "the vector-memory counter holds 63 operations");
    const BufferRsrc out_rsrc = make_rsrc(epi.base());
    char* stage = smem + RING + wave * EPI_BYTES;

    // Per column tile: filter rows 0 and 1 multiply image rows the ring has held since
    // the tile before; behind filter row 0 its slot takes the row the NEXT tile needs
    // last; only filter row 2 waits for a request, the one issued a whole tile ago.
    bool fresh = true;   // the ring holds none of the rows of the current column tile
    for (int i = 0; i < count; i++) {
        const int slot[FR] = {ph, next_phase(ph), next_phase(next_phase(ph))};
        if (fresh) {
            // every wavefront is done with the rows of the column tile before
            __syncthreads();
            set_strip();
            issue_row(y, 0, slot[0]);
            issue_row(y, 1, slot[1]);
            issue_row(y, 2, slot[2]);
            __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
            __syncthreads();
        }
        run_steps(std::integral_constant<int, 0>{}, std::integral_constant<int, ROW_STEPS>{}, slot);
        // the next column tile lies below this one: its third row goes where row y-1 was
        const bool below = (i + 1 < count) && (y + 1 < bg.out_rows);
        if (below) {
            __syncthreads();
            issue_row(y + 1, 2, slot[0]);
        }
        run_steps(std::integral_constant<int, ROW_STEPS>{}, std::integral_constant<int, 2 * ROW_STEPS>{}, slot);
        if (!fresh) {
            // row y+1 was requested behind filter row 0 of the tile before; since then this
            // wavefront has issued that tile's NS stores and, if the next tile lies below,
            // the requests just above (vector-memory operations complete in issue order)
            if (below) __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<NS + ROW_LOADS>::IMM);
            else       __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<NS>::IMM);
            __syncthreads();
        }
        run_steps(std::integral_constant<int, 2 * ROW_STEPS>{}, std::integral_constant<int, 3 * ROW_STEPS>{}, slot);
        const int n0 = (y * bg.out_width + x0) * NIMG;
        StreamBandsNarrow<TM, TN, WTN, EPITCH, 0>::run(acc, stage, lane, wm * (BM / WM), n0 + wn * WTN, out_rsrc, epi);
#pragma unroll
        for (int m = 0; m < TM; m++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[m][j][v] = 0.0f;
        fresh = !below;
        ph = slot[1];
        if (++y == bg.out_rows) { y = 0; ph = 0; x0 += PX; }
    }
}

// one workgroup per CU (the ring takes the LDS)
template <typename T, int BM, int PX, int BK, int WM, int WN, int KT, int LA, class AL, class Epi>
inline void launch_stream_taps(const AL& al, const RowSegStream<T>& bg, const Epi& epi, int tiles, hipStream_t stream)
{
    const int grid = std::min(tiles, device_cu_count());
    hipLaunchKernelGGL((conv_stream_taps_kernel<T, BM, PX, BK, WM, WN, KT, LA, AL, Epi>), dim3(grid), dim3(WM * WN * 64), 0,
                       stream, al, bg, epi, tiles);
}

}  // namespace ng
