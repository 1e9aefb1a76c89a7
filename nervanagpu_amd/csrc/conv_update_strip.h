// Weight gradient of 3x3 filters (unit strides, padding 1, one image plane) with at most
// 64 channels and at most 64 output maps on 64 images: all nine taps share their
// activations.
//
// gF[(c,r,s)][k] = sum over output pixels (y,q) and images n of I[c, y+r-1, q+s-1, n] * E[k, y, q, n].
// The ring kernel of conv_update_ring.h shares the three horizontal taps: a step requests
// one pixel of I per row (c,r), i.e. every pixel of I three times in the course of a walk
// (once per vertical tap), 192 lines of 128 bytes per step that all lie one channel stride
// apart.  Here a workgroup walks down a strip of WT output columns and keeps, per channel
// only, the last two strip rows of input pixels and the current one in a ring of LDS
// slots: a step requests ONE new input pixel of 64 channels (64 lines) and one pixel of E,
// and tap (r,s) reads the slot that was requested (2-r) strip rows and -s positions ago.
// Every input pixel of the strip (WT + 2 columns wide, so strips overlap by two) is
// requested once.
//
// Walk: a strip has WS = WT + 2 positions per row and H + 2 rows yy = -2 .. H-1 (the two
// rows before the image fill the ring; their steps multiply nothing).  Position
// p = (strip * (H + 2) + yy + 2) * WS + xs.  The A stream holds input pixel
// (row yy + 1, column x0 + xs - 1) at position p (rows -1 and H and columns -1 and W are
// the zero padding); the B stream holds output pixel (yy, x0 + xs) for yy >= 0, xs < WT
// (else nothing: the step only moves the ring).  Tap (r,s) of step p reads A position
// p + s - (2 - r) * WS.  A contraction slice is a range of positions; its first
// 2 * WS + 2 requests refill the ring.
#pragma once
#include "conv_plan.h"

namespace ng {

struct UpdateStripGeom {
    const _Float16* I;
    const _Float16* E;
    int C, K;
    int H, W;           // input = output extents (padding 1, unit strides)
    int strips;         // ceil(W / WT)
    int chan_stride;    // elements between channels of I: H*W*N
    int kdim;           // row length of E: H*W*N
    int steps;          // strips * (H + 2) * WS
    FastDiv ws_div, rows_div;   // by WS, by H + 2
};

// WT output columns per strip; LEAD: steps a request is issued ahead of its use
// (ring of 2 * WS + 3 + LEAD slots of 8 KB, 1 + LEAD stages of E)
template <int WT, int LEAD, class Epi>
__global__ __launch_bounds__(768)
void conv_update_strip_kernel(UpdateStripGeom g, Epi epi, CoreShape s)
{
    typedef _Float16 T;
    constexpr int N = 64;                          // images per pixel = contraction elements per step
    constexpr int CB = 64, BN = 64;                // channels (rows of a slot), output maps
    constexpr int WS = WT + 2, TAPS = 3;
    constexpr int WM = 6, WN = 2, NT = WM * WN * 64;   // wavefront rows: (channel block, vertical tap)
    constexpr int RING = 2 * WS + TAPS + LEAD, BST = 1 + LEAD;
    using TA = SwizzledTile<T, KC, CB, N>;         // one input pixel: 64 channels x 128 bytes
    using TB = SwizzledTile<T, KC, BN, N>;         // one pixel of E: 64 maps x 128 bytes
    using FA = SwizzledFrag<KC, TA>;
    using FB = SwizzledFrag<KC, TB>;
    static_assert(TA::CHUNKS == 512 && TB::CHUNKS == 512, "eight wavefronts request a slot, four request a stage twice");
    constexpr int A_BYTES = RING * TA::BYTES, B_BYTES = BST * TB::BYTES;
    static_assert(A_BYTES + B_BYTES <= 160 * 1024, "ring exceeds the LDS");
    constexpr int WTN = BN / WN;
    constexpr int EPITCH = WTN * 4 + 16;
    constexpr int EPI_BYTES = 32 * EPITCH;
    constexpr int SMEM_BYTES = (A_BYTES + B_BYTES > EPI_BYTES * WM * WN) ? A_BYTES + B_BYTES : EPI_BYTES * WM * WN;
    __shared__ __attribute__((aligned(16))) char smem[SMEM_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int cb = wm & 1, rtap = wm >> 1;         // 32-channel block and vertical tap of this wavefront

    int tm, tn, split;
    if (!block_work(s, tm, tn, split)) return;
    const int per = (g.steps + s.splits - 1) / s.splits;
    const int i_begin = split * per;
    const int i_end = min(i_begin + per, g.steps);
    const int nsteps = i_end - i_begin;

    // wavefronts 0..7 request the input pixel (one chunk a lane), 8..11 the pixel of E (two)
    const bool loads_a = wave < 8;
    int a_chan = 0;          // what of the address does not move with the walk
    bool a_valid = false;
    unsigned b_off[2] = {NG_OOB_OFFSET, NG_OOB_OFFSET};
    if (loads_a) {
        int r, k;
        TA::chunk_pos(tid, r, k);
        a_valid = r < g.C;
        a_chan = min(r, g.C - 1) * g.chan_stride + k;
    } else {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int chunk = (tid - 512) + i * 256;
            int r, k;
            TB::chunk_pos(chunk, r, k);
            b_off[i] = (r < g.K) ? ((unsigned)r * (unsigned)g.kdim + (unsigned)k) * 2u : NG_OOB_OFFSET;
        }
    }
    const BufferRsrc a_rsrc = make_rsrc(g.I), b_rsrc = make_rsrc(g.E);

    // walkers (wavefront-uniform).  A: next position to request; starts 2 * WS positions before the slice
    struct Walk { int strip, yy, xs; };
    auto walk_at = [&](int p) {
        Walk w;
        if (p < 0) { w.strip = -1; w.yy = -2; w.xs = p; return w; }     // before the first strip: nothing
        const int row = (int)g.ws_div.div((unsigned)p);
        w.xs = p - row * WS;
        w.strip = (int)g.rows_div.div((unsigned)row);
        w.yy = row - w.strip * (g.H + 2) - 2;
        return w;
    };
    auto advance = [&](Walk& w) {
        if (w.strip < 0) { if (++w.xs == 0) { w.strip = 0; w.yy = -2; } return; }
        if (++w.xs == WS) { w.xs = 0; if (++w.yy == g.H) { w.yy = -2; w.strip++; } }
    };
    Walk aw = walk_at(i_begin - 2 * WS), bw = walk_at(i_begin), cw = bw;

    auto issue_a = [&](int slot) {
        if (loads_a) {
            const int row = aw.yy + 1, col = aw.strip * WT + aw.xs - 1;
            const bool ok = a_valid & (aw.strip >= 0) & (aw.strip < g.strips) & ((unsigned)row < (unsigned)g.H) &
                            ((unsigned)col < (unsigned)g.W);
            const unsigned off = ok ? (unsigned)(a_chan + (row * g.W + col) * N) * 2u : NG_OOB_OFFSET;
            buffer_load_chunk_to_lds(a_rsrc, smem + slot * TA::BYTES + (wave * 64) * 16, off);
        }
        advance(aw);
    };
    auto issue_b = [&](int stage) {
        if (!loads_a) {
            const int q = bw.strip * WT + bw.xs;
            const bool ok = (bw.strip < g.strips) & (bw.yy >= 0) & (bw.xs < WT) & (q < g.W);
            const unsigned pix = (unsigned)(bw.yy * g.W + q) * (unsigned)(N * 2);
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const unsigned off = (ok & (b_off[i] != NG_OOB_OFFSET)) ? b_off[i] + pix : NG_OOB_OFFSET;
                // chunk (wave - 8) * 64 + lane + i * 256: the hardware adds 16 * lane to the wavefront's base
                buffer_load_chunk_to_lds(b_rsrc, smem + A_BYTES + stage * TB::BYTES + ((i * 4 + (wave - 8)) * 64) * 16, off);
            }
        }
        advance(bw);
    };

    float16_t acc[TAPS][1];
#pragma unroll
    for (int t = 0; t < TAPS; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][0][v] = 0.0f;

    const int fa_base = FA::base(cb, lane);
    const int fb_base = FB::base(wn, lane);

    // slot / stage indices advance by counters (the ring lengths are not powers of two)
    auto next = [](int v, int n) { return v + 1 == n ? 0 : v + 1; };
    int a_wr = 0, b_wr = 0;         // where the next requests go
    // slot of A position (step + s - (2 - rtap) * WS) for s = 0: the ring starts at position i_begin - 2 * WS
    int a_rd = rtap * WS, b_rd = 0;
    int issued = 0;                 // steps whose B request (and A request of position + 2) are out
    auto issue_step = [&]() {
        issue_a(a_wr); a_wr = next(a_wr, RING);
        issue_b(b_wr); b_wr = next(b_wr, BST);
        issued++;
    };
    if (nsteps > 0) {
        // refill: A positions i_begin - 2 * WS .. i_begin + 1, then LEAD whole steps
#pragma unroll 1
        for (int l = 0; l < 2 * WS + 2; l++) { issue_a(a_wr); a_wr = next(a_wr, RING); }
#pragma unroll
        for (int l = 0; l < LEAD; l++)
            if (issued < nsteps) issue_step();
    }
    for (int j = 0; j < nsteps; j++) {
        // the requests of step j have landed (those of later steps may still be in flight:
        // vector-memory operations complete in issue order), and nobody still reads what the
        // next requests overwrite (the oldest slot, the stage of step j-1)
        if (LEAD > 1 && issued - j - 1 >= LEAD - 1) {
            if (loads_a) __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(LEAD - 1) * 1>::IMM);
            else         __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(LEAD - 1) * 2>::IMM);
        } else {
            __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
        }
        __syncthreads();
        if (issued < nsteps) issue_step();
        const bool multiply = (cw.strip < g.strips) & (cw.yy >= 0) & (cw.xs < WT) & (cw.strip * WT + cw.xs < g.W);
        if (multiply) {
            const char* bt = smem + A_BYTES + b_rd * TB::BYTES;
            const int a1 = next(a_rd, RING), a2 = next(a1, RING);
            const char* at[TAPS] = {smem + a_rd * TA::BYTES, smem + a1 * TA::BYTES, smem + a2 * TA::BYTES};
#pragma unroll
            for (int kk = 0; kk < N / 16; kk++) {
                const Frag<T> b = FB::load(bt, fb_base, kk);
#pragma unroll
                for (int t = 0; t < TAPS; t++) {
                    const Frag<T> a = FA::load(at[t], fa_base, kk);
                    mfma_step(a, b, acc[t][0]);
                }
            }
        }
        a_rd = next(a_rd, RING); b_rd = next(b_rd, BST);
        advance(cw);
    }

    __syncthreads();
    char* stage = smem + wave * EPI_BYTES;
    // band s of this wavefront holds filter rows ((cb * 32 + i) * 3 + rtap) * 3 + s
    EpilogueBands<TAPS, 1, WTN, EPITCH, 0, TAPS, 3>::run(acc, stage, lane, cb * 96 + rtap, wn * WTN, 0, split, epi);
}

}  // namespace ng
