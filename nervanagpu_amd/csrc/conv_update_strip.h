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
// Walk: a strip has H + 2 rows yy = -2 .. H-1 (the two rows before the image fill the
// ring; their steps multiply nothing) of WS = WT + 2 positions xs.  Strip row
// gr = strip * (H + 2) + yy + 2, position p = gr * WS + xs.  The A stream holds input pixel
// (row yy + 1, column x0 + xs - 1) at position p (rows -1 and H and columns -1 and W are
// the zero padding); the B stream holds output pixel (yy, x0 + xs) for yy >= 0, xs < WT
// (else nothing: the step only moves the ring).  Tap (r,s) of step p reads A position
// p + s - (2 - r) * WS.  A contraction slice is a range of strip rows; the loop starts three
// rows early with the products switched off, which refills the ring.
//
// Everything that depends on the strip row (addresses, which positions exist) is decoded
// once per row on the scalar unit into an offset and a bit mask per stream; the WS steps of
// a row are unrolled, so what depends on xs is a compile-time constant: twelve wavefronts
// repeat the scalar part of a step, and it has to stay well below the 12 MFMAs of the step.
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
    int rows;           // strip rows: strips * (H + 2)
    FastDiv rows_div;   // by H + 2
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
    constexpr int WM = 6, WN = 2;                  // wavefront rows: (channel block, vertical tap)
    constexpr int A_LEAD = 2 + LEAD;               // positions the A stream runs ahead of the step
    constexpr int RING = 2 * WS + TAPS + LEAD, BST = 1 + LEAD;
    static_assert(WS % BST == 0, "the stage of E of a step is a constant of its xs");
    static_assert(A_LEAD < WS, "requests reach into the next strip row at most");
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
    const int per = (g.rows + s.splits - 1) / s.splits;
    const int r_begin = split * per;
    const int r_end = min(r_begin + per, g.rows);

    // wavefronts 0..7 request the input pixel (one chunk a lane), 8..11 the pixel of E (two)
    const bool loads_a = wave < 8;
    unsigned a_lane = 0;     // lane part of the byte offset: channel and image chunk
    bool a_valid = false;
    unsigned b_lane[2] = {NG_OOB_OFFSET, NG_OOB_OFFSET};
    if (loads_a) {
        int r, k;
        TA::chunk_pos(tid, r, k);
        a_valid = r < g.C;
        a_lane = (unsigned)(min(r, g.C - 1) * g.chan_stride + k) * 2u;
    } else {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            int r, k;
            TB::chunk_pos((tid - 512) + i * 256, r, k);
            b_lane[i] = (r < g.K) ? ((unsigned)r * (unsigned)g.kdim + (unsigned)k) * 2u : NG_OOB_OFFSET;
        }
    }
    const BufferRsrc a_rsrc = make_rsrc(g.I), b_rsrc = make_rsrc(g.E);

    // one strip row, decoded on the scalar unit: byte offset of position xs = 0 and the
    // positions that exist, for the A stream (input pixels) and the B stream (pixels of E)
    struct Row { unsigned a_off, a_mask, b_off, b_mask; };
    auto decode = [&](int gr) {
        Row r{0u, 0u, 0u, 0u};
        if (gr < 0 || gr >= g.rows) return r;
        const int st = (int)g.rows_div.div((unsigned)gr);
        const int yy = gr - st * (g.H + 2) - 2;
        const int x0 = st * WT;
        if ((unsigned)(yy + 1) < (unsigned)g.H) {
            // column x0 - 1 + xs: not before the image (strip 0, xs = 0), not past it
            const int hi = min(WS, g.W - x0 + 1);
            r.a_mask = ((1u << hi) - 1u) & (x0 == 0 ? ~1u : ~0u);
            r.a_off = (unsigned)(((yy + 1) * g.W + x0 - 1) * N) * 2u;      // of xs = 0; wraps below zero for x0 = 0, where xs = 0 is masked
        }
        if (yy >= 0 && gr >= r_begin && gr < r_end) {
            r.b_mask = (1u << min(WT, g.W - x0)) - 1u;
            r.b_off = (unsigned)((yy * g.W + x0) * N) * 2u;
        }
        return r;
    };

    float16_t acc[TAPS][1];
#pragma unroll
    for (int t = 0; t < TAPS; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][0][v] = 0.0f;

    const int fa_base = FA::base(cb, lane);
    const int fb_base = FB::base(wn, lane);

    // Ring slots as byte offsets.  The first request (made at the first step, for the position
    // A_LEAD ahead) goes to slot 0, so the slot of tap (rtap, 0) of the first step is
    // -A_LEAD - (2 - rtap) * WS modulo the ring; it only matters once real rows are multiplied.
    auto wrap = [](int off) { return off + TA::BYTES == A_BYTES ? 0 : off + TA::BYTES; };
    int a_wr = 0;
    int rd0 = (((-A_LEAD - (2 - rtap) * WS) % RING + RING) % RING) * TA::BYTES;
    int rd1 = wrap(rd0), rd2 = wrap(rd1);

    Row cur = decode(r_begin - 3);
    for (int gr = r_begin - 3; gr < r_end; gr++) {
        const Row nxt = decode(gr + 1);
#pragma unroll
        for (int xs = 0; xs < WS; xs++) {
            // the requests of this step have landed (those of the next LEAD - 1 steps may still be in
            // flight: vector-memory operations complete in issue order), and nobody still reads what
            // the next requests overwrite (the oldest slot, the stage of the previous step)
            if (loads_a) __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(LEAD - 1) * 1>::IMM);
            else         __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(LEAD - 1) * 2>::IMM);
            __syncthreads();
            if (loads_a) {
                const int xa = (xs + A_LEAD) % WS;       // constants once the loop is unrolled
                const Row& r = (xs + A_LEAD < WS) ? cur : nxt;
                const bool ok = (r.a_mask >> xa) & 1u;
                const unsigned off = (ok & a_valid) ? a_lane + r.a_off + (unsigned)(xa * N * 2) : NG_OOB_OFFSET;
                buffer_load_chunk_to_lds(a_rsrc, smem + a_wr + (wave * 64) * 16, off);
            } else {
                const int xb = (xs + LEAD) % WS;
                const Row& r = (xs + LEAD < WS) ? cur : nxt;
                const bool ok = (r.b_mask >> xb) & 1u;
                const unsigned pix = r.b_off + (unsigned)(xb * N * 2);
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const unsigned off = (ok & (b_lane[i] != NG_OOB_OFFSET)) ? b_lane[i] + pix : NG_OOB_OFFSET;
                    // chunk (wave - 8) * 64 + lane + i * 256: the hardware adds 16 * lane to the wavefront's base
                    buffer_load_chunk_to_lds(b_rsrc, smem + A_BYTES + (xb % BST) * TB::BYTES + ((i * 4 + (wave - 8)) * 64) * 16, off);
                }
            }
            a_wr = wrap(a_wr);
            if ((cur.b_mask >> xs) & 1u) {
                const char* bt = smem + A_BYTES + (xs % BST) * TB::BYTES;
                const char* at[TAPS] = {smem + rd0, smem + rd1, smem + rd2};
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
            rd0 = rd1; rd1 = rd2; rd2 = wrap(rd2);
        }
        cur = nxt;
    }

    // requests of the last steps (positions past the slice) may still be landing in the ring
    __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
    __syncthreads();
    char* stage = smem + wave * EPI_BYTES;
    // band s of this wavefront holds filter rows ((cb * 32 + i) * 3 + rtap) * 3 + s
    EpilogueBands<TAPS, 1, WTN, EPITCH, 0, TAPS, 3>::run(acc, stage, lane, cb * 96 + rtap, wn * WTN, 0, split, epi);
}

}  // namespace ng
