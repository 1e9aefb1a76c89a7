// Weight gradient of filters with three horizontal taps, unit strides and few output
// maps (at most 128): the taps share their activations.
//
// gF[(c,t,r,s)][k] = sum over output pixels (m,p,q) and images n of
//                    I[c, m+t-pad_d, p+r-pad_h, q+s-1, n] * E[k, m, p, q, n].
// The kernel of gemm_core.h with a gathered A operand fetches, for every output pixel,
// one 128-byte run of I per filter row (c,t,r,s): three runs per (c,t,r), and the run of
// tap s at pixel q is the run of tap s+1 at pixel q-1.  With 64 or 128 columns of E per
// tile the CU's vector-memory path (64 bytes a clock) then is what the kernel waits for
// (VGG conv1.2: 32 KB requested per 48 MFMAs).  Here a workgroup owns CRB rows (c,t,r) and
// all three taps of each, walks along the image rows, and keeps the input pixels in a
// ring of LDS slots: a step requests ONE new input pixel (CRB rows x 128 bytes) and one
// pixel of E, and multiplies E(q) with the slots of the input pixels q-1, q, q+1 into the
// accumulators of taps 0, 1, 2.
//
// Walk: positions i = row * (W+2) + x over the output rows (m,p), x = 0 .. W+1.  The A
// stream holds input pixel x-1 at position i (x-1 = -1 and x-1 = W are the zero padding),
// the B stream output pixel q = x (x >= W: nothing, the step only moves the ring).  Tap s
// of step i reads A position i+s.  A contraction slice is a range of positions.
#pragma once
#include "conv_plan.h"

namespace ng {

struct UpdateRingGeom {
    const _Float16* I;
    const _Float16* E;
    int CR;             // rows (c,t,r)
    int TR, R;          // T*R, R
    int D, H, W;        // input extents
    int MP, P;          // output rows M*P, P (output row length Q == W)
    int pad_d, pad_h;
    int K;
    int chan_stride;    // elements between channels of I: D*H*W*N
    int kdim;           // row length of E: M*P*Q*N
    int steps;          // M*P*(W+2)
    FastDiv tr_div, r_div, w2_div, p_div;
};

// CRB rows (c,t,r) per workgroup (32 per wavefront row), BN columns on two wavefront columns;
// LEAD: steps a request is issued ahead of its use (ring of 3 + LEAD slots, 1 + LEAD stages of E)
template <int CRB, int BN, int LEAD, class Epi>
__global__ __launch_bounds__(CRB / 32 * 2 * 64)
void conv_update_ring_kernel(UpdateRingGeom g, Epi epi, CoreShape s)
{
    typedef _Float16 T;
    constexpr int N = 64;                          // images per pixel = contraction elements per step
    constexpr int WM = CRB / 32, WN = 2, NT = WM * WN * 64, TAPS = 3, RING = TAPS + LEAD, BST = 1 + LEAD;
    constexpr int TN = BN / WN / 32;
    using TA = SwizzledTile<T, KC, CRB, N>;        // one input pixel: 64 rows x 128 bytes
    using TB = SwizzledTile<T, KC, BN, N>;         // one pixel of E: BN rows x 128 bytes
    using FA = SwizzledFrag<KC, TA>;
    using FB = SwizzledFrag<KC, TB>;
    constexpr int CPT_A = TA::CHUNKS / NT;
    // the chunks of E may not cover all wavefronts in the last round (768 threads on 512 chunks)
    constexpr int CPT_B = (TB::CHUNKS + NT - 1) / NT;
    static_assert(TA::CHUNKS % NT == 0 && TB::CHUNKS % 64 == 0, "tile chunks must divide evenly over threads / wavefronts");
    static_assert(SwizzledTile<T, KC, CRB, N>::BYTES * (TAPS + LEAD) + SwizzledTile<T, KC, BN, N>::BYTES * (1 + LEAD) <= 160 * 1024, "ring exceeds the LDS");
    constexpr int A_BYTES = RING * TA::BYTES, B_BYTES = BST * TB::BYTES;
    constexpr int WTN = BN / WN;
    constexpr int EPITCH = WTN * 4 + 16;
    constexpr int EPI_BYTES = 32 * EPITCH;
    constexpr int SMEM_BYTES = (A_BYTES + B_BYTES > EPI_BYTES * WM * WN) ? A_BYTES + B_BYTES : EPI_BYTES * WM * WN;
    __shared__ __attribute__((aligned(16))) char smem[SMEM_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    int tm, tn, split;
    if (!block_work(s, tm, tn, split)) return;
    const int cr0 = tm * CRB, n0 = tn * BN;
    const int per = (g.steps + s.splits - 1) / s.splits;
    const int i_begin = split * per;
    const int i_end = min(i_begin + per, g.steps);

    // A chunks of this lane: row (c,t,r) and image offset; what of the address does not move with the walk
    int a_base[CPT_A], a_dz[CPT_A], a_dy[CPT_A];
#pragma unroll
    for (int i = 0; i < CPT_A; i++) {
        int r, k;
        TA::chunk_pos(tid + i * NT, r, k);
        const int cr = cr0 + r;
        const int crc = min(cr, g.CR - 1);          // rows past the filter decode as the last row (never read)
        const int c = (int)g.tr_div.div((unsigned)crc), tr = crc - c * g.TR;
        const int t = (int)g.r_div.div((unsigned)tr), rf = tr - t * g.R;
        a_dz[i] = (cr < g.CR) ? t - g.pad_d : (1 << 20);       // rows past the filter never pass the range test
        a_dy[i] = rf - g.pad_h;
        a_base[i] = c * g.chan_stride + ((t - g.pad_d) * g.H + (rf - g.pad_h)) * g.W * N + k;
    }
    unsigned b_off[CPT_B];
#pragma unroll
    for (int i = 0; i < CPT_B; i++) {
        int r, k;
        TB::chunk_pos(min(tid + i * NT, TB::CHUNKS - 1), r, k);
        b_off[i] = (n0 + r < g.K) ? ((unsigned)(n0 + r) * (unsigned)g.kdim + (unsigned)k) * 2u : NG_OOB_OFFSET;
    }
    // whether this wavefront takes part in the last round of E requests (wavefront-uniform)
    const bool b_last = (CPT_B - 1) * NT + wave * 64 < TB::CHUNKS;
    const BufferRsrc a_rsrc = make_rsrc(g.I), b_rsrc = make_rsrc(g.E);

    // walkers (wavefront-uniform): the A stream runs three positions ahead of the B stream
    const int W2 = g.W + 2;
    int a_row = (int)g.w2_div.div((unsigned)i_begin), a_x = i_begin - a_row * W2;
    int b_row = a_row, b_x = a_x;         // next position to request
    int c_x = a_x;                        // position being multiplied
    bool a_ok[CPT_A];
    int a_rowbase = 0;
    auto a_enter_row = [&]() {
        const int m = (int)g.p_div.div((unsigned)a_row), p = a_row - m * g.P;
        a_rowbase = (m * g.H + p) * g.W * N;
#pragma unroll
        for (int i = 0; i < CPT_A; i++)
            a_ok[i] = (a_row < g.MP) & ((unsigned)(m + a_dz[i]) < (unsigned)g.D) & ((unsigned)(p + a_dy[i]) < (unsigned)g.H);
    };
    a_enter_row();
    auto issue_a = [&](int slot) {
        const int xin = a_x - 1;
        const bool xok = (unsigned)xin < (unsigned)g.W;
        const int pix = a_rowbase + xin * N;
#pragma unroll
        for (int i = 0; i < CPT_A; i++) {
            const unsigned off = (a_ok[i] & xok) ? (unsigned)(a_base[i] + pix) * 2u : NG_OOB_OFFSET;
            buffer_load_chunk_to_lds(a_rsrc, smem + slot * TA::BYTES + (i * NT + wave * 64) * 16, off);
        }
        if (++a_x == W2) { a_x = 0; a_row++; a_enter_row(); }
    };
    auto issue_b = [&](int stage) {
        const bool ok = (b_x < g.W) & (b_row < g.MP);
        const unsigned pix = (unsigned)(b_row * g.W + b_x) * (unsigned)(N * 2);
#pragma unroll
        for (int i = 0; i < CPT_B; i++) {
            const unsigned off = (ok & (b_off[i] != NG_OOB_OFFSET)) ? b_off[i] + pix : NG_OOB_OFFSET;
            if (i + 1 < CPT_B || b_last)
                buffer_load_chunk_to_lds(b_rsrc, smem + A_BYTES + stage * TB::BYTES + (i * NT + wave * 64) * 16, off);
        }
        if (++b_x == W2) { b_x = 0; b_row++; }
    };

    float16_t acc[TAPS][TN];
#pragma unroll
    for (int t = 0; t < TAPS; t++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[t][j][v] = 0.0f;

    const int fa_base = FA::base(wm, lane);
    int fb_base[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) fb_base[j] = FB::base(wn * TN + j, lane);

    const int nsteps = i_end - i_begin;
    // slot / stage indices advance by counters (the ring lengths are not powers of two)
    auto next = [](int v, int n) { return v + 1 == n ? 0 : v + 1; };
    int a_wr = 0, b_wr = 0;         // where the next requests go
    int a_rd = 0, b_rd = 0;         // slot of position i, stage of step i
    int issued = 0;                 // steps whose B request (and A request of position + 2) are out
    auto issue_step = [&]() {
        issue_a(a_wr); a_wr = next(a_wr, RING);
        issue_b(b_wr); b_wr = next(b_wr, BST);
        issued++;
    };
    if (nsteps > 0) {
        issue_a(a_wr); a_wr = next(a_wr, RING);
        issue_a(a_wr); a_wr = next(a_wr, RING);
#pragma unroll
        for (int l = 0; l < LEAD; l++)
            if (issued < nsteps) issue_step();
    }
    constexpr int PER_STEP = CPT_A + CPT_B;
    for (int j = 0; j < nsteps; j++) {
        // the requests of step j have landed (those of later steps may still be in flight:
        // vector-memory operations complete in issue order), and nobody still reads what the
        // next requests overwrite (the slot of position j-1, the stage of step j-1)
        if (LEAD > 1 && issued - j - 1 >= LEAD - 1) {
            if (b_last) __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(LEAD - 1) * PER_STEP>::IMM);
            else        __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(LEAD - 1) * (PER_STEP - 1)>::IMM);
        } else {
            __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
        }
        __syncthreads();
        if (issued < nsteps) issue_step();
        if (c_x < g.W) {
            const char* bt = smem + A_BYTES + b_rd * TB::BYTES;
            const int a1 = next(a_rd, RING), a2 = next(a1, RING);
            const char* at[TAPS] = {smem + a_rd * TA::BYTES, smem + a1 * TA::BYTES, smem + a2 * TA::BYTES};
#pragma unroll
            for (int kk = 0; kk < N / 16; kk++) {
                Frag<T> b[TN];
#pragma unroll
                for (int jn = 0; jn < TN; jn++) b[jn] = FB::load(bt, fb_base[jn], kk);
#pragma unroll
                for (int t = 0; t < TAPS; t++) {
                    const Frag<T> a = FA::load(at[t], fa_base, kk);
#pragma unroll
                    for (int jn = 0; jn < TN; jn++) mfma_step(a, b[jn], acc[t][jn]);
                }
            }
        }
        a_rd = next(a_rd, RING); b_rd = next(b_rd, BST);
        if (++c_x == W2) c_x = 0;
    }

    __syncthreads();
    char* stage = smem + wave * EPI_BYTES;
    EpilogueBands<TAPS, TN, WTN, EPITCH, 0, TAPS>::run(acc, stage, lane, cr0 + wm * 32, n0 + wn * WTN, 0, split, epi);
}

}  // namespace ng
