// Streaming contraction kernel for problems whose A operand is tiny (a first
// layer's filter: at most 64 rows, a few contraction tiles) and whose B operand
// and output are long streams of columns.
//
// The generic core gives such a problem one workgroup per column tile whose life
// is: wait for the gathered tile, a handful of MFMAs, store the tile.  Nothing
// overlaps inside a workgroup, and with two or three resident per CU little
// overlaps between them: gather time and store time add up (VGG conv1.1 forward:
// 61 us without the stores, 88 us without the gathers, 164 us with both).
//
// Here a workgroup owns a contiguous run of column tiles.  The whole A operand
// is read once into registers as MFMA fragments; the B tiles of all its column
// tiles form one stream that runs through a ring of NSTAGE LDS stages without
// draining between column tiles, so the requests of the next column tiles are in
// flight while the current one is multiplied and stored.
#pragma once

#include "gemm_core.h"

#include <algorithm>

namespace ng {

// rows of the fp32 tile a whole-tile epilogue wants parked in LDS (it declares MAX_ROWS)
template <class E, class = void> struct EpilogueStagedRows { static constexpr int value = 32; };
template <class E> struct EpilogueStagedRows<E, std::enable_if_t<(E::MAX_ROWS > 0)>> { static constexpr int value = E::MAX_ROWS; };

// f(std::integral_constant<int, I>) for I = BEGIN .. END-1, unrolled at compile time
template <int BEGIN, int END, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}

// A gather whose contraction rows differ only by a uniform stride inside a tile
// declares `static constexpr bool FIXED_PER_TILE = true`, Fixed fixed(first row of
// the tile) and offset(Fixed, row inside the tile, Col): one Fixed per contraction
// tile is kept (in scalar registers) instead of one per request.
template <class G, class = void> struct GatherFixedPerTile { static constexpr bool value = false; };
template <class G> struct GatherFixedPerTile<G, std::enable_if_t<G::FIXED_PER_TILE>> { static constexpr bool value = true; };

// A gather that derives what a contraction row contributes from the row number alone, with a few
// operations on the scalar unit, declares `static constexpr bool FIXED_ON_DEMAND = true` and
// Fixed fixed(row), offset(Fixed, Col): nothing is kept per contraction tile, so the tiles may be
// many (the 363 filter rows of an 11x11 first layer).  A line of its tiles must be one wavefront
// request, so that the row is uniform.
template <class G, class = void> struct GatherFixedOnDemand { static constexpr bool value = false; };
template <class G> struct GatherFixedOnDemand<G, std::enable_if_t<G::FIXED_ON_DEMAND>> { static constexpr bool value = true; };

template <class E, class = void> struct StoresPerThread { static constexpr int value = 0; };
template <class E> struct StoresPerThread<E, std::enable_if_t<(E::STORES_PER_THREAD > 0)>> { static constexpr int value = E::STORES_PER_THREAD; };

// iterations p in [kt - d, kt - 1] (contraction tile index modulo kt_count) that
// end a column tile, i.e. ran an epilogue
constexpr int epilogues_in_window(int kt, int d, int kt_count)
{
    int n = 0;
    for (int p = kt - d; p < kt; p++) n += (((p % kt_count) + kt_count) % kt_count == kt_count - 1) ? 1 : 0;
    return n;
}

// EpilogueBands with descriptor stores: one 32-row band of a wavefront's
// accumulators through its private LDS staging; every lane stores every piece.
// SR: the epilogue's store may round stochastically (store8_buffer_sr); row0 is the
// first row of the workgroup's row block
template <int TM, int TN, int WTN, int EPITCH, int I, bool SR = false>
struct StreamBands {
    template <class Epi>
    static __device__ __forceinline__ void run(float16_t (&acc)[TM][TN], char* stage, int lane, int nbase,
                                               BufferRsrc rsrc, const Epi& epi, int row0 = 0)
    {
        constexpr int CPW = 32 * WTN / 8;
        static_assert(CPW % 64 == 0, "a band must be whole store instructions");
        const int col = lane & 31;
        const int rsub = (lane >> 5) * 4;
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                *reinterpret_cast<float*>(stage + ((v >> 2) * 8 + rsub + (v & 3)) * EPITCH + (j * 32 + col) * 4) =
                    acc[I][j][v];
        wave_lds_fence();
#pragma unroll
        for (int c = 0; c < CPW / 64; c++) {
            const int id = lane + c * 64;
            const int r = id / (WTN / 8);
            const int cc = (id % (WTN / 8)) * 8;
            const float4_t lo = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4);
            const float4_t hi = *reinterpret_cast<const float4_t*>(stage + r * EPITCH + cc * 4 + 16);
            const float vals[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            if constexpr (SR) epi.store8_buffer_sr(rsrc, row0 + I * 32 + r, nbase + cc, 0, vals);
            else              epi.store8_buffer(rsrc, row0 + I * 32 + r, nbase + cc, vals);
        }
        wave_lds_fence();
        if constexpr (I + 1 < TM) StreamBands<TM, TN, WTN, EPITCH, I + 1, SR>::run(acc, stage, lane, nbase, rsrc, epi, row0);
    }
};

// B operand of the streaming kernel.  A gather functor supplies
//   Fixed fixed(j)       what contraction row j contributes (constant per thread
//                        and contraction tile: kept in registers for the whole run)
//   Col   col(c)         what virtual column c contributes (once per column tile)
//   unsigned offset(Fixed, Col)   byte offset of the chunk, NG_OOB_OFFSET for zeros
//   const T* X           the tensor
//
// LB: layout of the B tiles in LDS (MC: columns contiguous, the gathered activations
// of a convolution; KC: contraction contiguous, the rows of a dense matrix).
// gridDim.y > 1: blockIdx.y numbers blocks of BM rows of A and of the output, each
// with its own run of workgroups along the columns (a dense product with a short
// contraction: the rows of A stay in registers, the rows of B stream).
// SR: the store may round stochastically (the epilogue's store8_buffer_sr).
template <typename T, int BM, int BN, int BK, int WN, int KT, int LA, int NSTAGE, class ALoad, class BGather, class Epi,
          int LB = MC, bool SR = false>
__global__ __launch_bounds__(WN * 64)
void mfma_stream_kernel(ALoad aload, BGather bg, Epi epi, int tiles)
{
    static_assert(sizeof(T) == 2 && ALoad::DIRECT, "16-bit operands through direct LDS loads");
    static_assert(NSTAGE >= 2 && KT >= 1, "need two stages and one contraction tile");
    constexpr int NT = WN * 64;
    constexpr int KSTEP = Elem<T>::KSTEP;
    constexpr int KS = BK / KSTEP;
    constexpr int TM = BM / 32, TN = BN / WN / 32, WTN = BN / WN;
    using TA = SwizzledTile<T, LA, BM, BK>;
    using TB = SwizzledTile<T, LB, BN, BK>;
    using FA = SwizzledFrag<LA, TA>;
    using FB = SwizzledFrag<LB, TB>;
    constexpr int CPT_B = TB::CHUNKS / NT;
    static_assert(TB::CHUNKS % NT == 0, "B tile chunks must divide evenly over threads");
    static_assert(TA::CHUNKS % 64 == 0 && TA::BYTES <= NSTAGE * TB::BYTES, "A tile is staged through the ring, wavefront by wavefront");
    static_assert(BM % 32 == 0 && BN % (WN * 32) == 0 && BK % KSTEP == 0, "bad tile shape");
    constexpr bool WHOLE = EpilogueWholeTile<Epi>::value;
    static_assert(!WHOLE || BM == 32, "whole-tile epilogues take one block of 32 rows");
    static_assert(!WHOLE || !SR, "whole-tile epilogues round to nearest");
    constexpr int EPITCH = WTN * 4 + 16;
    constexpr int EPI_BYTES = 32 * EPITCH;
    // a whole-tile epilogue parks its rows in the ring stage that was just multiplied
    // (free until the request behind the next barrier), so it needs no LDS of its own
    constexpr int EPI_REGION = WHOLE ? 0 : EPI_BYTES * WN;
    static_assert(!WHOLE || EpilogueStagedRows<Epi>::value * BN * 4 <= TB::BYTES, "parked rows must fit one ring stage");
    constexpr int RING = NSTAGE * TB::BYTES;
    static_assert(RING + EPI_REGION <= 160 * 1024, "ring and epilogue staging exceed the LDS of a compute unit");
    __shared__ __attribute__((aligned(16))) char smem[RING + EPI_REGION];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // contiguous share of the column tiles (uniform over the workgroup)
    const int per = (tiles + (int)gridDim.x - 1) / (int)gridDim.x;
    const int first = (int)blockIdx.x * per;
    const int count = min(per, tiles - first);
    if (count <= 0) return;
    const int m0 = (int)blockIdx.y * BM;    // first row of this workgroup's block of A

    // ---- A: every contraction tile once through LDS into fragments ----
    Frag<T> fa[KT][KS][TM];
    int fa_base[TM];
#pragma unroll
    for (int i = 0; i < TM; i++) fa_base[i] = FA::base(i, lane);
    const typename ALoad::Wave a_wave = aload.wave_init(lane);
#pragma unroll
    for (int kt = 0; kt < KT; kt++) {
        const typename ALoad::Tile ta = aload.tile(kt, kt * BK, 0, a_wave);
#pragma unroll
        for (int i = 0; i * NT < TA::CHUNKS; i++) {
            if (i * NT + wave * 64 < TA::CHUNKS) {   // uniform over the wavefront
                int r, k;
                TA::chunk_pos(tid + i * NT, r, k);
                buffer_load_chunk_to_lds(ta.rsrc, smem + (i * NT + wave * 64) * 16, aload.offset(ta, aload.prepare(m0 + r, k)));
            }
        }
        __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
        __syncthreads();
#pragma unroll
        for (int st = 0; st < KS; st++)
#pragma unroll
            for (int i = 0; i < TM; i++) fa[kt][st][i] = FA::load(smem, fa_base[i], st);
        __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
        __syncthreads();
    }

    // ---- B stream ----
    constexpr bool PER_TILE = GatherFixedPerTile<BGather>::value;
    constexpr bool ON_DEMAND = GatherFixedOnDemand<BGather>::value;
    static_assert(!(PER_TILE || ON_DEMAND) || TB::CPR == 64, "a tile line must be one wavefront request for its row to be uniform");
    static_assert(!(ON_DEMAND && PER_TILE), "one or the other");
    int rc[CPT_B], kc[CPT_B];
    typename BGather::Fixed fx[ON_DEMAND ? 1 : KT][(PER_TILE || ON_DEMAND) ? 1 : CPT_B];
#pragma unroll
    for (int c = 0; c < CPT_B; c++) {
        int k;
        TB::chunk_pos(tid + c * NT, rc[c], k);
        kc[c] = (PER_TILE || ON_DEMAND) ? __builtin_amdgcn_readfirstlane(k) : k;
        if constexpr (!PER_TILE && !ON_DEMAND) {
#pragma unroll
            for (int kt = 0; kt < KT; kt++) fx[kt][c] = bg.fixed(kt * BK + k);
        }
    }
    if constexpr (PER_TILE) {
#pragma unroll
        for (int kt = 0; kt < KT; kt++) fx[kt][0] = bg.fixed(kt * BK);
    }
    const BufferRsrc rsrc = make_rsrc(bg.X);
    typename BGather::Col col[CPT_B];
    int wr_off = 0;   // ring stage (byte offset) the next request goes to
    // request contraction tile `ktn` of this workgroup's column tile `in`
    auto issue = [&](int in, int ktn) {
        if (in < count) {
            if (ktn == 0) {
#pragma unroll
                for (int c = 0; c < CPT_B; c++) col[c] = bg.col((first + in) * BN + rc[c]);
            }
#pragma unroll
            for (int c = 0; c < CPT_B; c++) {
                unsigned off = NG_OOB_OFFSET;
#pragma unroll
                for (int q = 0; q < KT; q++)
                    if (q == ktn) {
                        if constexpr (ON_DEMAND)     off = bg.offset(bg.fixed(q * BK + kc[c]), col[c]);   // q is a constant here
                        else if constexpr (PER_TILE) off = bg.offset(fx[q][0], kc[c], col[c]);
                        else                    off = bg.offset(fx[q][c], col[c]);
                    }
                buffer_load_chunk_to_lds(rsrc, smem + wr_off + (c * NT + wave * 64) * 16, off);
            }
        }
        wr_off = (wr_off + TB::BYTES == RING) ? 0 : wr_off + TB::BYTES;
    };

    float16_t acc[TM][TN];
    auto clear = [&]() {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
    };
    clear();
    int fb_base[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) fb_base[j] = FB::base(wave * TN + j, lane);

    // D tiles of the stream are requested ahead of the one being multiplied
    constexpr int D = NSTAGE - 1;
    // store instructions every wavefront issues per epilogue
    constexpr int NS = WHOLE ? StoresPerThread<Epi>::value : TM * (32 * WTN / 8 / 64);
    static_assert((D - 1) * CPT_B + NS * D < 64, "the vector-memory counter holds 63 operations");
    static_assert(!WHOLE || NT == 256, "whole-tile epilogues are laid out for 256 threads");
    const BufferRsrc out_rsrc = make_rsrc(epi.base());
#pragma unroll
    for (int q = 0; q < D; q++) issue(q / KT, q % KT);

    const int total = count * KT;
    int rd_off = 0, q = 0;
    for (int i = 0; i < count; i++) {
        static_for<0, KT>([&](auto kt_c) {
            constexpr int kt = decltype(kt_c)::value;
            // Tile q has landed when at most the vector-memory operations issued
            // after its requests are outstanding (they complete in issue order):
            // the requests of D-1 tiles and the stores of the epilogues that ran
            // in the last D iterations, a number fixed by kt because every
            // wavefront issues exactly NS store instructions per epilogue.  The
            // first D iterations have run fewer epilogues and count the requests
            // only, which waits longer than needed but never too little.
            constexpr int EPILOGUES = epilogues_in_window(kt, D, KT);
            if (q + D - 1 >= total) __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<0>::IMM);
            else if (q < D)         __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(D - 1) * CPT_B>::IMM);
            else                    __builtin_amdgcn_s_waitcnt(WaitVmLgkm0<(D - 1) * CPT_B + NS * EPILOGUES>::IMM);
            __syncthreads();
            // behind the barrier nobody reads the stage of tile q-1 any more
            issue(i + (kt + D) / KT, (kt + D) % KT);
            const int stage_off = rd_off;
            const char* tile = smem + stage_off;
#pragma unroll
            for (int st = 0; st < KS; st++) {
                Frag<T> fb[TN];
#pragma unroll
                for (int j = 0; j < TN; j++) fb[j] = FB::load(tile, fb_base[j], st);
#pragma unroll
                for (int m = 0; m < TM; m++)
#pragma unroll
                    for (int j = 0; j < TN; j++) mfma_step(fa[kt][st][m], fb[j], acc[m][j]);
            }
            rd_off = (rd_off + TB::BYTES == RING) ? 0 : rd_off + TB::BYTES;
            if (kt == KT - 1) {
                const int n0 = (first + i) * BN;
                if constexpr (WHOLE) {
                    float* g = reinterpret_cast<float*>(smem + stage_off);
                    const int nrows = epi.rows;
                    __syncthreads();   // every wavefront is done with the fragments of this stage
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int v = 0; v < 16; v++) {
                            const int row = (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                            if (row < nrows) g[row * BN + wave * WTN + j * 32 + (lane & 31)] = acc[0][j][v];
                        }
                    __syncthreads();
                    epi.tile_buffer(out_rsrc, g, tid, n0);
                    // the stage is requested into again behind the next barrier, which every
                    // thread reaches only after it has read the parked rows
                } else {
                    StreamBands<TM, TN, WTN, EPITCH, 0, SR>::run(acc, smem + RING + wave * EPI_BYTES, lane, n0 + wave * WTN, out_rsrc, epi, m0);
                }
                clear();
            }
            q++;
        });
    }
}

// `wgs_per_cu`: workgroups of this shape that fit a CU; the grid is that many per
// CU (or one per column tile if there are fewer)
template <typename T, int BM, int BN, int BK, int WN, int KT, int LA, int NSTAGE, class AL, class BG, class Epi>
inline void launch_stream(const AL& al, const BG& bg, const Epi& epi, int tiles, int wgs_per_cu, hipStream_t stream)
{
    const int grid = std::min(tiles, device_cu_count() * wgs_per_cu);
    hipLaunchKernelGGL((mfma_stream_kernel<T, BM, BN, BK, WN, KT, LA, NSTAGE, AL, BG, Epi>), dim3(grid), dim3(WN * 64), 0,
                       stream, al, bg, epi, tiles);
}

// the dense form: `row_blocks` blocks of BM rows (blockIdx.y), `col_groups` workgroups
// sharing the column tiles of each
template <typename T, int BM, int BN, int BK, int WN, int KT, int LA, int LB, int NSTAGE, bool SR, class AL, class BG, class Epi>
inline void launch_stream_rows(const AL& al, const BG& bg, const Epi& epi, int tiles, int row_blocks, int col_groups,
                               hipStream_t stream)
{
    hipLaunchKernelGGL((mfma_stream_kernel<T, BM, BN, BK, WN, KT, LA, NSTAGE, AL, BG, Epi, LB, SR>),
                       dim3((unsigned)col_groups, (unsigned)row_blocks), dim3(WN * 64), 0, stream, al, bg, epi, tiles);
}

}  // namespace ng
