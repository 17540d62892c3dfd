// Tile kernels, epilogues and launch logic of the MFMA GEMM, shared by the two translation units that
// instantiate them: gemm.hip (ptj_gemm: every operand layout, bias / GELU epilogues, K splits) and
// gemm_mul.hip (ptj_gemm_mul_colsum: the multiplying epilogue with column sums).  Everything here lives in
// an unnamed namespace, so each unit gets its own copy of what it uses; the two units compile side by side.
//
// MFMA GEMM for gfx950: C[n,m] = sum_k A(n,k) B(k,m) (+bias[m]) (gelu), fp32 accumulation.
//
// Tiling: one 512-thread workgroup (8 wavefronts, 4 along rows x 2 along columns) owns a
// 256x192 tile of C; each wavefront owns 64x96 = 2x3 MFMA tiles of 32x32
// (v_mfma_f32_32x32x16_bf16, or four v_mfma_f32_32x32x2_f32 per step for fp32 storage).
// 192 divides every feature width of the model (768, 2304, 3072) and 256 divides B*T, so
// the big products fill the 256 CUs in whole rounds.  K advances in panels of 128 BYTES
// per row (64 bf16 / 32 fp32), double-buffered in LDS (2 x 56 KiB): while the MFMAs
// consume buffer p, the next panels travel HBM -> registers -> buffer p^1, one barrier
// per step; two wavefronts per SIMD overlap one's MFMAs with the other's copies.  The
// kernel is persistent (one workgroup per CU); without a K split the panel pipeline runs
// on across a workgroup's tiles, so only its first tile pays the load latency up front.
//
// LDS panels and their swizzle are described in mma_tile.h.  Operands whose contiguous
// axis is K are copied 16 bytes at a time; operands whose contiguous axis is the
// row/column axis (.t() views: the dX and dW products) are transposed in registers on
// the way in.
//
// The MFMA roles are swapped (MFMA-A = B panel, MFMA-B = A panel) so that each lane ends
// up with 4 consecutive columns of one C row; the tile is staged through LDS in fp32 and
// written back with row-contiguous stores after the bias/GELU epilogue.
//
// Workgroup -> tile mapping: ids are first regrouped so that the workgroups that land on
// one XCD (id mod 8) cover a contiguous range of tiles (they share that XCD's L2), then
// walked in groups of 8 tile-rows.  Small outputs with a long K (the dW products) are
// split along K across gridDim.z into an fp32 workspace and reduced in fixed order.
#pragma once
#include "common.h"
#include "mma_tile.h"
#include <type_traits>

// Problem description handed to the kernels.  It has a name of its own (every translation unit sees the same type)
// because the plain product is instantiated per storage type in separate units: gemm.hip (bf16) and gemm_f32.hip.
namespace ptj_gemm_detail {
struct GemmArgs {
    const void* a;
    const void* b;
    void* c;
    const void* bias;
    void* c_aux;      // optional second output: A.B + bias before the GELU (nullptr = none)
    int64_t c_aux_rs;
    float* partial;   // split-K workspace [splits][n][m] (nullptr when splits == 1)
    int n, m, k;
    int64_t a_row, a_k;   // strides of A(row=n, k)
    int64_t b_row, b_k;   // strides of B(row=m, k)  (b_row = b_cs, b_k = b_rs)
    int64_t c_rs;
    int k_per_split;      // multiple of BK
    int splits;
    int tail_first;       // > 0: tiles [tail_first, tiles) -- the last, partly filled round -- are K-split
    int tail_splits;      //      into tail_splits items each (dense fp32 partial tiles in `partial`)
    int tail_kps;         //      of tail_kps contraction elements (multiple of BK)
    int stream;           // no K split and K is a whole even number of panels: tiles are pipelined back to back
    int vec_out;          // every output (C, pre-activation, partials) and the bias allow aligned 16-byte rows
    int epilogue;
    // gemm_kernel<..., MUL = true> only: C = round(A.B) * mul element-wise, and the column sums of the
    // stored C over each block of 64 rows go to colpart[row / 64][m]
    const void* mul;
    int64_t mul_rs;
    float* colpart;
};
int launch_plain_f32(const GemmArgs& g, int splits, hipStream_t st);   // gemm_f32.hip
}  // namespace ptj_gemm_detail

namespace {
using ptj_gemm_detail::GemmArgs;

constexpr int BM = 256, BN = 192;   // C tile (rows from A, columns from B)
// Register sets that stage operand panels between HBM and LDS: with 2, the loads of panel
// kt+2 are issued during step kt and have one step to arrive; with 3, panel kt+3 is requested
// during step kt and has two.
constexpr int GEMM_MAX_STAGES = 3;
// per operand layout and element size: only 2-byte operands that are copied as they are leave registers for a third
// set (a transposing load holds its panel twice while it permutes: 104-126 spilled registers with three sets;
// 4-byte storage: 50)
constexpr int stages_for(int amode, int bmode, int elt) {
    return (amode == KMAJOR && bmode == KMAJOR && elt == 2) ? GEMM_MAX_STAGES : 2;
}
constexpr int TM = 2, TN = 3;               // 32x32 MFMA tiles per wavefront (rows x columns)
constexpr int WROWS = TM * 32;              // C rows per wavefront
constexpr int WAVES_N = 2;                  // (BM/WROWS) x 2 wavefronts, each WROWS rows x 96 columns
constexpr int GEMM_THREADS = (BM / WROWS) * WAVES_N * 64;

inline int num_cus() { return ptj_num_cus(); }   // persistent grid: one workgroup per CU

// threadIdx.x behind an opaque barrier: everything derived from it (LDS and global
// offsets) is recomputed per call instead of being hoisted out of the persistent tile
// loop, where it would stay live through every phase and spill.
__device__ __forceinline__ int fresh_tid() {
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}


// A run of K panels [kt0, kt1) of one C tile through the element-wise edge loader (tiles
// that cross the matrix border, partial panels, unaligned operands).  Written as one flat
// function (no closures) so that the prefetch registers are plain SSA values.
template <typename T, int AMODE, int BMODE>
__device__ __forceinline__ void gemm_run(const GemmArgs& g, f32x16 (&acc)[TN][TM], char* __restrict__ smem, int row0,
                                         int col0, int kbeg, int kend, int kt0, int kt1) {
    constexpr int BK = BKB / (int)sizeof(T);
    if (kt0 >= kt1) return;
    const int tid = fresh_tid();
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int lr = lane & 31, lg = lane >> 5;
    const T* A = (const T*)g.a;
    const T* B = (const T*)g.b;
    char* sA0 = smem;
    char* sB0 = smem + 2 * BM * BKB;
    TileLoader<T, AMODE, BM, GEMM_THREADS> la;
    TileLoader<T, BMODE, BN, GEMM_THREADS> lb;
#define GEMM_FETCH(KT)                                                        \
    do {                                                                      \
        const int k0__ = kbeg + (KT) * BK;                                    \
        la.load_edge(A, g.a_row, g.a_k, row0, g.n, k0__, kend, tid);          \
        lb.load_edge(B, g.b_row, g.b_k, col0, g.m, k0__, kend, tid);          \
    } while (0)
    GEMM_FETCH(kt0);
    la.store(sA0, tid);
    lb.store(sB0, tid);
    __syncthreads();
    for (int kt = kt0; kt < kt1; ++kt) {
        const int p = (kt - kt0) & 1;
        // Straight-line body: the last step re-fetches its own panels (discarded) instead
        // of branching, so the prefetch registers never cross a control-flow edge.
        GEMM_FETCH(kt + 1 < kt1 ? kt + 1 : kt);
        // Keep the copies of the next panels in flight across the MFMA block: without the
        // fences the scheduler sinks the LDS stores (and their vmcnt waits) up here.
        __builtin_amdgcn_sched_barrier(0);
        const char* cA = sA0 + p * (BM * BKB);
        const char* cB = sB0 + p * (BN * BKB);
        // MFMA operands are double-buffered by hand: chunk c+1 is read from LDS while
        // the MFMAs of chunk c run; the fences keep the reads from piling up at the top.
        typename Frag<T>::type fa[2][TM], fb[2][TN];
#define GEMM_READ_CHUNK(C, BUF)                                                                              \
    do {                                                                                                     \
        const int q__ = (C) * 2 + lg;                                                                        \
        _Pragma("unroll") for (int t = 0; t < TM; ++t) fa[BUF][t] = read_frag<T>(cA, wm * WROWS + t * 32 + lr, q__); \
        _Pragma("unroll") for (int t = 0; t < TN; ++t) fb[BUF][t] = read_frag<T>(cB, wn * 96 + t * 32 + lr, q__); \
    } while (0)
        GEMM_READ_CHUNK(0, 0);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            if (c < 3) GEMM_READ_CHUNK(c + 1, (c + 1) & 1);
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm) mma_chunk(acc[tn][tm], fb[c & 1][tn], fa[c & 1][tm]);  // A-role = B panel
            __builtin_amdgcn_sched_barrier(0);
        }
        la.store(sA0 + (p ^ 1) * (BM * BKB), tid);
        lb.store(sB0 + (p ^ 1) * (BN * BKB), tid);
        __syncthreads();
    }
#undef GEMM_FETCH
#undef GEMM_READ_CHUNK
}

// Whole K panels [0, nk) of an interior C tile, software-pipelined two panels deep:
// while the MFMAs consume LDS buffer p (panel kt), panel kt+1 moves registers -> buffer
// p^1 and panel kt+2 moves HBM -> registers.  A panel is four contraction chunks of six
// MFMAs.  The instruction order is fixed by hand (every piece ends in a scheduling
// fence): during chunks 0 and 1 the row-side operands of the next chunk are read up
// front and each column-side operand is re-read right after its last use, with the
// global loads and the LDS stores slotted between MFMA pairs; chunk 2 reads all of chunk
// 3 first (the staging registers are free by then), so the single barrier of a step
// finds no LDS read outstanding, and chunk 3 starts by reading chunk 0 of the other
// buffer under its own MFMAs.  Loads past the last panel re-fetch it (discarded), so the
// body has no branches and the staging registers stay plain values.  CLAMP: the tile
// crosses the border of C; rows / columns past it re-read the last valid one (their
// results are discarded by the bounds-checked epilogue).
template <typename T, int AMODE, int BMODE, bool CLAMP>
__device__ __forceinline__ void gemm_run_fast(const GemmArgs& g, f32x16 (&acc)[TN][TM], char* __restrict__ smem,
                                              int row0, int col0, int kbeg, int nk) {
    constexpr int BK = BKB / (int)sizeof(T);
    constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB;
    constexpr int STAGES = stages_for(AMODE, BMODE, (int)sizeof(T));
    static_assert(TN == 3, "the pipeline below is written for three MFMA tile columns per wavefront");
    if (nk <= 0) return;
    const int tid = fresh_tid();
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int lr = lane & 31, lg = lane >> 5;
    const T* A = (const T*)g.a;
    const T* B = (const T*)g.b;
    char* sA = smem;
    char* sB = smem + 2 * A_BYTES;
    TileLoader<T, AMODE, BM, GEMM_THREADS, true> la0, la1, la2;
    TileLoader<T, BMODE, BN, GEMM_THREADS, true> lb0, lb1, lb2;
    typename Frag<T>::type fa[2][TM], fb[TN], fx[TN];
    const int last = nk - 1;
    const int arow = wm * WROWS + lr, brow = wn * 96 + lr;

#define SB() __builtin_amdgcn_sched_barrier(0)
#define K0_OF(KT) (kbeg + ((KT) < last ? (KT) : last) * BK)
#define ROW_A(KT) row0
#define ROW_B(KT) col0
#define RD_A(P, C, BUF)                                                                                   \
    do {                                                                                                  \
        _Pragma("unroll") for (int t = 0; t < TM; ++t)                                                    \
            fa[BUF][t] = read_frag<T>(sA + (P) * A_BYTES, arow + t * 32, (C) * 2 + lg);                   \
    } while (0)
#define RD_B(DST, P, C, TNI) DST = read_frag<T>(sB + (P) * B_BYTES, brow + (TNI) * 32, (C) * 2 + lg)
#define MM(TNI, FB, BUF)                                                                                  \
    do {                                                                                                  \
        _Pragma("unroll") for (int tm = 0; tm < TM; ++tm) mma_chunk(acc[TNI][tm], FB, fa[BUF][tm]);       \
    } while (0)
    // One K step on buffer P.  LWA/LWB hold panel kt+1 (stored to buffer P^1), LFA/LFB
    // receive panel KTF = kt+2.  On entry fa[0] and fb hold chunk 0 of buffer P.
#define ST_A(I, LWA, P) LWA.template store_slice<I, 4>(sA + ((P) ^ 1) * A_BYTES, tid)
#define ST_B(I, LWB, P) LWB.template store_slice<I, 3>(sB + ((P) ^ 1) * B_BYTES, tid)
#define LD_A(I, LFA, KTF) LFA.template load_fast_slice<I, 4, CLAMP>(A, g.a_row, g.a_k, ROW_A(KTF), K0_OF(KTF), tid, g.n)
#define LD_B(I, LFB, KTF) LFB.template load_fast_slice<I, 3, CLAMP>(B, g.b_row, g.b_k, ROW_B(KTF), K0_OF(KTF), tid, g.m)
#define MV_A(I, LWA, LFA, P, KTF) do { ST_A(I, LWA, P); LD_A(I, LFA, KTF); } while (0)
#define MV_B(I, LWB, LFB, P, KTF) do { ST_B(I, LWB, P); LD_B(I, LFB, KTF); } while (0)
#define RF_STEP(P, LWA, LWB, LFA, LFB, KTF)                                                               \
    do {                                                                                                  \
        RD_A(P, 1, 1); SB();                                                                              \
        MM(0, fb[0], 0); SB();                                                                            \
        RD_B(fb[0], P, 1, 0); MV_A(0, LWA, LFA, P, KTF); SB();                                            \
        MM(1, fb[1], 0); SB();                                                                            \
        RD_B(fb[1], P, 1, 1); MV_A(1, LWA, LFA, P, KTF); SB();                                            \
        MM(2, fb[2], 0); SB();                                                                            \
        RD_B(fb[2], P, 1, 2); MV_A(2, LWA, LFA, P, KTF); SB();                                            \
        RD_A(P, 2, 0); SB();                                                                              \
        MM(0, fb[0], 1); SB();                                                                            \
        RD_B(fb[0], P, 2, 0); MV_A(3, LWA, LFA, P, KTF); SB();                                            \
        MM(1, fb[1], 1); SB();                                                                            \
        RD_B(fb[1], P, 2, 1); MV_B(0, LWB, LFB, P, KTF); SB();                                            \
        MM(2, fb[2], 1); SB();                                                                            \
        RD_B(fb[2], P, 2, 2); MV_B(1, LWB, LFB, P, KTF); SB();                                            \
        RD_A(P, 3, 1); RD_B(fx[0], P, 3, 0); RD_B(fx[1], P, 3, 1); RD_B(fx[2], P, 3, 2); SB();            \
        MM(0, fb[0], 0); SB();                                                                            \
        MV_B(2, LWB, LFB, P, KTF); SB();                                                                  \
        MM(1, fb[1], 0); MM(2, fb[2], 0); SB();                                                           \
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");                                   \
        RD_A((P) ^ 1, 0, 0); RD_B(fb[0], (P) ^ 1, 0, 0); RD_B(fb[1], (P) ^ 1, 0, 1);                      \
        RD_B(fb[2], (P) ^ 1, 0, 2); SB();                                                                 \
        MM(0, fx[0], 1); MM(1, fx[1], 1); MM(2, fx[2], 1); SB();                                          \
    } while (0)

    la0.template load_fast_slice<0, 1, CLAMP>(A, g.a_row, g.a_k, row0, K0_OF(0), tid, g.n);
    lb0.template load_fast_slice<0, 1, CLAMP>(B, g.b_row, g.b_k, col0, K0_OF(0), tid, g.m);
    la1.template load_fast_slice<0, 1, CLAMP>(A, g.a_row, g.a_k, row0, K0_OF(1), tid, g.n);
    lb1.template load_fast_slice<0, 1, CLAMP>(B, g.b_row, g.b_k, col0, K0_OF(1), tid, g.m);
    if constexpr (STAGES == 3) {
        la2.template load_fast_slice<0, 1, CLAMP>(A, g.a_row, g.a_k, row0, K0_OF(2), tid, g.n);
        lb2.template load_fast_slice<0, 1, CLAMP>(B, g.b_row, g.b_k, col0, K0_OF(2), tid, g.m);
    }
    la0.store(sA, tid);
    lb0.store(sB, tid);
    __syncthreads();
    RD_A(0, 0, 0); RD_B(fb[0], 0, 0, 0); RD_B(fb[1], 0, 0, 1); RD_B(fb[2], 0, 0, 2); SB();
    int kt = 0;
    if constexpr (STAGES == 2) {
        for (; kt + 1 < nk; kt += 2) {
            RF_STEP(0, la1, lb1, la0, lb0, kt + 2);
            RF_STEP(1, la0, lb0, la1, lb1, kt + 3);
        }
        if (kt < nk) RF_STEP(0, la1, lb1, la0, lb0, kt + 2);
    } else {
        // panel p waits in register set p mod 3; the LDS buffer alternates every step, so its
        // index is a variable here (three steps flip it once)
        int pb = 0;
        for (; kt + 2 < nk; kt += 3) {
            RF_STEP(pb, la1, lb1, la0, lb0, kt + 3);
            RF_STEP(pb ^ 1, la2, lb2, la1, lb1, kt + 4);
            RF_STEP(pb, la0, lb0, la2, lb2, kt + 5);
            pb ^= 1;
        }
        if (kt < nk) RF_STEP(pb, la1, lb1, la0, lb0, kt + 3);
        if (kt + 1 < nk) RF_STEP(pb ^ 1, la2, lb2, la1, lb1, kt + 4);
    }
#undef K0_OF
#undef ROW_A
#undef ROW_B
}

// LDS: two operand panel buffers (2 x 56 KiB) followed by one 6 KiB output staging area per
// wavefront; the staging areas are separate from the panels so that a wavefront can write
// its part of a finished tile while the others already load the next tile.
constexpr int PANEL_BYTES = 2 * (BM + BN) * BKB;
constexpr int STAGE_BYTES = 6144;
constexpr int SMEM_BYTES = PANEL_BYTES + (GEMM_THREADS / 64) * STAGE_BYTES;

// Writes the wave's 64x96 accumulator block to `dst` (row pitch dst_rs elements of OUT)
// through the wave-private staging area: 32 rows per pass for 2-byte outputs, 16 for
// 4-byte outputs.  A staged row is 96 outputs = three groups of 32 columns (LPR 16-byte
// chunks each); inside a group the chunk index is XORed with bits of the row number, which
// spreads both the column-wise writes of the accumulator layout and the row-wise reads
// over all banks and keeps every address a per-lane base plus a compile-time offset.
// The write-back gives each row of a group to LPR consecutive lanes (64 or 128 contiguous
// bytes per row, 16 or 8 rows per store instruction).
// BIAS: add g.bias here (false when the accumulators were started from the bias).
// ACT: 1 = apply the GELU when the epilogue asks for it (both GELU epilogues); 2 = the GELU's
// derivative instead (the second output of PTJ_EPI_BIAS_GELU_DERIV).  One pass that evaluates the
// exponential once for both outputs was built as well: holding the second output of a pass in
// registers costs more in spills than the second evaluation.
// MUL: the stored value is round(acc) * g.mul[row, col], and its column sums over the
// wavefront's 64 rows are written to g.colpart (fixed order: deterministic).
// FULL: the tile lies inside C and dst / bias are vector-aligned, so the write-back is
// straight-line 16-byte stores; otherwise every element is bounds-checked.  The two
// variants are separate instantiations on purpose: when both appear behind one per-lane
// condition the compiler merges them into partial (12 + 2 + 2 byte) stores.  The global
// stores are not waited for.
template <typename OUT, typename T, bool BIAS, int ACT, bool FULL, bool MUL = false>
__device__ __forceinline__ void gemm_store_block(const GemmArgs& g, const f32x16 (&acc)[TN][TM], char* __restrict__ smem,
                                                 int row0, int col0, OUT* __restrict__ dst, int64_t dst_rs) {
    constexpr int RB = 96 * (int)sizeof(OUT);                    // bytes per staged row
    constexpr int ROWS = STAGE_BYTES / RB;                       // rows per pass
    constexpr int V = 16 / (int)sizeof(OUT);                     // elements per 16-byte vector
    constexpr int LPR = 32 / V;                                  // chunks per 32-column group = lanes per row
    constexpr int KS = sizeof(OUT) == 2 ? 2 : 1;                 // swizzle key = (row >> KS) & (LPR - 1)
    constexpr int RPI = 64 / LPR;                                // rows per store instruction
    static_assert(ROWS == 32 || ROWS == 16, "staging pass");
    const int tid = fresh_tid();
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int lr = lane & 31, lg = lane >> 5;
    char* stage = smem + PANEL_BYTES + wave * STAGE_BYTES;
    const int gcol0 = col0 + wn * 96;
    const int grow0 = row0 + wm * WROWS;
    const int sr = lr & (ROWS - 1);                              // staged row of this lane
    const bool has_bias = BIAS && g.epilogue != PTJ_EPI_NONE;
    const bool act = ACT == 1 && (g.epilogue == PTJ_EPI_BIAS_GELU || g.epilogue == PTJ_EPI_BIAS_GELU_DERIV);
    static_assert(!MUL || (WROWS == 64 && !BIAS && ACT == 0 && sizeof(OUT) == sizeof(T)), "MUL epilogue");

    // bias of this lane's 12 column quads
    float bias[TN * 4][4];
    if constexpr (BIAS) {
#pragma unroll
        for (int q = 0; q < TN * 4; ++q) {
            const int cc = (q >> 2) * 32 + (q & 3) * 8 + lg * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) bias[q][e] = 0.f;
            if (has_bias) {
                if constexpr (FULL) {
                    load_vec<T, 4>((const T*)g.bias + gcol0 + cc, bias[q]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gcol0 + cc + e < g.m) bias[q][e] = to_f32(((const T*)g.bias)[gcol0 + cc + e]);
                }
            }
        }
    }
    // write side: the lane's 4 columns of quad i4 sit in chunk (i4 [*2 + lg]) of group tn
    const int wkey = (sr >> KS) & (LPR - 1);
    char* wrow = stage + sr * RB + (sizeof(OUT) == 2 ? lg * 8 : 0);
    int woff[4];
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) woff[i4] = (((sizeof(OUT) == 2 ? i4 : i4 * 2 + lg) ^ wkey) << 4);
    // read side: lane -> row (lane / LPR) of the instruction's RPI rows, chunk lane % LPR
    const int rrow = lane / LPR, rch = lane % LPR;
    const char* rbase[ROWS / RPI];
#pragma unroll
    for (int h = 0; h < ROWS / RPI; ++h) {
        const int r = h * RPI + rrow;
        rbase[h] = stage + r * RB + ((rch ^ ((r >> KS) & (LPR - 1))) << 4);
    }
    OUT* gbase = dst + (int64_t)(grow0 + rrow) * dst_rs + gcol0 + rch * V;
    // MUL: the multiplier element beside every stored element, and this lane's column sums: its V
    // columns of each 32-column group over the rows it writes
    const OUT* mbase = nullptr;
    float cs[3][V];
    if constexpr (MUL) {
        mbase = (const OUT*)g.mul + (int64_t)(grow0 + rrow) * g.mul_rs + gcol0 + rch * V;
#pragma unroll
        for (int g3 = 0; g3 < 3; ++g3)
#pragma unroll
            for (int e = 0; e < V; ++e) cs[g3][e] = 0.f;
    }
#pragma unroll
    for (int pass = 0; pass < WROWS / ROWS; ++pass) {
        const int tm = pass * ROWS / 32;
        const bool mine = ROWS == 32 || (lr >> 4) == (pass & 1);
        // the multipliers of this pass are requested before the block is staged
        Pack<OUT, V> mv[ROWS / RPI][3];
        if constexpr (MUL && FULL) {
#pragma unroll
            for (int h = 0; h < ROWS / RPI; ++h)
#pragma unroll
                for (int g3 = 0; g3 < 3; ++g3)
                    mv[h][g3] = *reinterpret_cast<const Pack<OUT, V>*>(mbase + (int64_t)(pass * ROWS + h * RPI) * g.mul_rs +
                                                                        g3 * 32);
        }
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = acc[tn][tm][i4 * 4 + e];
                if constexpr (BIAS) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] += bias[tn * 4 + i4][e];
                }
                if constexpr (ACT == 1) {
                    if (act) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = gelu_f(o[e]);
                    }
                }
                if constexpr (ACT == 2) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = gelu_grad_f(o[e]);
                }
                if (ROWS == 32 || mine) store_vec<OUT, 4>(reinterpret_cast<OUT*>(wrow + tn * (LPR * 16) + woff[i4]), o);
            }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");   // the wave re-reads only its own area
#pragma unroll
        for (int h = 0; h < ROWS / RPI; ++h)
#pragma unroll
            for (int g3 = 0; g3 < 3; ++g3) {
                const int r = pass * ROWS + h * RPI;             // block row of the instruction's first row
                Pack<OUT, V> val = *reinterpret_cast<const Pack<OUT, V>*>(rbase[h] + g3 * (LPR * 16));
                OUT* p = gbase + (int64_t)r * dst_rs + g3 * 32;
                if constexpr (FULL) {
                    if constexpr (MUL) {
#pragma unroll
                        for (int e = 0; e < V; ++e) {
                            val.v[e] = from_f32<OUT>(to_f32(val.v[e]) * to_f32(mv[h][g3].v[e]));
                            cs[g3][e] += to_f32(val.v[e]);
                        }
                    }
                    *reinterpret_cast<Pack<OUT, V>*>(p) = val;
                } else {
                    if (grow0 + r + rrow < g.n) {
                        const int gcol = gcol0 + g3 * 32 + rch * V;
#pragma unroll
                        for (int e = 0; e < V; ++e)
                            if (gcol + e < g.m) {
                                if constexpr (MUL) {
                                    val.v[e] = from_f32<OUT>(to_f32(val.v[e]) *
                                                             to_f32(mbase[(int64_t)r * g.mul_rs + g3 * 32 + e]));
                                    cs[g3][e] += to_f32(val.v[e]);
                                }
                                p[e] = val.v[e];
                            }
                    }
                }
            }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    }
    if constexpr (MUL) {
        // lanes with equal (lane mod LPR) hold the same columns for different rows: butterfly over
        // the row bits, then the lanes of row 0 write the wavefront's 96 sums
#pragma unroll
        for (int g3 = 0; g3 < 3; ++g3)
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float v = cs[g3][e];
#pragma unroll
                for (int off = LPR; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
                cs[g3][e] = v;
            }
        if (rrow == 0 && grow0 < g.n) {
            float* cp = g.colpart + (int64_t)(grow0 / 64) * g.m + gcol0 + rch * V;
#pragma unroll
            for (int g3 = 0; g3 < 3; ++g3)
#pragma unroll
                for (int e = 0; e < V; ++e)
                    if (FULL || gcol0 + g3 * 32 + rch * V + e < g.m) cp[g3 * 32 + e] = cs[g3][e];
        }
    }
}

// Work item -> origin of its C tile: ids are regrouped so that the items of one XCD (id mod
// 8) cover a contiguous range of tiles, then walked in groups of 8 tile-rows.
__device__ __forceinline__ void tile_origin(int pid, int total, int num_m, int num_n, int& row0, int& col0) {
    {
        const int chunk = total >> 3, rem = total & 7, x = pid & 7;
        pid = x * chunk + (x < rem ? x : rem) + (pid >> 3);
    }
    constexpr int GROUP = 8;
    const int width = GROUP * num_n;
    const int group_id = pid / width;
    const int first_m = group_id * GROUP;
    const int gsz = (num_m - first_m) < GROUP ? (num_m - first_m) : GROUP;
    const int tile_m = first_m + (pid % width) % gsz;
    const int tile_n = (pid % width) / gsz;
    row0 = tile_m * BM;
    col0 = tile_n * BN;
}

// Epilogue of one tile.  acc[tn][tm][i] of lane (lr, lg) is
//   C[wm*64 + tm*32 + lr][wn*96 + tn*32 + (i/4)*8 + lg*4 + (i%4)].
// Bias / GELU are applied in registers, the block is converted to the output type,
// staged in the wave-private LDS area and written back as 16-byte vectors that run
// along whole 96-column rows.  Only wave-local ordering is needed.
template <typename T, bool BIAS, bool SPLIT = true, bool MUL = false>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& g, const f32x16 (&acc)[TN][TM], char* __restrict__ smem,
                                              int row0, int col0, int z) {
    const bool full = row0 + BM <= g.n && col0 + BN <= g.m && g.vec_out;
    if constexpr (MUL) {
        if (full) gemm_store_block<T, T, false, 0, true, true>(g, acc, smem, row0, col0, (T*)g.c, g.c_rs);
        else gemm_store_block<T, T, false, 0, false, true>(g, acc, smem, row0, col0, (T*)g.c, g.c_rs);
    } else if (SPLIT && g.partial != nullptr) {
        float* part = g.partial + (int64_t)z * g.n * (int64_t)g.m;
        if (full) gemm_store_block<float, T, false, 0, true>(g, acc, smem, row0, col0, part, g.m);
        else gemm_store_block<float, T, false, 0, false>(g, acc, smem, row0, col0, part, g.m);
    } else if (full) {
        if (g.c_aux != nullptr) {
            if (g.epilogue == PTJ_EPI_BIAS_GELU_DERIV)
                gemm_store_block<T, T, BIAS, 2, true>(g, acc, smem, row0, col0, (T*)g.c_aux, g.c_aux_rs);
            else
                gemm_store_block<T, T, BIAS, 0, true>(g, acc, smem, row0, col0, (T*)g.c_aux, g.c_aux_rs);
        }
        gemm_store_block<T, T, BIAS, 1, true>(g, acc, smem, row0, col0, (T*)g.c, g.c_rs);
    } else {
        if (g.c_aux != nullptr) {
            if (g.epilogue == PTJ_EPI_BIAS_GELU_DERIV)
                gemm_store_block<T, T, BIAS, 2, false>(g, acc, smem, row0, col0, (T*)g.c_aux, g.c_aux_rs);
            else
                gemm_store_block<T, T, BIAS, 0, false>(g, acc, smem, row0, col0, (T*)g.c_aux, g.c_aux_rs);
        }
        gemm_store_block<T, T, BIAS, 1, false>(g, acc, smem, row0, col0, (T*)g.c, g.c_rs);
    }
}

// Bias of this lane's 12 column quads of the tile at column col0, in storage type (zeros
// without a bias, or on request: K slices get their bias in the second stage).  CLAMP: the tile may cross the right border; columns past it re-read
// the last valid one.
template <typename T, bool CLAMP>
__device__ __forceinline__ void load_bias_quads(const GemmArgs& g, int col0, Pack<T, 4> (&b)[TN * 4], bool zero) {
    const int tid = fresh_tid();
    const int lg = (tid & 63) >> 5, wn = (tid >> 6) % WAVES_N;
    const int gcol0 = col0 + wn * 96 + lg * 4;
    const T* bias = (const T*)g.bias;
    if (zero || g.epilogue == PTJ_EPI_NONE || bias == nullptr) {
#pragma unroll
        for (int q = 0; q < TN * 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) b[q].v[e] = from_f32<T>(0.f);
        return;
    }
    bool whole = true;
    if constexpr (CLAMP) whole = col0 + BN <= g.m;
    if (whole) {
#pragma unroll
        for (int q = 0; q < TN * 4; ++q)
            b[q] = *reinterpret_cast<const Pack<T, 4>*>(bias + gcol0 + (q >> 2) * 32 + (q & 3) * 8);
    } else {
#pragma unroll
        for (int q = 0; q < TN * 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int c = gcol0 + (q >> 2) * 32 + (q & 3) * 8 + e;
                b[q].v[e] = bias[c < g.m ? c : g.m - 1];
            }
    }
}

// The pipelined loop of gemm_run_fast carried across the tiles of a workgroup (no K
// split, K a whole even number of panels): the two panel fetches that run past the end
// of a tile bring in the first two panels of the workgroup's next tile instead of
// re-reading the last one, so after the last step the LDS buffer, the staging registers
// and the operand registers are exactly in the state the loop expects on entry.  The
// epilogue (which stages through its own LDS area) runs between two tiles while those
// loads are in flight.  A workgroup without a next tile re-fetches its own first panels.
// The accumulators start from the bias (loaded while the previous tile's epilogue runs)
// instead of zero, so the epilogue neither waits for bias loads nor adds them.
template <typename T, int AMODE, int BMODE, bool CLAMP, bool MUL>
__device__ __forceinline__ void gemm_stream(const GemmArgs& g, char* __restrict__ smem) {
    constexpr int BK = BKB / (int)sizeof(T);
    constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB;
    constexpr int STAGES = stages_for(AMODE, BMODE, (int)sizeof(T));
    const int num_m = (g.n + BM - 1) / BM, num_n = (g.m + BN - 1) / BN;
    const int total = num_m * num_n;
    // work items: whole tiles, then (with a K-split last round) the K slices of its tiles
    const int work = g.tail_splits > 1 ? g.tail_first + (total - g.tail_first) * g.tail_splits : total;
    const T* A = (const T*)g.a;
    const T* B = (const T*)g.b;
    char* sA = smem;
    char* sB = smem + 2 * A_BYTES;
    TileLoader<T, AMODE, BM, GEMM_THREADS, true> la0, la1, la2;
    TileLoader<T, BMODE, BN, GEMM_THREADS, true> lb0, lb1, lb2;
    typename Frag<T>::type fa[2][TM], fb[TN], fx[TN];
    int pb = 0;   // LDS buffer that holds the current tile's first panel (three staging sets only)
    // item -> tile origin, first contraction element, number of panels (even), partial tile
#define STREAM_ITEM(ITEM, ROW0, COL0, KBEG, NK, PART)                                                    \
    do {                                                                                                 \
        if (g.tail_splits > 1 && (ITEM) >= g.tail_first) {                                               \
            const int r__ = (ITEM) - g.tail_first;                                                       \
            const int t__ = r__ / g.tail_splits, z__ = r__ - t__ * g.tail_splits;                        \
            tile_origin(g.tail_first + t__, total, num_m, num_n, ROW0, COL0);                            \
            KBEG = z__ * g.tail_kps;                                                                     \
            NK = ((KBEG + g.tail_kps < g.k ? g.tail_kps : g.k - KBEG)) / BK;                             \
            PART = g.partial + (int64_t)r__ * (BM * BN);                                                 \
        } else {                                                                                         \
            tile_origin(ITEM, total, num_m, num_n, ROW0, COL0);                                          \
            KBEG = 0;                                                                                    \
            NK = g.k / BK;                                                                               \
            PART = nullptr;                                                                              \
        }                                                                                                \
    } while (0)
    int item = blockIdx.x;
    int row0, col0, kbeg, nk;
    float* part;
    STREAM_ITEM(item, row0, col0, kbeg, nk, part);
    Pack<T, 4> braw[TN * 4];
    load_bias_quads<T, CLAMP>(g, col0, braw, part != nullptr);
    {
        const int tid = fresh_tid();
        const int lane = tid & 63, wave = tid >> 6;
        const int lr = lane & 31, lg = lane >> 5;
        const int arow = (wave / WAVES_N) * WROWS + lr, brow = (wave % WAVES_N) * 96 + lr;
        la0.template load_fast_slice<0, 1, CLAMP>(A, g.a_row, g.a_k, row0, kbeg, tid, g.n);
        lb0.template load_fast_slice<0, 1, CLAMP>(B, g.b_row, g.b_k, col0, kbeg, tid, g.m);
        la1.template load_fast_slice<0, 1, CLAMP>(A, g.a_row, g.a_k, row0, kbeg + BK, tid, g.n);
        lb1.template load_fast_slice<0, 1, CLAMP>(B, g.b_row, g.b_k, col0, kbeg + BK, tid, g.m);
        if constexpr (STAGES == 3) {
            la2.template load_fast_slice<0, 1, CLAMP>(A, g.a_row, g.a_k, row0, kbeg + 2 * BK, tid, g.n);
            lb2.template load_fast_slice<0, 1, CLAMP>(B, g.b_row, g.b_k, col0, kbeg + 2 * BK, tid, g.m);
        }
        la0.store(sA, tid);
        lb0.store(sB, tid);
        __syncthreads();
        RD_A(0, 0, 0); RD_B(fb[0], 0, 0, 0); RD_B(fb[1], 0, 0, 1); RD_B(fb[2], 0, 0, 2); SB();
    }
    for (;;) {
        const int nitem = item + (int)gridDim.x;
        const bool more = nitem < work;
        int nrow0, ncol0, nkbeg, nnk;
        float* npart;
        STREAM_ITEM(more ? nitem : item, nrow0, ncol0, nkbeg, nnk, npart);
        f32x16 acc[TN][TM];
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = to_f32(braw[i * 4 + (e >> 2)].v[e & 3]);
        {
            const int tid = fresh_tid();
            const int lane = tid & 63, wave = tid >> 6;
            const int lr = lane & 31, lg = lane >> 5;
            const int arow = (wave / WAVES_N) * WROWS + lr, brow = (wave % WAVES_N) * 96 + lr;
#define K0_OF(KT) ((KT) < nk ? kbeg + (KT) * BK : nkbeg + ((KT) - nk) * BK)
#define ROW_A(KT) ((KT) < nk ? row0 : nrow0)
#define ROW_B(KT) ((KT) < nk ? col0 : ncol0)
            if constexpr (STAGES == 2) {
                for (int kt = 0; kt < nk; kt += 2) {
                    RF_STEP(0, la1, lb1, la0, lb0, kt + 2);
                    RF_STEP(1, la0, lb0, la1, lb1, kt + 3);
                }
            } else {
                // nk is a multiple of 3 here: every tile starts with its panels 0, 1, 2 in LDS
                // buffer pb, set 1 and set 2
                for (int kt = 0; kt < nk; kt += 3) {
                    RF_STEP(pb, la1, lb1, la0, lb0, kt + 3);
                    RF_STEP(pb ^ 1, la2, lb2, la1, lb1, kt + 4);
                    RF_STEP(pb, la0, lb0, la2, lb2, kt + 5);
                    pb ^= 1;
                }
            }
#undef K0_OF
#undef ROW_A
#undef ROW_B
        }
        load_bias_quads<T, CLAMP>(g, ncol0, braw, npart != nullptr);
        if (part != nullptr) gemm_store_block<float, T, false, 0, true>(g, acc, smem, 0, 0, part, BN);
        else gemm_epilogue<T, false, false, MUL>(g, acc, smem, row0, col0, 0);
        if (!more) break;
        item = nitem;
        row0 = nrow0;
        col0 = ncol0;
        kbeg = nkbeg;
        nk = nnk;
        part = npart;
    }
#undef STREAM_ITEM
}
#undef SB
#undef RD_A
#undef RD_B
#undef MM
#undef RF_STEP
#undef ST_A
#undef ST_B
#undef LD_A
#undef LD_B
#undef MV_A
#undef MV_B

// Persistent kernel: workgroup b handles work items b, b + gridDim.x, ... where an item is
// one (C tile, K split) pair; the stores of a finished tile drain while the next tile's
// panels are loaded and multiplied.
template <typename T, int AMODE, int BMODE, bool MUL = false>
__global__ __launch_bounds__(GEMM_THREADS, 1) void gemm_kernel(const GemmArgs g) {
    constexpr int BK = BKB / (int)sizeof(T);
    __shared__ __attribute__((aligned(16))) char smem[SMEM_BYTES];
    constexpr bool VECTOR_OK = AMODE != GENERIC && BMODE != GENERIC;
    if constexpr (VECTOR_OK) {
        if (g.stream) {
            if (g.n % BM == 0 && g.m % BN == 0) gemm_stream<T, AMODE, BMODE, false, MUL>(g, smem);
            else gemm_stream<T, AMODE, BMODE, true, MUL>(g, smem);
            return;
        }
    }

    const int num_m = (g.n + BM - 1) / BM, num_n = (g.m + BN - 1) / BN;
    const int total = num_m * num_n;
    const int work = g.tail_splits > 1 ? g.tail_first + (total - g.tail_first) * g.tail_splits : total * g.splits;
    for (int item = blockIdx.x; item < work; item += gridDim.x) {
        int z = 0, row0, col0;
        int kbeg = 0, kend = g.k;
        float* tail_part = nullptr;
        if (g.tail_splits > 1 && item >= g.tail_first) {
            // a tile of the last round: one of its K slices, written as a dense partial tile
            const int r = item - g.tail_first;
            const int t = r / g.tail_splits;
            z = r - t * g.tail_splits;
            tile_origin(g.tail_first + t, total, num_m, num_n, row0, col0);
            kbeg = z * g.tail_kps;
            kend = (kbeg + g.tail_kps) < g.k ? (kbeg + g.tail_kps) : g.k;
            tail_part = g.partial + (int64_t)r * (BM * BN);
        } else if (g.splits > 1) {
            // K-split products are bound by operand traffic: the items of one XCD (a contiguous
            // index range after the regrouping, all resident at once) are chosen to share operand
            // slices.  Index order: the tiles along the smaller C dimension fastest (they share
            // the K slice of the larger operand), then the tiles along the larger one, then the
            // K split -- so every slice of the larger operand is fetched by one XCD only.
            const int chunk = work >> 3, rem = work & 7, x = item & 7;
            const int idx = x * chunk + (x < rem ? x : rem) + (item >> 3);
            int tile_m, tile_n;
            if (g.n >= g.m) {
                tile_n = idx % num_n;
                const int pair = idx / num_n;
                tile_m = pair % num_m;
                z = pair / num_m;
            } else {
                tile_m = idx % num_m;
                const int pair = idx / num_m;
                tile_n = pair % num_n;
                z = pair / num_n;
            }
            row0 = tile_m * BM;
            col0 = tile_n * BN;
            kbeg = z * g.k_per_split;
            kend = (kbeg + g.k_per_split) < g.k ? (kbeg + g.k_per_split) : g.k;
        } else {
            tile_origin(item, total, num_m, num_n, row0, col0);
        }
        const int nk = (kend - kbeg + BK - 1) / BK;

        f32x16 acc[TN][TM];
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

        const bool interior = row0 + BM <= g.n && col0 + BN <= g.m;
        const int nk_full = (kend - kbeg) / BK;  // whole panels
        if constexpr (VECTOR_OK) {
            // tiles that cross the border of C run the same pipeline with clamped row indices
            if (interior) gemm_run_fast<T, AMODE, BMODE, false>(g, acc, smem, row0, col0, kbeg, nk_full);
            else gemm_run_fast<T, AMODE, BMODE, true>(g, acc, smem, row0, col0, kbeg, nk_full);
            if (nk_full < nk) {
                __syncthreads();   // the pipelined loop leaves LDS reads in flight
                gemm_run<T, AMODE, BMODE>(g, acc, smem, row0, col0, kbeg, kend, nk_full, nk);
            }
        } else {
            gemm_run<T, AMODE, BMODE>(g, acc, smem, row0, col0, kbeg, kend, 0, nk);
        }
        if constexpr (MUL) gemm_epilogue<T, false, false, true>(g, acc, smem, row0, col0, 0);
        else if (tail_part != nullptr) gemm_store_block<float, T, false, 0, true>(g, acc, smem, 0, 0, tail_part, BN);
        else if (g.tail_splits > 1) gemm_epilogue<T, true, false>(g, acc, smem, row0, col0, z);
        else gemm_epilogue<T, true, true>(g, acc, smem, row0, col0, z);
    }
}

// Split-K second stage: C = epilogue(sum_z partial[z]) in z order.
template <typename T>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ partial, int splits, int n,
                                                                  int m, T* __restrict__ c, int64_t c_rs,
                                                                  const T* __restrict__ bias, int epilogue,
                                                                  T* __restrict__ c_aux, int64_t c_aux_rs) {
    const int64_t total = (int64_t)n * m;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        float s = 0.f;
        for (int z = 0; z < splits; ++z) s += partial[z * total + i];
        const int row = (int)(i / m), col = (int)(i - (int64_t)row * m);
        if (epilogue != PTJ_EPI_NONE) s += to_f32(bias[col]);
        if (c_aux != nullptr)
            c_aux[(int64_t)row * c_aux_rs + col] = from_f32<T>(epilogue == PTJ_EPI_BIAS_GELU_DERIV ? gelu_grad_f(s) : s);
        if (epilogue == PTJ_EPI_BIAS_GELU || epilogue == PTJ_EPI_BIAS_GELU_DERIV) s = gelu_f(s);
        c[(int64_t)row * c_rs + col] = from_f32<T>(s);
    }
}

// The same, four consecutive columns per thread (16-byte loads of the partials, one vector
// store): m % 4 == 0 and 4-element aligned C / bias.  Same summation order per element.
template <typename T>
__global__ __launch_bounds__(256) void gemm_splitk_reduce4_kernel(const float* __restrict__ partial, int splits, int n,
                                                                   int m, T* __restrict__ c, int64_t c_rs,
                                                                   const T* __restrict__ bias, int epilogue,
                                                                   T* __restrict__ c_aux, int64_t c_aux_rs) {
    const int64_t total = (int64_t)n * m, quads = total >> 2;
    for (int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x; q < quads; q += (int64_t)gridDim.x * 256) {
        const int64_t i = q << 2;
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int z = 0; z < splits; ++z) s += *reinterpret_cast<const f32x4*>(partial + z * total + i);
        const int row = (int)(i / m), col = (int)(i - (int64_t)row * m);
        if (epilogue != PTJ_EPI_NONE) {
            const Pack<T, 4> b = *reinterpret_cast<const Pack<T, 4>*>(bias + col);
#pragma unroll
            for (int e = 0; e < 4; ++e) s[e] += to_f32(b.v[e]);
        }
        Pack<T, 4> o;
        const bool deriv = epilogue == PTJ_EPI_BIAS_GELU_DERIV;
        if (c_aux != nullptr) {
#pragma unroll
            for (int e = 0; e < 4; ++e) o.v[e] = from_f32<T>(deriv ? gelu_grad_f(s[e]) : s[e]);
            *reinterpret_cast<Pack<T, 4>*>(c_aux + (int64_t)row * c_aux_rs + col) = o;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
            o.v[e] = from_f32<T>(epilogue == PTJ_EPI_BIAS_GELU || deriv ? gelu_f(s[e]) : s[e]);
        *reinterpret_cast<Pack<T, 4>*>(c + (int64_t)row * c_rs + col) = o;
    }
}

// Second stage for the K-split tiles of the last round: tile t (work item tail_first + t) =
// epilogue(sum_z partial[t*splits + z]) in z order; partial tiles are dense BM x BN.
template <typename T>
__global__ __launch_bounds__(256) void gemm_tail_reduce_kernel(const GemmArgs g) {
    const int num_m = (g.n + BM - 1) / BM, num_n = (g.m + BN - 1) / BN;
    const int t = blockIdx.x;
    int row0, col0;
    tile_origin(g.tail_first + t, num_m * num_n, num_m, num_n, row0, col0);
    const float* base = g.partial + (int64_t)t * g.tail_splits * (BM * BN);
    // four consecutive columns per thread: 16-byte loads of the partial tiles; a quad that lies
    // wholly inside C is stored as one vector when the outputs allow it
    for (int q = blockIdx.y * 256 + threadIdx.x; q < BM * BN / 4; q += gridDim.y * 256) {
        const int i = q * 4;
        const int r = i / BN, c = i - r * BN;
        const int row = row0 + r, col = col0 + c;
        if (row >= g.n || col >= g.m) continue;
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int z = 0; z < g.tail_splits; ++z) s += *reinterpret_cast<const f32x4*>(base + (int64_t)z * (BM * BN) + i);
        const bool whole = col + 4 <= g.m;
        if (g.epilogue != PTJ_EPI_NONE) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (whole || col + e < g.m) s[e] += to_f32(((const T*)g.bias)[col + e]);
        }
        T* ca = g.c_aux != nullptr ? (T*)g.c_aux + (int64_t)row * g.c_aux_rs + col : nullptr;
        T* cc = (T*)g.c + (int64_t)row * g.c_rs + col;
        Pack<T, 4> pre, out;
        const bool deriv = g.epilogue == PTJ_EPI_BIAS_GELU_DERIV;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pre.v[e] = from_f32<T>(deriv ? gelu_grad_f(s[e]) : s[e]);
            out.v[e] = from_f32<T>(g.epilogue == PTJ_EPI_BIAS_GELU || deriv ? gelu_f(s[e]) : s[e]);
        }
        if (whole && g.vec_out) {
            if (ca != nullptr) *reinterpret_cast<Pack<T, 4>*>(ca) = pre;
            *reinterpret_cast<Pack<T, 4>*>(cc) = out;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (col + e >= g.m) break;
                if (ca != nullptr) ca[e] = pre.v[e];
                cc[e] = out.v[e];
            }
        }
    }
}

#include "gemm_direct.h"

template <typename T>
int pick_mode(const void* p, int64_t s_row, int64_t s_k) {
    constexpr int VEC = VecOf<T>::N;
    if (!ptj_aligned16(p)) return GENERIC;
    if (s_k == 1 && s_row % VEC == 0) return KMAJOR;
    if (s_row == 1 && s_k % VEC == 0) return MNMAJOR;
    return GENERIC;
}

template <typename T, bool MUL = false>
int gemm_impl(GemmArgs g, int splits, hipStream_t st) {
    const int am = pick_mode<T>(g.a, g.a_row, g.a_k), bm = pick_mode<T>(g.b, g.b_row, g.b_k);
    {
        // the streamed loop takes K panels in groups of as many as there are staging sets
        const int sg = stages_for(am, bm, (int)sizeof(T)), bk = BKB / (int)sizeof(T);
        if (g.stream && !(g.k >= sg * bk && g.k % (sg * bk) == 0)) g.stream = 0;
        if (sg != 2 && g.tail_splits > 1) {      // K slices of the last round come in pairs of panels
            g.tail_first = 0; g.tail_splits = 1; g.tail_kps = 0;
            if (splits == 1) g.partial = nullptr;
        }
    }
    const int num_m = (g.n + BM - 1) / BM, num_n = (g.m + BN - 1) / BN;
    int64_t work = (int64_t)num_m * num_n * splits;
    if (g.tail_splits > 1) work = g.tail_first + ((int64_t)num_m * num_n - g.tail_first) * g.tail_splits;
    const int cus = num_cus();
    dim3 grid((unsigned)(work < cus ? work : cus)), block(GEMM_THREADS);
    bool direct = false;
    if constexpr (sizeof(T) == 2) {
        // Operands that need a transpose on their way to the MFMAs (.t() views: the dX and dW products) take the
        // loop with asynchronous copies and transposing LDS reads.  Two K-major operands stay on the register-staged
        // loop, whose third staging set gives their loads two steps to arrive: inside a training step it is the
        // faster of the two for them (4.67 against 4.90 ms over the step's 49 forward products), back to back
        // in a loop it is the slower one.
        direct = !(am == KMAJOR && bm == KMAJOR) && dg_eligible(g, am, bm);
        // only the loop with asynchronous copies starts its accumulators from the stored C
        if (g.epilogue == PTJ_EPI_ACCUMULATE && !(direct && g.vec_out && splits == 1 && g.tail_splits <= 1))
            return ptj_set_error(PTJ_ERR_INVALID, "gemm: the accumulating epilogue needs a transposed 16-byte aligned "
                                 "operand layout, k a multiple of 64 and vector-aligned C");
        if (direct) {
#define DG_LAUNCH(AM, BMD) hipLaunchKernelGGL((gemm_direct_kernel<AM, BMD, MUL>), grid, block, 0, st, g)
            switch (am * 3 + bm) {
                case 1: DG_LAUNCH(KMAJOR, MNMAJOR); break;
                case 3: DG_LAUNCH(MNMAJOR, KMAJOR); break;
                default: DG_LAUNCH(MNMAJOR, MNMAJOR); break;
            }
#undef DG_LAUNCH
        }
    }
    if (!direct) {
#define GEMM_LAUNCH(AM, BMD) hipLaunchKernelGGL((gemm_kernel<T, AM, BMD, MUL>), grid, block, 0, st, g)
    if constexpr (MUL) {
        // the multiplying epilogue exists for vector-loadable operands only (the caller checks)
        switch (am * 3 + bm) {
            case 0: GEMM_LAUNCH(KMAJOR, KMAJOR); break;
            case 1: GEMM_LAUNCH(KMAJOR, MNMAJOR); break;
            case 3: GEMM_LAUNCH(MNMAJOR, KMAJOR); break;
            case 4: GEMM_LAUNCH(MNMAJOR, MNMAJOR); break;
            default: return ptj_set_error(PTJ_ERR_INVALID, "gemm: operand layout without a multiplying epilogue");
        }
    } else {
        switch (am * 3 + bm) {
            case 0: GEMM_LAUNCH(KMAJOR, KMAJOR); break;
            case 1: GEMM_LAUNCH(KMAJOR, MNMAJOR); break;
            case 2: GEMM_LAUNCH(KMAJOR, GENERIC); break;
            case 3: GEMM_LAUNCH(MNMAJOR, KMAJOR); break;
            case 4: GEMM_LAUNCH(MNMAJOR, MNMAJOR); break;
            case 5: GEMM_LAUNCH(MNMAJOR, GENERIC); break;
            case 6: GEMM_LAUNCH(GENERIC, KMAJOR); break;
            case 7: GEMM_LAUNCH(GENERIC, MNMAJOR); break;
            default: GEMM_LAUNCH(GENERIC, GENERIC); break;
        }
    }
#undef GEMM_LAUNCH
    }
    PTJ_CHECK_LAUNCH();
    if (splits > 1) {
        const int64_t total = (int64_t)g.n * g.m;
        const bool quad = g.vec_out && g.m % 4 == 0 && ptj_aligned16(g.partial);
        int64_t blocks = ((quad ? total / 4 : total) + 255) / 256;
        if (blocks > 256 * 8) blocks = 256 * 8;
        if (quad)
            hipLaunchKernelGGL((gemm_splitk_reduce4_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st,
                               (const float*)g.partial, splits, g.n, g.m, (T*)g.c, g.c_rs, (const T*)g.bias, g.epilogue,
                               (T*)g.c_aux, g.c_aux_rs);
        else
            hipLaunchKernelGGL((gemm_splitk_reduce_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st,
                               (const float*)g.partial, splits, g.n, g.m, (T*)g.c, g.c_rs, (const T*)g.bias, g.epilogue,
                               (T*)g.c_aux, g.c_aux_rs);
        PTJ_CHECK_LAUNCH();
    }
    if (g.tail_splits > 1) {
        hipLaunchKernelGGL((gemm_tail_reduce_kernel<T>), dim3((unsigned)(num_m * num_n - g.tail_first), 12), dim3(256), 0,
                           st, g);
        PTJ_CHECK_LAUNCH();
    }
    return PTJ_OK;
}

// Number of K splits for an (n, m, k) problem given `ws_bytes` of workspace.
// Picks the split count that minimises a small cost model: the workgroups run in rounds
// of one per CU, a workgroup costs a fixed prologue/epilogue plus a per-panel time, and
// every split writes and re-reads an fp32 copy of C.
int choose_splits(int64_t n, int64_t m, int64_t k, int elt, size_t ws_bytes) {
    const int CUS = num_cus();
    constexpr double T_FIXED_US = 6.0, T_PANEL_US = 1.6, BYTES_PER_US = 4.0e6;
    const int64_t tiles = ((n + BM - 1) / BM) * ((m + BN - 1) / BN);
    const int bk = BKB / elt;
    const int64_t panels = (k + bk - 1) / bk;
    if (tiles >= CUS || panels < 16) return 1;
    int best = 1;
    double best_cost = 0.0;
    for (int s = 1; s <= 32; ++s) {
        if (s > 1 && (panels / s < 8 || (size_t)s * n * m * sizeof(float) > ws_bytes)) break;
        const int64_t rounds = (tiles * s + CUS - 1) / CUS;
        const int64_t per_split = (panels + s - 1) / s;
        double cost = (double)rounds * (T_FIXED_US + (double)per_split * T_PANEL_US);
        if (s > 1) cost += 2.0 * (double)s * (double)n * (double)m * sizeof(float) / BYTES_PER_US;
        if (s == 1 || cost < best_cost) { best = s; best_cost = cost; }
    }
    return best;
}

// K split of the last, partly filled round of tiles.  When the tile count is not a multiple
// of the CU count and the contraction is long, the leftover tiles would keep a few CUs busy
// for a whole tile time; they are cut into `*splits` K slices each so that the last round
// fills the chip and takes 1/splits of a tile time.  Returns the workspace bytes (0 = off).
size_t choose_tail_split(int64_t n, int64_t m, int64_t k, int elt, size_t ws_bytes, int* first, int* splits, int* kps) {
    const int CUS = num_cus();
    const int64_t tiles = ((n + BM - 1) / BM) * ((m + BN - 1) / BN);
    const int bk = BKB / elt;
    const int64_t panels = k / bk;
    *first = 0; *splits = 1; *kps = 0;
    const int64_t tail = tiles % CUS, rounds = tiles / CUS;
    if (tiles <= CUS || tail == 0 || tail > CUS / 2 || rounds > 16 || panels < 32 || k % bk != 0) return 0;
    int64_t s = CUS / tail;
    if (s > panels / 8) s = panels / 8;
    if (s > 32) s = 32;
    if (s < 2) return 0;
    int64_t per_panels = (panels + s - 1) / s;
    per_panels += per_panels & 1;                       // the streamed loop takes panels in pairs
    const int64_t per = per_panels * bk;
    s = (k + per - 1) / per;
    if (panels % 2 != 0 || k - (s - 1) * per < 2 * bk) return 0;
    const size_t need = (size_t)tail * s * BM * BN * sizeof(float);
    if (s < 2 || need > ws_bytes) return 0;
    *first = (int)(tiles - tail); *splits = (int)s; *kps = (int)per;
    return need;
}

}  // namespace
