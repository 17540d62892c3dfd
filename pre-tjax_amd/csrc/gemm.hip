// MFMA GEMM for gfx950: C[n,m] = sum_k A(n,k) B(k,m) (+bias[m]) (gelu), fp32 accumulation.
//
// Tiling: one 512-thread workgroup (8 wavefronts, 4 along rows x 2 along columns) owns a
// 256x192 tile of C; each wavefront owns 64x96 = 2x3 MFMA tiles of 32x32
// (v_mfma_f32_32x32x16_bf16, or four v_mfma_f32_32x32x2_f32 per step for fp32 storage).
// 192 divides every feature width of the model (768, 2304, 3072) and 256 divides B*T, so
// the big products fill the 256 CUs in whole rounds.  K advances in panels of 128 BYTES
// per row (64 bf16 / 32 fp32), double-buffered in LDS (2 x 56 KiB): while the MFMAs
// consume buffer p, the next panels travel HBM -> registers -> buffer p^1, one barrier
// per step; two wavefronts per SIMD overlap one's MFMAs with the other's copies.
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
#include "common.h"
#include "mma_tile.h"
#include <type_traits>

namespace {

#ifndef PTJ_GEMM_BM
#define PTJ_GEMM_BM 256
#endif
constexpr int BM = PTJ_GEMM_BM, BN = 192;   // C tile (rows from A, columns from B)
constexpr int WAVES_N = 2;                  // (BM/64) x 2 wavefronts, each 64 rows x 96 columns
constexpr int GEMM_THREADS = (BM / 64) * WAVES_N * 64;
constexpr int TM = 2, TN = 3;           // 32x32 MFMA tiles per wavefront

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
    int epilogue;
};

// A run of K panels [kt0, kt1) of one C tile.  FAST: straight-line vector loads (interior
// tile, whole panels); otherwise the element-wise edge loader.  Written as one flat
// function (no closures) so that the prefetch registers are plain SSA values.
template <typename T, int AMODE, int BMODE, bool FAST>
__device__ __forceinline__ void gemm_run(const GemmArgs& g, f32x16 (&acc)[TN][TM], char* __restrict__ smem, int row0,
                                         int col0, int kbeg, int kend, int kt0, int kt1) {
    constexpr int BK = BKB / (int)sizeof(T);
    if (kt0 >= kt1) return;
    const int tid = threadIdx.x;
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
        if constexpr (FAST) {                                                 \
            la.load_fast(A, g.a_row, g.a_k, row0, k0__, tid);                 \
            lb.load_fast(B, g.b_row, g.b_k, col0, k0__, tid);                 \
        } else {                                                              \
            la.load_edge(A, g.a_row, g.a_k, row0, g.n, k0__, kend, tid);      \
            lb.load_edge(B, g.b_row, g.b_k, col0, g.m, k0__, kend, tid);      \
        }                                                                     \
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
        _Pragma("unroll") for (int t = 0; t < TM; ++t) fa[BUF][t] = read_frag<T>(cA, wm * 64 + t * 32 + lr, q__); \
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

// Writes the wave's 64x96 accumulator block to `dst` (row pitch dst_rs elements of OUT),
// ROWS (32 or 64) rows per pass through a wave-private LDS staging area.
template <typename OUT, typename T, int ROWS, bool EPILOGUE, bool NO_ACT = false>
__device__ __forceinline__ void gemm_store_block(const GemmArgs& g, const f32x16 (&acc)[TN][TM], char* __restrict__ smem,
                                                 int row0, int col0, OUT* __restrict__ dst, int64_t dst_rs) {
    constexpr int PITCH = 96 * (int)sizeof(OUT) + 16;            // bytes per staged row
    constexpr int V = 16 / (int)sizeof(OUT);                     // elements per 16-byte vector
    constexpr int VPR = 96 / V;                                  // vectors per row
    static_assert((GEMM_THREADS / 64) * ROWS * PITCH <= 2 * (BM + BN) * BKB, "staging area");
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int lr = lane & 31, lg = lane >> 5;
    char* stage = smem + wave * (ROWS * PITCH);
    const int gcol0 = col0 + wn * 96;
    const int grow0 = row0 + wm * 64;
    const bool aligned = ((reinterpret_cast<uintptr_t>(dst) & 15) == 0) && (dst_rs % V == 0);
#pragma unroll
    for (int pass = 0; pass < 64 / ROWS; ++pass) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int i4 = 0; i4 < 4; ++i4) {
                const int cc = tn * 32 + i4 * 8 + lg * 4;        // first of 4 columns, block-relative
                float bias4[4] = {0.f, 0.f, 0.f, 0.f};
                if constexpr (EPILOGUE) {
                    if (g.epilogue != PTJ_EPI_NONE) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (gcol0 + cc + e < g.m) bias4[e] = to_f32(((const T*)g.bias)[gcol0 + cc + e]);
                    }
                }
#pragma unroll
                for (int tmi = 0; tmi < ROWS / 32; ++tmi) {
                    const int tm = pass * (ROWS / 32) + tmi;
                    float o[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        o[e] = acc[tn][tm][i4 * 4 + e];
                        if constexpr (EPILOGUE) {
                            o[e] += bias4[e];
                            if (!NO_ACT && g.epilogue == PTJ_EPI_BIAS_GELU) o[e] = gelu_f(o[e]);
                        }
                    }
                    store_vec<OUT, 4>(reinterpret_cast<OUT*>(stage + (tmi * 32 + lr) * PITCH) + cc, o);
                }
            }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");   // the wave re-reads only its own area
#pragma unroll
        for (int it = 0; it < ROWS * VPR / 64; ++it) {
            const int v = it * 64 + lane;
            const int r = v / VPR, c = (v % VPR) * V;
            const int grow = grow0 + pass * ROWS + r;
            const int gcol = gcol0 + c;
            const Pack<OUT, V> val = *reinterpret_cast<const Pack<OUT, V>*>(stage + r * PITCH + c * (int)sizeof(OUT));
            if (grow >= g.n || gcol >= g.m) continue;
            OUT* p = dst + (int64_t)grow * dst_rs + gcol;
            if (aligned && gcol + V <= g.m) {
                *reinterpret_cast<Pack<OUT, V>*>(p) = val;
            } else {
#pragma unroll
                for (int e = 0; e < V; ++e)
                    if (gcol + e < g.m) p[e] = val.v[e];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    }
}

template <typename T, int AMODE, int BMODE>
__global__ __launch_bounds__(GEMM_THREADS, BM == 128 ? 2 : 1) void gemm_kernel(const GemmArgs g) {
    constexpr int BK = BKB / (int)sizeof(T);
    constexpr int TILE_BYTES = 2 * (BM + BN) * BKB;             // 112 KiB of operand panels
    __shared__ __attribute__((aligned(16))) char smem[TILE_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int lr = lane & 31, lg = lane >> 5;

    // ---- workgroup -> tile ---------------------------------------------------------
    const int num_m = (g.n + BM - 1) / BM, num_n = (g.m + BN - 1) / BN;
    const int total = num_m * num_n;
    int pid = blockIdx.x;
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
    const int row0 = tile_m * BM, col0 = tile_n * BN;

    const int kbeg = blockIdx.z * g.k_per_split;
    const int kend = (kbeg + g.k_per_split) < g.k ? (kbeg + g.k_per_split) : g.k;
    const int nk = (kend - kbeg + BK - 1) / BK;

    f32x16 acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    constexpr bool VECTOR_OK = AMODE != GENERIC && BMODE != GENERIC;
    const bool interior = row0 + BM <= g.n && col0 + BN <= g.m;
    const int nk_full = (kend - kbeg) / BK;  // whole panels
    if constexpr (VECTOR_OK) {
        if (interior) {
            gemm_run<T, AMODE, BMODE, true>(g, acc, smem, row0, col0, kbeg, kend, 0, nk_full);
            gemm_run<T, AMODE, BMODE, false>(g, acc, smem, row0, col0, kbeg, kend, nk_full, nk);
        } else {
            gemm_run<T, AMODE, BMODE, false>(g, acc, smem, row0, col0, kbeg, kend, 0, nk);
        }
    } else {
        gemm_run<T, AMODE, BMODE, false>(g, acc, smem, row0, col0, kbeg, kend, 0, nk);
    }

    // ---- epilogue.  acc[tn][tm][i] of lane (lr, lg) is
    //   C[wm*64 + tm*32 + lr][wn*96 + tn*32 + (i/4)*8 + lg*4 + (i%4)].
    // Bias / GELU are applied in registers, the block is converted to the output type and
    // staged in a wave-private LDS area ([rows][96 columns]), then written back as 16-byte
    // vectors that run along whole 96-column rows.  Only wave-local ordering is needed.
    if (g.partial != nullptr) {
        // split-K partial sums: fp32, one 32-row half at a time
        gemm_store_block<float, T, 32, false>(g, acc, smem, row0, col0,
                                              g.partial + (int64_t)blockIdx.z * g.n * (int64_t)g.m, g.m);
    } else {
        if (g.c_aux != nullptr)
            gemm_store_block<T, T, sizeof(T) == 2 ? 64 : 32, true, true>(g, acc, smem, row0, col0, (T*)g.c_aux,
                                                                         g.c_aux_rs);
        gemm_store_block<T, T, sizeof(T) == 2 ? 64 : 32, true>(g, acc, smem, row0, col0, (T*)g.c, g.c_rs);
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
        if (c_aux != nullptr) c_aux[(int64_t)row * c_aux_rs + col] = from_f32<T>(s);
        if (epilogue == PTJ_EPI_BIAS_GELU) s = gelu_f(s);
        c[(int64_t)row * c_rs + col] = from_f32<T>(s);
    }
}

template <typename T>
int pick_mode(const void* p, int64_t s_row, int64_t s_k) {
    constexpr int VEC = VecOf<T>::N;
    if (!ptj_aligned16(p)) return GENERIC;
    if (s_k == 1 && s_row % VEC == 0) return KMAJOR;
    if (s_row == 1 && s_k % VEC == 0) return MNMAJOR;
    return GENERIC;
}

template <typename T>
int gemm_impl(GemmArgs g, int splits, hipStream_t st) {
    const int am = pick_mode<T>(g.a, g.a_row, g.a_k), bm = pick_mode<T>(g.b, g.b_row, g.b_k);
    const int num_m = (g.n + BM - 1) / BM, num_n = (g.m + BN - 1) / BN;
    dim3 grid(num_m * num_n, 1, splits), block(GEMM_THREADS);
#define GEMM_LAUNCH(AM, BMD) hipLaunchKernelGGL((gemm_kernel<T, AM, BMD>), grid, block, 0, st, g)
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
#undef GEMM_LAUNCH
    PTJ_CHECK_LAUNCH();
    if (splits > 1) {
        const int64_t total = (int64_t)g.n * g.m;
        int64_t blocks = (total + 255) / 256;
        if (blocks > 256 * 8) blocks = 256 * 8;
        hipLaunchKernelGGL((gemm_splitk_reduce_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st,
                           (const float*)g.partial, splits, g.n, g.m, (T*)g.c, g.c_rs, (const T*)g.bias, g.epilogue,
                           (T*)g.c_aux, g.c_aux_rs);
        PTJ_CHECK_LAUNCH();
    }
    return PTJ_OK;
}

// Number of K splits for an (n, m, k) problem given `ws_bytes` of workspace.
// Picks the split count that minimises a small cost model: the workgroups run in rounds
// of one per CU, a workgroup costs a fixed prologue/epilogue plus a per-panel time, and
// every split writes and re-reads an fp32 copy of C.
int choose_splits(int64_t n, int64_t m, int64_t k, int elt, size_t ws_bytes) {
    constexpr int CUS = 256;
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

}  // namespace

extern "C" {

size_t ptj_gemm_workspace_bytes(int64_t n, int64_t m, int64_t k, int dtype) {
    if (n <= 0 || m <= 0 || k <= 0) return 0;
    const int elt = dtype == PTJ_BF16 ? 2 : 4;
    const int s = choose_splits(n, m, k, elt, (size_t)-1);
    return s > 1 ? (size_t)s * n * m * sizeof(float) : 0;
}

int ptj_gemm(const void* a, const void* b, void* c, const void* bias, int64_t n, int64_t m, int64_t k, int64_t a_rs,
             int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t c_rs, int epilogue, void* c_pre, int64_t c_pre_rs,
             void* workspace, size_t workspace_bytes, int dtype, void* stream) {
    PTJ_CHECK_ARG(n >= 0 && m >= 0 && k >= 0, "gemm: negative dimension");
    PTJ_CHECK_ARG(n < (1ll << 31) && m < (1ll << 31) && k < (1ll << 31), "gemm: dimension exceeds 31 bits");
    PTJ_CHECK_ARG(epilogue >= PTJ_EPI_NONE && epilogue <= PTJ_EPI_BIAS_GELU, "gemm: unknown epilogue %d", epilogue);
    PTJ_CHECK_ARG(epilogue == PTJ_EPI_NONE || bias, "gemm: epilogue %d needs a bias", epilogue);
    PTJ_CHECK_ARG(dtype == PTJ_F32 || dtype == PTJ_BF16, "gemm: unknown dtype %d", dtype);
    if (n == 0 || m == 0) return PTJ_OK;
    PTJ_CHECK_ARG(c && (k == 0 || (a && b)), "gemm: null pointer");
    PTJ_CHECK_ARG(c_rs >= m, "gemm: c row stride %lld < m %lld", (long long)c_rs, (long long)m);
    PTJ_CHECK_ARG(!c_pre || (epilogue == PTJ_EPI_BIAS_GELU && c_pre_rs >= m),
                  "gemm: c_pre needs the bias+GELU epilogue and a row stride >= m");
    const int elt = dtype == PTJ_BF16 ? 2 : 4;
    const int bk = BKB / elt;
    GemmArgs g;
    g.a = a; g.b = b; g.c = c; g.bias = bias;
    g.n = (int)n; g.m = (int)m; g.k = (int)k;
    g.a_row = a_rs; g.a_k = a_cs;
    g.b_row = b_cs; g.b_k = b_rs;
    g.c_rs = c_rs;
    g.c_aux = c_pre;
    g.c_aux_rs = c_pre_rs;
    g.epilogue = epilogue;
    int splits = workspace ? choose_splits(n, m, k, elt, workspace_bytes) : 1;
    int64_t kps = k;
    if (splits > 1) {
        kps = ((k + splits - 1) / splits + bk - 1) / bk * bk;
        splits = (int)((k + kps - 1) / kps);
    }
    if (kps < 1) kps = bk;  // k == 0: one empty pass writes bias / zeros
    g.k_per_split = (int)kps;
    g.partial = splits > 1 ? (float*)workspace : nullptr;
    hipStream_t st = (hipStream_t)stream;
    return dtype == PTJ_F32 ? gemm_impl<float>(g, splits, st) : gemm_impl<bf16>(g, splits, st);
}

}  // extern "C"
