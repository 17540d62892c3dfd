// Main loop of the bf16 GEMM whose operand panels travel HBM -> LDS by asynchronous copies
// (global_load_lds, 16 bytes per lane): no staging registers, no LDS store instructions, no
// register transposes.  Included by gemm_core.h inside its unnamed namespace; uses its tile
// geometry (256x192 tile of C, eight wavefronts of 64x96), epilogues and work-item order.
//
// LDS map: [A stage 0][A stage 1][B stage 0][B stage 1][output staging of gemm_store_block];
// a stage holds one K panel of 64 contraction elements (32 KiB of A rows, 24 KiB of B rows).
//
// An operand whose contiguous axis is K (KMAJOR) is stored as in the staged kernel: [row][128
// bytes], 16-byte chunks XOR-swizzled by sw(row); a copy instruction covers eight rows and the
// swizzle is applied by choosing which global chunk each lane fetches.  A fragment is one
// ds_read_b128.
//
// An operand whose contiguous axis is the row axis (MNMAJOR: the .t() views of the dX and dW
// products) is stored as it lies in memory: [k][rows], whole cache lines per copy, and a
// fragment is two transposing reads (ds_read_b64_tr_b16: sixteen lanes fetch a 4 (k) x 16
// (rows) block and each ends up with four consecutive k of one row).  The 16-byte pieces of a
// k-row are XORed with a function of k mod 4 so that the four k-rows a lane group reads fall
// into different banks.
//
// Schedule of one K step (24 MFMAs per wavefront): the fragments of contraction chunk c+1 are
// requested in a burst while the six MFMAs of chunk c run; before the last chunk every
// wavefront waits for its own copies of the next panel and for its LDS reads, one barrier
// follows, and right after it the stage just vacated is refilled with the panel two steps
// ahead (also across work items: the copies run ahead into the next tile, and the epilogue,
// which stages through its own LDS area, overlaps them).  LDS reads and their waits are
// written by hand: the compiler does not see the asynchronous copies as producers of what a
// later ds_read returns.
#pragma once

typedef uint32_t dg_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t dg_u32x4 __attribute__((ext_vector_type(4)));

constexpr int DG_A_BYTES = BM * BKB;              // one stage of A: 32 KiB
constexpr int DG_B_BYTES = BN * BKB;              // one stage of B: 24 KiB
constexpr int DG_B_BASE = 2 * DG_A_BYTES;         // the B stages follow the two A stages
static_assert(2 * (DG_A_BYTES + DG_B_BYTES) == PANEL_BYTES, "same panel area as the staged kernel");
static_assert(BM == 256 && BN == 192 && TM == 2 && TN == 3 && GEMM_THREADS == 512, "geometry of the direct loop");

__device__ __forceinline__ uint32_t dg_lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
// piece swizzle of an MNMAJOR stage: XORed into the index of a 16-byte piece inside its k-row
template <int ROWS> __device__ __forceinline__ int dg_mn_swz(int k) { return (ROWS == 256 ? 10 : 2) * (k & 3); }

// One MFMA operand fragment (eight bf16 per lane) and how it is read from a stage.
template <int MODE> struct DgFrag;
template <> struct DgFrag<KMAJOR> {
    dg_u32x4 v;
    // OFF: byte offset of the tile's first row (t * 32 rows); the chunk is in the address
    template <int OFF, int PITCH, int KOFF>
    __device__ __forceinline__ void read(uint32_t addr) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    }
    __device__ __forceinline__ void landed() { asm volatile("" : "+v"(v)); }
    __device__ __forceinline__ bf16x8 get() const { return __builtin_bit_cast(bf16x8, v); }
};
template <> struct DgFrag<MNMAJOR> {
    dg_u32x2 lo, hi;
    // KOFF: first k-row of the contraction chunk (16 c); the two reads fetch k + 0..3 and k + 4..7
    template <int OFF, int PITCH, int KOFF>
    __device__ __forceinline__ void read(uint32_t addr) {
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(addr), "n"(KOFF * PITCH));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"((KOFF + 4) * PITCH));
    }
    __device__ __forceinline__ void landed() { asm volatile("" : "+v"(lo), "+v"(hi)); }
    __device__ __forceinline__ bf16x8 get() const {
        const dg_u32x4 q = {lo[0], lo[1], hi[0], hi[1]};
        return __builtin_bit_cast(bf16x8, q);
    }
};

// Per-lane state of one operand: where its copies fetch from and where its fragments are read.
//   ROWS  256 (A: rows of C) or 192 (B: columns of C);  NT tiles of 32 rows per wavefront (2 / 3)
template <int MODE, int ROWS, int NT>
struct DgOperand {
    static constexpr int PER = ROWS / 64;                  // copies per wavefront and stage: 4 / 3
    static constexpr int PITCH = ROWS * 2;                 // MNMAJOR: bytes per k-row
    static constexpr int NADDR = MODE == KMAJOR ? 4 : NT;  // fragment base addresses (per chunk / per tile)
    uint32_t goff[PER];     // byte offset of the lane's 16 bytes from the panel's base, per copy
    uint32_t raddr[NADDR];  // LDS byte address of the lane's fragments in stage 0

    // copy geometry for the tile whose first row is row0 (CLAMP: rows past nrows - 1 re-read the last one)
    template <bool CLAMP>
    __device__ __forceinline__ void set_tile(int64_t s_row, int64_t s_k, int row0, int nrows, int tid) {
        const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int inst = wave * PER + i;
            if constexpr (MODE == KMAJOR) {
                const int r = inst * 8 + (lane >> 3);
                const int chunk = (lane & 7) ^ sw(r);
                int grow = row0 + r;
                if (CLAMP) grow = grow < nrows ? grow : nrows - 1;
                goff[i] = ((uint32_t)grow * (uint32_t)s_row + (uint32_t)chunk * 8u) * 2u;
            } else {
                constexpr int PPR = ROWS / 8;              // 16-byte pieces per k-row
                const int p = inst * 64 + lane;
                const int k = p / PPR, pos = p - k * PPR;
                int grow = row0 + (pos ^ dg_mn_swz<ROWS>(k)) * 8;
                if (CLAMP) {
                    const int lastv = ((nrows - 1) >> 3) << 3;   // a .t() view's pitch covers this vector
                    grow = grow < lastv ? grow : lastv;
                }
                goff[i] = ((uint32_t)k * (uint32_t)s_k + (uint32_t)grow) * 2u;
            }
        }
    }

    // fragment addresses of the wavefront whose first row inside the tile is wrow
    __device__ __forceinline__ void set_reads(uint32_t region, int wrow, int tid) {
        const int lane = tid & 63;
        if constexpr (MODE == KMAJOR) {
            const int row = wrow + (lane & 31), lg = lane >> 5;
#pragma unroll
            for (int c = 0; c < 4; ++c) raddr[c] = region + row * BKB + (((c * 2 + lg) ^ sw(row)) << 4);
        } else {
            const int l16 = lane & 15, mhalf = (lane >> 4) & 1, lg = lane >> 5;
            const int kq = l16 >> 2;                        // k mod 4 of the k-row this lane addresses
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int piece = (wrow >> 3) + t * 4 + 2 * mhalf + ((l16 & 3) >> 1);
                raddr[t] = region + (8 * lg + kq) * PITCH + ((piece ^ dg_mn_swz<ROWS>(kq)) << 4) + 8 * (l16 & 1);
            }
        }
    }

    // copies [I0, I1) of the panel whose base is `panel` into the stage at LDS address `stage` (wave-uniform)
    template <int I0, int I1>
    __device__ __forceinline__ void copy(const char* __restrict__ panel, char* __restrict__ stage, int wave) const {
#pragma unroll
        for (int i = I0; i < I1; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(panel + goff[i]),
                                             (__attribute__((address_space(3))) void*)(stage + (wave * PER + i) * 1024),
                                             16, 0, 0);
    }

    // fragments of contraction chunk C of the stage at byte offset soff
    template <int C>
    __device__ __forceinline__ void read_chunk(DgFrag<MODE> (&f)[NT], uint32_t soff) const {
        if constexpr (MODE == KMAJOR) {
            const uint32_t a = raddr[C] + soff;
            f[0].template read<0, 0, 0>(a);
            f[1].template read<32 * BKB, 0, 0>(a);
            if constexpr (NT == 3) f[2].template read<64 * BKB, 0, 0>(a);
        } else {
            f[0].template read<0, PITCH, 16 * C>(raddr[0] + soff);
            f[1].template read<0, PITCH, 16 * C>(raddr[1] + soff);
            if constexpr (NT == 3) f[2].template read<0, PITCH, 16 * C>(raddr[2] + soff);
        }
    }
};

// A work item of the persistent grid: a C tile, or one K slice of one.
struct DgItem {
    int row0, col0, kbeg, nk, z;
    float* part;   // dense partial tile of a K-split tile of the last round (nullptr otherwise)
};
__device__ __forceinline__ DgItem dg_item(const GemmArgs& g, int item, int num_m, int num_n) {
    const int total = num_m * num_n;
    DgItem d;
    d.z = 0;
    d.part = nullptr;
    if (g.tail_splits > 1 && item >= g.tail_first) {
        const int r = item - g.tail_first;
        const int t = r / g.tail_splits;
        d.z = r - t * g.tail_splits;
        tile_origin(g.tail_first + t, total, num_m, num_n, d.row0, d.col0);
        d.kbeg = d.z * g.tail_kps;
        d.nk = ((d.kbeg + g.tail_kps < g.k ? d.kbeg + g.tail_kps : g.k) - d.kbeg) / 64;
        d.part = g.partial + (int64_t)r * (BM * BN);
    } else if (g.splits > 1) {
        // the items of one XCD share operand slices: the tiles along the smaller C dimension vary
        // fastest, then the tiles along the larger one, then the K split
        const int work = total * g.splits;
        const int chunk = work >> 3, rem = work & 7, x = item & 7;
        const int idx = x * chunk + (x < rem ? x : rem) + (item >> 3);
        int tile_m, tile_n;
        if (g.n >= g.m) {
            tile_n = idx % num_n;
            const int pair = idx / num_n;
            tile_m = pair % num_m;
            d.z = pair / num_m;
        } else {
            tile_m = idx % num_m;
            const int pair = idx / num_m;
            tile_n = pair % num_n;
            d.z = pair / num_n;
        }
        d.row0 = tile_m * BM;
        d.col0 = tile_n * BN;
        d.kbeg = d.z * g.k_per_split;
        d.nk = ((d.kbeg + g.k_per_split < g.k ? d.kbeg + g.k_per_split : g.k) - d.kbeg) / 64;
    } else {
        tile_origin(item, total, num_m, num_n, d.row0, d.col0);
        d.kbeg = 0;
        d.nk = g.k / 64;
    }
    return d;
}

// PTJ_EPI_ACCUMULATE: the accumulators of the tile at (row0, col0) start from the stored C.  acc[tn][tm][i] of
// lane (lr, lg) is C[row0 + wm*64 + tm*32 + lr][col0 + wn*96 + tn*32 + (i/4)*8 + lg*4 + i%4]: four consecutive
// columns per load.  Elements outside C start from zero (their results are never stored).
template <bool CLAMP>
__device__ __forceinline__ void dg_load_c_tile(const GemmArgs& g, f32x16 (&acc)[TN][TM], int row0, int col0) {
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lg = lane >> 5;
    const int r0 = row0 + (wave / WAVES_N) * WROWS + lr, c0 = col0 + (wave % WAVES_N) * 96 + lg * 4;
    const bf16* C = (const bf16*)g.c;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int row = r0 + tm * 32, col = c0 + tn * 32 + q * 8;
                Pack<bf16, 4> v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v.v[e] = from_f32<bf16>(0.f);
                if (!CLAMP || (row < g.n && col + 4 <= g.m)) {
                    v = *reinterpret_cast<const Pack<bf16, 4>*>(C + (int64_t)row * g.c_rs + col);
                } else if (row < g.n) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < g.m) v.v[e] = C[(int64_t)row * g.c_rs + col + e];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[tn][tm][q * 4 + e] = to_f32(v.v[e]);
            }
}

template <int AMODE, int BMODE, bool CLAMP, bool MUL>
__device__ __forceinline__ void gemm_direct(const GemmArgs& g, char* __restrict__ smem) {
    typedef bf16 T;
    const int num_m = (g.n + BM - 1) / BM, num_n = (g.m + BN - 1) / BN;
    const int total = num_m * num_n;
    const int work = g.tail_splits > 1 ? g.tail_first + (total - g.tail_first) * g.tail_splits : total * g.splits;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    DgOperand<AMODE, BM, TM> oa;
    DgOperand<BMODE, BN, TN> ob;
    oa.set_reads(dg_lds_addr(smem), wm * WROWS, tid);
    ob.set_reads(dg_lds_addr(smem) + DG_B_BASE, wn * 96, tid);
    const int64_t a_step = AMODE == KMAJOR ? 2 : 2 * g.a_k;   // bytes per contraction element along the panel axis
    const int64_t b_step = BMODE == KMAJOR ? 2 : 2 * g.b_k;

    // ---- fetch cursor: runs two panels ahead of the multiplications, across work items
    int f_item = blockIdx.x;
    DgItem f = dg_item(g, f_item, num_m, num_n);
    int f_k = f.kbeg, f_left = f.nk;
    bool f_valid = true;
    oa.template set_tile<CLAMP>(g.a_row, g.a_k, f.row0, g.n, tid);
    ob.template set_tile<CLAMP>(g.b_row, g.b_k, f.col0, g.m, tid);
#define DG_COPY_A(I0, I1, ST)                                                                               \
    do {                                                                                                    \
        if (f_valid) oa.template copy<I0, I1>((const char*)g.a + (int64_t)f_k * a_step, smem + (ST) * DG_A_BYTES, wave); \
    } while (0)
#define DG_COPY_B(I0, I1, ST)                                                                               \
    do {                                                                                                    \
        if (f_valid) ob.template copy<I0, I1>((const char*)g.b + (int64_t)f_k * b_step, smem + DG_B_BASE + (ST) * DG_B_BYTES, wave); \
    } while (0)
#define DG_ADVANCE()                                                                                        \
    do {                                                                                                    \
        f_k += 64;                                                                                          \
        if (--f_left == 0) {                                                                                \
            f_item += (int)gridDim.x;                                                                       \
            if (f_item < work) {                                                                            \
                f = dg_item(g, f_item, num_m, num_n);                                                       \
                f_k = f.kbeg;                                                                               \
                f_left = f.nk;                                                                              \
                oa.template set_tile<CLAMP>(g.a_row, g.a_k, f.row0, g.n, tid);                              \
                ob.template set_tile<CLAMP>(g.b_row, g.b_k, f.col0, g.m, tid);                              \
            } else {                                                                                        \
                f_valid = false;                                                                            \
            }                                                                                               \
        }                                                                                                   \
    } while (0)
#define DG_SB() __builtin_amdgcn_sched_barrier(0)

    DgFrag<AMODE> fa[2][TM];
    DgFrag<BMODE> fb[2][TN];
#define DG_READ(SET, C, SOFF_A, SOFF_B)                                                                     \
    do {                                                                                                    \
        oa.template read_chunk<C>(fa[SET], SOFF_A);                                                         \
        ob.template read_chunk<C>(fb[SET], SOFF_B);                                                         \
    } while (0)
#define DG_LANDED(SET)                                                                                      \
    do {                                                                                                    \
        _Pragma("unroll") for (int t = 0; t < TM; ++t) fa[SET][t].landed();                                 \
        _Pragma("unroll") for (int t = 0; t < TN; ++t) fb[SET][t].landed();                                 \
    } while (0)
#define DG_MM(SET, TNI)                                                                                     \
    do {                                                                                                    \
        const bf16x8 b__ = fb[SET][TNI].get();                                                              \
        _Pragma("unroll") for (int tm = 0; tm < TM; ++tm) mma_chunk(acc[TNI][tm], b__, fa[SET][tm].get());  \
    } while (0)

    // ---- prologue: the first panel lands, the second is requested, the first fragments are read
    DG_COPY_A(0, 4, 0);
    DG_COPY_B(0, 3, 0);
    DG_ADVANCE();
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    DG_COPY_A(0, 4, 1);
    DG_COPY_B(0, 3, 1);
    DG_ADVANCE();
    DG_READ(0, 0, 0u, 0u);
    int pb = 0;   // stage that holds the panel being multiplied

    int item = blockIdx.x;
    DgItem cur = dg_item(g, item, num_m, num_n);
    Pack<T, 4> braw[TN * 4];
    load_bias_quads<T, CLAMP>(g, cur.col0, braw, cur.part != nullptr || g.splits > 1);
    for (;;) {
        const int nitem = item + (int)gridDim.x;
        const bool more = nitem < work;
        const DgItem nxt = dg_item(g, more ? nitem : item, num_m, num_n);
        f32x16 acc[TN][TM];
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
            for (int j = 0; j < TM; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = to_f32(braw[i * 4 + (e >> 2)].v[e & 3]);
        if constexpr (!MUL) {
            if (g.epilogue == PTJ_EPI_ACCUMULATE) dg_load_c_tile<CLAMP>(g, acc, cur.row0, cur.col0);
        }
        for (int kt = 0; kt < cur.nk; ++kt) {
            const uint32_t sa = pb * DG_A_BYTES, sb = pb * DG_B_BYTES;
            const uint32_t na = (pb ^ 1) * DG_A_BYTES, nb = (pb ^ 1) * DG_B_BYTES;
            // chunk 0 (set 0) while chunk 1 is read into set 1
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            DG_LANDED(0);
            DG_READ(1, 1, sa, sb); DG_SB();
            DG_MM(0, 0); DG_MM(0, 1); DG_MM(0, 2); DG_SB();
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            DG_LANDED(1);
            DG_READ(0, 2, sa, sb); DG_SB();
            DG_MM(1, 0); DG_MM(1, 1); DG_MM(1, 2); DG_SB();
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            DG_LANDED(0);
            DG_READ(1, 3, sa, sb); DG_SB();
            DG_MM(0, 0); DG_MM(0, 1); DG_MM(0, 2); DG_SB();
            // this wavefront's copies of the next panel have landed and its reads of this stage are
            // done; after the barrier that holds for every wavefront: the next panel may be read and
            // this stage refilled
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
            DG_LANDED(1);
            DG_READ(0, 0, na, nb); DG_SB();
            DG_MM(1, 0); DG_SB();
            DG_COPY_A(0, 3, pb); DG_SB();
            DG_MM(1, 1); DG_SB();
            DG_COPY_A(3, 4, pb); DG_COPY_B(0, 1, pb); DG_SB();
            DG_MM(1, 2); DG_SB();
            DG_COPY_B(1, 3, pb);
            DG_ADVANCE();
            DG_SB();
            pb ^= 1;
        }
        load_bias_quads<T, CLAMP>(g, nxt.col0, braw, nxt.part != nullptr || g.splits > 1);
        if (cur.part != nullptr) gemm_store_block<float, T, false, 0, true>(g, acc, smem, 0, 0, cur.part, BN);
        else if (g.splits > 1) gemm_epilogue<T, false, true>(g, acc, smem, cur.row0, cur.col0, cur.z);
        else gemm_epilogue<T, false, false, MUL>(g, acc, smem, cur.row0, cur.col0, 0);
        if (!more) break;
        item = nitem;
        cur = nxt;
    }
    // nothing of this workgroup may still be on its way into LDS when its wavefronts end
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
#undef DG_COPY_A
#undef DG_COPY_B
#undef DG_ADVANCE
#undef DG_SB
#undef DG_READ
#undef DG_LANDED
#undef DG_MM
}

// Persistent kernel around gemm_direct: one workgroup per CU, eight wavefronts.
template <int AMODE, int BMODE, bool MUL>
__global__ __launch_bounds__(GEMM_THREADS, 1) void gemm_direct_kernel(const GemmArgs g) {
    __shared__ __attribute__((aligned(1024))) char smem[SMEM_BYTES];
    if (g.n % BM == 0 && g.m % BN == 0) gemm_direct<AMODE, BMODE, false, MUL>(g, smem);
    else gemm_direct<AMODE, BMODE, true, MUL>(g, smem);
}

// Whether a launch can take the direct loop: 2-byte operands in one of the two vector layouts, whole
// panels of 64 contraction elements, and 32-bit byte offsets inside a tile's panels.
inline bool dg_eligible(const GemmArgs& g, int am, int bm) {
    if (am == GENERIC || bm == GENERIC || g.k < 64 || g.k % 64 != 0) return false;
    if (g.splits > 1 && g.k_per_split % 64 != 0) return false;
    if (g.tail_splits > 1 && g.tail_kps % 64 != 0) return false;
    const double lim = 2147483648.0;
    const double ao = am == KMAJOR ? (double)g.n * (double)g.a_row * 2 : 64.0 * (double)g.a_k * 2 + (double)g.n * 2;
    const double bo = bm == KMAJOR ? (double)g.m * (double)g.b_row * 2 : 64.0 * (double)g.b_k * 2 + (double)g.m * 2;
    return ao < lim && bo < lim && g.a_row >= 0 && g.a_k >= 0 && g.b_row >= 0 && g.b_k >= 0;
}
