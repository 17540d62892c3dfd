// Causal flash attention for gfx950, head dimension 64: forward, and a backward that
// recomputes P from the saved row max / row sum-exp.
//
// Layout trick shared by the three MFMA kernels: scores are produced TRANSPOSED.  With
// 32x32 MFMA tiles, D[m][n] of lane l sits at n = l & 31, m = 8*(i/4) + 4*(l>>5) + i%4
// (register i).  Forward and the dQ pass compute S^T = K Q^T, so a lane owns ONE query
// (n) and 16 keys per 32-key tile (m): row max / row sum / rescaling are per-lane
// scalars (one cross-lane exchange with lane^32), and the probabilities are already in
// MFMA B-operand position for O^T = V^T P^T (contraction over keys, which live in the
// lane's registers), so P never travels through LDS.  The dK/dV pass computes S = Q K^T
// with the same trick mirrored: a lane owns one key, dV^T = dO^T P and dK^T = Q^T dS.
// The operand that must be read "across" its memory layout (V^T, K^T, Q^T, dO^T: row
// index d, contraction along keys / queries) is transposed once while it is written to
// LDS (MNMAJOR panel loader, quads paired so that the eight positions a lane holds of an
// accumulator tile are one 16-byte chunk) and shared by the four wavefronts.
//
// Softmax is evaluated in base 2 (scores pre-multiplied by log2(e)/sqrt(dh)); the saved
// statistics `ms` are converted back to natural units.  Masked scores take the
// reference's fill value -1e9 (not -inf); the running maximum starts above it, so a masked
// element contributes exactly 0.  A row without any visible key therefore has sum-exp 0: its
// output row is 0, its saved statistics are (ms, ls) = (-1e9, 0), and the backward gives it
// (and takes from it) no gradient.
//
// An explicit mask arrives bit-packed in both orientations together with one class per 32x32
// tile of (mask AND causal): hidden everywhere / mixed / equal to the causal pattern.  Hidden
// tiles are skipped, tiles equal to the causal pattern run the index-masked code, and only
// mixed tiles read their mask words -- a plain lower-triangular tensor costs what mask = NULL
// costs, and packed documents cost what they attend to.
//
// Dropout on the probabilities: element (q, k) of batch-head g is kept iff
// philox(seed + g, q + k) passes the threshold -- the offset depends on q + k only, so
// one line of 2T keep bits per batch-head is generated once (attn_keepbits_kernel); the
// kernels read it through the scalar unit and turn it into 64-lane select masks.
//
// The backward is two passes without atomics: dQ over query tiles (it also forms
// delta = rowsum(dO * O) of its queries and stores it), then (dK, dV) over key tiles,
// which reads delta; both recompute S and dP.
#include "common.h"
#include "mma_tile.h"

namespace {

constexpr int DH = 64;
constexpr int ATT_THREADS = 256;
constexpr int PANEL = 64 * BKB;  // bytes of one 64-row LDS panel
constexpr int MAX_T = 8192;
constexpr int MAX_BITWORDS = 2 * MAX_T / 32 + 2;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr float NEG_NAT = -1e9f;
constexpr float NEG2 = NEG_NAT * LOG2E;

template <typename T> struct AT {
    static constexpr int ROWB = DH * (int)sizeof(T);   // bytes per q/k/v row: 128 / 256
    static constexpr int NP = ROWB / BKB;               // panels per 64-element axis: 1 / 2
    static constexpr int NC = ROWB / 32;                // contraction chunks along d: 4 / 8
    static constexpr int EPP = BKB / (int)sizeof(T);    // elements per panel row: 64 / 32
    typedef typename Frag<T>::type F;
};

struct AttnArgs {
    const void *q, *k, *v, *o, *d_o;
    void *out0, *out1;            // fwd: out0 = O.  bwd dkdv: out0 = dK, out1 = dV.  bwd dq: out0 = dQ
    // nullptr = causal by index; else the mask bit-packed in both orientations (ptj_attn_pack_mask):
    //   words [0, B*T/32*T):   word (b, q/32, k) holds M[b, 32*(q/32) + r, k] in bit r   (lane = query)
    //   then the same amount:  word (b, k/32, q) holds M[b, q, 32*(k/32) + r] in bit r   (lane = key)
    //   then B*(T/32)^2 words:  class of tile (b, q/32, k/32), then the same indexed (b, k/32, q/32)
    const uint32_t* mask;
    float *ms, *ls;               // [BH, T]
    float* delta;                 // [BH, T] rowsum(dO * O)  (backward: written by the dQ pass, read by the dK/dV pass)
    const uint32_t* keepbits;     // [BH, bitwords]  (train)
    int B, H, T, bitwords;
    // element strides: batch, head, row (the head dimension itself has unit stride)
    int64_t q_bs, q_hs, q_rs, k_bs, k_hs, k_rs, v_bs, v_hs, v_rs, o_bs, o_hs, o_rs, do_bs, do_hs, do_rs;
    int64_t out0_bs, out0_hs, out0_rs, out1_bs, out1_hs, out1_rs;
    int train;
    float scale;                  // 1/sqrt(dh)
};

// ---- small device helpers -----------------------------------------------------------
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }
// max / sum of a value with its partner in the other half of the wavefront (lane ^ 32), the same
// in both lanes: v_permlane32_swap exchanges the upper half of one register with the lower half
// of another inside the vector ALU (no LDS round trip); with both registers holding v the two
// results are {lo, lo} and {hi, hi}.
__device__ __forceinline__ float max_xor32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_xor32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The 16-byte operand pieces of one 64-element row held in registers (lane half lg).
template <typename T>
__device__ __forceinline__ void load_row_frags(typename AT<T>::F (&f)[AT<T>::NC], const T* __restrict__ row, int lg) {
#pragma unroll
    for (int c = 0; c < AT<T>::NC; ++c)
        f[c] = *reinterpret_cast<const typename AT<T>::F*>(reinterpret_cast<const char*>(row) + c * 32 + lg * 16);
}

// s += panel_rows(j*32 + lr) x register_rows : panel rows become MFMA rows (m), the
// lane's register row the MFMA column (n); contraction over the 64-element axis d.
template <typename T>
__device__ __forceinline__ void rows_x_frags_one(f32x16& s, const char* __restrict__ panels,
                                                 const typename AT<T>::F (&f)[AT<T>::NC], int j, int lr, int lg) {
#pragma unroll
    for (int c = 0; c < AT<T>::NC; ++c) {
        typename AT<T>::F a = read_frag<T>(panels + (c / 4) * PANEL, j * 32 + lr, (c % 4) * 2 + lg);
        mma_chunk(s, a, f[c]);
    }
}
template <typename T>
__device__ __forceinline__ void rows_x_frags(f32x16 (&s)[2], const char* __restrict__ panels,
                                             const typename AT<T>::F (&f)[AT<T>::NC], int lr, int lg) {
#pragma unroll
    for (int c = 0; c < AT<T>::NC; ++c) {
        const char* pp = panels + (c / 4) * PANEL;
        const int q = (c % 4) * 2 + lg;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            typename AT<T>::F a = read_frag<T>(pp, j * 32 + lr, q);
            mma_chunk(s[j], a, f[c]);
        }
    }
}

// Eight floats -> eight bf16, converted two at a time (one packed conversion per pair).
__device__ __forceinline__ bf16x8 pack8_bf16(const float* __restrict__ p) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    u32x4_t w;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const f32x2_t f = {p[2 * e], p[2 * e + 1]};
        w[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
    }
    return __builtin_bit_cast(bf16x8, w);
}

// o[t] += transposed_panel_rows(t*32 + lr) x p : contraction over the 32 positions of
// sub-tile j whose values p[i] the lane holds in accumulator order
// (position = j*32 + 8*(i/4) + 4*lg + i%4).
__device__ __forceinline__ void tp_x_regs_one(f32x16 (&o)[2], const char* __restrict__ panels, const float (&p)[16],
                                              int j, int lr, int lg, bf16) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const bf16x8 b = pack8_bf16(&p[8 * h]);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            // the panel was stored with paired quads: chunk 4j + 2h + lg holds exactly the eight
            // positions of b, in the same order
            const bf16x8 a = read_frag<bf16>(panels, t * 32 + lr, 4 * j + 2 * h + lg);
            o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, o[t], 0, 0, 0);
        }
    }
}
__device__ __forceinline__ void tp_x_regs_one(f32x16 (&o)[2], const char* __restrict__ panels, const float (&p)[16],
                                              int j, int lr, int lg, float) {
    const char* pp = panels + j * PANEL;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const f32x4 v = read_frag<float>(pp, t * 32 + lr, 2 * a + lg);
#pragma unroll
            for (int b = 0; b < 4; ++b) o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(v[b], p[4 * a + b], o[t], 0, 0, 0);
        }
}
template <typename T>
__device__ __forceinline__ void tp_x_regs(f32x16 (&o)[2], const char* __restrict__ panels, const float (&p)[2][16],
                                          int lr, int lg, T tag) {
#pragma unroll
    for (int j = 0; j < 2; ++j) tp_x_regs_one(o, panels, p[j], j, lr, lg, tag);
}

// Keep bits of one wavefront tile as wave-uniform (scalar) words.  Element (q, k) is kept
// iff bit q + k of the batch-head's line is set.  In the kernels whose lanes are queries
// (keys), the element in accumulator register i of sub-tile j sits at
//   q + k = base + C + (lane & 31) + 4 * (lane >> 5),   C = 32 j + 8 (i / 4) + i % 4,
// with base = (wave's first query) + (tile's first key), a multiple of 32.  So the keep
// decision of ONE register across the 64 lanes is two 32-bit windows of the line at the
// constant offsets C and C + 4: a lane mask that the scalar unit extracts with two
// shifts and that a single v_cndmask applies -- no per-lane bit arithmetic at all.
struct KeepWords { uint32_t d0, d1, d2; };
__device__ __forceinline__ KeepWords load_keep_words(const uint32_t* __restrict__ line, int base) {
    const uint32_t* p = line + (base >> 5);   // wave-uniform address: scalar loads
    KeepWords w;
    w.d0 = p[0];
    w.d1 = p[1];
    w.d2 = p[2];
    return w;
}
template <int C> __device__ __forceinline__ uint32_t keep_win32(const KeepWords& w) {
    static_assert(C >= 0 && C < 64, "window offset");
    const uint64_t v = C < 32 ? (((uint64_t)w.d1 << 32) | w.d0) : (((uint64_t)w.d2 << 32) | w.d1);
    return (uint32_t)(v >> (C & 31));
}
template <int C> __device__ __forceinline__ uint64_t keep_lane_mask(const KeepWords& w) {
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    const u32x2_t halves = {keep_win32<C>(w), keep_win32<C + 4>(w)};
    return __builtin_bit_cast(uint64_t, halves);
}
// The same for an offset that is a constant only after loop unrolling.
__device__ __forceinline__ uint64_t keep_lane_mask_at(const KeepWords& w, int c) {
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    const uint64_t lo_pair = ((uint64_t)w.d1 << 32) | w.d0, hi_pair = ((uint64_t)w.d2 << 32) | w.d1;
    const int c4 = c + 4;
    const u32x2_t halves = {(uint32_t)((c < 32 ? lo_pair : hi_pair) >> (c & 31)),
                            (uint32_t)((c4 < 32 ? lo_pair : hi_pair) >> (c4 & 31))};
    return __builtin_bit_cast(uint64_t, halves);
}
// v where the lane's bit of `mask` is set, else 0.  The builtin turns a wave-uniform 64-bit
// mask into a per-lane condition, i.e. one v_cndmask with the mask in scalar registers
// (left to the compiler rather than inline assembly so that its hazard handling --
// e.g. the wait state after a transcendental -- still applies).
__device__ __forceinline__ float keep_select(float v, uint64_t mask) {
    return __builtin_amdgcn_inverse_ballot_w64(mask) ? v : 0.f;
}
// Attention-mask words -> lane mask of accumulator register i of a 32x32 sub-tile: the
// register holds column c = (i/4)*8 + i%4 for lanes 0..31 and column c + 4 for lanes 32..63,
// and word w[c] carries the mask bits of the 32 lanes' rows for column c.
__device__ __forceinline__ uint64_t mask_lanes(const uint32_t (&w)[32], int i) {
    const int c = (i >> 2) * 8 + (i & 3);
    return (uint64_t)w[c] | ((uint64_t)w[c + 4] << 32);
}
__device__ __forceinline__ float mask_select(float v, float other, uint64_t mask) {
    return __builtin_amdgcn_inverse_ballot_w64(mask) ? v : other;
}
// p[i] = keep ? p[i] : 0 for the 16 registers of sub-tile J
template <int J, int I = 0>
__device__ __forceinline__ void keep_apply(float (&p)[16], const KeepWords& w) {
    if constexpr (I < 16) {
        p[I] = keep_select(p[I], keep_lane_mask<J * 32 + (I >> 2) * 8 + (I & 3)>(w));
        keep_apply<J, I + 1>(p, w);
    }
}

// Store the transposed accumulators acc[t][i] (row = the lane's position `pos`, column
// d = t*32 + 8*(i/4) + 4*lg + i%4) scaled by `f` as rows of a [.., 64] tensor.
template <typename T>
__device__ __forceinline__ void store_rows(T* __restrict__ row, const f32x16 (&acc)[2], float f, int lg) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            float v[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) v[b] = acc[t][4 * a + b] * f;
            store_vec<T, 4>(row + t * 32 + a * 8 + lg * 4, v);
        }
}

// ---- keep-bit line per batch-head ---------------------------------------------------
__global__ __launch_bounds__(256) void attn_keepbits_kernel(uint32_t* __restrict__ bits, int bitwords, uint64_t seed) {
    const int bh = blockIdx.y;
    const int o = blockIdx.x * 256 + threadIdx.x;
    const uint64_t s = seed + (uint64_t)bh;
    const bool keep = philox_keep((uint32_t)o, (uint32_t)s, (uint32_t)(s >> 32));
    const uint64_t m = __ballot(keep);
    if ((threadIdx.x & 63) == 0) {
        const int w = o >> 5;
        uint32_t* dst = bits + (int64_t)bh * bitwords;
        if (w < bitwords) dst[w] = (uint32_t)m;
        if (w + 1 < bitwords) dst[w + 1] = (uint32_t)(m >> 32);
    }
}

// ---- attention mask, bit-packed in both orientations ----------------------------------
// out word (o, b, g, x), o = 0: bits r = mask[b, 32g + r, x] (a word per key x: 32 queries);
//                        o = 1: bits r = mask[b, x, 32g + r] (a word per query x: 32 keys).
__global__ __launch_bounds__(256) void attn_pack_mask_kernel(const uint8_t* __restrict__ mask,
                                                              uint32_t* __restrict__ out, int B, int T) {
    const int64_t per = (int64_t)B * (T >> 5) * T;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < 2 * per; i += (int64_t)gridDim.x * 256) {
        const int o = i >= per;
        const int64_t r = i - (o ? per : 0);
        const int x = (int)(r % T);
        const int g = (int)((r / T) % (T >> 5));
        const int64_t b = r / ((int64_t)T * (T >> 5));
        const uint8_t* m = mask + b * (int64_t)T * T;
        uint32_t w = 0;
        if (o == 0) {
            for (int k = 0; k < 32; ++k) w |= (m[(int64_t)(32 * g + k) * T + x] != 0 ? 1u : 0u) << k;
        } else {
            for (int k = 0; k < 32; ++k) w |= (m[(int64_t)x * T + 32 * g + k] != 0 ? 1u : 0u) << k;
        }
        out[i] = w;
    }
}

// Class of every 32x32 tile of (mask AND causal), from the packed words of orientation 0:
//   TILE_CAUSAL  the tile equals the causal pattern (also every tile above the diagonal, where
//                both are empty): index masking alone is exact
//   TILE_HIDDEN  no element visible
//   TILE_MIXED   anything else: the mask words are needed
// written twice: cq[(b, q/32, k/32)] and ck[(b, k/32, q/32)].
enum { TILE_HIDDEN = 0, TILE_MIXED = 1, TILE_CAUSAL = 2 };
__global__ __launch_bounds__(256) void attn_mask_classes_kernel(const uint32_t* __restrict__ packed,
                                                                 uint32_t* __restrict__ cq, uint32_t* __restrict__ ck,
                                                                 int B, int T) {
    const int G = T >> 5;
    const int64_t total = (int64_t)B * G * G;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int kg = (int)(i % G), qg = (int)((i / G) % G);
        const int64_t b = i / ((int64_t)G * G);
        const uint32_t* w = packed + (b * G + qg) * (int64_t)T + 32 * kg;
        bool any = false, same = true;
        for (int c = 0; c < 32; ++c) {
            const int d = 32 * kg + c - 32 * qg;   // query bit r is causally visible iff r >= d
            const uint32_t cw = d <= 0 ? 0xffffffffu : (d >= 32 ? 0u : (0xffffffffu << d));
            const uint32_t eff = w[c] & cw;
            any |= eff != 0;
            same &= eff == cw;
        }
        const uint32_t cls = same ? TILE_CAUSAL : (any ? TILE_MIXED : TILE_HIDDEN);
        cq[i] = cls;
        ck[(b * G + kg) * (int64_t)G + qg] = cls;
    }
}
// classes of the two 32-wide halves of tile step `t` in the class row at `row` (wave-uniform)
struct TileClasses { uint32_t c0, c1; };
__device__ __forceinline__ TileClasses load_classes(const uint32_t* __restrict__ row, int t) {
    TileClasses c;
    c.c0 = row[2 * t];
    c.c1 = row[2 * t + 1];
    return c;
}

// ---- element-wise pieces (VALU budget: a wave64 VALU op costs 4 cycles, v_exp 16, and one
//      K tile gives each lane 32 score elements against 16 MFMAs = 512 cycles; every
//      instruction per element counts, so masks and dropout are compiled in only where used)
constexpr float NEG_RAW = -8e9f;          // masked raw score: NEG_RAW * (1/sqrt(64)) = -1e9
constexpr float RESCALE_SLACK = 8.0f;     // forward: the reference point of the exponentials may lag the row maximum by 2^8
constexpr float M_START = -1e8f;          // log2-domain start of the running maximum: above every masked score
                                          // (-1.44e9), below every real one, so exp2(masked - m) is exactly 0

// Causal visibility of the lane's 16 elements of a sub-tile written into the raw scores
// (invisible -> NEG_RAW).
//   pos0 = (lane's own index) - (first index of the sub-tile along registers) - 4*lg
//   element i = 4a+b sits at register offset 8a+b: visible iff 8a+b <= pos0 (causal part).
template <bool LANE_IS_QUERY>
__device__ __forceinline__ void apply_causal(f32x16& s, int pos0) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int off = (i >> 2) * 8 + (i & 3);
        // lane = query: key offset must be <= query;  lane = key: query offset must be >= key
        const bool ok = LANE_IS_QUERY ? (off <= pos0) : (off >= pos0);
        s[i] = ok ? s[i] : NEG_RAW;
    }
}


// ---- forward -------------------------------------------------------------------------
// grid (B*H, ceil(T/128)); wave w owns queries q0 + 32w .. +31; K/V tiles of 64 keys.
template <typename T, bool HAS_MASK, bool TRAIN>
// (2-byte storage: three workgroups per CU = three wavefronts per SIMD, 168 registers each)
__global__ __launch_bounds__(ATT_THREADS, sizeof(T) == 2 ? 3 : 1) void attn_fwd_kernel(const AttnArgs a) {
    typedef AT<T> X;
    constexpr int STAGE = 2 * X::NP * PANEL;  // K panels then V^T panels
    __shared__ __attribute__((aligned(16))) char smem[2 * STAGE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lg = lane >> 5;
    // grid (B*H, T/128): the batch-head index is the fast dispatch dimension and the query
    // tiles go from the longest (last) to the shortest, so the workgroups that start last
    // are the cheapest ones (causal work per tile grows with the query position).
    const int bh = blockIdx.x, bidx = bh / a.H, hidx = bh % a.H;
    const int q0 = (gridDim.y - 1 - blockIdx.y) * 128;
    const int qw0 = q0 + wave * 32;
    const int query = qw0 + lr;
    const int qrow = query < a.T ? query : a.T - 1;

    const T* Qb = (const T*)a.q + bidx * a.q_bs + hidx * a.q_hs;
    const T* Kb = (const T*)a.k + bidx * a.k_bs + hidx * a.k_hs;
    const T* Vb = (const T*)a.v + bidx * a.v_bs + hidx * a.v_hs;

    typename X::F qf[X::NC];
    load_row_frags<T>(qf, Qb + (int64_t)qrow * a.q_rs, lg);

    int nkt = (q0 + 128) / 64;
    if (nkt > a.T / 64) nkt = a.T / 64;

    // Flat code (no closures) keeps the prefetch registers plain SSA values; the last step
    // re-fetches its own tile instead of branching.
    TileLoader<T, KMAJOR, 64, ATT_THREADS> lk[X::NP];
    TileLoader<T, MNMAJOR, 64, ATT_THREADS, false, true> lv[X::NP];
#define FWD_FETCH(KT)                                                                  \
    _Pragma("unroll") for (int p = 0; p < X::NP; ++p) {                                \
        lk[p].load_fast(Kb, a.k_rs, 1, (KT) * 64, p * X::EPP, tid);                    \
        lv[p].load_fast(Vb, 1, a.v_rs, 0, (KT) * 64 + p * X::EPP, tid);                \
    }
#define FWD_STASH(ST)                                                                  \
    _Pragma("unroll") for (int p = 0; p < X::NP; ++p) {                                \
        lk[p].store(smem + (ST) * STAGE + p * PANEL, tid);                             \
        lv[p].store(smem + (ST) * STAGE + (X::NP + p) * PANEL, tid);                   \
    }

    FWD_FETCH(0)
    // keep-bit line of this batch-head and the wave's first query as scalars
    const uint32_t* __restrict__ kline = a.keepbits + (int64_t)bh * a.bitwords;
    const int qw0u = q0 + __builtin_amdgcn_readfirstlane(wave) * 32;
    FWD_STASH(0)
    __syncthreads();

    const float sc = a.scale * LOG2E;
    float m_run = M_START, m_true = M_START, l_run = 0.f;
    f32x16 o[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[t][e] = 0.f;

    KeepWords kw_next;
    if constexpr (TRAIN) kw_next = load_keep_words(kline, qw0u);
    // tile classes of the wave's 32 queries against every 32-key group (explicit mask only)
    const uint32_t* __restrict__ crow = nullptr;
    TileClasses tc_next = {TILE_CAUSAL, TILE_CAUSAL};
    if constexpr (HAS_MASK) {
        const int G = a.T >> 5;
        crow = a.mask + 2 * (int64_t)a.B * G * a.T + ((int64_t)bidx * G + (qw0u >> 5)) * G;
        tc_next = load_classes(crow, 0);
    }
    for (int kt = 0; kt < nkt; ++kt) {
        const int st = kt & 1;
        FWD_FETCH(kt + 1 < nkt ? kt + 1 : kt)
        // keep bits and classes of this tile were requested one step ago; request the next tile's now
        const KeepWords kw = kw_next;
        if constexpr (TRAIN) kw_next = load_keep_words(kline, qw0u + (kt + 1) * 64);
        const TileClasses tc = tc_next;
        if constexpr (HAS_MASK) tc_next = load_classes(crow, kt + 1 < nkt ? kt + 1 : kt);
        __builtin_amdgcn_sched_barrier(0);
        const int key0 = kt * 64;
        // some key of this tile is visible to some query of the wave
        if (key0 <= qw0 + 31 && (!HAS_MASK || (tc.c0 | tc.c1) != TILE_HIDDEN)) {
            const char* kp = smem + st * STAGE;
            const char* vp = kp + X::NP * PANEL;
            f32x16 s[2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) s[j][e] = 0.f;
            rows_x_frags<T>(s, kp, qf, lr, lg);

            if (key0 + 63 > qw0) {   // tile touches the diagonal for this wave
#pragma unroll
                for (int j = 0; j < 2; ++j) apply_causal<true>(s[j], query - key0 - j * 32 - lg * 4);
            }
            if constexpr (HAS_MASK) {
                // one word per key: the mask bits of the wave's 32 queries (wave-uniform loads), read
                // only for a half whose tile is not already described by the causal pattern
                const uint32_t* mw = a.mask + ((int64_t)bidx * (a.T >> 5) + (qw0u >> 5)) * a.T + key0;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if ((j == 0 ? tc.c0 : tc.c1) == TILE_CAUSAL) continue;
                    uint32_t w[32];
#pragma unroll
                    for (int t = 0; t < 32; ++t) w[t] = mw[j * 32 + t];
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[j][i] = mask_select(s[j][i], NEG_RAW, mask_lanes(w, i));
                }
            }
            float tmax = s[0][0];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, s[j][i]);
            tmax = max_xor32(tmax) * sc;
            m_true = fmaxf(m_true, tmax);
            // The exponentials are taken relative to m_run, which follows the true row maximum
            // only when some row of the wavefront has outgrown it by more than 2^RESCALE_SLACK:
            // softmax does not depend on the reference point, p stays below 2^RESCALE_SLACK, and
            // the 32 rescaling multiplies of the accumulators are skipped on most tiles.  The
            // saved statistics are converted to the true maximum at the end.
            if (__builtin_amdgcn_ballot_w64(tmax > m_run + RESCALE_SLACK) != 0) {
                const float m_new = fmaxf(m_run, tmax);
                const float alpha = fast_exp2(m_run - m_new);
                l_run *= alpha;
                m_run = m_new;
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[t][e] *= alpha;
            }
            float p[2][16];
            float lsum = 0.f;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float e = fast_exp2(fmaf(s[j][i], sc, -m_run));
                    p[j][i] = e;
                    lsum += e;
                }
            l_run += sum_xor32(lsum);
            if constexpr (TRAIN) {
                keep_apply<0>(p[0], kw);
                keep_apply<1>(p[1], kw);
            }
            tp_x_regs(o, vp, p, lr, lg, T());
        }
        __builtin_amdgcn_sched_barrier(0);
        FWD_STASH(st ^ 1)
        __syncthreads();
    }
#undef FWD_FETCH
#undef FWD_STASH

    if (query < a.T) {
        // l_run = 0: no key of the row is visible (a row with a visible key has l_run >= 1)
        const bool empty = l_run == 0.f;
        const float f = empty ? 0.f : (TRAIN ? 1.0f : 0.9f) / l_run;
        store_rows<T>((T*)a.out0 + bidx * a.out0_bs + hidx * a.out0_hs + (int64_t)query * a.out0_rs, o, f, lg);
        if (lg == 0) {
            // statistics relative to the true row maximum: sum exp(s - m_true) = l_run 2^(m_run - m_true)
            a.ms[(int64_t)bh * a.T + query] = empty ? NEG_NAT : m_true * LN2;
            a.ls[(int64_t)bh * a.T + query] = empty ? 0.f : l_run * fast_exp2(m_run - m_true);
        }
    }
}

// ---- backward pass 1: dK, dV ------------------------------------------------------------
// grid (B*H, ceil(T/128)); wave w owns keys key0 + 32w .. +31 (lane = key); query tiles of 64.
template <typename T, bool HAS_MASK, bool TRAIN>
__global__ __launch_bounds__(ATT_THREADS, sizeof(T) == 2 ? 2 : 1) void attn_bwd_dkdv_kernel(const AttnArgs a) {
    typedef AT<T> X;
    constexpr int STAGE = 4 * X::NP * PANEL;  // Q, dO, Q^T, dO^T
    __shared__ __attribute__((aligned(16))) char smem[2 * STAGE];
    __shared__ __attribute__((aligned(16))) float sstat[2][3][64];  // m2, 1/l, delta per stage

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lg = lane >> 5;
    const int bh = blockIdx.x, bidx = bh / a.H, hidx = bh % a.H;
    const int key0 = blockIdx.y * 128;                    // first key tiles see the most queries: heavy first
    const int kw0 = key0 + wave * 32;
    const int key = kw0 + lr;
    const int krow = key < a.T ? key : a.T - 1;

    const T* Qb = (const T*)a.q + bidx * a.q_bs + hidx * a.q_hs;
    const T* Kb = (const T*)a.k + bidx * a.k_bs + hidx * a.k_hs;
    const T* Vb = (const T*)a.v + bidx * a.v_bs + hidx * a.v_hs;
    const T* dOb = (const T*)a.d_o + bidx * a.do_bs + hidx * a.do_hs;

    typename X::F kf[X::NC], vf[X::NC];
    load_row_frags<T>(kf, Kb + (int64_t)krow * a.k_rs, lg);
    load_row_frags<T>(vf, Vb + (int64_t)krow * a.v_rs, lg);

    const int qt0 = key0 / 64, nqt = a.T / 64;

    TileLoader<T, KMAJOR, 64, ATT_THREADS> lq[X::NP], ld[X::NP];
    TileLoader<T, MNMAJOR, 64, ATT_THREADS, false, true> lqt[X::NP], ldt[X::NP];
    float st_m = 0.f, st_l = 1.f, st_d = 0.f;
    // 2-byte storage: 1/l goes into the exponent (p = 2^(s - m - log2 l)), one multiplication less
    // per element.  A row without a visible key (saved l = 0) gets m = 0 and 1/l = 0 instead: all
    // of its scores are masked (-1.44e9 in the exponent), so its p is exactly 0.
    constexpr bool FOLD_L = sizeof(T) == 2;
    const int64_t stat0 = (int64_t)bh * a.T + (tid & 63);
#define KV_FETCH(QT)                                                                   \
    {                                                                                  \
        const int q0__ = (QT) * 64;                                                    \
        _Pragma("unroll") for (int p = 0; p < X::NP; ++p) {                            \
            lq[p].load_fast(Qb, a.q_rs, 1, q0__, p * X::EPP, tid);                     \
            ld[p].load_fast(dOb, a.do_rs, 1, q0__, p * X::EPP, tid);                   \
            lqt[p].load_fast(Qb, 1, a.q_rs, 0, q0__ + p * X::EPP, tid);                \
            ldt[p].load_fast(dOb, 1, a.do_rs, 0, q0__ + p * X::EPP, tid);              \
        }                                                                              \
        st_m = a.ms[stat0 + q0__];                                                     \
        st_l = a.ls[stat0 + q0__];                                                     \
        st_d = a.delta[stat0 + q0__];                                                  \
    }
#define KV_STASH(ST)                                                                   \
    {                                                                                  \
        char* base__ = smem + (ST) * STAGE;                                            \
        _Pragma("unroll") for (int p = 0; p < X::NP; ++p) {                            \
            lq[p].store(base__ + p * PANEL, tid);                                      \
            ld[p].store(base__ + (X::NP + p) * PANEL, tid);                            \
            lqt[p].store(base__ + (2 * X::NP + p) * PANEL, tid);                       \
            ldt[p].store(base__ + (3 * X::NP + p) * PANEL, tid);                       \
        }                                                                              \
        if (tid < 64) {                                                                \
            const bool none__ = st_l == 0.f;                                           \
            const float m2__ = FOLD_L ? fmaf(st_m, LOG2E, __builtin_amdgcn_logf(st_l)) : st_m * LOG2E; \
            sstat[ST][0][tid] = none__ ? 0.f : m2__;                                   \
            sstat[ST][1][tid] = none__ ? 0.f : 1.0f / st_l;                            \
            sstat[ST][2][tid] = st_d;                                                  \
        }                                                                              \
    }

    f32x16 dk[2], dv[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) dk[t][e] = dv[t][e] = 0.f;

    if (qt0 < nqt) {
        KV_FETCH(qt0)
        KV_STASH(0)
    }
    __syncthreads();

    const float sc = a.scale * LOG2E;
    // keep-bit line of this batch-head and the wave's first key as scalars
    const uint32_t* __restrict__ kline = a.keepbits + (int64_t)bh * a.bitwords;
    const int kw0u = key0 + __builtin_amdgcn_readfirstlane(wave) * 32;
    KeepWords kw_next;
    if constexpr (TRAIN) kw_next = load_keep_words(kline, kw0u + qt0 * 64);
    // tile classes of the wave's 32 keys against every 32-query group (explicit mask only)
    const uint32_t* __restrict__ crow = nullptr;
    TileClasses tc_next = {TILE_CAUSAL, TILE_CAUSAL};
    if constexpr (HAS_MASK) {
        const int G = a.T >> 5;
        crow = a.mask + 2 * (int64_t)a.B * G * a.T + (int64_t)a.B * G * G + ((int64_t)bidx * G + (kw0u >> 5)) * G;
        if (qt0 < nqt) tc_next = load_classes(crow, qt0);
    }
    for (int qt = qt0; qt < nqt; ++qt) {
        const int st = (qt - qt0) & 1;
        KV_FETCH(qt + 1 < nqt ? qt + 1 : qt)
        const KeepWords kw = kw_next;   // requested one step ago
        if constexpr (TRAIN) kw_next = load_keep_words(kline, kw0u + (qt + 1) * 64);
        const TileClasses tc = tc_next;
        if constexpr (HAS_MASK) tc_next = load_classes(crow, qt + 1 < nqt ? qt + 1 : qt);
        __builtin_amdgcn_sched_barrier(0);
        const int q0 = qt * 64;
        if (q0 + 63 >= kw0) {   // some query of the tile sees some key of the wave
            const char* base = smem + st * STAGE;
            // The two 32-query halves are processed one after the other: half the live
            // accumulators, which keeps two wavefronts per SIMD resident.
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (q0 + j * 32 + 31 < kw0) continue;   // every query of this half precedes the wave's keys
                const uint32_t cls = j == 0 ? tc.c0 : tc.c1;
                if (HAS_MASK && cls == TILE_HIDDEN) continue;
                f32x16 s, dp;
#pragma unroll
                for (int e = 0; e < 16; ++e) s[e] = dp[e] = 0.f;
                rows_x_frags_one<T>(s, base, kf, j, lr, lg);                      // S  [query][key]
                rows_x_frags_one<T>(dp, base + X::NP * PANEL, vf, j, lr, lg);     // dP [query][key]

                const bool diag = q0 + j * 32 < kw0 + 31;
                if (diag) apply_causal<false>(s, key - q0 - j * 32 - lg * 4);
                if (HAS_MASK && cls != TILE_CAUSAL) {
                    // one word per query: the mask bits of the wave's 32 keys (wave-uniform loads)
                    const uint32_t* mw = a.mask + (int64_t)a.B * (a.T >> 5) * a.T +
                                         ((int64_t)bidx * (a.T >> 5) + (kw0u >> 5)) * a.T + q0 + j * 32;
                    uint32_t mwords[32];
#pragma unroll
                    for (int t = 0; t < 32; ++t) mwords[t] = mw[t];
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[i] = mask_select(s[i], NEG_RAW, mask_lanes(mwords, i));
                }
                float pd[16], ds[16];
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const int qi = j * 32 + g4 * 8 + lg * 4;  // first of 4 consecutive queries (tile-relative)
                    const f32x4 m4 = *reinterpret_cast<const f32x4*>(&sstat[st][0][qi]);
                    f32x4 l4 = {1.f, 1.f, 1.f, 1.f};
                    if constexpr (!FOLD_L) l4 = *reinterpret_cast<const f32x4*>(&sstat[st][1][qi]);
                    const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sstat[st][2][qi]);
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        const int i = g4 * 4 + b;
                        float p = fast_exp2(fmaf(s[i], sc, -m4[b]));
                        if constexpr (!FOLD_L) p *= l4[b];
                        if constexpr (TRAIN) {
                            // dS = P (keep ? dP : 0) - P delta = (keep ? P : 0) dP - P delta: the dropped
                            // probability is needed anyway, so one select serves both products
                            const uint64_t km = keep_lane_mask_at(kw, j * 32 + g4 * 8 + b);
                            pd[i] = keep_select(p, km);
                            ds[i] = fmaf(pd[i], dp[i], -(p * d4[b]));
                        } else {
                            pd[i] = 0.9f * p;
                            ds[i] = p * fmaf(dp[i], 0.9f, -d4[b]);
                        }
                    }
                }
                // Hidden elements (causal or masked) need no separate dS masking: their score is the
                // fill value and the row's reference point is a real maximum (or 0 for a row without
                // visible keys), so p, hence dS, is exactly 0 there.
                tp_x_regs_one(dv, base + 3 * X::NP * PANEL, pd, j, lr, lg, T());  // dV^T += dO^T P
                tp_x_regs_one(dk, base + 2 * X::NP * PANEL, ds, j, lr, lg, T());  // dK^T += Q^T dS
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        KV_STASH(st ^ 1)
        __syncthreads();
    }
#undef KV_FETCH
#undef KV_STASH

    if (key < a.T) {
        store_rows<T>((T*)a.out0 + bidx * a.out0_bs + hidx * a.out0_hs + (int64_t)key * a.out0_rs, dk, a.scale, lg);
        store_rows<T>((T*)a.out1 + bidx * a.out1_bs + hidx * a.out1_hs + (int64_t)key * a.out1_rs, dv, 1.0f, lg);
    }
}

// ---- backward pass 2: dQ ----------------------------------------------------------------
// Same geometry as the forward (lane = query, key tiles of 64).
template <typename T, bool HAS_MASK, bool TRAIN>
// (2-byte storage without an explicit mask fits three wavefronts per SIMD; the bound keeps it there)
__global__ __launch_bounds__(ATT_THREADS, sizeof(T) == 2 ? 3 : 1) void attn_bwd_dq_kernel(const AttnArgs a) {
    typedef AT<T> X;
    constexpr int STAGE = 3 * X::NP * PANEL;  // K, V, K^T
    __shared__ __attribute__((aligned(16))) char smem[2 * STAGE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lg = lane >> 5;
    const int bh = blockIdx.x, bidx = bh / a.H, hidx = bh % a.H;
    const int q0 = (gridDim.y - 1 - blockIdx.y) * 128;    // longest query tiles first
    const int qw0 = q0 + wave * 32;
    const int query = qw0 + lr;
    const int qrow = query < a.T ? query : a.T - 1;

    const T* Qb = (const T*)a.q + bidx * a.q_bs + hidx * a.q_hs;
    const T* Kb = (const T*)a.k + bidx * a.k_bs + hidx * a.k_hs;
    const T* Vb = (const T*)a.v + bidx * a.v_bs + hidx * a.v_hs;
    const T* dOb = (const T*)a.d_o + bidx * a.do_bs + hidx * a.do_hs;

    typename X::F qf[X::NC], dof[X::NC];
    load_row_frags<T>(qf, Qb + (int64_t)qrow * a.q_rs, lg);
    load_row_frags<T>(dof, dOb + (int64_t)qrow * a.do_rs, lg);
    const int64_t si = (int64_t)bh * a.T + qrow;
    // as in the dK/dV pass: 1/l folded into the exponent for 2-byte storage; a row without a
    // visible key (saved l = 0) takes m = 0 and 1/l = 0, which makes its p exactly 0
    constexpr bool FOLD_L = sizeof(T) == 2;
    const float lsum = a.ls[si];
    const bool none = lsum == 0.f;
    const float linv = none ? 0.f : 1.0f / lsum;
    // delta = rowsum(dO * O) of the lane's query: each lane of the pair (lr, lg) holds one half
    // of the dO row already; the dK/dV pass (launched after this one) reads the stored values.
    float delta;
    {
        typename X::F of[X::NC];
        load_row_frags<T>(of, (const T*)a.o + bidx * a.o_bs + hidx * a.o_hs + (int64_t)qrow * a.o_rs, lg);
        constexpr int FE = (int)(sizeof(typename X::F) / sizeof(T));
        float part = 0.f;
#pragma unroll
        for (int c = 0; c < X::NC; ++c)
#pragma unroll
            for (int e = 0; e < FE; ++e) part += (float)dof[c][e] * (float)of[c][e];
        delta = part + xor32(part);
        if (lg == 0 && query < a.T) a.delta[si] = delta;
    }
    const float m2 = none ? 0.f : (FOLD_L ? fmaf(a.ms[si], LOG2E, __builtin_amdgcn_logf(lsum)) : a.ms[si] * LOG2E);

    int nkt = (q0 + 128) / 64;
    if (nkt > a.T / 64) nkt = a.T / 64;

    TileLoader<T, KMAJOR, 64, ATT_THREADS> lk[X::NP], lv[X::NP];
    TileLoader<T, MNMAJOR, 64, ATT_THREADS, false, true> lkt[X::NP];
#define DQ_FETCH(KT)                                                                   \
    _Pragma("unroll") for (int p = 0; p < X::NP; ++p) {                                \
        lk[p].load_fast(Kb, a.k_rs, 1, (KT) * 64, p * X::EPP, tid);                    \
        lv[p].load_fast(Vb, a.v_rs, 1, (KT) * 64, p * X::EPP, tid);                    \
        lkt[p].load_fast(Kb, 1, a.k_rs, 0, (KT) * 64 + p * X::EPP, tid);               \
    }
#define DQ_STASH(ST)                                                                   \
    _Pragma("unroll") for (int p = 0; p < X::NP; ++p) {                                \
        lk[p].store(smem + (ST) * STAGE + p * PANEL, tid);                             \
        lv[p].store(smem + (ST) * STAGE + (X::NP + p) * PANEL, tid);                   \
        lkt[p].store(smem + (ST) * STAGE + (2 * X::NP + p) * PANEL, tid);              \
    }

    DQ_FETCH(0)
    DQ_STASH(0)
    __syncthreads();

    const float sc = a.scale * LOG2E;
    f32x16 dq[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) dq[t][e] = 0.f;

    const uint32_t* __restrict__ kline = a.keepbits + (int64_t)bh * a.bitwords;
    const int qw0u = q0 + __builtin_amdgcn_readfirstlane(wave) * 32;
    KeepWords kw_next;
    if constexpr (TRAIN) kw_next = load_keep_words(kline, qw0u);
    const uint32_t* __restrict__ crow = nullptr;
    TileClasses tc_next = {TILE_CAUSAL, TILE_CAUSAL};
    if constexpr (HAS_MASK) {
        const int G = a.T >> 5;
        crow = a.mask + 2 * (int64_t)a.B * G * a.T + ((int64_t)bidx * G + (qw0u >> 5)) * G;
        tc_next = load_classes(crow, 0);
    }
    for (int kt = 0; kt < nkt; ++kt) {
        const int st = kt & 1;
        DQ_FETCH(kt + 1 < nkt ? kt + 1 : kt)
        const KeepWords kw = kw_next;   // requested one step ago
        if constexpr (TRAIN) kw_next = load_keep_words(kline, qw0u + (kt + 1) * 64);
        const TileClasses tc = tc_next;
        if constexpr (HAS_MASK) tc_next = load_classes(crow, kt + 1 < nkt ? kt + 1 : kt);
        __builtin_amdgcn_sched_barrier(0);
        const int key0 = kt * 64;
        if (key0 <= qw0 + 31) {
            const char* base = smem + st * STAGE;
            // The two 32-key halves one after the other: half the live accumulators, and a half
            // whose keys all follow the wave's queries is skipped.
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int kh0 = key0 + j * 32;
                if (kh0 > qw0 + 31) continue;
                const uint32_t cls = j == 0 ? tc.c0 : tc.c1;
                if (HAS_MASK && cls == TILE_HIDDEN) continue;
                f32x16 s, dp;
#pragma unroll
                for (int e = 0; e < 16; ++e) s[e] = dp[e] = 0.f;
                rows_x_frags_one<T>(s, base, qf, j, lr, lg);                       // S^T  [key][query]
                rows_x_frags_one<T>(dp, base + X::NP * PANEL, dof, j, lr, lg);     // dP^T [key][query]

                const bool masked = kh0 + 31 > qw0;
                if (masked) apply_causal<true>(s, query - kh0 - lg * 4);
                if (HAS_MASK && cls != TILE_CAUSAL) {
                    // one word per key: the mask bits of the wave's 32 queries (wave-uniform loads)
                    const uint32_t* mw = a.mask + ((int64_t)bidx * (a.T >> 5) + (qw0u >> 5)) * a.T + kh0;
                    uint32_t mwords[32];
#pragma unroll
                    for (int t = 0; t < 32; ++t) mwords[t] = mw[t];
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[i] = mask_select(s[i], NEG_RAW, mask_lanes(mwords, i));
                }
                float ds[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    float p = fast_exp2(fmaf(s[i], sc, -m2));
                    if constexpr (!FOLD_L) p *= linv;
                    if constexpr (TRAIN)
                        ds[i] = p * (keep_select(dp[i], keep_lane_mask_at(kw, j * 32 + (i >> 2) * 8 + (i & 3))) - delta);
                    else
                        ds[i] = p * fmaf(dp[i], 0.9f, -delta);
                }
                // as in the dK/dV pass: p, hence dS, is exactly 0 on hidden elements
                tp_x_regs_one(dq, base + 2 * X::NP * PANEL, ds, j, lr, lg, T());   // dQ^T += K^T dS^T
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        DQ_STASH(st ^ 1)
        __syncthreads();
    }
#undef DQ_FETCH
#undef DQ_STASH

    if (query < a.T)
        store_rows<T>((T*)a.out0 + bidx * a.out0_bs + hidx * a.out0_hs + (int64_t)query * a.out0_rs, dq, a.scale, lg);
}

// Launch one of the (mask, train) specialisations.
#define ATTN_LAUNCH(KERNEL, T_, grid, st, args)                                                        \
    do {                                                                                               \
        const bool hm__ = (args).mask != nullptr, tr__ = (args).train != 0;                            \
        if (hm__ && tr__) hipLaunchKernelGGL((KERNEL<T_, true, true>), grid, dim3(ATT_THREADS), 0, st, args);        \
        else if (hm__) hipLaunchKernelGGL((KERNEL<T_, true, false>), grid, dim3(ATT_THREADS), 0, st, args);          \
        else if (tr__) hipLaunchKernelGGL((KERNEL<T_, false, true>), grid, dim3(ATT_THREADS), 0, st, args);          \
        else hipLaunchKernelGGL((KERNEL<T_, false, false>), grid, dim3(ATT_THREADS), 0, st, args);                   \
    } while (0)

// ---- host side ----------------------------------------------------------------------------
inline size_t bits_bytes(int64_t BH, int64_t T) { return (size_t)BH * (2 * T / 32 + 2) * sizeof(uint32_t); }
inline size_t delta_bytes(int64_t BH, int64_t T) { return (size_t)BH * T * sizeof(float); }

int check_common(const char* what, int64_t B, int64_t H, int64_t T, int64_t dh, int dtype,
                 std::initializer_list<const void*> ptrs, std::initializer_list<int64_t> strides) {
    if (B < 1 || H < 1) return ptj_set_error(PTJ_ERR_INVALID, "%s: B and H must be positive", what);
    if (dh != DH) return ptj_set_error(PTJ_ERR_INVALID, "%s: head dimension %lld unsupported (64 only)", what, (long long)dh);
    if (T < 64 || T % 64 != 0 || T > MAX_T)
        return ptj_set_error(PTJ_ERR_INVALID, "%s: T=%lld must be a multiple of 64 in [64, %d]", what, (long long)T, MAX_T);
    if (dtype != PTJ_F32 && dtype != PTJ_BF16) return ptj_set_error(PTJ_ERR_INVALID, "%s: unknown dtype %d", what, dtype);
    const int vec = dtype == PTJ_BF16 ? 8 : 4;
    for (const void* p : ptrs)
        if (!p || !ptj_aligned16(p)) return ptj_set_error(PTJ_ERR_INVALID, "%s: null or not 16-byte aligned pointer", what);
    for (int64_t s : strides)
        if (s % vec != 0 || s < 0) return ptj_set_error(PTJ_ERR_INVALID, "%s: strides must be multiples of 16 bytes", what);
    return PTJ_OK;
}

int launch_keepbits(uint32_t* bits, int64_t BH, int bitwords, int64_t seed, hipStream_t st) {
    hipLaunchKernelGGL(attn_keepbits_kernel, dim3((bitwords * 32 + 255) / 256, (unsigned)BH), dim3(256), 0, st, bits,
                       bitwords, (uint64_t)seed);
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

}  // namespace

extern "C" {

size_t ptj_attn_workspace_bytes(int64_t B, int64_t H, int64_t T) {
    if (B < 1 || H < 1 || T < 1) return 0;
    return bits_bytes(B * H, T) + delta_bytes(B * H, T);
}

size_t ptj_attn_packed_mask_bytes(int64_t B, int64_t T) {
    if (B < 1 || T < 32 || T % 32) return 0;
    // the mask words in both orientations, then the tile classes in both index orders
    return ((size_t)2 * B * (T / 32) * T + (size_t)2 * B * (T / 32) * (T / 32)) * sizeof(uint32_t);
}

int ptj_attn_pack_mask(const uint8_t* mask, uint32_t* packed, int64_t B, int64_t T, void* stream) {
    PTJ_CHECK_ARG(mask && packed, "attn_pack_mask: null pointer");
    PTJ_CHECK_ARG(B >= 1 && T >= 32 && T % 32 == 0 && T < (1 << 24), "attn_pack_mask: need B >= 1 and T a multiple of 32");
    const int64_t words = 2 * B * (T / 32) * T;
    int64_t blocks = (words + 255) / 256;
    if (blocks > (int64_t)ptj_num_cus() * 16) blocks = (int64_t)ptj_num_cus() * 16;
    hipLaunchKernelGGL(attn_pack_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, mask, packed, (int)B,
                       (int)T);
    PTJ_CHECK_LAUNCH();
    const int64_t tiles = B * (T / 32) * (T / 32);
    uint32_t* cq = packed + words;
    hipLaunchKernelGGL(attn_mask_classes_kernel, dim3((unsigned)((tiles + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint32_t*)packed, cq, cq + tiles, (int)B, (int)T);
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

int ptj_attn_fwd(const void* q, const void* k, const void* v, const uint32_t* mask, void* o, float* ms, float* ls,
                 void* workspace, size_t workspace_bytes, int64_t B, int64_t H, int64_t T, int64_t dh,
                 int64_t q_bs, int64_t q_hs, int64_t q_rs, int64_t k_bs, int64_t k_hs, int64_t k_rs,
                 int64_t v_bs, int64_t v_hs, int64_t v_rs, int64_t o_bs, int64_t o_hs, int64_t o_rs,
                 int train, int64_t seed, int dtype, void* stream) {
    int rc = check_common("attn_fwd", B, H, T, dh, dtype, {q, k, v, o},
                          {q_bs, q_hs, q_rs, k_bs, k_hs, k_rs, v_bs, v_hs, v_rs, o_bs, o_hs, o_rs});
    if (rc) return rc;
    PTJ_CHECK_ARG(ms && ls, "attn_fwd: null statistics pointer");
    PTJ_CHECK_ARG(!mask || (reinterpret_cast<uintptr_t>(mask) & 3) == 0, "attn_fwd: mask must be 4-byte aligned");
    const int64_t BH = B * H;
    hipStream_t st = (hipStream_t)stream;
    AttnArgs a = {};
    a.q = q; a.k = k; a.v = v; a.out0 = o; a.mask = mask; a.ms = ms; a.ls = ls;
    a.B = (int)B; a.H = (int)H; a.T = (int)T; a.bitwords = (int)(2 * T / 32 + 2);
    a.q_bs = q_bs; a.q_hs = q_hs; a.q_rs = q_rs; a.k_bs = k_bs; a.k_hs = k_hs; a.k_rs = k_rs;
    a.v_bs = v_bs; a.v_hs = v_hs; a.v_rs = v_rs;
    a.out0_bs = o_bs; a.out0_hs = o_hs; a.out0_rs = o_rs;
    a.train = train != 0; a.scale = 0.125f;
    if (a.train) {
        if (!workspace || workspace_bytes < bits_bytes(BH, T))
            return ptj_set_error(PTJ_ERR_WORKSPACE, "attn_fwd: workspace %zu < %zu bytes", workspace_bytes, bits_bytes(BH, T));
        a.keepbits = (const uint32_t*)workspace;
        rc = launch_keepbits((uint32_t*)workspace, BH, a.bitwords, seed, st);
        if (rc) return rc;
    }
    dim3 grid((unsigned)BH, (unsigned)((T + 127) / 128));
    if (dtype == PTJ_F32) ATTN_LAUNCH(attn_fwd_kernel, float, grid, st, a);
    else ATTN_LAUNCH(attn_fwd_kernel, bf16, grid, st, a);
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

int ptj_attn_bwd(const void* d_o, const void* q, const void* k, const void* v, const void* o, const float* ms,
                 const float* ls, const uint32_t* mask, void* dq, void* dk, void* dv, void* workspace,
                 size_t workspace_bytes, int64_t B, int64_t H, int64_t T, int64_t dh,
                 int64_t do_bs, int64_t do_hs, int64_t do_rs, int64_t q_bs, int64_t q_hs, int64_t q_rs,
                 int64_t k_bs, int64_t k_hs, int64_t k_rs, int64_t v_bs, int64_t v_hs, int64_t v_rs,
                 int64_t o_bs, int64_t o_hs, int64_t o_rs, int64_t dq_bs, int64_t dq_hs, int64_t dq_rs,
                 int64_t dk_bs, int64_t dk_hs, int64_t dk_rs, int64_t dv_bs, int64_t dv_hs, int64_t dv_rs,
                 int train, int64_t seed, int dtype, void* stream) {
    int rc = check_common("attn_bwd", B, H, T, dh, dtype, {d_o, q, k, v, o, dq, dk, dv},
                          {do_bs, do_hs, do_rs, q_bs, q_hs, q_rs, k_bs, k_hs, k_rs, v_bs, v_hs, v_rs, o_bs, o_hs, o_rs,
                           dq_bs, dq_hs, dq_rs, dk_bs, dk_hs, dk_rs, dv_bs, dv_hs, dv_rs});
    if (rc) return rc;
    PTJ_CHECK_ARG(ms && ls, "attn_bwd: null statistics pointer");
    PTJ_CHECK_ARG(!mask || (reinterpret_cast<uintptr_t>(mask) & 3) == 0, "attn_bwd: mask must be 4-byte aligned");
    const int64_t BH = B * H;
    if (!workspace || workspace_bytes < ptj_attn_workspace_bytes(B, H, T))
        return ptj_set_error(PTJ_ERR_WORKSPACE, "attn_bwd: workspace %zu < %zu bytes", workspace_bytes,
                             ptj_attn_workspace_bytes(B, H, T));
    hipStream_t st = (hipStream_t)stream;
    uint32_t* bits = (uint32_t*)workspace;
    float* delta = (float*)((char*)workspace + bits_bytes(BH, T));
    AttnArgs a = {};
    a.q = q; a.k = k; a.v = v; a.o = o; a.d_o = d_o; a.mask = mask;
    a.ms = const_cast<float*>(ms); a.ls = const_cast<float*>(ls); a.delta = delta; a.keepbits = bits;
    a.B = (int)B; a.H = (int)H; a.T = (int)T; a.bitwords = (int)(2 * T / 32 + 2);
    a.q_bs = q_bs; a.q_hs = q_hs; a.q_rs = q_rs; a.k_bs = k_bs; a.k_hs = k_hs; a.k_rs = k_rs;
    a.v_bs = v_bs; a.v_hs = v_hs; a.v_rs = v_rs; a.o_bs = o_bs; a.o_hs = o_hs; a.o_rs = o_rs;
    a.do_bs = do_bs; a.do_hs = do_hs; a.do_rs = do_rs;
    a.train = train != 0; a.scale = 0.125f;
    if (a.train) {
        rc = launch_keepbits(bits, BH, a.bitwords, seed, st);
        if (rc) return rc;
    }
    dim3 grid((unsigned)BH, (unsigned)((T + 127) / 128));
    AttnArgs a1 = a;
    a1.out0 = dk; a1.out0_bs = dk_bs; a1.out0_hs = dk_hs; a1.out0_rs = dk_rs;
    a1.out1 = dv; a1.out1_bs = dv_bs; a1.out1_hs = dv_hs; a1.out1_rs = dv_rs;
    AttnArgs a2 = a;
    a2.out0 = dq; a2.out0_bs = dq_bs; a2.out0_hs = dq_hs; a2.out0_rs = dq_rs;
    if (dtype == PTJ_F32) {
        ATTN_LAUNCH(attn_bwd_dq_kernel, float, grid, st, a2);      // also writes delta ...
        ATTN_LAUNCH(attn_bwd_dkdv_kernel, float, grid, st, a1);    // ... which this pass reads
    } else {
        ATTN_LAUNCH(attn_bwd_dq_kernel, bf16, grid, st, a2);
        ATTN_LAUNCH(attn_bwd_dkdv_kernel, bf16, grid, st, a1);
    }
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

}  // extern "C"
