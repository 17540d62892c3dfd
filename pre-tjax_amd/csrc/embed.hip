// Token + position embedding, forward and backward, as single passes.
//
// Forward: out[i] = dropout(round(wemb[token_i] * scale) + pos[i mod seq]) -- the gather,
// the scaling, the position add and the embedding dropout of the model's first step, with
// the storage rounding after each of them that separate kernels would apply.
//
// Backward: dwemb[tok] += scale * sum_{i: token_i = tok} d[i].  The caller passes the
// token ids sorted (stable) together with the sorting permutation; a workgroup that sits
// on the first position of a run of equal tokens sums the run's gradient rows in fp32 in
// sorted order (four row slots folded through LDS in slot order) and updates that table
// row in place, so the result is deterministic and no [vocab, dim] scratch is touched.
#include "common.h"

namespace {

constexpr int EMB_COLT = 128;            // column threads (one 16-byte vector each per sweep)
constexpr int EMB_SLOTS = 4;             // row slots of the backward workgroup
constexpr int EMB_BWD_THREADS = EMB_COLT * EMB_SLOTS;

template <typename T, int VEC>
__global__ __launch_bounds__(256) void embed_fwd_kernel(const T* __restrict__ wemb, const T* __restrict__ pos,
                                                         const int64_t* __restrict__ tokens, T* __restrict__ out,
                                                         int64_t n, int dim, int64_t seq, int64_t vocab, float scale,
                                                         int train, uint64_t seed) {
#pragma clang fp contract(off)   // product and sum are rounded separately, as two kernels would
    const int vpr = dim / VEC;
    const int64_t total = n * vpr;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t row = (int64_t)((uint64_t)i / (uint32_t)vpr);
        const int c0 = (int)(i - row * vpr) * VEC;
        int64_t tok = tokens[row];
        tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);   // ids are required to be in range; never read outside the table
        float w[VEC], p[VEC];
        load_vec<T, VEC>(wemb + tok * dim + c0, w);
        load_vec<T, VEC>(pos + (row % seq) * dim + c0, p);
        const uint64_t s = seed + (uint64_t)row;
        const uint32_t k0 = (uint32_t)s, k1 = (uint32_t)(s >> 32);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            float v = to_f32(from_f32<T>(w[j] * scale));
            v = to_f32(from_f32<T>(v + p[j]));
            if (train) v = philox_keep((uint32_t)(c0 + j), k0, k1) ? v : 0.f;
            else v *= 0.9f;
            w[j] = v;
        }
        store_vec<T, VEC>(out + row * dim + c0, w);
    }
}

// Row of `d` behind sorted position j, clamped so that a bad permutation cannot read outside d.
__device__ __forceinline__ int64_t src_row(const int64_t* __restrict__ order, int64_t j, int64_t n) {
    const int64_t r = order[j];
    return r < 0 ? 0 : (r >= n ? n - 1 : r);
}

template <typename T, int VEC>
__global__ __launch_bounds__(EMB_BWD_THREADS) void embed_bwd_kernel(const T* __restrict__ d,
                                                                    const int64_t* __restrict__ sorted_tok,
                                                                    const int64_t* __restrict__ order,
                                                                    T* __restrict__ dwemb, int64_t n, int dim,
                                                                    int64_t vocab, float scale) {
    __shared__ float red[EMB_SLOTS][EMB_COLT * VEC];
    __shared__ int64_t s_end;
    const int64_t first = blockIdx.x;
    const int64_t tok = sorted_tok[first];
    if (first > 0 && sorted_tok[first - 1] == tok) return;      // not the head of a run (uniform)
    if (tok < 0 || tok >= vocab) return;
    if (threadIdx.x == 0) {
        // end of the run: first position after `first` with a different token (binary search)
        int64_t lo = first + 1, hi = n;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (sorted_tok[mid] == tok) lo = mid + 1;
            else hi = mid;
        }
        s_end = lo;
    }
    __syncthreads();
    const int64_t end = s_end;
    const int ct = threadIdx.x % EMB_COLT, slot = threadIdx.x / EMB_COLT;
    const int nvec = dim / VEC;
    for (int v0 = 0; v0 < nvec; v0 += EMB_COLT) {
        const int vi = v0 + ct;
        const bool active = vi < nvec;
        float acc[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
        if (active) {
            constexpr int U = 4;
            int64_t j = first + slot;
            for (; j + (U - 1) * EMB_SLOTS < end; j += U * EMB_SLOTS) {
                float r[U][VEC];
#pragma unroll
                for (int u = 0; u < U; ++u) load_vec<T, VEC>(d + src_row(order, j + u * EMB_SLOTS, n) * dim + vi * VEC, r[u]);
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[e] += r[u][e];
            }
            for (; j < end; j += EMB_SLOTS) {
                float r[VEC];
                load_vec<T, VEC>(d + src_row(order, j, n) * dim + vi * VEC, r);
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] += r[e];
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) red[slot][ct * VEC + e] = acc[e];
        }
        __syncthreads();
        if (active && slot == 0) {
            float row[VEC];
            load_vec<T, VEC>(dwemb + tok * dim + vi * VEC, row);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float s = red[0][ct * VEC + e];
#pragma unroll
                for (int k = 1; k < EMB_SLOTS; ++k) s += red[k][ct * VEC + e];
                row[e] += s * scale;
            }
            store_vec<T, VEC>(dwemb + tok * dim + vi * VEC, row);
        }
        __syncthreads();
    }
}

template <typename T>
int embed_fwd_impl(const void* wemb, const void* pos, const int64_t* tokens, void* out, int64_t n, int64_t dim,
                   int64_t seq, int64_t vocab, float scale, int train, int64_t seed, hipStream_t st) {
    constexpr int FV = VecOf<T>::N;
    const bool vok = dim % FV == 0 && ptj_aligned16(wemb) && ptj_aligned16(pos) && ptj_aligned16(out);
    const int64_t work = n * (vok ? dim / FV : dim);
    int64_t blocks = (work + 255) / 256;
    if (blocks > (int64_t)ptj_num_cus() * 16) blocks = (int64_t)ptj_num_cus() * 16;
    if (vok)
        hipLaunchKernelGGL((embed_fwd_kernel<T, FV>), dim3((unsigned)blocks), dim3(256), 0, st, (const T*)wemb, (const T*)pos,
                           tokens, (T*)out, n, (int)dim, seq, vocab, scale, train, (uint64_t)seed);
    else
        hipLaunchKernelGGL((embed_fwd_kernel<T, 1>), dim3((unsigned)blocks), dim3(256), 0, st, (const T*)wemb, (const T*)pos,
                           tokens, (T*)out, n, (int)dim, seq, vocab, scale, train, (uint64_t)seed);
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

template <typename T>
int embed_bwd_impl(const void* d, const int64_t* sorted_tok, const int64_t* order, void* dwemb, int64_t n, int64_t dim,
                   int64_t vocab, float scale, hipStream_t st) {
    constexpr int FV = VecOf<T>::N;
    const bool vok = dim % FV == 0 && ptj_aligned16(d) && ptj_aligned16(dwemb);
    if (vok)
        hipLaunchKernelGGL((embed_bwd_kernel<T, FV>), dim3((unsigned)n), dim3(EMB_BWD_THREADS), 0, st, (const T*)d,
                           sorted_tok, order, (T*)dwemb, n, (int)dim, vocab, scale);
    else
        hipLaunchKernelGGL((embed_bwd_kernel<T, 1>), dim3((unsigned)n), dim3(EMB_BWD_THREADS), 0, st, (const T*)d,
                           sorted_tok, order, (T*)dwemb, n, (int)dim, vocab, scale);
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

}  // namespace

extern "C" {

int ptj_embed_fwd(const void* wemb, const void* pos, const int64_t* tokens, void* out, int64_t n, int64_t dim,
                  int64_t seq, int64_t vocab, float scale, int train, int64_t seed, int dtype, void* stream) {
    PTJ_CHECK_ARG(n >= 0 && dim >= 1 && dim < (1ll << 31) && seq >= 1 && vocab >= 1, "embed_fwd: bad shape");
    PTJ_CHECK_ARG(dtype == PTJ_F32 || dtype == PTJ_BF16, "embed_fwd: unknown dtype %d", dtype);
    if (n == 0) return PTJ_OK;
    PTJ_CHECK_ARG(wemb && pos && tokens && out, "embed_fwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    return dtype == PTJ_F32 ? embed_fwd_impl<float>(wemb, pos, tokens, out, n, dim, seq, vocab, scale, train, seed, st)
                            : embed_fwd_impl<bf16>(wemb, pos, tokens, out, n, dim, seq, vocab, scale, train, seed, st);
}

int ptj_embed_bwd(const void* d, const int64_t* sorted_tokens, const int64_t* order, void* dwemb, int64_t n,
                  int64_t dim, int64_t vocab, float scale, int dtype, void* stream) {
    PTJ_CHECK_ARG(n >= 0 && n < (1ll << 31) && dim >= 1 && dim < (1ll << 31) && vocab >= 1, "embed_bwd: bad shape");
    PTJ_CHECK_ARG(dtype == PTJ_F32 || dtype == PTJ_BF16, "embed_bwd: unknown dtype %d", dtype);
    if (n == 0) return PTJ_OK;
    PTJ_CHECK_ARG(d && sorted_tokens && order && dwemb, "embed_bwd: null pointer");
    hipStream_t st = (hipStream_t)stream;
    return dtype == PTJ_F32 ? embed_bwd_impl<float>(d, sorted_tokens, order, dwemb, n, dim, vocab, scale, st)
                            : embed_bwd_impl<bf16>(d, sorted_tokens, order, dwemb, n, dim, vocab, scale, st);
}

}  // extern "C"
