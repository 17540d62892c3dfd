// Fused AdamW step: one pass over (gradient, master weight, first and second moment) that
// also refreshes the low-precision copy the kernels compute with.  HBM-bound: 14 bytes
// read and 14 written per parameter with bf16 gradients and a bf16 shadow.
#include "common.h"

namespace {

template <typename G, typename S, bool HAS_SHADOW>
__global__ __launch_bounds__(256) void adamw_kernel(float* __restrict__ p, float* __restrict__ m, float* __restrict__ v,
                                                     const G* __restrict__ g, S* __restrict__ shadow, int64_t n4,
                                                     int64_t n, float lr, float b1, float b2, float eps, float wd,
                                                     float bc1, float bc2) {
    // body: 4 parameters per thread as 16-byte vectors
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
        float pp[4], mm[4], vv[4], gg[4];
        load_vec<float, 4>(p + i * 4, pp);
        load_vec<float, 4>(m + i * 4, mm);
        load_vec<float, 4>(v + i * 4, vv);
        load_vec<G, 4>(g + i * 4, gg);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            mm[j] = mm[j] * b1 + (1.0f - b1) * gg[j];
            vv[j] = vv[j] * b2 + (1.0f - b2) * gg[j] * gg[j];
            const float mh = mm[j] * bc1, vh = vv[j] * bc2;
            pp[j] = pp[j] + (-lr * (mh / (sqrtf(vh) + eps) + wd * pp[j]));
        }
        store_vec<float, 4>(p + i * 4, pp);
        store_vec<float, 4>(m + i * 4, mm);
        store_vec<float, 4>(v + i * 4, vv);
        if constexpr (HAS_SHADOW) store_vec<S, 4>(shadow + i * 4, pp);
    }
    // tail (n % 4 elements) by the first threads of block 0
    if (blockIdx.x == 0 && threadIdx.x < (unsigned)(n - n4 * 4)) {
        const int64_t i = n4 * 4 + threadIdx.x;
        const float gi = to_f32(g[i]);
        const float mi = m[i] * b1 + (1.0f - b1) * gi;
        const float vi = v[i] * b2 + (1.0f - b2) * gi * gi;
        const float pi = p[i] + (-lr * ((mi * bc1) / (sqrtf(vi * bc2) + eps) + wd * p[i]));
        m[i] = mi;
        v[i] = vi;
        p[i] = pi;
        if constexpr (HAS_SHADOW) shadow[i] = from_f32<S>(pi);
    }
}

// Multi-tensor form: one launch updates up to ADAMW_MAX tensors.  The descriptors travel in
// the kernel arguments; workgroup b belongs to the last tensor whose first_block <= b.
constexpr int ADAMW_MAX = 32;
struct AdamwItem {
    float* p;
    float* m;
    float* v;
    const void* g;
    void* shadow;
    int64_t n;
    float wd;
    int first_block;   // first workgroup of this tensor
    int nblocks;
    int pad;
};
struct AdamwBatch {
    AdamwItem it[ADAMW_MAX];
    int count;
};

template <typename G, typename S, bool HAS_SHADOW>
__global__ __launch_bounds__(256) void adamw_multi_kernel(const AdamwBatch b, float lr, float b1, float b2, float eps,
                                                           float bc1, float bc2) {
    int idx = 0;
    for (int k = 1; k < b.count; ++k)
        if ((int)blockIdx.x >= b.it[k].first_block) idx = k;
    const AdamwItem& t = b.it[idx];
    float* __restrict__ p = t.p;
    float* __restrict__ m = t.m;
    float* __restrict__ v = t.v;
    const G* __restrict__ g = (const G*)t.g;
    S* __restrict__ shadow = (S*)t.shadow;
    const int64_t n = t.n, n4 = n / 4;
    const float wd = t.wd;
    const int lb = (int)blockIdx.x - t.first_block;
    for (int64_t i = (int64_t)lb * 256 + threadIdx.x; i < n4; i += (int64_t)t.nblocks * 256) {
        float pp[4], mm[4], vv[4], gg[4];
        load_vec<float, 4>(p + i * 4, pp);
        load_vec<float, 4>(m + i * 4, mm);
        load_vec<float, 4>(v + i * 4, vv);
        load_vec<G, 4>(g + i * 4, gg);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            mm[j] = mm[j] * b1 + (1.0f - b1) * gg[j];
            vv[j] = vv[j] * b2 + (1.0f - b2) * gg[j] * gg[j];
            const float mh = mm[j] * bc1, vh = vv[j] * bc2;
            pp[j] = pp[j] + (-lr * (mh / (sqrtf(vh) + eps) + wd * pp[j]));
        }
        store_vec<float, 4>(p + i * 4, pp);
        store_vec<float, 4>(m + i * 4, mm);
        store_vec<float, 4>(v + i * 4, vv);
        if constexpr (HAS_SHADOW) store_vec<S, 4>(shadow + i * 4, pp);
    }
    if (lb == 0 && threadIdx.x < (unsigned)(n - n4 * 4)) {
        const int64_t i = n4 * 4 + threadIdx.x;
        const float gi = to_f32(g[i]);
        const float mi = m[i] * b1 + (1.0f - b1) * gi;
        const float vi = v[i] * b2 + (1.0f - b2) * gi * gi;
        const float pi = p[i] + (-lr * ((mi * bc1) / (sqrtf(vi * bc2) + eps) + wd * p[i]));
        m[i] = mi;
        v[i] = vi;
        p[i] = pi;
        if constexpr (HAS_SHADOW) shadow[i] = from_f32<S>(pi);
    }
}

}  // namespace

extern "C" {

int ptj_adamw_multi(int64_t count, float* const* p, float* const* m, float* const* v, const void* const* g,
                    void* const* shadow, const int64_t* n, const float* weight_decay, float lr, float beta1,
                    float beta2, float eps, int64_t t, int grad_dtype, int shadow_dtype, void* stream) {
    PTJ_CHECK_ARG(count >= 0 && t >= 1, "adamw_multi: need count >= 0 and step t >= 1");
    if (count == 0) return PTJ_OK;
    PTJ_CHECK_ARG(p && m && v && g && n && weight_decay, "adamw_multi: null table");
    PTJ_CHECK_ARG(grad_dtype == PTJ_F32 || grad_dtype == PTJ_BF16, "adamw_multi: unknown gradient dtype %d", grad_dtype);
    PTJ_CHECK_ARG(!shadow || shadow_dtype == PTJ_F32 || shadow_dtype == PTJ_BF16,
                  "adamw_multi: unknown shadow dtype %d", shadow_dtype);
    const uintptr_t gmask = grad_dtype == PTJ_BF16 ? 7 : 15, smask = shadow_dtype == PTJ_BF16 ? 7 : 15;
    for (int64_t i = 0; i < count; ++i) {
        PTJ_CHECK_ARG(n[i] >= 0, "adamw_multi: tensor %lld has a negative size", (long long)i);
        if (n[i] == 0) continue;
        PTJ_CHECK_ARG(p[i] && m[i] && v[i] && g[i] && (!shadow || shadow[i]), "adamw_multi: tensor %lld: null pointer",
                      (long long)i);
        PTJ_CHECK_ARG(ptj_aligned16(p[i]) && ptj_aligned16(m[i]) && ptj_aligned16(v[i]),
                      "adamw_multi: tensor %lld: state must be 16-byte aligned", (long long)i);
        PTJ_CHECK_ARG((reinterpret_cast<uintptr_t>(g[i]) & gmask) == 0 &&
                          (!shadow || (reinterpret_cast<uintptr_t>(shadow[i]) & smask) == 0),
                      "adamw_multi: tensor %lld: gradient / shadow must be aligned to 4 elements", (long long)i);
    }
    const float bc1 = (float)(1.0 / (1.0 - pow((double)beta1, (double)t)));
    const float bc2 = (float)(1.0 / (1.0 - pow((double)beta2, (double)t)));
    hipStream_t st = (hipStream_t)stream;
    int64_t i = 0;
    while (i < count) {
        AdamwBatch b;
        b.count = 0;
        int blocks = 0;
        for (; i < count && b.count < ADAMW_MAX; ++i) {
            if (n[i] == 0) continue;
            AdamwItem& it = b.it[b.count++];
            it.p = p[i]; it.m = m[i]; it.v = v[i]; it.g = g[i];
            it.shadow = shadow ? shadow[i] : nullptr;
            it.n = n[i];
            it.wd = weight_decay[i];
            int64_t nb = (n[i] / 4 + 255) / 256;
            if (nb > 2048) nb = 2048;
            if (nb < 1) nb = 1;
            it.first_block = blocks;
            it.nblocks = (int)nb;
            it.pad = 0;
            blocks += (int)nb;
        }
        if (b.count == 0) break;
#define ADAMW_MULTI(G_, S_, HS_)                                                                              \
    hipLaunchKernelGGL((adamw_multi_kernel<G_, S_, HS_>), dim3((unsigned)blocks), dim3(256), 0, st, b, lr, beta1, \
                       beta2, eps, bc1, bc2)
        if (grad_dtype == PTJ_BF16) {
            if (!shadow) ADAMW_MULTI(bf16, bf16, false);
            else if (shadow_dtype == PTJ_BF16) ADAMW_MULTI(bf16, bf16, true);
            else ADAMW_MULTI(bf16, float, true);
        } else {
            if (!shadow) ADAMW_MULTI(float, float, false);
            else if (shadow_dtype == PTJ_BF16) ADAMW_MULTI(float, bf16, true);
            else ADAMW_MULTI(float, float, true);
        }
#undef ADAMW_MULTI
        PTJ_CHECK_LAUNCH();
    }
    return PTJ_OK;
}

int ptj_adamw(float* p, float* m, float* v, const void* g, void* shadow, int64_t n, float lr, float beta1, float beta2,
              float eps, float weight_decay, int64_t t, int grad_dtype, int shadow_dtype, void* stream) {
    PTJ_CHECK_ARG(n >= 0 && t >= 1, "adamw: need n >= 0 and step t >= 1");
    if (n == 0) return PTJ_OK;
    PTJ_CHECK_ARG(p && m && v && g, "adamw: null pointer");
    PTJ_CHECK_ARG(ptj_aligned16(p) && ptj_aligned16(m) && ptj_aligned16(v), "adamw: state must be 16-byte aligned");
    PTJ_CHECK_ARG(grad_dtype == PTJ_F32 || grad_dtype == PTJ_BF16, "adamw: unknown gradient dtype %d", grad_dtype);
    PTJ_CHECK_ARG(!shadow || shadow_dtype == PTJ_F32 || shadow_dtype == PTJ_BF16, "adamw: unknown shadow dtype %d",
                  shadow_dtype);
    const bool g_al = (reinterpret_cast<uintptr_t>(g) & (grad_dtype == PTJ_BF16 ? 7 : 15)) == 0;
    const bool s_al = !shadow || (reinterpret_cast<uintptr_t>(shadow) & (shadow_dtype == PTJ_BF16 ? 7 : 15)) == 0;
    PTJ_CHECK_ARG(g_al && s_al, "adamw: gradient / shadow must be aligned to 4 elements");
    const float bc1 = (float)(1.0 / (1.0 - pow((double)beta1, (double)t)));
    const float bc2 = (float)(1.0 / (1.0 - pow((double)beta2, (double)t)));
    const int64_t n4 = n / 4;
    int64_t blocks = (n4 + 255) / 256;
    if (blocks > (int64_t)ptj_num_cus() * 8) blocks = (int64_t)ptj_num_cus() * 8;
    if (blocks < 1) blocks = 1;
    hipStream_t st = (hipStream_t)stream;
#define ADAMW_LAUNCH(G_, S_, HS_)                                                                                  \
    hipLaunchKernelGGL((adamw_kernel<G_, S_, HS_>), dim3((unsigned)blocks), dim3(256), 0, st, p, m, v, (const G_*)g, \
                       (S_*)shadow, n4, n, lr, beta1, beta2, eps, weight_decay, bc1, bc2)
    if (grad_dtype == PTJ_BF16) {
        if (!shadow) ADAMW_LAUNCH(bf16, bf16, false);
        else if (shadow_dtype == PTJ_BF16) ADAMW_LAUNCH(bf16, bf16, true);
        else ADAMW_LAUNCH(bf16, float, true);
    } else {
        if (!shadow) ADAMW_LAUNCH(float, float, false);
        else if (shadow_dtype == PTJ_BF16) ADAMW_LAUNCH(float, bf16, true);
        else ADAMW_LAUNCH(float, float, true);
    }
#undef ADAMW_LAUNCH
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

}  // extern "C"
