// Shared device/host helpers for the gfx950 kernels of libptj.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/ptj.h"

typedef __bf16 bf16;
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define PTJ_WAVE 64

// ---- host-side error plumbing -------------------------------------------------
int ptj_set_error(int code, const char* fmt, ...);
int ptj_num_cus();   // compute units of the current device (256 when no device can be asked)

#define PTJ_CHECK_ARG(cond, ...)                                   \
    do {                                                           \
        if (!(cond)) return ptj_set_error(PTJ_ERR_INVALID, __VA_ARGS__); \
    } while (0)

#define PTJ_CHECK_LAUNCH()                                                         \
    do {                                                                           \
        hipError_t e__ = hipGetLastError();                                        \
        if (e__ != hipSuccess)                                                     \
            return ptj_set_error(PTJ_ERR_LAUNCH, "%s: %s", __func__, hipGetErrorString(e__)); \
    } while (0)

static inline bool ptj_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ---- element <-> float conversion ---------------------------------------------
__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }

// 16-byte vector of T: 4 floats or 8 bf16.
template <typename T> struct VecOf;
template <> struct VecOf<float> { static constexpr int N = 4; };
template <> struct VecOf<bf16> { static constexpr int N = 8; };

template <typename T, int N> struct alignas(sizeof(T) * N) Pack { T v[N]; };

// Load N elements (N*sizeof(T) bytes, naturally aligned) and widen to float.
template <typename T, int N>
__device__ __forceinline__ void load_vec(const T* __restrict__ p, float (&out)[N]) {
    Pack<T, N> t = *reinterpret_cast<const Pack<T, N>*>(p);
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = to_f32(t.v[i]);
}
template <typename T, int N>
__device__ __forceinline__ void store_vec(T* __restrict__ p, const float (&in)[N]) {
    Pack<T, N> t;
#pragma unroll
    for (int i = 0; i < N; ++i) t.v[i] = from_f32<T>(in[i]);
    *reinterpret_cast<Pack<T, N>*>(p) = t;
}

// ---- wavefront (64 lanes) reductions --------------------------------------------
// All 64 lanes must be active.  Lanes are combined inside each row of 16 with DPP lane
// permutations (quad swaps, then row rotations by 4 and 8: no LDS crossbar round trips),
// and the four row results are read out and combined in row order, so every lane returns
// the same value and the order of the additions is fixed.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_move<0x124>(v);   // row_ror 4
    v += dpp_move<0x128>(v);   // row_ror 8
    return ((lane_value(v, 0) + lane_value(v, 16)) + lane_value(v, 32)) + lane_value(v, 48);
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x124>(v));
    v = fmaxf(v, dpp_move<0x128>(v));
    return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

__device__ __forceinline__ int wave_min_int(int v) {
    auto mv = [](int x, int y) { return y < x ? y : x; };
    v = mv(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false));
    v = mv(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false));
    v = mv(v, __builtin_amdgcn_update_dpp(0, v, 0x124, 0xf, 0xf, false));
    v = mv(v, __builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, false));
    return mv(mv(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
              mv(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

// Reduction over the TPR threads that share one row.  TPR == 64: one wave, no LDS.
// TPR > 64: TPR == blockDim.x, `smem` holds TPR/64 floats per call site; every
// thread of the block must call it (uses __syncthreads).
template <int TPR, bool IS_MAX>
__device__ __forceinline__ float row_reduce(float v, float* smem) {
    v = IS_MAX ? wave_max(v) : wave_sum(v);
    if constexpr (TPR > 64) {
        constexpr int NW = TPR / 64;
        const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
        __syncthreads();  // protect smem reuse between consecutive reductions
        if (l == 0) smem[w] = v;
        __syncthreads();
        float r = smem[0];
#pragma unroll
        for (int i = 1; i < NW; ++i) r = IS_MAX ? fmaxf(r, smem[i]) : r + smem[i];
        v = r;
    }
    return v;
}

// ---- Philox4x32-10, first output word -------------------------------------------
// Counter (offset,0,0,0), key (seed_lo, seed_hi): the generator behind the
// reference's dropout (Triton's tl.rand).  Only word 0 is produced, so the last
// two rounds are partly dead code the compiler removes.
__device__ __forceinline__ uint32_t philox_word0(uint32_t offset, uint32_t k0, uint32_t k1) {
    constexpr uint32_t KA = 0x9E3779B9u, KB = 0xBB67AE85u, RA = 0xD2511F53u, RB = 0xCD9E8D57u;
    uint32_t c0 = offset, c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t pa = (uint64_t)RA * c0;
        const uint64_t pb = (uint64_t)RB * c2;
        const uint32_t n0 = (uint32_t)(pb >> 32) ^ c1 ^ k0;
        const uint32_t n2 = (uint32_t)(pa >> 32) ^ c3 ^ k1;
        c1 = (uint32_t)pb;
        c3 = (uint32_t)pa;
        c0 = n0;
        c2 = n2;
        k0 += KA;
        k1 += KB;
    }
    return c0;
}

// Keep decision of the reference's dropout for rate p = 0.1:
//   x = int32(word); x = x < 0 ? -x-1 : x; keep iff float(x) * 4.6566127342e-10f > 0.1f.
// float(x)*scale is monotone in x, so this equals the integer compare x > 214748392
// (the largest x whose product is <= 0.1f); tests check the equivalence on the host.
#define PTJ_DROPOUT_KEEP_THRESHOLD 214748392
__device__ __forceinline__ bool philox_keep(uint32_t offset, uint32_t k0, uint32_t k1) {
    int32_t x = (int32_t)philox_word0(offset, k0, k1);
    x ^= (x >> 31);  // x < 0 ? -x-1 : x
    return x > PTJ_DROPOUT_KEEP_THRESHOLD;
}

// tanh-GELU.  The reference evaluates tanh(z) as 2*sigmoid(2z) - 1, so that
//   gelu(x)  = 0.5 x (1 + tanh z)                       = x * s
//   gelu'(x) = 0.5 (1 + tanh z) + 0.5 x (1 - tanh^2 z) z' = s + 2 x s (1 - s) z'
// with s = sigmoid(2z), z = k (x + 0.044715 x^3), z' = k (1 + 3*0.044715 x^2).
// s and 1-s are both formed from a = exp(-2|z|) <= 1, which avoids the cancellation
// of (1 + tanh z) for very negative z and any overflow.
struct SigPair { float s, om; };  // s = sigmoid(2z), om = 1 - s
__device__ __forceinline__ SigPair sigmoid2z(float z) {
    const float a = __expf(-2.0f * fabsf(z));
    const float r = __builtin_amdgcn_rcpf(1.0f + a);   // denominator in [1, 2]: the 1-ulp hardware reciprocal
    SigPair o;
    o.s = z >= 0.f ? r : a * r;
    o.om = z >= 0.f ? a * r : r;
    return o;
}
// Forward only needs s = 1 / (1 + exp(-2z)), which is accurate for every z as it stands
// (exp overflowing to +inf gives s = 0); -2 z log2(e) = x (c1 + c3 x^2) feeds the hardware exp2.
__device__ __forceinline__ float gelu_f(float x) {
    constexpr float k = 0.7978845608028654f, l2e = 1.4426950408889634f;
    constexpr float c1 = -2.0f * l2e * k, c3 = -2.0f * l2e * k * 0.044715f;
    const float e = __builtin_amdgcn_exp2f(x * fmaf(x * x, c3, c1));
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float gelu_grad_f(float x) {
    constexpr float k = 0.7978845608028654f;
    const float x2 = x * x;
    const SigPair sp = sigmoid2z(k * (x + 0.044715f * x * x2));
    return sp.s * (1.0f + 2.0f * x * sp.om * k * (1.0f + 3.0f * 0.044715f * x2));
}
