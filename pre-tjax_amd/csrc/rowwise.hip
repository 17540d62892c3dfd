// Row-wise, HBM-bound kernels: LayerNorm fwd/bwd, tanh-GELU fwd/bwd, Philox dropout,
// log-softmax fwd/bwd.  One row is owned by TPR threads (one wavefront for short rows,
// a 256- or 1024-thread workgroup for long ones) and lives in registers between the
// single HBM read and the single HBM write; all global accesses are 16-byte vectors
// when shapes allow (VEC = 16/sizeof(T)), scalar otherwise.
#include "common.h"

#include <mutex>

namespace {

// ---------------------------------------------------------------------------------
// Row holder: thread `t` of the TPR threads owning a row holds vectors
// t, t+TPR, t+2*TPR, ... (ITERS of them), each VEC consecutive elements.
// ---------------------------------------------------------------------------------
template <typename T, int VEC, int TPR, int ITERS>
struct RowRegs {
    float v[ITERS][VEC];
    __device__ __forceinline__ void load(const T* __restrict__ row, int nvec, int t, float fill) {
#pragma unroll
        // Branch-free: lanes past the end of the row re-read its last vector and discard it,
        // so that all loads of a row are in flight together (a load inside a per-lane branch
        // is followed by a full wait).
        for (int it = 0; it < ITERS; ++it) {
            const int vi = t + it * TPR;
            const int vc = vi < nvec ? vi : nvec - 1;
            load_vec<T, VEC>(row + (int64_t)vc * VEC, v[it]);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[it][j] = vi < nvec ? v[it][j] : fill;
        }
    }
    __device__ __forceinline__ void store(T* __restrict__ row, int nvec, int t) const {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int vi = t + it * TPR;
            if (vi < nvec) store_vec<T, VEC>(row + (int64_t)vi * VEC, v[it]);
        }
    }
};

// One row in storage type (ITERS 16-byte vectors per thread), for operands that are used
// once and late: they wait in a quarter (bf16) of the registers of their float form.
template <typename T, int VEC, int TPR, int ITERS>
struct RawRow {
    Pack<T, VEC> p[ITERS];
    __device__ __forceinline__ void load(const T* __restrict__ row, int nvec, int t) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int vi = t + it * TPR;
            const int vc = vi < nvec ? vi : nvec - 1;   // lanes past the row re-read its last vector
            p[it] = *reinterpret_cast<const Pack<T, VEC>*>(row + (int64_t)vc * VEC);
        }
    }
    __device__ __forceinline__ float get(int it, int j) const { return to_f32(p[it].v[j]); }
};

template <int TPR> struct RowGeom {
    static constexpr int BLOCK = TPR == 64 ? 256 : TPR;
    static constexpr int ROWS_PER_BLOCK = BLOCK / TPR;
};

// ---------------------------------------------------------------------------------
// LayerNorm forward
// ---------------------------------------------------------------------------------
template <typename T, int VEC, int TPR, int ITERS>
__global__ __launch_bounds__(RowGeom<TPR>::BLOCK) void layernorm_fwd_kernel(
    const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ beta, T* __restrict__ y,
    int64_t rows, int cols, int64_t xs, int64_t ys) {
    __shared__ float smem[16];
    constexpr int RPB = RowGeom<TPR>::ROWS_PER_BLOCK;
    const int t = threadIdx.x % TPR;
    const int sub = threadIdx.x / TPR;
    const int nvec = cols / VEC;
    RowRegs<T, VEC, TPR, ITERS> g, b;
    g.load(gamma, nvec, t, 0.f);
    b.load(beta, nvec, t, 0.f);
    const float inv_n = 1.0f / (float)cols;
    const float inv_nm1 = 1.0f / (float)(cols - 1);
    for (int64_t row = (int64_t)blockIdx.x * RPB + sub; row < rows; row += (int64_t)gridDim.x * RPB) {
        RowRegs<T, VEC, TPR, ITERS> r;
        r.load(x + row * xs, nvec, t, 0.f);
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) s += r.v[it][j];
        const float mu = row_reduce<TPR, false>(s, smem) * inv_n;
        float q = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const bool valid = (t + it * TPR) < nvec;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float d = valid ? r.v[it][j] - mu : 0.f;
                r.v[it][j] = d;
                q += d * d;
            }
        }
        const float var = row_reduce<TPR, false>(q, smem) * inv_nm1;
        const float rstd = 1.0f / sqrtf(var);
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[it][j] = g.v[it][j] * (r.v[it][j] * rstd) + b.v[it][j];
        r.store(y + row * ys, nvec, t);
    }
}

// ---------------------------------------------------------------------------------
// Residual update fused with the LayerNorm that consumes it, one row per wave / workgroup:
//   y = res + dropout(x)    exactly as dropout_kernel<ADD> (keep bytes recorded on request)
//   h = layernorm(y)        exactly as layernorm_fwd_kernel on the stored y
// A row's Philox key is uniform over its wave, so the key schedule runs on the scalar unit
// and y is never re-read.
// ---------------------------------------------------------------------------------
template <typename T, int VEC, int TPR, int ITERS>
__global__ __launch_bounds__(RowGeom<TPR>::BLOCK) void dropout_add_layernorm_kernel(
    const T* __restrict__ x, const T* __restrict__ res, const T* __restrict__ gamma, const T* __restrict__ beta,
    T* __restrict__ y, T* __restrict__ h, uint8_t* __restrict__ keep_out, int64_t rows, int cols, int train,
    uint64_t seed) {
    __shared__ float smem[16];
    constexpr int RPB = RowGeom<TPR>::ROWS_PER_BLOCK;
    const int t = threadIdx.x % TPR;
    const int sub = threadIdx.x / TPR;
    const int nvec = cols / VEC;
    RawRow<T, VEC, TPR, ITERS> g, b;
    g.load(gamma, nvec, t);
    b.load(beta, nvec, t);
    const float inv_n = 1.0f / (float)cols;
    const float inv_nm1 = 1.0f / (float)(cols - 1);
    for (int64_t row = (int64_t)blockIdx.x * RPB + sub; row < rows; row += (int64_t)gridDim.x * RPB) {
        RowRegs<T, VEC, TPR, ITERS> r;
        RawRow<T, VEC, TPR, ITERS> rr;
        r.load(x + row * (int64_t)cols, nvec, t, 0.f);
        rr.load(res + row * (int64_t)cols, nvec, t);
        const uint64_t sd = seed + (uint64_t)row;
        // the row, and so the key, is the same for all lanes of the wave
        const uint32_t k0 = __builtin_amdgcn_readfirstlane((uint32_t)sd);
        const uint32_t k1 = __builtin_amdgcn_readfirstlane((uint32_t)(sd >> 32));
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int vi = t + it * TPR;
            const bool valid = vi < nvec;
            if (train) {
                uint32_t bits = 0;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const bool keep = philox_keep((uint32_t)(vi * VEC + j), k0, k1);
                    r.v[it][j] = keep ? r.v[it][j] : 0.f;
                    bits |= keep ? (1u << j) : 0u;
                }
                if constexpr (sizeof(T) == 2 && (VEC == 8 || VEC == 4)) {
                    if (keep_out != nullptr) {   // one byte per 8 columns
                        if constexpr (VEC == 8) {
                            if (valid) keep_out[row * (int64_t)(cols >> 3) + vi] = (uint8_t)bits;
                        } else {
                            // lanes 2i and 2i+1 hold the two halves of a byte
                            const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)bits, 0xB1, 0xf, 0xf, false);
                            if (valid && (vi & 1) == 0)
                                keep_out[row * (int64_t)(cols >> 3) + (vi >> 1)] = (uint8_t)(bits | (other << 4));
                        }
                    }
                }
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) r.v[it][j] *= 0.9f;
            }
            // dropout(x) is rounded to the storage type before the add, the sum again on store
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float v = rr.get(it, j) + to_f32(from_f32<T>(r.v[it][j]));
                r.v[it][j] = valid ? to_f32(from_f32<T>(v)) : 0.f;
            }
        }
        r.store(y + row * (int64_t)cols, nvec, t);
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) s += r.v[it][j];
        const float mu = row_reduce<TPR, false>(s, smem) * inv_n;
        float q = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const bool valid = (t + it * TPR) < nvec;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float d = valid ? r.v[it][j] - mu : 0.f;
                r.v[it][j] = d;
                q += d * d;
            }
        }
        const float var = row_reduce<TPR, false>(q, smem) * inv_nm1;
        const float rstd = 1.0f / sqrtf(var);
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[it][j] = g.get(it, j) * (r.v[it][j] * rstd) + b.get(it, j);
        r.store(h + row * (int64_t)cols, nvec, t);
    }
}

// ---------------------------------------------------------------------------------
// LayerNorm backward: dx and/or per-block partial sums of dgamma, dbeta.
// Partials layout: part[p][0][cols] = sum dy*xhat, part[p][1][cols] = sum dy over the
// rows handled by row-slot p (p = blockIdx.x*RPB + sub).
// ---------------------------------------------------------------------------------
template <int TPR> struct LnBwdGeom {
    static constexpr int BLOCK = TPR == 64 ? 512 : TPR;
    static constexpr int ROWS_PER_BLOCK = BLOCK / TPR;
};
constexpr int LN_BWD_MAX_WAVE_COLS = 64 * 4 * 8;  // widest row a single wave holds (bf16, ITERS 4)

// DROP selects the code for the second (dropout) output at compile time, which keeps the
// Philox generator out of the register budget of the common variants: 0 = no second
// output, 1 = mask read from recorded keep bytes, 2 = mask recomputed (or eval scaling).
template <typename T, int VEC, int TPR, int ITERS, bool DX, bool DGB, int DROP>
__global__ __launch_bounds__(LnBwdGeom<TPR>::BLOCK, (TPR == 64 && ITERS <= 3 && DROP != 2) ? 4 : 2) void layernorm_bwd_kernel(
    const T* __restrict__ dy, const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ res,
    T* __restrict__ dx, float* __restrict__ part, int64_t rows, int cols, int64_t dys, int64_t xs, int64_t dxs,
    T* __restrict__ drop, int drop_train, uint64_t drop_seed, const uint8_t* __restrict__ keep, int np,
    int has_res, int64_t ress) {
    // res is always a readable row source (the host passes dy when there is no residual), so
    // that its load is unconditional; has_res says whether it is added.
    // np: partial sums per workgroup and column: dgamma, dbeta and, with np == 3, the
    // column sums of the `drop` output
    __shared__ float smem[16];
    constexpr int RPB = LnBwdGeom<TPR>::ROWS_PER_BLOCK;
    const int t = threadIdx.x % TPR;
    const int sub = threadIdx.x / TPR;
    const int nvec = cols / VEC;
    RawRow<T, VEC, TPR, ITERS> g;
    if constexpr (DX) g.load(gamma, nvec, t);
    float acc_g[ITERS][VEC], acc_b[ITERS][VEC], acc_d[ITERS][VEC];
    if constexpr (DGB) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc_g[it][j] = acc_b[it][j] = acc_d[it][j] = 0.f;
    }
    const float inv_n = 1.0f / (float)cols;
    const float inv_nm1 = 1.0f / (float)(cols - 1);
    const float n_adj = (float)cols * inv_nm1;
    // Every thread of a >64-thread row group must take the same trip count because
    // row_reduce synchronises the block; with RPB == 1 all threads share `row`.
#pragma unroll 1
    for (int64_t row = (int64_t)blockIdx.x * RPB + sub; row < rows; row += (int64_t)gridDim.x * RPB) {
        RowRegs<T, VEC, TPR, ITERS> r, d;
        RawRow<T, VEC, TPR, ITERS> rr;
        r.load(x + row * xs, nvec, t, 0.f);
        d.load(dy + row * dys, nvec, t, 0.f);
        if constexpr (DX) {
            // residual row, in flight under the reductions
            rr.load(res + row * ress, nvec, t);
        }
        uint32_t kbits[ITERS];
        if constexpr (DROP == 1) {
            // keep bytes of this row (one per vector), fetched with the row instead of after it
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int vi = t + it * TPR;
                const int c0 = (vi < nvec ? vi : nvec - 1) * VEC;          // one keep byte per 8 columns
                kbits[it] = (uint32_t)keep[row * (int64_t)(cols >> 3) + (c0 >> 3)] >> (c0 & 7);
            }
        }
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) s += r.v[it][j];
        const float mu = row_reduce<TPR, false>(s, smem) * inv_n;
        float q = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const bool valid = (t + it * TPR) < nvec;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float c = valid ? r.v[it][j] - mu : 0.f;
                r.v[it][j] = c;
                q += c * c;
            }
        }
        const float var = row_reduce<TPR, false>(q, smem) * inv_nm1;
        const float rstd = 1.0f / sqrtf(var);
        float sg = 0.f, sgx = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float xh = r.v[it][j] * rstd;
                r.v[it][j] = xh;
                if constexpr (DGB) {
                    acc_g[it][j] += d.v[it][j] * xh;
                    acc_b[it][j] += d.v[it][j];
                }
                if constexpr (DX) {
                    const float gg = d.v[it][j] * g.get(it, j);
                    d.v[it][j] = gg;
                    sg += gg;
                    sgx += gg * xh;
                }
            }
        if constexpr (DX) {
            const float mg = row_reduce<TPR, false>(sg, smem) * inv_n;
            const float mgx = row_reduce<TPR, false>(sgx, smem) * inv_n * n_adj;
#pragma unroll
            for (int it = 0; it < ITERS; ++it)
#pragma unroll
                for (int j = 0; j < VEC; ++j) d.v[it][j] = (d.v[it][j] - mg - r.v[it][j] * mgx) * rstd;
            if (has_res) {
                // residual branch: the sum is formed from the storage-rounded LayerNorm gradient,
                // as two separate passes would
#pragma unroll
                for (int it = 0; it < ITERS; ++it)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) d.v[it][j] = rr.get(it, j) + to_f32(from_f32<T>(d.v[it][j]));
            }
            d.store(dx + row * dxs, nvec, t);
            if constexpr (DROP != 0) {
                // second output: dropout applied to the stored (rounded) dx, i.e. the backward
                // of the dropout that feeds this residual stream -- saves a pass over dx
                const uint64_t sd = drop_seed + (uint64_t)row;
                const uint32_t k0 = (uint32_t)sd, k1 = (uint32_t)(sd >> 32);
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    const int vi = t + it * TPR;
                    // keep bits of this vector: recorded by the forward dropout (one byte per
                    // 8 columns) when available, else recomputed
                    uint32_t bits = 0;
                    if constexpr (DROP == 1) {
                        bits = kbits[it];
                    } else {
                        if (drop_train) {
#pragma unroll
                            for (int j = 0; j < VEC; ++j)
                                bits |= philox_keep((uint32_t)(vi * VEC + j), k0, k1) ? (1u << j) : 0u;
                        }
                    }
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        const float r = to_f32(from_f32<T>(d.v[it][j]));
                        d.v[it][j] = drop_train ? (((bits >> j) & 1u) ? r : 0.f) : r * 0.9f;
                        if constexpr (DGB) {
                            if (np == 3) acc_d[it][j] += to_f32(from_f32<T>(d.v[it][j]));   // the stored value
                        }
                    }
                }
                d.store(drop + row * (int64_t)cols, nvec, t);
            }
        }
    }
    if constexpr (DGB) {
        // One partial per workgroup.  With several row slots per workgroup the slots are
        // folded through LDS in slot order (deterministic).
        float* pg = part + (int64_t)blockIdx.x * np * (int64_t)cols;
        float* pb = pg + cols;
        float* pd = pb + cols;
        if constexpr (RPB > 1) {
            __shared__ float red[3][LN_BWD_MAX_WAVE_COLS];
            for (int s = 0; s < RPB; ++s) {
                if (sub == s) {
#pragma unroll
                    for (int it = 0; it < ITERS; ++it) {
                        const int vi = t + it * TPR;
                        if (vi < nvec) {
#pragma unroll
                            for (int j = 0; j < VEC; ++j) {
                                const int c = vi * VEC + j;
                                red[0][c] = s == 0 ? acc_g[it][j] : red[0][c] + acc_g[it][j];
                                red[1][c] = s == 0 ? acc_b[it][j] : red[1][c] + acc_b[it][j];
                                red[2][c] = s == 0 ? acc_d[it][j] : red[2][c] + acc_d[it][j];
                            }
                        }
                    }
                }
                __syncthreads();
            }
            for (int c = threadIdx.x; c < cols; c += LnBwdGeom<TPR>::BLOCK) {
                pg[c] = red[0][c];
                pb[c] = red[1][c];
                if (np == 3) pd[c] = red[2][c];
            }
        } else {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int vi = t + it * TPR;
                if (vi < nvec) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        pg[vi * VEC + j] = acc_g[it][j];
                        pb[vi * VEC + j] = acc_b[it][j];
                        if (np == 3) pd[vi * VEC + j] = acc_d[it][j];
                    }
                }
            }
        }
    }
}

// layernorm_bwd_kernel<T, VEC, 64, ITERS, true, true, DROP> (DROP 0 or 1) for rows of exactly
// 64 * VEC * ITERS columns: every lane holds whole vectors, so nothing is masked, and the row after
// the current one is requested -- all of its vectors at once, in storage form -- before the current
// row's arithmetic starts (the general kernel's loads end up interleaved with the conversions that
// consume them, a row at a time).  Same operations in the same order as the general kernel: the
// results are bit-equal to it.
template <typename T, int VEC, int ITERS, int DROP>
__global__ __launch_bounds__(512, DROP == 1 ? 2 : 4) void layernorm_bwd_exact_kernel(
    const T* __restrict__ dy, const T* __restrict__ x, const T* __restrict__ gamma, const T* __restrict__ res,
    T* __restrict__ dx, float* __restrict__ part, int64_t rows, int64_t dys, int64_t xs, int64_t dxs,
    T* __restrict__ drop, int drop_train, const uint8_t* __restrict__ keep, int np, int has_res, int64_t ress) {
    constexpr int TPR = 64, RPB = 8;
    constexpr int cols = TPR * VEC * ITERS;
    static_assert(DROP == 0 || DROP == 1, "keep-byte or no dropout output");
    static_assert(DROP == 0 || (VEC == 4 || VEC == 8), "one keep byte per 8 columns");
    const int t = threadIdx.x & 63;
    const int sub = threadIdx.x >> 6;
    Pack<T, VEC> graw[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) graw[it] = *reinterpret_cast<const Pack<T, VEC>*>(gamma + (t + it * TPR) * VEC);
    float acc_g[ITERS][VEC], acc_b[ITERS][VEC], acc_d[ITERS][VEC];
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc_g[it][j] = acc_b[it][j] = acc_d[it][j] = 0.f;
    const float inv_n = 1.0f / (float)cols;
    const float inv_nm1 = 1.0f / (float)(cols - 1);
    const float n_adj = (float)cols * inv_nm1;
    const int64_t stride = (int64_t)gridDim.x * RPB;
    Pack<T, VEC> nx[ITERS], nd[ITERS], nr[ITERS];
    uint8_t nk[ITERS];
#define LNX_REQUEST(ROW)                                                                                  \
    do {                                                                                                  \
        const T* xr__ = x + (ROW) * xs;                                                                   \
        const T* dr__ = dy + (ROW) * dys;                                                                 \
        const T* rr__ = res + (ROW) * ress;                                                               \
        _Pragma("unroll") for (int it = 0; it < ITERS; ++it) {                                            \
            const int c__ = (t + it * TPR) * VEC;                                                         \
            nx[it] = *reinterpret_cast<const Pack<T, VEC>*>(xr__ + c__);                                  \
            nd[it] = *reinterpret_cast<const Pack<T, VEC>*>(dr__ + c__);                                  \
            nr[it] = *reinterpret_cast<const Pack<T, VEC>*>(rr__ + c__);                                  \
            if constexpr (DROP == 1) nk[it] = keep[(ROW) * (int64_t)(cols >> 3) + (c__ >> 3)];            \
        }                                                                                                 \
    } while (0)
    int64_t row = (int64_t)blockIdx.x * RPB + sub;
    if (row < rows) LNX_REQUEST(row);
#pragma unroll 1
    for (; row < rows; row += stride) {
        float xv[ITERS][VEC], dv[ITERS][VEC];
        Pack<T, VEC> rr[ITERS];
        uint32_t kbits[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                xv[it][j] = to_f32(nx[it].v[j]);
                dv[it][j] = to_f32(nd[it].v[j]);
            }
            rr[it] = nr[it];
            if constexpr (DROP == 1) kbits[it] = (uint32_t)nk[it] >> (((t + it * TPR) * VEC) & 7);
        }
        // the next row of this slot (the last one asks for its own row again: no branch around the loads)
        const int64_t nrow = row + stride < rows ? row + stride : row;
        LNX_REQUEST(nrow);
        __builtin_amdgcn_sched_barrier(0);
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) s += xv[it][j];
        const float mu = wave_sum(s) * inv_n;
        float q = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float c = xv[it][j] - mu;
                xv[it][j] = c;
                q += c * c;
            }
        const float var = wave_sum(q) * inv_nm1;
        const float rstd = 1.0f / sqrtf(var);
        float sg = 0.f, sgx = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float xh = xv[it][j] * rstd;
                xv[it][j] = xh;
                acc_g[it][j] += dv[it][j] * xh;
                acc_b[it][j] += dv[it][j];
                const float gg = dv[it][j] * to_f32(graw[it].v[j]);
                dv[it][j] = gg;
                sg += gg;
                sgx += gg * xh;
            }
        const float mg = wave_sum(sg) * inv_n;
        const float mgx = wave_sum(sgx) * inv_n * n_adj;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) dv[it][j] = (dv[it][j] - mg - xv[it][j] * mgx) * rstd;
        if (has_res) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it)
#pragma unroll
                for (int j = 0; j < VEC; ++j) dv[it][j] = to_f32(rr[it].v[j]) + to_f32(from_f32<T>(dv[it][j]));
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) store_vec<T, VEC>(dx + row * dxs + (t + it * TPR) * VEC, dv[it]);
        if constexpr (DROP == 1) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const float r = to_f32(from_f32<T>(dv[it][j]));
                    dv[it][j] = drop_train ? (((kbits[it] >> j) & 1u) ? r : 0.f) : r * 0.9f;
                    if (np == 3) acc_d[it][j] += to_f32(from_f32<T>(dv[it][j]));   // the stored value
                }
                store_vec<T, VEC>(drop + row * (int64_t)cols + (t + it * TPR) * VEC, dv[it]);
            }
        }
    }
#undef LNX_REQUEST
    // one partial per workgroup: the eight row slots are folded through LDS in slot order
    float* pg = part + (int64_t)blockIdx.x * np * (int64_t)cols;
    float* pb = pg + cols;
    float* pd = pb + cols;
    __shared__ float red[3][cols];
    for (int sl = 0; sl < RPB; ++sl) {
        if (sub == sl) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it)
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const int c = (t + it * TPR) * VEC + j;
                    red[0][c] = sl == 0 ? acc_g[it][j] : red[0][c] + acc_g[it][j];
                    red[1][c] = sl == 0 ? acc_b[it][j] : red[1][c] + acc_b[it][j];
                    red[2][c] = sl == 0 ? acc_d[it][j] : red[2][c] + acc_d[it][j];
                }
        }
        __syncthreads();
    }
    for (int c = threadIdx.x; c < cols; c += 512) {
        pg[c] = red[0][c];
        pb[c] = red[1][c];
        if (np == 3) pd[c] = red[2][c];
    }
}

// Sum over partials for one column, shared by the second-stage reducers: 1024 threads =
// 32 columns x 32 slices; slice py adds partials py, py+32, ... (four independent chains so
// that the loads overlap), then the slices are folded through LDS in slice order.
constexpr int RED_THREADS = 1024;
__device__ __forceinline__ float reduce_partials(const float* __restrict__ col_base, int64_t stride, int nparts,
                                                 bool active, float (&sm)[32][33]) {
    const int cx = threadIdx.x & 31, py = threadIdx.x >> 5;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (active) {
        int p = py;
        for (; p + 96 < nparts; p += 128) {
            s0 += col_base[(int64_t)p * stride];
            s1 += col_base[(int64_t)(p + 32) * stride];
            s2 += col_base[(int64_t)(p + 64) * stride];
            s3 += col_base[(int64_t)(p + 96) * stride];
        }
        for (; p < nparts; p += 32) s0 += col_base[(int64_t)p * stride];
    }
    sm[py][cx] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    float r = 0.f;
    if (py == 0) {
#pragma unroll
        for (int i = 0; i < 32; ++i) r += sm[i][cx];
    }
    return r;
}

// Second stage: out[which][c] = sum_p part[p][which][c], fixed order.  grid = (ceil(cols/32), np)
// with np = 2 (dgamma, dbeta) or 3 (and the column sums of the dropped output).
template <typename T>
__global__ __launch_bounds__(RED_THREADS) void layernorm_bwd_reduce_kernel(const float* __restrict__ part, int nparts,
                                                                            int cols, T* __restrict__ dgamma,
                                                                            T* __restrict__ dbeta, T* __restrict__ dsum) {
    __shared__ float sm[32][33];
    const int c = blockIdx.x * 32 + (threadIdx.x & 31);
    const int which = blockIdx.y, np = gridDim.y;
    const float r = reduce_partials(part + (int64_t)which * cols + c, np * (int64_t)cols, nparts, c < cols, sm);
    if ((threadIdx.x >> 5) == 0 && c < cols) (which == 0 ? dgamma : which == 1 ? dbeta : dsum)[c] = from_f32<T>(r);
}

// ---------------------------------------------------------------------------------
// log-softmax forward / backward
// ---------------------------------------------------------------------------------
template <typename T, int VEC, int TPR, int ITERS>
__global__ __launch_bounds__(RowGeom<TPR>::BLOCK) void log_softmax_fwd_kernel(const T* __restrict__ x,
                                                                               T* __restrict__ y, int64_t rows,
                                                                               int cols, int64_t xs, int64_t ys) {
    __shared__ float smem[16];
    constexpr int RPB = RowGeom<TPR>::ROWS_PER_BLOCK;
    const int t = threadIdx.x % TPR;
    const int sub = threadIdx.x / TPR;
    const int nvec = cols / VEC;
    for (int64_t row = (int64_t)blockIdx.x * RPB + sub; row < rows; row += (int64_t)gridDim.x * RPB) {
        RowRegs<T, VEC, TPR, ITERS> r;
        r.load(x + row * xs, nvec, t, -INFINITY);
        float m = -INFINITY;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) m = fmaxf(m, r.v[it][j]);
        m = row_reduce<TPR, true>(m, smem);
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                r.v[it][j] -= m;
                s += __expf(r.v[it][j]);
            }
        const float lse = logf(row_reduce<TPR, false>(s, smem));
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) r.v[it][j] -= lse;
        r.store(y + row * ys, nvec, t);
    }
}

template <typename T, int VEC, int TPR, int ITERS>
__global__ __launch_bounds__(RowGeom<TPR>::BLOCK) void log_softmax_bwd_kernel(
    const T* __restrict__ dy, const T* __restrict__ x, T* __restrict__ dx, int64_t rows, int cols, int64_t dys,
    int64_t xs, int64_t dxs) {
    __shared__ float smem[16];
    constexpr int RPB = RowGeom<TPR>::ROWS_PER_BLOCK;
    const int t = threadIdx.x % TPR;
    const int sub = threadIdx.x / TPR;
    const int nvec = cols / VEC;
    for (int64_t row = (int64_t)blockIdx.x * RPB + sub; row < rows; row += (int64_t)gridDim.x * RPB) {
        RowRegs<T, VEC, TPR, ITERS> r, d;
        r.load(x + row * xs, nvec, t, -INFINITY);
        d.load(dy + row * dys, nvec, t, 0.f);
        float m = -INFINITY, sd = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                m = fmaxf(m, r.v[it][j]);
                sd += d.v[it][j];
            }
        m = row_reduce<TPR, true>(m, smem);
        sd = row_reduce<TPR, false>(sd, smem);
        float s = 0.f;
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                r.v[it][j] = __expf(r.v[it][j] - m);
                s += r.v[it][j];
            }
        const float c = sd / row_reduce<TPR, false>(s, smem);
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j) d.v[it][j] -= r.v[it][j] * c;
        d.store(dx + row * dxs, nvec, t);
    }
}

// ---------------------------------------------------------------------------------
// Elementwise: GELU fwd/bwd (flat), dropout (+ residual add)
// ---------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gelu_fwd_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t nvec) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        float v[VEC];
        load_vec<T, VEC>(x + i * VEC, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = gelu_f(v[j]);
        store_vec<T, VEC>(y + i * VEC, v);
    }
}
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gelu_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                        T* __restrict__ dx, int64_t nvec) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        float v[VEC], d[VEC];
        load_vec<T, VEC>(x + i * VEC, v);
        load_vec<T, VEC>(dy + i * VEC, d);
#pragma unroll
        for (int j = 0; j < VEC; ++j) d[j] *= gelu_grad_f(v[j]);
        store_vec<T, VEC>(dx + i * VEC, d);
    }
}

// One thread per VEC-wide chunk; chunks never straddle rows (cols % VEC == 0).
template <typename T, int VEC, bool ADD>
__global__ __launch_bounds__(256) void dropout_kernel(const T* __restrict__ x, const T* __restrict__ res,
                                                       T* __restrict__ y, int64_t rows, int cols, int64_t xs,
                                                       int64_t ys, int train, uint64_t seed,
                                                       uint8_t* __restrict__ keep_out) {
    const int vpr = cols / VEC;  // vectors per row
    const int64_t total = rows * vpr;
    const bool small = total <= 0x7fffffffll;  // 32-bit division is several times cheaper
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t row = small ? (int64_t)((uint32_t)i / (uint32_t)vpr) : i / vpr;
        const int c0 = (int)(i - row * vpr) * VEC;
        float v[VEC];
        load_vec<T, VEC>(x + row * xs + c0, v);
        if (train) {
            const uint64_t s = seed + (uint64_t)row;
            const uint32_t k0 = (uint32_t)s, k1 = (uint32_t)(s >> 32);
            uint32_t bits = 0;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const bool keep = philox_keep((uint32_t)(c0 + j), k0, k1);
                v[j] = keep ? v[j] : 0.f;
                bits |= keep ? (1u << j) : 0u;
            }
            // keep byte of this 8-column group (only requested on the 8-wide path)
            if (VEC == 8 && keep_out != nullptr) keep_out[i] = (uint8_t)bits;
        } else {
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= 0.9f;
        }
        if constexpr (ADD) {
            float r[VEC];
            load_vec<T, VEC>(res + row * (int64_t)cols + c0, r);
            // The reference rounds dropout(x) to the storage type before adding it.
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] = r[j] + to_f32(from_f32<T>(v[j]));
        }
        store_vec<T, VEC>(y + row * ys + c0, v);
    }
}

// ---------------------------------------------------------------------------------
// Column sums, two stages.  Stage 1: block (bx, by) sums rows [by*rps, (by+1)*rps) of the
// 128*VEC columns starting at bx*128*VEC into part[by][col].  Stage 2 reuses the
// LayerNorm partial reducer layout (part[p][1][cols] with a single "which").
// ---------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(128) void colsum_stage1_kernel(const T* __restrict__ x, float* __restrict__ part,
                                                            int64_t rows, int cols, int64_t xs, int rows_per_split) {
    const int c0 = (blockIdx.x * 128 + threadIdx.x) * VEC;
    if (c0 >= cols) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_split;
    const int64_t r1 = r0 + rows_per_split < rows ? r0 + rows_per_split : rows;
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
    constexpr int U = 8;   // independent row loads in flight per thread
    int64_t r = r0;
    for (; r + U <= r1; r += U) {
        float v[U][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u) load_vec<T, VEC>(x + (r + u) * xs + c0, v[u]);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j] += v[u][j];
    }
    for (; r < r1; ++r) {
        float v[VEC];
        load_vec<T, VEC>(x + r * xs + c0, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[j] += v[j];
    }
    float* dst = part + (int64_t)blockIdx.y * cols + c0;
#pragma unroll
    for (int j = 0; j < VEC; ++j) dst[j] = acc[j];
}
template <typename T>
__global__ __launch_bounds__(RED_THREADS) void colsum_stage2_kernel(const float* __restrict__ part, int nparts, int cols,
                                                                     T* __restrict__ out) {
    __shared__ float sm[32][33];
    const int c = blockIdx.x * 32 + (threadIdx.x & 31);
    const float r = reduce_partials(part + c, (int64_t)cols, nparts, c < cols, sm);
    if ((threadIdx.x >> 5) == 0 && c < cols) out[c] = from_f32<T>(r);
}

// Second stage for a few partial rows (wide tensors with few rows, e.g. the sum over the batch
// that is the positional table's gradient): one thread per column, the partials added in order.
template <typename T>
__global__ __launch_bounds__(256) void colsum_stage2_few_kernel(const float* __restrict__ part, int nparts, int cols,
                                                                 T* __restrict__ out) {
    for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < cols; c += (int64_t)gridDim.x * 256) {
        float s = 0.f;
        for (int p = 0; p < nparts; ++p) s += part[(int64_t)p * cols + c];
        out[c] = from_f32<T>(s);
    }
}

// GELU backward with the column sums of its own output (the bias gradient of the linear
// layer in front of the GELU).  A workgroup owns whole rows: `tpr` threads cover a row
// (thread t the 16-byte vectors t, t + tpr, ... : contiguous accesses) and the workgroup
// holds blockDim / tpr such row slots, which take the rows of the workgroup's range
// [b*rps, (b+1)*rps) in turn.  dx is written, the sums of the stored (storage-rounded) dx
// values are folded over the slots through LDS in slot order and left in part[b][col].
// NV = vectors per thread.
constexpr int GELU_CS_MAX_LDS_COLS = 8192;   // floats of LDS for the slot fold
template <typename T, int VEC, int NV>
__global__ __launch_bounds__(1024) void gelu_bwd_colsum_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                               T* __restrict__ dx, float* __restrict__ part,
                                                               int64_t rows, int cols, int rows_per_split, int tpr) {
    __shared__ float red[GELU_CS_MAX_LDS_COLS];
    const int nvec = cols / VEC;
    const int slots = blockDim.x / tpr, slot = threadIdx.x / tpr, tx = threadIdx.x - slot * tpr;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_split;
    const int64_t r1 = r0 + rows_per_split < rows ? r0 + rows_per_split : rows;
    float acc[NV][VEC];
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
        for (int j = 0; j < VEC; ++j) acc[k][j] = 0.f;
    constexpr int U = NV == 1 ? 4 : 2;   // independent rows in flight per thread
    int64_t r = r0 + slot;
    for (; r + (int64_t)(U - 1) * slots < r1; r += (int64_t)U * slots) {
        float v[U][NV][VEC], d[U][NV][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int vi = tx + k * tpr;
                const int vc = vi < nvec ? vi : nvec - 1;
                load_vec<T, VEC>(x + (r + u * slots) * (int64_t)cols + (int64_t)vc * VEC, v[u][k]);
                load_vec<T, VEC>(dy + (r + u * slots) * (int64_t)cols + (int64_t)vc * VEC, d[u][k]);
            }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int vi = tx + k * tpr;
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    d[u][k][j] = to_f32(from_f32<T>(d[u][k][j] * gelu_grad_f(v[u][k][j])));
                    acc[k][j] += d[u][k][j];
                }
                if (vi < nvec) store_vec<T, VEC>(dx + (r + u * slots) * (int64_t)cols + (int64_t)vi * VEC, d[u][k]);
            }
    }
    for (; r < r1; r += slots) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int vi = tx + k * tpr;
            const int vc = vi < nvec ? vi : nvec - 1;
            float v[VEC], d[VEC];
            load_vec<T, VEC>(x + r * (int64_t)cols + (int64_t)vc * VEC, v);
            load_vec<T, VEC>(dy + r * (int64_t)cols + (int64_t)vc * VEC, d);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                d[j] = to_f32(from_f32<T>(d[j] * gelu_grad_f(v[j])));
                acc[k][j] += d[j];
            }
            if (vi < nvec) store_vec<T, VEC>(dx + r * (int64_t)cols + (int64_t)vi * VEC, d);
        }
    }
    // fold the slots in slot order (only used with slots > 1, which the host allows when
    // the row fits the LDS array)
    for (int s = 1; s < slots; ++s) {
        if (slot == s) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int vi = tx + k * tpr;
                if (vi < nvec) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) red[vi * VEC + j] = acc[k][j];
                }
            }
        }
        __syncthreads();
        if (slot == 0) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int vi = tx + k * tpr;
                if (vi < nvec) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[k][j] += red[vi * VEC + j];
                }
            }
        }
        __syncthreads();
    }
    if (slot == 0) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int vi = tx + k * tpr;
            if (vi < nvec) {
                float* dst = part + (int64_t)blockIdx.x * cols + (int64_t)vi * VEC;
#pragma unroll
                for (int j = 0; j < VEC; ++j) dst[j] = acc[k][j];
            }
        }
    }
}

inline void colsum_geometry(int64_t rows, int64_t cols, int vec, int* gx, int* splits, int* rps) {
    *gx = (int)((cols + 128 * vec - 1) / (128 * vec));
    int64_t s = 2048 / *gx;
    if (s > 512) s = 512;
    if (s < 1) s = 1;
    if (s > (rows + 31) / 32) s = (rows + 31) / 32;
    if (s < 1) s = 1;
    *rps = (int)((rows + s - 1) / s);
    *splits = (int)((rows + *rps - 1) / *rps);
}

template <typename T>
int colsum_impl(const void* x, void* out, void* ws, size_t ws_bytes, int64_t rows, int64_t cols, int64_t xs,
                hipStream_t st) {
    constexpr int FV = VecOf<T>::N;
    const bool vok = (cols % FV == 0) && (xs % FV == 0) && ptj_aligned16(x);
    const int vec = vok ? FV : 1;
    int gx, splits, rps;
    colsum_geometry(rows, cols, vec, &gx, &splits, &rps);
    const size_t need = (size_t)splits * cols * sizeof(float);
    if (!ws || ws_bytes < need) return ptj_set_error(PTJ_ERR_WORKSPACE, "colsum: workspace %zu < %zu bytes", ws_bytes, need);
    if (vok)
        hipLaunchKernelGGL((colsum_stage1_kernel<T, FV>), dim3(gx, splits), dim3(128), 0, st, (const T*)x, (float*)ws,
                           rows, (int)cols, xs, rps);
    else
        hipLaunchKernelGGL((colsum_stage1_kernel<T, 1>), dim3(gx, splits), dim3(128), 0, st, (const T*)x, (float*)ws,
                           rows, (int)cols, xs, rps);
    PTJ_CHECK_LAUNCH();
    if (splits <= 8) {
        int64_t blocks = (cols + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL((colsum_stage2_few_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st, (const float*)ws, splits,
                           (int)cols, (T*)out);
    } else {
        hipLaunchKernelGGL((colsum_stage2_kernel<T>), dim3((unsigned)((cols + 31) / 32)), dim3(RED_THREADS), 0, st,
                           (const float*)ws, splits, (int)cols, (T*)out);
    }
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

template <typename T>
int gelu_impl(const void* dy, const void* x, void* out, int64_t n, bool bwd, hipStream_t st);

// Rows per workgroup of the fused GELU backward: two workgroups per CU, at most 512 partial
// rows.
inline void gelu_bwd_colsum_geometry(int64_t rows, int64_t max_splits, int* splits, int* rps) {
    int64_t s = (rows + 31) / 32;
    if (s > 512) s = 512;
    if (s > max_splits) s = max_splits;   // the partials must fit the caller's workspace
    if (s < 1) s = 1;
    *rps = (int)((rows + s - 1) / s);
    *splits = (int)((rows + *rps - 1) / *rps);
}

template <typename T>
int gelu_bwd_colsum_impl(const void* dy, const void* x, void* dx, void* colsum, void* ws, size_t ws_bytes, int64_t rows,
                         int64_t cols, hipStream_t st) {
    constexpr int FV = VecOf<T>::N;
    const bool vok = (cols % FV == 0) && ptj_aligned16(x) && ptj_aligned16(dy) && ptj_aligned16(dx);
    int splits, rps;
    if (!ws || ws_bytes < (size_t)cols * sizeof(float))
        return ptj_set_error(PTJ_ERR_WORKSPACE, "gelu_bwd_colsum: workspace %zu < %zu bytes", ws_bytes,
                             (size_t)cols * sizeof(float));
    gelu_bwd_colsum_geometry(rows, (int64_t)(ws_bytes / ((size_t)cols * sizeof(float))), &splits, &rps);
    const int64_t nvec = vok ? cols / FV : cols;
    // threads per row: a multiple of 64 that covers the row in one, two or four sweeps
    const int nv = nvec <= 512 ? 1 : nvec <= 1024 ? 2 : 4;
    const int tpr = (int)(((nvec + nv - 1) / nv + 63) / 64 * 64);
    if (tpr > 512) {
        // wider rows: separate passes
        int rc = gelu_impl<T>(dy, x, dx, rows * cols, true, st);
        if (rc != PTJ_OK) return rc;
        return colsum_impl<T>(dx, colsum, ws, ws_bytes, rows, cols, cols, st);
    }
    // row slots per workgroup: up to 1024 threads, as long as a row fits the fold buffer
    int slots = 1024 / tpr;
    if (slots > 4) slots = 4;
    if (cols > GELU_CS_MAX_LDS_COLS || slots < 1) slots = 1;
    const int threads = tpr * slots;
#define LAUNCH(V_, NV_)                                                                                          \
    hipLaunchKernelGGL((gelu_bwd_colsum_kernel<T, V_, NV_>), dim3(splits), dim3(threads), 0, st, (const T*)dy,   \
                       (const T*)x, (T*)dx, (float*)ws, rows, (int)cols, rps, tpr)
    if (vok) {
        if (nv == 1) LAUNCH(FV, 1);
        else if (nv == 2) LAUNCH(FV, 2);
        else LAUNCH(FV, 4);
    } else {
        if (nv == 1) LAUNCH(1, 1);
        else if (nv == 2) LAUNCH(1, 2);
        else LAUNCH(1, 4);
    }
#undef LAUNCH
    PTJ_CHECK_LAUNCH();
    hipLaunchKernelGGL((colsum_stage2_kernel<T>), dim3((unsigned)((cols + 31) / 32)), dim3(RED_THREADS), 0, st,
                       (const float*)ws, splits, (int)cols, (T*)colsum);
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

// ---------------------------------------------------------------------------------
// Dispatch helpers
// ---------------------------------------------------------------------------------
struct RowCfg {
    int vec;   // VEC or 1
    int tpr;   // 64, 256, 1024
    int iters64;  // ITERS of the 64-thread row group: 1, 2 or 4
};

// Picks the smallest row-group that holds `cols` elements in registers.
// ITERS per TPR: 64 -> 1, 2 or 4 (the smallest that covers the row), 256 -> 4, 1024 -> 8.
inline bool pick_row_cfg(int64_t cols, int full_vec, bool vec_ok, RowCfg* cfg) {
    const int vec = vec_ok ? full_vec : 1;
    const int64_t nvec = cols / vec;
    cfg->vec = vec;
    cfg->iters64 = nvec <= 64 ? 1 : nvec <= 128 ? 2 : 4;
    if (nvec <= 64 * 4) cfg->tpr = 64;
    else if (nvec <= 256 * 4) cfg->tpr = 256;
    else if (nvec <= 1024 * 8) cfg->tpr = 1024;
    else return false;
    return true;
}

inline int row_grid(int64_t rows, int tpr) {
    const int rpb = tpr == 64 ? 4 : 1;
    const int64_t need = (rows + rpb - 1) / rpb;
    const int64_t cap = (int64_t)ptj_num_cus() * 8;  // 8 workgroups per CU
    return (int)(need < cap ? need : cap);
}

#define ROW_DISPATCH(T, cfg, LAUNCH)                                     \
    do {                                                                 \
        constexpr int FV = VecOf<T>::N;                                  \
        if (cfg.vec == 1) {                                              \
            if (cfg.tpr == 64) {                                         \
                if (cfg.iters64 == 1) { LAUNCH(T, 1, 64, 1); }           \
                else if (cfg.iters64 == 2) { LAUNCH(T, 1, 64, 2); }      \
                else { LAUNCH(T, 1, 64, 4); }                            \
            }                                                            \
            else if (cfg.tpr == 256) { LAUNCH(T, 1, 256, 4); }           \
            else { LAUNCH(T, 1, 1024, 8); }                              \
        } else {                                                         \
            if (cfg.tpr == 64) {                                         \
                if (cfg.iters64 == 1) { LAUNCH(T, FV, 64, 1); }          \
                else if (cfg.iters64 == 2) { LAUNCH(T, FV, 64, 2); }     \
                else { LAUNCH(T, FV, 64, 4); }                           \
            }                                                            \
            else if (cfg.tpr == 256) { LAUNCH(T, FV, 256, 4); }          \
            else { LAUNCH(T, FV, 1024, 8); }                             \
        }                                                                \
    } while (0)

template <typename T>
bool rows_vec_ok(int64_t cols, std::initializer_list<const void*> ptrs, std::initializer_list<int64_t> strides) {
    constexpr int FV = VecOf<T>::N;
    if (cols % FV) return false;
    for (const void* p : ptrs)
        if (p && !ptj_aligned16(p)) return false;
    for (int64_t s : strides)
        if (s % FV) return false;
    return true;
}

template <typename T>
int layernorm_fwd_impl(const void* x, const void* gamma, const void* beta, void* y, int64_t rows, int64_t cols,
                       int64_t xs, int64_t ys, hipStream_t st) {
    RowCfg cfg;
    const bool vok = rows_vec_ok<T>(cols, {x, gamma, beta, y}, {xs, ys});
    if (!pick_row_cfg(cols, VecOf<T>::N, vok, &cfg))
        return ptj_set_error(PTJ_ERR_INVALID, "layernorm_fwd: cols=%lld too large for the register-resident row kernel",
                             (long long)cols);
    const int grid = row_grid(rows, cfg.tpr);
#define LAUNCH(T_, V_, TPR_, IT_)                                                                           \
    hipLaunchKernelGGL((layernorm_fwd_kernel<T_, V_, TPR_, IT_>), dim3(grid), dim3(RowGeom<TPR_>::BLOCK), 0, st, \
                       (const T_*)x, (const T_*)gamma, (const T_*)beta, (T_*)y, rows, (int)cols, xs, ys)
    // 2-byte rows of 513..768 columns: three 8-byte vectors per lane keep all 64 lanes busy
    // (the same layout, and so the same summation order, as the fused residual + norm kernel)
    bool launched = false;
    if constexpr (sizeof(T) == 2) {
        if (cfg.vec == 8 && cfg.tpr == 64 && cols > 512 && cols <= 768) {
            LAUNCH(T, 4, 64, 3);
            launched = true;
        }
    }
    if (!launched) ROW_DISPATCH(T, cfg, LAUNCH);
#undef LAUNCH
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

template <typename T>
int dropout_add_layernorm_impl(const void* x, const void* res, const void* gamma, const void* beta, void* y, void* h,
                               void* keep, int64_t rows, int64_t cols, int train, int64_t seed, hipStream_t st) {
    RowCfg cfg;
    const bool vok = rows_vec_ok<T>(cols, {x, res, gamma, beta, y, h}, {});
    if (keep != nullptr && !(vok && VecOf<T>::N == 8))
        return ptj_set_error(PTJ_ERR_INVALID, "dropout_add_layernorm: keep bytes need 2-byte elements, cols %% 8 == 0 and 16-byte aligned rows");
    if (!pick_row_cfg(cols, VecOf<T>::N, vok, &cfg))
        return ptj_set_error(PTJ_ERR_INVALID, "dropout_add_layernorm: cols=%lld too large for the register-resident row kernel",
                             (long long)cols);
    const int grid = row_grid(rows, cfg.tpr);
#define LAUNCH(T_, V_, TPR_, IT_)                                                                                  \
    hipLaunchKernelGGL((dropout_add_layernorm_kernel<T_, V_, TPR_, IT_>), dim3(grid), dim3(RowGeom<TPR_>::BLOCK), 0, st, \
                       (const T_*)x, (const T_*)res, (const T_*)gamma, (const T_*)beta, (T_*)y, (T_*)h, (uint8_t*)keep, \
                       rows, (int)cols, train, (uint64_t)seed)
    // 2-byte rows of 513..768 columns: three 8-byte vectors per lane keep all 64 lanes busy
    bool launched = false;
    if constexpr (sizeof(T) == 2) {
        if (cfg.vec == 8 && cfg.tpr == 64 && cols > 512 && cols <= 768) {
            LAUNCH(T, 4, 64, 3);
            launched = true;
        }
    }
    if (!launched) ROW_DISPATCH(T, cfg, LAUNCH);
#undef LAUNCH
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

// Grid of the backward kernel = number of dgamma/dbeta partials (one per workgroup).
inline int ln_bwd_grid(int64_t rows, int tpr) {
    const int rpb = tpr == 64 ? LnBwdGeom<64>::ROWS_PER_BLOCK : 1;
    const int64_t need = (rows + rpb - 1) / rpb;
    const int64_t cap = tpr == 64 ? 512 * (512 / LnBwdGeom<64>::BLOCK) : 512;  // bounds the partials
    return (int)(need < cap ? need : cap);
}

template <typename T>
int layernorm_bwd_impl(const void* dy, const void* x, const void* gamma, const void* res, void* dx, void* dgamma,
                       void* dbeta,
                       void* ws, size_t ws_bytes, int64_t rows, int64_t cols, int64_t dys, int64_t xs, int64_t dxs,
                       void* drop, int drop_train, int64_t drop_seed, const void* keep, void* drop_sum, hipStream_t st) {
    RowCfg cfg;
    const bool vok = rows_vec_ok<T>(cols, {dy, x, gamma, dx, res, drop}, {dys, xs, dx ? dxs : 0});
    if (keep != nullptr && !(vok && VecOf<T>::N == 8))
        return ptj_set_error(PTJ_ERR_INVALID, "layernorm_bwd: keep bytes need 2-byte elements and the vector path");
    if (!pick_row_cfg(cols, VecOf<T>::N, vok, &cfg))
        return ptj_set_error(PTJ_ERR_INVALID, "layernorm_bwd: cols=%lld too large", (long long)cols);
    const int grid = ln_bwd_grid(rows, cfg.tpr);
    const int nparts = grid;
    const bool want_dx = dx != nullptr, want_dgb = dgamma != nullptr;
    const int np = drop_sum != nullptr ? 3 : 2;
    // keep bytes are read by the variant with dgamma/dbeta only; elsewhere the mask is recomputed
    const int drop_mode = drop == nullptr ? 0 : (keep != nullptr && want_dgb && drop_train) ? 1 : 2;
    if (drop_sum != nullptr && !(want_dgb && drop != nullptr))
        return ptj_set_error(PTJ_ERR_INVALID, "layernorm_bwd: the column sums of the dropped output need dgamma/dbeta and the dropped output");
    if (want_dgb) {
        const size_t need = (size_t)nparts * np * (size_t)cols * sizeof(float);
        if (!ws || ws_bytes < need)
            return ptj_set_error(PTJ_ERR_WORKSPACE, "layernorm_bwd: workspace %zu < %zu bytes", ws_bytes, need);
    }
#define LAUNCH_F(T_, V_, TPR_, IT_, DX_, DGB_, DROP_)                                                            \
    hipLaunchKernelGGL((layernorm_bwd_kernel<T_, V_, TPR_, IT_, DX_, DGB_, DROP_>), dim3(grid),                  \
                       dim3(LnBwdGeom<TPR_>::BLOCK), 0, st, (const T_*)dy, (const T_*)x, (const T_*)gamma,       \
                       (const T_*)(res ? res : dy), (T_*)dx,                                                     \
                       (float*)ws, rows, (int)cols, dys, xs, dxs, (T_*)drop, drop_train, (uint64_t)drop_seed,    \
                       (const uint8_t*)keep, np, res ? 1 : 0, res ? cols : dys)
#define LAUNCH(T_, V_, TPR_, IT_)                                     \
    do {                                                              \
        if (want_dx && want_dgb) {                                    \
            if (drop_mode == 0) LAUNCH_F(T_, V_, TPR_, IT_, true, true, 0);        \
            else if (drop_mode == 1) LAUNCH_F(T_, V_, TPR_, IT_, true, true, 1);   \
            else LAUNCH_F(T_, V_, TPR_, IT_, true, true, 2);          \
        } else if (want_dx) {                                         \
            if (drop_mode == 0) LAUNCH_F(T_, V_, TPR_, IT_, true, false, 0);       \
            else LAUNCH_F(T_, V_, TPR_, IT_, true, false, 2);         \
        } else LAUNCH_F(T_, V_, TPR_, IT_, false, true, 0);           \
    } while (0)
    // 2-byte rows of 513..768 columns: three 8-byte vectors per lane keep all 64 lanes busy and
    // need a quarter fewer registers than two 16-byte vectors (one more wave per SIMD)
    bool launched = false;
    if constexpr (sizeof(T) == 2) {
        if (cfg.vec == 8 && cfg.tpr == 64 && cols == 768 && want_dx && want_dgb && drop_mode != 2) {
            // whole vectors in every lane: the pipelined kernel (bit-equal to the general one)
#define LAUNCH_X(DROP_)                                                                                           \
    hipLaunchKernelGGL((layernorm_bwd_exact_kernel<T, 4, 3, DROP_>), dim3(grid), dim3(512), 0, st, (const T*)dy,  \
                       (const T*)x, (const T*)gamma, (const T*)(res ? res : dy), (T*)dx, (float*)ws, rows, dys,   \
                       xs, dxs, (T*)drop, drop_train, (const uint8_t*)keep, np, res ? 1 : 0, res ? cols : dys)
            if (drop_mode == 0) LAUNCH_X(0);
            else LAUNCH_X(1);
#undef LAUNCH_X
            launched = true;
        } else if (cfg.vec == 8 && cfg.tpr == 64 && cols > 512 && cols <= 768) {
            LAUNCH(T, 4, 64, 3);
            launched = true;
        }
    }
    if (!launched) ROW_DISPATCH(T, cfg, LAUNCH);
#undef LAUNCH
#undef LAUNCH_F
    PTJ_CHECK_LAUNCH();
    if (want_dgb) {
        hipLaunchKernelGGL((layernorm_bwd_reduce_kernel<T>), dim3((unsigned)((cols + 31) / 32), np), dim3(RED_THREADS), 0, st,
                           (const float*)ws, nparts, (int)cols, (T*)dgamma, (T*)dbeta, (T*)drop_sum);
        PTJ_CHECK_LAUNCH();
    }
    return PTJ_OK;
}

template <typename T>
int log_softmax_fwd_impl(const void* x, void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys, hipStream_t st) {
    RowCfg cfg;
    const bool vok = rows_vec_ok<T>(cols, {x, y}, {xs, ys});
    if (!pick_row_cfg(cols, VecOf<T>::N, vok, &cfg))
        return ptj_set_error(PTJ_ERR_INVALID, "log_softmax_fwd: cols=%lld too large", (long long)cols);
    const int grid = row_grid(rows, cfg.tpr);
#define LAUNCH(T_, V_, TPR_, IT_)                                                                              \
    hipLaunchKernelGGL((log_softmax_fwd_kernel<T_, V_, TPR_, IT_>), dim3(grid), dim3(RowGeom<TPR_>::BLOCK), 0, st, \
                       (const T_*)x, (T_*)y, rows, (int)cols, xs, ys)
    ROW_DISPATCH(T, cfg, LAUNCH);
#undef LAUNCH
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

template <typename T>
int log_softmax_bwd_impl(const void* dy, const void* x, void* dx, int64_t rows, int64_t cols, int64_t dys, int64_t xs,
                         int64_t dxs, hipStream_t st) {
    RowCfg cfg;
    const bool vok = rows_vec_ok<T>(cols, {dy, x, dx}, {dys, xs, dxs});
    if (!pick_row_cfg(cols, VecOf<T>::N, vok, &cfg))
        return ptj_set_error(PTJ_ERR_INVALID, "log_softmax_bwd: cols=%lld too large", (long long)cols);
    const int grid = row_grid(rows, cfg.tpr);
#define LAUNCH(T_, V_, TPR_, IT_)                                                                              \
    hipLaunchKernelGGL((log_softmax_bwd_kernel<T_, V_, TPR_, IT_>), dim3(grid), dim3(RowGeom<TPR_>::BLOCK), 0, st, \
                       (const T_*)dy, (const T_*)x, (T_*)dx, rows, (int)cols, dys, xs, dxs)
    ROW_DISPATCH(T, cfg, LAUNCH);
#undef LAUNCH
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

inline int flat_grid(int64_t nthreads_needed) {
    int64_t b = (nthreads_needed + 255) / 256;
    const int64_t cap = (int64_t)ptj_num_cus() * 16;
    if (b > cap) b = cap;
    if (b < 1) b = 1;
    return (int)b;
}

template <typename T>
int gelu_impl(const void* dy, const void* x, void* out, int64_t n, bool bwd, hipStream_t st) {
    constexpr int FV = VecOf<T>::N;
    const bool vok = (n % FV == 0) && ptj_aligned16(x) && ptj_aligned16(out) && (!dy || ptj_aligned16(dy));
    if (n == 0) return PTJ_OK;
    if (vok) {
        const int64_t nvec = n / FV;
        if (bwd)
            hipLaunchKernelGGL((gelu_bwd_kernel<T, FV>), dim3(flat_grid(nvec)), dim3(256), 0, st, (const T*)dy,
                               (const T*)x, (T*)out, nvec);
        else
            hipLaunchKernelGGL((gelu_fwd_kernel<T, FV>), dim3(flat_grid(nvec)), dim3(256), 0, st, (const T*)x, (T*)out,
                               nvec);
    } else {
        if (bwd)
            hipLaunchKernelGGL((gelu_bwd_kernel<T, 1>), dim3(flat_grid(n)), dim3(256), 0, st, (const T*)dy,
                               (const T*)x, (T*)out, n);
        else
            hipLaunchKernelGGL((gelu_fwd_kernel<T, 1>), dim3(flat_grid(n)), dim3(256), 0, st, (const T*)x, (T*)out, n);
    }
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

template <typename T>
int dropout_impl(const void* x, const void* res, void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys,
                 int train, int64_t seed, hipStream_t st, void* keep_out = nullptr) {
    constexpr int FV = VecOf<T>::N;
    if (rows == 0 || cols == 0) return PTJ_OK;
    const bool vok = (cols % FV == 0) && (xs % FV == 0) && (ys % FV == 0) && ptj_aligned16(x) && ptj_aligned16(y) &&
                     (!res || ptj_aligned16(res));
    if (keep_out != nullptr && !(vok && FV == 8))
        return ptj_set_error(PTJ_ERR_INVALID, "dropout: keep bytes need 2-byte elements, cols %% 8 == 0 and 16-byte aligned rows");
#define LAUNCH(V_, ADD_)                                                                                       \
    hipLaunchKernelGGL((dropout_kernel<T, V_, ADD_>), dim3(flat_grid(rows * (cols / V_))), dim3(256), 0, st,     \
                       (const T*)x, (const T*)res, (T*)y, rows, (int)cols, xs, ys, train, (uint64_t)seed,       \
                       (uint8_t*)keep_out)
    if (vok) {
        if (res) LAUNCH(FV, true); else LAUNCH(FV, false);
    } else {
        if (res) LAUNCH(1, true); else LAUNCH(1, false);
    }
#undef LAUNCH
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

#define DTYPE_SWITCH(dtype, CALL_F32, CALL_BF16)                                  \
    switch (dtype) {                                                              \
        case PTJ_F32: return CALL_F32;                                            \
        case PTJ_BF16: return CALL_BF16;                                          \
        default: return ptj_set_error(PTJ_ERR_INVALID, "%s: unknown dtype %d", __func__, dtype); \
    }

}  // namespace

// ---- ptj_colsum without a caller workspace ---------------------------------------------
// The stage-1 partial sums live in a file-scope device array instead of a buffer the caller
// brings.  Every GPU holds its own copy of the array at its own address, so the address is
// looked up once per device (with that device current) and kept; kernels receive that
// pointer, never the array's name, which in host code is only a stand-in.
static __device__ __align__(256) unsigned char scratch[PTJ_COLSUM_STATIC_SCRATCH_BYTES];
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[PTJ_MAX_DEVICES] = {};

static int colsum_static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return ptj_set_error(PTJ_ERR_LAUNCH, "colsum_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= PTJ_MAX_DEVICES) return ptj_set_error(PTJ_ERR_INVALID, "colsum_static: device index %d", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return ptj_set_error(PTJ_ERR_LAUNCH, "colsum_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return PTJ_OK;
}

extern "C" {

int ptj_layernorm_fwd(const void* x, const void* gamma, const void* beta, void* y, int64_t rows, int64_t cols,
                      int64_t xs, int64_t ys, int dtype, void* stream) {
    PTJ_CHECK_ARG(x && gamma && beta && y, "layernorm_fwd: null pointer");
    PTJ_CHECK_ARG(rows >= 0 && cols >= 2, "layernorm_fwd: need rows >= 0 and cols >= 2 (unbiased std), got %lld x %lld",
                  (long long)rows, (long long)cols);
    PTJ_CHECK_ARG(xs >= cols && ys >= cols, "layernorm_fwd: row stride smaller than cols");
    if (rows == 0) return PTJ_OK;
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (layernorm_fwd_impl<float>(x, gamma, beta, y, rows, cols, xs, ys, st)),
                 (layernorm_fwd_impl<bf16>(x, gamma, beta, y, rows, cols, xs, ys, st)));
}

int ptj_dropout_add_layernorm(const void* x, const void* res, const void* gamma, const void* beta, void* y, void* h,
                              void* keep_bytes, int64_t rows, int64_t cols, int train, int64_t seed, int dtype,
                              void* stream) {
    PTJ_CHECK_ARG(rows >= 0 && cols >= 2, "dropout_add_layernorm: need rows >= 0 and cols >= 2");
    if (rows == 0) return PTJ_OK;
    PTJ_CHECK_ARG(x && res && gamma && beta && y && h, "dropout_add_layernorm: null pointer");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (dropout_add_layernorm_impl<float>(x, res, gamma, beta, y, h, keep_bytes, rows, cols, train, seed, st)),
                 (dropout_add_layernorm_impl<bf16>(x, res, gamma, beta, y, h, keep_bytes, rows, cols, train, seed, st)));
}

size_t ptj_layernorm_bwd_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    // Upper bound over the row configurations the dispatcher can pick.
    return (size_t)(512 * (512 / LnBwdGeom<64>::BLOCK)) * 3 * (size_t)cols * sizeof(float);
}

int ptj_layernorm_bwd_dropout(const void* dy, const void* x, const void* gamma, const void* residual, void* dx,
                              void* dgamma, void* dbeta, void* dropped, void* dropped_colsum, int drop_train, int64_t drop_seed,
                              const void* keep_bytes, void* workspace, size_t workspace_bytes, int64_t rows, int64_t cols, int64_t dys,
                              int64_t xs, int64_t dxs, int dtype, void* stream) {
    PTJ_CHECK_ARG(dy && x, "layernorm_bwd: null dy/x");
    PTJ_CHECK_ARG(dx || dgamma, "layernorm_bwd: nothing to compute (dx and dgamma both null)");
    PTJ_CHECK_ARG(!dx || gamma, "layernorm_bwd: dx requested without gamma");
    PTJ_CHECK_ARG(!residual || dx, "layernorm_bwd: residual given without dx");
    PTJ_CHECK_ARG(!dropped || dx, "layernorm_bwd: dropout output requested without dx");
    PTJ_CHECK_ARG(!dropped_colsum || (dropped && dgamma), "layernorm_bwd: dropped_colsum needs dropped and dgamma/dbeta");
    PTJ_CHECK_ARG((dgamma == nullptr) == (dbeta == nullptr), "layernorm_bwd: dgamma and dbeta must be given together");
    PTJ_CHECK_ARG(rows >= 1 && cols >= 2, "layernorm_bwd: need rows >= 1 and cols >= 2");
    PTJ_CHECK_ARG(dys >= cols && xs >= cols && (!dx || dxs >= cols), "layernorm_bwd: row stride smaller than cols");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype,
                 (layernorm_bwd_impl<float>(dy, x, gamma, residual, dx, dgamma, dbeta, workspace, workspace_bytes, rows, cols,
                                            dys, xs, dxs, dropped, drop_train, drop_seed, keep_bytes, dropped_colsum, st)),
                 (layernorm_bwd_impl<bf16>(dy, x, gamma, residual, dx, dgamma, dbeta, workspace, workspace_bytes, rows, cols, dys,
                                           xs, dxs, dropped, drop_train, drop_seed, keep_bytes, dropped_colsum, st)));
}

int ptj_layernorm_bwd(const void* dy, const void* x, const void* gamma, const void* residual, void* dx, void* dgamma,
                      void* dbeta,
                      void* workspace, size_t workspace_bytes, int64_t rows, int64_t cols, int64_t dys, int64_t xs,
                      int64_t dxs, int dtype, void* stream) {
    return ptj_layernorm_bwd_dropout(dy, x, gamma, residual, dx, dgamma, dbeta, nullptr, nullptr, 0, 0, nullptr, workspace, workspace_bytes,
                                     rows, cols, dys, xs, dxs, dtype, stream);
}

size_t ptj_colsum_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    int gx, splits, rps;
    colsum_geometry(rows, cols, 1, &gx, &splits, &rps);   // scalar geometry bounds the vector one
    int gx2, splits2, rps2;
    colsum_geometry(rows, cols, 8, &gx2, &splits2, &rps2);
    int gx3, splits3, rps3;
    colsum_geometry(rows, cols, 4, &gx3, &splits3, &rps3);
    int m = splits > splits2 ? splits : splits2;
    m = m > splits3 ? m : splits3;
    return (size_t)m * cols * sizeof(float);
}

int ptj_colsum(const void* x, void* out, void* workspace, size_t workspace_bytes, int64_t rows, int64_t cols,
               int64_t xs, int dtype, void* stream) {
    PTJ_CHECK_ARG(rows >= 1 && cols >= 1 && cols < (1ll << 31), "colsum: bad shape");
    PTJ_CHECK_ARG(x && out, "colsum: null pointer");
    PTJ_CHECK_ARG(xs >= cols, "colsum: row stride smaller than cols");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (colsum_impl<float>(x, out, workspace, workspace_bytes, rows, cols, xs, st)),
                 (colsum_impl<bf16>(x, out, workspace, workspace_bytes, rows, cols, xs, st)));
}

int ptj_init(void) {
    // per-device state that entry points otherwise look up on their first call: the address of
    // the built-in scratch array and the CU count
    void* ws = nullptr;
    const int rc = colsum_static_scratch(&ws);
    if (rc != PTJ_OK) return rc;
    (void)ptj_num_cus();
    return PTJ_OK;
}

int ptj_colsum_static(const void* x, void* out, int64_t rows, int64_t cols, int64_t xs, int dtype, void* stream) {
    PTJ_CHECK_ARG(rows >= 1 && cols >= 1 && cols < (1ll << 31), "colsum_static: bad shape");
    PTJ_CHECK_ARG(x && out, "colsum_static: null pointer");
    PTJ_CHECK_ARG(xs >= cols, "colsum_static: row stride smaller than cols");
    const size_t need = ptj_colsum_workspace_bytes(rows, cols);
    PTJ_CHECK_ARG(need <= (size_t)PTJ_COLSUM_STATIC_SCRATCH_BYTES,
                  "colsum_static: [%lld, %lld] needs %zu bytes of partial sums, the built-in scratch holds %zu; "
                  "use ptj_colsum with a workspace", (long long)rows, (long long)cols, need,
                  (size_t)PTJ_COLSUM_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    const int rc = colsum_static_scratch(&ws);
    if (rc != PTJ_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    // every partial that stage 2 reads is written by stage 1 of the same call: nothing in the
    // scratch needs clearing between calls
    DTYPE_SWITCH(dtype, (colsum_impl<float>(x, out, ws, need, rows, cols, xs, st)),
                 (colsum_impl<bf16>(x, out, ws, need, rows, cols, xs, st)));
}

int ptj_gelu_fwd(const void* x, void* y, int64_t n, int dtype, void* stream) {
    PTJ_CHECK_ARG(n >= 0 && (n == 0 || (x && y)), "gelu_fwd: bad arguments");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (gelu_impl<float>(nullptr, x, y, n, false, st)), (gelu_impl<bf16>(nullptr, x, y, n, false, st)));
}

int ptj_gelu_bwd(const void* dy, const void* x, void* dx, int64_t n, int dtype, void* stream) {
    PTJ_CHECK_ARG(n >= 0 && (n == 0 || (dy && x && dx)), "gelu_bwd: bad arguments");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (gelu_impl<float>(dy, x, dx, n, true, st)), (gelu_impl<bf16>(dy, x, dx, n, true, st)));
}

int ptj_gelu_bwd_colsum(const void* dy, const void* x, void* dx, void* colsum, void* workspace, size_t workspace_bytes,
                        int64_t rows, int64_t cols, int dtype, void* stream) {
    PTJ_CHECK_ARG(rows >= 1 && cols >= 1 && cols < (1ll << 31), "gelu_bwd_colsum: bad shape");
    PTJ_CHECK_ARG(dy && x && dx && colsum, "gelu_bwd_colsum: null pointer");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (gelu_bwd_colsum_impl<float>(dy, x, dx, colsum, workspace, workspace_bytes, rows, cols, st)),
                 (gelu_bwd_colsum_impl<bf16>(dy, x, dx, colsum, workspace, workspace_bytes, rows, cols, st)));
}

int ptj_dropout(const void* x, void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys, int train, int64_t seed,
                int dtype, void* stream) {
    PTJ_CHECK_ARG(rows >= 0 && cols >= 0, "dropout: negative shape");
    PTJ_CHECK_ARG(rows * cols == 0 || (x && y), "dropout: null pointer");
    PTJ_CHECK_ARG(xs >= cols && ys >= cols, "dropout: row stride smaller than cols");
    PTJ_CHECK_ARG(cols < (1ll << 31), "dropout: cols must fit in 31 bits");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (dropout_impl<float>(x, nullptr, y, rows, cols, xs, ys, train, seed, st)),
                 (dropout_impl<bf16>(x, nullptr, y, rows, cols, xs, ys, train, seed, st)));
}

int ptj_dropout_add(const void* x, const void* res, void* y, int64_t rows, int64_t cols, int train, int64_t seed,
                    int dtype, void* stream) {
    PTJ_CHECK_ARG(rows >= 0 && cols >= 0, "dropout_add: negative shape");
    PTJ_CHECK_ARG(rows * cols == 0 || (x && res && y), "dropout_add: null pointer");
    PTJ_CHECK_ARG(cols < (1ll << 31), "dropout_add: cols must fit in 31 bits");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (dropout_impl<float>(x, res, y, rows, cols, cols, cols, train, seed, st)),
                 (dropout_impl<bf16>(x, res, y, rows, cols, cols, cols, train, seed, st)));
}

int ptj_dropout_add_keep(const void* x, const void* res, void* y, void* keep_bytes, int64_t rows, int64_t cols,
                         int train, int64_t seed, int dtype, void* stream) {
    PTJ_CHECK_ARG(rows >= 0 && cols >= 0, "dropout_add_keep: negative shape");
    PTJ_CHECK_ARG(rows * cols == 0 || (x && res && y && keep_bytes), "dropout_add_keep: null pointer");
    PTJ_CHECK_ARG(cols < (1ll << 31), "dropout_add_keep: cols must fit in 31 bits");
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (dropout_impl<float>(x, res, y, rows, cols, cols, cols, train, seed, st, keep_bytes)),
                 (dropout_impl<bf16>(x, res, y, rows, cols, cols, cols, train, seed, st, keep_bytes)));
}

int ptj_log_softmax_fwd(const void* x, void* y, int64_t rows, int64_t cols, int64_t xs, int64_t ys, int dtype,
                        void* stream) {
    PTJ_CHECK_ARG(rows >= 0 && cols >= 1, "log_softmax_fwd: bad shape");
    PTJ_CHECK_ARG(rows == 0 || (x && y), "log_softmax_fwd: null pointer");
    PTJ_CHECK_ARG(xs >= cols && ys >= cols, "log_softmax_fwd: row stride smaller than cols");
    if (rows == 0) return PTJ_OK;
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (log_softmax_fwd_impl<float>(x, y, rows, cols, xs, ys, st)),
                 (log_softmax_fwd_impl<bf16>(x, y, rows, cols, xs, ys, st)));
}

int ptj_log_softmax_bwd(const void* dy, const void* x, void* dx, int64_t rows, int64_t cols, int64_t dys, int64_t xs,
                        int64_t dxs, int dtype, void* stream) {
    PTJ_CHECK_ARG(rows >= 0 && cols >= 1, "log_softmax_bwd: bad shape");
    PTJ_CHECK_ARG(rows == 0 || (dy && x && dx), "log_softmax_bwd: null pointer");
    PTJ_CHECK_ARG(dys >= cols && xs >= cols && dxs >= cols, "log_softmax_bwd: row stride smaller than cols");
    if (rows == 0) return PTJ_OK;
    hipStream_t st = (hipStream_t)stream;
    DTYPE_SWITCH(dtype, (log_softmax_bwd_impl<float>(dy, x, dx, rows, cols, dys, xs, dxs, st)),
                 (log_softmax_bwd_impl<bf16>(dy, x, dx, rows, cols, dys, xs, dxs, st)));
}

}  // extern "C"
