// LDS operand panels for the 32x32 MFMA kernels (GEMM and attention).
//
// A panel is [ROWS][128 bytes of the contraction axis] (64 bf16 or 32 fp32 per row), no
// padding; the eight 16-byte chunks of a row are XOR-swizzled by sw(row).  A lane's MFMA
// operand for one contraction chunk (16 bf16 / 8 fp32 values of k, 32 bytes per row) is
// the 16-byte half selected by lane>>5, read with one ds_read_b128.
#pragma once
#include "common.h"

constexpr int BKB = 128;  // bytes of the contraction axis per panel row

enum LoadMode { KMAJOR = 0, MNMAJOR = 1, GENERIC = 2 };

__device__ __forceinline__ int sw(int row) { return (row ^ (row >> 3)) & 7; }

template <typename T> struct Frag;
template <> struct Frag<bf16> { typedef bf16x8 type; };
template <> struct Frag<float> { typedef f32x4 type; };

__device__ __forceinline__ void mma_chunk(f32x16& acc, const bf16x8& a, const bf16x8& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}
__device__ __forceinline__ void mma_chunk(f32x16& acc, const f32x4& a, const f32x4& b) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[j], acc, 0, 0, 0);
}

// ---------------------------------------------------------------------------------
// Operand panel loader (THREADS threads): ROWS rows x BK = BKB/sizeof(T) k-values,
// HBM -> registers -> LDS.  `row` indexes the panel row, `k` the contraction index.
//   KMAJOR : element(row,k) = p[row*s_row + k]       16-byte vectors along k, copied
//   MNMAJOR: element(row,k) = p[k*s_k + row]         16-byte vectors along rows; a thread
//            takes the same row-vector at 4 consecutive k ("quad") and transposes it in
//            registers, so each row receives 4 consecutive k in one 8/16-byte LDS write
//   GENERIC: element(row,k) = p[row*s_row + k*s_k]   scalar loads, any strides/alignment
// Rows >= nrows and k >= kend read as zero.
// ---------------------------------------------------------------------------------
template <typename T, int MODE, int ROWS, int THREADS>
struct TileLoader {
    static constexpr int VEC = VecOf<T>::N;
    static constexpr int BK = BKB / (int)sizeof(T);
    // KMAJOR / GENERIC geometry
    static constexpr int RP = THREADS / 8;          // rows per pass (8 threads cover one 128-byte row)
    static constexpr int NV = (ROWS + RP - 1) / RP; // vectors per thread
    // MNMAJOR geometry: a block = 8 row-vectors x 8 quads = one wave-wide instruction
    static constexpr int JB = ROWS / VEC / 8;       // blocks along rows
    static constexpr int KB = BK / 4 / 8;           // blocks along k (bf16: 2, fp32: 1)
    static constexpr int NBLK = JB * KB;
    static constexpr int NW = THREADS / 64;
    static constexpr int NQ = (NBLK + NW - 1) / NW; // quads per thread
    static_assert(ROWS % (VEC * 8) == 0 && BK % 32 == 0, "panel shape");
    static constexpr int NREG = MODE == MNMAJOR ? NQ * 4 : NV;
    Pack<T, VEC> r[NREG];

    // Interior panels: every vector is fully inside the operand; straight-line 16-byte loads
    // (no predicates, no branches, so all of them stay in flight together).
    __device__ __forceinline__ void load_fast(const T* __restrict__ p, int64_t s_row, int64_t s_k, int row0, int k0,
                                              int tid) {
        static_assert(MODE != GENERIC, "GENERIC panels have no vector path");
        if constexpr (MODE == KMAJOR) {
            const T* base = p + (int64_t)(row0 + (tid >> 3)) * s_row + k0 + (tid & 7) * VEC;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                if (ROWS % RP != 0 && (tid >> 3) + RP * i >= ROWS) break;
                r[i] = *reinterpret_cast<const Pack<T, VEC>*>(base + (int64_t)(RP * i) * s_row);
            }
        } else {
            const int jc_lo = tid & 7, kq_lo = (tid >> 3) & 7, w = tid >> 6;
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi) {
                const int b = w + qi * NW;
                if (NBLK % NW != 0 && b >= NBLK) break;
                const int row = row0 + ((b % JB) * 8 + jc_lo) * VEC;
                const int kq = k0 + ((b / JB) * 8 + kq_lo) * 4;
                const T* base = p + (int64_t)kq * s_k + row;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    r[qi * 4 + i] = *reinterpret_cast<const Pack<T, VEC>*>(base + (int64_t)i * s_k);
            }
        }
    }

    // Edge panels and GENERIC operands: element-wise loads with the address clamped to
    // the operand's first element when out of range (branch-free), zero-filled.
    __device__ __forceinline__ void load_edge(const T* __restrict__ p, int64_t s_row, int64_t s_k, int row0, int nrows,
                                              int k0, int kend, int tid) {
        if constexpr (MODE == KMAJOR || MODE == GENERIC) {
            const int c = tid & 7;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int prow = (tid >> 3) + RP * i;
                if (ROWS % RP != 0 && prow >= ROWS) break;
                const int row = row0 + prow;
                const int k = k0 + c * VEC;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const bool ok = row < nrows && k + e < kend;
                    const T v = p[ok ? (int64_t)row * s_row + (int64_t)(k + e) * s_k : 0];
                    r[i].v[e] = ok ? v : from_f32<T>(0.f);
                }
            }
        } else {
            const int jc_lo = tid & 7, kq_lo = (tid >> 3) & 7, w = tid >> 6;
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi) {
                const int b = w + qi * NW;
                if (NBLK % NW != 0 && b >= NBLK) break;
                const int row = row0 + ((b % JB) * 8 + jc_lo) * VEC;
                const int kq = k0 + ((b / JB) * 8 + kq_lo) * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const bool ok = kq + i < kend && row + e < nrows;
                        const T v = p[ok ? (int64_t)(kq + i) * s_k + row + e : 0];
                        r[qi * 4 + i].v[e] = ok ? v : from_f32<T>(0.f);
                    }
            }
        }
    }

    __device__ __forceinline__ void store(char* __restrict__ lds, int tid) const {
        if constexpr (MODE == KMAJOR || MODE == GENERIC) {
            const int c = tid & 7;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int row = (tid >> 3) + RP * i;
                if (ROWS % RP != 0 && row >= ROWS) break;
                *reinterpret_cast<Pack<T, VEC>*>(lds + row * BKB + ((c ^ sw(row)) << 4)) = r[i];
            }
        } else {
            const int jc_lo = tid & 7, kq_lo = (tid >> 3) & 7, w = tid >> 6;
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi) {
                const int b = w + qi * NW;
                if (NBLK % NW != 0 && b >= NBLK) break;
                const int prow = ((b % JB) * 8 + jc_lo) * VEC;
                const int kb = ((b / JB) * 8 + kq_lo) * 4 * (int)sizeof(T);  // byte offset of the quad in the row
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const int row = prow + e;
                    Pack<T, 4> t;
#pragma unroll
                    for (int i = 0; i < 4; ++i) t.v[i] = r[qi * 4 + i].v[e];
                    *reinterpret_cast<Pack<T, 4>*>(lds + row * BKB + (((kb >> 4) ^ sw(row)) << 4) + (kb & 15)) = t;
                }
            }
        }
    }
};

template <typename T>
__device__ __forceinline__ typename Frag<T>::type read_frag(const char* __restrict__ lds, int row, int q) {
    return *reinterpret_cast<const typename Frag<T>::type*>(lds + row * BKB + ((q ^ sw(row)) << 4));
}

