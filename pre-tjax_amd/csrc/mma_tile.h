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

// Depends on row mod 32 only, so the rows of one lane's MFMA operands (32 apart) share a
// swizzle and differ by a constant LDS offset.
__device__ __forceinline__ int sw(int row) { return (row ^ ((row >> 3) & 3)) & 7; }

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
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Sets the raw bits of element e of a 16-byte vector of T (used by the edge path; the
// staging registers are plain 4 x u32 vectors so that they are always promoted to registers).
template <typename T> __device__ __forceinline__ void vec_set(u32x4& v, int e, uint32_t bits) {
    if constexpr (sizeof(T) == 4) v[e] = bits;
    else v[e >> 1] = (e & 1) ? ((v[e >> 1] & 0xffffu) | (bits << 16)) : ((v[e >> 1] & 0xffff0000u) | bits);
}
template <typename T> __device__ __forceinline__ uint32_t elem_bits(const T* p) {
    if constexpr (sizeof(T) == 4) return *reinterpret_cast<const uint32_t*>(p);
    else return *reinterpret_cast<const uint16_t*>(p);
}

// WRAP (MNMAJOR only): when the 8x8 blocks do not divide evenly among the wavefronts, the
// spare wavefronts repeat earlier blocks (same data to the same place) instead of idling,
// which keeps the loader free of branches.
// PAIRQ (MNMAJOR panels of 2-byte elements only): within every 16 positions of the k axis the
// two middle quads trade places (k bits 2 and 3 swapped), so that positions {4g .. 4g+3} and
// {8 + 4g .. 8 + 4g+3} form one 16-byte chunk -- the k order in which a lane holds a 32x32
// accumulator tile, which lets such a tile be multiplied from registers against one
// 16-byte LDS read per MFMA.
template <typename T, int MODE, int ROWS, int THREADS, bool WRAP = false, bool PAIRQ = false>
struct TileLoader {
    static constexpr int VEC = VecOf<T>::N;
    static constexpr int BK = BKB / (int)sizeof(T);
    // KMAJOR / GENERIC geometry
    static constexpr int RP = THREADS / 8;          // rows per pass (8 threads cover one 128-byte row)
    static constexpr int NV = (ROWS + RP - 1) / RP; // vectors per thread
    // MNMAJOR geometry: a block = RB row-vectors x QB quads = one wave-wide instruction.  QB
    // quads span a whole 128-byte panel row (2-byte elements: 16 quads of 8 bytes, 4-byte: 8
    // quads of 16 bytes), so one LDS store instruction writes RB complete rows -- every bank
    // equally often, whatever the swizzle.
    static constexpr int QB = BK / 4;               // quads of one block along k: 16 / 8
    static constexpr int RB = 64 / QB;              // row vectors of one block: 4 / 8
    static constexpr int JB = ROWS / VEC / RB;      // blocks along rows
    static constexpr int KB = 1;                    // blocks along k
    static constexpr int NBLK = JB * KB;
    static constexpr int NW = THREADS / 64;
    static constexpr int NQ = (NBLK + NW - 1) / NW; // quads per thread
    static_assert(ROWS % (VEC * RB) == 0 && BK % 32 == 0, "panel shape");
    static constexpr int NREG = MODE == MNMAJOR ? NQ * 4 : NV;
    u32x4 r[NREG];

    // Interior panels: every vector is fully inside the operand; straight-line 16-byte loads
    // (no predicates, no branches, so all of them stay in flight together).  The address is
    // split into a wave-uniform 64-bit part (scalar registers) and one 32-bit per-lane
    // offset that does not change along K.
    __device__ __forceinline__ void load_fast(const T* __restrict__ p, int64_t s_row, int64_t s_k, int row0, int k0,
                                              int tid) {
        load_fast_slice<0, 1, false>(p, s_row, s_k, row0, k0, tid, 0);
    }

    // Slice I of N of load_fast (every N-th load), so that a caller can spread the loads of
    // one panel between other work.  CLAMP: the panel may extend past the last row of the
    // operand (nrows); rows past it re-read the last valid row / row vector instead, so the
    // loads stay straight-line and in bounds and the caller discards those rows' results.
    template <int I, int N, bool CLAMP>
    __device__ __forceinline__ void load_fast_slice(const T* __restrict__ p, int64_t s_row, int64_t s_k, int row0,
                                                    int k0, int tid, int nrows) {
        static_assert(MODE != GENERIC, "GENERIC panels have no vector path");
        // Byte addressing: wave-uniform 64-bit base + one unsigned 32-bit lane offset.
        if constexpr (MODE == KMAJOR) {
            if constexpr (!CLAMP) {
                const char* ub = reinterpret_cast<const char*>(p + (int64_t)row0 * s_row + k0);   // uniform
                const uint32_t loff = ((uint32_t)(tid >> 3) * (uint32_t)s_row + (tid & 7) * VEC) * (uint32_t)sizeof(T);
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    if (i % N != I) continue;
                    if ((ROWS % RP == 0) || ((tid >> 3) + RP * i < ROWS))
                        r[i] = *reinterpret_cast<const u32x4*>(ub + (int64_t)(RP * i) * s_row * (int64_t)sizeof(T) + loff);
                }
            } else {
                // rows past the operand's last one re-read it; both addresses are a uniform
                // base plus a 32-bit lane offset, so the clamp costs a compare and selects
                const int64_t rstep = s_row * (int64_t)sizeof(T);
                const char* ub = reinterpret_cast<const char*>(p + (int64_t)row0 * s_row + k0);   // uniform
                const int lim = nrows - 1 - row0;
                const char* last = ub + (int64_t)lim * rstep;                                      // uniform
                const uint32_t col = (uint32_t)((tid & 7) * VEC * (int)sizeof(T));
                const uint32_t loff = (uint32_t)(tid >> 3) * (uint32_t)s_row * (uint32_t)sizeof(T) + col;
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    if (i % N != I) continue;
                    if ((ROWS % RP == 0) || ((tid >> 3) + RP * i < ROWS)) {
                        const bool in = (tid >> 3) + RP * i <= lim;
                        const char* a = in ? ub + (int64_t)(RP * i) * rstep + loff : last + col;
                        r[i] = *reinterpret_cast<const u32x4*>(a);
                    }
                }
            }
        } else {
            const int jc_lo = tid & (RB - 1), kq_lo = (tid & 63) / RB, w = tid >> 6;
            const char* ub = reinterpret_cast<const char*>(p + (int64_t)k0 * s_k + (CLAMP ? 0 : row0));   // uniform
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi) {
                const int b = WRAP ? (w + qi * NW) % NBLK : w + qi * NW;
                if (WRAP || (NBLK % NW == 0) || (b < NBLK)) {
                    int rowv = ((b % JB) * RB + jc_lo) * VEC;              // first row of the lane's row vector
                    if constexpr (CLAMP) {
                        const int lastv = ((nrows - 1) / VEC) * VEC;        // a .t() view's pitch covers this vector
                        rowv = row0 + rowv < lastv ? row0 + rowv : lastv;
                    }
                    const uint32_t loff =
                        ((uint32_t)(((b / JB) * QB + kq_lo) * 4) * (uint32_t)s_k + (uint32_t)rowv) * (uint32_t)sizeof(T);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if ((qi * 4 + i) % N != I) continue;
                        r[qi * 4 + i] = *reinterpret_cast<const u32x4*>(ub + (int64_t)i * s_k * (int64_t)sizeof(T) + loff);
                    }
                }
            }
        }
    }

    // Edge panels and GENERIC operands: element-wise loads, zero-filled out of range.
    __device__ __forceinline__ void load_edge(const T* __restrict__ p, int64_t s_row, int64_t s_k, int row0, int nrows,
                                              int k0, int kend, int tid) {
        if constexpr (MODE == KMAJOR || MODE == GENERIC) {
            const int c = tid & 7;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int prow = (tid >> 3) + RP * i;
                const int row = row0 + prow;
                const int k = k0 + c * VEC;
                u32x4 v = {0u, 0u, 0u, 0u};
                if ((ROWS % RP == 0 || prow < ROWS) && row < nrows) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        if (k + e < kend) vec_set<T>(v, e, elem_bits<T>(p + (int64_t)row * s_row + (int64_t)(k + e) * s_k));
                }
                r[i] = v;
            }
        } else {
            const int jc_lo = tid & (RB - 1), kq_lo = (tid & 63) / RB, w = tid >> 6;
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi) {
                const int b = WRAP ? (w + qi * NW) % NBLK : w + qi * NW;
                const int row = row0 + ((b % JB) * RB + jc_lo) * VEC;
                const int kq = k0 + ((b / JB) * QB + kq_lo) * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    u32x4 v = {0u, 0u, 0u, 0u};
                    if ((WRAP || NBLK % NW == 0 || b < NBLK) && kq + i < kend) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            if (row + e < nrows) vec_set<T>(v, e, elem_bits<T>(p + (int64_t)(kq + i) * s_k + row + e));
                    }
                    r[qi * 4 + i] = v;
                }
            }
        }
    }

    __device__ __forceinline__ void store(char* __restrict__ lds, int tid) const { store_slice<0, 1>(lds, tid); }

    // Slice I of N of store (every N-th LDS write).
    template <int I, int N>
    __device__ __forceinline__ void store_slice(char* __restrict__ lds, int tid) const {
        if constexpr (MODE == KMAJOR || MODE == GENERIC) {
            const int c = tid & 7;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                if (i % N != I) continue;
                const int row = (tid >> 3) + RP * i;
                if ((ROWS % RP == 0) || (row < ROWS))
                    *reinterpret_cast<u32x4*>(lds + row * BKB + ((c ^ sw(row)) << 4)) = r[i];
            }
        } else {
            const int jc_lo = tid & (RB - 1), kq_lo = (tid & 63) / RB, w = tid >> 6;
#pragma unroll
            for (int qi = 0; qi < NQ; ++qi) {
                const int b = WRAP ? (w + qi * NW) % NBLK : w + qi * NW;
                if (WRAP || (NBLK % NW == 0) || (b < NBLK)) {
                    const int prow = ((b % JB) * RB + jc_lo) * VEC;
                    int kq = (b / JB) * QB + kq_lo;
                    if constexpr (PAIRQ && sizeof(T) == 2) kq = (kq & ~3) | ((kq & 1) << 1) | ((kq >> 1) & 1);
                    const int kb = kq * 4 * (int)sizeof(T);  // byte offset of the quad in the row
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        if ((qi * VEC + e) % N != I) continue;
                        const int row = prow + e;
                        char* dst = lds + row * BKB + (((kb >> 4) ^ sw(row)) << 4) + (kb & 15);
                        if constexpr (sizeof(T) == 4) {
                            u32x4 t = {r[qi * 4 + 0][e], r[qi * 4 + 1][e], r[qi * 4 + 2][e], r[qi * 4 + 3][e]};
                            *reinterpret_cast<u32x4*>(dst) = t;
                        } else {
                            // element e of two row vectors side by side: one byte permute per dword
                            // (low halves 0x05040100, high halves 0x07060302 of {second, first})
                            const uint32_t SEL = (e & 1) ? 0x07060302u : 0x05040100u;
                            u32x2 t = {__builtin_amdgcn_perm(r[qi * 4 + 1][e >> 1], r[qi * 4 + 0][e >> 1], SEL),
                                       __builtin_amdgcn_perm(r[qi * 4 + 3][e >> 1], r[qi * 4 + 2][e >> 1], SEL)};
                            *reinterpret_cast<u32x2*>(dst) = t;
                        }
                    }
                }
            }
        }
    }
};

template <typename T>
__device__ __forceinline__ typename Frag<T>::type read_frag(const char* __restrict__ lds, int row, int q) {
    return *reinterpret_cast<const typename Frag<T>::type*>(lds + row * BKB + ((q ^ sw(row)) << 4));
}

