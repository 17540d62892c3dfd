// Fused log-softmax + mean cross-entropy, forward and backward in one pass over the
// logits: each row (vocabulary-wide, e.g. 50257) is read from HBM once into the
// registers of a 1024-thread workgroup, reduced (max, sum-exp), and the gradient row
// is written once.  Rows are not 16-byte aligned when the vocabulary size is odd, so
// vectors are taken relative to the aligned address below the row start and the two
// boundary vectors of a row are masked element-wise.
#include "common.h"

namespace {

constexpr int CE_THREADS = 1024;
constexpr float CE_LOG2E = 1.4426950408889634f;

typedef uint32_t ce_u32x4 __attribute__((ext_vector_type(4)));

// Asynchronous copy of 16 bytes per lane from global memory straight into LDS: lane l of a
// wavefront lands at lds_wave_base + 16*l (the destination is wave-uniform by construction).
__device__ __forceinline__ void ce_load_to_lds(const void* gsrc, void* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

// Waits until the asynchronous row copies of this wavefront have landed while up to `younger`
// vector stores that were issued AFTER them may still be in flight (vector memory operations
// of one wavefront complete in issue order, so "all but the newest N" covers the copies).
// `younger` is wave-uniform; anything outside 0..8 waits for everything.
// The count is exact only while every gradient vector of a row is ONE store instruction
// (ce_exact_store_count says for which wavefronts that is so); a count that is too high would read
// a landing area that has not filled yet.  CE_RELAXED_ROW_WAIT = false takes that assumption out
// (every wait then drains the stores too): measured 0.79 against 0.76 ms for the 16384 x 50257 pass.
// The parity tests against the CPU oracle and against the plain pass run with the relaxed wait.
constexpr bool CE_RELAXED_ROW_WAIT = true;
__device__ __forceinline__ void ce_wait_row_landed(int younger) {
    if (!CE_RELAXED_ROW_WAIT) younger = -1;
    switch (younger) {
        case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
        case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
        case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
        case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
        case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
        case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
}
// Number of gradient-row stores a wavefront issues per row after it has requested the next
// row's copies, when that number is known exactly: whole 16-byte vectors only (the wavefront
// holds neither end of the row, whose vectors are stored element by element) and no other
// store (wavefront 0 also writes the row's loss and argmax).  Otherwise -1.
template <int ITERS>
__device__ __forceinline__ int ce_exact_store_count(int nvec, int mis, int cols, int vec) {
    const int wbase = __builtin_amdgcn_readfirstlane((int)threadIdx.x & ~63);
    if (wbase == 0) return -1;
    int n = 0;
    bool exact = true;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v0 = wbase + it * CE_THREADS;
        if (v0 < nvec) ++n;
        // the last vector of the row is partial unless the row ends on a vector boundary
        if (v0 <= nvec - 1 && nvec - 1 < v0 + 64 && (cols + mis) % vec != 0) exact = false;
    }
    return exact ? n : -1;
}

__global__ __launch_bounds__(1024) void ce_count_kernel(const int64_t* __restrict__ labels, int64_t rows,
                                                         int64_t* __restrict__ count) {
    __shared__ int sm[16];
    int c = 0;
    for (int64_t i = threadIdx.x; i < rows; i += 1024) c += labels[i] != 0;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t t = 0;
        for (int i = 0; i < 16; ++i) t += sm[i];
        *count = t;
    }
}

// Writes one vector of the gradient row: subtracts 1/count at the label column (label < 0:
// dead row) and stores, element-wise where the vector crosses a row boundary.  A plain
// function rather than a closure so that `g` stays in registers.
template <typename T>
__device__ __forceinline__ void ce_emit(float (&g)[VecOf<T>::N], int vi, int mis, int cols, int64_t label,
                                        float inv_cnt, T* __restrict__ db, T* __restrict__ dr) {
    constexpr int VEC = VecOf<T>::N;
    const int e0 = vi * VEC - mis;
    const int64_t lj = label - e0;
    if (label >= 0 && lj >= 0 && lj < VEC) {   // the one vector of the row that holds the label column
#pragma unroll
        for (int j = 0; j < VEC; ++j) g[j] -= lj == j ? inv_cnt : 0.f;
    }
    if (e0 >= 0 && e0 + VEC <= cols) {
        store_vec<T, VEC>(db + (int64_t)vi * VEC, g);
    } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const int e = e0 + j;
            if (e >= 0 && e < cols) dr[e] = from_f32<T>(g[j]);
        }
    }
}

// Issues the asynchronous copies of row `xr_` (cols elements) into the landing area:
// thread t owns slots t, t + CE_THREADS, ...; threads past the row re-read its last vector.
template <typename T, int ITERS>
__device__ __forceinline__ void ce_issue_row(const T* xr_, int cols, int t, char* land) {
    constexpr int VEC = VecOf<T>::N;
    const int mis_ = (int)((reinterpret_cast<uintptr_t>(xr_) & 15) / sizeof(T));
    const T* xb_ = xr_ - mis_;
    const int nvec_ = (cols + mis_ + VEC - 1) / VEC;
    const char* gb = reinterpret_cast<const char*>(xb_);
    // a rolled loop on purpose: unrolled, the eight 64-bit addresses are hoisted out of the
    // row loop and spilled
#pragma unroll 1
    for (int it = 0; it < ITERS; ++it) {
        const int vi = t + it * CE_THREADS;
        const uint32_t vc = (uint32_t)(vi < nvec_ ? vi : nvec_ - 1);
        ce_load_to_lds(gb + vc * 16u, land + ((t & ~63) + it * CE_THREADS) * 16);
    }
}

// CACHED: the row is kept in registers (ITERS vectors per thread).  Otherwise the
// row is streamed from memory three times (max, sum, gradient).
template <typename T, int ITERS, bool CACHED>
__global__ __launch_bounds__(1024) void ce_row_kernel(const int64_t* __restrict__ labels, const T* logits,
                                                       T* dlogits, float* __restrict__ row_loss,
                                                       int64_t* __restrict__ pred,
                                                       const int64_t* __restrict__ count, int64_t rows, int cols,
                                                       int64_t xs, int64_t dxs) {
    constexpr int VEC = VecOf<T>::N;
    // 2-byte rows are fetched with asynchronous global->LDS copies: every vector of the row
    // is in flight at once at no register cost, a thread reads back only the slots it
    // filled itself (no barrier), and the next row's copies are issued as soon as this
    // row sits in registers, so they overlap the reductions and the gradient stores.
    constexpr bool LAND = CACHED && sizeof(T) == 2;
    __shared__ __attribute__((aligned(16))) char land[LAND ? CE_THREADS * ITERS * 16 : 16];
    __shared__ float smem[16];
    __shared__ int s_best;
    __shared__ float s_xy;
    const float inv_cnt = 1.0f / (float)(*count);
    int younger_stores = -1;
    if constexpr (LAND) {
        // exact only when every row has the same 16-byte phase (row pitches multiples of a vector)
        if (xs % VEC == 0 && dxs % VEC == 0) {
            const int mis0 = (int)((reinterpret_cast<uintptr_t>(logits) & 15) / sizeof(T));
            younger_stores = ce_exact_store_count<ITERS>((cols + mis0 + VEC - 1) / VEC, mis0, cols, VEC);
        }
        if ((int64_t)blockIdx.x < rows) ce_issue_row<T, ITERS>(logits + (int64_t)blockIdx.x * xs, cols, threadIdx.x, land);
    }
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const int t = threadIdx.x;
        const T* xr = logits + row * xs;
        T* dr = dlogits + row * dxs;
        const int mis = (int)((reinterpret_cast<uintptr_t>(xr) & 15) / sizeof(T));
        const T* xb = xr - mis;  // 16-byte aligned
        T* db = dr - mis;        // 16-byte aligned too (checked on the host)
        const int nvec = (cols + mis + VEC - 1) / VEC;
        const int64_t label = labels[row];
        if (t == 0 && label != 0) s_xy = to_f32(xr[label]);  // read before any in-place write
        if (t == 0) s_best = 0x7fffffff;   // ordered before this row's candidates by the max reduction's barrier

        float v[ITERS][VEC];
        float m = -INFINITY;
        if constexpr (LAND) {
            // this row's copies have landed; the previous row's gradient stores, issued after
            // the copies were requested, need not have
            ce_wait_row_landed(row == (int64_t)blockIdx.x ? -1 : younger_stores);
            // thread index behind an opaque barrier: the slot offsets are recomputed here
            // instead of being hoisted out of the row loop and spilled
            int tr = t;
            asm volatile("" : "+v"(tr));
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int vi = tr + it * CE_THREADS;
                ce_u32x4 raw = *reinterpret_cast<const ce_u32x4*>(land + vi * 16);
                // only the vectors that cross the ends of the row (and the slots past it) have
                // positions outside it: those get -inf, in storage form, before widening
                if (vi == 0 || vi >= nvec - 1) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        const int e = vi * VEC + j - mis;
                        if (e < 0 || e >= cols)
                            raw[j >> 1] = (j & 1) ? ((raw[j >> 1] & 0x0000ffffu) | 0xff800000u)
                                                  : ((raw[j >> 1] & 0xffff0000u) | 0x0000ff80u);
                    }
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    v[it][j] = __uint_as_float((j & 1) ? (raw[j >> 1] & 0xffff0000u) : (raw[j >> 1] << 16));
                    m = fmaxf(m, v[it][j]);
                }
                // two LDS reads in flight are enough; more would only cost registers
                if (it & 1) __builtin_amdgcn_sched_barrier(0);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // slots are free again
            if (row + gridDim.x < rows) ce_issue_row<T, ITERS>(logits + (row + gridDim.x) * xs, cols, t, land);
        } else if constexpr (CACHED) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int vi = t + it * CE_THREADS;
                if (vi < nvec) {
                    load_vec<T, VEC>(xb + (int64_t)vi * VEC, v[it]);
                    if (vi == 0 || vi == nvec - 1) {   // the two vectors that cross the ends of the row
#pragma unroll
                        for (int j = 0; j < VEC; ++j) {
                            const int e = vi * VEC + j - mis;
                            if (e < 0 || e >= cols) v[it][j] = -INFINITY;
                        }
                    }
#pragma unroll
                    for (int j = 0; j < VEC; ++j) m = fmaxf(m, v[it][j]);
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) v[it][j] = -INFINITY;
                }
            }
        } else {
            for (int vi = t; vi < nvec; vi += CE_THREADS) {
                float w[VEC];
                load_vec<T, VEC>(xb + (int64_t)vi * VEC, w);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const int e = vi * VEC + j - mis;
                    if (e >= 0 && e < cols) m = fmaxf(m, w[j]);
                }
            }
        }
        const float m_own = m;                       // maximum of this thread's elements
        m = row_reduce<CE_THREADS, true>(m, smem);
        if (pred != nullptr) {
            // argmax = lowest column whose logit equals the row maximum
            int best = 0x7fffffff;
            if constexpr (CACHED) {
                // only a thread that holds the maximum searches for its position (typically one
                // thread of the row; the others skip the scan)
                if (m_own == m) {
                    // from the thread's last element down to its first, so the lowest match is the
                    // one that stays: a compare and a select on a constant per element
                    int off = 0x7fffffff;
#pragma unroll
                    for (int it = ITERS - 1; it >= 0; --it)
#pragma unroll
                        for (int j = VEC - 1; j >= 0; --j) off = v[it][j] == m ? it * CE_THREADS * VEC + j : off;
                    if (off != 0x7fffffff) best = off + t * VEC - mis;
                }
            } else {
                for (int vi = t; vi < nvec; vi += CE_THREADS) {
                    float w[VEC];
                    load_vec<T, VEC>(xb + (int64_t)vi * VEC, w);
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        const int e = vi * VEC + j - mis;
                        if (e >= 0 && e < cols && w[j] == m && e < best) best = e;
                    }
                }
            }
            // the few threads that hold the maximum post their lowest column; thread 0 reads the
            // result after the barriers of the sum reduction below
            if (best != 0x7fffffff) atomicMin(&s_best, best);
        }
        float s = 0.f;
        if constexpr (CACHED) {
            // exp(x - m) = 2^(x log2(e) - m log2(e)): one fused multiply-add and the hardware exponential
            const float m2 = m * CE_LOG2E;
#pragma unroll
            for (int it = 0; it < ITERS; ++it)
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    v[it][j] = __builtin_amdgcn_exp2f(fmaf(v[it][j], CE_LOG2E, -m2));
                    s += v[it][j];
                }
        } else {
            for (int vi = t; vi < nvec; vi += CE_THREADS) {
                float w[VEC];
                load_vec<T, VEC>(xb + (int64_t)vi * VEC, w);
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const int e = vi * VEC + j - mis;
                    if (e >= 0 && e < cols) s += __expf(w[j] - m);
                }
            }
        }
        s = row_reduce<CE_THREADS, false>(s, smem);  // contains __syncthreads: s_xy is visible after it
        const bool live = label != 0;
        if (t == 0 && pred != nullptr) pred[row] = s_best;
        if (t == 0) row_loss[row] = live ? -(s_xy - m - logf(s)) : 0.f;
        const float scale = live ? inv_cnt / s : 0.f;

        if constexpr (CACHED) {
            int ts = t;
            asm volatile("" : "+v"(ts));   // as above: keep the store offsets out of the spill area
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int vi = ts + it * CE_THREADS;
                if (vi < nvec) {
                    float g[VEC];
#pragma unroll
                    for (int j = 0; j < VEC; ++j) g[j] = v[it][j] * scale;
                    ce_emit<T>(g, vi, mis, cols, live ? label : -1, inv_cnt, db, dr);
                }
            }
        } else {
            for (int vi = t; vi < nvec; vi += CE_THREADS) {
                float g[VEC];
                load_vec<T, VEC>(xb + (int64_t)vi * VEC, g);
#pragma unroll
                for (int j = 0; j < VEC; ++j) g[j] = __expf(g[j] - m) * scale;
                ce_emit<T>(g, vi, mis, cols, live ? label : -1, inv_cnt, db, dr);
            }
        }
        __syncthreads();  // s_xy is rewritten by thread 0 at the top of the next row
    }
}

// ---- 2-byte logits: the same pass that also sums the gradient's columns -------------------
// ce_row_kernel<bf16, 8, true> plus per-workgroup column sums of the STORED gradient (the
// bias gradient of the layer that produced the logits: what a separate column-sum pass over
// the gradient would return, without reading the gradient again).  A thread owns the same
// 64 columns of every row (all rows share one 16-byte phase: the host checks that the row
// pitches are multiples of 8 elements), so the sums are 64 fp32 registers per thread.  To
// make room for them the row waits in registers in storage type (32 registers instead of
// 64) and is widened on the fly in each of the three sweeps; the exponential is evaluated
// twice.  One workgroup per CU; its sums over the rows it handled go to part[workgroup].
constexpr int CE_CS_MAX_ITERS = 7;   // 16-byte vectors per thread: 7 * 8 column sums + 7 * 4 row registers fit, 8 would spill

__device__ __forceinline__ float ce_bf16_at(const ce_u32x4& raw, int j) {
    return __uint_as_float((j & 1) ? (raw[j >> 1] & 0xffff0000u) : (raw[j >> 1] << 16));
}

template <int ITERS>
__global__ __launch_bounds__(1024) void ce_row_colsum_kernel(const int64_t* __restrict__ labels, const bf16* logits,
                                                              bf16* dlogits, float* __restrict__ row_loss,
                                                              int64_t* __restrict__ pred,
                                                              const int64_t* __restrict__ count, int64_t rows, int cols,
                                                              int64_t xs, int64_t dxs, float* __restrict__ part,
                                                              int pcols, int resume) {
    typedef bf16 T;
    constexpr int VEC = 8;
    __shared__ __attribute__((aligned(16))) char land[CE_THREADS * ITERS * 16];
    __shared__ float smem[16];
    __shared__ int s_best;
    __shared__ float s_xy;
    const float inv_cnt = 1.0f / (float)(*count);
    const int t = threadIdx.x;
    // identical for every row
    const int mis = (int)((reinterpret_cast<uintptr_t>(logits) & 15) / sizeof(T));
    const int nvec = (cols + mis + VEC - 1) / VEC;
    // resume: the rows given continue an earlier call's (same workgroup, same columns): the sums
    // go on from the partial row that call left, so the additions keep the order of one call
    float acc[ITERS][VEC];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int vi = t + it * CE_THREADS;
        f32x4 lo4 = {0.f, 0.f, 0.f, 0.f}, hi4 = {0.f, 0.f, 0.f, 0.f};
        if (resume && vi < nvec) {
            const float* pr0 = part + (int64_t)blockIdx.x * pcols + vi * VEC;
            lo4 = *reinterpret_cast<const f32x4*>(pr0);
            hi4 = *reinterpret_cast<const f32x4*>(pr0 + 4);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) { acc[it][j] = lo4[j]; acc[it][4 + j] = hi4[j]; }
    }
    const int younger_stores = ce_exact_store_count<ITERS>(nvec, mis, cols, VEC);
    if ((int64_t)blockIdx.x < rows) ce_issue_row<T, ITERS>(logits + (int64_t)blockIdx.x * xs, cols, t, land);
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const T* xr = logits + row * xs;
        T* dr = dlogits + row * dxs;
        T* db = dr - mis;        // 16-byte aligned
        const int64_t label = labels[row];
        if (t == 0 && label != 0) s_xy = to_f32(xr[label]);  // read before any in-place write
        if (t == 0) s_best = 0x7fffffff;

        ce_u32x4 raw[ITERS];
        float m = -INFINITY;
        // this row's copies have landed; the previous row's gradient stores, issued after
        // the copies were requested, need not have
        ce_wait_row_landed(row == (int64_t)blockIdx.x ? -1 : younger_stores);
        int tr = t;
        asm volatile("" : "+v"(tr));
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int vi = tr + it * CE_THREADS;
            raw[it] = *reinterpret_cast<const ce_u32x4*>(land + vi * 16);
            // the two vectors that cross the ends of the row (and the slots past it) get -inf
            // in the positions outside the row, once, in storage form
            if (vi == 0 || vi >= nvec - 1) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const int e = vi * VEC + j - mis;
                    if (e < 0 || e >= cols)
                        raw[it][j >> 1] = (j & 1) ? ((raw[it][j >> 1] & 0x0000ffffu) | 0xff800000u)
                                                  : ((raw[it][j >> 1] & 0xffff0000u) | 0x0000ff80u);
                }
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) m = fmaxf(m, ce_bf16_at(raw[it], j));
            if (it & 1) __builtin_amdgcn_sched_barrier(0);
        }
        const float m_own = m;
        m = row_reduce<CE_THREADS, true>(m, smem);
        if (pred != nullptr && m_own == m) {
            // argmax = lowest column whose logit equals the row maximum.  Only a thread that
            // holds the maximum (typically one of the row) searches, and it searches its slots
            // of the landing area -- still this row's, the next row is requested below -- in a
            // rolled loop: scanning the registers would cost this kernel registers it lacks.
            int best = 0x7fffffff;
#pragma unroll 1
            for (int it = ITERS - 1; it >= 0; --it) {
                const int vi = t + it * CE_THREADS;
                const uint16_t* slot = reinterpret_cast<const uint16_t*>(land + vi * 16);
#pragma unroll 1
                for (int j = VEC - 1; j >= 0; --j) {
                    const int e = vi * VEC + j - mis;
                    const float x = __uint_as_float((uint32_t)slot[j] << 16);
                    if (e >= 0 && e < cols && x == m) best = e;
                }
            }
            if (best != 0x7fffffff) atomicMin(&s_best, best);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slots are free again
        if (row + gridDim.x < rows) ce_issue_row<T, ITERS>(logits + (row + gridDim.x) * xs, cols, t, land);
        float s = 0.f;
        const float m2 = m * CE_LOG2E;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            // opaque to the optimiser: the widened values (and, below, the exponentials) are formed
            // again in every sweep instead of being kept, which would not fit the register file
            asm volatile("" : "+v"(raw[it][0]), "+v"(raw[it][1]), "+v"(raw[it][2]), "+v"(raw[it][3]));
#pragma unroll
            for (int j = 0; j < VEC; ++j) s += __builtin_amdgcn_exp2f(fmaf(ce_bf16_at(raw[it], j), CE_LOG2E, -m2));
            __builtin_amdgcn_sched_barrier(0);   // one vector at a time: registers are scarce here
        }
        s = row_reduce<CE_THREADS, false>(s, smem);  // contains __syncthreads: s_xy is visible after it
        const bool live = label != 0;
        if (t == 0 && pred != nullptr) pred[row] = s_best;
        if (t == 0) row_loss[row] = live ? -(s_xy - m - logf(s)) : 0.f;
        const float scale = live ? inv_cnt / s : 0.f;
        const int64_t lab = live ? label : -1;

        int ts = t;
        asm volatile("" : "+v"(ts));
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int vi = ts + it * CE_THREADS;
            if (vi < nvec) {
                float g[VEC];
                asm volatile("" : "+v"(raw[it][0]), "+v"(raw[it][1]), "+v"(raw[it][2]), "+v"(raw[it][3]));
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    g[j] = __builtin_amdgcn_exp2f(fmaf(ce_bf16_at(raw[it], j), CE_LOG2E, -m2)) * scale;
                const int e0 = vi * VEC - mis;
                const int64_t lj = lab - e0;
                if (lj >= 0 && lj < VEC) {   // the vector that holds the label column (one per row)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) g[j] -= lj == j ? inv_cnt : 0.f;
                }
                // storage rounding first: the sums are those of the stored values
#pragma unroll
                for (int j = 0; j < VEC; ++j) g[j] = to_f32(from_f32<T>(g[j]));
                if (e0 >= 0 && e0 + VEC <= cols) {
                    store_vec<T, VEC>(db + (int64_t)vi * VEC, g);
                } else {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        const int e = e0 + j;
                        if (e >= 0 && e < cols) dr[e] = from_f32<T>(g[j]);
                        else g[j] = 0.f;
                    }
                }
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[it][j] += g[j];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();  // s_xy is rewritten by thread 0 at the top of the next row
    }
    // slot (vi, j) is column vi*8 + j - mis; the partial row is stored by slot (pcols slots)
    float* pr = part + (int64_t)blockIdx.x * pcols;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int vi = t + it * CE_THREADS;
        if (vi < nvec) {
            *reinterpret_cast<f32x4*>(pr + vi * VEC) = f32x4{acc[it][0], acc[it][1], acc[it][2], acc[it][3]};
            *reinterpret_cast<f32x4*>(pr + vi * VEC + 4) = f32x4{acc[it][4], acc[it][5], acc[it][6], acc[it][7]};
        }
    }
}

// out[c] = sum over workgroups of part[w][c + mis], in workgroup order (fixed).
__global__ __launch_bounds__(256) void ce_colsum_reduce_kernel(const float* __restrict__ part, int nparts, int pcols,
                                                                int mis, int cols, bf16* __restrict__ out) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    const float* p = part + c + mis;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int w = 0;
    for (; w + 3 < nparts; w += 4) {
        s0 += p[(int64_t)w * pcols];
        s1 += p[(int64_t)(w + 1) * pcols];
        s2 += p[(int64_t)(w + 2) * pcols];
        s3 += p[(int64_t)(w + 3) * pcols];
    }
    for (; w < nparts; ++w) s0 += p[(int64_t)w * pcols];
    out[c] = from_f32<bf16>((s0 + s1) + (s2 + s3));
}

// loss = (sum of row losses in index order) / count.  One workgroup, fixed order.
__global__ __launch_bounds__(1024) void ce_finalize_kernel(const float* __restrict__ row_loss, int64_t rows,
                                                            const int64_t* __restrict__ count,
                                                            float* __restrict__ loss) {
    __shared__ float sm[1024];
    // Each thread sums a contiguous slice so the summation order is fixed.
    const int64_t per = (rows + 1023) / 1024;
    const int64_t b = threadIdx.x * per;
    const int64_t e = b + per < rows ? b + per : rows;
    float s = 0.f;
    for (int64_t i = b; i < e; ++i) s += row_loss[i];
    sm[threadIdx.x] = s;
    __syncthreads();
    for (int o = 512; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) sm[threadIdx.x] += sm[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) *loss = sm[0] / (float)(*count);
}

template <typename T>
int ce_impl(const int64_t* labels, const void* logits, float* loss, int64_t* count, void* dlogits, int64_t* pred,
            void* ws, int64_t rows, int64_t cols, int64_t xs, int64_t dxs, hipStream_t st) {
    constexpr int VEC = VecOf<T>::N;
    constexpr int ITERS = 64 / VEC;  // 64 cached floats per thread
    float* row_loss = (float*)ws;
    hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(1024), 0, st, labels, rows, count);
    PTJ_CHECK_LAUNCH();
    const int64_t two_per_cu = 2 * (int64_t)ptj_num_cus();
    const int grid = (int)(rows < two_per_cu ? rows : two_per_cu);
    const bool cached = (cols + VEC) <= (int64_t)CE_THREADS * ITERS * VEC;
    if (cached)
        hipLaunchKernelGGL((ce_row_kernel<T, ITERS, true>), dim3(grid), dim3(1024), 0, st, labels, (const T*)logits,
                           (T*)dlogits, row_loss, pred, (const int64_t*)count, rows, (int)cols, xs, dxs);
    else
        hipLaunchKernelGGL((ce_row_kernel<T, 1, false>), dim3(grid), dim3(1024), 0, st, labels, (const T*)logits,
                           (T*)dlogits, row_loss, pred, (const int64_t*)count, rows, (int)cols, xs, dxs);
    PTJ_CHECK_LAUNCH();
    hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(1024), 0, st, (const float*)row_loss, rows,
                       (const int64_t*)count, loss);
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

inline int ce_cs_grid() { return ptj_num_cus(); }   // one workgroup per CU (its LDS landing area fills the CU)
inline int ce_cs_pcols(int64_t cols) { return (int)((cols + 8 + 7) / 8 * 8); }

}  // namespace

extern "C" {

size_t ptj_ce_workspace_bytes(int64_t rows) { return rows > 0 ? (size_t)rows * sizeof(float) : 0; }

size_t ptj_ce_colsum_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    return ((size_t)rows * sizeof(float) + 255) / 256 * 256 + (size_t)ce_cs_grid() * ce_cs_pcols(cols) * sizeof(float);
}

int ptj_ce_fwd_bwd_colsum_rows(const int64_t* labels, const void* logits, float* loss, int64_t* count, void* dlogits,
                               int64_t* pred, void* colsum, void* workspace, size_t workspace_bytes, int64_t rows_total,
                               int64_t row0, int64_t rows, int64_t cols, int64_t xs, int64_t dxs, int dtype,
                               void* stream) {
    PTJ_CHECK_ARG(labels && logits && loss && count && dlogits && colsum, "ce_fwd_bwd_colsum: null pointer");
    PTJ_CHECK_ARG(dtype == PTJ_BF16, "ce_fwd_bwd_colsum: 2-byte storage only (dtype %d)", dtype);
    PTJ_CHECK_ARG(rows_total >= 1 && cols >= 1 && cols + 8 <= (int64_t)CE_THREADS * CE_CS_MAX_ITERS * 8,
                  "ce_fwd_bwd_colsum: bad shape %lld x %lld (at most %d columns)", (long long)rows_total, (long long)cols,
                  CE_THREADS * CE_CS_MAX_ITERS * 8 - 8);
    PTJ_CHECK_ARG(xs >= cols && dxs >= cols && xs % 8 == 0 && dxs % 8 == 0,
                  "ce_fwd_bwd_colsum: row pitches must be multiples of 8 elements and at least cols");
    PTJ_CHECK_ARG(((reinterpret_cast<uintptr_t>(logits) ^ reinterpret_cast<uintptr_t>(dlogits)) & 15) == 0,
                  "ce_fwd_bwd_colsum: logits and dlogits must have equal 16-byte misalignment");
    if (!workspace || workspace_bytes < ptj_ce_colsum_workspace_bytes(rows_total, cols))
        return ptj_set_error(PTJ_ERR_WORKSPACE, "ce_fwd_bwd_colsum: workspace %zu < %zu bytes", workspace_bytes,
                             ptj_ce_colsum_workspace_bytes(rows_total, cols));
    // one workgroup per CU over the WHOLE problem: workgroup w owns the rows w, w + grid, ... of it
    const int grid = (int)(rows_total < ce_cs_grid() ? rows_total : ce_cs_grid());
    PTJ_CHECK_ARG(rows >= 1 && row0 >= 0 && row0 + rows <= rows_total && row0 % grid == 0 &&
                      (rows >= grid || row0 + rows == rows_total),
                  "ce_fwd_bwd_colsum: rows [%lld, %lld) of %lld: chunks start at multiples of %d rows", (long long)row0,
                  (long long)(row0 + rows), (long long)rows_total, grid);
    hipStream_t st = (hipStream_t)stream;
    float* row_loss = (float*)workspace;
    float* part = (float*)((char*)workspace + ((size_t)rows_total * sizeof(float) + 255) / 256 * 256);
    const int pcols = ce_cs_pcols(cols);
    const int mis = (int)((reinterpret_cast<uintptr_t>(logits) & 15) / 2);
    if (row0 == 0) {
        hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(1024), 0, st, labels, rows_total, count);
        PTJ_CHECK_LAUNCH();
    }
    const int launch = (int)(rows < grid ? rows : grid);
    const int resume = row0 > 0 ? 1 : 0;
    int64_t* pred_rows = pred ? pred + row0 : nullptr;
    if (cols + 8 <= (int64_t)CE_THREADS * 4 * 8)
        hipLaunchKernelGGL(ce_row_colsum_kernel<4>, dim3(launch), dim3(1024), 0, st, labels + row0, (const bf16*)logits,
                           (bf16*)dlogits, row_loss + row0, pred_rows, (const int64_t*)count, rows, (int)cols, xs, dxs,
                           part, pcols, resume);
    else
        hipLaunchKernelGGL(ce_row_colsum_kernel<CE_CS_MAX_ITERS>, dim3(launch), dim3(1024), 0, st, labels + row0,
                           (const bf16*)logits, (bf16*)dlogits, row_loss + row0, pred_rows, (const int64_t*)count, rows,
                           (int)cols, xs, dxs, part, pcols, resume);
    PTJ_CHECK_LAUNCH();
    if (row0 + rows == rows_total) {
        hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(1024), 0, st, (const float*)row_loss, rows_total,
                           (const int64_t*)count, loss);
        PTJ_CHECK_LAUNCH();
        hipLaunchKernelGGL(ce_colsum_reduce_kernel, dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, st,
                           (const float*)part, grid, pcols, mis, (int)cols, (bf16*)colsum);
        PTJ_CHECK_LAUNCH();
    }
    return PTJ_OK;
}

int ptj_ce_fwd_bwd_colsum(const int64_t* labels, const void* logits, float* loss, int64_t* count, void* dlogits,
                          int64_t* pred, void* colsum, void* workspace, size_t workspace_bytes, int64_t rows,
                          int64_t cols, int64_t xs, int64_t dxs, int dtype, void* stream) {
    return ptj_ce_fwd_bwd_colsum_rows(labels, logits, loss, count, dlogits, pred, colsum, workspace, workspace_bytes, rows,
                                      0, rows, cols, xs, dxs, dtype, stream);
}

int ptj_ce_fwd_bwd(const int64_t* labels, const void* logits, float* loss, int64_t* count, void* dlogits,
                   int64_t* pred, void* workspace, size_t workspace_bytes, int64_t rows, int64_t cols, int64_t xs, int64_t dxs,
                   int dtype, void* stream) {
    PTJ_CHECK_ARG(labels && logits && loss && count && dlogits, "ce_fwd_bwd: null pointer");
    PTJ_CHECK_ARG(rows >= 1 && cols >= 1 && cols < (1ll << 30), "ce_fwd_bwd: bad shape %lld x %lld", (long long)rows,
                  (long long)cols);
    PTJ_CHECK_ARG(xs >= cols && dxs >= cols, "ce_fwd_bwd: row stride smaller than cols");
    if (!workspace || workspace_bytes < ptj_ce_workspace_bytes(rows))
        return ptj_set_error(PTJ_ERR_WORKSPACE, "ce_fwd_bwd: workspace %zu < %zu bytes", workspace_bytes,
                             ptj_ce_workspace_bytes(rows));
    const size_t es = dtype == PTJ_BF16 ? 2 : 4;
    // Every gradient row must share its logits row's offset inside a 16-byte line.
    PTJ_CHECK_ARG(((reinterpret_cast<uintptr_t>(logits) ^ reinterpret_cast<uintptr_t>(dlogits)) & 15) == 0 &&
                      (((xs - dxs) * (int64_t)es) % 16 == 0 || rows == 1),
                  "ce_fwd_bwd: logits and dlogits rows must have equal 16-byte misalignment");
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case PTJ_F32: return ce_impl<float>(labels, logits, loss, count, dlogits, pred, workspace, rows, cols, xs, dxs, st);
        case PTJ_BF16: return ce_impl<bf16>(labels, logits, loss, count, dlogits, pred, workspace, rows, cols, xs, dxs, st);
        default: return ptj_set_error(PTJ_ERR_INVALID, "ce_fwd_bwd: unknown dtype %d", dtype);
    }
}

}  // extern "C"
