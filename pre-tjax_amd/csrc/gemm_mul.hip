// ptj_gemm_mul_colsum: the GEMM whose epilogue multiplies by a same-shaped tensor and sums the columns of what it
// stores (kernels and launch logic in gemm_core.h), the second stage of those sums, and the two-pass form
// for operand layouts that the GEMM reads element by element.
#include "gemm_core.h"

namespace {

// Second stage of the MUL epilogue: out[col] = sum over the 64-row blocks of colpart[block][col].  A
// workgroup owns 64 columns; its four wavefronts take the blocks b = w, w + 4, ... (independent,
// coalesced loads, eight in flight) and their sums are combined in wavefront order: the order of
// the additions is fixed.
template <typename T>
__global__ __launch_bounds__(256) void gemm_colpart_reduce_kernel(const float* __restrict__ colpart, int blocks, int m,
                                                                   T* __restrict__ out) {
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int col = blockIdx.x * 64 + lane;
    float s = 0.f;
    if (col < m) {
        int b = w;
        for (; b + 28 < blocks; b += 32) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = colpart[(int64_t)(b + 4 * u) * m + col];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; b < blocks; b += 4) s += colpart[(int64_t)b * m + col];
    }
    part[w][lane] = s;
    __syncthreads();
    if (w == 0 && col < m) out[col] = from_f32<T>((part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]));
}

// The multiplying epilogue as a pass of its own, for operand layouts the GEMM reads element by
// element: C = round(C * mul) in place and the column sums of the result per block of 64 rows.
// One thread per column of a row block.
template <typename T>
__global__ __launch_bounds__(256) void gemm_mul_colpart_kernel(T* __restrict__ c, int64_t c_rs, const T* __restrict__ mul,
                                                                int64_t mul_rs, int n, int m, float* __restrict__ colpart) {
    const int col = blockIdx.x * 256 + threadIdx.x;
    const int rb = blockIdx.y;
    if (col >= m) return;
    const int r1 = (rb + 1) * 64 < n ? (rb + 1) * 64 : n;
    float s = 0.f;
    for (int r = rb * 64; r < r1; ++r) {
        const T v = from_f32<T>(to_f32(c[(int64_t)r * c_rs + col]) * to_f32(mul[(int64_t)r * mul_rs + col]));
        c[(int64_t)r * c_rs + col] = v;
        s += to_f32(v);
    }
    colpart[(int64_t)rb * m + col] = s;
}

}  // namespace

extern "C" {

size_t ptj_gemm_mul_colsum_workspace_bytes(int64_t n, int64_t m) {
    if (n <= 0 || m <= 0) return 0;
    return (size_t)((n + 63) / 64) * (size_t)m * sizeof(float);
}

int ptj_gemm_mul_colsum(const void* a, const void* b, const void* mul, void* c, void* colsum, int64_t n, int64_t m,
                        int64_t k, int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t mul_rs, int64_t c_rs,
                        void* workspace, size_t workspace_bytes, int dtype, void* stream) {
    PTJ_CHECK_ARG(n >= 0 && m >= 0 && k >= 0, "gemm_mul_colsum: negative dimension");
    PTJ_CHECK_ARG(n < (1ll << 31) && m < (1ll << 31) && k < (1ll << 31), "gemm_mul_colsum: dimension exceeds 31 bits");
    PTJ_CHECK_ARG(dtype == PTJ_F32 || dtype == PTJ_BF16, "gemm_mul_colsum: unknown dtype %d", dtype);
    if (m == 0) return PTJ_OK;
    PTJ_CHECK_ARG(colsum, "gemm_mul_colsum: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const size_t need = ptj_gemm_mul_colsum_workspace_bytes(n, m);
    if (n > 0) {
        PTJ_CHECK_ARG(c && mul && (k == 0 || (a && b)), "gemm_mul_colsum: null pointer");
        PTJ_CHECK_ARG(c_rs >= m && mul_rs >= m, "gemm_mul_colsum: row stride below m %lld", (long long)m);
        if (!workspace || workspace_bytes < need)
            return ptj_set_error(PTJ_ERR_WORKSPACE, "gemm_mul_colsum: workspace %zu < %zu bytes", workspace_bytes, need);
        const int elt = dtype == PTJ_BF16 ? 2 : 4;
        const int bk = BKB / elt;
        GemmArgs g;
        g.a = a; g.b = b; g.c = c; g.bias = nullptr;
        g.n = (int)n; g.m = (int)m; g.k = (int)k;
        g.a_row = a_rs; g.a_k = a_cs;
        g.b_row = b_cs; g.b_k = b_rs;
        g.c_rs = c_rs;
        g.c_aux = nullptr; g.c_aux_rs = 0;
        g.epilogue = PTJ_EPI_NONE;
        g.mul = mul; g.mul_rs = mul_rs; g.colpart = (float*)workspace;
        g.k_per_split = k > 0 ? (int)k : bk;
        g.splits = 1;
        g.tail_first = 0; g.tail_splits = 1; g.tail_kps = 0;
        g.partial = nullptr;
        const int64_t v = 16 / elt;
        g.vec_out = (ptj_aligned16(c) && c_rs % v == 0 && ptj_aligned16(mul) && mul_rs % v == 0 && ptj_aligned16(workspace) &&
                     m % 4 == 0) ? 1 : 0;
        g.stream = (g.vec_out && k >= 2 * bk && k % bk == 0) ? 1 : 0;
        const bool vector_operands =
            dtype == PTJ_F32 ? (pick_mode<float>(a, g.a_row, g.a_k) != GENERIC && pick_mode<float>(b, g.b_row, g.b_k) != GENERIC)
                             : (pick_mode<bf16>(a, g.a_row, g.a_k) != GENERIC && pick_mode<bf16>(b, g.b_row, g.b_k) != GENERIC);
        if (vector_operands) {
            const int rc = dtype == PTJ_F32 ? gemm_impl<float, true>(g, 1, st) : gemm_impl<bf16, true>(g, 1, st);
            if (rc != PTJ_OK) return rc;
        } else {
            // plain product first, then the multiplication and the sums as a pass over C
            const int rc = ptj_gemm(a, b, c, nullptr, n, m, k, a_rs, a_cs, b_rs, b_cs, c_rs, PTJ_EPI_NONE, nullptr, 0, nullptr, 0,
                                    dtype, stream);
            if (rc != PTJ_OK) return rc;
            const dim3 grid2((unsigned)((m + 255) / 256), (unsigned)((n + 63) / 64));
            if (dtype == PTJ_F32)
                hipLaunchKernelGGL((gemm_mul_colpart_kernel<float>), grid2, dim3(256), 0, st, (float*)c, c_rs, (const float*)mul,
                                   mul_rs, (int)n, (int)m, (float*)workspace);
            else
                hipLaunchKernelGGL((gemm_mul_colpart_kernel<bf16>), grid2, dim3(256), 0, st, (bf16*)c, c_rs, (const bf16*)mul,
                                   mul_rs, (int)n, (int)m, (float*)workspace);
            PTJ_CHECK_LAUNCH();
        }
    }
    const int blocks = (int)((n + 63) / 64);
    const dim3 grid((unsigned)((m + 63) / 64));
    if (dtype == PTJ_F32)
        hipLaunchKernelGGL((gemm_colpart_reduce_kernel<float>), grid, dim3(256), 0, st, (const float*)workspace, blocks,
                           (int)m, (float*)colsum);
    else
        hipLaunchKernelGGL((gemm_colpart_reduce_kernel<bf16>), grid, dim3(256), 0, st, (const float*)workspace, blocks,
                           (int)m, (bf16*)colsum);
    PTJ_CHECK_LAUNCH();
    return PTJ_OK;
}

}  // extern "C"
