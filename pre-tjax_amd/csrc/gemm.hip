// ptj_gemm: C = A.B (+bias) (gelu) for every operand layout; kernels and launch logic in gemm_core.h.  The bf16
// kernels are instantiated here, the fp32 ones in gemm_f32.hip (the two compile side by side).
#include "gemm_core.h"

extern "C" {

size_t ptj_gemm_workspace_bytes(int64_t n, int64_t m, int64_t k, int dtype) {
    if (n <= 0 || m <= 0 || k <= 0) return 0;
    const int elt = dtype == PTJ_BF16 ? 2 : 4;
    const int s = choose_splits(n, m, k, elt, (size_t)-1);
    if (s > 1) return (size_t)s * n * m * sizeof(float);
    int first, ts, tkps;
    return choose_tail_split(n, m, k, elt, (size_t)-1, &first, &ts, &tkps);
}

int ptj_gemm(const void* a, const void* b, void* c, const void* bias, int64_t n, int64_t m, int64_t k, int64_t a_rs,
             int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t c_rs, int epilogue, void* c_pre, int64_t c_pre_rs,
             void* workspace, size_t workspace_bytes, int dtype, void* stream) {
    PTJ_CHECK_ARG(n >= 0 && m >= 0 && k >= 0, "gemm: negative dimension");
    PTJ_CHECK_ARG(n < (1ll << 31) && m < (1ll << 31) && k < (1ll << 31), "gemm: dimension exceeds 31 bits");
    PTJ_CHECK_ARG(epilogue >= PTJ_EPI_NONE && epilogue <= PTJ_EPI_ACCUMULATE, "gemm: unknown epilogue %d", epilogue);
    PTJ_CHECK_ARG(epilogue != PTJ_EPI_BIAS_GELU_DERIV || c_pre, "gemm: the derivative epilogue needs its second output");
    PTJ_CHECK_ARG(epilogue == PTJ_EPI_NONE || epilogue == PTJ_EPI_ACCUMULATE || bias, "gemm: epilogue %d needs a bias", epilogue);
    PTJ_CHECK_ARG(epilogue != PTJ_EPI_ACCUMULATE || (!bias && !c_pre && dtype == PTJ_BF16),
                  "gemm: the accumulating epilogue takes no bias and no second output, 2-byte storage only");
    PTJ_CHECK_ARG(dtype == PTJ_F32 || dtype == PTJ_BF16, "gemm: unknown dtype %d", dtype);
    if (n == 0 || m == 0) return PTJ_OK;
    PTJ_CHECK_ARG(c && (k == 0 || (a && b)), "gemm: null pointer");
    PTJ_CHECK_ARG(c_rs >= m, "gemm: c row stride %lld < m %lld", (long long)c_rs, (long long)m);
    PTJ_CHECK_ARG(!c_pre || ((epilogue == PTJ_EPI_BIAS_GELU || epilogue == PTJ_EPI_BIAS_GELU_DERIV) && c_pre_rs >= m),
                  "gemm: c_pre needs a bias+GELU epilogue and a row stride >= m");
    const int elt = dtype == PTJ_BF16 ? 2 : 4;
    const int bk = BKB / elt;
    GemmArgs g;
    g.a = a; g.b = b; g.c = c; g.bias = bias;
    g.n = (int)n; g.m = (int)m; g.k = (int)k;
    g.a_row = a_rs; g.a_k = a_cs;
    g.b_row = b_cs; g.b_k = b_rs;
    g.c_rs = c_rs;
    g.c_aux = c_pre;
    g.c_aux_rs = c_pre_rs;
    g.epilogue = epilogue;
    g.mul = nullptr; g.mul_rs = 0; g.colpart = nullptr;
    if (epilogue == PTJ_EPI_ACCUMULATE) workspace = nullptr;   // no K split: the partial sums would not see the stored C
    int splits = workspace ? choose_splits(n, m, k, elt, workspace_bytes) : 1;
    int64_t kps = k;
    if (splits > 1) {
        kps = ((k + splits - 1) / splits + bk - 1) / bk * bk;
        splits = (int)((k + kps - 1) / kps);
    }
    if (kps < 1) kps = bk;  // k == 0: one empty pass writes bias / zeros
    g.k_per_split = (int)kps;
    g.splits = splits;
    g.tail_first = 0; g.tail_splits = 1; g.tail_kps = 0;
    if (splits == 1 && workspace && ptj_aligned16(workspace))
        choose_tail_split(n, m, k, elt, workspace_bytes, &g.tail_first, &g.tail_splits, &g.tail_kps);
    {
        const int64_t v = 16 / elt;
        bool ok = ptj_aligned16(c) && c_rs % v == 0;
        if (c_pre) ok = ok && ptj_aligned16(c_pre) && c_pre_rs % v == 0;
        if (bias) ok = ok && (reinterpret_cast<uintptr_t>(bias) % (4 * (size_t)elt)) == 0;
        if (splits > 1) ok = ok && ptj_aligned16(workspace) && m % 4 == 0;
        g.vec_out = ok ? 1 : 0;
    }
    g.partial = (splits > 1 || g.tail_splits > 1) ? (float*)workspace : nullptr;
    // streamed tiles need whole, evenly many K panels (the two-step loop body) and vector-aligned outputs
    g.stream = (splits == 1 && g.vec_out && k >= 2 * bk && k % bk == 0) ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    return dtype == PTJ_F32 ? ptj_gemm_detail::launch_plain_f32(g, splits, st) : gemm_impl<bf16>(g, splits, st);
}

}  // extern "C"
