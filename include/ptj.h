/*
 * libptj -- C ABI of the MI355X (gfx950) kernel path that replaces the Triton
 * kernels of martin-kukla/pre-tjax (model_triton.py, loss_and_optimizer_triton.py).
 *
 * Conventions shared by every entry point
 *   - plain pointers and sizes only; every pointer is a DEVICE pointer unless said
 *     otherwise; the caller owns all buffers (inputs, outputs, workspaces);
 *   - no entry point allocates, frees or synchronises; work is enqueued on
 *     `stream` (a hipStream_t passed as void*, NULL = the default stream);
 *   - `dtype` selects the storage type of all float tensors of the call
 *     (PTJ_F32 or PTJ_BF16); statistics and accumulators are always fp32;
 *   - strides are in ELEMENTS;
 *   - return value 0 on success, negative PTJ_ERR_* otherwise, in which case
 *     ptj_last_error() (thread local) describes the failure.  Nothing is launched
 *     when an argument check fails.
 * The reference interface each entry point replaces is cited as
 * `model_triton.py:<line>` (kernel / wrapper) relative to the reference tree.
 */
#ifndef PTJ_H
#define PTJ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PTJ_F32 0
#define PTJ_BF16 1

#define PTJ_OK 0
#define PTJ_ERR_INVALID (-1)     /* bad argument / unsupported shape */
#define PTJ_ERR_LAUNCH (-2)      /* HIP reported a launch error */
#define PTJ_ERR_WORKSPACE (-3)   /* workspace too small */

/* GEMM epilogues (ptj_gemm) */
#define PTJ_EPI_NONE 0
#define PTJ_EPI_BIAS 1           /* C = A.B + bias[m]                       */
#define PTJ_EPI_BIAS_GELU 2      /* C = gelu(A.B + bias[m])                 */
#define PTJ_EPI_BIAS_GELU_DERIV 3 /* the same C; c_pre = gelu'(A.B + bias[m]) */
#define PTJ_EPI_ACCUMULATE 4     /* C = C + A.B (C is read, widened, and rounded once more) */

int ptj_version(void);
const char* ptj_last_error(void);
/* Optional, once per GPU with that GPU current: resolves the per-device state that entry points
 * otherwise look up on their first call there (the CU count that sizes the persistent grids, the
 * device address of ptj_colsum_static's built-in scratch array), so that from the first compute
 * call on nothing but kernel launches happens.  No counterpart in the reference. */
int ptj_init(void);

/* ---- row-wise kernels ---------------------------------------------------- */

/* LayerNorm forward: y = gamma*(x-mean)/std_unbiased + beta, no epsilon.
 * Replaces t_layernorm_fwd_k / t_layernorm_fwd_t (model_triton.py:1582-1637). */
int ptj_layernorm_fwd(const void* x, const void* gamma, const void* beta, void* y,
                      int64_t rows, int64_t cols, int64_t x_row_stride, int64_t y_row_stride,
                      int dtype, void* stream);

/* LayerNorm backward.  dx (nullable) replaces t_layernorm_bkwd2_x_k/_t
 * (model_triton.py:1799-1867); dgamma/dbeta (both nullable together) replace
 * t_layernorm_bkwd2_p_k/_t (model_triton.py:1664-1726) with a deterministic
 * two-stage reduction instead of float atomics.  `workspace` must hold
 * ptj_layernorm_bwd_workspace_bytes(rows, cols) bytes when dgamma != NULL
 * (may be NULL otherwise).  gamma may be NULL when dx == NULL.  `residual` (nullable,
 * contiguous [rows, cols]) is added to dx: the `blck_dloss_dx + dloss_dx` of the block
 * backward (model_triton.py:2036, 2190) without a separate pass. */
size_t ptj_layernorm_bwd_workspace_bytes(int64_t rows, int64_t cols);
int ptj_layernorm_bwd(const void* dy, const void* x, const void* gamma, const void* residual,
                      void* dx, void* dgamma, void* dbeta, void* workspace, size_t workspace_bytes,
                      int64_t rows, int64_t cols, int64_t dy_row_stride, int64_t x_row_stride,
                      int64_t dx_row_stride, int dtype, void* stream);

/* ptj_layernorm_bwd with a second output: `dropped` (nullable, contiguous [rows, cols]) =
 * dropout(dx) computed from the stored dx with the mask of ptj_dropout(train, seed) --
 * the t_dropout_bkwd2_t that the block backward applies to every residual-stream gradient
 * (model_triton.py:2021-2024, 2175-2178) without another pass over dx.  Bit-identical to
 * ptj_layernorm_bwd followed by ptj_dropout.  `keep_bytes` (nullable) are the keep bits
 * that ptj_dropout_add_keep recorded for the same (seed, shape); with them the mask is
 * read instead of recomputed (2-byte element types only).  `dropped_colsum` (nullable,
 * [cols]; needs dropped and dgamma) receives the column sums of the stored `dropped`: the
 * `.sum(dim=0)` bias gradient of the linear layer that `dropped` is the output gradient of
 * (model_triton.py:426), from the same two-stage reduction as dgamma/dbeta. */
int ptj_layernorm_bwd_dropout(const void* dy, const void* x, const void* gamma, const void* residual,
                              void* dx, void* dgamma, void* dbeta,
                              void* dropped, void* dropped_colsum, int drop_train, int64_t drop_seed,
                              const void* keep_bytes,
                              void* workspace, size_t workspace_bytes,
                              int64_t rows, int64_t cols, int64_t dy_row_stride, int64_t x_row_stride,
                              int64_t dx_row_stride, int dtype, void* stream);

/* Column sums out[c] = sum_r x[r, c] (bias gradients: the `.sum(dim=0)` of
 * t_linear_bkwd2_p, model_triton.py:426).  Two-stage, fixed order.  `workspace`:
 * ptj_colsum_workspace_bytes(rows, cols) bytes. */
size_t ptj_colsum_workspace_bytes(int64_t rows, int64_t cols);
int ptj_colsum(const void* x, void* out, void* workspace, size_t workspace_bytes,
               int64_t rows, int64_t cols, int64_t x_row_stride, int dtype, void* stream);

/* ptj_colsum without a workspace argument, for callers that cannot allocate one (code under
 * HIP graph capture, serving loops and harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The stage-1 partial sums go to a device array built into
 * the library (PTJ_COLSUM_STATIC_SCRATCH_BYTES per GPU, held until the process ends); shapes
 * whose partial sums do not fit -- ptj_colsum_workspace_bytes(rows, cols) above that size --
 * are rejected with PTJ_ERR_INVALID and nothing is launched.  No hipMalloc, hipFree or other
 * allocating call is made; the array's device address is looked up on the first call on a GPU
 * unless ptj_init() has done so before (callers under graph capture call ptj_init first).
 * The GPU that `stream` belongs to must be the current device.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two
 * streams, two threads) race; calls ordered on one stream are safe.  Results are bit-equal
 * to ptj_colsum's. */
#define PTJ_COLSUM_STATIC_SCRATCH_BYTES (16u << 20)
#define PTJ_MAX_DEVICES 64
int ptj_colsum_static(const void* x, void* out, int64_t rows, int64_t cols, int64_t x_row_stride,
                      int dtype, void* stream);

/* tanh-GELU forward / backward on a flat array of n elements.
 * Replace t_gelu_fwd_k/_t (model_triton.py:237-260) and t_gelu_bkwd2_k/_t (:274-304). */
int ptj_gelu_fwd(const void* x, void* y, int64_t n, int dtype, void* stream);
int ptj_gelu_bwd(const void* dy, const void* x, void* dx, int64_t n, int dtype, void* stream);
/* GELU backward on [rows, cols] (contiguous) that also returns the column sums of dx:
 * dx = dy * gelu'(x), colsum[c] = sum_r dx[r, c] over the stored (rounded) values -- the
 * gradient of the bias in front of the GELU (t_gelu_bkwd2_t followed by the `.sum(dim=0)`
 * of t_linear_bkwd2_p, model_triton.py:296-304 and :426) in one pass over dx.
 * `workspace`: ptj_colsum_workspace_bytes(rows, cols) bytes. */
int ptj_gelu_bwd_colsum(const void* dy, const void* x, void* dx, void* colsum, void* workspace,
                        size_t workspace_bytes, int64_t rows, int64_t cols, int dtype, void* stream);

/* Dropout, rate 0.1, non-inverted: train != 0 -> y = keep ? x : 0 with
 * keep = tl.rand(seed + row, col) > 0.1 (Philox4x32-10); train == 0 -> y = 0.9*x.
 * The backward applies the same function to dy, so one entry point serves
 * t_dropout_fwd_k/_t (model_triton.py:1471-1506) and t_dropout_bkwd2_k/_t (:1538-1572). */
int ptj_dropout(const void* x, void* y, int64_t rows, int64_t cols,
                int64_t x_row_stride, int64_t y_row_stride,
                int train, int64_t seed, int dtype, void* stream);

/* Fused residual update used by the block composites: y = res + dropout(x) with
 * the same mask as ptj_dropout (model_triton.py:1898, 2069: y + t_dropout_fwd_t(...)).
 * All three tensors are contiguous [rows, cols]. */
int ptj_dropout_add(const void* x, const void* res, void* y, int64_t rows, int64_t cols,
                    int train, int64_t seed, int dtype, void* stream);

/* ptj_dropout_add that also records its keep mask: keep_bytes[r * cols/8 + g] holds, in
 * bit j, whether column 8g + j of row r was kept (train != 0).  The backward
 * (ptj_layernorm_bwd_dropout) can then read the mask instead of re-running Philox.
 * Needs a 2-byte element type, cols % 8 == 0 and 16-byte aligned tensors. */
int ptj_dropout_add_keep(const void* x, const void* res, void* y, void* keep_bytes,
                         int64_t rows, int64_t cols, int train, int64_t seed, int dtype, void* stream);

/* Embedding forward: out[i, :] = dropout(round(wemb[tokens[i], :] * scale) + pos[i mod seq, :])
 * for i < n, with the mask of ptj_dropout(train, seed) on [n, dim] -- t_embed_fwd
 * (model_triton.py:166-167), the position add and the embedding dropout of
 * t_gpt2_tlayers_fwd3_t (model_triton.py:2334-2351) in one pass.  Token ids must lie in
 * [0, vocab). */
int ptj_embed_fwd(const void* wemb, const void* pos, const int64_t* tokens, void* out,
                  int64_t n, int64_t dim, int64_t seq, int64_t vocab, float scale,
                  int train, int64_t seed, int dtype, void* stream);

/* Embedding backward, in place on the table gradient:
 * dwemb[t, :] += scale * sum_{i: tokens[i] = t} d[i, :] -- the scatter-add of
 * t_embed_bkwd (model_triton.py:2489-2521) accumulated onto the tied LM-head gradient
 * (:2591).  `sorted_tokens` are the n token ids in ascending (stable) order and `order`
 * the permutation that sorts them (sorted_tokens[j] = tokens[order[j]]); every run of equal
 * ids is summed in that order in fp32, so the result is deterministic. */
int ptj_embed_bwd(const void* d, const int64_t* sorted_tokens, const int64_t* order, void* dwemb,
                  int64_t n, int64_t dim, int64_t vocab, float scale, int dtype, void* stream);

/* ptj_dropout_add[_keep] followed by ptj_layernorm_fwd on its result, in one pass:
 * y = res + dropout(x), h = layernorm(y) with the values of y as stored -- the residual
 * update of one sub-block and the normalisation that opens the next one
 * (model_triton.py:1898 / :2069 then :1625-1637).  All tensors contiguous [rows, cols];
 * `keep_bytes` (nullable) as in ptj_dropout_add_keep.  Bit-identical to the two calls. */
int ptj_dropout_add_layernorm(const void* x, const void* res, const void* gamma, const void* beta,
                              void* y, void* h, void* keep_bytes, int64_t rows, int64_t cols,
                              int train, int64_t seed, int dtype, void* stream);

/* Row-wise log-softmax forward / backward (dx = dy - softmax(x)*sum(dy)).
 * Replace t_log_softmax_fwd_k/_t (model_triton.py:30-72) and
 * t_log_softmax_bkwd2_k/_t (:122-164). */
int ptj_log_softmax_fwd(const void* x, void* y, int64_t rows, int64_t cols,
                        int64_t x_row_stride, int64_t y_row_stride, int dtype, void* stream);
int ptj_log_softmax_bwd(const void* dy, const void* x, void* dx, int64_t rows, int64_t cols,
                        int64_t dy_row_stride, int64_t x_row_stride, int64_t dx_row_stride,
                        int dtype, void* stream);

/* Fused log-softmax + mean cross-entropy forward and backward over rows whose
 * label != 0.  Replaces t_avg_cross_entropy_loss_bkwd3_k/_t
 * (loss_and_optimizer_triton.py:108-197).
 *   labels  int64 [rows];  logits/dlogits [rows, cols] with row strides;
 *   loss    float [1]  (fp32 regardless of dtype) = -mean_{label!=0} log_softmax(x)[label];
 *   count   int64 [1]  = number of labels != 0;
 *   dlogits = (softmax(x) - onehot(label))/count on rows with label != 0, else 0.
 *   pred    int64 [rows] or NULL: argmax of each logits row (lowest index on ties), the
 *           input of the reference's accuracy() (loss_and_optimizer_triton.py:199-200);
 * dlogits may alias logits (in-place).  `workspace`: ptj_ce_workspace_bytes(rows) bytes.
 * Deterministic (no atomics).  count == 0 gives loss = NaN as the reference does. */
size_t ptj_ce_workspace_bytes(int64_t rows);
int ptj_ce_fwd_bwd(const int64_t* labels, const void* logits, float* loss, int64_t* count,
                   void* dlogits, int64_t* pred, void* workspace, size_t workspace_bytes,
                   int64_t rows, int64_t cols, int64_t logits_row_stride, int64_t dlogits_row_stride,
                   int dtype, void* stream);

/* ptj_ce_fwd_bwd that also returns the column sums of the stored gradient,
 * colsum[c] = sum_r dlogits[r, c] -- the `.sum(dim=0)` bias gradient of t_linear_bkwd2_p
 * (model_triton.py:426) for the layer that produced the logits (the tied LM head,
 * model_triton.py:2538) -- from the same pass, so the gradient is not read again.
 * 2-byte storage only (dtype PTJ_BF16); both row strides must be multiples of 8 elements
 * (all rows then share one 16-byte phase); cols + 8 <= 57344.  Other layouts: call
 * ptj_ce_fwd_bwd and ptj_colsum.  `workspace`: ptj_ce_colsum_workspace_bytes(rows, cols)
 * bytes (per-row losses and one fp32 partial row per workgroup).  Fixed summation order. */
size_t ptj_ce_colsum_workspace_bytes(int64_t rows, int64_t cols);
int ptj_ce_fwd_bwd_colsum(const int64_t* labels, const void* logits, float* loss, int64_t* count,
                          void* dlogits, int64_t* pred, void* colsum, void* workspace,
                          size_t workspace_bytes, int64_t rows, int64_t cols, int64_t logits_row_stride,
                          int64_t dlogits_row_stride, int dtype, void* stream);

/* ptj_ce_fwd_bwd_colsum over the rows [row0, row0 + rows) of a problem of rows_total rows, for a caller
 * that holds only a chunk of the logits at a time (LM head -> loss -> dX in row chunks: the
 * reference materialises all [B, T, V] logits, model_triton.py:2538).  `labels` and `pred` are the
 * whole arrays (rows_total entries), `logits` / `dlogits` point at the chunk's first row, the
 * workspace is that of the whole problem (ptj_ce_colsum_workspace_bytes(rows_total, cols)) and must
 * be left alone between the calls.  The call with row0 == 0 counts the labels != 0 of ALL rows
 * (`count`), the call that reaches rows_total writes `loss` and `colsum`.  Chunks must be
 * processed in row order with row0 a multiple of the device's CU count; then every addition
 * happens in the order of the one-call form and the results are bit-equal to it. */
int ptj_ce_fwd_bwd_colsum_rows(const int64_t* labels, const void* logits, float* loss, int64_t* count,
                               void* dlogits, int64_t* pred, void* colsum, void* workspace,
                               size_t workspace_bytes, int64_t rows_total, int64_t row0, int64_t rows,
                               int64_t cols, int64_t logits_row_stride, int64_t dlogits_row_stride,
                               int dtype, void* stream);

/* ---- dense contraction --------------------------------------------------- */

/* C[n,m] = sum_k A(n,k) * B(k,m) (+ bias[m]) (gelu) with fp32 accumulation on MFMA.
 * A(n,k) = a[n*a_rs + k*a_cs], B(k,m) = b[k*b_rs + m*b_cs]; for each operand one
 * of the two strides must be 1 (row- or column-major views, as produced by
 * `.t()`), C is row-major with row stride c_rs.  Replaces t_matmul_k / t_matmul_t
 * (model_triton.py:313-398) and the two launches of t_tlayer_ffn_fwd_t (:1258-1313);
 * also the torch.matmul / einsum call sites of the training path
 * (:306, :436, :460-472, :495-508, :423-428).
 * Operands that are 16-byte aligned with a leading stride that is a multiple of
 * 16 bytes take the vectorised path; anything else (any strides) is still computed,
 * through scalar loads.  `workspace` (nullable) lets small outputs with a long k be
 * split along k: pass ptj_gemm_workspace_bytes(n, m, k, dtype) bytes; the split
 * partials are reduced in fixed order, so results are deterministic.  `c_pre`
 * (nullable, PTJ_EPI_BIAS_GELU only) additionally receives A.B + bias before the GELU:
 * the activation the backward needs (the reference recomputes it, model_triton.py:1415-1418).
 * With PTJ_EPI_BIAS_GELU_DERIV `c_pre` (required) receives gelu'(A.B + bias) instead, taken from
 * the fp32 accumulators with the exponential the GELU needs anyway: what the backward multiplies
 * the incoming gradient by (t_gelu_bkwd2_k, model_triton.py:274-294).
 * PTJ_EPI_ACCUMULATE (no bias; 2-byte storage, 16-byte aligned operands with unit stride along one
 * axis, k a multiple of 64, no K split: anything else is refused) starts the fp32 accumulators from
 * the stored C: a weight gradient summed over row chunks of the batch (the reference forms it in one
 * product over all rows, model_triton.py:423-428). */
size_t ptj_gemm_workspace_bytes(int64_t n, int64_t m, int64_t k, int dtype);
int ptj_gemm(const void* a, const void* b, void* c, const void* bias,
             int64_t n, int64_t m, int64_t k,
             int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t c_rs,
             int epilogue, void* c_pre, int64_t c_pre_rs,
             void* workspace, size_t workspace_bytes, int dtype, void* stream);

/* C[n,m] = round(A.B) * mul[n,m] element-wise, and colsum[m] = the column sums of the stored C:
 * the product that carries a gradient back through the feed-forward block's second linear layer
 * (t_proj_bkwd2_x, model_triton.py:495-508), the GELU backward (t_gelu_bkwd2_k, :274-294; `mul` =
 * gelu' kept by PTJ_EPI_BIAS_GELU_DERIV) and the first layer's bias gradient (:426) in one
 * launch plus a small fixed-order reduction.  A.B is rounded to the storage type before the
 * multiplication, as when the product is stored and re-read.  Operands as for ptj_gemm; `mul`
 * and C are row-major with row strides mul_rs / c_rs.  `workspace` must hold
 * ptj_gemm_mul_colsum_workspace_bytes(n, m) bytes (one fp32 row of sums per 64 rows of C). */
size_t ptj_gemm_mul_colsum_workspace_bytes(int64_t n, int64_t m);
int ptj_gemm_mul_colsum(const void* a, const void* b, const void* mul, void* c, void* colsum,
                        int64_t n, int64_t m, int64_t k,
                        int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t mul_rs, int64_t c_rs,
                        void* workspace, size_t workspace_bytes, int dtype, void* stream);

/* ---- optimizer ----------------------------------------------------------- */

/* Fused AdamW update of one tensor, in place on the fp32 master weight and moments
 * (replaces the per-tensor Python loops of adam_w_in_place,
 * loss_and_optimizer_triton.py:376-401): with step t = i+1,
 *   m = b1 m + (1-b1) g;  v = b2 v + (1-b2) g^2;
 *   p += -lr * ( (m/(1-b1^t)) / (sqrt(v/(1-b2^t)) + eps) + weight_decay * p ).
 * `g` has grad_dtype (fp32 or bf16); `shadow` (nullable, shadow_dtype) receives the
 * updated weight rounded to the compute type. */
int ptj_adamw(float* p, float* m, float* v, const void* g, void* shadow, int64_t n,
              float lr, float beta1, float beta2, float eps, float weight_decay, int64_t t,
              int grad_dtype, int shadow_dtype, void* stream);

/* The same update for `count` tensors in as few launches as possible (the whole
 * parameter nest of adam_w_in_place, loss_and_optimizer_triton.py:376-401, in one call).
 * p, m, v, g, shadow, n and weight_decay are HOST arrays of `count` entries (shadow may be
 * NULL: no low-precision copies); all gradients share grad_dtype and all shadows
 * shadow_dtype.  Each tensor is updated exactly as by ptj_adamw. */
int ptj_adamw_multi(int64_t count, float* const* p, float* const* m, float* const* v,
                    const void* const* g, void* const* shadow, const int64_t* n,
                    const float* weight_decay, float lr, float beta1, float beta2, float eps,
                    int64_t t, int grad_dtype, int shadow_dtype, void* stream);

/* ---- attention ----------------------------------------------------------- */

/* Causal flash-attention forward.  q/k/v/o are [B, H, T, dh] views with explicit
 * (batch, head, row) strides and unit stride along dh -- e.g. slices of the
 * [B*T, H*3*dh] output of one fused QKV product; `mask` is NULL (pure causal:
 * key j visible to query i iff j <= i) or the [B, T, T] mask (shared by the heads, as in
 * the reference, model_triton.py:637) in the bit-packed form that ptj_attn_pack_mask
 * writes; it is ANDed with the causal block structure exactly as the reference kernel
 * does (tiles strictly above the diagonal are never visited; model_triton.py:659-661).
 * Saves ms (running row max of the scaled, masked scores) and ls (sum of
 * exp(score - ms)) as fp32 [BH, T].  Dropout (train != 0) keeps probability
 * (i, j) of batch-head g iff tl.rand(seed + g, i + j) > 0.1; train == 0 scales
 * probabilities by 0.9.  Replaces t_scaled_dot_prod_attn_fwd3_k/_t
 * (model_triton.py:616-754).  ms/ls are contiguous [B*H, T].  Requires dh == 64, T % 64 == 0, 16-byte aligned
 * pointers and strides that are multiples of 16 bytes.  A non-NULL mask is applied
 * as (mask AND key <= query): masks must be sub-masks of the causal mask, as the
 * training path produces them.  A query without any visible key (a padding row) gets an
 * all-zero output row and the statistics (ms, ls) = (-1e9, 0), and the backward passes no
 * gradient through it; the reference's kernel averages V over the keys of the tiles it
 * happens to visit there (model_triton.py:678-682), its torch twin over all T keys -- such
 * rows carry label 0 and are ignored by the loss.  `workspace` is needed when train != 0
 * only (ptj_attn_workspace_bytes(B, H, T) bytes; the dropout keep bits live there). */
size_t ptj_attn_workspace_bytes(int64_t B, int64_t H, int64_t T);

/* Packs a uint8 [B, T, T] mask (nonzero = visible; contiguous) for the attention kernels:
 * one bit per (query, key), stored twice -- as words of 32 queries per key and as words of
 * 32 keys per query -- so that a wavefront fetches the mask of a 32x32 score tile with
 * scalar loads and applies it with lane-mask selects -- followed by one class word per
 * 32x32 tile of (mask AND causal), in both index orders: hidden / mixed / equal to the causal
 * pattern.  The kernels skip hidden tiles, read mask words only for mixed ones and mask by
 * index elsewhere, so a plain lower-triangular mask tensor runs at the speed of mask = NULL.
 * `packed` holds ptj_attn_packed_mask_bytes(B, T) bytes (about a quarter of the byte mask).
 * T % 32 == 0.
 * The reference passes the bool mask itself to its kernels (model_triton.py:637, 672). */
size_t ptj_attn_packed_mask_bytes(int64_t B, int64_t T);
int ptj_attn_pack_mask(const uint8_t* mask, uint32_t* packed, int64_t B, int64_t T, void* stream);

int ptj_attn_fwd(const void* q, const void* k, const void* v, const uint32_t* mask,
                 void* o, float* ms, float* ls, void* workspace, size_t workspace_bytes,
                 int64_t B, int64_t H, int64_t T, int64_t dh,
                 int64_t q_b_stride, int64_t q_h_stride, int64_t q_row_stride,
                 int64_t k_b_stride, int64_t k_h_stride, int64_t k_row_stride,
                 int64_t v_b_stride, int64_t v_h_stride, int64_t v_row_stride,
                 int64_t o_b_stride, int64_t o_h_stride, int64_t o_row_stride,
                 int train, int64_t seed, int dtype, void* stream);

/* Flash-attention backward with P recomputed from (ms, ls).  Outputs dq/dk/dv
 * [BH, T, dh] with explicit strides.  Deterministic: dK/dV and dQ are produced by
 * two passes, no atomics (the dQ pass runs first and leaves rowsum(dO*O) in the
 * workspace for the dK/dV pass), so no output may overlap an input.  `workspace`
 * (always required here) holds
 * ptj_attn_workspace_bytes(B, H, T) bytes.  Replaces
 * t_scaled_dot_prod_attn_bkwd3_k/_t (model_triton.py:829-1003). */
int ptj_attn_bwd(const void* d_o, const void* q, const void* k, const void* v, const void* o,
                 const float* ms, const float* ls, const uint32_t* mask,
                 void* dq, void* dk, void* dv, void* workspace, size_t workspace_bytes,
                 int64_t B, int64_t H, int64_t T, int64_t dh,
                 int64_t do_b_stride, int64_t do_h_stride, int64_t do_row_stride,
                 int64_t q_b_stride, int64_t q_h_stride, int64_t q_row_stride,
                 int64_t k_b_stride, int64_t k_h_stride, int64_t k_row_stride,
                 int64_t v_b_stride, int64_t v_h_stride, int64_t v_row_stride,
                 int64_t o_b_stride, int64_t o_h_stride, int64_t o_row_stride,
                 int64_t dq_b_stride, int64_t dq_h_stride, int64_t dq_row_stride,
                 int64_t dk_b_stride, int64_t dk_h_stride, int64_t dk_row_stride,
                 int64_t dv_b_stride, int64_t dv_h_stride, int64_t dv_row_stride,
                 int train, int64_t seed, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PTJ_H */
