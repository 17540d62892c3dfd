"""Loss-side wrappers with the reference's names (loss_and_optimizer_triton.py of
martin-kukla/pre-tjax) on top of libptj.so."""
import ctypes
import math

import torch

from ._lib import check, dtype_code, lib, ptr, require_gpu, stream
from .model_triton import _workspace
from .spec_torch import accuracy, t_avg_cross_entropy_loss, t_avg_cross_entropy_loss_bkwd3  # noqa: F401  (torch twins)


def t_avg_cross_entropy_loss_bkwd3_t(y_labels: torch.Tensor, x_logits: torch.Tensor, inplace=False, want_pred=False,
                                     want_colsum=False):
    """Fused log-softmax + mean cross-entropy forward and backward
    (reference: loss_and_optimizer_triton.py:176-197).

    Returns ``(loss[1] fp32, nonzero_count 0-d int64, dloss_dlogits like x_logits)``.
    With ``inplace=True`` the gradient overwrites ``x_logits`` (an extension: the
    reference always allocates).  With ``want_pred=True`` a further value is returned:
    the row-wise argmax of the logits (int64, shaped like ``y_labels``), computed in
    the same pass -- the input of ``accuracy``.  With ``want_colsum=True`` the last value
    returned is the column sum of the stored gradient over all rows (``[V]``: the gradient
    of the bias that was added to the logits, model_triton.py:426), from the same pass for
    2-byte logits whose row pitch is a multiple of 8 elements, else from ``colsum_t``."""
    require_gpu(y_labels, x_logits)
    shape = x_logits.shape
    labels = y_labels.reshape(-1).to(torch.int64).contiguous()
    x2 = x_logits.reshape(labels.numel(), -1)     # a view for row-padded logits buffers
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    rows, cols = x2.shape
    loss = torch.empty(1, dtype=torch.float32, device=x2.device)
    count = torch.empty((), dtype=torch.int64, device=x2.device)
    if inplace:
        dx = x2
    else:  # same row pitch and the same offset inside a 16-byte line as the logits, so rows keep their phase
        mis = (x2.data_ptr() % 16) // x2.element_size()
        flat = torch.empty((rows - 1) * x2.stride(0) + cols + mis, dtype=x2.dtype, device=x2.device)
        dx = flat[mis:].as_strided((rows, cols), (x2.stride(0), 1))
    pred = torch.empty(rows, dtype=torch.int64, device=x2.device) if want_pred else None
    colsum = None
    fused = (want_colsum and x2.dtype == torch.bfloat16 and x2.stride(0) % 8 == 0 and dx.stride(0) % 8 == 0
             and cols + 8 <= 1024 * 56 and (x2.data_ptr() - dx.data_ptr()) % 16 == 0)
    if fused:
        colsum = torch.empty(cols, dtype=x2.dtype, device=x2.device)
        ws_bytes = lib().ptj_ce_colsum_workspace_bytes(rows, cols)
        ws = _workspace(ws_bytes, x2.device, "ce")
        check(lib().ptj_ce_fwd_bwd_colsum(ptr(labels), ptr(x2), ptr(loss), ptr(count), ptr(dx), ptr(pred), ptr(colsum),
                                          ptr(ws), ws_bytes, rows, cols, x2.stride(0), dx.stride(0), dtype_code(x2),
                                          stream()), "ptj_ce_fwd_bwd_colsum")
    else:
        ws_bytes = lib().ptj_ce_workspace_bytes(rows)
        ws = _workspace(ws_bytes, x2.device, "ce")
        check(lib().ptj_ce_fwd_bwd(ptr(labels), ptr(x2), ptr(loss), ptr(count), ptr(dx), ptr(pred), ptr(ws), ws_bytes, rows,
                                   cols, x2.stride(0), dx.stride(0), dtype_code(x2), stream()), "ptj_ce_fwd_bwd")
        if want_colsum:
            from .model_triton import colsum_t
            colsum = colsum_t(dx)
    dx = dx.view(shape) if inplace else dx.reshape(shape)
    out = (loss, count, dx)
    if want_pred:
        out += (pred.reshape(y_labels.shape),)
    if want_colsum:
        out += (colsum,)
    return out


def accuracy_from_pred(y_labels, pred):
    """loss_and_optimizer_triton.py:199-200 given the row-wise argmax."""
    hit = (y_labels == pred).to(torch.float32)
    return torch.nanmean(torch.where(y_labels != 0, hit, torch.full_like(hit, float("nan"))))


LM_HEAD_CHUNK_ROWS = 8192   # rows of logits alive at a time in t_loss_bkwd3_t (0: all of them, one pass)


def _lm_head_loss_in_row_chunks(params, h, y_out, chunk):
    """LM head -> loss -> the head's three gradient products, `chunk` rows at a time: only
    [chunk, V] logits exist at any moment (the reference materialises [B, T, V],
    model_triton.py:2538, and a same-sized gradient, loss_and_optimizer_triton.py:176-197).
    Per chunk: logits = h_c @ Wemb^T + bemb into one reused row-padded buffer, the loss pass
    overwrites them with their gradient (continuing the loss sum, the argmax and the column sums of
    the previous chunks), dh_c = dlogits_c @ Wemb, and dWemb += dlogits_c^T @ h_c (accumulating
    epilogue: the stored sum is widened, added to and rounded once per chunk).
    Returns (loss[1], count, pred [B,T], dh [N,D], dwemb [V,D], dbemb [V])."""
    from .model_triton import _padded_logits, matmul_t
    wemb, bemb = params[0]
    V, D = wemb.shape
    N = y_out.numel()
    h2d = h.reshape(N, D)
    labels = y_out.reshape(-1).to(torch.int64).contiguous()
    dev = h.device
    loss = torch.empty(1, dtype=torch.float32, device=dev)
    count = torch.empty((), dtype=torch.int64, device=dev)
    pred = torch.empty(N, dtype=torch.int64, device=dev)
    dbemb = torch.empty(V, dtype=h.dtype, device=dev)
    dh = torch.empty((N, D), dtype=h.dtype, device=dev)
    dwemb = torch.empty((V, D), dtype=h.dtype, device=dev)
    buf = _padded_logits(chunk, V, h.dtype, dev)
    ws_bytes = lib().ptj_ce_colsum_workspace_bytes(N, V)
    ws = _workspace(ws_bytes, dev, "ce")
    for r0 in range(0, N, chunk):
        rows = min(chunk, N - r0)
        lg = buf[:rows]
        matmul_t(h2d[r0:r0 + rows], wemb.t(), bemb, out=lg)
        check(lib().ptj_ce_fwd_bwd_colsum_rows(ptr(labels), ptr(lg), ptr(loss), ptr(count), ptr(lg), ptr(pred), ptr(dbemb),
                                               ptr(ws), ws_bytes, N, r0, rows, V, lg.stride(0), lg.stride(0),
                                               dtype_code(lg), stream()), "ptj_ce_fwd_bwd_colsum_rows")
        matmul_t(lg, wemb, out=dh[r0:r0 + rows])
        matmul_t(lg.t(), h2d[r0:r0 + rows], out=dwemb, accumulate=r0 > 0)
    return loss, count, pred.reshape(y_out.shape), dh, dwemb, dbemb


def _chunked_head_applies(params, n_rows, chunk):
    """Row chunks need the fused loss pass (2-byte logits, vocabulary within its register budget)
    and chunk starts at multiples of the loss pass's workgroup count (one per CU)."""
    wemb = params[0][0]
    return (chunk > 0 and n_rows > chunk and wemb.dtype == torch.bfloat16 and wemb.shape[0] + 8 <= 1024 * 56
            and chunk % 1024 == 0 and wemb.shape[1] % 64 == 0 and chunk % 64 == 0)


def t_loss_bkwd3_t(params, y, y_mask, y_indices, train, p_gen_aux=None):
    """One forward+backward (reference: loss_and_optimizer_triton.py:279-289).
    y int [B,T+1] -> (grads nest, (loss, acc, non-pad fraction)).  With more than
    LM_HEAD_CHUNK_ROWS positions in 2-byte storage, the LM head, the loss and the head's gradient
    products run in row chunks (see _lm_head_loss_in_row_chunks); otherwise in one pass over a
    [B, T, V] logits buffer."""
    from .model_triton import (gpt2_bkwd_below_head_t, t_gpt2_bkwd3_p_t, t_gpt2_forward_with_acts_t,
                               t_gpt2_tlayers_fwd3_t)
    y_in = y[:, :-1]
    y_out = y[:, 1:]
    if _chunked_head_applies(params, y_out.numel(), LM_HEAD_CHUNK_ROWS):
        h, acts = t_gpt2_tlayers_fwd3_t(params, y_in, y_mask, y_indices, train, p_gen_aux)
        loss_val, tokens_count, pred, dh, dwemb, dbemb = _lm_head_loss_in_row_chunks(params, h, y_out, LM_HEAD_CHUNK_ROWS)
        grads = gpt2_bkwd_below_head_t(dh, dwemb, dbemb, [acts, h], params, y_in, y_mask, train, p_gen_aux)
        acc = accuracy_from_pred(y_out, pred)
        return grads, (loss_val, acc, tokens_count / y_out.numel())
    logits, acts = t_gpt2_forward_with_acts_t(params, y_in, y_mask, y_indices, train, p_gen_aux)
    # the bias gradient of the tied head (column sums of the loss gradient) comes out of the loss pass
    loss_val, tokens_count, dloss_dx, pred, dbemb = t_avg_cross_entropy_loss_bkwd3_t(y_out, logits, inplace=True,
                                                                                    want_pred=True, want_colsum=True)
    grads = t_gpt2_bkwd3_p_t(dloss_dx, acts, params, y_in, y_mask, y_indices, train, p_gen_aux, dbemb=dbemb)
    acc = accuracy_from_pred(y_out, pred)
    return grads, (loss_val, acc, tokens_count / y_out.numel())


def sample_p_gen_aux(params, generator=None):
    """1 + 3L dropout seeds in [0, 1e6) (loss_and_optimizer_triton.py:318-325) drawn on
    the host: no device round trips."""
    n = 1 + 3 * (len(params) - 3)
    return torch.randint(0, 1_000_000, (n,), generator=generator).tolist()


def t_acc_grad_loss3_t(acc_grads, params, y, y_mask, y_indices):
    """One micro-step of gradient accumulation on the kernel path
    (loss_and_optimizer_triton.py:336-337): -> (acc_grads, (loss, acc, non-pad fraction))."""
    return _acc_grad_loss(t_loss_bkwd3_t, acc_grads, params, y, y_mask, y_indices)


def _acc_grad_loss(grad_loss_fn, acc_grads, params, y, y_mask, y_indices):
    """loss_and_optimizer_triton.py:340-348: fresh dropout seeds, one forward+backward, and
    the step's gradients added onto `acc_grads` (entries are rebound, as in the reference;
    the sums are formed in the accumulator's dtype by multi-tensor adds, a few launches for
    the whole nest)."""
    step_grads, rest = grad_loss_fn(params, y, y_mask, y_indices, train=True, p_gen_aux=sample_p_gen_aux(params))
    flat_acc = [a for grp in acc_grads for a in grp]
    flat_new = [g.to(a.dtype).reshape(a.shape) for grp_a, grp_g in zip(acc_grads, step_grads)
                for a, g in zip(grp_a, grp_g)]
    summed = iter(torch._foreach_add(flat_acc, flat_new))
    for grp in acc_grads:
        for pi in range(len(grp)):
            grp[pi] = next(summed)
    return acc_grads, rest


def _sq_norms(tensors):
    return [n * n for n in torch._foreach_norm([t.float() for t in tensors])]


def grads_l2norm(grads):
    """Global L2 norm of a gradient nest as a Python float (reference :411-414)."""
    return math.sqrt(float(torch.stack(_sq_norms([g for grp in grads for g in grp])).sum()))


def grads_grps_l2norms(grads):
    """Per-group L2 norms of a gradient nest as Python floats (reference :415-416)."""
    return [math.sqrt(float(torch.stack(_sq_norms(list(grp))).sum())) for grp in grads]


def elwise(params_and_grads, func):
    """Apply `func` leaf by leaf over nests of equal shape (reference :355-356)."""
    return [[func(*leaves) for leaves in zip(*groups)] for groups in zip(*params_and_grads)]


def sgd(params, grads, lr):
    """reference :358-359."""
    return elwise((params, grads), lambda p, g: p - lr * g)


def init_adam_w(params):
    """(zero gradient accumulators, [first moments, second moments]), each shaped like
    `params` (loss_and_optimizer_triton.py:362-363).  The moments are fp32 whatever the
    parameter dtype; the accumulators take the parameters' dtype."""
    zeros = lambda dt: [[torch.zeros_like(p, dtype=dt or p.dtype) for p in grp] for grp in params]
    return zeros(None), [zeros(torch.float32), zeros(torch.float32)]


def adam_w_in_place(params, grads, lr, betas, epsilon, moments, i, weight_decay=0.0, weight_decay_mask=None,
                    shadow=None):
    """AdamW of the reference (:376-401: t = i+1, bias-corrected moments, decay scaled by
    lr) on fp32 master weights: one fused HIP pass over the whole nest (a few launches)
    instead of ~10 torch ops per tensor.
    `params` are the fp32 master weights, updated in place; `shadow` (optional nest of
    low-precision copies) is refreshed from them."""
    master = params
    t = i + 1
    ps, ms_, vs, gs, ss, ns, wds = [], [], [], [], [], [], []
    keep = []                                    # contiguous gradient copies must outlive the launch
    gdt = sdt = None
    for gi, grp in enumerate(master):
        for pi, p in enumerate(grp):
            g = grads[gi][pi]
            if not g.is_contiguous():
                g = g.contiguous()
                keep.append(g)
            sh = shadow[gi][pi] if shadow is not None else None
            assert p.dtype == torch.float32 and p.is_contiguous() and g.numel() == p.numel()
            assert gdt in (None, g.dtype) and (sh is None or sdt in (None, sh.dtype)), "mixed gradient / shadow dtypes"
            gdt = g.dtype
            if sh is not None:
                sdt = sh.dtype
            ps.append(p.data_ptr())
            ms_.append(moments[0][gi][pi].data_ptr())
            vs.append(moments[1][gi][pi].data_ptr())
            gs.append(g.data_ptr())
            ss.append(sh.data_ptr() if sh is not None else 0)
            ns.append(p.numel())
            wds.append(weight_decay if (weight_decay_mask is None or weight_decay_mask[gi][pi]) else 0.0)
    cnt = len(ps)
    if cnt:
        arr = lambda vals: (ctypes.c_void_p * cnt)(*vals)
        code = {torch.float32: 0, torch.bfloat16: 1}
        check(lib().ptj_adamw_multi(cnt, arr(ps), arr(ms_), arr(vs), arr(gs), arr(ss) if shadow is not None else None,
                                    (ctypes.c_int64 * cnt)(*ns), (ctypes.c_float * cnt)(*wds), lr, betas[0], betas[1],
                                    epsilon, t, code[gdt], code[sdt] if sdt is not None else -1, stream()),
              "ptj_adamw_multi")
    return master, moments
