"""Loss-side wrappers with the reference's names (loss_and_optimizer_triton.py of
martin-kukla/pre-tjax) on top of libptj.so."""
import torch

from ._lib import check, dtype_code, lib, ptr, require_gpu, stream
from .model_triton import _workspace


def t_avg_cross_entropy_loss_bkwd3_t(y_labels: torch.Tensor, x_logits: torch.Tensor, inplace=False):
    """Fused log-softmax + mean cross-entropy forward and backward
    (reference: loss_and_optimizer_triton.py:176-197).

    Returns ``(loss[1] fp32, nonzero_count 0-d int64, dloss_dlogits like x_logits)``.
    With ``inplace=True`` the gradient overwrites ``x_logits`` (an extension: the
    reference always allocates)."""
    require_gpu(y_labels, x_logits)
    shape = x_logits.shape
    labels = y_labels.reshape(-1).to(torch.int64).contiguous()
    x2 = x_logits.reshape(labels.numel(), -1)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    rows, cols = x2.shape
    loss = torch.empty(1, dtype=torch.float32, device=x2.device)
    count = torch.empty((), dtype=torch.int64, device=x2.device)
    dx = x2 if inplace else torch.empty_like(x2)
    ws_bytes = lib().ptj_ce_workspace_bytes(rows)
    ws = _workspace(ws_bytes, x2.device, "ce")
    check(lib().ptj_ce_fwd_bwd(ptr(labels), ptr(x2), ptr(loss), ptr(count), ptr(dx), ptr(ws), ws_bytes, rows, cols,
                               x2.stride(0), dx.stride(0), dtype_code(x2), stream()), "ptj_ce_fwd_bwd")
    return loss, count, dx.reshape(shape)
