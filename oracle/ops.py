"""Per-operator CPU restatement of the reference's functional ops (torch, any
float dtype; tests run it in float64 and float32).  TEST INFRASTRUCTURE ONLY.

Every function cites the reference lines it restates.  None of them is used by
the product; see oracle/__init__.py.
"""
import math

import numpy as np
import torch

from . import philox

DROPOUT_RATE = 0.1  # model_torch_func.py:2


def log_softmax(x):
    """model_torch_func.py:50-52 / model_triton.py:25-27."""
    x = x - x.max(dim=-1, keepdim=True)[0]
    return x - torch.logsumexp(x, dim=-1, keepdim=True)


def log_softmax_bkwd2(dy, x):
    """model_triton.py:91-102: dy - softmax(x) * sum(dy)."""
    x = x - x.max(dim=-1, keepdim=True)[0]
    e = torch.exp(x)
    return dy - dy.sum(-1, keepdim=True) * e / e.sum(-1, keepdim=True)


def gelu(x):
    """model_torch_func.py:60-62 / model_triton.py:221-223 (tanh form)."""
    k = math.sqrt(2 / math.pi)
    return 0.5 * x * (1 + torch.tanh(k * (x + 0.044715 * x ** 3)))


def gelu_bkwd2(dy, x):
    """model_triton.py:262-271."""
    k = math.sqrt(2 / math.pi)
    t = torch.tanh(k * (x + 0.044715 * x ** 3))
    dt = (1 - t * t) * k * (1 + 3 * 0.044715 * x * x)
    return dy * (0.5 * (1 + t) + 0.5 * x * dt)


def layernorm_fwd(params, x):
    """model_torch_func.py:104-108: unbiased std (N-1), no epsilon."""
    mu = x.mean(dim=-1, keepdim=True)
    sd = x.std(dim=-1, keepdim=True)  # torch default: unbiased
    return (x - mu) / sd * params[0] + params[1]


def layernorm_bkwd2_p(dy, params, x):
    """model_triton.py:1652-1660."""
    mu = x.mean(dim=-1, keepdim=True)
    sd = x.std(dim=-1, keepdim=True)
    xh = (x - mu) / sd
    red = tuple(range(x.dim() - 1))
    return (dy * xh).sum(dim=red), dy.sum(dim=red)


def layernorm_bkwd2_x(dy, params, x):
    """model_triton.py:1773-1795 (llm.c-style form with the N/(N-1) correction)."""
    n = x.shape[-1]
    mu = x.mean(dim=-1, keepdim=True)
    rstd = 1 / x.std(dim=-1, keepdim=True)
    xh = (x - mu) * rstd
    g = dy * params[0]
    out = g - g.mean(-1, keepdim=True) - xh * (g * xh).mean(-1, keepdim=True) * (n / (n - 1))
    return out * rstd


def rowwise_keep(x_shape, seed):
    """Keep mask of the row-wise dropout kernels as a bool tensor of `x_shape`
    (rows = all leading dims flattened; model_triton.py:1496-1505)."""
    cols = x_shape[-1]
    rows = int(np.prod(x_shape[:-1])) if len(x_shape) > 1 else 1
    m = philox.rowwise_keep_mask(seed, rows, cols, DROPOUT_RATE)
    return torch.from_numpy(m.reshape(x_shape))


def dropout(x, train=True, p_gen_aux=None):
    """model_triton.py:1460-1468,1471-1506: non-inverted dropout; eval scales by
    (1-p).  The mask is the Triton-kernel mask (Philox), not torch.bernoulli."""
    if not train:
        return x * (1 - DROPOUT_RATE)
    return torch.where(rowwise_keep(tuple(x.shape), p_gen_aux), x, torch.zeros_like(x))


def dropout_bkwd2(dy, x, train=True, p_gen_aux=None):
    """model_triton.py:1527-1572: same mask applied to dy."""
    return dropout(dy, train, p_gen_aux)


def attn_keep(B, H, T, seed):
    m = philox.attn_keep_mask(seed, B * H, T, T, DROPOUT_RATE)
    return torch.from_numpy(m.reshape(B, H, T, T))


def softmax_attn(q, k, mask, train, p_gen_aux=None, keep=None):
    """model_triton.py:510-517 / model_torch_func.py:70-77.  q,k: [B,H,T,dh];
    mask [B,T,T] bool.  Returns (P, P_dropped)."""
    dh = q.shape[-1]
    s = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(dh)
    s = torch.where(mask.unsqueeze(1), s, torch.full_like(s, -1e9))
    p = torch.exp(log_softmax(s))
    if not train:
        return p, p * (1 - DROPOUT_RATE)
    if keep is None:
        B, H, T, _ = q.shape
        keep = attn_keep(B, H, T, p_gen_aux)
    return p, torch.where(keep, p, torch.zeros_like(p))


def scaled_dot_prod_attn_fwd(qkv, mask, train=True, p_gen_aux=None):
    """model_triton.py:608-611.  qkv [B,H,3,T,dh] -> O [B,H,T,dh]."""
    q, k, v = torch.unbind(qkv, dim=2)
    _, pd = softmax_attn(q, k, mask, train, p_gen_aux)
    return torch.matmul(pd, v)


def scaled_dot_prod_attn_stats(qkv, mask):
    """Row max `ms` and sum-exp `ls` the flash kernel saves (model_triton.py:655-700):
    ms = max_j s_ij, ls = sum_j exp(s_ij - ms)."""
    q, k, _ = torch.unbind(qkv, dim=2)
    dh = q.shape[-1]
    s = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(dh)
    s = torch.where(mask.unsqueeze(1), s, torch.full_like(s, -1e9))
    ms = s.max(dim=-1)[0]
    ls = torch.exp(s - ms.unsqueeze(-1)).sum(-1)
    return ms, ls


def scaled_dot_prod_attn_bkwd(dO, qkv, mask, train=True, p_gen_aux=None):
    """model_triton.py:801-811 + 550-606 restated as closed-form VJP:
    dV = Pd^T dO; dPd = dO V^T; dP = dPd*keep (or *(1-p) in eval);
    dS = P*(dP - rowsum(dP*P)); masked entries 0; dQ = dS K/sqrt(dh); dK = dS^T Q/sqrt(dh)."""
    q, k, v = torch.unbind(qkv, dim=2)
    dh = q.shape[-1]
    B, H, T, _ = q.shape
    if train:
        keep = attn_keep(B, H, T, p_gen_aux)
        p, pd = softmax_attn(q, k, mask, True, keep=keep)
    else:
        p, pd = softmax_attn(q, k, mask, False)
    dv = torch.matmul(pd.transpose(-2, -1), dO)
    dpd = torch.matmul(dO, v.transpose(-2, -1))
    dp = torch.where(keep, dpd, torch.zeros_like(dpd)) if train else dpd * (1 - DROPOUT_RATE)
    ds = p * (dp - (dp * p).sum(-1, keepdim=True))
    ds = torch.where(mask.unsqueeze(1), ds, torch.zeros_like(ds)) / math.sqrt(dh)
    dq = torch.matmul(ds, k)
    dk = torch.matmul(ds.transpose(-2, -1), q)
    return dq, dk, dv


def avg_cross_entropy_loss(y_labels, x_logits):
    """loss_and_optimizer_triton.py:26-32: mean over positions with label != 0."""
    y = y_labels.reshape(-1).to(torch.int64)
    x = x_logits.reshape(y.numel(), -1)
    el = log_softmax(x)[torch.arange(y.numel()), y]
    el = torch.where(y != 0, el, torch.full_like(el, float("nan")))
    return -torch.nanmean(el), torch.count_nonzero(y)


def avg_cross_entropy_loss_bkwd3(y_labels, x_logits):
    """loss_and_optimizer_triton.py:83-106: (loss, count, dlogits)."""
    shape = x_logits.shape
    y = y_labels.reshape(-1, 1).to(torch.int64)
    x = x_logits.reshape(y.numel(), -1)
    cnt = torch.count_nonzero(y)
    loss, _ = avg_cross_entropy_loss(y_labels, x_logits)
    sm = torch.exp(log_softmax(x))
    onehot = torch.zeros_like(sm).scatter_(1, y, 1.0)
    dx = torch.where(y != 0, (sm - onehot) / cnt, torch.zeros_like(sm))
    return loss, cnt, dx.reshape(shape)


def accuracy(y_labels, x_logits):
    """loss_and_optimizer_triton.py:199-200."""
    hit = (y_labels == torch.argmax(x_logits, dim=-1)).to(x_logits.dtype)
    return torch.nanmean(torch.where(y_labels != 0, hit, torch.full_like(hit, float("nan"))))


def matmul_bruteforce(a, b):
    """Triple loop for tiny shapes (pins the GEMM convention C[n,m]=sum_k A[n,k]B[k,m])."""
    n, kk = a.shape
    _, m = b.shape
    c = torch.zeros(n, m, dtype=a.dtype)
    for i in range(n):
        for j in range(m):
            acc = 0.0
            for t in range(kk):
                acc += float(a[i, t]) * float(b[t, j])
            c[i, j] = acc
    return c
