"""Plain-torch twins of the kernel wrappers, under the reference's names without the
``_t`` suffix (model_triton.py:25, 91, 221, 269, 306, 436, 510, 608, 756, 801, 1244, 1450,
1518, 1574, 1652, 1790; loss_and_optimizer_triton.py:83).

The reference's accuracy and speed tests import these as the "naive" side they compare the
kernels with, and pass ``t_gelu_fwd`` around as the ``activation_fn`` marker; they are
differentiable torch code that runs on whatever device its inputs live on.  They are not on
the hot path: no ``*_t`` wrapper and no composite calls them.
"""
import math

import torch

DROPOUT_RATE = 0.1  # model_torch_func.py:2
_GELU_K = math.sqrt(2.0 / math.pi)
_GELU_C = 0.044715


def t_log_softmax_fwd(x_logits):
    z = x_logits - x_logits.amax(dim=-1, keepdim=True)
    return z - torch.logsumexp(z, dim=-1, keepdim=True)


def t_log_softmax_bkwd2(dloss_dx, x_logits):
    """VJP of log-softmax: dy - softmax(x) * sum(dy)."""
    sm = torch.softmax(x_logits, dim=-1)
    return dloss_dx - sm * dloss_dx.sum(dim=-1, keepdim=True)


def t_gelu_fwd(x):
    return 0.5 * x * (1.0 + torch.tanh(_GELU_K * (x + _GELU_C * x * x * x)))


def t_gelu_bkwd2(dloss_dx, x):
    th = torch.tanh(_GELU_K * (x + _GELU_C * x * x * x))
    dth = (1.0 - th * th) * _GELU_K * (1.0 + 3.0 * _GELU_C * x * x)
    return dloss_dx * (0.5 * (1.0 + th) + 0.5 * x * dth)


def t_linear_fwd(layer_params, x):
    return x @ layer_params[0].transpose(0, 1) + layer_params[1]


def t_proj_fwd(layer_params, x):
    return x @ layer_params.transpose(-2, -1)


def _bernoulli_keep(like, p_gen_aux):
    """The spec's own mask: torch.bernoulli on a generator seeded with p_gen_aux
    (model_triton.py:1455-1457) -- NOT the Philox mask of the kernels."""
    assert p_gen_aux is not None
    gen = torch.Generator(device=like.device).manual_seed(int(p_gen_aux))
    return torch.bernoulli(torch.full_like(like, 1.0 - DROPOUT_RATE), generator=gen)


def t_dropout_fwd(x, train=True, p_gen_aux=None):
    if not train:
        return x * (1.0 - DROPOUT_RATE)
    return x * _bernoulli_keep(x, p_gen_aux)


def t_dropout_bkwd2(dloss_dx, x, train=True, p_gen_aux=None):
    if not train:
        return dloss_dx * (1.0 - DROPOUT_RATE)
    return dloss_dx * _bernoulli_keep(x, p_gen_aux)


def _normalize(x):
    mu = x.mean(dim=-1, keepdim=True)
    rstd = 1.0 / x.std(dim=-1, keepdim=True)          # unbiased, no epsilon
    return (x - mu) * rstd, rstd


def t_layernorm_fwd(layer_params, x):
    xh, _ = _normalize(x)
    return xh * layer_params[0] + layer_params[1]


def t_layernorm_bkwd2_p(dloss_dx, layer_params, x):
    xh, _ = _normalize(x)
    lead = tuple(range(x.dim() - 1))
    return (dloss_dx * xh).sum(dim=lead), dloss_dx.sum(dim=lead)


def t_layernorm_bkwd2_x(dloss_dx, layer_params, x):
    n = x.shape[-1]
    xh, rstd = _normalize(x)
    g = dloss_dx * layer_params[0]
    proj = (g * xh).mean(dim=-1, keepdim=True) * (n / (n - 1.0))
    return (g - g.mean(dim=-1, keepdim=True) - xh * proj) * rstd


def t_softmax_attn_fwd(q, k, mask, train, p_gen_aux=None):
    s = (q @ k.transpose(-2, -1)) / math.sqrt(q.shape[-1])
    s = torch.where(mask.unsqueeze(1), s, torch.full_like(s, -1e9))
    return t_dropout_fwd(torch.exp(t_log_softmax_fwd(s)), train, p_gen_aux)


def t_softmax_attn_bkwd2(dloss_dx, q, k, mask, train, p_gen_aux=None):
    """(dq, dk) of t_softmax_attn_fwd for an incoming gradient of the dropped probabilities."""
    scale = 1.0 / math.sqrt(q.shape[-1])
    s = (q @ k.transpose(-2, -1)) * scale
    s = torch.where(mask.unsqueeze(1), s, torch.full_like(s, -1e9))
    p = torch.softmax(s, dim=-1)
    ds = t_log_softmax_bkwd2(t_dropout_bkwd2(dloss_dx, p, train, p_gen_aux) * p, s)
    ds = torch.where(mask.unsqueeze(1), ds, torch.zeros_like(ds))
    return (ds @ k) * scale, (ds.transpose(-2, -1) @ q) * scale


def t_scaled_dot_prod_attn_fwd(qkv, mask, train=True, p_gen_aux=None):
    q, k, v = torch.unbind(qkv, dim=2)
    return t_softmax_attn_fwd(q, k, mask, train, p_gen_aux) @ v


def t_scaled_dot_prod_attn_fwd3(qkv, mask, train=True, p_gen_aux=None):
    q, k, v = torch.unbind(qkv, dim=2)
    sa = t_softmax_attn_fwd(q, k, mask, train, p_gen_aux)
    return sa @ v, [sa]


def t_scaled_dot_prod_attn_bkwd3(dloss_dx, acts, qkv, mask, train=True, p_gen_aux=None):
    """acts = [dropped probabilities] as returned by t_scaled_dot_prod_attn_fwd3."""
    q, k, v = torch.unbind(qkv, dim=2)
    scale = 1.0 / math.sqrt(q.shape[-1])
    sa = acts[0]
    dv = sa.transpose(-2, -1) @ dloss_dx
    dsa = dloss_dx @ v.transpose(-2, -1)
    s = (q @ k.transpose(-2, -1)) * scale
    s = torch.where(mask.unsqueeze(1), s, torch.full_like(s, -1e9))
    p = torch.softmax(s, dim=-1)
    dp = t_dropout_bkwd2(dsa, p, train, p_gen_aux) * p
    ds = t_log_softmax_bkwd2(dp, s)
    ds = torch.where(mask.unsqueeze(1), ds, torch.zeros_like(ds))
    return (ds @ k) * scale, (ds.transpose(-2, -1) @ q) * scale, dv


def t_tlayer_ffn_fwd(layer_params, x, activation_fn):
    h = activation_fn(t_linear_fwd(layer_params[:2], x))
    return t_linear_fwd(layer_params[2:4], h)


def t_avg_cross_entropy_loss(y_labels, x_logits):
    y = y_labels.reshape(-1).to(torch.int64)
    lp = t_log_softmax_fwd(x_logits.reshape(y.numel(), -1)).gather(1, y[:, None])[:, 0]
    lp = torch.where(y != 0, lp, torch.full_like(lp, float("nan")))
    return -torch.nanmean(lp), torch.count_nonzero(y_labels)


def t_avg_cross_entropy_loss_bkwd3(y_labels, x_logits):
    shape = x_logits.shape
    y = y_labels.reshape(-1, 1).to(torch.int64)
    x = x_logits.reshape(y.numel(), -1)
    cnt = torch.count_nonzero(y)
    loss, _ = t_avg_cross_entropy_loss(y_labels, x_logits)
    d = torch.softmax(x, dim=-1)
    d.scatter_add_(1, y, -torch.ones_like(y, dtype=d.dtype))
    d = torch.where(y != 0, d / cnt, torch.zeros_like(d))
    return loss, cnt, d.reshape(shape)


def accuracy(y_labels, x_logits):
    """loss_and_optimizer_triton.py:199-200."""
    hit = (y_labels == x_logits.argmax(dim=-1)).to(torch.float32)
    return torch.nanmean(torch.where(y_labels != 0, hit, torch.full_like(hit, float("nan"))))
