"""CPU restatement of the reference's functional GPT-2 (torch.func mode) and its
loss.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows model_torch_func.py:12-46 (parameter layout and init scales), :50-135
(ops, block, model) and loss_and_optimizer_triton.py:20-32,199-200,221-229.
Differences, all deliberate and stated:
  * the batch/head ``torch.vmap`` of the reference (:84,:135) is written as plain
    batched tensor ops (same arithmetic);
  * train-mode dropout uses the Philox masks of the Triton path
    (model_triton.py:1460-1468) driven by ``p_gen_aux`` instead of
    ``torch.bernoulli`` on the global generator (:98-102), so that train-mode
    results are reproducible and comparable bit-for-bit in the mask;
  * the positional table is sliced to the sequence length (identical to the
    reference whenever T equals the table length, model_torch_func.py:121).
"""
import math

import torch

from . import ops

INIT_SCALE = 2e-2  # model_torch_func.py:3


def init_transformer_gpt2(vocab_size, emb_dim, layers, num_heads, ffn_dim, seq_len, seed=0,
                          dtype=torch.float32):
    """Parameter nest of model_torch_func.py:36-43, drawn from a seeded CPU generator."""
    g = torch.Generator(device="cpu").manual_seed(seed)

    def rn(*shape, scale=INIT_SCALE):
        return (scale * torch.randn(*shape, generator=g, dtype=torch.float32)).to(dtype)

    res = INIT_SCALE / math.sqrt(2 * layers)
    dh = emb_dim // num_heads
    params = [[rn(vocab_size, emb_dim), torch.zeros(vocab_size, dtype=dtype)],
              [rn(seq_len, emb_dim)]]
    for _ in range(layers):
        params.append([
            torch.ones(emb_dim, dtype=dtype), torch.zeros(emb_dim, dtype=dtype),
            rn(num_heads, 3, dh, emb_dim), rn(emb_dim, emb_dim, scale=res),
            torch.ones(emb_dim, dtype=dtype), torch.zeros(emb_dim, dtype=dtype),
            rn(ffn_dim, emb_dim), torch.zeros(ffn_dim, dtype=dtype),
            rn(emb_dim, ffn_dim, scale=res), torch.zeros(emb_dim, dtype=dtype)])
    params.append([torch.ones(emb_dim, dtype=dtype), torch.zeros(emb_dim, dtype=dtype)])
    return params


def tlayer_attn_fwd(layer_params, x, mask, train, seed):
    """model_torch_func.py:80-90 (+ :70-78).  layer_params = (Wqkv[H,3,dh,D], Wo[D,D])."""
    wqkv, wo = layer_params
    B, T, D = x.shape
    H = wqkv.shape[0]
    # proj_qkv[b,h,c,t,:] = x[b,t,:] @ wqkv[h,c].T
    qkv = torch.einsum("btd,hced->bhcte", x, wqkv)
    o = ops.scaled_dot_prod_attn_fwd(qkv, mask, train, seed)          # [B,H,T,dh]
    o = o.transpose(1, 2).reshape(B, T, D)                            # concat heads (:89)
    return torch.matmul(o, wo.t())


def tlayer_ffn_fwd(layer_params, x):
    """model_torch_func.py:92-96 with gelu."""
    w1, b1, w2, b2 = layer_params
    h = ops.gelu(torch.matmul(x, w1.t()) + b1)
    return torch.matmul(h, w2.t()) + b2


def tlayer_fwd_gpt2(lp, y, mask, train, seeds):
    """model_torch_func.py:110-117; seeds = [attn-prob, post-attn, post-ffn]
    (model_triton.py:2214-2222)."""
    yd = ops.layernorm_fwd(lp[:2], y)
    y = y + ops.dropout(tlayer_attn_fwd(lp[2:4], yd, mask, train, seeds[0]), train, seeds[1])
    yd = ops.layernorm_fwd(lp[4:6], y)
    y = y + ops.dropout(tlayer_ffn_fwd(lp[6:], yd), train, seeds[2])
    return y


def forward_gpt2(params, y, mask, train, p_gen_aux=None):
    """model_torch_func.py:119-133 batched: y int [B,T] -> logits [B,T,V]."""
    L = len(params) - 3
    if not train:
        p_gen_aux = [0] * (1 + 3 * L)
    wemb, bemb = params[0]
    T = y.shape[1]
    h = wemb[y] * math.sqrt(wemb.shape[1])
    h = ops.dropout(h + params[1][0][:T], train, p_gen_aux[0])
    for i, lp in enumerate(params[2:-1]):
        h = tlayer_fwd_gpt2(lp, h, mask, train, p_gen_aux[1 + 3 * i:4 + 3 * i])
    h = ops.layernorm_fwd(params[-1], h)
    return torch.matmul(h, wemb.t()) + bemb


def loss_fn(params, y, mask, train, p_gen_aux=None):
    """loss_and_optimizer_triton.py:221-229: y [B,T+1]; returns (loss, (loss, acc, frac))."""
    y_in, y_out = y[:, :-1], y[:, 1:]
    logits = forward_gpt2(params, y_in, mask, train, p_gen_aux)
    loss, cnt = ops.avg_cross_entropy_loss(y_out, logits)
    acc = ops.accuracy(y_out, logits)
    return loss, (loss, acc, cnt / y_out.numel())


def grad_loss(params, y, mask, train, p_gen_aux=None):
    """torch.func.grad(loss_train) of loss_and_optimizer_triton.py:234 via autograd.
    Returns (grads nest, aux)."""
    leaves = [[p.detach().clone().requires_grad_(True) for p in grp] for grp in params]
    loss, aux = loss_fn(leaves, y, mask, train, p_gen_aux)
    flat = [p for grp in leaves for p in grp]
    gs = torch.autograd.grad(loss, flat, allow_unused=True)
    it = iter(gs)
    grads = [[(next(it)) for _ in grp] for grp in leaves]
    grads = [[torch.zeros_like(p) if g is None else g for g, p in zip(gg, pg)]
             for gg, pg in zip(grads, leaves)]
    return grads, tuple(a.detach() for a in aux)


def adam_w(params, grads, lr, betas, eps, moments, i, weight_decay=0.0, weight_decay_mask=None):
    """loss_and_optimizer_triton.py:376-401 (t = i+1; decoupled decay scaled by lr)."""
    t = i + 1
    for b, mom, pw in zip(betas, moments, (1, 2)):
        for gi, grp in enumerate(grads):
            for pi, g in enumerate(grp):
                mom[gi][pi] = mom[gi][pi] * b + (1 - b) * g ** pw
    for gi, grp in enumerate(grads):
        for pi, _ in enumerate(grp):
            m = moments[0][gi][pi] / (1 - betas[0] ** t)
            v = moments[1][gi][pi] / (1 - betas[1] ** t)
            wd = weight_decay if (weight_decay_mask is None or weight_decay_mask[gi][pi]) else 0.0
            p = params[gi][pi]
            params[gi][pi] = p + (-lr * (m / (torch.sqrt(v) + eps) + wd * p))
    return params, moments
