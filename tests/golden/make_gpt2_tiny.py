"""Writes tests/golden/gpt2_tiny_v1.npz: logits, loss and every parameter gradient of a tiny
GPT-2 (V97 D32 L2 H4 F64 T16 B2, non-trivial gains, shifts and biases) in eval mode, computed in
float64 by `library_forward` below -- a per-sequence, per-head rebuild of the reference model
(model_torch_func.py:110-133) out of torch LIBRARY routines only:

  F.embedding * sqrt(D) + positions            (model_torch_func.py:54-55, :120-121)
  F.layer_norm(eps=0) * sqrt((D-1)/D)          (unbiased std without epsilon, :104-108)
  F.scaled_dot_product_attention(is_causal)    (:70-78; eval dropout scales the probabilities,
                                                hence the output, by 0.9)
  F.linear, F.gelu(approximate="tanh")         (:60-68, :92-96)
  F.cross_entropy(ignore_index=0)              (loss_and_optimizer_triton.py:26-32)
  torch.autograd                               (the torch.func.grad of :234)

It shares no code with oracle/ and imports nothing of the reference.  The flags of
`library_forward` switch on four structural mistakes (no sqrt(D) embedding scale, post-norm
instead of pre-norm, no positional add, heads merged without the transpose); the tests use
them to show that the comparison with the oracle notices each.  Run from the repository root:

    python tests/golden/make_gpt2_tiny.py
"""
import math
import os

import numpy as np
import torch
import torch.nn.functional as F

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpt2_tiny_v1.npz")
V, D, L, H, FF, T, B = 97, 32, 2, 4, 64, 16, 2
EVAL_KEEP = 0.9            # eval-mode dropout multiplies by 1 - DROPOUT_RATE (model_torch_func.py:98-100)


def tiny_params(seed=11):
    """Parameter nest of model_torch_func.py:36-43 with every tensor random (so that gains,
    shifts and biases matter), float64."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s, sc=0.2: sc * torch.randn(*s, generator=g, dtype=torch.float64)
    near1 = lambda n: 1 + 0.3 * torch.randn(n, generator=g, dtype=torch.float64)
    dh = D // H
    p = [[rn(V, D), rn(V)], [rn(T, D)]]
    for _ in range(L):
        p.append([near1(D), rn(D), rn(H, 3, dh, D), rn(D, D), near1(D), rn(D), rn(FF, D), rn(FF), rn(D, FF), rn(D)])
    p.append([near1(D), rn(D)])
    return p


def tiny_tokens(seed=12):
    g = torch.Generator().manual_seed(seed)
    y = torch.randint(1, V, (B, T + 1), generator=g)
    y[0, 5] = 0            # two ignored labels (pad id 0), one of them also an input token
    y[1, T] = 0
    return y


def _ln(gamma, beta, x):
    d = x.shape[-1]
    return F.layer_norm(x, (d,), None, None, 0.0) * math.sqrt((d - 1) / d) * gamma + beta


def library_forward(params, y_in, scale_emb=True, pre_norm=True, add_pos=True, head_transpose=True):
    """y_in int [B,T] -> logits [B,T,V], eval mode, one sequence and one head at a time."""
    wemb, bemb = params[0]
    out = []
    for b in range(y_in.shape[0]):
        x = F.embedding(y_in[b], wemb)
        if scale_emb:
            x = x * math.sqrt(D)
        if add_pos:
            x = x + params[1][0]
        x = x * EVAL_KEEP
        for ln1g, ln1b, wqkv, wo, ln2g, ln2b, w1, b1, w2, b2 in params[2:-1]:
            def attn(h):
                heads = []
                for hd in range(H):
                    q, k, v = (F.linear(h, wqkv[hd, c]) for c in range(3))
                    heads.append(F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
                                 * EVAL_KEEP)
                if head_transpose:
                    merged = torch.cat(heads, dim=-1)                              # [T, H*dh]
                else:
                    merged = torch.stack(heads, 0).reshape(T, D)                   # the mistake
                return F.linear(merged, wo) * EVAL_KEEP

            def ffn(h):
                return F.linear(F.gelu(F.linear(h, w1, b1), approximate="tanh"), w2, b2) * EVAL_KEEP

            if pre_norm:
                x = x + attn(_ln(ln1g, ln1b, x))
                x = x + ffn(_ln(ln2g, ln2b, x))
            else:
                x = _ln(ln1g, ln1b, x + attn(x))
                x = _ln(ln2g, ln2b, x + ffn(x))
        x = _ln(params[-1][0], params[-1][1], x)
        out.append(F.linear(x, wemb, bemb))
    return torch.stack(out)


def library_loss_and_grads(params, y, **flags):
    leaves = [[t.clone().requires_grad_(True) for t in grp] for grp in params]
    logits = library_forward(leaves, y[:, :-1], **flags)
    loss = F.cross_entropy(logits.reshape(-1, V), y[:, 1:].reshape(-1), ignore_index=0)
    flat = [t for grp in leaves for t in grp]
    grads = torch.autograd.grad(loss, flat, allow_unused=True)      # unused only under a mistake flag
    grads = [torch.zeros_like(t) if g is None else g for g, t in zip(grads, flat)]
    return logits.detach(), loss.detach(), grads


def main():
    params, y = tiny_params(), tiny_tokens()
    logits, loss, grads = library_loss_and_grads(params, y)
    d = {"y": y.numpy(), "logits": logits.numpy(), "loss": loss.numpy()}
    for i, t in enumerate(t for grp in params for t in grp):
        d["param_%02d" % i] = t.numpy()
    for i, g in enumerate(grads):
        d["grad_%02d" % i] = g.numpy()
    np.savez_compressed(OUT, **d)
    print("wrote", OUT, os.path.getsize(OUT), "bytes; loss", float(loss))


if __name__ == "__main__":
    main()
