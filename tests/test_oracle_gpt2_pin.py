"""Pins oracle/gpt2.py (forward_gpt2, tlayer_*, loss_fn, grad_loss) -- the checker behind
every full-model parity figure -- against a rebuild of the model from torch library routines
(tests/golden/make_gpt2_tiny.py) and against the tensors that rebuild committed
(tests/golden/gpt2_tiny_v1.npz).  Four structural mistakes are switched on in the rebuild to
show that the comparison notices each of them; train mode is pinned by a second rebuild that
applies the Philox keep masks (themselves pinned by the Triton package's values) by hand."""
import importlib.util
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gpt2, ops, philox

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_gpt2_tiny", os.path.join(HERE, "golden", "make_gpt2_tiny.py"))
tiny = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(tiny)

TOL = 1e-10


def _mask(B, T):
    return torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T)


def _flat(nest):
    return [t for grp in nest for t in grp]


def _rel(a, b):
    return ((a - b).norm() / b.norm().clamp_min(1e-300)).item()


@pytest.fixture(scope="module")
def fx():
    with np.load(os.path.join(HERE, "golden", "gpt2_tiny_v1.npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _fixture_params(fx):
    shapes = tiny.tiny_params()
    it = iter(range(10 ** 6))
    return [[torch.from_numpy(fx["param_%02d" % next(it)]) for _ in grp] for grp in shapes]


def test_oracle_eval_forward_loss_and_gradients_equal_committed_library_values(fx):
    params = _fixture_params(fx)
    y = torch.from_numpy(fx["y"])
    mask = _mask(tiny.B, tiny.T)
    logits = gpt2.forward_gpt2(params, y[:, :-1], mask, False)
    assert _rel(logits, torch.from_numpy(fx["logits"])) < TOL
    grads, (loss, acc, frac) = gpt2.grad_loss(params, y, mask, False)
    assert abs(loss.item() - float(fx["loss"])) < TOL
    assert frac.item() == pytest.approx((2 * tiny.T - 2) / (2 * tiny.T))        # two pad labels
    for i, g in enumerate(_flat(grads)):
        assert _rel(g, torch.from_numpy(fx["grad_%02d" % i])) < 1e-9, i


def test_library_rebuild_still_reproduces_the_fixture(fx):
    logits, loss, grads = tiny.library_loss_and_grads(tiny.tiny_params(), tiny.tiny_tokens())
    assert _rel(logits, torch.from_numpy(fx["logits"])) < 1e-12
    for i, g in enumerate(grads):
        assert _rel(g, torch.from_numpy(fx["grad_%02d" % i])) < 1e-10, i


@pytest.mark.parametrize("flag", ["scale_emb", "pre_norm", "add_pos", "head_transpose"])
def test_comparison_notices_structural_mistakes(fx, flag):
    """The same comparison with one mistake in the library rebuild: no sqrt(D) embedding scale,
    post-norm blocks, no positional add, heads merged without the transpose.  Each moves the
    logits and the gradients far outside the tolerance the oracle is held to."""
    params, y = tiny.tiny_params(), tiny.tiny_tokens()
    mask = _mask(tiny.B, tiny.T)
    logits_m, loss_m, grads_m = tiny.library_loss_and_grads(params, y, **{flag: False})
    logits = gpt2.forward_gpt2(params, y[:, :-1], mask, False)
    grads, (loss, _, _) = gpt2.grad_loss(params, y, mask, False)
    assert _rel(logits, logits_m) > 1e-3
    assert abs(loss.item() - loss_m.item()) > 1e-4
    assert max(_rel(g, gm) for g, gm in zip(_flat(grads), grads_m)) > 1e-3


def _train_forward_by_hand(params, y_in, seeds):
    """Train-mode forward, one sequence at a time, dropout applied with explicitly indexed
    keep masks: row-wise masks are addressed (seed + flattened row, column) with rows counted
    over [B,T] (model_triton.py:1486-1505), attention masks (seed + b*H + h, q + k) (:688)."""
    wemb, bemb = params[0]
    Bn, T = y_in.shape
    D = wemb.shape[1]
    H = params[2][2].shape[0]

    def drop_rows(x, b, seed):
        keep = philox.tl_rand(np.int64(seed) + np.arange(b * T, (b + 1) * T, dtype=np.int64)[:, None],
                              np.arange(x.shape[-1], dtype=np.int64)[None, :]) > np.float32(0.1)
        return x * torch.from_numpy(keep)

    out = []
    for b in range(Bn):
        x = drop_rows(F.embedding(y_in[b], wemb) * math.sqrt(D) + params[1][0][:T], b, seeds[0])
        for li, (ln1g, ln1b, wqkv, wo, ln2g, ln2b, w1, b1, w2, b2) in enumerate(params[2:-1]):
            s_attn, s_post, s_ffn = seeds[1 + 3 * li:4 + 3 * li]
            h = tiny._ln(ln1g, ln1b, x)
            heads = []
            for hd in range(H):
                q, k, v = (F.linear(h, wqkv[hd, c]) for c in range(3))
                s = (q @ k.t()) / math.sqrt(q.shape[-1])
                s = s.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), float("-inf"))
                qi, ki = np.meshgrid(np.arange(T), np.arange(T), indexing="ij")
                keep = philox.tl_rand(np.int64(s_attn + b * H + hd), qi + ki) > np.float32(0.1)
                heads.append((F.softmax(s, dim=-1) * torch.from_numpy(keep)) @ v)
            x = x + drop_rows(F.linear(torch.cat(heads, -1), wo), b, s_post)
            h = tiny._ln(ln2g, ln2b, x)
            x = x + drop_rows(F.linear(F.gelu(F.linear(h, w1, b1), approximate="tanh"), w2, b2), b, s_ffn)
        out.append(F.linear(tiny._ln(params[-1][0], params[-1][1], x), wemb, bemb))
    return torch.stack(out)


def test_oracle_train_mode_equals_hand_masked_library_rebuild():
    params, y = tiny.tiny_params(), tiny.tiny_tokens()
    seeds = [31, 977, 12345, 999999, 5, (1 << 32) + 7, 424242]
    mask = _mask(tiny.B, tiny.T)
    leaves = [[t.clone().requires_grad_(True) for t in grp] for grp in params]
    logits = _train_forward_by_hand(leaves, y[:, :-1], seeds)
    loss = F.cross_entropy(logits.reshape(-1, tiny.V), y[:, 1:].reshape(-1), ignore_index=0)
    want = torch.autograd.grad(loss, _flat(leaves))
    got_logits = gpt2.forward_gpt2(params, y[:, :-1], mask, True, seeds)
    assert _rel(got_logits, logits.detach()) < TOL
    grads, (got_loss, _, _) = gpt2.grad_loss(params, y, mask, True, seeds)
    assert abs(got_loss.item() - loss.item()) < TOL
    for i, (g, w) in enumerate(zip(_flat(grads), want)):
        assert _rel(g, w) < 1e-9, i
    # dropout really acted: train differs from eval
    assert _rel(got_logits, gpt2.forward_gpt2(params, y[:, :-1], mask, False)) > 1e-2


def test_accuracy_and_pad_handling_against_library_routines():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(3, 7, 19, generator=g, dtype=torch.float64)
    y = torch.randint(0, 19, (3, 7), generator=g)
    y[0, :3] = 0
    pred = logits.argmax(-1)
    keep = y != 0
    assert ops.accuracy(y, logits).item() == pytest.approx((pred[keep] == y[keep]).double().mean().item())
