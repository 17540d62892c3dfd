"""GPU checks of the boundary functions beyond the single-kernel wrappers: the
feed-forward VJP without saved activations (the reference's tests/test_t_tlayer_ffn_bkwd.py
shape and tolerances, against autograd of the oracle's feed-forward), gradient accumulation
over micro-steps, and the gradient-norm helpers."""
import math

import pytest
import torch

from oracle import gpt2 as ogpt2
from util import f64, gen, randn, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ffn_bkwd2_reference_test_shape(mt, dtype):
    BS, N, D = 8, 512, 768
    F = 4 * D
    g = gen(3)
    x = randn(g, BS, N, D, dtype=dtype)
    dy = randn(g, BS, N, D, dtype=dtype)
    p = (randn(g, F, D, dtype=dtype, std=0.02), randn(g, F, dtype=dtype, std=0.02),
         randn(g, D, F, dtype=dtype, std=0.02), randn(g, D, dtype=dtype, std=0.02))
    leaves = [t.double().requires_grad_(True) for t in p]
    xr = x.double().requires_grad_(True)
    out = ogpt2.tlayer_ffn_fwd(leaves, xr)
    want = torch.autograd.grad(out, [xr] + leaves, dy.double())
    dx, dps = mt.t_tlayer_ffn_bkwd2_t(dy.to(DEV), tuple(t.to(DEV) for t in p), x.to(DEV), mt.t_gelu_fwd)
    assert dx.shape == x.shape and len(dps) == 4
    got = [dx] + list(dps)
    if dtype == torch.float32:
        # the reference's own absolute bars (tests/test_t_tlayer_ffn_bkwd.py:41-56) ...
        for a, b, atol in zip(got, want, (5e-3, 5e-3, 1e-3, 1e-3, 1e-3)):
            assert torch.allclose(f64(a), b, atol=atol, rtol=1e-7)
    # ... and the relative bars of this build
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for a, b, name in zip(got, want, ("dx", "dW1", "db1", "dW2", "db2")):
        assert a.shape == b.shape, name
        assert rel_l2(a, b) <= tol, (name, rel_l2(a, b))


def test_acc_grad_loss3_t_accumulates_micro_steps(lo):
    V, D, L, H, F, T, B = 211, 128, 2, 2, 256, 64, 2
    params = ogpt2.init_transformer_gpt2(V, D, L, H, F, T, seed=5)
    dparams = [[p.to(DEV) for p in grp] for grp in params]
    acc, moments = lo.init_adam_w(dparams)
    g = torch.Generator().manual_seed(6)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T).contiguous().to(DEV)
    ys = [torch.randint(1, V, (B, T + 1), generator=g).to(DEV) for _ in range(2)]
    torch.manual_seed(123)                               # sample_p_gen_aux draws from the global generator
    for y in ys:
        acc, (loss, acc_val, frac) = lo.t_acc_grad_loss3_t(acc, dparams, y, mask, None)
        assert loss.shape == (1,) and math.isfinite(loss.item()) and frac.item() == 1.0
    torch.manual_seed(123)
    want = None
    for y in ys:
        seeds = lo.sample_p_gen_aux(dparams)
        grads, _ = lo.t_loss_bkwd3_t(dparams, y, mask, None, train=True, p_gen_aux=seeds)
        want = grads if want is None else [[a + b for a, b in zip(ga, gb)] for ga, gb in zip(want, grads)]
    for ga, gw in zip(acc, want):
        for a, w in zip(ga, gw):
            assert torch.equal(a, w.reshape(a.shape))
    # norms: python floats, equal to the norm of the concatenated gradient
    flat = torch.cat([a.double().flatten() for grp in acc for a in grp])
    assert lo.grads_l2norm(acc) == pytest.approx(flat.norm().item(), rel=1e-5)
    per = lo.grads_grps_l2norms(acc)
    assert len(per) == len(acc) and per[0] == pytest.approx(
        torch.cat([a.double().flatten() for a in acc[0]]).norm().item(), rel=1e-5)
