"""GPU parity of the composite GPT-2 forward/backward (the reference's fwd3_t / bkwd3_t call
chain on the HIP kernels) against the CPU oracle (functional model + autograd, fp64) on the
same seeded parameters and tokens.  Metric: per-tensor relative L2 error
||g - g_ref|| / ||g_ref||; bars: fp32 storage 1e-5 on the loss and 5e-5 on gradients (1e-5
per kernel, compounded over the depth of the model), bf16 storage 2e-2."""
import math

import pytest
import torch

from oracle import gpt2 as ogpt2
from util import f64, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"


def to_dev(params, dtype):
    return [[p.to(dtype).to(DEV) for p in grp] for grp in params]


def to64(params, dtype):
    return [[p.to(dtype).to(torch.float64) for p in grp] for grp in params]


def run_case(lo, V, D, L, H, F, T, B, dtype, train, seed=0, pad=True, mask_as="tensor"):
    params = ogpt2.init_transformer_gpt2(V, D, L, H, F, T, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    # make biases / layernorm parameters non-trivial so their gradients are exercised
    for grp in params:
        for i, p in enumerate(grp):
            if p.dim() == 1:
                grp[i] = p + 0.05 * torch.randn(p.shape, generator=g)
    y = torch.randint(0, V, (B, T + 1), generator=g)
    if pad:
        y[0, -5:] = 0                                    # padded tail: labels ignored by the loss
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T).contiguous()
    seeds = [1000 + 17 * i for i in range(1 + 3 * L)]
    dmask = mask.to(DEV) if mask_as == "tensor" else None         # None: the index-masked causal path
    grads, (loss, acc, frac) = lo.t_loss_bkwd3_t(to_dev(params, dtype), y.to(DEV), dmask, None, train, seeds)
    want_g, (wl, wacc, wfrac) = ogpt2.grad_loss(to64(params, dtype), y, mask, train, seeds)
    return grads, loss, acc, frac, want_g, wl, wacc, wfrac


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("train", [False, True])
@pytest.mark.parametrize("mask_as", ["tensor", "none"])
def test_small_model_grads(lo, dtype, train, mask_as):
    grads, loss, acc, frac, want_g, wl, wacc, wfrac = run_case(lo, V=331, D=128, L=2, H=2, F=256, T=128, B=2,
                                                               dtype=dtype, train=train, mask_as=mask_as)
    ltol, gtol = (1e-5, 5e-5) if dtype == torch.float32 else (5e-3, 2e-2)
    assert abs(loss.item() - wl.item()) <= ltol * abs(wl.item()), (loss.item(), wl.item())
    assert abs(frac.item() - wfrac.item()) < 1e-6
    worst = 0.0
    for gi, (gg, wg) in enumerate(zip(grads, want_g)):
        assert len(gg) == len(wg)
        for pi, (a, b) in enumerate(zip(gg, wg)):
            assert a.shape == b.shape, (gi, pi, a.shape, b.shape)
            e = rel_l2(a, b)
            worst = max(worst, e)
            assert e <= gtol, "grad[%d][%d] rel L2 %.3e" % (gi, pi, e)
    if dtype == torch.float32:
        assert abs(acc.item() - wacc.item()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("train", [False, True])
def test_small_model_grads_head_size_32(lo, dtype, train):
    """Head size 32 (the reference's two-layer test model, tests/test_fwd3_t.ipynb cell 0: D64, H2)
    through the composite forward and backward: the attention wrappers run it on zero-padded heads."""
    grads, loss, acc, frac, want_g, wl, wacc, wfrac = run_case(lo, V=128, D=64, L=2, H=2, F=256, T=128, B=2,
                                                               dtype=dtype, train=train, seed=7)
    ltol, gtol = (1e-5, 5e-5) if dtype == torch.float32 else (5e-3, 2e-2)
    assert abs(loss.item() - wl.item()) <= ltol * abs(wl.item()), (loss.item(), wl.item())
    for gi, (gg, wg) in enumerate(zip(grads, want_g)):
        for pi, (a, b) in enumerate(zip(gg, wg)):
            assert a.shape == b.shape, (gi, pi, a.shape, b.shape)
            assert rel_l2(a, b) <= gtol, "grad[%d][%d] rel L2 %.3e" % (gi, pi, rel_l2(a, b))


def test_gpt2_small_config1_fp32(lo):
    # BASELINE config 1: full GPT-2 small, fp32, B=2, T=256, dropout off (eval semantics, x0.9)
    grads, loss, acc, frac, want_g, wl, wacc, wfrac = run_case(lo, V=50257, D=768, L=12, H=12, F=3072, T=256, B=2,
                                                               dtype=torch.float32, train=False, seed=1234, pad=False,
                                                               mask_as="none")
    assert abs(loss.item() - wl.item()) <= 1e-5 * abs(wl.item()), (loss.item(), wl.item())
    worst = 0.0
    for gi, (gg, wg) in enumerate(zip(grads, want_g)):
        for pi, (a, b) in enumerate(zip(gg, wg)):
            e = rel_l2(a, b)
            worst = max(worst, e)
            assert e <= 5e-5, "grad[%d][%d] rel L2 %.3e" % (gi, pi, e)
    print("config1 fp32: loss %.6f (oracle %.6f), worst grad rel L2 %.2e" % (loss.item(), wl.item(), worst))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_loss_curve_short_run(lo, dtype):
    """A short synthetic training run (dropout on, AdamW every step, a fresh batch of learnable sequences per step) on
    the HIP path next to the same run in the oracle (fp64 autograd + its AdamW, identical
    Philox seeds).  Bars on the per-step loss: 1e-4 relative for fp32 storage (the 1e-5
    per-step bar compounded over the steps), 2e-2 for bf16 compute on fp32 master weights."""
    V, D, L, H, F, T, B, steps = 331, 128, 2, 2, 256, 128, 4, 20
    lr, betas, eps, wd = 3e-3, (0.9, 0.95), 1e-8, 0.1
    params = ogpt2.init_transformer_gpt2(V, D, L, H, F, T, seed=7)
    wd_mask = [[p.dim() > 1 for p in grp] for grp in params]
    g = torch.Generator().manual_seed(8)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T).contiguous()
    master = [[p.clone().to(DEV) for p in grp] for grp in params]
    shadow = None if dtype == torch.float32 else to_dev(params, dtype)
    _, moments = lo.init_adam_w(master)
    o_params = [[p.double() for p in grp] for grp in params]
    o_mom = [[[torch.zeros_like(p) for p in grp] for grp in o_params] for _ in range(2)]
    got, want = [], []
    for i in range(steps):
        # learnable data: arithmetic token sequences with a random start and stride
        start = torch.randint(1, V, (B, 1), generator=g)
        stride = torch.randint(1, 4, (B, 1), generator=g)
        y = 1 + (start + stride * torch.arange(T + 1)[None, :]) % (V - 1)
        seeds = [5000 + 101 * i + j for j in range(1 + 3 * L)]
        compute = master if shadow is None else shadow
        grads, (loss, _, _) = lo.t_loss_bkwd3_t(compute, y.to(DEV), mask.to(DEV), None, True, seeds)
        lo.adam_w_in_place(master, grads, lr, betas, eps, moments, i, wd, wd_mask, shadow=shadow)
        # the oracle computes in the storage dtype's values: for bf16 it sees the rounded weights
        o_compute = o_params if shadow is None else [[p.to(dtype).double() for p in grp] for grp in o_params]
        o_grads, (o_loss, _, _) = ogpt2.grad_loss(o_compute, y, mask, True, seeds)
        o_params, o_mom = ogpt2.adam_w(o_params, o_grads, lr, betas, eps, o_mom, i, wd, wd_mask)
        got.append(loss.item())
        want.append(o_loss.item())
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    worst = max(abs(a - b) / abs(b) for a, b in zip(got, want))
    print("loss curve (%s): hip %s\n             oracle %s\nworst rel diff %.2e" %
          (dtype, ["%.4f" % x for x in got], ["%.4f" % x for x in want], worst))
    assert want[-1] < want[0] - 0.2, "the run must actually learn: %s" % want
    assert worst <= tol, (got, want)
