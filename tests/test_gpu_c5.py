"""BASELINE config 5 at its real size on the GPU: full GPT-2 small (12 x 768, 12 heads, MLP
3072, vocab 50257, context 1024), bf16 storage with fp32 master weights, dropout 0.1 in
train mode, AdamW (lr 6e-4, betas 0.9/0.95, wd 0.1).

* one forward+backward at B=2, T=1024 against the oracle's autograd on the same bf16-rounded
  weights: loss to 5e-3, every gradient tensor to 2e-2 relative L2 -- with the causal mask
  given both ways (mask=None: masked by index; a bool tensor: bit-packed on the device);
* 200 optimizer steps at B=16, T=1024 with the oracle beside it: at a few steps the oracle
  evaluates the train-mode loss of the GPU's CURRENT bf16 weights on the first 4 sequences of
  that step's batch with the same Philox seeds, next to the GPU's loss on the same 4
  sequences (an oracle forward pass over the whole batch takes 30 s on 16 host cores and a
  full oracle training step 90 s: 200 of them would take five hours), so every checked point
  is an independent comparison of the weights the run has reached.  The curve is written to
  the directory named by PTJ_TEST_OUTPUT_DIR when that is set.

The oracle runs in fp32 here (its own error, 1e-6, is far below the bf16 bars; fp64 would
double its memory: the [B,H,T,T] probabilities of 12 layers are kept for autograd)."""
import json
import math
import os
import sys
import time

import pytest
import torch

from oracle import gpt2 as ogpt2
from oracle import ops as oracle_ops
from util import rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda"
CFG = dict(V=50257, D=768, L=12, H=12, F=3072, T=1024)


def say(msg):
    print(msg)
    sys.stdout.flush()


def init_params(seed):
    c = CFG
    params = ogpt2.init_transformer_gpt2(c["V"], c["D"], c["L"], c["H"], c["F"], c["T"], seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    for grp in params:                                   # non-trivial gains, shifts and biases
        for i, p in enumerate(grp):
            if p.dim() == 1:
                grp[i] = p + 0.02 * torch.randn(p.shape, generator=g)
    return params


def test_c5_one_step_b2_t1024_bf16_train_vs_oracle(lo):
    c = CFG
    B, T, L = 2, c["T"], c["L"]
    params = init_params(55)
    g = torch.Generator().manual_seed(56)
    y = torch.randint(0, c["V"], (B, T + 1), generator=g)
    y[1, -7:] = 0                                        # a padded tail: labels the loss ignores
    seeds = [777 + 13 * i for i in range(1 + 3 * L)]
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T).contiguous()
    bf = [[p.to(torch.bfloat16) for p in grp] for grp in params]
    t0 = time.time()
    want_g, (wl, wacc, wfrac) = ogpt2.grad_loss([[p.float() for p in grp] for grp in bf], y, mask, True, seeds)
    say("oracle fwd+bwd B2 T1024 fp32: %.1f s, loss %.5f" % (time.time() - t0, wl.item()))
    # Two gradient tensors are column sums with heavy cancellation at this initialisation: the
    # tied head makes every position predict its own input token with a logit near 15, which is
    # also the previous position's label, so in the head bias gradient sum_r dlogits[r, v] the
    # +p/count of one row and the -1/count of the row before cancel to about a tenth, and the
    # final norm's shift gradient sum_r dlogits[r, :] @ Wemb inherits it.  bf16 logits carry a
    # rounding error of up to 0.03 at that magnitude, i.e. 3 % of (1 - p); what the 2e-2 bar
    # can hold for such a sum is the error relative to the summed magnitudes of its terms.
    with torch.no_grad():
        f32 = [[p.float() for p in grp] for grp in bf]
        o_logits = ogpt2.forward_gpt2(f32, y[:, :-1], mask, True, seeds)
        _, _, o_dlog = oracle_ops.avg_cross_entropy_loss_bkwd3(y[:, 1:], o_logits)
        o_dlog = o_dlog.reshape(B * T, -1)
        cancel = {(0, 1): o_dlog.abs().sum(0).double().norm().item(),
                  (L + 2, 1): (o_dlog @ f32[0][0]).abs().sum(0).double().norm().item()}
        del o_logits, o_dlog
    dparams = [[p.to(DEV) for p in grp] for grp in bf]
    for mask_as in ("none", "tensor"):
        dmask = mask.to(DEV) if mask_as == "tensor" else None
        # the 2048 positions fit one pass of the LM head; the tensor-mask run takes it in two row
        # chunks instead, so that the chunked form of the head is held to the oracle as well
        chunk_rows = lo.LM_HEAD_CHUNK_ROWS
        lo.LM_HEAD_CHUNK_ROWS = 1024 if mask_as == "tensor" else chunk_rows
        try:
            grads, (loss, acc, frac) = lo.t_loss_bkwd3_t(dparams, y.to(DEV), dmask, None, True, seeds)
        finally:
            lo.LM_HEAD_CHUNK_ROWS = chunk_rows
        assert abs(loss.item() - wl.item()) <= 5e-3 * abs(wl.item()), (mask_as, loss.item(), wl.item())
        assert abs(frac.item() - wfrac.item()) < 1e-6
        worst, where = 0.0, None
        for gi, (gg, wg) in enumerate(zip(grads, want_g)):
            for pi, (a, b) in enumerate(zip(gg, wg)):
                assert a.shape == b.shape and a.dtype == torch.bfloat16
                e = rel_l2(a, b.double())
                if (gi, pi) in cancel:
                    e_terms = (a.double().cpu() - b.double()).norm().item() / cancel[(gi, pi)]
                    say("grad[%d][%d]: rel L2 %.2e of the sum, %.2e of its terms' magnitudes" % (gi, pi, e, e_terms))
                    assert e <= 6e-2 and e_terms <= 2e-2, (mask_as, gi, pi, e, e_terms)
                    continue
                if e > worst:
                    worst, where = e, (gi, pi)
                assert e <= 2e-2, "mask=%s grad[%d][%d] rel L2 %.3e" % (mask_as, gi, pi, e)
        say("mask=%s: loss %.5f (oracle %.5f), worst gradient tensor rel L2 %.2e at %s"
            % (mask_as, loss.item(), wl.item(), worst, where))


@pytest.mark.parametrize("data", ["uniform", "learnable"])
def test_c5_loss_curve_200_steps_b16_t1024(lo, data):
    """`uniform`: BASELINE's data (uniform token ids: the loss can only fall from its initial
    value to ln V); `learnable`: arithmetic token sequences, on which the loss really falls."""
    c = CFG
    B, T, L, V, steps = 16, c["T"], c["L"], c["V"], 200
    lr, betas, eps, wd = 6e-4, (0.9, 0.95), 1e-8, 0.1
    check_at = (0, 1, 199) if data == "uniform" else (0, 60, 199)
    SUB = 4
    params = init_params(91)
    wd_mask = [[p.dim() > 1 for p in grp] for grp in params]
    master = [[p.clone().to(DEV) for p in grp] for grp in params]
    shadow = [[p.to(torch.bfloat16) for p in grp] for grp in master]
    _, moments = lo.init_adam_w(master)
    g = torch.Generator().manual_seed(92)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T)
    curve, checks = [], []
    for i in range(steps):
        if data == "uniform":
            y = torch.randint(0, V, (B, T + 1), generator=g)
        else:
            start = torch.randint(1, V, (B, 1), generator=g)
            stride = torch.randint(1, 4, (B, 1), generator=g)
            y = 1 + (start + stride * torch.arange(T + 1)[None, :]) % (V - 1)
        seeds = lo.sample_p_gen_aux(master, g)
        if i in check_at:                                # the oracle on the weights this step starts from
            t0 = time.time()
            with torch.no_grad():
                cpu_w = [[p.float().cpu() for p in grp] for grp in shadow]
                want = ogpt2.loss_fn(cpu_w, y[:SUB], mask[:SUB], True, seeds)[0].item()
            _, (sub_loss, _, _) = lo.t_loss_bkwd3_t(shadow, y[:SUB].to(DEV), None, None, True, seeds)
            got = sub_loss.item()
            checks.append((i, got, want))
            say("step %d: loss on %d sequences %.5f, oracle %.5f (%.1f s), rel diff %.2e"
                % (i, SUB, got, want, time.time() - t0, abs(got - want) / abs(want)))
            assert abs(got - want) <= 5e-3 * abs(want), (i, got, want)
        grads, (loss, _, _) = lo.t_loss_bkwd3_t(shadow, y.to(DEV), None, None, True, seeds)
        lo.adam_w_in_place(master, grads, lr, betas, eps, moments, i, wd, wd_mask, shadow=shadow)
        curve.append(loss)
    curve = [x.item() for x in curve]
    assert all(math.isfinite(x) for x in curve)
    if data == "uniform":
        # at initialisation the tied head predicts each position's own input token (loss about
        # ln V + 2.4); nothing but the token frequencies can be learnt from uniform ids
        assert curve[0] > math.log(V) + 1.0 and abs(curve[-1] - math.log(V)) < 0.15
    else:
        assert curve[-1] < curve[0] - 3.0, (curve[0], curve[-1])
    out_dir = os.environ.get("PTJ_TEST_OUTPUT_DIR", "")
    if out_dir and os.path.isdir(out_dir):
        with open(os.path.join(out_dir, "loss_curve_c5_%s.json" % data), "w") as f:
            json.dump({"data": data, "steps": steps, "B": B, "T": T, "loss": curve,
                       "oracle_checks_first_%d_sequences" % SUB: [{"step": s, "hip": a, "oracle": b}
                                                                  for s, a, b in checks]}, f)
    say("%s: loss %.4f -> %.4f over %d steps; every 20th: %s"
        % (data, curve[0], curve[-1], steps, " ".join("%.3f" % x for x in curve[::20])))
