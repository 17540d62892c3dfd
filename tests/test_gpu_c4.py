"""BASELINE configuration 4 at its own size: x[8192,768] times the tied table W[50257,768]
(+ bias) into the row-padded logits buffer, then the fused log-softmax / mean cross-entropy
forward and backward, in fp32 and in bf16.

The fp64 checks run on a slice (every 32nd row: 256 rows that fall into every tile row of the
product); what covers all 8192 rows is size-independent: the loss against the library's
cross_entropy on the kernel's own logits, sum_v dlogits = 0 per row, exact zero rows for
label 0, the argmax attaining the row maximum, and the bias gradient against the column sums
of the stored gradient."""
import pytest
import torch
import torch.nn.functional as F

from oracle import ops
from util import DTYPES, f64, gen, randn
from util import gemm_bound as bound_of

pytestmark = pytest.mark.gpu
DEV = "cuda"
N, D, V = 8192, 768, 50257


@pytest.mark.parametrize("dtype", DTYPES)
def test_c4_lm_head_and_cross_entropy_at_8192_rows(mt, lo, dtype):
    g = gen(1234 + 4)
    x = randn(g, N, D, dtype=dtype)
    w = randn(g, V, D, dtype=dtype, std=0.02)
    b = randn(g, V, dtype=dtype, std=0.02)
    y = torch.randint(0, V, (N,), generator=g)
    y[::97] = 0                                             # ignored positions
    xd, wd, bd, yd = x.to(DEV), w.to(DEV), b.to(DEV), y.to(DEV)

    logits = mt._padded_logits(N, V, dtype, DEV)
    assert logits.stride(0) == 50304
    mt.matmul_t(xd, wd.t(), bd, out=logits)

    # ---- the product, against fp64 on 256 rows spread over all tile rows
    rows = torch.arange(5, N, 32)
    got = f64(logits[rows.to(DEV)])
    x64, w64, b64 = f64(x[rows]), f64(w), f64(b)
    want = x64 @ w64.t() + b64
    scale = x64.abs() @ w64.abs().t() + b64.abs()
    ratio = ((got - want).abs() / bound_of(want, scale, dtype)).max().item()
    assert ratio <= 1.0, "LM-head product: max err/bound %.3f" % ratio

    # ---- loss pass (out of place, so the logits stay for the checks)
    if dtype == torch.bfloat16:
        loss, cnt, dx, pred, sums = lo.t_avg_cross_entropy_loss_bkwd3_t(yd, logits, want_pred=True, want_colsum=True)
    else:
        loss, cnt, dx, pred = lo.t_avg_cross_entropy_loss_bkwd3_t(yd, logits, want_pred=True)
    n_kept = int((y != 0).sum())
    assert cnt.item() == n_kept and dx.shape == (N, V) and dx.dtype == dtype

    # loss over all rows: the library routine in fp64 on the kernel's own logits, in row chunks
    total = 0.0
    for r0 in range(0, N, 1024):
        total += F.cross_entropy(logits[r0:r0 + 1024].double(), yd[r0:r0 + 1024], ignore_index=0, reduction="sum").item()
    want_loss = total / n_kept
    assert abs(loss.item() - want_loss) <= 1e-5 * want_loss, (loss.item(), want_loss)

    # gradient rows of the slice against the oracle (its mean is over the slice's own kept rows)
    wl, wc, wdx = ops.avg_cross_entropy_loss_bkwd3(y[rows], got)
    wdx = wdx * (wc.item() / n_kept)
    err = (f64(dx[rows.to(DEV)]) - wdx).abs()
    tol = (1e-5 if dtype == torch.float32 else 2.0 ** -8) * wdx.abs() + 1e-12
    assert not (err > tol).any(), (err / tol).max().item()

    # every row: the gradient sums to zero, rows with label 0 are exactly zero
    rsum = dx.double().sum(1).abs().max().item()
    assert rsum <= (1e-5 if dtype == torch.float32 else 2.0 ** -8) / n_kept, rsum
    assert not dx[yd == 0].any().item()
    assert dx[yd != 0].abs().sum(1).min().item() > 0
    # the reported argmax attains the row maximum
    assert torch.equal(logits.gather(1, pred.view(-1, 1))[:, 0], logits.max(dim=1).values)

    if dtype == torch.bfloat16:
        ref = dx.double().sum(0)
        mag = dx.double().abs().sum(0)
        assert ((sums.double() - ref).abs() <= 2.0 ** -8 * ref.abs() + 1e-6 * mag + 1e-12).all()
