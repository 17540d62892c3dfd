"""GPU parity of the row-wise kernels (through the C ABI) against the CPU oracle.
Tolerances: fp32 rtol 1e-5 (+atol 1e-6); bf16 rtol 2e-2 (+atol 2e-3) against the fp64
oracle evaluated on the bf16-rounded inputs.  Dropout masks are compared bit-exactly."""
import pytest
import torch

from oracle import ops
from util import DTYPES, assert_close, f64, gen, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(8192, 768), (3, 5, 768), (7, 100), (33, 1000), (5, 4096), (2, 12000), (1, 2)])
def test_layernorm_fwd(mt, dtype, shape):
    g = gen(1)
    x = randn(g, *shape, dtype=dtype)
    D = shape[-1]
    gamma, beta = randn(g, D, dtype=dtype, mean=1.0, std=0.1), randn(g, D, dtype=dtype, std=0.1)
    y = mt.t_layernorm_fwd_t((gamma.to(DEV), beta.to(DEV)), x.to(DEV))
    assert y.shape == x.shape and y.dtype == dtype
    want = ops.layernorm_fwd((f64(gamma), f64(beta)), f64(x))
    # D=2 rows have |xhat| = 1/sqrt(2) exactly; generic tolerance is fine
    assert_close(y, want, dtype, what="layernorm_fwd")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(8192, 768), (4, 6, 768), (7, 100), (300, 1000), (5, 4096)])
def test_layernorm_bwd(mt, dtype, shape):
    g = gen(2)
    x, dy = randn(g, *shape, dtype=dtype), randn(g, *shape, dtype=dtype)
    D = shape[-1]
    gamma, beta = randn(g, D, dtype=dtype, mean=1.0, std=0.1), randn(g, D, dtype=dtype, std=0.1)
    p = (gamma.to(DEV), beta.to(DEV))
    dx = mt.t_layernorm_bkwd2_x_t(dy.to(DEV), p, x.to(DEV))
    dg, db = mt.t_layernorm_bkwd2_p_t(dy.to(DEV), p, x.to(DEV))
    dx2, (dg2, db2) = mt.layernorm_bkwd2_t(dy.to(DEV), p, x.to(DEV))
    want_dx = ops.layernorm_bkwd2_x(f64(dy), (f64(gamma),), f64(x))
    want_dg, want_db = ops.layernorm_bkwd2_p(f64(dy), None, f64(x))
    rows = x.numel() // D
    # dx: cancellation of three terms of size ~|g|; atol scaled to the terms
    assert_close(dx, want_dx, dtype, atol=2e-5 if dtype == torch.float32 else 3e-2, what="ln dx")
    # column sums over `rows` terms of size ~1: absolute error grows like sqrt(rows)*eps
    a = (3e-6 if dtype == torch.float32 else 8e-3) * max(1.0, rows ** 0.5)
    assert_close(dg, want_dg, dtype, atol=a, what="ln dgamma")
    assert_close(db, want_db, dtype, atol=a, what="ln dbeta")
    assert torch.equal(dx, dx2) and torch.equal(dg, dg2) and torch.equal(db, db2)   # fused == separate, bitwise
    # determinism (no atomics)
    dg3, db3 = mt.t_layernorm_bkwd2_p_t(dy.to(DEV), p, x.to(DEV))
    assert torch.equal(dg, dg3) and torch.equal(db, db3)
    if dtype == torch.float32:
        # row invariants of the unbiased-std layernorm VJP
        xh = ops.layernorm_fwd((torch.ones(D, dtype=torch.float64), torch.zeros(D, dtype=torch.float64)), f64(x))
        assert f64(dx).sum(-1).abs().max() < 1e-3
        assert (f64(dx) * xh).sum(-1).abs().max() < 1e-3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(8192, 3072), (3, 1001), (0,), (5,)])
def test_gelu(mt, dtype, shape):
    g = gen(3)
    x, dy = randn(g, *shape, dtype=dtype, std=2.0), randn(g, *shape, dtype=dtype)
    y = mt.t_gelu_fwd_t(x.to(DEV))
    dx = mt.t_gelu_bkwd2_t(dy.to(DEV), x.to(DEV))
    assert y.shape == x.shape and dx.shape == x.shape
    assert_close(y, ops.gelu(f64(x)), dtype, atol=2e-6 if dtype == torch.float32 else 2e-3, what="gelu fwd")
    assert_close(dx, ops.gelu_bkwd2(f64(dy), f64(x)), dtype, atol=2e-6 if dtype == torch.float32 else 2e-3,
                 what="gelu bwd")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4096, 768), (333, 768), (64, 1024), (17, 4096), (5, 100), (3, 1001), (2, 16384)])
def test_dropout_add_layernorm_matches_separate_calls(mt, dtype, shape):
    """Residual update + LayerNorm in one pass: bit-exact against dropout_add_t followed by
    t_layernorm_fwd_t (both outputs and the recorded keep bytes), train and eval."""
    g = gen(31)
    x, res = randn(g, *shape, dtype=dtype).to(DEV), randn(g, *shape, dtype=dtype).to(DEV)
    gamma, beta = randn(g, shape[1], dtype=dtype).to(DEV), randn(g, shape[1], dtype=dtype).to(DEV)
    for train in (True, False):
        y0, keep0 = mt.dropout_add_t(x, res, train, 9191, want_keep=True)
        h0 = mt.t_layernorm_fwd_t((gamma, beta), y0)
        y1, h1, keep1 = mt.dropout_add_layernorm_t(x, res, (gamma, beta), train, 9191, want_keep=True)
        assert torch.equal(y0, y1) and torch.equal(h0, h1)
        assert (keep0 is None) == (keep1 is None)
        if keep0 is not None:
            assert torch.equal(keep0, keep1)
        y2, h2, keep2 = mt.dropout_add_layernorm_t(x, res, (gamma, beta), train, 9191)
        assert keep2 is None and torch.equal(y0, y2) and torch.equal(h0, h2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(16384, 3072), (1000, 768), (37, 101), (1, 8), (2, 3, 64)])
def test_gelu_bwd_with_colsum_matches_separate_calls(mt, dtype, shape):
    """The fused entry point writes exactly the dx of t_gelu_bkwd2_t and the column sums of
    that stored dx (compared with an fp64 sum of the rounded values)."""
    g = gen(11)
    x, dy = randn(g, *shape, dtype=dtype, std=2.0).to(DEV), randn(g, *shape, dtype=dtype).to(DEV)
    dx, sums = mt.t_gelu_bkwd2_colsum_t(dy, x)
    want = mt.t_gelu_bkwd2_t(dy, x)
    assert dx.shape == x.shape and torch.equal(dx, want)
    rows = x.numel() // shape[-1]
    ref = f64(want).reshape(rows, shape[-1]).sum(0)
    tol = (3e-6 if dtype == torch.float32 else 8e-3) * max(1.0, rows ** 0.5)
    assert (f64(sums) - ref).abs().max().item() <= tol + (0 if dtype == torch.float32 else 1e-2 * ref.abs().max().item())
    dx2, sums2 = mt.t_gelu_bkwd2_colsum_t(dy, x)
    assert torch.equal(sums, sums2) and torch.equal(dx, dx2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,seed", [((8192, 768), 42), ((2, 3, 768), 7), ((5, 100), 123456), ((3, 1001), 999999),
                                        ((4, 8), (1 << 32) + 5)])
def test_dropout_mask_bit_exact(mt, dtype, shape, seed):
    g = gen(4)
    x = randn(g, *shape, dtype=dtype).abs() + 1.0    # strictly positive so y != 0 <=> kept
    y = mt.t_dropout_fwd_t(x.to(DEV), True, seed).cpu()
    keep = ops.rowwise_keep(tuple(shape), seed)
    assert torch.equal(y != 0, keep)                  # mask bit-exact
    assert torch.equal(y[keep], x[keep])              # no rescale: values pass through bitwise
    dy = randn(g, *shape, dtype=dtype).abs() + 1.0
    d = mt.t_dropout_bkwd2_t(dy.to(DEV), x.to(DEV), True, seed).cpu()
    assert torch.equal(d != 0, keep) and torch.equal(d[keep], dy[keep])
    # eval mode: x * 0.9
    e = mt.t_dropout_fwd_t(x.to(DEV), False)
    assert_close(e, f64(x) * 0.9, dtype, what="dropout eval")
    # fused residual form
    r = randn(g, *shape, dtype=dtype)
    ya = mt.dropout_add_t(x.to(DEV), r.to(DEV), True, seed).cpu()
    assert torch.equal(ya, (r.to(torch.float32) + y.to(torch.float32)).to(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(8, 12, 64, 512), (4096, 1024), (3, 37), (2, 4096), (5, 1)])
def test_log_softmax(mt, dtype, shape):
    g = gen(5)
    x, dy = randn(g, *shape, dtype=dtype, std=3.0), randn(g, *shape, dtype=dtype)
    y = mt.t_log_softmax_fwd_t(x.to(DEV))
    dx = mt.t_log_softmax_bkwd2_t(dy.to(DEV), x.to(DEV))
    a = 1e-5 if dtype == torch.float32 else 6e-2      # |y| ~ 10: bf16 spacing there is 6e-2
    assert_close(y, ops.log_softmax(f64(x)), dtype, atol=a, what="log_softmax fwd")
    assert_close(dx, ops.log_softmax_bkwd2(f64(dy), f64(x)), dtype, atol=1e-5 if dtype == torch.float32 else 2e-2,
                 what="log_softmax bwd")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,V", [(512, 50257), (64, 35374), (33, 1000), (7, 101), (4, 70001), (1, 5)])
def test_ce_fwd_bwd(lo, dtype, rows, V):
    g = gen(6)
    x = randn(g, rows, V, dtype=dtype)
    y = torch.randint(0, V, (rows,), generator=g)
    y[::7] = 0
    if rows == 1:
        y[0] = 3
    loss, cnt, dx = lo.t_avg_cross_entropy_loss_bkwd3_t(y.to(DEV), x.to(DEV))
    wl, wc, wdx = ops.avg_cross_entropy_loss_bkwd3(y, f64(x))
    assert cnt.item() == wc.item() and cnt.dtype == torch.int64
    assert loss.shape == (1,) and loss.dtype == torch.float32
    assert abs(loss.item() - wl.item()) <= (1e-5 if dtype == torch.float32 else 1e-4) * abs(wl.item())
    assert dx.shape == x.shape and dx.dtype == dtype
    assert_close(dx, wdx, dtype, atol=1e-9 if dtype == torch.float32 else 1e-6, what="ce dlogits")
    assert torch.equal(dx.cpu()[y == 0], torch.zeros_like(x)[y == 0])
    # determinism + in-place variant
    loss2, _, dx2 = lo.t_avg_cross_entropy_loss_bkwd3_t(y.to(DEV), x.to(DEV))
    assert torch.equal(loss, loss2) and torch.equal(dx, dx2)
    xin = x.to(DEV).clone()
    loss3, _, dx3 = lo.t_avg_cross_entropy_loss_bkwd3_t(y.to(DEV), xin, inplace=True)
    assert dx3.data_ptr() == xin.data_ptr() and torch.equal(dx3, dx) and torch.equal(loss3, loss)


@pytest.mark.parametrize("rows,V,pitch", [(512, 50257, 50304), (300, 1000, 1000), (64, 35374, 35376), (5, 17, 24),
                                          (1030, 4099, 4104)])
def test_ce_with_column_sums_equals_separate_passes(lo, mt, rows, V, pitch):
    """The loss pass that also sums the gradient's columns (2-byte logits, row pitch a multiple
    of 8): loss, count, gradient and argmax bit-equal to the plain pass, and the sums equal to
    the fp64 column sums of the stored gradient within the rounding of the 2-byte result."""
    g = gen(66)
    buf = randn(g, rows, pitch, dtype=torch.bfloat16).to(DEV)
    x = buf[:, :V]
    y = torch.randint(0, V, (rows,), generator=g)
    y[::5] = 0
    y = y.to(DEV)
    loss0, cnt0, dx0, pred0 = lo.t_avg_cross_entropy_loss_bkwd3_t(y, x, want_pred=True)
    loss1, cnt1, dx1, pred1, sums = lo.t_avg_cross_entropy_loss_bkwd3_t(y, x, want_pred=True, want_colsum=True)
    assert torch.equal(loss0, loss1) and torch.equal(cnt0, cnt1) and torch.equal(pred0, pred1)
    assert torch.equal(dx0, dx1)
    want = f64(dx1).sum(0)
    assert sums.shape == (V,) and sums.dtype == torch.bfloat16
    err = (f64(sums) - want).abs()
    assert (err <= 2 ** -8 * want.abs() + 1e-9).all(), err.max().item()
    # against the two-pass form the fused call replaces (fp32 partial sums in another order)
    ref = mt.colsum_t(dx0)
    assert (f64(sums) - f64(ref)).abs().max().item() <= 2 ** -7 * want.abs().max().item() + 1e-9
    # in place, as the training step calls it; a second call gives the same bits
    xin = buf.clone()[:, :V]
    loss2, _, dx2, _, sums2 = lo.t_avg_cross_entropy_loss_bkwd3_t(y, xin, inplace=True, want_pred=True, want_colsum=True)
    assert dx2.data_ptr() == xin.data_ptr() and torch.equal(dx2, dx0) and torch.equal(sums2, sums)
    assert torch.equal(loss2, loss0)


@pytest.mark.parametrize("shift,inplace", [(3, False), (3, True), (5, True), (8, False)])
def test_ce_with_column_sums_rows_off_the_16_byte_grid(lo, mt, shift, inplace):
    """Logits whose rows start `shift` elements into 16-byte aligned, 8-element-pitched rows (a column
    slice of a wider buffer): the vectors that hold a row's two ends are stored element by element
    and the partial column sums are indexed by slot.  Against the plain pass and the fp64 sums."""
    rows, V, pitch = 300, 4099, 4112
    g = gen(67 + shift)
    buf = randn(g, rows, pitch, dtype=torch.bfloat16).to(DEV)
    x = buf[:, shift:shift + V]
    assert (x.data_ptr() % 16 != 0) == (shift % 8 != 0)
    y = torch.randint(0, V, (rows,), generator=g)
    y[::4] = 0
    y = y.to(DEV)
    loss0, cnt0, dx0, pred0 = lo.t_avg_cross_entropy_loss_bkwd3_t(y, x, want_pred=True)
    wl, wc, wdx = ops.avg_cross_entropy_loss_bkwd3(y.cpu(), f64(x))
    assert abs(loss0.item() - wl.item()) <= 1e-4 * abs(wl.item())
    assert_close(dx0, wdx, torch.bfloat16, atol=1e-6, what="ce dlogits (shifted rows)")
    xin = buf.clone()[:, shift:shift + V] if inplace else x
    keep_left, keep_right = buf[:, :shift].clone(), buf[:, shift + V:].clone()
    loss1, cnt1, dx1, pred1, sums = lo.t_avg_cross_entropy_loss_bkwd3_t(y, xin, inplace=inplace, want_pred=True,
                                                                     want_colsum=True)
    assert torch.equal(loss0, loss1) and torch.equal(cnt0, cnt1) and torch.equal(pred0, pred1) and torch.equal(dx0, dx1)
    if inplace:
        assert dx1.data_ptr() == xin.data_ptr()
    want = f64(dx1).sum(0)
    assert ((f64(sums) - want).abs() <= 2 ** -8 * want.abs() + 1e-9).all()
    # nothing outside the rows was written
    if not inplace:
        assert torch.equal(buf[:, :shift], keep_left) and torch.equal(buf[:, shift + V:], keep_right)


@pytest.mark.parametrize("dtype,pitch", [(torch.float32, 1000), (torch.bfloat16, 1003)])
def test_ce_column_sums_where_the_fused_pass_does_not_apply(lo, mt, dtype, pitch):
    """fp32 logits, or a row pitch that is not a multiple of 8: want_colsum routes to the plain pass
    plus colsum_t and returns the same values as the two calls made by hand."""
    rows, V = 130, 1000
    g = gen(68)
    x = randn(g, rows, pitch, dtype=dtype).to(DEV)[:, :V]
    y = torch.randint(0, V, (rows,), generator=g).to(DEV)
    loss0, cnt0, dx0 = lo.t_avg_cross_entropy_loss_bkwd3_t(y, x)
    loss1, cnt1, dx1, sums = lo.t_avg_cross_entropy_loss_bkwd3_t(y, x, want_colsum=True)
    assert torch.equal(loss0, loss1) and torch.equal(dx0, dx1) and torch.equal(sums, mt.colsum_t(dx0))
    want = f64(dx0).sum(0)
    tol = 1e-5 if dtype == torch.float32 else 2 ** -8
    assert ((f64(sums) - want).abs() <= tol * want.abs() + 1e-9).all()


def test_ce_all_labels_zero_is_nan(lo):
    x = torch.randn(4, 50, device=DEV)
    loss, cnt, dx = lo.t_avg_cross_entropy_loss_bkwd3_t(torch.zeros(4, dtype=torch.int64, device=DEV), x)
    assert torch.isnan(loss).all() and cnt.item() == 0 and (dx == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4096, 768), (1000, 768), (37, 768), (33, 200), (7, 2048), (3, 5000)])
def test_layernorm_bwd_with_dropout_output_matches_separate_calls(mt, dtype, shape):
    """The LayerNorm backward that also emits dropout_bkwd(dx): bit-exact against the
    LayerNorm backward followed by the dropout kernel, train and eval."""
    g = gen(21)
    dy, x, res = (randn(g, *shape, dtype=dtype).to(DEV) for _ in range(3))
    gamma, beta = randn(g, shape[1], dtype=dtype).to(DEV), randn(g, shape[1], dtype=dtype).to(DEV)
    for train in (True, False):
        dx0, (dg0, db0) = mt.layernorm_bkwd2_t(dy, (gamma, beta), x, residual=res)
        want = mt.t_dropout_bkwd2_t(dx0, None, train, 4242)
        dx1, (dg1, db1), got = mt.layernorm_bkwd2_t(dy, (gamma, beta), x, residual=res, drop=(train, 4242))
        assert torch.equal(dx0, dx1) and torch.equal(dg0, dg1) and torch.equal(db0, db1)
        assert torch.equal(got, want)
        # same again with the keep mask recorded by the forward dropout instead of recomputed
        out, keep = mt.dropout_add_t(x, res, train, 4242, want_keep=True)
        assert torch.equal(out, mt.dropout_add_t(x, res, train, 4242))
        if keep is not None:
            assert train and dtype == torch.bfloat16 and shape[1] % 8 == 0
            _, _, got2 = mt.layernorm_bkwd2_t(dy, (gamma, beta), x, residual=res, drop=(train, 4242, keep))
            assert torch.equal(got2, want)
        else:
            assert not (train and dtype == torch.bfloat16 and shape[1] % 8 == 0)
        # and with the column sums of the dropped output (a bias gradient) from the same pass
        dx3, (dg3, db3), got3, sums = mt.layernorm_bkwd2_t(dy, (gamma, beta), x, residual=res, drop=(train, 4242),
                                                           drop_sum=True)
        assert torch.equal(dx3, dx0) and torch.equal(dg3, dg0) and torch.equal(db3, db0) and torch.equal(got3, want)
        ref = f64(want).sum(0)
        rows = shape[0]
        tol = (3e-6 if dtype == torch.float32 else 8e-3) * max(1.0, rows ** 0.5)
        assert (f64(sums) - ref).abs().max().item() <= tol + (0 if dtype == torch.float32 else 1e-2 * ref.abs().max().item())
