"""GPU parity of the MFMA GEMM (through the C ABI) against fp64 matmul of the same inputs.

Error bound per element.  The products of two bf16 (or fp32) values are exact in the fp32
accumulator, so the only errors are the fp32 additions -- at most K * 2^-24 and typically
sqrt(K) * 2^-24 of sum_k |a_ik b_kj| -- and the rounding of the result to the storage type
(2^-9 relative for bf16).  Bound: ACC * sum_k |a_ik b_kj| + OUT * |want| with ACC = 1e-5 and
OUT = 2^-8 for bf16 storage (one rounding with a factor two of slack), 0 for fp32.  At K = 768
and N(0,1) operands that is about 0.5 % of a typical |c| = sqrt(K): a dropped 16-wide MFMA
contraction chunk (14 % of a typical element) fails it, which
test_bound_fails_when_one_contraction_chunk_is_dropped shows on the expected-value side."""
import pytest
import torch

from oracle import ops
from util import DTYPES, OUT_BF16, f64, gen, randn
from util import gemm_bound as bound_of

pytestmark = pytest.mark.gpu
DEV = "cuda"


def worst_ratio(c, a, b, dtype, bias=None, gelu=False):
    """max over elements of |c - want| / bound."""
    a64, b64 = f64(a), f64(b)
    want = a64 @ b64
    scale = a64.abs() @ b64.abs()
    if bias is not None:
        want = want + f64(bias)
        scale = scale + f64(bias).abs()
    if gelu:
        want = ops.gelu(want)        # |gelu'| <= 1.13: the accumulation error carries over times that
    assert c.shape == want.shape
    return ((f64(c) - want).abs() / bound_of(want, scale, dtype, 1.2 if gelu else 1.0)).max().item()


def check(c, a, b, dtype, bias=None, gelu=False):
    r = worst_ratio(c, a, b, dtype, bias, gelu)
    assert r <= 1.0, "max err/bound %.3f" % r


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layout", ["nt", "tn"])
def test_bound_fails_when_one_contraction_chunk_is_dropped(mt, dtype, layout):
    """The bound is tight enough to see a lost MFMA step: the kernel's result passes against the
    true product and fails against the product without contraction indices 16..31."""
    n, m, k = 512, 384, 768
    g = gen(99)
    a = randn(g, n, k, dtype=dtype) if layout[0] == "n" else randn(g, k, n, dtype=dtype).t()
    b = randn(g, k, m, dtype=dtype) if layout[1] == "n" else randn(g, m, k, dtype=dtype).t()
    ad = (a.t().contiguous().to(DEV).t() if layout[0] == "t" else a.to(DEV))
    bd = (b.t().contiguous().to(DEV).t() if layout[1] == "t" else b.to(DEV))
    c = mt.matmul_t(ad, bd)
    assert worst_ratio(c, a, b, dtype) <= 1.0
    a_cut = a.clone()
    a_cut[:, 16:32] = 0
    assert worst_ratio(c, a_cut, b, dtype) > 20.0


SHAPES = [(128, 128, 64), (256, 384, 512), (100, 37, 19), (513, 129, 65), (1, 1, 1), (64, 768, 3072),
          (33, 2, 200), (300, 50257, 64)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,m,k", SHAPES)
@pytest.mark.parametrize("layout", ["nn", "nt", "tn", "tt"])
def test_gemm_layouts(mt, dtype, n, m, k, layout):
    g = gen(n * 7 + m * 3 + k)
    a = randn(g, n, k, dtype=dtype) if layout[0] == "n" else randn(g, k, n, dtype=dtype).t()
    b = randn(g, k, m, dtype=dtype) if layout[1] == "n" else randn(g, m, k, dtype=dtype).t()
    ad = (a.t().contiguous().to(DEV).t() if layout[0] == "t" else a.to(DEV))
    bd = (b.t().contiguous().to(DEV).t() if layout[1] == "t" else b.to(DEV))
    assert ad.stride() == a.stride() and bd.stride() == b.stride()
    c = mt.matmul_t(ad, bd)
    check(c, a, b, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_bruteforce_tiny(mt, dtype):
    g = gen(5)
    a, b = randn(g, 9, 13, dtype=dtype), randn(g, 13, 6, dtype=dtype)
    c = mt.t_matmul_t(a.to(DEV), b.to(DEV))
    want = ops.matmul_bruteforce(f64(a), f64(b))
    assert torch.allclose(f64(c), want, rtol=1e-5 if dtype == torch.float32 else OUT_BF16, atol=1e-5 if dtype == torch.float32 else 1e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,m,k", [(768, 768, 16384), (2304, 768, 8192), (50257, 64, 4096), (130, 70, 5000)])
def test_gemm_split_k_dw_shapes(mt, dtype, n, m, k):
    # dW-like products: both operands contiguous along the output axes, long contraction
    g = gen(11)
    dy, x = randn(g, k, n, dtype=dtype), randn(g, k, m, dtype=dtype)
    c = mt.matmul_t(dy.to(DEV).t(), x.to(DEV))
    check(c, dy.t(), x, dtype)
    c2 = mt.matmul_t(dy.to(DEV).t(), x.to(DEV))
    assert torch.equal(c, c2)      # split-K partials are reduced in fixed order


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,m,k,layout", [(16640, 768, 2048, "tn"), (16500, 770, 2048, "nt"), (16640, 768, 4096, "nn")])
def test_gemm_split_last_round(mt, dtype, n, m, k, layout):
    """More tiles than CUs with a small remainder and a long contraction: the tiles of the
    last round are K-split (dense partial tiles + a second stage), with and without tiles that
    cross the border of C, with bias; the result does not depend on the run."""
    g = gen(13)
    a = randn(g, n, k, dtype=dtype, std=0.5) if layout[0] == "n" else randn(g, k, n, dtype=dtype, std=0.5).t()
    b = randn(g, k, m, dtype=dtype, std=0.5) if layout[1] == "n" else randn(g, m, k, dtype=dtype, std=0.5).t()
    bias = randn(g, m, dtype=dtype)
    ad = (a.t().contiguous().to(DEV).t() if layout[0] == "t" else a.to(DEV))
    bd = (b.t().contiguous().to(DEV).t() if layout[1] == "t" else b.to(DEV))
    c = mt.matmul_t(ad, bd, bias.to(DEV))
    check(c, a, b, dtype, bias=bias)
    assert torch.equal(c, mt.matmul_t(ad, bd, bias.to(DEV)))


def _random_cases():
    import random
    rnd = random.Random(20240611)
    cases = []
    for i in range(28):
        # many tiles (several rounds of the persistent grid at small sizes are not reachable, but
        # streamed multi-tile workgroups, border tiles, K tails and odd panel counts all are)
        n = rnd.choice([256, 512, 1000, 1280, 2048, 2304, 3000, 4096])
        m = rnd.choice([192, 384, 200, 768, 770, 960, 1536])
        k = rnd.choice([64, 128, 192, 256, 320, 768, 1000, 1024, 2048])
        layout = rnd.choice(["nn", "nt", "tn", "tt"])
        epi = rnd.choice(["none", "bias", "gelu", "gelu_pre"])
        cases.append((n, m, k, layout, epi))
    # more tiles than workgroups: every workgroup streams through two or three tiles
    cases += [(16384, 1536, 256, "nt", "gelu_pre"), (16384, 2304, 128, "nn", "bias"), (12288, 1540, 256, "nt", "gelu"),
              (8192, 3072, 192, "tn", "none")]
    return cases


@pytest.mark.parametrize("n,m,k,layout,epi", _random_cases())
def test_gemm_random_shapes_layouts_epilogues(mt, n, m, k, layout, epi):
    """Seeded sweep over shapes x operand layouts x epilogues in bf16 (the storage type of the
    training step): exercises the streamed tile loop, border tiles, K tails and every epilogue
    variant in combinations the fixed cases above do not list."""
    dtype = torch.bfloat16
    g = gen(n + 3 * m + 7 * k)
    a = randn(g, n, k, dtype=dtype, std=0.5) if layout[0] == "n" else randn(g, k, n, dtype=dtype, std=0.5).t()
    b = randn(g, k, m, dtype=dtype, std=0.5) if layout[1] == "n" else randn(g, m, k, dtype=dtype, std=0.5).t()
    bias = randn(g, m, dtype=dtype) if epi != "none" else None
    ad = (a.t().contiguous().to(DEV).t() if layout[0] == "t" else a.to(DEV))
    bd = (b.t().contiguous().to(DEV).t() if layout[1] == "t" else b.to(DEV))
    biasd = bias.to(DEV) if bias is not None else None
    if epi == "gelu_pre":
        pre = torch.empty(n, m, dtype=dtype, device=DEV)
        c = mt.matmul_t(ad, bd, biasd, gelu=True, pre_out=pre)
        check(pre, a, b, dtype, bias=bias)
    else:
        c = mt.matmul_t(ad, bd, biasd, gelu=(epi == "gelu"))
    check(c, a, b, dtype, bias=bias, gelu=epi.startswith("gelu"))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_bias_gelu_and_ffn(mt, dtype):
    g = gen(12)
    x = randn(g, 4, 96, 768, dtype=dtype)
    w1, b1 = randn(g, 3072, 768, dtype=dtype, std=0.02), randn(g, 3072, dtype=dtype, std=0.1)
    w2, b2 = randn(g, 768, 3072, dtype=dtype, std=0.02), randn(g, 768, dtype=dtype, std=0.1)
    x2 = x.reshape(-1, 768)
    h = mt.matmul_t(x2.to(DEV), w1.to(DEV).t(), b1.to(DEV), gelu=True)
    check(h, x2, w1.t(), dtype, bias=b1, gelu=True)
    y = mt.t_tlayer_ffn_fwd_t((w1.to(DEV), b1.to(DEV), w2.to(DEV), b2.to(DEV)), x.to(DEV), mt.t_gelu_fwd)
    assert y.shape == x.shape
    want = ops.gelu(f64(x2) @ f64(w1).t() + f64(b1)) @ f64(w2).t() + f64(b2)
    rel = ((f64(y).reshape(-1, 768) - want).norm() / want.norm()).item()
    assert rel < (1e-5 if dtype == torch.float32 else 1e-2), rel


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_strided_output_and_misaligned_inputs(mt, dtype):
    g = gen(13)
    a, b = randn(g, 70, 41, dtype=dtype), randn(g, 41, 50, dtype=dtype)
    buf = torch.zeros(70, 64, dtype=dtype, device=DEV)
    mt.matmul_t(a.to(DEV), b.to(DEV), out=buf[:, :50])
    check(buf[:, :50], a, b, dtype)
    assert (buf[:, 50:] == 0).all()
    # operands starting 1 element into an allocation (not 16-byte aligned)
    pa = torch.zeros(70 * 41 + 1, dtype=dtype, device=DEV)
    pa[1:] = a.to(DEV).reshape(-1)
    c = mt.matmul_t(pa[1:].view(70, 41), b.to(DEV))
    check(c, a, b, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_gelu_dual_output(mt, dtype):
    g = gen(14)
    x, w, b = randn(g, 300, 200, dtype=dtype), randn(g, 260, 200, dtype=dtype, std=0.1), randn(g, 260, dtype=dtype)
    pre = torch.empty(300, 260, dtype=dtype, device=DEV)
    act = mt.matmul_t(x.to(DEV), w.to(DEV).t(), b.to(DEV), gelu=True, pre_out=pre)
    check(pre, x, w.t(), dtype, bias=b)
    check(act, x, w.t(), dtype, bias=b, gelu=True)
    # the activation is computed from the unrounded pre-activation, exactly as the single-output epilogue
    assert torch.equal(act, mt.matmul_t(x.to(DEV), w.to(DEV).t(), b.to(DEV), gelu=True))


def _gelu_deriv64(x64):
    """gelu'(x) in fp64 through the oracle's backward with a unit incoming gradient."""
    return ops.gelu_bkwd2(torch.ones_like(x64), x64)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,m,k", [(300, 260, 200), (512, 384, 128), (256, 192, 768), (64, 100, 4096)])
def test_gemm_gelu_derivative_output(mt, dtype, n, m, k):
    """Second output of the derivative epilogue = gelu'(a @ b + bias); first output unchanged.
    Shapes: edge tiles, whole tiles on the pipelined path, and a long K that is split."""
    g = gen(15 + n)
    x, w, b = randn(g, n, k, dtype=dtype), randn(g, m, k, dtype=dtype, std=0.1), randn(g, m, dtype=dtype)
    der = torch.empty(n, m, dtype=dtype, device=DEV)
    act = mt.matmul_t(x.to(DEV), w.to(DEV).t(), b.to(DEV), gelu=True, deriv_out=der)
    check(act, x, w.t(), dtype, bias=b, gelu=True)
    assert torch.equal(act, mt.matmul_t(x.to(DEV), w.to(DEV).t(), b.to(DEV), gelu=True))
    pre64 = f64(x) @ f64(w).t() + f64(b)
    want = _gelu_deriv64(pre64)
    # |gelu''| <= 1.1: the error of the pre-activation carries over, plus the output rounding
    scale = f64(x).abs() @ f64(w).t().abs() + f64(b).abs()
    bound = bound_of(want, scale, dtype, 1.2) + 1e-6
    err = (f64(der) - want).abs()
    assert not (err > bound).any(), (err / bound).max().item()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,m,k,layout", [(512, 384, 128, "nn"), (256, 192, 768, "nt"), (300, 260, 200, "nn"),
                                          (130, 70, 96, "tn"), (1024, 768, 256, "nn"), (33, 5, 7, "nn"),
                                          (64, 100, 4096, "nn")])
def test_gemm_multiply_epilogue_with_column_sums(mt, dtype, n, m, k, layout):
    """(a @ b) * mul and its column sums against fp64; the product is the stored, rounded a @ b
    times mul, and the sums are those of the stored result."""
    g = gen(16 + n + m)
    a = randn(g, n, k, dtype=dtype) if layout[0] == "n" else randn(g, k, n, dtype=dtype).t()
    b = randn(g, k, m, dtype=dtype, std=0.1) if layout[1] == "n" else randn(g, m, k, dtype=dtype, std=0.1).t()
    mul = randn(g, n, m, dtype=dtype)
    ad = (a.t().contiguous().to(DEV).t() if layout[0] == "t" else a.to(DEV))
    bd = (b.t().contiguous().to(DEV).t() if layout[1] == "t" else b.to(DEV))
    c, sums = mt.matmul_mul_colsum_t(ad, bd, mul.to(DEV))
    assert c.shape == (n, m) and sums.shape == (m,) and c.dtype == dtype and sums.dtype == dtype
    # element-wise: the rounded a @ b (same bound as the plain product, which may sum a long K in
    # another order) times mul, rounded once more
    a64, b64, m64 = f64(a), f64(b), f64(mul)
    # the product rounded to storage (bound_of), times mul, rounded once more
    bound = bound_of(a64 @ b64, a64.abs() @ b64.abs(), dtype) * m64.abs()
    bound = bound + (1e-30 if dtype == torch.float32 else OUT_BF16 * (a64 @ b64 * m64).abs() + 1e-6)
    err = (f64(c) - a64 @ b64 * m64).abs()
    assert not (err > bound).any(), (err / bound).max().item()
    if dtype == torch.bfloat16 and k <= 768:             # one summation order: bit-equal to the two-step form
        plain = mt.matmul_t(ad, bd)
        assert torch.equal(c, (plain.float() * mul.to(DEV).float()).to(dtype))
    want_s = f64(c).sum(0)
    mag = f64(c).abs().sum(0)
    tol = 1e-6 if dtype == torch.float32 else 5e-3       # fp32 accumulation, output rounded to storage
    assert ((f64(sums) - want_s).abs() <= tol * mag + 1e-30).all(), ((f64(sums) - want_s).abs() / (mag + 1e-30)).max()


@pytest.mark.parametrize("dtype", DTYPES)
def test_ffn_backward_through_the_fused_epilogues(mt, dtype):
    """t_tlayer_ffn_bkwd2_t (derivative epilogue forward, multiply + column-sum epilogue backward)
    against autograd of the fp64 restatement."""
    g = gen(17)
    N, D, F = 384, 192, 576
    x = randn(g, N, D, dtype=dtype)
    w1, b1 = randn(g, F, D, dtype=dtype, std=0.05), randn(g, F, dtype=dtype, std=0.1)
    w2, b2 = randn(g, D, F, dtype=dtype, std=0.05), randn(g, D, dtype=dtype, std=0.1)
    dy = randn(g, N, D, dtype=dtype)
    leaves = [f64(t).requires_grad_() for t in (x, w1, b1, w2, b2)]
    out = ops.gelu(leaves[0] @ leaves[1].t() + leaves[2]) @ leaves[3].t() + leaves[4]
    want = torch.autograd.grad(out, leaves, f64(dy))
    dx, (dw1, db1, dw2, db2) = mt.t_tlayer_ffn_bkwd2_t(dy.to(DEV), tuple(t.to(DEV) for t in (w1, b1, w2, b2)), x.to(DEV))
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for name, got, w in zip(("dx", "dw1", "db1", "dw2", "db2"), (dx, dw1, db1, dw2, db2), want):
        rel = ((f64(got) - w).norm() / w.norm()).item()
        assert got.shape == w.shape and rel < tol, (name, rel)
