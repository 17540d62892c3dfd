"""LM head -> loss -> head gradients in row chunks (only [chunk, V] logits alive at a time)
against the one-pass form over a [B, T, V] buffer, at BASELINE configuration 5's size
(B16 T1024, V50257, bf16), and the two entry points the chunks rest on: the loss pass that
continues over row ranges and the GEMM epilogue that adds onto the stored C."""
import importlib

import pytest
import torch

from oracle import gpt2 as ogpt2
from util import OUT_BF16, f64, gen, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_gemm_accumulating_epilogue(mt):
    """C = round(round(A1^T B1) + A2^T B2) against fp64: one extra rounding of the stored partial sum;
    border tiles (50257 rows), the dW layout (both operands transposed), contraction 2 x 4096."""
    g = gen(41)
    K, N, M = 4096, 50257, 192
    # rows of 50257 elements in a buffer whose pitch keeps them 16-byte aligned (as the logits buffer does)
    a1 = randn(g, K, 50304, dtype=torch.bfloat16, std=0.05)
    a2 = randn(g, K, 50304, dtype=torch.bfloat16, std=0.05)
    b1, b2 = randn(g, K, M, dtype=torch.bfloat16), randn(g, K, M, dtype=torch.bfloat16)
    d = [a1.to(DEV)[:, :N], a2.to(DEV)[:, :N], b1.to(DEV), b2.to(DEV)]
    a1, a2 = a1[:, :N], a2[:, :N]
    assert d[0].stride() == (50304, 1)
    c = mt.matmul_t(d[0].t(), d[2])
    first = c.clone()
    mt.matmul_t(d[1].t(), d[3], out=c, accumulate=True)
    rows = torch.arange(0, N, 97)                        # every tile row, incl. the partly filled last one
    p1 = f64(a1[:, rows]).t() @ f64(b1)
    p2 = f64(a2[:, rows]).t() @ f64(b2)
    s1 = f64(a1[:, rows]).abs().t() @ f64(b1).abs()
    s2 = f64(a2[:, rows]).abs().t() @ f64(b2).abs()
    got = f64(c[rows.to(DEV)])
    bound = 1e-5 * (s1 + s2) + OUT_BF16 * (p1.abs() + (p1 + p2).abs()) + 1e-6
    assert not ((got - (p1 + p2)).abs() > bound).any()
    # the same bits on a second run (fixed summation order), and the first product was really added onto
    c2 = first.clone()
    mt.matmul_t(d[1].t(), d[3], out=c2, accumulate=True)
    assert torch.equal(c, c2) and not torch.equal(c, first)
    _lib = importlib.import_module("pre-tjax_amd._lib")
    with pytest.raises(_lib.PtjError):                   # a K-major x K-major product has no accumulating form
        mt.matmul_t(d[0].t().contiguous(), d[2].t().contiguous().t(), out=c.clone(), accumulate=True)


@pytest.mark.parametrize("rows_total,chunks", [(2048, [1024, 1024]), (2304, [1024, 768, 512]), (700, [512, 188])])
def test_loss_pass_over_row_ranges_is_bit_equal_to_one_call(lo, rows_total, chunks):
    """ptj_ce_fwd_bwd_colsum_rows chunk by chunk (chunk starts at multiples of the CU count) against
    the one-call form: loss, count, gradient, argmax and column sums, bit for bit."""
    _lib = importlib.import_module("pre-tjax_amd._lib")
    V, pitch = 50257, 50304
    g = gen(rows_total)
    x = randn(g, rows_total, pitch, dtype=torch.bfloat16).to(DEV)
    y = torch.randint(0, V, (rows_total,), generator=g)
    y[::9] = 0
    y = y.to(DEV)
    loss0, cnt0, dx0, pred0, sums0 = lo.t_avg_cross_entropy_loss_bkwd3_t(y, x[:, :V], want_pred=True, want_colsum=True)
    lib = _lib.lib()
    loss = torch.empty(1, dtype=torch.float32, device=DEV)
    cnt = torch.empty((), dtype=torch.int64, device=DEV)
    pred = torch.empty(rows_total, dtype=torch.int64, device=DEV)
    sums = torch.empty(V, dtype=torch.bfloat16, device=DEV)
    ws_bytes = lib.ptj_ce_colsum_workspace_bytes(rows_total, V)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    work = x.clone()
    r0 = 0
    for rows in chunks:
        lg = work[r0:r0 + rows]
        _lib.check(lib.ptj_ce_fwd_bwd_colsum_rows(y.data_ptr(), lg.data_ptr(), loss.data_ptr(), cnt.data_ptr(), lg.data_ptr(),
                                                  pred.data_ptr(), sums.data_ptr(), ws.data_ptr(), ws_bytes, rows_total, r0,
                                                  rows, V, pitch, pitch, _lib.PTJ_BF16, _lib.stream()), "rows")
        r0 += rows
    assert r0 == rows_total
    assert torch.equal(loss, loss0) and torch.equal(cnt, cnt0) and torch.equal(pred, pred0)
    assert torch.equal(work[:, :V], dx0) and torch.equal(sums, sums0)
    # a chunk that does not start at a multiple of the CU count is refused
    with pytest.raises(_lib.PtjError):
        _lib.check(lib.ptj_ce_fwd_bwd_colsum_rows(y.data_ptr(), work.data_ptr(), loss.data_ptr(), cnt.data_ptr(),
                                                  work.data_ptr(), pred.data_ptr(), sums.data_ptr(), ws.data_ptr(), ws_bytes,
                                                  rows_total, 100, 300, V, pitch, pitch, _lib.PTJ_BF16, _lib.stream()), "rows")


def test_chunked_head_equals_one_pass_at_b16_t1024(lo, mt):
    """B16 T1024 bf16, train mode, the head in chunks of 8192 rows against one pass over [B, T, V] logits.
    The head by itself: loss, count, argmax and the bias gradient bit-equal; the head's weight
    gradient, which the chunks round once more per chunk, and dh, whose 50257-long contraction an
    8192-row product splits in two for the 256 CUs (another fp32 summation order), within one bf16
    unit.  Then the whole t_loss_bkwd3_t: loss and accuracy bit-equal, every gradient tensor within
    1e-2 relative L2, half the bar against the oracle (the two forms are two roundings of one result,
    and each is held to the oracle elsewhere); peak memory drops by half the logits buffer."""
    V, D, L, H, F, T, B = 50257, 768, 12, 12, 3072, 1024, 16
    params = ogpt2.init_transformer_gpt2(V, D, L, H, F, T, seed=3)
    dparams = [[p.to(torch.bfloat16).to(DEV) for p in grp] for grp in params]
    g = torch.Generator().manual_seed(4)
    y = torch.randint(0, V, (B, T + 1), generator=g)
    y[3, -20:] = 0
    y = y.to(DEV)
    y_in, y_out = y[:, :-1], y[:, 1:]
    seeds = [31 + 7 * i for i in range(1 + 3 * L)]
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool, device=DEV)).expand(B, T, T).contiguous()

    # ---- the head alone, on the same final-norm output
    h, _ = mt.t_gpt2_tlayers_fwd3_t(dparams, y_in, mask, None, True, seeds)
    wemb, bemb = dparams[0]
    logits = mt._padded_logits(B * T, V, h.dtype, DEV)
    mt.matmul_t(h.view(B * T, D), wemb.t(), bemb, out=logits)
    loss0, cnt0, dlog, pred0, db0 = lo.t_avg_cross_entropy_loss_bkwd3_t(y_out, logits, inplace=True, want_pred=True,
                                                                      want_colsum=True)
    head0 = mt.matmul_t(dlog.t(), h.view(B * T, D))
    dh0 = mt.matmul_t(dlog, wemb)
    loss1, cnt1, pred1, dh1, head1, db1 = lo._lm_head_loss_in_row_chunks(dparams, h, y_out, 8192)
    assert torch.equal(loss0, loss1) and torch.equal(cnt0, cnt1) and torch.equal(pred0.reshape(-1), pred1.reshape(-1))
    assert torch.equal(db0, db1)
    unit = 2.0 ** -7
    # dh: two fp32 summation orders of a 50257-long contraction (1e-5 of sum |terms|) and the output rounding
    d = (dh0.float() - dh1.float()).abs()
    terms = mt.matmul_t(dlog.abs(), wemb.abs()).float()
    bound = unit * torch.maximum(dh0.float().abs(), dh1.float().abs()) + 1e-5 * terms
    assert (d <= bound).all(), ("dh", (d - bound).max().item())
    del terms
    # the head's weight gradient: the first chunk's product is stored (rounded: half a unit of ITS magnitude)
    # before the second chunk's is added, then the sum is rounded
    first = mt.matmul_t(dlog[:8192].t(), h.view(B * T, D)[:8192]).float().abs()
    d = (head0.float() - head1.float()).abs()
    bound = 0.5 * unit * first + unit * torch.maximum(head0.float().abs(), head1.float().abs())
    assert (d <= bound).all(), ("dWemb (head part)", (d - bound).max().item())
    del logits, dlog, dh0, dh1, head0, head1, first

    # ---- the whole step, both ways
    keep = lo.LM_HEAD_CHUNK_ROWS
    try:
        lo.LM_HEAD_CHUNK_ROWS = 0
        torch.cuda.reset_peak_memory_stats()
        g0, (l0, a0, f0) = lo.t_loss_bkwd3_t(dparams, y, mask, None, True, seeds)
        peak0 = torch.cuda.max_memory_allocated()
        lo.LM_HEAD_CHUNK_ROWS = 8192
        torch.cuda.reset_peak_memory_stats()
        g1, (l1, a1, f1) = lo.t_loss_bkwd3_t(dparams, y, mask, None, True, seeds)
        peak1 = torch.cuda.max_memory_allocated()
    finally:
        lo.LM_HEAD_CHUNK_ROWS = keep
    assert torch.equal(l0, l1) and torch.equal(a0, a1) and torch.equal(f0, f1)
    assert torch.equal(g0[0][1], g1[0][1])                       # the head's bias gradient: same additions
    for gi, (grp0, grp1) in enumerate(zip(g0, g1)):
        for pi, (t0, t1) in enumerate(zip(grp0, grp1)):
            rel = ((t0.double() - t1.double()).norm() / t0.double().norm().clamp_min(1e-30)).item()
            # dh differs in the last bf16 bit of some elements; twelve blocks of bf16 backward carry that on
            assert rel < 1e-2, (gi, pi, rel)
    # half of the [N, V] logits buffer (0.82 GB) is gone
    assert peak0 - peak1 > 0.7e9, (peak0, peak1)
