"""GPU parity of the flash-attention kernels (through the C ABI) against the fp64 oracle on
the same (dtype-rounded) inputs.  Tolerances: fp32 rtol 1e-5 relative to the tensor's scale
(atol = 1e-5 * max|want|) ; bf16 2e-2 likewise.  Dropout masks are exercised through the
train-mode output (the oracle applies the Philox keep mask of the reference kernel)."""
import pytest
import torch

from oracle import ops
from util import DTYPES, f64, gen, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


def close(got, want, dtype, what):
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    scale = want.abs().max().item()
    err = (f64(got) - want).abs().max().item()
    assert err <= tol * max(scale, 1e-30), "%s: max err %.3e vs scale %.3e (tol %g)" % (what, err, scale, tol)


def make(B, H, T, dtype, seed=0):
    g = gen(seed)
    qkv = randn(g, B, H, 3, T, 64, dtype=dtype)
    dO = randn(g, B, H, T, 64, dtype=dtype)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T).contiguous()
    return qkv, dO, mask


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,H,T", [(1, 1, 64), (2, 3, 128), (1, 2, 192), (2, 2, 256), (1, 12, 512)])
@pytest.mark.parametrize("train", [False, True])
@pytest.mark.parametrize("mask_as", ["tensor", "none"])
def test_attn_fwd_bwd_causal(mt, dtype, B, H, T, train, mask_as):
    """`tensor`: the lower-triangular mask as a bool tensor (bit-packed on the device, applied
    from the packed words); `none`: mask=None, the kernels' index-masked causal path."""
    qkv, dO, mask = make(B, H, T, dtype, seed=T + B)
    seed = 4242
    dmask = mask.to(DEV) if mask_as == "tensor" else None
    o, acts = mt.t_scaled_dot_prod_attn_fwd3_t(qkv.to(DEV), dmask, train, seed)
    want_o = ops.scaled_dot_prod_attn_fwd(f64(qkv), mask, train, seed)
    close(o, want_o, dtype, "O")
    ms, ls = ops.scaled_dot_prod_attn_stats(f64(qkv), mask)
    assert acts[2] is o and acts[0].shape == (B, H, T)
    close(acts[0], ms, torch.float32 if dtype == torch.float32 else dtype, "ms")
    close(acts[1], ls, torch.float32 if dtype == torch.float32 else dtype, "ls")
    dq, dk, dv = mt.t_scaled_dot_prod_attn_bkwd3_t(dO.to(DEV), acts, qkv.to(DEV), dmask, train, seed)
    wq, wk, wv = ops.scaled_dot_prod_attn_bkwd(f64(dO), f64(qkv), mask, train, seed)
    close(dq, wq, dtype, "dq")
    close(dk, wk, dtype, "dk")
    close(dv, wv, dtype, "dv")
    # deterministic (no atomics)
    dq2, dk2, dv2 = mt.t_scaled_dot_prod_attn_bkwd3_t(dO.to(DEV), acts, qkv.to(DEV), dmask, train, seed)
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mask_as", ["tensor", "none"])
def test_attn_config2_shape(mt, dtype, mask_as):
    # BASELINE config 2: B=8, H=12, T=1024, dh=64 (oracle on a 2-batch slice to bound CPU time)
    B, H, T = 8, 12, 1024
    qkv, dO, mask = make(B, H, T, dtype, seed=2)
    dmask = mask.to(DEV) if mask_as == "tensor" else None
    o, acts = mt.t_scaled_dot_prod_attn_fwd3_t(qkv.to(DEV), dmask, False)
    dq, dk, dv = mt.t_scaled_dot_prod_attn_bkwd3_t(dO.to(DEV), acts, qkv.to(DEV), dmask, False)
    sl = slice(6, 8)
    want_o = ops.scaled_dot_prod_attn_fwd(f64(qkv[sl]), mask[sl], False)
    close(o[sl], want_o, dtype, "O")
    wq, wk, wv = ops.scaled_dot_prod_attn_bkwd(f64(dO[sl]), f64(qkv[sl]), mask[sl], False)
    close(dq[sl], wq, dtype, "dq")
    close(dk[sl], wk, dtype, "dk")
    close(dv[sl], wv, dtype, "dv")
    # size-independent property at full size: T=1 prefix -> first output row equals 0.9 * v[0]
    assert torch.allclose(o[:, :, 0].float().cpu(), 0.9 * qkv[:, :, 2, 0].float(), rtol=2e-2, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("train", [False, True])
def test_attn_padding_mask(mt, dtype, train):
    # tril AND key-padding AND packing (block-diagonal) -- sub-masks of the causal mask, as the
    # training collator builds them; every row keeps its diagonal.
    B, H, T = 2, 2, 256
    qkv, dO, mask = make(B, H, T, dtype, seed=9)
    mask = mask.clone()
    mask[0, :, 100:130] = False                      # padded keys ...
    mask[0, 200:, :200] = False                      # second packed sequence cannot see the first
    mask[1, 64:, :64] = False
    idx = torch.arange(T)
    mask[:, idx, idx] = True                         # ... but a token always sees itself
    seed = 77
    o, acts = mt.t_scaled_dot_prod_attn_fwd3_t(qkv.to(DEV), mask.to(DEV), train, seed)
    close(o, ops.scaled_dot_prod_attn_fwd(f64(qkv), mask, train, seed), dtype, "O")
    dq, dk, dv = mt.t_scaled_dot_prod_attn_bkwd3_t(dO.to(DEV), acts, qkv.to(DEV), mask.to(DEV), train, seed)
    wq, wk, wv = ops.scaled_dot_prod_attn_bkwd(f64(dO), f64(qkv), mask, train, seed)
    close(dq, wq, dtype, "dq")
    close(dk, wk, dtype, "dk")
    close(dv, wv, dtype, "dv")


def _packed_documents_mask(B, T, seed):
    """What the packing collator emits for a row of three documents and a padded tail:
    lower triangular AND same document AND neither side padding.  Returns (mask [B,T,T] bool,
    pad [B,T] bool: the queries without any visible key)."""
    g = gen(seed)
    doc = torch.zeros(B, T, dtype=torch.int64)
    for b in range(B):
        cuts = sorted(torch.randint(1, T - 40, (2,), generator=g).tolist())
        end = int(torch.randint(T - 39, T - 3, (1,), generator=g))        # a padded tail of 4..39 positions
        doc[b, :cuts[0]] = 1
        doc[b, cuts[0]:cuts[1]] = 2
        doc[b, cuts[1]:end] = 3                                            # 0 = padding
    real = doc != 0
    same = doc.unsqueeze(2) == doc.unsqueeze(1)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)) & same & real.unsqueeze(2) & real.unsqueeze(1)
    return mask, ~real


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("train", [False, True])
def test_attn_three_packed_documents_per_row(mt, dtype, train):
    """Three packed documents and a padded tail per row at T = 512: hidden tiles (a later
    document against an earlier one) are skipped, tiles inside a document run the index path,
    tiles that straddle a document boundary or the padding read their mask words.  Rows with a
    visible key against the oracle; padding queries (no visible key at all) give zero output
    rows, statistics (-1e9, 0) and neither receive nor pass on gradient, so the oracle's
    gradients are taken with dO zeroed on those rows."""
    B, H, T, seed = 2, 3, 512, 515
    qkv, dO, _ = make(B, H, T, dtype, seed=41)
    mask, pad = _packed_documents_mask(B, T, 17)
    assert pad.any() and (mask.sum(-1) == 0).equal(pad)
    o, acts = mt.t_scaled_dot_prod_attn_fwd3_t(qkv.to(DEV), mask.to(DEV), train, seed)
    want_o = ops.scaled_dot_prod_attn_fwd(f64(qkv), mask, train, seed)
    live = (~pad).view(B, 1, T, 1)
    close(o * live.to(DEV), want_o * live, dtype, "O (rows with a visible key)")
    padq = pad.view(B, 1, T).expand(B, H, T)
    assert not o.cpu()[padq].any()                                          # exact zeros
    assert (acts[0].cpu()[padq] == -1e9).all() and (acts[1].cpu()[padq] == 0).all()
    ms, ls = ops.scaled_dot_prod_attn_stats(f64(qkv), mask)
    st = torch.float32 if dtype == torch.float32 else dtype
    close(torch.where(padq.to(DEV), 0, acts[0]), torch.where(padq, 0, ms), st, "ms")
    close(torch.where(padq.to(DEV), 0, acts[1]), torch.where(padq, 0, ls), st, "ls")
    dq, dk, dv = mt.t_scaled_dot_prod_attn_bkwd3_t(dO.to(DEV), acts, qkv.to(DEV), mask.to(DEV), train, seed)
    wq, wk, wv = ops.scaled_dot_prod_attn_bkwd(f64(dO) * live, f64(qkv), mask, train, seed)
    close(dq, wq, dtype, "dq")
    close(dk, wk, dtype, "dk")
    close(dv, wv, dtype, "dv")
    assert not dq.cpu()[padq].any()
    # keys that nobody sees (the padding) get no gradient either
    assert not dk.cpu()[padq].any() and not dv.cpu()[padq].any()


@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_rows_without_visible_keys_closed_forms(mt, dtype):
    """What the kernels do on rows the mask hides completely, next to rows with one visible key
    (the reference's mask notebook, tests/test_t_scaled_dot_prod_attn_fwd_diff_masks.ipynb cells
    1-3, compares such masks): a row whose only visible key is j returns 0.9 v_j (eval) whatever
    the scores; a row with none returns 0 and has (ms, ls) = (-1e9, 0) -- also when every row of
    its 32-query group is hidden (all tiles skipped) and when it sits in a group with live rows."""
    B, H, T = 1, 2, 192
    qkv, dO, _ = make(B, H, T, dtype, seed=5)
    mask = torch.zeros(B, T, T, dtype=torch.bool)
    idx = torch.arange(T)
    one_key = (idx * 7) % (idx + 1)                       # some key <= query
    mask[0, idx, one_key] = True
    mask[0, 64:96] = False                                # a whole 32-query group without keys
    mask[0, 130] = False                                  # single rows inside live groups
    mask[0, 5] = False
    hidden = mask.sum(-1) == 0
    o, acts = mt.t_scaled_dot_prod_attn_fwd3_t(qkv.to(DEV), mask.to(DEV), False)
    want = 0.9 * f64(qkv)[:, :, 2][:, :, one_key] * (~hidden).view(B, 1, T, 1)
    close(o, want, dtype, "O")
    hq = hidden.view(B, 1, T).expand(B, H, T)
    assert not o.cpu()[hq].any()
    assert (acts[0].cpu()[hq] == -1e9).all() and (acts[1].cpu()[hq] == 0).all()
    assert (acts[1].cpu()[~hq] - 1).abs().max().item() < 1e-5   # one visible key: sum-exp = 1
    dq, dk, dv = mt.t_scaled_dot_prod_attn_bkwd3_t(dO.to(DEV), acts, qkv.to(DEV), mask.to(DEV), False)
    # one visible key per row: P is a one-hot row, so dS = 0 (dq = dk = 0 up to the rounding of the
    # stored O inside rowsum(dO * O)) and dV_j = 0.9 * sum of dO_i over the live rows i whose key is j
    want_dv = torch.zeros(B, H, T, 64, dtype=torch.float64)
    want_dv.index_add_(2, one_key[~hidden[0]], 0.9 * f64(dO)[:, :, ~hidden[0]])
    close(dv, want_dv, dtype, "dv")
    tol = (1e-5 if dtype == torch.float32 else 2e-2) * want_dv.abs().max().item()
    assert dq.abs().max().item() <= tol and dk.abs().max().item() <= tol
    assert not dq.cpu()[hq].any()                         # rows without keys: exactly nothing


@pytest.mark.parametrize("train", [False, True])
def test_attn_lower_triangular_tensor_equals_mask_none_bitwise(mt, train):
    """A plain lower-triangular mask tensor is classified tile by tile as the causal pattern and
    runs the same index-masked code as mask=None: identical bits, forward and backward."""
    B, H, T, seed = 2, 4, 512, 7
    qkv, dO, mask = make(B, H, T, torch.bfloat16, seed=77)
    qd, dd = qkv.to(DEV), dO.to(DEV)
    o0, a0 = mt.t_scaled_dot_prod_attn_fwd3_t(qd, None, train, seed)
    o1, a1 = mt.t_scaled_dot_prod_attn_fwd3_t(qd, mask.to(DEV), train, seed)
    assert torch.equal(o0, o1) and torch.equal(a0[0], a1[0]) and torch.equal(a0[1], a1[1])
    g0 = mt.t_scaled_dot_prod_attn_bkwd3_t(dd, a0, qd, None, train, seed)
    g1 = mt.t_scaled_dot_prod_attn_bkwd3_t(dd, a1, qd, mask.to(DEV), train, seed)
    for x, y in zip(g0, g1):
        assert torch.equal(x, y)


def test_attn_fresh_mask_tensor_every_call(mt):
    """The collator builds a new mask every batch: each call below gets a mask tensor that did
    not exist before, alternating between two contents, so that a freed mask's address is
    likely handed to a tensor with other content.  Nothing may be carried over from the
    previous tensor at that address, and no call may need the host (the packed words are
    made on the device from the tensor given)."""
    B, H, T = 2, 2, 256
    qkv, _, tril = make(B, H, T, torch.float32, seed=3)
    qd = qkv.to(DEV)
    padded = tril.clone()
    padded[:, 128:, :128] = False
    want = {"tril": ops.scaled_dot_prod_attn_fwd(f64(qkv), tril, False, 0),
            "padded": ops.scaled_dot_prod_attn_fwd(f64(qkv), padded, False, 0)}
    for it in range(8):
        name, host = (("tril", tril), ("padded", padded))[it % 2]
        m = host.to(DEV)                                 # a fresh device tensor
        o, _ = mt.t_scaled_dot_prod_attn_fwd3_t(qd, m, False, 0)
        close(o, want[name], torch.float32, "O %s call %d" % (name, it))
        del m                                            # its memory may be handed out again
    # a mask rewritten in place (same address, new version) is packed again
    m = tril.to(DEV)
    mt.t_scaled_dot_prod_attn_fwd3_t(qd, m, False, 0)
    m.copy_(padded.to(DEV))
    o, _ = mt.t_scaled_dot_prod_attn_fwd3_t(qd, m, False, 0)
    close(o, want["padded"], torch.float32, "O after in-place rewrite")


def test_attn_dropout_mask_bits(mt):
    # P with q = 0, k = 0 is uniform over visible keys; with v = one-hot(key % 64) the train-mode
    # output row i, column c is (#kept keys j<=i with j%64==c)/(i+1): recovers the keep mask exactly.
    B, H, T = 1, 2, 128
    qkv = torch.zeros(B, H, 3, T, 64)
    qkv[:, :, 2, torch.arange(T), torch.arange(T) % 64] = 1.0
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T).contiguous()
    seed = 31337
    o, _ = mt.t_scaled_dot_prod_attn_fwd3_t(qkv.to(DEV), mask.to(DEV), True, seed)
    keep = ops.attn_keep(B, H, T, seed).to(torch.float64)
    want = torch.einsum("bhqk,kc->bhqc", keep * mask.unsqueeze(1), torch.eye(64, dtype=torch.float64).repeat(2, 1))
    want = want / torch.arange(1, T + 1, dtype=torch.float64).view(1, 1, T, 1)
    assert torch.allclose(f64(o), want, rtol=1e-5, atol=1e-7)


def test_attn_full_size_train_properties(mt):
    """BASELINE config 5 shape (B16 H12 T1024, bf16, dropout on): properties that need no oracle.
    (1) the backward is linear in dO, and a scaling by 2 commutes with every rounding, so
        bwd(2 dO) == 2 bwd(dO) bit for bit -- which also holds only if the dK/dV pass reads the
        row sums rowsum(dO*O) of THIS call (the dQ pass of the same call writes them);
    (2) with v = 1 and dO = 1: O[q, :] = sum_k Pdrop[q, k] and dV[k, :] = sum_q Pdrop[q, k], so both
        have the same grand total per batch-head -- forward and backward apply one dropout mask."""
    B, H, T, seed = 16, 12, 1024, 99
    g = gen(8)
    q = randn(g, B, H, T, 64, dtype=torch.bfloat16).to(DEV)
    k = randn(g, B, H, T, 64, dtype=torch.bfloat16).to(DEV)
    v = randn(g, B, H, T, 64, dtype=torch.bfloat16).to(DEV)
    dO = randn(g, B, H, T, 64, dtype=torch.bfloat16).to(DEV)
    o, ms, ls = mt.attn_fwd_t(q, k, v, None, True, seed)
    d1 = [t.clone() for t in mt.attn_bwd_t(dO, q, k, v, o, ms, ls, None, True, seed)]
    d2 = mt.attn_bwd_t(dO * 2, q, k, v, o, ms, ls, None, True, seed)
    for a, b, name in zip(d1, d2, ("dq", "dk", "dv")):
        assert torch.equal(a * 2, b), name
    again = mt.attn_bwd_t(dO, q, k, v, o, ms, ls, None, True, seed)
    for a, b, name in zip(d1, again, ("dq", "dk", "dv")):
        assert torch.equal(a, b), name + " not reproducible"

    ones = torch.ones_like(v)
    o1, ms1, ls1 = mt.attn_fwd_t(q, k, ones, None, True, seed)
    _, _, dv1 = mt.attn_bwd_t(ones, q, k, ones, o1, ms1, ls1, None, True, seed)
    tot_o = o1[..., 0].double().sum(dim=-1)          # [B, H]
    tot_dv = dv1[..., 0].double().sum(dim=-1)
    assert torch.allclose(tot_o, tot_dv, rtol=2e-3), (tot_o - tot_dv).abs().max().item()
    # about a tenth of the probability mass is dropped
    assert 0.85 * T < tot_o.mean().item() < 0.95 * T


def test_attn_strided_views_fused_qkv_layout(mt):
    # q/k/v as column slices of one [B*T, H*3*dh] buffer, O written into [B,T,H*dh]
    B, H, T = 2, 4, 128
    g = gen(21)
    buf = randn(g, B * T, H * 3 * 64, dtype=torch.bfloat16).to(DEV)
    v5 = buf.view(B, T, H, 3, 64)
    q, k, v = (v5[:, :, :, c].permute(0, 2, 1, 3) for c in range(3))
    out = torch.empty(B, T, H * 64, dtype=torch.bfloat16, device=DEV)
    o, ms, ls = mt.attn_fwd_t(q, k, v, None, False, 0, out=out.view(B, T, H, 64).permute(0, 2, 1, 3))
    qkv = torch.stack((q, k, v), dim=2).contiguous()
    o_ref, _ = mt.t_scaled_dot_prod_attn_fwd3_t(qkv, None, False)
    assert torch.equal(o, o_ref)
    assert torch.equal(out.view(B, T, H, 64).permute(0, 2, 1, 3), o_ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dh", [16, 32])
@pytest.mark.parametrize("train", [False, True])
def test_attn_smaller_head_dimensions(mt, dtype, dh, train):
    """Head sizes below 64 (the reference's mask notebook uses 16): forward and backward against
    the oracle through the padded path of the wrappers."""
    B, H, T, seed = 2, 3, 128, 909
    g = gen(dh)
    qkv = randn(g, B, H, 3, T, dh, dtype=dtype)
    dO = randn(g, B, H, T, dh, dtype=dtype)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool)).expand(B, T, T).contiguous()
    o, acts = mt.t_scaled_dot_prod_attn_fwd3_t(qkv.to(DEV), None, train, seed)
    assert o.shape == (B, H, T, dh)
    close(o, ops.scaled_dot_prod_attn_fwd(f64(qkv), mask, train, seed), dtype, "O")
    dq, dk, dv = mt.t_scaled_dot_prod_attn_bkwd3_t(dO.to(DEV), acts, qkv.to(DEV), None, train, seed)
    wq, wk, wv = ops.scaled_dot_prod_attn_bkwd(f64(dO), f64(qkv), mask, train, seed)
    # sqrt(64/32) is not a power of two: q is rounded once more in 2-byte storage
    for got, want, name in ((dq, wq, "dq"), (dk, wk, "dk"), (dv, wv, "dv")):
        assert got.shape == want.shape
        close(got, want, dtype, name)


def test_attn_rejects_bad_shapes(mt):
    _lib = __import__("importlib").import_module("pre-tjax_amd._lib")
    qkv = torch.zeros(1, 1, 3, 96, 64, device=DEV)
    with pytest.raises(AssertionError):
        mt.t_scaled_dot_prod_attn_fwd3_t(qkv, None, False)
    # the C ABI itself takes dh = 64 only (the wrappers pad smaller heads)
    q = torch.zeros(1, 1, 64, 32, device=DEV)
    o, ms = torch.empty_like(q), torch.empty(1, 1, 64, device=DEV)
    st = (q.stride(0), q.stride(1), q.stride(2))
    rc = _lib.lib().ptj_attn_fwd(q.data_ptr(), q.data_ptr(), q.data_ptr(), None, o.data_ptr(), ms.data_ptr(), ms.data_ptr(),
                                 None, 0, 1, 1, 64, 32, *st, *st, *st, *st, 0, 0, _lib.PTJ_F32, _lib.stream())
    assert rc != 0 and b"head dimension" in _lib.lib().ptj_last_error()
    o2, _, _ = mt.attn_fwd_t(q, q, q, None, False, 0)
    assert o2.shape == q.shape
    with pytest.raises(AssertionError):
        mt.t_scaled_dot_prod_attn_fwd3_t(torch.zeros(1, 1, 3, 64, 128, device=DEV), None, False)
