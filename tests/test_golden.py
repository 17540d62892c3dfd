"""Golden vectors (tests/golden/vectors_v1.npz, written by tests/golden/make_golden.py):
the CPU oracle must keep reproducing them, and the HIP kernels must match them through the
C ABI -- dropout masks bit for bit, float results to 1e-5 relative in fp32 storage."""
import os

import numpy as np
import pytest
import torch

from oracle import ops, philox

HERE = os.path.dirname(os.path.abspath(__file__))
DEV = "cuda"


@pytest.fixture(scope="module")
def gold():
    with np.load(os.path.join(HERE, "golden", "vectors_v1.npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def t64(a):
    return torch.from_numpy(np.asarray(a)).to(torch.float64)


def close(got, want, rtol=1e-5, atol=1e-6):
    got = got.detach().to("cpu").to(torch.float64)
    assert got.shape == want.shape
    assert torch.allclose(got, want, rtol=rtol, atol=atol), (got - want).abs().max().item()


# ---------------------------------------------------------------------------- CPU: the oracle
def test_oracle_reproduces_golden_masks(gold):
    assert (philox.rowwise_keep_mask(42, 6, 72) == gold["rowwise_mask_seed42"]).all()
    assert (philox.rowwise_keep_mask((1 << 32) + 5, 3, 16) == gold["rowwise_mask_seedbig"]).all()
    assert (philox.attn_keep_mask(9, 3, 64, 64) == gold["attn_mask_seed9"]).all()


def test_oracle_reproduces_golden_floats(gold):
    # fp64 to 1e-12: the host's math library may differ in the last bits of exp/tanh
    same = lambda a, b: torch.allclose(a, b, rtol=1e-12, atol=1e-14)
    p4 = (torch.ones(4, dtype=torch.float64), torch.zeros(4, dtype=torch.float64))
    assert same(ops.layernorm_fwd(p4, t64(gold["ln4_x"])), t64(gold["ln4_y"]))
    assert same(ops.layernorm_bkwd2_x(t64(gold["ln4_dy"]), p4, t64(gold["ln4_x"])), t64(gold["ln4_dx"]))
    p = (t64(gold["ln_gamma"]), t64(gold["ln_beta"]))
    assert same(ops.layernorm_fwd(p, t64(gold["ln_x"])), t64(gold["ln_y"]))
    assert same(ops.layernorm_bkwd2_x(t64(gold["ln_dy"]), p, t64(gold["ln_x"])), t64(gold["ln_dx"]))
    assert same(ops.gelu(t64(gold["gelu_x"])), t64(gold["gelu_y"]))
    assert same(ops.gelu_bkwd2(torch.ones(49, dtype=torch.float64), t64(gold["gelu_x"])), t64(gold["gelu_dx"]))
    loss, cnt, dlg = ops.avg_cross_entropy_loss_bkwd3(torch.from_numpy(gold["ce_labels"]), t64(gold["ce_logits"]))
    assert abs(float(loss) - float(gold["ce_loss"])) < 1e-12 and int(cnt) == int(gold["ce_count"])
    assert same(dlg, t64(gold["ce_dlogits"]))
    # hand check of the literal row: unbiased std, so sum(y) = 0 and sum(y^2) = D - 1
    y4 = t64(gold["ln4_y"])
    assert abs(y4.sum().item()) < 1e-12 and abs((y4 ** 2).sum().item() - 3.0) < 1e-12


# ---------------------------------------------------------------------------- GPU: the kernels
@pytest.mark.gpu
def test_gpu_dropout_masks_equal_golden(mt, gold):
    for seed, key in ((42, "rowwise_mask_seed42"), ((1 << 32) + 5, "rowwise_mask_seedbig")):
        want = torch.from_numpy(gold[key])
        for dtype in (torch.float32, torch.bfloat16):
            x = torch.ones(want.shape, dtype=dtype, device=DEV)
            got = mt.t_dropout_fwd_t(x, True, seed)
            assert torch.equal(got.cpu() != 0, want)
            assert torch.equal(mt.t_dropout_bkwd2_t(x, None, True, seed), got)


@pytest.mark.gpu
def test_gpu_dropout_masks_equal_triton_package_values(mt):
    """Keep decisions written by the installed Triton package's own tl.rand
    (tests/golden/make_tl_rand.py), row-wise and attention addressing, all four seeds."""
    with np.load(os.path.join(HERE, "golden", "tl_rand_v1.npz"), allow_pickle=False) as z:
        fx = {k: z[k] for k in z.files}
    for seed in fx["seeds"].tolist():
        want = torch.from_numpy(fx["rows_keep_%d" % seed])
        for dtype in (torch.float32, torch.bfloat16):
            got = mt.t_dropout_fwd_t(torch.ones(want.shape, dtype=dtype, device=DEV), True, seed)
            assert torch.equal(got.cpu() != 0, want), seed
        # attention: the fixture covers q, k < 16; V = identity shows the kept probabilities
        want = torch.from_numpy(fx["attn_keep_%d" % seed])                  # [3, 16, 16]
        B, H, T, dh = 1, want.shape[0], 64, 64
        z4 = torch.zeros(B, H, T, dh, device=DEV)
        v = torch.eye(T, dh, device=DEV).expand(B, H, T, dh).contiguous()
        o, _, _ = mt.attn_fwd_t(z4, z4.clone(), v, None, True, seed)
        n = want.shape[1]
        tril = torch.tril(torch.ones(n, n, dtype=torch.bool))
        assert torch.equal((o[0, :, :n, :n].cpu() != 0) & tril, want & tril), seed


@pytest.mark.gpu
def test_gpu_attention_dropout_mask_equals_golden(mt, gold):
    # V = identity padded to dh columns makes row q of O the dropped probabilities of q: the
    # zero pattern below the diagonal is the keep mask (seed + batch-head, offset q + k)
    want = torch.from_numpy(gold["attn_mask_seed9"])          # [3, 64, 64]
    B, H, T, dh = 1, 3, 64, 64
    q = torch.zeros(B, H, T, dh, device=DEV)
    k = torch.zeros(B, H, T, dh, device=DEV)
    v = torch.eye(T, dh, device=DEV).expand(B, H, T, dh).contiguous()
    o, _, _ = mt.attn_fwd_t(q, k, v, None, True, 9)
    tril = torch.tril(torch.ones(T, T, dtype=torch.bool))
    got = o[0].cpu() != 0                                      # [H, q, k]
    assert torch.equal(got & tril, want & tril)


@pytest.mark.gpu
def test_gpu_rowwise_kernels_match_golden(mt, lo, gold):
    dev = lambda a: torch.from_numpy(np.asarray(a)).to(torch.float32).to(DEV)
    p4 = (torch.ones(4, device=DEV), torch.zeros(4, device=DEV))
    close(mt.t_layernorm_fwd_t(p4, dev(gold["ln4_x"])), t64(gold["ln4_y"]))
    close(mt.t_layernorm_bkwd2_x_t(dev(gold["ln4_dy"]), p4, dev(gold["ln4_x"])), t64(gold["ln4_dx"]))
    p = (dev(gold["ln_gamma"]), dev(gold["ln_beta"]))
    close(mt.t_layernorm_fwd_t(p, dev(gold["ln_x"])), t64(gold["ln_y"]))
    close(mt.t_layernorm_bkwd2_x_t(dev(gold["ln_dy"]), p, dev(gold["ln_x"])), t64(gold["ln_dx"]))
    dg, db = mt.t_layernorm_bkwd2_p_t(dev(gold["ln_dy"]), p, dev(gold["ln_x"]))
    close(dg, t64(gold["ln_dgamma"]))
    close(db, t64(gold["ln_dbeta"]))
    close(mt.t_gelu_fwd_t(dev(gold["gelu_x"])), t64(gold["gelu_y"]))
    close(mt.t_gelu_bkwd2_t(torch.ones(49, device=DEV), dev(gold["gelu_x"])), t64(gold["gelu_dx"]))
    loss, cnt, dlg = lo.t_avg_cross_entropy_loss_bkwd3_t(torch.from_numpy(gold["ce_labels"]).to(DEV),
                                                         dev(gold["ce_logits"]))
    close(loss.reshape(()), t64(gold["ce_loss"]))
    assert int(cnt) == int(gold["ce_count"])
    close(dlg, t64(gold["ce_dlogits"]))


@pytest.mark.gpu
def test_gpu_attention_matches_golden(mt, gold):
    qkv = torch.from_numpy(gold["attn_qkv"]).to(torch.float32).to(DEV)
    mask = torch.tril(torch.ones(64, 64, dtype=torch.bool, device=DEV)).expand(1, 64, 64)
    o, (ms, ls, _) = mt.t_scaled_dot_prod_attn_fwd3_t(qkv, mask, train=False)
    # eval mode scales the probabilities by 0.9 (non-inverted dropout); the oracle output has it
    close(o, t64(gold["attn_o"]))
    close(ms, t64(gold["attn_ms"]))
    close(ls, t64(gold["attn_ls"]))
