"""The drop-in boundary as data: every name the reference's callers import from the two
modules this package stands in for, with the reference's positional parameter list
(model_triton.py / loss_and_optimizer_triton.py at the cited lines), checked against
inspect.signature of the export -- without a GPU.  Extra parameters are allowed only after
the reference's, and only with defaults, so a reference-style call binds the same way."""
import inspect
import types

import pytest
import torch

# name -> (reference line, positional parameters in order, names that have defaults in the reference)
MODEL_TRITON = {
    "t_log_softmax_fwd_t": (62, ["x"], []),
    "t_log_softmax_bkwd2_t": (153, ["dloss_dx", "x"], []),
    "t_gelu_fwd_t": (254, ["x"], []),
    "t_gelu_bkwd2_t": (296, ["dloss_dx", "x"], []),
    "t_matmul_t": (373, ["a", "b"], []),
    "t_tlayer_ffn_fwd_t": (1258, ["layer_params", "x", "activation_fn"], []),
    "t_tlayer_ffn_bkwd2_t": (1410, ["dloss_dx", "layer_params", "x", "activation_fn"], []),
    "t_softmax_attn_fwd_t": (519, ["q", "k", "mask", "train", "p_gen_aux"], ["p_gen_aux"]),
    "t_softmax_attn_bkwd2_t": (579, ["dloss_dx", "q", "k", "mask", "train", "p_gen_aux"], ["p_gen_aux"]),
    "t_scaled_dot_prod_attn_fwd3_t": (706, ["qkv", "mask", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_scaled_dot_prod_attn_bkwd3_t": (951, ["dloss_dx", "acts", "qkv", "mask", "train", "p_gen_aux"],
                                       ["train", "p_gen_aux"]),
    "t_dropout_fwd_t": (1496, ["x", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_dropout_bkwd2_t": (1562, ["dloss_dx", "x", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_layernorm_fwd_t": (1625, ["layer_params", "x"], []),
    "t_layernorm_bkwd2_p_t": (1710, ["dloss_dx", "layer_params", "x"], []),
    "t_layernorm_bkwd2_x_t": (1853, ["dloss_dx", "layer_params", "x"], []),
    "t_gpt2_tlayer_fwd3_t": (2214, ["layer_params", "y", "mask", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_gpt2_tlayer_bkwd3_t": (2291, ["dloss_dx", "acts", "layer_params", "y", "mask", "train", "p_gen_aux"],
                              ["train", "p_gen_aux"]),
    "t_gpt2_tlayers_fwd3_t": (2334, ["params", "y", "mask", "indices", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_gpt2_forward_with_acts_t": (2535, ["params", "y", "y_mask", "y_indices", "train", "p_gen_aux"], ["p_gen_aux"]),
    "t_gpt2_bkwd3_p_t": (2583, ["dloss_dx", "acts", "params", "y", "y_mask", "y_indices", "train", "p_gen_aux"],
                         ["p_gen_aux"]),
    # plain-torch twins (the "naive" side of the reference's tests)
    "t_log_softmax_fwd": (25, ["x_logits"], []),
    "t_log_softmax_bkwd2": (91, ["dloss_dx", "x_logits"], []),
    "t_gelu_fwd": (221, ["x"], []),
    "t_gelu_bkwd2": (269, ["dloss_dx", "x"], []),
    "t_linear_fwd": (306, ["layer_params", "x"], []),
    "t_proj_fwd": (436, ["layer_params", "x"], []),
    "t_softmax_attn_fwd": (510, ["q", "k", "mask", "train", "p_gen_aux"], ["p_gen_aux"]),
    "t_softmax_attn_bkwd2": (550, ["dloss_dx", "q", "k", "mask", "train", "p_gen_aux"], ["p_gen_aux"]),
    "t_scaled_dot_prod_attn_fwd": (608, ["qkv", "mask", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_scaled_dot_prod_attn_fwd3": (756, ["qkv", "mask", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_scaled_dot_prod_attn_bkwd3": (801, ["dloss_dx", "acts", "qkv", "mask", "train", "p_gen_aux"],
                                     ["train", "p_gen_aux"]),
    "t_tlayer_ffn_fwd": (1244, ["layer_params", "x", "activation_fn"], []),
    "t_dropout_fwd": (1450, ["x", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_dropout_bkwd2": (1518, ["dloss_dx", "x", "train", "p_gen_aux"], ["train", "p_gen_aux"]),
    "t_layernorm_fwd": (1574, ["layer_params", "x"], []),
    "t_layernorm_bkwd2_p": (1652, ["dloss_dx", "layer_params", "x"], []),
    "t_layernorm_bkwd2_x": (1790, ["dloss_dx", "layer_params", "x"], []),
    "t_embed_fwd": (166, ["layer_params", "x"], []),
}
LOSS_AND_OPTIMIZER = {
    "t_avg_cross_entropy_loss_bkwd3_t": (176, ["y_labels", "x_logits"], []),
    "t_avg_cross_entropy_loss_bkwd3": (83, ["y_labels", "x_logits"], []),
    "t_avg_cross_entropy_loss": (23, ["y_labels", "x_logits"], []),
    "accuracy": (199, ["y_labels", "x_logits"], []),
    "t_loss_bkwd3_t": (279, ["params", "y", "y_mask", "y_indices", "train", "p_gen_aux"], ["p_gen_aux"]),
    "t_acc_grad_loss3_t": (336, ["acc_grads", "params", "y", "y_mask", "y_indices"], []),
    "_acc_grad_loss": (340, ["grad_loss_fn", "acc_grads", "params", "y", "y_mask", "y_indices"], []),
    "sample_p_gen_aux": (318, ["params"], []),
    "init_adam_w": (362, ["params"], []),
    "adam_w_in_place": (376, ["params", "grads", "lr", "betas", "epsilon", "moments", "i", "weight_decay",
                              "weight_decay_mask"], ["weight_decay", "weight_decay_mask"]),
    "grads_l2norm": (413, ["grads"], []),
    "grads_grps_l2norms": (415, ["grads"], []),
    "sgd": (358, ["params", "grads", "lr"], []),
    "elwise": (355, ["params_and_grads", "func"], []),
}


def _check(mod, table):
    for name, (_, want, defaults) in table.items():
        fn = getattr(mod, name, None)
        assert callable(fn), "%s.%s is missing" % (mod.__name__, name)
        ps = list(inspect.signature(fn).parameters.values())
        pos = [p for p in ps if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)]
        # same names in the same order: positional and keyword calls written for the
        # reference bind identically
        assert [p.name for p in pos[:len(want)]] == want, (name, [p.name for p in pos], want)
        for p in pos[:len(want)]:
            if p.name in defaults:
                assert p.default is not p.empty, (name, p.name)
        # anything beyond the reference's list must be optional
        for p in pos[len(want):] + [p for p in ps if p.kind == p.KEYWORD_ONLY]:
            assert p.default is not p.empty, "%s: extra parameter %s needs a default" % (name, p.name)


def test_model_triton_exports_and_signatures(mt):
    _check(mt, MODEL_TRITON)


def test_loss_and_optimizer_exports_and_signatures(lo):
    _check(lo, LOSS_AND_OPTIMIZER)


def test_adam_w_in_place_parameter_names(lo):
    names = list(inspect.signature(lo.adam_w_in_place).parameters)[:9]
    assert names[1:] == ["grads", "lr", "betas", "epsilon", "moments", "i", "weight_decay", "weight_decay_mask"]


def test_init_adam_w_returns_accumulators_and_two_moment_nests(lo):
    params = [[torch.ones(3, 2), torch.zeros(3)], [torch.ones(4, dtype=torch.bfloat16)]]
    grads, moments = lo.init_adam_w(params)             # unpacks as train_gpt2_triton.py:267 does
    assert len(moments) == 2
    for nest in (grads, moments[0], moments[1]):
        assert [[t.shape for t in g] for g in nest] == [[p.shape for p in g] for g in params]
        assert all(float(t.abs().sum()) == 0 for g in nest for t in g)
    assert grads[1][0].dtype == torch.bfloat16 and moments[0][1][0].dtype == torch.float32


def test_gradient_norm_helpers_on_cpu_tensors(lo):
    g = [[torch.tensor([3.0, 4.0]), torch.tensor([[12.0]])], [torch.tensor([0.0, 5.0])]]
    assert lo.grads_grps_l2norms(g) == pytest.approx([13.0, 5.0])
    assert lo.grads_l2norm(g) == pytest.approx((169.0 + 25.0) ** 0.5)


def test_acc_grad_loss_accumulates_and_forwards_aux(lo):
    params = [[torch.zeros(2)], [torch.zeros(1)], [torch.zeros(1)]]          # "L = 0" nest: one seed
    seen = {}

    def fake_grad_loss(p, y, y_mask, y_indices, train, p_gen_aux):
        seen["train"], seen["seeds"] = train, p_gen_aux
        return [[torch.tensor([1.0, 2.0])], [torch.tensor([3.0])], [torch.tensor([4.0])]], ("loss", "acc", "frac")

    acc = [[torch.tensor([10.0, 10.0])], [torch.tensor([0.0])], [torch.tensor([1.0])]]
    out, rest = lo._acc_grad_loss(fake_grad_loss, acc, params, None, None, None)
    assert rest == ("loss", "acc", "frac") and seen["train"] is True and len(seen["seeds"]) == 1
    assert out is acc and out[0][0].tolist() == [11.0, 12.0] and out[1][0].tolist() == [3.0] and out[2][0].tolist() == [5.0]


def test_spec_twins_agree_with_library_routines(mt, lo):
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4, 6, 10, generator=g, dtype=torch.float64)
    dy = torch.randn(4, 6, 10, generator=g, dtype=torch.float64)
    p = (torch.randn(10, generator=g, dtype=torch.float64), torch.randn(10, generator=g, dtype=torch.float64))
    assert torch.allclose(mt.t_gelu_fwd(x), F.gelu(x, approximate="tanh"), atol=1e-12)
    assert torch.allclose(mt.t_log_softmax_fwd(x), torch.log_softmax(x, -1), atol=1e-12)
    assert torch.allclose(mt.t_layernorm_fwd(p, x), F.layer_norm(x, (10,), None, None, 0.0) * (0.9 ** 0.5) * p[0] + p[1],
                          atol=1e-12)
    xr = x.clone().requires_grad_(True)
    for fwd, bwd in ((lambda t: mt.t_gelu_fwd(t), lambda: mt.t_gelu_bkwd2(dy, x)),
                     (lambda t: mt.t_log_softmax_fwd(t), lambda: mt.t_log_softmax_bkwd2(dy, x)),
                     (lambda t: mt.t_layernorm_fwd(p, t), lambda: mt.t_layernorm_bkwd2_x(dy, p, x))):
        (want,) = torch.autograd.grad(fwd(xr), xr, dy)
        assert torch.allclose(bwd(), want, atol=1e-11)
    dg, db = mt.t_layernorm_bkwd2_p(dy, p, x)
    gr = [t.clone().requires_grad_(True) for t in p]
    wg, wb = torch.autograd.grad(mt.t_layernorm_fwd(gr, x), gr, dy)
    assert torch.allclose(dg, wg, atol=1e-11) and torch.allclose(db, wb, atol=1e-11)
    assert torch.equal(mt.t_dropout_fwd(x, False), x * 0.9)
    a, b = mt.t_dropout_fwd(x, True, 7), mt.t_dropout_bkwd2(x, x, True, 7)
    assert torch.equal(a, b) and 0.8 < float((a != 0).double().mean()) < 0.97
    qkv = torch.randn(2, 3, 3, 5, 4, generator=g, dtype=torch.float64)
    mask = torch.tril(torch.ones(5, 5, dtype=torch.bool)).expand(2, 5, 5)
    q, k, v = qkv.unbind(2)
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True) * 0.9
    assert torch.allclose(mt.t_scaled_dot_prod_attn_fwd(qkv, mask, False), want, atol=1e-12)
    o, acts = mt.t_scaled_dot_prod_attn_fwd3(qkv, mask, False)
    dO = torch.randn_like(o)
    qr = qkv.clone().requires_grad_(True)
    (wq,) = torch.autograd.grad(mt.t_scaled_dot_prod_attn_fwd(qr, mask, False), qr, dO)
    for got, c in zip(mt.t_scaled_dot_prod_attn_bkwd3(dO, acts, qkv, mask, False), range(3)):
        assert torch.allclose(got, wq[:, :, c], atol=1e-11)
    lg = torch.randn(3, 5, 11, generator=g, dtype=torch.float64)
    y = torch.randint(0, 11, (3, 5), generator=g)
    y[0, 0] = 0
    loss, cnt, dlg = lo.t_avg_cross_entropy_loss_bkwd3(y, lg)
    lr = lg.clone().requires_grad_(True)
    want = F.cross_entropy(lr.reshape(-1, 11), y.reshape(-1), ignore_index=0)
    assert abs(float(loss) - float(want)) < 1e-12 and int(cnt) == int((y != 0).sum())
    assert torch.allclose(dlg, torch.autograd.grad(want, lr)[0], atol=1e-12)


def test_install_patches_the_reference_modules_by_attribute(pkg):
    import importlib
    dropin = importlib.import_module("pre-tjax_amd.dropin")
    mt = importlib.import_module("pre-tjax_amd.model_triton")
    ref_mt = types.ModuleType("model_triton")
    ref_lo = types.ModuleType("loss_and_optimizer_triton")
    keep = object()
    ref_mt.t_layernorm_fwd_t = ref_mt.t_gpt2_bkwd3_p_t = "triton version"
    ref_lo.loss_train = ref_lo.grad_loss = keep                  # torch.func side stays the reference's
    ref_lo.t_gpt2_forward_with_acts_t = "imported by value"      # from model_triton import ...
    ref_lo.t_loss_bkwd3_t = "triton version"
    done = dropin.install(ref_mt, ref_lo)
    assert ref_mt.t_layernorm_fwd_t is mt.t_layernorm_fwd_t and ref_mt.t_gpt2_bkwd3_p_t is mt.t_gpt2_bkwd3_p_t
    assert ref_lo.loss_train is keep and ref_lo.grad_loss is keep
    assert ref_lo.t_gpt2_forward_with_acts_t is mt.t_gpt2_forward_with_acts_t
    assert callable(ref_lo.t_loss_bkwd3_t) and callable(ref_lo.t_acc_grad_loss3_t)
    assert ("loss_and_optimizer_triton", "init_adam_w") in done
    for name in dropin.MODEL_NAMES:
        assert name in MODEL_TRITON, name
    for name in dropin.LOSS_NAMES:
        assert name in LOSS_AND_OPTIMIZER, name


def test_ffn_wrappers_accept_the_reference_modules_own_gelu_marker(pkg):
    """After an attribute-level install the callers pass THEIR module's `t_gelu_fwd` object
    (model_triton.py:2184, tests/test_t_tlayer_ffn_fwd.py:21), which is not this package's twin:
    the marker is recognised by name.  On CPU tensors the call then gets past the marker check
    and stops at the no-fallback guard; anything that is not the GELU marker is refused."""
    import importlib
    dropin = importlib.import_module("pre-tjax_amd.dropin")
    mt = importlib.import_module("pre-tjax_amd.model_triton")
    lib = importlib.import_module("pre-tjax_amd._lib")
    ref_mt = types.ModuleType("model_triton")

    def t_gelu_fwd(x):                      # a distinct object with the reference's name
        return x

    ref_mt.t_gelu_fwd = t_gelu_fwd
    dropin.install(ref_mt)
    assert ref_mt.t_gelu_fwd is t_gelu_fwd and ref_mt.t_gelu_fwd is not mt.t_gelu_fwd
    params = (torch.zeros(8, 4), torch.zeros(8), torch.zeros(4, 8), torch.zeros(4))
    x = torch.zeros(2, 4)
    for call in (lambda f: ref_mt.t_tlayer_ffn_fwd_t(params, x, f),
                 lambda f: ref_mt.t_tlayer_ffn_bkwd2_t(x, params, x, f)):
        with pytest.raises(lib.PtjError):
            call(ref_mt.t_gelu_fwd)
        with pytest.raises(AssertionError):
            call(torch.relu)


def test_softmax_attn_twin_backward_is_the_vjp_of_its_forward(mt):
    g = torch.Generator().manual_seed(3)
    q = torch.randn(2, 3, 5, 4, generator=g, dtype=torch.float64)
    k = torch.randn(2, 3, 5, 4, generator=g, dtype=torch.float64)
    mask = torch.tril(torch.ones(5, 5, dtype=torch.bool)).expand(2, 5, 5)
    d = torch.randn(2, 3, 5, 5, generator=g, dtype=torch.float64)
    qr, kr = q.clone().requires_grad_(True), k.clone().requires_grad_(True)
    wq, wk = torch.autograd.grad(mt.t_softmax_attn_fwd(qr, kr, mask, False), (qr, kr), d)
    gq, gk = mt.t_softmax_attn_bkwd2(d, q, k, mask, False)
    assert torch.allclose(gq, wq, atol=1e-12) and torch.allclose(gk, wk, atol=1e-12)
