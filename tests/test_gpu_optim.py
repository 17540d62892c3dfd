"""GPU parity of the fused AdamW kernel and the column-sum kernel against the CPU oracle."""
import importlib

import pytest
import torch

from oracle import gpt2 as ogpt2
from util import f64, gen, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("gdtype", [torch.float32, torch.bfloat16])
def test_adamw_matches_oracle(lo, gdtype):
    g = gen(3)
    shapes = [(257, 33), (1000,), (7,), (64, 64)]
    params = [[randn(g, *s) for s in shapes[:2]], [randn(g, *s) for s in shapes[2:]]]
    wd_mask = [[True, False], [False, True]]
    master = [[p.clone().to(DEV) for p in grp] for grp in params]
    shadow = [[p.to(torch.bfloat16).to(DEV) for p in grp] for grp in params]
    _, moments = lo.init_adam_w(master)
    o_params = [[p.double() for p in grp] for grp in params]
    o_mom = [[[torch.zeros_like(p) for p in grp] for grp in o_params] for _ in range(2)]
    for i in range(4):
        grads = [[randn(g, *p.shape, dtype=gdtype) for p in grp] for grp in params]
        lo.adam_w_in_place(master, [[x.to(DEV) for x in grp] for grp in grads], 6e-4, (0.9, 0.95), 1e-8, moments, i,
                           0.1, wd_mask, shadow=shadow)
        o_params, o_mom = ogpt2.adam_w(o_params, [[x.double() for x in grp] for grp in grads], 6e-4, (0.9, 0.95), 1e-8,
                                       o_mom, i, 0.1, wd_mask)
    for gi in range(2):
        for pi in range(2):
            assert torch.allclose(f64(master[gi][pi]), o_params[gi][pi], rtol=1e-5, atol=1e-6)
            assert torch.allclose(f64(moments[0][gi][pi]), o_mom[0][gi][pi], rtol=1e-5, atol=1e-7)
            assert torch.allclose(f64(moments[1][gi][pi]), o_mom[1][gi][pi], rtol=1e-5, atol=1e-7)
            assert torch.equal(shadow[gi][pi], master[gi][pi].to(torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(16384, 768), (1000, 50257), (37, 101), (1, 8), (4, 6, 64), (16, 98304), (150, 20000)])
def test_colsum(mt, dtype, shape):
    g = gen(4)
    x = randn(g, *shape, dtype=dtype)
    got = mt.colsum_t(x.to(DEV))
    want = f64(x).reshape(-1, shape[-1]).sum(0)
    rows = x.numel() // shape[-1]
    tol = (3e-6 if dtype == torch.float32 else 8e-3) * max(1.0, rows ** 0.5)
    assert (f64(got) - want).abs().max().item() <= tol + (0 if dtype == torch.float32 else 1e-2 * want.abs().max().item())
    assert torch.equal(got, mt.colsum_t(x.to(DEV)))


def test_adamw_multi_equals_single_tensor_calls(lo, pkg):
    """The multi-tensor entry point updates every tensor exactly as ptj_adamw does (bit-exact),
    across the chunking of its launches (more tensors than one launch holds, odd sizes)."""
    _lib = importlib.import_module("pre-tjax_amd._lib")
    g = gen(9)
    sizes = [1, 3, 4, 5, 1023, 1024, 4099] * 6 + [300000]
    params = [[randn(g, n) for n in sizes]]
    grads = [[randn(g, n, dtype=torch.bfloat16).to(DEV) for n in sizes]]
    wd_mask = [[i % 2 == 0 for i in range(len(sizes))]]
    a_p = [[p.clone().to(DEV) for p in params[0]]]
    a_sh = [[p.to(torch.bfloat16).to(DEV) for p in params[0]]]
    _, a_mom = lo.init_adam_w(a_p)
    b_p = [p.clone().to(DEV) for p in params[0]]
    b_sh = [p.to(torch.bfloat16).to(DEV) for p in params[0]]
    b_m = [torch.zeros_like(p) for p in b_p]
    b_v = [torch.zeros_like(p) for p in b_p]
    for i in range(3):
        lo.adam_w_in_place(a_p, grads, 1e-3, (0.9, 0.95), 1e-8, a_mom, i, 0.1, wd_mask, shadow=a_sh)
        for k, n in enumerate(sizes):
            _lib.check(_lib.lib().ptj_adamw(_lib.ptr(b_p[k]), _lib.ptr(b_m[k]), _lib.ptr(b_v[k]), _lib.ptr(grads[0][k]),
                                            _lib.ptr(b_sh[k]), n, 1e-3, 0.9, 0.95, 1e-8, 0.1 if wd_mask[0][k] else 0.0,
                                            i + 1, 1, 1, _lib.stream()), "ptj_adamw")
    for k in range(len(sizes)):
        assert torch.equal(a_p[0][k], b_p[k]) and torch.equal(a_sh[0][k], b_sh[k])
        assert torch.equal(a_mom[0][0][k], b_m[k]) and torch.equal(a_mom[1][0][k], b_v[k])
