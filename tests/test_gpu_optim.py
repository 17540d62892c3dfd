"""GPU parity of the fused AdamW kernel and the column-sum kernel against the CPU oracle."""
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
    moments = lo.init_adam_w(master)
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
@pytest.mark.parametrize("shape", [(16384, 768), (1000, 50257), (37, 101), (1, 8), (4, 6, 64)])
def test_colsum(mt, dtype, shape):
    g = gen(4)
    x = randn(g, *shape, dtype=dtype)
    got = mt.colsum_t(x.to(DEV))
    want = f64(x).reshape(-1, shape[-1]).sum(0)
    rows = x.numel() // shape[-1]
    tol = (3e-6 if dtype == torch.float32 else 8e-3) * max(1.0, rows ** 0.5)
    assert (f64(got) - want).abs().max().item() <= tol + (0 if dtype == torch.float32 else 1e-2 * want.abs().max().item())
    assert torch.equal(got, mt.colsum_t(x.to(DEV)))
