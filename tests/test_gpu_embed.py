"""GPU parity of the fused embedding kernels: forward (gather * sqrt(D) + positions + dropout)
against the CPU oracle's formula and against the separate gather / add / dropout calls;
backward (scatter-add onto the tied table gradient) against an fp64 index_add."""
import math

import pytest
import torch

from oracle import philox
from util import DTYPES, assert_close, f64, gen, randn

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("train", [True, False])
@pytest.mark.parametrize("B,T,V,D", [(4, 64, 1000, 768), (2, 5, 11, 100), (1, 1, 3, 8)])
def test_embed_fwd(mt, dtype, train, B, T, V, D):
    g = gen(5)
    wemb, pos = randn(g, V, D, dtype=dtype, std=0.02), randn(g, T + 3, D, dtype=dtype, std=0.02)
    y = torch.randint(0, V, (B, T), generator=g)
    seed = 777
    got = mt.embed_pos_dropout_t(wemb.to(DEV), pos.to(DEV), y.to(DEV), train, seed)
    assert got.shape == (B, T, D)
    # the same three steps through the separate entry points: bit-identical
    x = mt.t_embed_fwd((wemb.to(DEV),), y.to(DEV)) + pos.to(DEV)[:T]
    assert torch.equal(got, mt.t_dropout_fwd_t(x, train, seed))
    # oracle: fp64 formula with the Philox keep mask of rows b*T + t
    h = f64(wemb)[y] * math.sqrt(D) + f64(pos)[:T]
    if train:
        keep = torch.from_numpy(philox.rowwise_keep_mask(seed, B * T, D)).reshape(B, T, D)
        want = torch.where(keep, h, torch.zeros_like(h))
    else:
        want = 0.9 * h
    assert_close(got, want, dtype, what="embed fwd")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,V,D,hot", [(16384, 50257, 768, 0), (4096, 50, 768, 0), (5000, 1000, 768, 3000),
                                       (37, 11, 100, 0), (1, 5, 8, 0)])
def test_embed_bwd(mt, dtype, N, V, D, hot):
    """`hot` positions share one token id (a long run in the sorted order)."""
    g = gen(6)
    y = torch.randint(0, V, (N,), generator=g)
    if hot:
        y[torch.randperm(N, generator=g)[:hot]] = 7
    d = randn(g, N, D, dtype=dtype)
    dw0 = randn(g, V, D, dtype=dtype)
    got = mt.embed_bkwd_add_t(dw0.clone().to(DEV), d.to(DEV), y.to(DEV))
    want = f64(dw0).index_add(0, y, f64(d) * math.sqrt(D))
    cnt = torch.bincount(y, minlength=V).max().item()
    if dtype == torch.float32:
        assert_close(got, want, dtype, rtol=1e-5, atol=2e-6 * math.sqrt(D) * max(1.0, cnt ** 0.5), what="embed bwd")
    else:
        assert_close(got, want, dtype, rtol=8e-3, atol=1e-2, what="embed bwd")
    # rows of tokens that do not occur are untouched; the result is deterministic
    absent = torch.ones(V, dtype=torch.bool)
    absent[y] = False
    assert torch.equal(got.cpu()[absent], dw0[absent])
    again = mt.embed_bkwd_add_t(dw0.clone().to(DEV), d.to(DEV), y.to(DEV))
    assert torch.equal(got, again)
