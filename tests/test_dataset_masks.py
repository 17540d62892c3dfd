"""The batch / mask contract of the collators (the caller side of the kernel path):
y_mask = lower-triangular AND padding AND packing, padded query rows empty, positions
restart per packed document; and that the attention kernels and the full model accept such
masks (padded rows included) and agree with the oracle on everything the loss can see."""
import importlib

import numpy as np
import pytest
import torch

from oracle import gpt2 as ogpt2
from oracle import ops

td = importlib.import_module("pre-tjax_amd.tokenized_dataset")


def test_build_masks_is_tril_and_padding_and_packing():
    y = np.array([5, 6, 7, 8, 9, 0, 0, 0])
    _, m, _ = td.build_masks(np.zeros(8, dtype=int), y)
    want = np.tril(np.ones((8, 8))) * np.outer(y != 0, y != 0)
    assert (m == want).all() and m[5:].sum() == 0 and m[:, 5:].sum() == 0
    packs = td.ones_block_diag([3, 2, 3], [3, 2, 3])
    _, mp, _ = td.build_masks(np.zeros(8, dtype=int), y, y_packs=packs)
    assert (mp == want * packs).all()
    assert mp[3, 2] == 0 and mp[4, 3] == 1 and mp[2, 0] == 1          # no attention across documents


def test_convert_batch_item_pads_cuts_and_restarts_positions():
    x, y1, xm, ym, yxm, xi, yi = td.convert_batch_item([], [1, 7, 8, 2, 1, 9, 2], 8, [0, 0], [4, 3])
    assert y1.tolist() == [1, 7, 8, 2, 1, 9, 2, 0, 0] and ym.shape == (8, 8)
    assert yi.tolist() == [0, 1, 2, 3, 0, 1, 2, 0]                        # filler document covers the tail
    assert ym[4, 3] == 0 and ym[6, 4] == 1 and ym[7].sum() == 0           # second document / padded row
    # too long: cut to seq_len (+1 for the shifted targets)
    _, y2, _, ym2, _, _, yi2 = td.convert_batch_item([], list(range(1, 20)), 8)
    assert y2.tolist() == list(range(1, 10)) and (ym2 == np.tril(np.ones((8, 8)))).all() and yi2.tolist() == list(range(8))


def test_batch_generators_shapes_and_packing():
    items = list(td.synthetic_items(40, 100, 3, 9, seed=1))
    batches = list(td.get_batched_examples(items, 4, 16, 1, 2))
    assert len(batches) == 10
    x, y, xm, ym, yxm, xi, yi = batches[0]
    assert y.shape == (4, 17) and ym.shape == (4, 16, 16) and yi.shape == (4, 16)
    assert (y[:, 0] == 1).all()
    last = list(td.get_batched_examples(items[:6], 4, 16, 1, 2, drop_last=False))[-1]
    assert (last[1][2:] == 0).all() and last[3][2:].sum() == 0           # completed with all-padding rows
    packed = list(td.get_batched_examples_packed(items, 4, 16, 1, 2, pack_frac=0.75))
    _, yp, _, ymp, _, _, yip = packed[0]
    assert yp.shape == (4, 17) and (yip[:, 0] == 0).all()
    assert ((yip == 0).sum(axis=1) >= 2).all()                            # at least two documents per row
    assert np.array_equal(ymp, np.tril(ymp))                              # never above the diagonal
    real = yp[:, :-1] != 0
    diag = ymp[:, np.arange(16), np.arange(16)]
    assert np.array_equal(diag.astype(bool), real)                        # a real token sees itself, a padded one nothing


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_on_packed_padded_batch_matches_oracle(lo, dtype):
    """A packed, padded batch from the collator through the kernel path, train mode: loss and
    every gradient against the oracle.  Padded queries have an empty mask row; their outputs
    differ between implementations by design (the reference's kernel averages V over the
    visited keys, its torch model over all keys) but no real token or scored label sees them."""
    V, D, L, H, F, T, B = 211, 128, 2, 2, 256, 128, 4
    items = list(td.synthetic_items(64, V, 10, 70, seed=3))
    batch = next(td.get_batched_examples_packed(items, B, T, 1, 2, pack_frac=0.75))
    y = torch.from_numpy(batch[1]).to(torch.int64)
    mask = torch.from_numpy(batch[3]).to(torch.bool)
    assert (y[:, :-1] == 0).any() and not mask.all(dim=-1).any()
    params = ogpt2.init_transformer_gpt2(V, D, L, H, F, T, seed=4)
    seeds = [300 + 7 * i for i in range(1 + 3 * L)]
    dev = [[p.to(dtype).to("cuda") for p in grp] for grp in params]
    grads, (loss, acc, frac) = lo.t_loss_bkwd3_t(dev, y.to("cuda"), mask.to("cuda"), None, True, seeds)
    want, (wl, wacc, wfrac) = ogpt2.grad_loss([[p.to(dtype).double() for p in grp] for grp in params], y, mask, True,
                                              seeds)
    ltol, gtol = (1e-5, 5e-5) if dtype == torch.float32 else (5e-3, 2e-2)
    assert abs(loss.item() - wl.item()) <= ltol * abs(wl.item())
    assert abs(frac.item() - wfrac.item()) < 1e-6 and frac.item() < 1.0
    for gi, (gg, wg) in enumerate(zip(grads, want)):
        for pi, (a, b) in enumerate(zip(gg, wg)):
            e = ((a.double().cpu() - b).norm() / b.norm().clamp_min(1e-30)).item()
            assert e <= gtol, "grad[%d][%d] rel L2 %.3e" % (gi, pi, e)
