"""Writes tests/golden/vectors_v1.npz: small fixed input/output vectors for the kernels of the
path, produced by the CPU oracle (oracle/), which is itself pinned by known-answer vectors,
library routines and closed forms (tests/test_oracle_*.py).  Nothing of the reference
implementation is imported or executed.  Run from the repository root:

    python tests/golden/make_golden.py

The fixture is data only (inputs and expected outputs); tests/test_golden.py checks that the
oracle still reproduces it (CPU) and that the HIP kernels match it (GPU)."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ops, philox  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors_v1.npz")


def main():
    g = torch.Generator().manual_seed(20240501)
    d = {}
    # Philox keep masks: row-wise (seed + row, column) and attention (seed + batch-head, q + k)
    d["rowwise_seed"] = np.array([42, (1 << 32) + 5], dtype=np.int64)
    d["rowwise_mask_seed42"] = philox.rowwise_keep_mask(42, 6, 72)
    d["rowwise_mask_seedbig"] = philox.rowwise_keep_mask((1 << 32) + 5, 3, 16)
    d["attn_mask_seed9"] = philox.attn_keep_mask(9, 3, 64, 64)
    # LayerNorm on the literal D=4 row the reference's own backward test prints
    # (tests/test_t_layernorm_bkwd-wip.py:13-16) and on a random [5, 12] block
    x4 = torch.tensor([[-0.2614, 0.9828, -0.1427, 0.1716]], dtype=torch.float64)
    dy4 = torch.tensor([[0.7227, 0.6544, -0.7753, 0.5889]], dtype=torch.float64)
    p4 = (torch.ones(4, dtype=torch.float64), torch.zeros(4, dtype=torch.float64))
    d["ln4_x"], d["ln4_dy"] = x4.numpy(), dy4.numpy()
    d["ln4_y"] = ops.layernorm_fwd(p4, x4).numpy()
    d["ln4_dx"] = ops.layernorm_bkwd2_x(dy4, p4, x4).numpy()
    x = torch.randn(5, 12, generator=g, dtype=torch.float64)
    dy = torch.randn(5, 12, generator=g, dtype=torch.float64)
    gam, bet = torch.randn(12, generator=g, dtype=torch.float64), torch.randn(12, generator=g, dtype=torch.float64)
    d["ln_x"], d["ln_dy"], d["ln_gamma"], d["ln_beta"] = x.numpy(), dy.numpy(), gam.numpy(), bet.numpy()
    d["ln_y"] = ops.layernorm_fwd((gam, bet), x).numpy()
    d["ln_dx"] = ops.layernorm_bkwd2_x(dy, (gam, bet), x).numpy()
    dg, db = ops.layernorm_bkwd2_p(dy, (gam, bet), x)
    d["ln_dgamma"], d["ln_dbeta"] = dg.numpy(), db.numpy()
    # GELU and its derivative on a fixed grid
    gx = torch.linspace(-6, 6, 49, dtype=torch.float64)
    d["gelu_x"], d["gelu_y"] = gx.numpy(), ops.gelu(gx).numpy()
    d["gelu_dx"] = ops.gelu_bkwd2(torch.ones_like(gx), gx).numpy()
    # mean cross-entropy over labels != 0 and its gradient, [6, 10] logits with an ignored row
    lg = torch.randn(6, 10, generator=g, dtype=torch.float64) * 2
    lab = torch.tensor([3, 0, 9, 1, 1, 7])
    loss, cnt, dlg = ops.avg_cross_entropy_loss_bkwd3(lab, lg)
    d["ce_logits"], d["ce_labels"] = lg.numpy(), lab.numpy()
    d["ce_loss"], d["ce_count"], d["ce_dlogits"] = np.array(float(loss)), np.array(int(cnt)), dlg.numpy()
    # causal attention, B1 H1 T64 dh64 (the kernels' tile), eval mode: output and statistics;
    # inputs stored in fp32 (exactly representable for the fp32 kernels)
    qkv = torch.randn(1, 1, 3, 64, 64, generator=g, dtype=torch.float32).to(torch.float64)
    mask = torch.tril(torch.ones(64, 64, dtype=torch.bool)).expand(1, 64, 64)
    o = ops.scaled_dot_prod_attn_fwd(qkv, mask, train=False)
    ms, ls = ops.scaled_dot_prod_attn_stats(qkv, mask)
    d["attn_qkv"] = qkv.to(torch.float32).numpy()
    d["attn_o"], d["attn_ms"], d["attn_ls"] = o.numpy(), ms.numpy(), ls.numpy()
    np.savez_compressed(OUT, **d)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(d), "arrays")


if __name__ == "__main__":
    main()
