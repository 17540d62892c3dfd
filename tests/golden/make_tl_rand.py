"""Writes tests/golden/tl_rand_v1.npz: uniform floats and keep decisions produced by the
INSTALLED third-party Triton package's own ``tl.rand`` (CPU interpreter, TRITON_INTERPRET=1),
for the two ways the reference addresses it: ``tl.rand(seed + row, col)`` of the row-wise
dropout kernels (model_triton.py:1463, 1486-1492) and ``tl.rand(seed + bs_h, q + k)`` of the
attention kernels (model_triton.py:688, 923).  The kernel below is a six-line stand-alone
Triton program, not reference code; nothing of the reference is imported or executed.
Run from the repository root in the build container (needs the `triton` package, no GPU):

    TRITON_INTERPRET=1 python tests/golden/make_tl_rand.py

tests/test_oracle_philox.py compares oracle/philox.py with the stored values (CPU), and
tests/test_golden.py compares the HIP dropout kernels with the stored keep decisions (GPU)."""
import os

os.environ["TRITON_INTERPRET"] = "1"

import numpy as np  # noqa: E402
import torch  # noqa: E402
import triton  # noqa: E402
import triton.language as tl  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tl_rand_v1.npz")
SEEDS = [42, 0, 999999, (1 << 32) + 5]
ROWS, COLS = 5, 96           # row-wise layout: seed + row, offset = column
BH, TQ, TK = 3, 16, 16       # attention layout: seed + batch-head, offset = q + k


@triton.jit
def rand_rows_k(out_ptr, seed, n_cols, BLOCK: tl.constexpr):
    row = tl.program_id(0)
    offs = tl.arange(0, BLOCK)
    r = tl.rand(seed + row, offs)
    tl.store(out_ptr + row * n_cols + offs, r, mask=offs < n_cols)


@triton.jit
def rand_attn_k(out_ptr, seed, BQ: tl.constexpr, BK: tl.constexpr):
    bh = tl.program_id(0)
    q = tl.arange(0, BQ)
    k = tl.arange(0, BK)
    r = tl.rand(seed + bh, q[:, None] + k[None, :])
    tl.store(out_ptr + bh * BQ * BK + q[:, None] * BK + k[None, :], r)


def main():
    d = {"seeds": np.array(SEEDS, dtype=np.int64), "triton_version": np.array(triton.__version__)}
    for s in SEEDS:
        rows = torch.zeros(ROWS, COLS, dtype=torch.float32)
        rand_rows_k[(ROWS,)](rows, s, COLS, BLOCK=128)
        attn = torch.zeros(BH, TQ, TK, dtype=torch.float32)
        rand_attn_k[(BH,)](attn, s, BQ=TQ, BK=TK)
        d["rows_u_%d" % s] = rows.numpy()
        d["rows_keep_%d" % s] = rows.numpy() > np.float32(0.1)
        d["attn_u_%d" % s] = attn.numpy()
        d["attn_keep_%d" % s] = attn.numpy() > np.float32(0.1)
    np.savez_compressed(OUT, **d)
    print("wrote", OUT, os.path.getsize(OUT), "bytes; triton", triton.__version__)


if __name__ == "__main__":
    main()
