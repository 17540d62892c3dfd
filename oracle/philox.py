"""Philox4x32-10 and the uniform-float / keep-mask derivation used by the
reference's dropout.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

The reference calls Triton's ``tl.rand(seed, offset)`` (model_triton.py:1463,
1530, 688, 923).  ``tl.rand`` is a third-party algorithm (package ``triton``,
pinned 3.2.0 in setup_torch_triton.py:30, not vendored in the reference):
Philox4x32 with 10 rounds, counter = (offset, 0, 0, 0), key = (seed_lo,
seed_hi) of the 64-bit seed, first output word reinterpreted as int32 ``x``,
``x = -x-1 if x < 0``, ``u = float32(x) * 4.6566127342e-10`` and the dropout
keeps an element iff ``u > 0.1`` (float32 compare).

Pinned by the Random123 known-answer vectors for philox4x32-10 in
tests/test_oracle_philox.py.
"""
import numpy as np

PHILOX_KEY_A = np.uint32(0x9E3779B9)
PHILOX_KEY_B = np.uint32(0xBB67AE85)
PHILOX_ROUND_A = np.uint64(0xD2511F53)
PHILOX_ROUND_B = np.uint64(0xCD9E8D57)
_M32 = np.uint64(0xFFFFFFFF)


def philox4x32(c0, c1, c2, c3, k0, k1, rounds=10):
    """Vectorised Philox4x32-`rounds`.  All inputs broadcastable uint32 arrays."""
    c0, c1, c2, c3, k0, k1 = [np.asarray(a, dtype=np.uint32) for a in (c0, c1, c2, c3, k0, k1)]
    shape = np.broadcast_shapes(c0.shape, c1.shape, c2.shape, c3.shape, k0.shape, k1.shape)
    c0, c1, c2, c3, k0, k1 = [np.broadcast_to(a, shape).copy() for a in (c0, c1, c2, c3, k0, k1)]
    with np.errstate(over="ignore"):
        for _ in range(rounds):
            pa = PHILOX_ROUND_A * c0.astype(np.uint64)   # A * c0 (64-bit product)
            pb = PHILOX_ROUND_B * c2.astype(np.uint64)   # B * c2
            hi_a = (pa >> np.uint64(32)).astype(np.uint32)
            lo_a = (pa & _M32).astype(np.uint32)
            hi_b = (pb >> np.uint64(32)).astype(np.uint32)
            lo_b = (pb & _M32).astype(np.uint32)
            c0, c1, c2, c3 = hi_b ^ c1 ^ k0, lo_b, hi_a ^ c3 ^ k1, lo_a
            k0 = k0 + PHILOX_KEY_A
            k1 = k1 + PHILOX_KEY_B
    return c0, c1, c2, c3


def tl_randint(seed, offset):
    """First Philox word for (seed: int or int64 array, offset: uint32 array)."""
    seed = np.asarray(seed, dtype=np.int64).astype(np.uint64)
    k0 = (seed & _M32).astype(np.uint32)
    k1 = ((seed >> np.uint64(32)) & _M32).astype(np.uint32)
    off = np.asarray(offset, dtype=np.int64).astype(np.uint64)
    c0 = (off & _M32).astype(np.uint32)
    z = np.zeros((), dtype=np.uint32)
    return philox4x32(c0, z, z, z, k0, k1)[0]


def uint_to_uniform_float(w):
    """uint32 word -> float32 in [0, 1) exactly as tl.rand does."""
    x = np.asarray(w, dtype=np.uint32).view(np.int32).astype(np.int64)
    x = np.where(x < 0, -x - 1, x)
    return x.astype(np.float32) * np.float32(4.6566127342e-10)


def tl_rand(seed, offset):
    return uint_to_uniform_float(tl_randint(seed, offset))


def rowwise_keep_mask(seed, n_rows, n_cols, p=0.1):
    """Keep mask [n_rows, n_cols] (bool) of the row-wise dropout kernels:
    seed of row r is ``seed + r``, offset is the column (model_triton.py:1486-1492)."""
    rows = np.arange(n_rows, dtype=np.int64)[:, None] + np.int64(seed)
    cols = np.arange(n_cols, dtype=np.int64)[None, :]
    return tl_rand(rows, cols) > np.float32(p)


def attn_keep_mask(seed, bs_h, n_q, n_k, p=0.1):
    """Keep mask [bs_h, n_q, n_k] of the attention kernels: seed ``seed + bs_h_index``,
    offset ``q_index + k_index`` (model_triton.py:688, 923)."""
    s = np.arange(bs_h, dtype=np.int64)[:, None] + np.int64(seed)       # [BH,1]
    off = np.arange(n_q + n_k - 1, dtype=np.int64)[None, :]             # [1, nq+nk-1]
    line = tl_rand(s, off) > np.float32(p)                              # [BH, nq+nk-1]
    idx = np.arange(n_q)[:, None] + np.arange(n_k)[None, :]
    return line[:, idx]


def keep_threshold(p=0.1):
    """Largest non-negative int32 ``t`` with float32(t)*scale <= p; an element is
    kept iff its folded word ``x`` (x<0 -> -x-1) is > t.  Used to cross-check the
    integer-compare form the device code uses."""
    lo, hi = 0, 2**31 - 1
    sc = np.float32(4.6566127342e-10)
    pf = np.float32(p)
    while lo < hi:
        mid = (lo + hi + 1) // 2
        if np.float32(mid) * sc > pf:
            hi = mid - 1
        else:
            lo = mid
    return lo
