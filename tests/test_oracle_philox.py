"""Pins oracle/philox.py: Random123 known-answer vectors for philox4x32-10, the
uniform-float conversion, and the integer form of the keep decision."""
import numpy as np

from oracle import philox


def test_philox_kat_random123():
    # kat_vectors of Random123 (philox4x32 10 rounds): counter, key -> output
    z = philox.philox4x32(0, 0, 0, 0, 0, 0)
    assert [int(w) for w in z] == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]
    f = 0xFFFFFFFF
    o = philox.philox4x32(f, f, f, f, f, f)
    assert [int(w) for w in o] == [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]
    p = philox.philox4x32(0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344, 0xa4093822, 0x299f31d0)
    assert [int(w) for w in p] == [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]


def test_randint_is_word0_with_offset_counter_and_seed_key():
    # seed 0, offset 0 is the all-zero KAT; seed = 2^32+5 puts 5 in k0 and 1 in k1.
    assert int(philox.tl_randint(0, 0)) == 0x6627e8d5
    a = philox.tl_randint((1 << 32) + 5, 7)
    b = philox.philox4x32(7, 0, 0, 0, 5, 1)[0]
    assert int(a) == int(b)


def test_uniform_float_range_and_fold():
    w = np.array([0, 1, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF], dtype=np.uint32)
    u = philox.uint_to_uniform_float(w)
    assert u.dtype == np.float32
    # 0 -> 0; 0xFFFFFFFF is int32 -1 -> folded to 0; 0x80000000 is INT_MIN -> 2^31-1
    assert u[0] == 0.0 and u[4] == 0.0
    assert u[2] == u[3]
    assert (u >= 0).all() and (u < 1).all()


def test_keep_threshold_matches_float_compare():
    t = philox.keep_threshold(0.1)
    assert t == 214748392
    sc, p = np.float32(4.6566127342e-10), np.float32(0.1)
    xs = np.arange(t - 2000, t + 2000, dtype=np.int64)
    keep_f = xs.astype(np.float32) * sc > p
    keep_i = xs > t
    assert (keep_f == keep_i).all()
    # and on random words through the full pipeline
    rng = np.random.default_rng(0)
    w = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    x = w.view(np.int32).astype(np.int64)
    x = np.where(x < 0, -x - 1, x)
    assert ((philox.uint_to_uniform_float(w) > p) == (x > t)).all()


def test_rowwise_mask_layout_and_rate():
    m = philox.rowwise_keep_mask(42, 16, 768)
    # row r of seed s equals row 0 of seed s+r
    m2 = philox.rowwise_keep_mask(42 + 5, 1, 768)
    assert (m[5] == m2[0]).all()
    big = philox.rowwise_keep_mask(7, 256, 768)
    assert abs(big.mean() - 0.9) < 0.005


def test_attn_mask_depends_on_q_plus_k_only():
    m = philox.attn_keep_mask(3, 2, 8, 8)
    # moving one step along an anti-diagonal leaves q+k, and so the keep bit, unchanged
    assert (m[:, 1:, :-1] == m[:, :-1, 1:]).all()
    q, k = np.meshgrid(np.arange(8), np.arange(8), indexing="ij")
    line = philox.tl_rand(np.int64(3 + 1), np.arange(15)) > np.float32(0.1)
    assert (m[1] == line[q + k]).all()


def _tl_rand_fixture():
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tl_rand_v1.npz")
    return np.load(path)


def test_tl_rand_matches_the_triton_package():
    """oracle.philox against values written by the installed Triton package's own tl.rand
    (tests/golden/make_tl_rand.py): the seed -> key split, the offset -> counter word, the
    choice of output word 0 and the float fold are all fixed by these, bit for bit."""
    fx = _tl_rand_fixture()
    for s in fx["seeds"].tolist():
        rows_u = fx["rows_u_%d" % s]
        n_rows, n_cols = rows_u.shape
        got = philox.tl_rand(np.arange(n_rows, dtype=np.int64)[:, None] + np.int64(s),
                             np.arange(n_cols, dtype=np.int64)[None, :])
        assert got.dtype == np.float32 and (got.view(np.uint32) == rows_u.view(np.uint32)).all(), s
        assert (philox.rowwise_keep_mask(s, n_rows, n_cols) == fx["rows_keep_%d" % s]).all(), s
        attn_keep = fx["attn_keep_%d" % s]
        bh, tq, tk = attn_keep.shape
        assert (philox.attn_keep_mask(s, bh, tq, tk) == attn_keep).all(), s
        q, k = np.meshgrid(np.arange(tq), np.arange(tk), indexing="ij")
        u = philox.tl_rand(np.arange(bh, dtype=np.int64)[:, None, None] + np.int64(s), (q + k)[None])
        assert (u.view(np.uint32) == fx["attn_u_%d" % s].view(np.uint32)).all(), s
    # the fixture exercises both decisions
    assert not fx["rows_keep_42"].all() and fx["rows_keep_42"].any()
