"""The gather / scatter-add oracle against properties that hold whatever the implementation."""
import numpy as np

from oracle import gather_ref


def test_gather_identity_permutation_and_inverse():
    rng = np.random.default_rng(1)
    a = rng.normal(size=(257, 24)).astype(np.float32)
    np.testing.assert_array_equal(gather_ref.gather_rows_ref(a, np.arange(257)), a)
    perm = rng.permutation(257)
    inv = np.empty_like(perm)
    inv[perm] = np.arange(257)
    g = gather_ref.gather_rows_ref(a, perm)
    assert not np.array_equal(g, a)
    np.testing.assert_array_equal(gather_ref.gather_rows_ref(g, inv), a)
    # row i of the result is row perm[i] of the input, not the other way round
    np.testing.assert_array_equal(g[3], a[perm[3]])
    # out-of-range indices give zeros, repeated indices repeat rows
    g2 = gather_ref.gather_rows_ref(a, np.array([5, -1, 5, 257]))
    np.testing.assert_array_equal(g2[0], a[5])
    np.testing.assert_array_equal(g2[2], a[5])
    assert not g2[1].any() and not g2[3].any()


def test_scatter_add_is_one_hot_product_and_counts():
    rng = np.random.default_rng(2)
    m, rows, c = 100, 150, 8
    idx = rng.permutation(rows)[:m]
    inp = rng.integers(-8, 9, size=(m, c)).astype(np.float32)     # small integers: sums are exact
    out = rng.integers(-8, 9, size=(rows, c)).astype(np.float32)
    onehot = np.zeros((rows, m), np.float32)
    onehot[idx, np.arange(m)] = 1.0
    np.testing.assert_array_equal(gather_ref.scatter_add_rows_ref(out, inp, idx), out + onehot @ inp)
    ones = gather_ref.scatter_add_rows_ref(np.zeros((rows, 1), np.float32), np.ones((m, 1), np.float32), idx)
    np.testing.assert_array_equal(ones[:, 0], np.bincount(idx, minlength=rows).astype(np.float32))
    # scatter-add undoes itself with the negated input; the caller's output is not modified
    back = gather_ref.scatter_add_rows_ref(gather_ref.scatter_add_rows_ref(out, inp, idx), -inp, idx)
    np.testing.assert_array_equal(back, out)
    # a dropped row
    drop = gather_ref.scatter_add_rows_ref(out, inp[:2], np.array([rows, 3]))
    np.testing.assert_array_equal(drop[3], out[3] + inp[1])
    assert np.array_equal(np.delete(drop, 3, axis=0), np.delete(out, 3, axis=0))


def test_scatter_add_f16_rounds_once():
    out = np.array([[2048.0]], np.float16)
    inp = np.array([[1.0]], np.float16)
    # 2049 is not representable in f16 (spacing 2 above 2048): ties to even = 2048
    assert gather_ref.scatter_add_rows_ref(out, inp, np.array([0]), "f16")[0, 0] == np.float16(2048.0)
    inp3 = np.array([[3.0]], np.float16)
    assert gather_ref.scatter_add_rows_ref(out, inp3, np.array([0]), "f16")[0, 0] == np.float16(2052.0)
