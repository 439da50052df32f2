"""Pins for the GEMM oracle: textbook identities that a dropped term, a swapped operand or a
wrong index would break, and the dense / gather-scatter plumbing case (A[512,256] @ B[256,384])."""
import numpy as np

from oracle import gemm_ref as gr
from oracle import numerics as nm


def _r(rng, shape):
    return rng.uniform(-1, 1, size=shape).astype(np.float32)


def test_config1_dense_and_gather_scatter_fp32():
    rng = np.random.default_rng(2024)
    a, b = _r(rng, (512, 256)), _r(rng, (256, 384))
    c = gr.matmul2_ref(a, b, np.zeros((512, 384), np.float32), dtype_a="f32", dtype_b="f32", dtype_c="f32")
    np.testing.assert_allclose(c, a @ b, rtol=1e-6, atol=1e-6)
    # gather 384 A rows by a random permutation prefix, scatter-add the rows into zeros[1024, 384]
    a_inds = rng.permutation(512)[:384].astype(np.int32)
    c_inds = rng.permutation(1024)[:384].astype(np.int32)
    out = gr.matmul2_ref(a, b, np.zeros((1024, 384), np.float32), dtype_a="f32", dtype_b="f32",
                         dtype_c="f32", shuffle=gr.SHUFFLE_AC, a_inds=a_inds, c_inds=c_inds, beta=1.0)
    want = np.zeros((1024, 384), np.float32)
    np.add.at(want, c_inds, a[a_inds] @ b)
    np.testing.assert_allclose(out, want, rtol=1e-6, atol=1e-6)
    untouched = np.setdiff1d(np.arange(1024), c_inds)
    assert not out[untouched].any()


def test_transposes_and_trans_c():
    rng = np.random.default_rng(1)
    m, n, k = 24, 40, 16
    A, B = _r(rng, (m, k)), _r(rng, (k, n))
    want = A @ B
    for ta in (False, True):
        for tb in (False, True):
            for tc in (False, True):
                a = np.ascontiguousarray(A.T) if ta else A
                b = np.ascontiguousarray(B.T) if tb else B
                c0 = np.zeros((n, m) if tc else (m, n), np.float32)
                got = gr.matmul2_ref(a, b, c0, dtype_a="f32", dtype_b="f32", dtype_c="f32",
                                     trans_a=ta, trans_b=tb, trans_c=tc)
                np.testing.assert_allclose(got.T if tc else got, want, rtol=1e-6, atol=1e-6)


def test_shuffle_ac_identity_indices_equal_dense_and_alpha_beta_bias():
    rng = np.random.default_rng(2)
    m, n, k = 50, 32, 16
    a, b, c0 = _r(rng, (m, k)), _r(rng, (k, n)), _r(rng, (m, n))
    ident = np.arange(m, dtype=np.int32)
    dense = gr.matmul2_ref(a, b, c0, dtype_a="f32", dtype_b="f32", dtype_c="f32", alpha=0.5, beta=2.0)
    np.testing.assert_allclose(dense, 0.5 * (a @ b) + 2.0 * c0, rtol=1e-6, atol=1e-6)
    sh = gr.matmul2_ref(a, b, c0, dtype_a="f32", dtype_b="f32", dtype_c="f32", shuffle=gr.SHUFFLE_AC,
                        a_inds=ident, c_inds=ident, alpha=0.5, beta=2.0)
    np.testing.assert_array_equal(sh, dense)
    bias = _r(rng, (n,))
    withb = gr.matmul2_ref(a, b, c0, dtype_a="f32", dtype_b="f32", dtype_c="f32", d=bias, beta=1.0,
                           act=nm.ACT_RELU)
    np.testing.assert_allclose(withb, np.maximum(a @ b + bias[None, :], 0), rtol=1e-6, atol=1e-6)
    # beta == 0: the old contents of C (even NaN) must not leak into the result
    poisoned = np.full((m, n), np.nan, np.float32)
    clean = gr.matmul2_ref(a, b, poisoned, dtype_a="f32", dtype_b="f32", dtype_c="f32")
    assert np.isfinite(clean).all()


def test_shuffle_ab_is_gathered_transposed_product():
    rng = np.random.default_rng(3)
    rows, kk, m, n = 70, 33, 8, 16
    a, b = _r(rng, (rows, m)), _r(rng, (rows, n))
    ai = rng.permutation(rows)[:kk].astype(np.int32)
    bi = rng.permutation(rows)[:kk].astype(np.int32)
    got = gr.matmul2_ref(a, b, np.zeros((m, n), np.float32), dtype_a="f32", dtype_b="f32", dtype_c="f32",
                         trans_a=True, shuffle=gr.SHUFFLE_AB, a_inds=ai, b_inds=bi)
    want = sum(np.outer(a[i], b[j]) for i, j in zip(ai, bi))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_int8_accumulator_is_exact_and_f16_rounds_once():
    rng = np.random.default_rng(4)
    a = rng.integers(-127, 128, size=(40, 512)).astype(np.int8)
    b = rng.integers(-127, 128, size=(512, 24)).astype(np.int8)
    acc = gr._matmul_acc(a, b, "s8", "s8")
    np.testing.assert_array_equal(acc, a.astype(np.int64) @ b.astype(np.int64))
    af, bf = rng.normal(0, 1, (16, 64)).astype(np.float16), rng.normal(0, 1, (64, 8)).astype(np.float16)
    got = gr.matmul2_ref(af, bf, np.zeros((16, 8), np.float16), dtype_a="f16", dtype_b="f16", dtype_c="f16")
    want = (af.astype(np.float64) @ bf.astype(np.float64))
    np.testing.assert_allclose(got.astype(np.float64), want, rtol=2e-3, atol=2e-3)
    assert got.dtype == np.float16


def test_s32_output_is_integer_arithmetic():
    """Output type s32 of s8 operands: alpha and beta become integers (C conversion, toward zero)
    and alpha*acc + beta*src is integer arithmetic.  Pinned by a brute-force product in Python
    integers, by the conversion numpy's C cast makes, and by wrap-around at 2^31."""
    rng = np.random.default_rng(11)
    m, n, k = 5, 7, 9
    a = rng.integers(-127, 128, size=(m, k)).astype(np.int8)
    b = rng.integers(-127, 128, size=(k, n)).astype(np.int8)
    c0 = rng.integers(-10 ** 6, 10 ** 6, size=(m, n)).astype(np.int32)
    brute = [[sum(int(a[i, t]) * int(b[t, j]) for t in range(k)) for j in range(n)] for i in range(m)]
    got = gr.matmul2_ref(a, b, c0, dtype_a="s8", dtype_b="s8", dtype_c="s32")
    assert got.dtype == np.int32 and got.tolist() == brute
    got = gr.matmul2_ref(a, b, c0, dtype_a="s8", dtype_b="s8", dtype_c="s32", alpha=3.0, beta=-2.0)
    assert got.tolist() == [[3 * brute[i][j] - 2 * int(c0[i, j]) for j in range(n)] for i in range(m)]
    # fractional parameters convert toward zero: 2.9 -> 2, -1.5 -> -1, 0.5 -> 0 (source not needed)
    for alpha, beta in ((2.9, -1.5), (-2.9, 0.5)):
        ai, bi = int(np.float32(alpha).astype(np.int32)), int(np.float32(beta).astype(np.int32))
        got = gr.matmul2_ref(a, b, c0, dtype_a="s8", dtype_b="s8", dtype_c="s32", alpha=alpha, beta=beta)
        assert got.tolist() == [[ai * brute[i][j] + bi * int(c0[i, j]) for j in range(n)] for i in range(m)]
    # ReLU and LeakyReLU on integers
    got = gr.matmul2_ref(a, b, c0, dtype_a="s8", dtype_b="s8", dtype_c="s32", act=nm.ACT_RELU)
    assert got.tolist() == [[max(v, 0) for v in row] for row in brute]
    got = gr.matmul2_ref(a, b, c0, dtype_a="s8", dtype_b="s8", dtype_c="s32", act=nm.ACT_LEAKY_RELU, act_alpha=3.7)
    assert got.tolist() == [[v if v >= 0 else 3 * v for v in row] for row in brute]
    # overflow wraps modulo 2^32
    big = gr.linear_combination_s32(np.array([2 ** 30 + 5], np.int32), None, 4.0, 0.0, nm.ACT_NONE, 0.0)
    assert int(big[0]) == ((4 * (2 ** 30 + 5) + 2 ** 31) % 2 ** 32) - 2 ** 31 == 20


def test_serial_split_k_slices_round_between_slices():
    """Slices are contiguous ranges of k of ceil(ceil(k / tile_k) / slices) * tile_k elements (the
    size is pinned against the reference's header in test_desp.py); every slice after the first
    adds onto the rounded result of the one before."""
    assert gr.split_k_ranges(656, 4, 32) == [(0, 192), (192, 384), (384, 576), (576, 656)]
    assert gr.split_k_ranges(64, 4, 32) == [(0, 32), (32, 64), (64, 64), (64, 64)]
    assert gr.split_k_ranges(100, 3, 64) == [(0, 64), (64, 100), (100, 100)]
    rng = np.random.default_rng(12)
    m, n, k = 6, 10, 100
    a = rng.normal(0, 1, size=(m, k)).astype(np.float16)
    b = rng.normal(0, 1, size=(k, n)).astype(np.float16)
    c0 = rng.normal(0, 1, size=(m, n)).astype(np.float16)
    got = gr.matmul2_ref(a, b, c0, dtype_a="f16", dtype_b="f16", dtype_c="f16", alpha=0.5, beta=2.0,
                         split_k_slices=3, tile_k=64)
    af, bf = a.astype(np.float32), b.astype(np.float32)
    step1 = (np.float32(0.5) * (af[:, :64] @ bf[:64]) + np.float32(2.0) * c0.astype(np.float32)).astype(np.float16)
    step2 = (np.float32(0.5) * (af[:, 64:] @ bf[64:]) + step1.astype(np.float32)).astype(np.float16)
    # (fused vs unfused multiply-add may differ in the last f16 digit)
    assert np.max(np.abs(got.astype(np.float32) - step2.astype(np.float32))) <= 2 * np.max(np.abs(np.spacing(step2)))
    one = gr.matmul2_ref(a, b, c0, dtype_a="f16", dtype_b="f16", dtype_c="f16", alpha=0.5, beta=2.0)
    assert np.any(one != got)        # a single rounding is not the same thing
    # integers: exact whatever the slicing
    ai = rng.integers(-127, 128, size=(m, 300)).astype(np.int8)
    bi = rng.integers(-127, 128, size=(300, n)).astype(np.int8)
    ci = rng.integers(-1000, 1000, size=(m, n)).astype(np.int32)
    s1 = gr.matmul2_ref(ai, bi, ci, dtype_a="s8", dtype_b="s8", dtype_c="s32", beta=1.0)
    s4 = gr.matmul2_ref(ai, bi, ci, dtype_a="s8", dtype_b="s8", dtype_c="s32", beta=1.0, split_k_slices=4, tile_k=64)
    np.testing.assert_array_equal(s1, s4)
