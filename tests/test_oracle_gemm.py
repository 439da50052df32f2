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
