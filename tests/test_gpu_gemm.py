"""GPU parity: GemmMainUnitTest.matmul2 (-> C ABI -> HIP kernels) against the CPU oracle.

Modelled on the reference's check scripts cumm/gemm/main_real.py:171-294 (ShuffleAC /
ShuffleAB with random permutations) and :97-168 (plain GEMM, odd sizes).
"""
import numpy as np
import pytest

from oracle import gemm_ref
from oracle import numerics as onm

from cumm_amd import tensorview as tv
from cumm_amd.gemm.main import GemmMainUnitTest
from cumm_amd.tensorview.gemm import Activation, GemmParams, ShuffleStrideType

import helpers as H

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _rand(rng, shape, dtype, scale=1.0):
    if dtype == "s8":
        return rng.integers(-127, 128, size=shape).astype(np.int8)
    return H.to_storage((rng.uniform(-1, 1, size=shape) * scale).astype(np.float32), dtype)


def _compare(got, ref, dtype):
    if dtype == "s8":
        np.testing.assert_array_equal(got, ref)
    else:
        assert H.rel_err(H.as_f32(got, dtype), H.as_f32(ref, dtype)) < TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16", "s8"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 64), (64, 128), (128, 128)])
@pytest.mark.parametrize("trans_b", [True, False])
def test_shuffle_ac(dtype, tile, trans_b):
    print("case shuffle_ac", dtype, tile, trans_b, flush=True)
    rng = np.random.default_rng(12315)
    rows, m, n, k = 5000, 3777, 128, 64
    a = _rand(rng, (rows, k), dtype)
    b = _rand(rng, (k, n), dtype, 0.1)
    a_inds = rng.permutation(rows)[:m].astype(np.int32)
    c_inds = rng.permutation(rows)[:m].astype(np.int32)
    c0 = _rand(rng, (rows, n), dtype)
    alpha = 1.0 if dtype != "s8" else 1e-4
    for beta in (0.0, 1.0):
        p = GemmParams()
        p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAC, *tile, False, trans_b)
        p.a = H.dev(a, dtype)
        p.b = H.dev(np.ascontiguousarray(b.T) if trans_b else b, dtype)
        p.c = H.dev(c0, dtype)
        p.a_inds, p.c_inds = H.dev(a_inds, "i32"), H.dev(c_inds, "i32")
        p.alpha, p.beta = alpha, beta
        GemmMainUnitTest.matmul2(p)
        ref = gemm_ref.matmul2_ref(a, np.ascontiguousarray(b.T) if trans_b else b, c0,
                                   dtype_a=dtype, dtype_b=dtype, dtype_c=dtype, trans_b=trans_b,
                                   shuffle=gemm_ref.SHUFFLE_AC, a_inds=a_inds, c_inds=c_inds,
                                   alpha=alpha, beta=beta)
        _compare(H.host(p.c), ref, dtype)


def test_shuffle_ac_identity_a_bias_relu():
    dtype = "f16"
    rng = np.random.default_rng(7)
    m, n, k = 1000, 64, 64
    a, b = _rand(rng, (m, k), dtype), _rand(rng, (n, k), dtype, 0.1)
    c_inds = rng.permutation(m).astype(np.int32)
    bias = _rand(rng, (n,), dtype)
    c0 = _rand(rng, (m, n), dtype)
    p = GemmParams()
    p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAC, 64, 64, False, True)
    p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(c0, dtype)
    p.d = H.dev(bias, dtype)
    p.c_inds = H.dev(c_inds, "i32")
    p.beta = 1.0
    p.act_type = Activation.ReLU
    GemmMainUnitTest.matmul2(p)
    ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype, trans_b=True,
                               shuffle=gemm_ref.SHUFFLE_AC, c_inds=c_inds, d=bias, beta=1.0,
                               act=onm.ACT_RELU)
    _compare(H.host(p.c), ref, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "s8"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 128)])
@pytest.mark.parametrize("trans", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("trans_c", [False, True])
def test_dense(dtype, tile, trans, trans_c):
    print("case dense", dtype, tile, trans, trans_c, flush=True)
    rng = np.random.default_rng(19260817)
    m, n, k = 336, 240, 656
    ta, tb = trans
    a = _rand(rng, (k, m) if ta else (m, k), dtype)
    b = _rand(rng, (n, k) if tb else (k, n), dtype, 0.1)
    c0 = _rand(rng, (n, m) if trans_c else (m, n), dtype)
    alpha = 1.0 if dtype != "s8" else 2e-5
    for beta, split in ((0.0, 1), (1.0, 1), (1.0, 4)):
        p = GemmParams()
        p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.NoShuffle, *tile, ta, tb, trans_c)
        p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(c0, dtype)
        p.alpha, p.beta = alpha, beta
        p.split_k_slices = split
        GemmMainUnitTest.matmul2(p)
        if split > 1:
            continue  # partial sums round to the output type per slice: covered by the wgrad test
        ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype,
                                   trans_a=ta, trans_b=tb, trans_c=trans_c, alpha=alpha, beta=beta)
        _compare(H.host(p.c), ref, dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("split", [1, 8])
def test_shuffle_ab(dtype, split):
    print("case shuffle_ab", dtype, split, flush=True)
    rng = np.random.default_rng(5)
    rows, kk, m, n = 6000, 4096, 64, 128
    a = _rand(rng, (rows, m), dtype)
    b = _rand(rng, (rows, n), dtype)
    a_inds = rng.permutation(rows)[:kk].astype(np.int32)
    b_inds = rng.permutation(rows)[:kk].astype(np.int32)
    c0 = _rand(rng, (m, n), dtype)
    p = GemmParams()
    p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAB, 64, 64, True, False)
    p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(c0, dtype)
    p.a_inds, p.b_inds = H.dev(a_inds, "i32"), H.dev(b_inds, "i32")
    p.split_k_slices = split
    p.alpha = 0.01
    GemmMainUnitTest.matmul2(p)
    ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype, trans_a=True,
                               shuffle=gemm_ref.SHUFFLE_AB, a_inds=a_inds, b_inds=b_inds, alpha=0.01)
    # with split-K the partial sums round to the output type between slices: allow for it
    assert H.rel_err(H.as_f32(H.host(p.c), dtype), H.as_f32(ref, dtype)) < (TOL if split == 1 else 2 * TOL)
