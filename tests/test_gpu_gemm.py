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
    if dtype in ("s8", "s32"):
        np.testing.assert_array_equal(got, ref)
    else:
        assert H.rel_err(H.as_f32(got, dtype), H.as_f32(ref, dtype)) < TOL


WIDE = {"s8": "s32", "f16": "f32", "bf16": "f32"}   # output in the accumulator's type
TILE_K = {"s8": 64, "f16": 32, "bf16": 32}


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
        # serial split-K: the oracle takes the same contiguous slices of k and rounds the partial
        # results to the output type between slices, in slice order
        ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype,
                                   trans_a=ta, trans_b=tb, trans_c=trans_c, alpha=alpha, beta=beta,
                                   split_k_slices=split, tile_k=TILE_K[dtype])
        _compare(H.host(p.c), ref, dtype)


@pytest.mark.parametrize("dtype", ["s8", "f16", "bf16"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 128)])
@pytest.mark.parametrize("trans", [(False, False), (False, True), (True, False), (True, True)])
def test_dense_accumulator_output(dtype, tile, trans):
    """Output in the accumulator's type: s8 x s8 -> s32 bit-exact (integer linear combination, also
    across serial split-K slices), f16 / bf16 -> f32."""
    print("case dense wide", dtype, tile, trans, flush=True)
    rng = np.random.default_rng(4242)
    m, n, k = 208, 144, 656
    ta, tb = trans
    out = WIDE[dtype]
    a = _rand(rng, (k, m) if ta else (m, k), dtype)
    b = _rand(rng, (n, k) if tb else (k, n), dtype, 0.1 if dtype != "s8" else 1.0)
    if out == "s32":
        c0 = rng.integers(-100000, 100000, size=(m, n)).astype(np.int32)
    else:
        c0 = rng.normal(0, 1, size=(m, n)).astype(np.float32)
    for alpha, beta, split, trans_c in ((1.0, 0.0, 1, False), (2.0, -3.0, 1, False), (1.0, 1.0, 4, False),
                                        (3.0, 1.0, 1, True)):
        cc = np.ascontiguousarray(c0.T) if trans_c else c0
        p = GemmParams()
        p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.NoShuffle, *tile, ta, tb, trans_c, dtype_c=out)
        p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(cc, out)
        p.alpha, p.beta = alpha, beta
        p.split_k_slices = split
        GemmMainUnitTest.matmul2(p)
        ref = gemm_ref.matmul2_ref(a, b, cc, dtype_a=dtype, dtype_b=dtype, dtype_c=out, trans_a=ta, trans_b=tb,
                                   trans_c=trans_c, alpha=alpha, beta=beta, split_k_slices=split,
                                   tile_k=TILE_K[dtype])
        got = H.host(p.c)
        if out == "s32":
            np.testing.assert_array_equal(got, ref)
            if alpha == 1.0 and beta == 0.0:   # the raw accumulators: the textbook integer product
                am = (a.T if ta else a).astype(np.int64)
                bm = (b.T if tb else b).astype(np.int64)
                np.testing.assert_array_equal(got.astype(np.int64), am @ bm)
        else:
            assert H.rel_err(got, ref) < 2e-3      # no output rounding: only the order of the fp32 sums differs


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("n,k", [(64, 64), (64, 128), (40, 96), (8, 8), (56, 32), (64, 24)])
@pytest.mark.parametrize("wide", [False, True])
def test_shuffle_ac_one_column_block(dtype, trans_b, n, k, wide):
    """Up to 64 output channels and 128 contraction elements: the kernel that keeps the weight matrix
    in registers and gathers rows straight into operand registers (csrc/rowgemm_wave.h); ragged
    row counts, identity and permuted rows, a 2-D source, a bias, ReLU, f32 outputs."""
    print("case shuffle_ac one block", dtype, trans_b, n, k, wide, flush=True)
    rng = np.random.default_rng(4242)
    rows = 3000
    out = WIDE[dtype] if wide else dtype
    b = _rand(rng, (k, n), dtype, 0.1)
    bb = np.ascontiguousarray(b.T) if trans_b else b
    a = _rand(rng, (rows, k), dtype)
    for m, with_a in ((2777, True), (33, True), (rows, False), (1, True)):
        a_inds = rng.permutation(rows)[:m].astype(np.int32)
        c_inds = rng.permutation(rows)[:m].astype(np.int32)
        c0 = rng.normal(0, 1, size=(rows, n)).astype(np.float32) if wide else _rand(rng, (rows, n), dtype)
        bias = rng.normal(0, 1, size=(n,)).astype(np.float32) if wide else _rand(rng, (n,), dtype)
        for alpha, beta, act, use_bias in ((1.0, 0.0, Activation.None_, False), (0.5, 1.0, Activation.ReLU, False),
                                           (1.0, 1.0, Activation.LeakyReLU, True)):
            p = GemmParams()
            p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAC, 64, 64, False, trans_b, dtype_c=out)
            p.a, p.b, p.c = H.dev(a, dtype), H.dev(bb, dtype), H.dev(c0, out)
            if with_a:
                p.a_inds = H.dev(a_inds, "i32")
            p.c_inds = H.dev(c_inds, "i32")
            if use_bias:
                p.d = H.dev(bias, out)
            p.alpha, p.beta, p.act_type, p.act_alpha = alpha, beta, act, 0.1
            GemmMainUnitTest.matmul2(p)
            ref = gemm_ref.matmul2_ref(a if with_a else a[:m], bb, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=out,
                                       trans_b=trans_b, shuffle=gemm_ref.SHUFFLE_AC,
                                       a_inds=a_inds if with_a else None, c_inds=c_inds,
                                       d=bias if use_bias else None, alpha=alpha, beta=beta, act=act.value,
                                       act_alpha=0.1)
            got = H.host(p.c)
            if wide:
                assert H.rel_err(got, ref) < 2e-3
            else:
                _compare(got, ref, dtype)


@pytest.mark.parametrize("dtype", ["s8", "f16", "bf16"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 64), (64, 128), (128, 128)])
@pytest.mark.parametrize("trans_b", [True, False])
def test_shuffle_ac_accumulator_output(dtype, tile, trans_b):
    print("case shuffle_ac wide", dtype, tile, trans_b, flush=True)
    rng = np.random.default_rng(777)
    rows, m, n, k = 4000, 3001, 144, 128
    out = WIDE[dtype]
    a = _rand(rng, (rows, k), dtype)
    b = _rand(rng, (k, n), dtype, 0.1 if dtype != "s8" else 1.0)
    bb = np.ascontiguousarray(b.T) if trans_b else b
    a_inds = rng.permutation(rows)[:m].astype(np.int32)
    c_inds = rng.permutation(rows)[:m].astype(np.int32)
    c0 = (rng.integers(-100000, 100000, size=(rows, n)).astype(np.int32) if out == "s32"
          else rng.normal(0, 1, size=(rows, n)).astype(np.float32))
    for alpha, beta, act in ((1.0, 0.0, Activation.None_), (2.0, 1.0, Activation.ReLU)):
        p = GemmParams()
        p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAC, *tile, False, trans_b, dtype_c=out)
        p.a, p.b, p.c = H.dev(a, dtype), H.dev(bb, dtype), H.dev(c0, out)
        p.a_inds, p.c_inds = H.dev(a_inds, "i32"), H.dev(c_inds, "i32")
        p.alpha, p.beta, p.act_type = alpha, beta, act
        GemmMainUnitTest.matmul2(p)
        ref = gemm_ref.matmul2_ref(a, bb, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=out, trans_b=trans_b,
                                   shuffle=gemm_ref.SHUFFLE_AC, a_inds=a_inds, c_inds=c_inds, alpha=alpha,
                                   beta=beta, act=act.value)
        got = H.host(p.c)
        if out == "s32":
            np.testing.assert_array_equal(got, ref)
        else:
            assert H.rel_err(got, ref) < 2e-3


@pytest.mark.parametrize("dtype", ["f16", "bf16", "s8"])
def test_shuffle_ac_long_contraction(dtype):
    """k beyond eight stage rows (512 two-byte / 1024 one-byte elements): the chunked
    register-gather kernel serves these shapes."""
    print("case shuffle_ac long k", dtype, flush=True)
    rng = np.random.default_rng(99)
    rows, m, n = 900, 700, 64
    k = 640 if dtype != "s8" else 1152
    a = _rand(rng, (rows, k), dtype)
    b = _rand(rng, (k, n), dtype, 0.1)
    a_inds = rng.permutation(rows)[:m].astype(np.int32)
    c_inds = rng.permutation(rows)[:m].astype(np.int32)
    c0 = _rand(rng, (rows, n), dtype)
    alpha = 1.0 if dtype != "s8" else 1e-5
    for trans_b in (True, False):
        bb = np.ascontiguousarray(b.T) if trans_b else b
        p = GemmParams()
        p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAC, 64, 64, False, trans_b)
        p.a, p.b, p.c = H.dev(a, dtype), H.dev(bb, dtype), H.dev(c0, dtype)
        p.a_inds, p.c_inds = H.dev(a_inds, "i32"), H.dev(c_inds, "i32")
        p.alpha, p.beta = alpha, 1.0
        GemmMainUnitTest.matmul2(p)
        ref = gemm_ref.matmul2_ref(a, bb, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype, trans_b=trans_b,
                                   shuffle=gemm_ref.SHUFFLE_AC, a_inds=a_inds, c_inds=c_inds, alpha=alpha, beta=1.0)
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
    # ... and follow it: the oracle with the same slices
    ref_s = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype, trans_a=True,
                                 shuffle=gemm_ref.SHUFFLE_AB, a_inds=a_inds, b_inds=b_inds, alpha=0.01,
                                 split_k_slices=split, tile_k=32)
    assert H.rel_err(H.as_f32(H.host(p.c), dtype), H.as_f32(ref_s, dtype)) < TOL


@pytest.mark.parametrize("out", ["s8", "s32"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 128)])
@pytest.mark.parametrize("split", [1, 4])
def test_shuffle_ab_s8(out, tile, split):
    """C = A[a_inds]^T B[b_inds] on one-byte operands: s32 sums bit-exact, s8 results through
    the float linear combination bit-exact too (same slices, same roundings)."""
    print("case shuffle_ab s8", out, tile, split, flush=True)
    rng = np.random.default_rng(6)
    rows, kk, m, n = 3000, 2048, 64, 144
    a = _rand(rng, (rows, m), "s8")
    b = _rand(rng, (rows, n), "s8")
    a_inds = rng.permutation(rows)[:kk].astype(np.int32)
    b_inds = rng.permutation(rows)[:kk].astype(np.int32)
    c0 = (rng.integers(-1000, 1000, size=(m, n)).astype(np.int32) if out == "s32"
          else rng.integers(-127, 128, size=(m, n)).astype(np.int8))
    alpha, beta = (1.0, 1.0) if out == "s32" else (1e-5, 1.0)
    p = GemmParams()
    p.algo_desp = H.find_gemm_desp("s8", ShuffleStrideType.ShuffleAB, *tile, True, False, dtype_c=out)
    p.a, p.b, p.c = H.dev(a, "s8"), H.dev(b, "s8"), H.dev(c0, out)
    p.a_inds, p.b_inds = H.dev(a_inds, "i32"), H.dev(b_inds, "i32")
    p.split_k_slices = split
    p.alpha, p.beta = alpha, beta
    GemmMainUnitTest.matmul2(p)
    ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a="s8", dtype_b="s8", dtype_c=out, trans_a=True,
                               shuffle=gemm_ref.SHUFFLE_AB, a_inds=a_inds, b_inds=b_inds, alpha=alpha, beta=beta,
                               split_k_slices=split, tile_k=64)
    np.testing.assert_array_equal(H.host(p.c), ref)


def test_split_k_time_out_is_reported():
    """A serial split-K slice waits for its turn at most a bounded number of polls.  With the
    bound forced to one poll (from the host; every kernel still runs to its end) slices give
    up, and the next synchronisation reports that as an error instead of returning silently
    with a sum that may be wrong; the call after that is clean again."""
    from cumm_amd import _capi
    import ctypes
    lib = _capi.lib()
    rng = np.random.default_rng(8)
    m, n, k = 128, 128, 64 * 64
    a, b = _rand(rng, (m, k), "f16"), _rand(rng, (n, k), "f16", 0.1)
    p = GemmParams()
    p.algo_desp = H.find_gemm_desp("f16", ShuffleStrideType.NoShuffle, 64, 64, False, True)
    p.a, p.b, p.c = H.dev(a, "f16"), H.dev(b, "f16"), H.dev(np.zeros((m, n), np.float16), "f16")
    p.split_k_slices = 64
    GemmMainUnitTest.device_synchronize()
    try:
        _capi.check(lib.cumm_hip_set_split_k_spin_limit(1))
        GemmMainUnitTest.matmul2(p)
        with pytest.raises(RuntimeError, match="split-K"):
            GemmMainUnitTest.device_synchronize()
    finally:
        _capi.check(lib.cumm_hip_set_split_k_spin_limit(0))
    GemmMainUnitTest.device_synchronize()          # reported once, then cleared
    p.c = H.dev(np.zeros((m, n), np.float16), "f16")
    GemmMainUnitTest.matmul2(p)
    GemmMainUnitTest.device_synchronize()          # the default bound: no time-out
    cnt = ctypes.c_int32(-1)
    _capi.check(lib.cumm_hip_take_async_errors(ctypes.byref(cnt)))
    assert cnt.value == 0
    ref = gemm_ref.matmul2_ref(a, b, np.zeros((m, n), np.float16), dtype_a="f16", dtype_b="f16", dtype_c="f16",
                               trans_b=True, split_k_slices=64, tile_k=32)
    assert H.rel_err(H.as_f32(H.host(p.c), "f16"), H.as_f32(ref, "f16")) < TOL
