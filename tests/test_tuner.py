"""Candidate selection of the tuner (host logic, no GPU) and, marked gpu, the timing loop."""
import numpy as np
import pytest

import helpers as H
from cumm_amd import pairs, tuner
from cumm_amd import tensorview as tv
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.gemm.main import GemmMainUnitTest
from cumm_amd.tensorview.gemm import ConvOpType, ConvParams, GemmParams, ShuffleStrideType


def _host_conv_params(op, dtype, c_in, k_out, n=500, kv=27):
    p = ConvParams(3, op)
    p.conv_algo_desp = H.find_conv_desp(dtype, op, 64, 64, int8_inference=(dtype == "s8"))
    np_dt = {"f16": np.float16, "s8": np.int8}[dtype]
    p.input = tv.from_numpy(np.zeros((n, c_in), np_dt))
    p.weight = tv.from_numpy(np.zeros((k_out, kv, c_in), np_dt))
    p.output = tv.from_numpy(np.zeros((n, k_out), np_dt))
    p.indices = tv.from_numpy(np.zeros((kv, n), np.int32))
    p.mask_width = 64
    return p


def test_conv_candidates_share_the_kind_and_accept_the_problem():
    p = _host_conv_params(ConvOpType.Forward, "f16", 64, 64)
    cands = tuner.conv_candidates(p)
    tiles = sorted(tuple(d.tile_shape[:2]) for d in cands)
    assert tiles == [(64, 64), (64, 128), (128, 64), (128, 128)]
    assert all(d.dtype_a == tv.float16 and ConvOpType(d.op_type) == ConvOpType.Forward and
               not d.is_int8_inference for d in cands)
    # channels that are not a multiple of the access width: nothing supports them
    assert tuner.conv_candidates(_host_conv_params(ConvOpType.Forward, "f16", 60, 64)) == []
    # a contraction of more than 128 bytes: the 128 x 128 tile is a candidate with two and with three stages
    long_c = tuner.conv_candidates(_host_conv_params(ConvOpType.Forward, "f16", 128, 64))
    assert sorted(d.num_stage for d in long_c if tuple(d.tile_shape[:2]) == (128, 128)) == [2, 3]
    assert all(d.num_stage == 2 for d in long_c if tuple(d.tile_shape[:2]) != (128, 128))
    # (backward-input contracts over the output channels)
    long_k = tuner.conv_candidates(_host_conv_params(ConvOpType.BackwardInput, "f16", 64, 128))
    assert sorted(d.num_stage for d in long_k if tuple(d.tile_shape[:2]) == (128, 128)) == [2, 3]
    # int8 inference descriptors stay among themselves
    s8 = tuner.conv_candidates(_host_conv_params(ConvOpType.Forward, "s8", 64, 128))
    assert s8 and all(d.is_int8_inference and d.dtype_a == tv.int8 for d in s8)
    # backward-weight: serial and balanced split-k variants are both candidates, and split_k_slices > 1
    # keeps only descriptors with a split-k variant
    pw = _host_conv_params(ConvOpType.BackwardWeight, "f16", 64, 64)
    pw.split_k_slices = 8
    cw = tuner.conv_candidates(pw)
    assert cw and all(d.split_k_serial or d.split_k_parallel for d in cw)
    assert {bool(d.split_k_parallel) for d in cw} == {False, True}
    # the key separates what must not share a cached answer
    k1 = tuner.Tuner.conv_key(p)
    assert k1 == tuner.Tuner.conv_key(_host_conv_params(ConvOpType.Forward, "f16", 64, 64, n=400))   # same bucket
    assert k1 != tuner.Tuner.conv_key(_host_conv_params(ConvOpType.Forward, "f16", 64, 64, n=5000))
    assert k1 != tuner.Tuner.conv_key(_host_conv_params(ConvOpType.BackwardInput, "f16", 64, 64))
    # two clouds of one size and a 10x different pair density do not share a cached tile
    n = p.indices.dim(1)
    assert tuner.Tuner.conv_key(p, num_pairs=2 * n) != tuner.Tuner.conv_key(p, num_pairs=20 * n)
    assert tuner.Tuner.conv_key(p, num_pairs=2 * n) == tuner.Tuner.conv_key(p, num_pairs=int(2.2 * n))
    assert tuner.Tuner.conv_key(p, num_pairs=2 * n) != k1      # unknown density is its own class
    # the light_prefix hint changes how the 64-row descriptors run: its share of the positions is in the key
    hinted = tuner.Tuner.conv_key(p)
    p.light_prefix = (n // 128) * 128
    assert tuner.Tuner.conv_key(p) != hinted
    p.light_prefix = 0
    assert tuner.Tuner.conv_key(p) == hinted


def test_gemm_candidates():
    p = GemmParams()
    p.algo_desp = H.find_gemm_desp("f16", ShuffleStrideType.ShuffleAC, 64, 64, False, True)
    p.a = tv.from_numpy(np.zeros((1000, 64), np.float16))
    p.b = tv.from_numpy(np.zeros((128, 64), np.float16))
    p.c = tv.from_numpy(np.zeros((1000, 128), np.float16))
    p.a_inds = tv.from_numpy(np.zeros((700,), np.int32))
    p.c_inds = tv.from_numpy(np.zeros((700,), np.int32))
    cands = tuner.gemm_candidates(p)
    assert len(cands) >= 2
    assert all(d.shuffle_type == p.algo_desp.shuffle_type and d.trans_b and not d.trans_a for d in cands)
    assert len({tuple(d.tile_shape[:2]) for d in cands}) == len(cands)


@pytest.mark.gpu
def test_tune_conv_picks_a_candidate_restores_the_output_and_caches():
    from oracle import conv_ref
    rng = np.random.default_rng(4)
    coords, grid = H.small_cloud(4, 3000)
    pt = pairs.subm_pairs(coords, grid)
    n = coords.shape[0]
    feat = H.to_storage(rng.normal(0, 1, size=(n, 64)).astype(np.float32), "f16")
    w = H.to_storage(rng.normal(0, 0.05, size=(64, 27, 64)).astype(np.float32), "f16")
    out0 = H.to_storage(rng.normal(0, 1, size=(n, 64)).astype(np.float32), "f16")
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp("f16", ConvOpType.Forward, 128, 128)
    p.input, p.weight, p.output = H.dev(feat, "f16"), H.dev(w, "f16"), H.dev(out0, "f16")
    p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_fwd, "i32"), H.dev(ms, "u32"), H.dev(order, "i32")
    p.mask_width = 64
    p.beta = 1.0                      # accumulating: the tuning runs must not leave traces
    t = tuner.Tuner(steps=2, warmup=1)
    res = t.tune_conv(p)
    assert len(res.tried) == 4 and res.ms == min(ms_ for _, ms_ in res.tried) and res.ms > 0
    assert p.conv_algo_desp is res.desp and str(res.desp) in [nm for nm, _ in res.tried]
    np.testing.assert_array_equal(H.host(p.output), out0)
    ConvMainUnitTest.implicit_gemm2(p)
    ref, _ = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=res.desp.tile_shape[0],
                                            dtype_in="f16", dtype_w="f16", dtype_out="f16", beta=1.0)
    assert H.rel_err(H.as_f32(H.host(p.output), "f16"), H.as_f32(ref, "f16")) < 1e-2
    # same shape again: answered from the cache, nothing is run
    p.conv_algo_desp = H.find_conv_desp("f16", ConvOpType.Forward, 128, 128)
    again = t.tune_conv(p)
    assert again is res and p.conv_algo_desp is res.desp


@pytest.mark.gpu
def test_tune_gemm_gather_scatter():
    from oracle import gemm_ref
    rng = np.random.default_rng(5)
    rows, m, n, k = 4000, 2500, 64, 64
    a = H.to_storage(rng.normal(0, 1, size=(rows, k)).astype(np.float32), "f16")
    b = H.to_storage(rng.normal(0, 0.1, size=(n, k)).astype(np.float32), "f16")
    c0 = H.to_storage(rng.normal(0, 1, size=(rows, n)).astype(np.float32), "f16")
    a_inds = rng.permutation(rows)[:m].astype(np.int32)
    c_inds = rng.permutation(rows)[:m].astype(np.int32)
    p = GemmParams()
    p.algo_desp = H.find_gemm_desp("f16", ShuffleStrideType.ShuffleAC, 128, 128, False, True)
    p.a, p.b, p.c = H.dev(a, "f16"), H.dev(b, "f16"), H.dev(c0, "f16")
    p.a_inds, p.c_inds = H.dev(a_inds, "i32"), H.dev(c_inds, "i32")
    p.alpha, p.beta = 1.0, 1.0
    res = tuner.Tuner(steps=2, warmup=1).tune_gemm(p)
    assert len(res.tried) >= 2 and p.algo_desp is res.desp
    np.testing.assert_array_equal(H.host(p.c), c0)
    GemmMainUnitTest.matmul2(p)
    ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a="f16", dtype_b="f16", dtype_c="f16", trans_b=True,
                               shuffle=gemm_ref.SHUFFLE_AC, a_inds=a_inds, c_inds=c_inds, alpha=1.0, beta=1.0)
    assert H.rel_err(H.as_f32(H.host(p.c), "f16"), H.as_f32(ref, "f16")) < 1e-2
