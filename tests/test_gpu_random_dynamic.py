"""Random kernel volumes above 32, against the oracle: the `dynamic_mask` descriptors (forward and
backward-input in one launch over masks of several words, pair table by row or by position, the
mask of the other direction read in reverse for submanifold tables, beta / bias / ReLU epilogues)
and the per-offset convolution (forward, backward-input, backward-weight over the pair lists).

Submanifold kernels of 1 / 3 / 5 / 7 per axis and strided kernels of 2 to 6 with strides 1 / 2 and
padding 0 to 2, 33 to 128 offsets, clouds from one voxel to 3000, channel counts from 8 to 160 that
need not fill a tile, f16 and bf16 to a relative error of 1e-2.  Each case prints its parameters first.
"""
import json

import numpy as np
import pytest

import helpers as H
from oracle import conv_ref, native_ref, numerics as onm
from cumm_amd import pairs, synth
from cumm_amd import tensorview as tv
from cumm_amd.conv import native
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.tensorview.gemm import Activation, ConvOpType, ConvParams

pytestmark = pytest.mark.gpu

TOL = 1e-2


def one_case(seed):
    rng = np.random.default_rng(seed)
    dtype = str(rng.choice(["f16", "bf16"]))
    strided = bool(rng.integers(0, 2))
    grid = (int(rng.integers(5, 14)), int(rng.integers(8, 30)), int(rng.integers(8, 30)))
    n = int(rng.choice([1, 40, 65, 300, 1500, 3000]))
    coords = synth.clustered_voxels(rng, n, grid, int(rng.integers(1, 5)), sigma=float(rng.uniform(1.0, 3.5)))
    while True:
        ksize = tuple(int(x) for x in rng.choice([1, 3, 5, 7] if not strided else [2, 3, 4, 5, 6], size=3))
        kv = ksize[0] * ksize[1] * ksize[2]
        if 32 < kv <= 128:
            break
    c_in = int(rng.choice([8, 16, 32, 64, 72, 128, 160]))
    k_out = int(rng.choice([8, 24, 64, 96, 128, 136]))
    tile = int(rng.choice([64, 128]))
    op = str(rng.choice(["fwd", "dgrad", "native"]))
    by_pos = bool(rng.integers(0, 2))
    desc = dict(seed=seed, dtype=dtype, strided=strided, n=int(coords.shape[0]), ksize=ksize, c=c_in, k=k_out, tile=tile, op=op, by_pos=by_pos)
    print("case", json.dumps(desc), flush=True)
    if strided:
        stride = tuple(int(x) for x in rng.choice([1, 2], size=3))
        padding = tuple(int(x) for x in rng.choice([0, 1, 2], size=3))
        host = pairs.sparse_conv_pairs(coords, grid, ksize, stride, padding)
        if min(host.out_shape) <= 0 or host.indices_fwd.shape[1] == 0:
            return True, 0.0, desc
        devt = pairs.sparse_conv_pairs_device(H.dev(coords, "i32"), grid, ksize, stride, padding)
    else:
        host = pairs.subm_pairs(coords, grid, ksize)
        devt = pairs.subm_pairs_device(H.dev(coords, "i32"), grid, ksize)
    n_in, n_out = coords.shape[0], host.indices_fwd.shape[1]
    words = (kv + 31) // 32
    feat = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
    w = H.to_storage(rng.normal(0, 0.03, size=(k_out, kv, c_in)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    if op == "fwd":
        mf_d = pairs.masks_from_pairs_device(devt.indices_fwd)
        ms_d, order_d = pairs.sort_by_mask_words_device(mf_d)
        ms, order = H.host(ms_d), H.host(order_d)
        out0 = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
        beta = float(rng.choice([0.0, 1.0]))
        use_bias = beta == 1.0 and bool(rng.integers(0, 2))
        bias = H.to_storage(rng.normal(0, 1, size=(k_out,)).astype(np.float32), dtype) if use_bias else None
        act = onm.ACT_RELU if rng.integers(0, 2) else onm.ACT_NONE
        ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, host.indices_fwd, ms, order, tile_m=tile, dtype_in=dtype,
                                                     dtype_w=dtype, dtype_out=dtype, beta=beta, bias=bias, act=act)
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, tile, tile, dynamic_mask=True)
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
        if bias is not None:
            p.bias = H.dev(bias, dtype)
        p.beta = beta
        p.act_type = Activation.ReLU if act == onm.ACT_RELU else Activation.None_
        p.indices = pairs.pairs_by_position_device(devt.indices_fwd, order_d) if by_pos else devt.indices_fwd
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort = ms_d, order_d
        tiles = (n_out + tile - 1) // tile
        p.mask_output = tv.zeros([tiles, words], tv.uint32, 0)
        p.mask_int_count = words
        ConvMainUnitTest.implicit_gemm2(p)
        err = H.rel_err(H.as_f32(H.host(p.output), dtype), H.as_f32(ref, dtype))
        ok = err < TOL and np.array_equal(H.host(p.mask_output), ref_mo)
    elif op == "dgrad":
        reverse = (not strided) and bool(rng.integers(0, 2))
        src = devt.indices_fwd if reverse else devt.indices_bwd
        m_d = pairs.masks_from_pairs_device(src)
        ms_d, order_d = pairs.sort_by_mask_words_device(m_d)
        din0 = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
        beta = float(rng.choice([0.0, 1.0]))
        ref = conv_ref.implicit_gemm_dgrad_ref(dout, w, din0, host.indices_bwd, H.host(ms_d), H.host(order_d), tile_m=tile,
                                               dtype_in=dtype, dtype_w=dtype, dtype_out=dtype, reverse_mask=reverse, beta=beta)
        p = ConvParams(3, ConvOpType.BackwardInput)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, tile, tile, dynamic_mask=True)
        p.input, p.weight, p.output = H.dev(din0, dtype), H.dev(w, dtype), H.dev(dout, dtype)
        p.indices = pairs.pairs_by_position_device(devt.indices_bwd, order_d) if by_pos else devt.indices_bwd
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort = ms_d, order_d
        p.reverse_mask = reverse
        p.beta = beta
        p.mask_int_count = words
        ConvMainUnitTest.implicit_gemm2(p)
        err = H.rel_err(H.as_f32(H.host(p.input), dtype), H.as_f32(ref, dtype))
        ok = err < TOL
    else:
        lists_h, lists_d = pairs.pair_lists(host.indices_fwd), pairs.pair_lists_device(devt.indices_fwd)
        which = str(rng.choice(["fwd", "dgrad", "wgrad"]))
        desc["which"] = which
        if which == "fwd":
            out = tv.zeros([n_out, k_out], H.TV_DTYPE[dtype], 0)
            native.forward(H.dev(feat, dtype), H.dev(w, dtype), out, lists_d)
            ref = native_ref.native_fwd_ref(feat, w, lists_h.pair_in, lists_h.pair_out, lists_h.counts, n_out, dtype=dtype)
            err = H.rel_err(H.as_f32(H.host(out), dtype), H.as_f32(ref, dtype))
        elif which == "dgrad":
            din = tv.zeros([n_in, c_in], H.TV_DTYPE[dtype], 0)
            native.backward_input(H.dev(dout, dtype), H.dev(w, dtype), din, lists_d)
            ref = native_ref.native_dgrad_ref(dout, w, lists_h.pair_in, lists_h.pair_out, lists_h.counts, n_in, dtype=dtype)
            err = H.rel_err(H.as_f32(H.host(din), dtype), H.as_f32(ref, dtype))
        else:
            dw = tv.zeros([k_out, kv, c_in], H.TV_DTYPE[dtype], 0)
            native.backward_weight(H.dev(dout, dtype), H.dev(feat, dtype), dw, lists_d)
            ref = native_ref.native_wgrad_ref(dout, feat, lists_h.pair_in, lists_h.pair_out, lists_h.counts, kv, dtype=dtype)
            err = H.rel_err(H.as_f32(H.host(dw), dtype), H.as_f32(ref, dtype))
        ok = err < TOL
    return ok, err, desc


@pytest.mark.parametrize("block", range(4))
def test_random_kernel_volumes_above_32(block):
    failures = []
    for it in range(60):
        ok, err, desc = one_case(7100000 + block * 1000 + it)
        if not ok:
            failures.append((desc, err))
    assert not failures, failures
