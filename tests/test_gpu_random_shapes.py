"""Random shapes through the mask kernels, against the oracle.

Forward, backward-input, backward-weight (tiled, balanced, fixed order) and the int8 inference
forward with channel counts, tiles, cloud sizes (1 to 9000 voxels), submanifold / strided tables,
sort orders (mask value, offset count), pair tables by row and by position, hints (looked up, off,
arbitrary), mask filters, alpha / beta, bias and ReLU drawn from a seeded generator: the
combinations the hand-picked cases of the other files do not reach.  Each case prints its
parameters before it runs.  f16 / bf16 within 1e-2 (tile masks bit-exact), int8 bit-exact.
"""
import json

import numpy as np
import pytest

import helpers as H
from oracle import conv_ref, numerics as onm
from cumm_amd import pairs, synth
from cumm_amd import tensorview as tv
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.tensorview.gemm import Activation, ConvOpType, ConvParams

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _one_case(seed):
    rng = np.random.default_rng(seed)
    dtype = rng.choice(["f16", "bf16"])
    strided = bool(rng.integers(0, 2))
    n = int(rng.choice([1, 7, 63, 64, 65, 129, 500, 2000, 4500, 9000]))
    grid = (int(rng.integers(6, 14)), int(rng.integers(10, 40)), int(rng.integers(10, 40)))
    coords = synth.clustered_voxels(rng, n, grid, int(rng.integers(1, 6)), sigma=float(rng.uniform(1.0, 4.0)))
    c_in = int(rng.choice([8, 16, 24, 32, 64, 72, 96, 128, 160, 200, 256]))
    k_out = int(rng.choice([8, 16, 40, 64, 72, 96, 128, 136, 192, 256]))
    tile = tuple(int(x) for x in rng.choice([64, 128], size=2))
    op = rng.choice(["fwd", "dgrad", "wgrad", "int8", "fwd", "dgrad"])
    by_count = bool(rng.integers(0, 2))
    by_pos = bool(rng.integers(0, 2))
    hint_mode = int(rng.integers(0, 3))       # 0 table lookup, 1 off, 2 explicit garbage
    filt = int(rng.choice([0x7FFFFFF, 0xFFFFFFFF, 0x2AAAAAA, 0x3FFF, 0x7FFC000]))
    beta = float(rng.choice([0.0, 1.0, 0.5]))
    alpha = float(rng.choice([1.0, 0.5]))
    desc = dict(seed=seed, dtype=str(dtype), strided=strided, n=coords.shape[0], c=c_in, k=k_out, tile=tile, op=str(op),
                by_count=by_count, by_pos=by_pos, hint=hint_mode, filt=hex(filt), beta=beta, alpha=alpha)
    print("case", json.dumps(desc), flush=True)
    pt = pairs.sparse_conv_pairs(coords, grid) if strided else pairs.subm_pairs(coords, grid)
    n_in, n_out = coords.shape[0], pt.indices_fwd.shape[1]
    if n_out == 0:
        return True, 0.0, desc
    feat = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
    w = H.to_storage(rng.normal(0, 0.05, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    sort_filt = filt & 0x7FFFFFF if by_count else filt
    if op == "int8":
        c8 = int(rng.choice([16, 32, 64, 96, 128, 192]))
        k8 = int(rng.choice([16, 32, 64, 128, 144]))
        feat8 = rng.integers(-127, 128, size=(n_in, c8)).astype(np.int8)
        w8 = rng.integers(-127, 128, size=(k8, 27, c8)).astype(np.int8)
        scale = rng.uniform(0.0005, 0.01, size=(k8,)).astype(np.float32)
        bias8 = rng.normal(0, 1, size=(k8,)).astype(np.float32)
        d_mask = H.dev(pt.mask_fwd, "u32")
        ms_d, order_d = pairs.sort_by_mask_device(d_mask, sort_filt, by_offset_count=by_count)
        ms, order = H.host(ms_d), H.host(order_d)
        out0 = np.zeros((n_out, k8), np.int8)
        use_add = bool(rng.integers(0, 2))
        add = rng.integers(-127, 128, size=(n_out, k8)).astype(np.int8)
        act = Activation.ReLU if rng.integers(0, 2) else Activation.None_
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp("s8", ConvOpType.Forward, *tile, int8_inference=True)
        p.input, p.weight, p.output = H.dev(feat8, "s8"), H.dev(w8, "s8"), H.dev(out0, "s8")
        p.scale, p.bias = H.dev(scale, "f32"), H.dev(bias8, "f32")
        if use_add:
            p.output_add = H.dev(add, "s8")
            p.beta = 0.5
        p.act_type = act
        d_ind = H.dev(pt.indices_fwd, "i32")
        p.indices = pairs.pairs_by_position_device(d_ind, order_d) if by_pos else d_ind
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort = ms_d, order_d
        p.mask_filter = sort_filt
        desc.update(c=c8, k=k8, add=use_add)
        ConvMainUnitTest.implicit_gemm2(p)
        ref, _ = conv_ref.implicit_gemm_fwd_ref(feat8, w8, out0, pt.indices_fwd, ms, order, tile_m=tile[0], dtype_in="s8",
                                                dtype_w="s8", dtype_out="s8", mask_filter=sort_filt, scale=scale, bias=bias8,
                                                output_add=add if use_add else None, beta=p.beta, act=act.value,
                                                int8_inference=True)
        err = float((H.host(p.output) != ref).sum())
        ok = err == 0
    elif op == "fwd":
        d_mask = H.dev(pt.mask_fwd, "u32")
        ms_d, order_d = pairs.sort_by_mask_device(d_mask, sort_filt, by_offset_count=by_count)
        ms, order = H.host(ms_d), H.host(order_d)
        # the sorted masks hold mask & filter: the conv filter is the same one
        out0 = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
        use_bias = bool(rng.integers(0, 2)) and beta == 1.0
        bias = H.to_storage(rng.normal(0, 1, size=(k_out,)).astype(np.float32), dtype) if use_bias else None
        act = rng.choice([onm.ACT_NONE, onm.ACT_RELU])
        ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=tile[0], dtype_in=dtype,
                                                     dtype_w=dtype, dtype_out=dtype, mask_filter=sort_filt, alpha=alpha, beta=beta,
                                                     bias=bias, act=act)
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, *tile)
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
        d_ind = H.dev(pt.indices_fwd, "i32")
        p.indices = pairs.pairs_by_position_device(d_ind, order_d) if by_pos else d_ind
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort = ms_d, order_d
        p.mask_filter = sort_filt
        tiles = (n_out + tile[0] - 1) // tile[0]
        p.mask_output = tv.zeros([tiles], tv.uint32, 0)
        p.alpha, p.beta = alpha, beta
        if bias is not None:
            p.bias = H.dev(bias, dtype)
        p.act_type = Activation.ReLU if act == onm.ACT_RELU else Activation.None_
        p.light_prefix = 0 if hint_mode == 0 else (-1 if hint_mode == 1 else int(rng.integers(1, n_out + 200)))
        ConvMainUnitTest.implicit_gemm2(p)
        got = H.as_f32(H.host(p.output), dtype)
        err = H.rel_err(got, H.as_f32(ref, dtype))
        ok = err < TOL and (H.host(p.mask_output) == ref_mo).all()
    elif op == "dgrad":
        reverse = (not strided) and bool(rng.integers(0, 2))
        src_mask = pt.mask_fwd if reverse else pt.mask_bwd
        d_mask = H.dev(src_mask, "u32")
        ms_d, order_d = pairs.sort_by_mask_device(d_mask, sort_filt, by_offset_count=by_count)
        ms, order = H.host(ms_d), H.host(order_d)
        din0 = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
        # with reverse_mask the filter applies to the reversed tile mask: keep all bits then
        f2 = 0x7FFFFFF if reverse else sort_filt
        if reverse:
            ms_d, order_d = pairs.sort_by_mask_device(d_mask, 0x7FFFFFF, by_offset_count=by_count)
            ms, order = H.host(ms_d), H.host(order_d)
        ref = conv_ref.implicit_gemm_dgrad_ref(dout, w, din0, pt.indices_bwd, ms, order, tile_m=tile[0], dtype_in=dtype,
                                               dtype_w=dtype, dtype_out=dtype, mask_filter=f2, reverse_mask=reverse,
                                               alpha=alpha, beta=beta)
        p = ConvParams(3, ConvOpType.BackwardInput)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, *tile)
        p.input, p.weight, p.output = H.dev(din0, dtype), H.dev(w, dtype), H.dev(dout, dtype)
        d_ind = H.dev(pt.indices_bwd, "i32")
        p.indices = pairs.pairs_by_position_device(d_ind, order_d) if by_pos else d_ind
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort = ms_d, order_d
        p.mask_filter = f2
        p.reverse_mask = reverse
        p.alpha, p.beta = alpha, beta
        p.light_prefix = 0 if hint_mode == 0 else (-1 if hint_mode == 1 else int(rng.integers(1, n_in + 200)))
        ConvMainUnitTest.implicit_gemm2(p)
        got = H.as_f32(H.host(p.input), dtype)
        err = H.rel_err(got, H.as_f32(ref, dtype))
        ok = err < TOL
    else:
        ms, order = pairs.sort_by_mask(pt.mask_fwd, sort_filt, by_offset_count=by_count)
        mask_width = int(rng.choice([32, 64, 128]))
        red = conv_ref.tile_masks(ms, mask_width)
        dw0 = H.to_storage(rng.normal(0, 1, size=(k_out, 27, c_in)).astype(np.float32), dtype)
        parallel = bool(rng.integers(0, 2))
        det = parallel and bool(rng.integers(0, 2))
        split_k = int(rng.choice([2, 4, 32])) if parallel else int(rng.choice([1, 4]))
        ref = conv_ref.implicit_gemm_wgrad_ref(dout, feat, dw0, pt.indices_fwd, red, order, mask_width=mask_width, dtype_dout=dtype,
                                               dtype_in=dtype, dtype_w=dtype, mask_filter=sort_filt, alpha=alpha, beta=beta,
                                               split_k_slices=1 if parallel else split_k, tile_k=32)
        p = ConvParams(3, ConvOpType.BackwardWeight)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True) if parallel \
            else H.find_conv_desp(dtype, ConvOpType.BackwardWeight, tile[0], tile[0])
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(dw0, dtype), H.dev(dout, dtype)
        p.indices = H.dev(pt.indices_fwd, "i32")
        p.mask, p.mask_argsort = H.dev(red, "u32"), H.dev(order, "i32")
        p.mask_width, p.split_k_slices = mask_width, split_k
        p.mask_filter = sort_filt
        p.alpha, p.beta = alpha, beta
        p.deterministic = det
        desc.update(mw=mask_width, parallel=parallel, det=det, split_k=split_k)
        ConvMainUnitTest.implicit_gemm2(p)
        got = H.as_f32(H.host(p.weight), dtype)
        err = H.rel_err(got, H.as_f32(ref, dtype))
        ok = err < TOL
    return ok, err, desc


@pytest.mark.parametrize("block", range(6))
def test_random_shapes_against_the_oracle(block):
    bad = []
    for it in range(60):
        ok, err, desc = _one_case(7000000 + block * 1000 + it)
        if not ok:
            bad.append((desc, err))
    assert not bad, bad
