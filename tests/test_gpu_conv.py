"""GPU parity: mask-based sparse convolution through ConvMainUnitTest.implicit_gemm2
(-> C ABI -> HIP kernels) against the CPU oracle on the same seeded inputs.

Modelled on the reference's own check script cumm/conv/main_real_spconv.py:54-411
(forward / backward-input / backward-weight vs per-offset gather-matmul-scatter).
Tolerance for f16/bf16: max relative error 1e-2 (fp32 accumulate); pair tables,
s32 accumulators and s8 outputs are compared bit-exactly.
"""
import numpy as np
import pytest

from oracle import conv_ref
from oracle import numerics as onm

from cumm_amd import _capi, pairs, synth
from cumm_amd import tensorview as tv
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.tensorview.gemm import Activation, ConvOpType, ConvParams

import helpers as H

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _case(seed, n, c_in, k_out, dtype, grid=(12, 40, 36), strided=False, clusters=6, sigma=3.0):
    rng = np.random.default_rng(seed)
    coords = synth.clustered_voxels(rng, n, grid, clusters, sigma=sigma)
    if strided:
        pt = pairs.sparse_conv_pairs(coords, grid)
    else:
        pt = pairs.subm_pairs(coords, grid)
    n_in = coords.shape[0]
    n_out = pt.indices_fwd.shape[1]
    if dtype == "s8":
        feat = rng.integers(-127, 128, size=(n_in, c_in)).astype(np.int8)
        w = rng.integers(-127, 128, size=(k_out, 27, c_in)).astype(np.int8)
    else:
        feat = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
        w = H.to_storage(rng.normal(0, 0.05, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    return rng, coords, pt, feat, w, n_in, n_out


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 64), (64, 128), (128, 128)])
@pytest.mark.parametrize("c_in,k_out", [(64, 64), (32, 96), (128, 128), (72, 40)])
def test_subm_forward(dtype, tile, c_in, k_out):
    print("case subm_forward", dtype, tile, c_in, k_out, flush=True)
    rng, coords, pt, feat, w, n_in, n_out = _case(1, 3000, c_in, k_out, dtype)
    mask_sorted, argsort = pairs.sort_by_mask(pt.mask_fwd)
    desp = H.find_conv_desp(dtype, ConvOpType.Forward, *tile)
    out0 = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    for beta in (0.0, 1.0):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = desp
        p.input, p.weight = H.dev(feat, dtype), H.dev(w, dtype)
        p.output = H.dev(out0, dtype)
        p.indices = H.dev(pt.indices_fwd, "i32")
        p.mask, p.mask_argsort = H.dev(mask_sorted, "u32"), H.dev(argsort, "i32")
        tiles = (n_out + tile[0] - 1) // tile[0]
        p.mask_output = tv.zeros([tiles], tv.uint32, 0)
        p.mask_width = tile[0]
        p.beta = beta
        ConvMainUnitTest.implicit_gemm2(p)
        got = H.host(p.output)
        ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(
            feat, w, out0, pt.indices_fwd, mask_sorted, argsort, tile_m=tile[0], dtype_in=dtype,
            dtype_w=dtype, dtype_out=dtype, beta=beta)
        assert H.rel_err(H.as_f32(got, dtype), H.as_f32(ref, dtype)) < TOL
        np.testing.assert_array_equal(H.host(p.mask_output), ref_mo)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_forward_bias_relu_and_mask_filter(dtype):
    rng, coords, pt, feat, w, n_in, n_out = _case(2, 2500, 64, 64, dtype)
    bias = H.to_storage(rng.normal(0, 1, size=(64,)).astype(np.float32), dtype)
    desp = H.find_conv_desp(dtype, ConvOpType.Forward, 64, 64)
    out0 = H.to_storage(np.zeros((n_out, 64), np.float32), dtype)
    # two mask splits as in cumm/conv/main_real_spconv.py:270-294: the second pass accumulates
    filters = [0x3FFF, 0x1FFF << 14]
    cur = out0
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = desp
    p.input, p.weight = H.dev(feat, dtype), H.dev(w, dtype)
    p.output = H.dev(out0, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    for j, f in enumerate(filters):
        ms, order = pairs.sort_by_mask(pt.mask_fwd, f)
        p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
        p.mask_filter = f
        p.beta = 0.0 if j == 0 else 1.0
        ConvMainUnitTest.implicit_gemm2(p)
        cur, _ = conv_ref.implicit_gemm_fwd_ref(
            feat, w, cur, pt.indices_fwd, ms, order, tile_m=64, dtype_in=dtype, dtype_w=dtype,
            dtype_out=dtype, mask_filter=f, beta=p.beta)
    assert H.rel_err(H.as_f32(H.host(p.output), dtype), H.as_f32(cur, dtype)) < TOL
    # bias as the source operand + ReLU (BN folded into the epilogue)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = desp
    p.input, p.weight = H.dev(feat, dtype), H.dev(w, dtype)
    p.output = H.dev(out0, dtype)
    p.bias = H.dev(bias, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
    p.beta = 1.0
    p.act_type = Activation.ReLU
    ConvMainUnitTest.implicit_gemm2(p)
    ref, _ = conv_ref.implicit_gemm_fwd_ref(
        feat, w, out0, pt.indices_fwd, ms, order, tile_m=64, dtype_in=dtype, dtype_w=dtype,
        dtype_out=dtype, beta=1.0, bias=bias, act=onm.ACT_RELU)
    got = H.as_f32(H.host(p.output), dtype)
    assert got.min() >= 0.0
    assert H.rel_err(got, H.as_f32(ref, dtype)) < TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 128)])
@pytest.mark.parametrize("strided", [False, True])
def test_backward_input(dtype, tile, strided):
    print("case backward_input", dtype, tile, strided, flush=True)
    c_in, k_out = 64, 96
    rng, coords, pt, feat, w, n_in, n_out = _case(3, 2500, c_in, k_out, dtype, strided=strided)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    din0 = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
    desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, *tile)
    if strided:
        ms, order = pairs.sort_by_mask(pt.mask_bwd)
        reverse = False
    else:
        # SubM: the forward mask is reused, bit-reversed inside the kernel
        ms, order = pairs.sort_by_mask(pt.mask_fwd)
        reverse = True
    p = ConvParams(3, ConvOpType.BackwardInput)
    p.conv_algo_desp = desp
    p.input, p.weight, p.output = H.dev(din0, dtype), H.dev(w, dtype), H.dev(dout, dtype)
    p.indices = H.dev(pt.indices_bwd, "i32")
    p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
    p.reverse_mask = reverse
    p.beta = 0.0
    ConvMainUnitTest.implicit_gemm2(p)
    ref = conv_ref.implicit_gemm_dgrad_ref(
        dout, w, din0, pt.indices_bwd, ms, order, tile_m=tile[0], dtype_in=dtype, dtype_w=dtype,
        dtype_out=dtype, reverse_mask=reverse)
    assert H.rel_err(H.as_f32(H.host(p.input), dtype), H.as_f32(ref, dtype)) < TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("c_in,k_out", [(64, 64), (32, 48)])
def test_light_prefix_hint_moves_work_not_results(dtype, c_in, k_out):
    """ConvParams.light_prefix sends the leading positions of the sorted order to 128-row tiles:
    whatever it says - the count pairs.light_prefix gives, too little, too much, everything - the
    output rows and the tile masks are the same bits as without it (and those are checked
    against the oracle)."""
    print("case light_prefix", dtype, c_in, k_out, flush=True)
    rng = np.random.default_rng(11)
    grid = (16, 200, 200)
    coords = synth.clustered_voxels(rng, 6000, grid, 8, sigma=4.0, noise_frac=0.6)
    pt = pairs.subm_pairs(coords, grid)
    n = coords.shape[0]
    feat = H.to_storage(rng.normal(0, 1, size=(n, c_in)).astype(np.float32), dtype)
    w = H.to_storage(rng.normal(0, 0.05, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    out0 = H.to_storage(rng.normal(0, 1, size=(n, k_out)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n, k_out)).astype(np.float32), dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    exact = pairs.light_prefix(ms)
    assert 256 <= exact <= n - 256, "the cloud should have a light end and a heavy end"
    d_ms, d_order = H.dev(ms, "u32"), H.dev(order, "i32")
    assert pairs.light_prefix_device(d_ms) == exact
    assert pairs.light_prefix_device(d_ms, mask_filter=1 << 13) == (n // 128) * 128    # the centre alone: all light
    tiles = (n + 63) // 64
    hints = (0, exact, 128, exact - 128, exact + 640, n - 1, n, n + 1000)

    def forward(hint, beta, relu, with_bias):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, 64, 64)
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
        p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_fwd, "i32"), d_ms, d_order
        p.mask_output = tv.zeros([tiles], tv.uint32, 0)
        p.beta = beta
        if with_bias:
            p.bias = H.dev(bias, dtype)
        if relu:
            p.act_type = Activation.ReLU
        p.light_prefix = hint
        ConvMainUnitTest.implicit_gemm2(p)
        return H.host(p.output), H.host(p.mask_output)

    bias = H.to_storage(rng.normal(0, 1, size=(k_out,)).astype(np.float32), dtype)
    for beta, relu, with_bias in ((0.0, False, False), (1.0, True, False), (1.0, True, True)):
        base, base_mo = forward(0, beta, relu, with_bias)
        ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(
            feat, w, out0, pt.indices_fwd, ms, order, tile_m=64, dtype_in=dtype, dtype_w=dtype, dtype_out=dtype,
            beta=beta, bias=bias if with_bias else None, act=onm.ACT_RELU if relu else onm.ACT_NONE)
        assert H.rel_err(H.as_f32(base, dtype), H.as_f32(ref, dtype)) < TOL
        np.testing.assert_array_equal(base_mo, ref_mo)
        for hint in hints[1:]:
            got, got_mo = forward(hint, beta, relu, with_bias)
            np.testing.assert_array_equal(got.view(np.uint16), base.view(np.uint16), err_msg="hint %d" % hint)
            np.testing.assert_array_equal(got_mo, base_mo, err_msg="hint %d" % hint)

    def backward_input(hint):
        p = ConvParams(3, ConvOpType.BackwardInput)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, 64, 64)
        din = H.dev(H.to_storage(np.zeros((n, c_in), np.float32), dtype), dtype)
        p.input, p.weight, p.output = din, H.dev(w, dtype), H.dev(dout, dtype)
        p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_bwd, "i32"), d_ms, d_order
        p.reverse_mask = True
        p.light_prefix = hint
        ConvMainUnitTest.implicit_gemm2(p)
        return H.host(din)

    if k_out <= 64 and c_in <= 64:
        base = backward_input(0)
        ref = conv_ref.implicit_gemm_dgrad_ref(
            dout, w, np.zeros_like(feat), pt.indices_bwd, ms, order, tile_m=64, dtype_in=dtype, dtype_w=dtype,
            dtype_out=dtype, reverse_mask=True)
        assert H.rel_err(H.as_f32(base, dtype), H.as_f32(ref, dtype)) < TOL
        for hint in hints[1:]:
            np.testing.assert_array_equal(backward_input(hint).view(np.uint16), base.view(np.uint16), err_msg="hint %d" % hint)


def test_light_prefix_leaves_skipped_rows_alone():
    """Backward-input of a stride-2 layer without padding: inputs on the last plane of an even axis
    feed no output, their masks are zero and lead the sorted order, and whole 64-row tiles of them
    are skipped (the caller zero-fills).  With the hint those positions sit in 128-row tiles: a
    half without any offset must stay untouched there as well - the gradient buffer starts from
    a sentinel here and has to come back the same with and without the hint."""
    print("case light_prefix strided backward-input", flush=True)
    dtype, c_in, k_out = "f16", 64, 64
    rng = np.random.default_rng(12)
    grid = (12, 40, 36)
    coords = synth.clustered_voxels(rng, 2500, grid, 6, sigma=3.0)
    zz, yy = np.meshgrid(np.arange(grid[0]), np.arange(grid[1]), indexing="ij")
    plane = np.stack([np.zeros(zz.size, np.int64), zz.ravel(), yy.ravel(), np.full(zz.size, grid[2] - 1)], axis=1)
    z2, x2 = np.meshgrid(np.arange(grid[0]), np.arange(7), indexing="ij")      # a strip of the last y plane as well
    edge = np.stack([np.zeros(z2.size, np.int64), z2.ravel(), np.full(z2.size, grid[1] - 1), x2.ravel()], axis=1)
    coords = np.unique(np.concatenate([coords, plane.astype(np.int32), edge.astype(np.int32)]), axis=0).astype(np.int32)
    pt = pairs.sparse_conv_pairs(coords, grid, padding=(0, 0, 0))
    n_in, n_out = coords.shape[0], pt.indices_fwd.shape[1]
    ms, order = pairs.sort_by_mask(pt.mask_bwd)
    empty = int((ms == 0).sum())
    assert empty >= 3 * 64 and (empty // 64) % 2 == 1, "an odd number of empty tiles: one 128-run is half empty"
    exact = pairs.light_prefix(ms)
    assert exact >= 256
    w = H.to_storage(rng.normal(0, 0.05, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    sentinel = H.to_storage(np.full((n_in, c_in), 7.0, np.float32), dtype)

    def run(hint):
        p = ConvParams(3, ConvOpType.BackwardInput)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, 64, 64)
        din = H.dev(sentinel, dtype)
        p.input, p.weight, p.output = din, H.dev(w, dtype), H.dev(dout, dtype)
        p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_bwd, "i32"), H.dev(ms, "u32"), H.dev(order, "i32")
        p.light_prefix = hint
        ConvMainUnitTest.implicit_gemm2(p)
        return H.host(din)

    base = run(0)
    skipped = order[:(empty // 64) * 64]
    assert (H.as_f32(base, dtype)[skipped] == 7.0).all()
    ref = conv_ref.implicit_gemm_dgrad_ref(dout, w, sentinel, pt.indices_bwd, ms, order, tile_m=64, dtype_in=dtype,
                                           dtype_w=dtype, dtype_out=dtype, reverse_mask=False)
    assert H.rel_err(H.as_f32(base, dtype), H.as_f32(ref, dtype)) < TOL
    for hint in (exact, 128, (empty // 128 + 1) * 128, n_in):
        np.testing.assert_array_equal(run(hint).view(np.uint16), base.view(np.uint16), err_msg="hint %d" % hint)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 128)])
@pytest.mark.parametrize("split_k", [1, 4, 32])
def test_backward_weight(dtype, tile, split_k):
    print("case backward_weight", dtype, tile, split_k, flush=True)
    c_in, k_out = 64, 96
    rng, coords, pt, feat, w, n_in, n_out = _case(4, 3000, c_in, k_out, dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    mask_width = 64
    red = conv_ref.tile_masks(ms, mask_width)
    dw0 = H.to_storage(np.zeros((k_out, 27, c_in), np.float32), dtype)
    desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, *tile)
    p = ConvParams(3, ConvOpType.BackwardWeight)
    p.conv_algo_desp = desp
    p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(dw0, dtype), H.dev(dout, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(red, "u32"), H.dev(order, "i32")
    p.mask_width = mask_width
    p.split_k_slices = split_k
    p.beta = 0.0
    ConvMainUnitTest.implicit_gemm2(p)
    got = H.as_f32(H.host(p.weight), dtype)
    ref = conv_ref.implicit_gemm_wgrad_ref(
        dout, feat, dw0, pt.indices_fwd, red, order, mask_width=mask_width, dtype_dout=dtype,
        dtype_in=dtype, dtype_w=dtype, split_k_slices=split_k, tile_k=32)
    assert H.rel_err(got, H.as_f32(ref, dtype)) < TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(64, 64, 64), (64, 96, 128), (40, 72, 32), (128, 128, 64), (72, 136, 64),
                                   (160, 200, 32)])
@pytest.mark.parametrize("strided", [False, True])
def test_backward_weight_balanced_atomic(dtype, shape, strided):
    """The split_k_parallel descriptor: work balanced over live tiles, fp32 atomic partial sums;
    compared with the oracle's once-rounded float32 sum, for two mask splits with beta."""
    c_in, k_out, mask_width = shape
    print("case backward_weight_atomic", dtype, shape, strided, flush=True)
    rng, coords, pt, feat, w, n_in, n_out = _case(14, 3000, c_in, k_out, dtype, strided=strided)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    red = conv_ref.tile_masks(ms, mask_width)
    dw0 = H.to_storage(rng.normal(0, 1, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)
    p = ConvParams(3, ConvOpType.BackwardWeight)
    p.conv_algo_desp = desp
    p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(dw0, dtype), H.dev(dout, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(red, "u32"), H.dev(order, "i32")
    p.mask_width = mask_width
    p.split_k_slices = 4
    cur = dw0
    for filt, beta in ((0x3FFF, 0.0), (0x1FFF << 14, 1.0)):
        p.mask_filter, p.beta, p.alpha = filt, beta, 0.5
        ConvMainUnitTest.implicit_gemm2(p)
        cur = conv_ref.implicit_gemm_wgrad_ref(
            dout, feat, cur, pt.indices_fwd, red, order, mask_width=mask_width, dtype_dout=dtype,
            dtype_in=dtype, dtype_w=dtype, mask_filter=filt, alpha=0.5, beta=beta,
            split_k_slices=1)
    got = H.as_f32(H.host(p.weight), dtype)
    assert H.rel_err(got, H.as_f32(cur, dtype)) < TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(64, 64, 64), (64, 192, 64), (128, 128, 64), (192, 136, 32), (40, 72, 128)])
@pytest.mark.parametrize("strided", [False, True])
def test_backward_weight_fixed_order(dtype, shape, strided):
    """ConvParams.deterministic with the split_k_parallel descriptor: partial sums kept per workgroup
    and added in a fixed order.  Against the oracle's once-rounded float32 sum (two mask splits,
    alpha and beta), and the same bits on a second run and on a run with other contents in the
    workspace; a workspace with room for fewer workgroups still gives a result within tolerance."""
    c_in, k_out, mask_width = shape
    print("case backward_weight_fixed_order", dtype, shape, strided, flush=True)
    rng, coords, pt, feat, w, n_in, n_out = _case(15, 3000, c_in, k_out, dtype, strided=strided)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    red = conv_ref.tile_masks(ms, mask_width)
    dw0 = H.to_storage(rng.normal(0, 1, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)

    def run(workspace=None):
        p = ConvParams(3, ConvOpType.BackwardWeight)
        p.conv_algo_desp = desp
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(dw0, dtype), H.dev(dout, dtype)
        p.indices = H.dev(pt.indices_fwd, "i32")
        p.mask, p.mask_argsort = H.dev(red, "u32"), H.dev(order, "i32")
        p.mask_width = mask_width
        p.split_k_slices = 4
        p.deterministic = True
        if workspace is not None:
            p.workspace = workspace
        for filt, beta in ((0x3FFF, 0.0), (0x1FFF << 14, 1.0)):
            p.mask_filter, p.beta, p.alpha = filt, beta, 0.5
            ConvMainUnitTest.implicit_gemm2(p)
        return H.host(p.weight), p.workspace

    cur = dw0
    for filt, beta in ((0x3FFF, 0.0), (0x1FFF << 14, 1.0)):
        cur = conv_ref.implicit_gemm_wgrad_ref(
            dout, feat, cur, pt.indices_fwd, red, order, mask_width=mask_width, dtype_dout=dtype,
            dtype_in=dtype, dtype_w=dtype, mask_filter=filt, alpha=0.5, beta=beta, split_k_slices=1)
    first, ws = run()
    assert H.rel_err(H.as_f32(first, dtype), H.as_f32(cur, dtype)) < TOL
    again, _ = run()
    np.testing.assert_array_equal(first, again)
    # same size of workspace, garbage inside: nothing in it has to start at zero
    dirty = H.dev(np.random.default_rng(1).integers(0, 255, size=ws.nbytes, dtype=np.uint8), "u8")
    third, _ = run(dirty)
    np.testing.assert_array_equal(first, third)
    need = int(_capi.lib().cumm_hip_query_wgrad_ordered_workspace(n_out, c_in, k_out, 27, mask_width))
    assert need == ws.nbytes
    # the reference's size for four slices: room for fewer workgroups (another split of the sum:
    # other bits, same tolerance) or, with many channel blocks, for none (the error names the least)
    m, n, k = k_out, 27 * c_in, n_out
    small = tv.empty([desp.query_conv_workspace_size(m, n, k, 4, 27)], tv.uint8, 0)
    assert small.nbytes < need
    try:
        fourth, _ = run(small)
        assert H.rel_err(H.as_f32(fourth, dtype), H.as_f32(cur, dtype)) < TOL
    except RuntimeError as e:
        assert "workspace at least" in str(e)
    with pytest.raises(RuntimeError, match="workspace at least"):
        run(tv.empty([4096], tv.uint8, 0))


def _wgrad_problem(seed, n, c_in, k_out, mask_width, dtype, grid=(12, 40, 36), strided=False, filt=0xFFFFFFFF,
                   alpha=1.0, beta=0.0, clusters=6, sigma=3.0):
    rng, coords, pt, feat, w, n_in, n_out = _case(seed, n, c_in, k_out, dtype, grid=grid, strided=strided,
                                                  clusters=clusters, sigma=sigma)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    red = conv_ref.tile_masks(ms, mask_width)
    dw0 = H.to_storage(rng.normal(0, 1, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    ref = conv_ref.implicit_gemm_wgrad_ref(
        dout, feat, dw0, pt.indices_fwd, red, order, mask_width=mask_width, dtype_dout=dtype,
        dtype_in=dtype, dtype_w=dtype, mask_filter=filt, alpha=alpha, beta=beta, split_k_slices=1)
    p = ConvParams(3, ConvOpType.BackwardWeight)
    p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)
    p.input, p.output = H.dev(feat, dtype), H.dev(dout, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(red, "u32"), H.dev(order, "i32")
    p.mask_width, p.split_k_slices = mask_width, 4
    p.mask_filter, p.alpha, p.beta = filt, alpha, beta
    return p, dw0, H.as_f32(ref, dtype), red


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_backward_weight_balanced_back_to_back(dtype):
    """Balanced backward-weight calls of different channel counts, mask widths, filters (offsets
    switched off, offsets without a live tile: a handful of voxels), alpha and beta, one after the
    other on one stream, twice over, then the same on a second stream of its own - every result
    against the oracle.  Each call prepares its own workspace (zeroed images, live-tile lists):
    nothing of an earlier problem may show in a later one."""
    print("case backward_weight_back_to_back", dtype, flush=True)
    lib = _capi.lib()
    problems = [
        _wgrad_problem(21, 3000, 64, 64, 64, dtype),
        _wgrad_problem(22, 2500, 24, 40, 32, dtype, alpha=0.5, beta=1.0),
        _wgrad_problem(23, 3000, 128, 128, 64, dtype, strided=True),
        _wgrad_problem(24, 40, 64, 64, 32, dtype, grid=(30, 60, 60), beta=1.0),      # most offsets have no pair
        _wgrad_problem(25, 3000, 72, 136, 64, dtype, filt=0x2AAAAAA, alpha=2.0, beta=0.5),
        _wgrad_problem(26, 9000, 64, 64, 32, dtype, grid=(20, 80, 80)),
    ]
    assert (problems[3][3] != 0).any() and bin(int(np.bitwise_or.reduce(problems[3][3]))).count("1") < 27
    other = tv.Context().create_cuda_stream()
    for stream in (0, other.cuda_stream_int()):
        for trip in range(2):
            for i, (p, dw0, ref, _) in enumerate(problems):
                p.stream = stream
                p.weight = H.dev(dw0, dtype)
                ConvMainUnitTest.implicit_gemm2(p)
                assert lib.cumm_hip_last_wgrad_path() in (2, 3), "problem %d" % i
                if stream:
                    other.synchronize_stream()
                got = H.as_f32(H.host(p.weight), dtype)
                assert H.rel_err(got, ref) < TOL, "stream %d trip %d problem %d" % (stream, trip, i)


@pytest.mark.parametrize("dtype", ["f16"])
def test_backward_weight_paths_by_size(dtype):
    """Which kernels serve a backward-weight call, as cumm_hip_last_wgrad_path reports them: the
    balanced units on live-tile lists (or, where a workgroup would walk several units of the centre
    offset, the fixed-order variant by itself), the fixed-order variant when asked for; both
    against the oracle."""
    print("case backward_weight_paths", dtype, flush=True)
    lib = _capi.lib()
    p, dw0, ref, red = _wgrad_problem(27, 150000, 64, 64, 32, dtype, grid=(40, 300, 300), clusters=60, sigma=15.0)
    assert red.shape[0] > 4096
    p.weight = H.dev(dw0, dtype)
    ConvMainUnitTest.implicit_gemm2(p)
    assert lib.cumm_hip_last_wgrad_path() in (2, 4)
    assert H.rel_err(H.as_f32(H.host(p.weight), dtype), ref) < TOL
    p, dw0, ref, red = _wgrad_problem(28, 3000, 64, 64, 64, dtype)
    p.deterministic = True
    p.weight = H.dev(dw0, dtype)
    ConvMainUnitTest.implicit_gemm2(p)
    assert lib.cumm_hip_last_wgrad_path() == 4
    assert H.rel_err(H.as_f32(H.host(p.weight), dtype), ref) < TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_backward_weight_balanced_atomic_small_workspace(dtype):
    """Few channels and many tiles: the two fp32 images that split_k_slices = 2 asks for have no
    room for the live-tile lists (27 * 94 words > 8 * 8 floats per offset), so the kernel that
    scans the reduced mask itself runs."""
    c_in, k_out, mask_width = 8, 8, 32
    print("case backward_weight_atomic small workspace", dtype, flush=True)
    rng, coords, pt, feat, w, n_in, n_out = _case(15, 3000, c_in, k_out, dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    red = conv_ref.tile_masks(ms, mask_width)
    assert 4 * 27 * red.shape[0] > 4 * k_out * 27 * c_in
    dw0 = H.to_storage(rng.normal(0, 1, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    p = ConvParams(3, ConvOpType.BackwardWeight)
    p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)
    p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(dw0, dtype), H.dev(dout, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(red, "u32"), H.dev(order, "i32")
    p.mask_width = mask_width
    p.split_k_slices = 2
    p.alpha, p.beta = 1.0, 1.0
    ConvMainUnitTest.implicit_gemm2(p)
    ref = conv_ref.implicit_gemm_wgrad_ref(
        dout, feat, dw0, pt.indices_fwd, red, order, mask_width=mask_width, dtype_dout=dtype,
        dtype_in=dtype, dtype_w=dtype, alpha=1.0, beta=1.0, split_k_slices=1)
    assert H.rel_err(H.as_f32(H.host(p.weight), dtype), H.as_f32(ref, dtype)) < TOL


@pytest.mark.parametrize("tile", [(64, 64), (128, 128), (64, 128)])
@pytest.mark.parametrize("strided", [False, True])
def test_int8_inference_bit_exact(tile, strided):
    print("case int8", tile, strided, flush=True)
    c_in, k_out = 64, 128
    rng, coords, pt, feat, w, n_in, n_out = _case(5, 3000, c_in, k_out, "s8", strided=strided)
    scale = rng.uniform(0.001, 0.01, size=(k_out,)).astype(np.float32)
    bias = rng.normal(0, 1, size=(k_out,)).astype(np.float32)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = np.zeros((n_out, k_out), np.int8)
    add = rng.integers(-127, 128, size=(n_out, k_out)).astype(np.int8)
    desp = H.find_conv_desp("s8", ConvOpType.Forward, *tile, int8_inference=True)
    for use_add, act in ((False, Activation.None_), (True, Activation.ReLU)):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = desp
        p.input, p.weight, p.output = H.dev(feat, "s8"), H.dev(w, "s8"), H.dev(out0, "s8")
        p.scale, p.bias = H.dev(scale, "f32"), H.dev(bias, "f32")
        if use_add:
            p.output_add = H.dev(add, "s8")
            p.beta = 0.5
        p.act_type = act
        p.indices = H.dev(pt.indices_fwd, "i32")
        p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
        ConvMainUnitTest.implicit_gemm2(p)
        ref, _ = conv_ref.implicit_gemm_fwd_ref(
            feat, w, out0, pt.indices_fwd, ms, order, tile_m=tile[0], dtype_in="s8", dtype_w="s8",
            dtype_out="s8", scale=scale, bias=bias, output_add=add if use_add else None,
            beta=p.beta, act=act.value, int8_inference=True)
        np.testing.assert_array_equal(H.host(p.output), ref)


def test_ragged_and_empty():
    """N not a multiple of the tile and a single voxel; each also with light_prefix hints that cover
    nothing, one run of 128, everything and more (few rows: the hint is cut to the whole runs)."""
    dtype = "f16"
    desp = H.find_conv_desp(dtype, ConvOpType.Forward, 64, 64)
    for n in (1, 65, 130, 257, 300):
        rng, coords, pt, feat, w, n_in, n_out = _case(6 + n, n, 64, 64, dtype, grid=(6, 10, 10))
        ms, order = pairs.sort_by_mask(pt.mask_fwd)
        out0 = H.to_storage(np.zeros((n_out, 64), np.float32), dtype)
        ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=64,
                                                     dtype_in=dtype, dtype_w=dtype, dtype_out=dtype)
        first = None
        for hint in (0, 128, 200, n_out, n_out + 500):
            p = ConvParams(3, ConvOpType.Forward)
            p.conv_algo_desp = desp
            p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
            p.indices = H.dev(pt.indices_fwd, "i32")
            p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
            p.mask_output = tv.zeros([(n_out + 63) // 64], tv.uint32, 0)
            p.light_prefix = hint
            ConvMainUnitTest.implicit_gemm2(p)
            got = H.host(p.output)
            assert H.rel_err(H.as_f32(got, dtype), H.as_f32(ref, dtype)) < TOL
            np.testing.assert_array_equal(H.host(p.mask_output), ref_mo)
            if first is None:
                first = got
            np.testing.assert_array_equal(got.view(np.uint16), first.view(np.uint16), err_msg="n %d hint %d" % (n, hint))


@pytest.mark.parametrize("geometry", [
    ("subm", (1, 3, 3), None, None),
    ("subm", (3, 1, 1), None, None),
    ("subm", (1, 1, 1), None, None),
    ("strided", (2, 2, 2), (2, 2, 2), (0, 0, 0)),
    ("strided", (2, 4, 4), (1, 2, 2), (0, 1, 1)),          # kernel volume 32: every mask bit in use
    ("strided", (3, 3, 3), (1, 1, 1), (1, 1, 1)),          # stride 1: a regular convolution on all sites
])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_kernel_volumes_forward_and_backward(dtype, geometry):
    """Kernel volumes other than 27 (1 to 32 offsets) through all three passes."""
    kind, ksize, stride, padding = geometry
    print("case kernel volume", dtype, geometry, flush=True)
    rng = np.random.default_rng(31)
    grid = (10, 24, 20)
    coords = synth.clustered_voxels(rng, 2200, grid, 5, sigma=3.0)
    if kind == "subm":
        pt = pairs.subm_pairs(coords, grid, ksize)
    else:
        pt = pairs.sparse_conv_pairs(coords, grid, ksize, stride, padding)
    kv = ksize[0] * ksize[1] * ksize[2]
    n_in, n_out = coords.shape[0], pt.indices_fwd.shape[1]
    c_in, k_out, tile = 64, 96, (64, 64)
    feat = H.to_storage(rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32), dtype)
    w = H.to_storage(rng.normal(0, 0.1, size=(k_out, kv, c_in)).astype(np.float32), dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    zero_out = H.to_storage(np.zeros((n_out, k_out), np.float32), dtype)

    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, *tile)
    p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(zero_out, dtype)
    p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_fwd, "i32"), H.dev(ms, "u32"), H.dev(order, "i32")
    p.mask_output = tv.zeros([(n_out + 63) // 64], tv.uint32, 0)
    ConvMainUnitTest.implicit_gemm2(p)
    ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, zero_out, pt.indices_fwd, ms, order, tile_m=64,
                                                 dtype_in=dtype, dtype_w=dtype, dtype_out=dtype)
    assert H.rel_err(H.as_f32(H.host(p.output), dtype), H.as_f32(ref, dtype)) < TOL
    np.testing.assert_array_equal(H.host(p.mask_output), ref_mo)

    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    zero_in = H.to_storage(np.zeros((n_in, c_in), np.float32), dtype)
    if kind == "subm":
        msb, orderb, reverse = ms, order, True
    else:
        msb, orderb = pairs.sort_by_mask(pt.mask_bwd)
        reverse = False
    pd = ConvParams(3, ConvOpType.BackwardInput)
    pd.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, *tile)
    pd.input, pd.weight, pd.output = H.dev(zero_in, dtype), p.weight, H.dev(dout, dtype)
    pd.indices, pd.mask, pd.mask_argsort = H.dev(pt.indices_bwd, "i32"), H.dev(msb, "u32"), H.dev(orderb, "i32")
    pd.reverse_mask = reverse
    ConvMainUnitTest.implicit_gemm2(pd)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, zero_in, pt.indices_bwd, msb, orderb, tile_m=64, dtype_in=dtype,
                                             dtype_w=dtype, dtype_out=dtype, reverse_mask=reverse)
    assert H.rel_err(H.as_f32(H.host(pd.input), dtype), H.as_f32(ref_d, dtype)) < TOL

    red = conv_ref.tile_masks(ms, 64)
    zero_w = H.to_storage(np.zeros((k_out, kv, c_in), np.float32), dtype)
    ref_w = conv_ref.implicit_gemm_wgrad_ref(dout, feat, zero_w, pt.indices_fwd, red, order, mask_width=64,
                                             dtype_dout=dtype, dtype_in=dtype, dtype_w=dtype, split_k_slices=1)
    for parallel, fixed_order in ((True, False), (True, True), (False, False)):
        pw = ConvParams(3, ConvOpType.BackwardWeight)
        pw.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=parallel)
        pw.input, pw.weight, pw.output = p.input, H.dev(zero_w, dtype), pd.output
        pw.indices, pw.mask, pw.mask_argsort = p.indices, H.dev(red, "u32"), p.mask_argsort
        pw.mask_width, pw.split_k_slices = 64, 4 if parallel else 1
        pw.deterministic = fixed_order
        ConvMainUnitTest.implicit_gemm2(pw)
        assert H.rel_err(H.as_f32(H.host(pw.weight), dtype), H.as_f32(ref_w, dtype)) < TOL


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("act,act_alpha", [(Activation.Sigmoid, 0.0), (Activation.LeakyReLU, 0.1),
                                           (Activation.LeakyReLU, 0.0)])
def test_forward_sigmoid_and_leaky_relu(dtype, act, act_alpha):
    """The other two activations of the epilogue (UnaryActivation, cumm/gemm/gemmmath/__init__.py:181-214),
    with a bias, on the LDS-streaming kernel (64 channels) and on the chunked one (160 channels)."""
    print("case activation", dtype, act, act_alpha, flush=True)
    for c_in, k_out, tile in ((64, 64, (64, 64)), (160, 96, (128, 128))):
        rng, coords, pt, feat, w, n_in, n_out = _case(41, 2500, c_in, k_out, dtype)
        bias = H.to_storage(rng.normal(0, 0.5, size=(k_out,)).astype(np.float32), dtype)
        ms, order = pairs.sort_by_mask(pt.mask_fwd)
        out0 = H.to_storage(np.zeros((n_out, k_out), np.float32), dtype)
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, *tile)
        p.input, p.weight, p.output, p.bias = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype), H.dev(bias, dtype)
        p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_fwd, "i32"), H.dev(ms, "u32"), H.dev(order, "i32")
        p.beta, p.act_type, p.act_alpha = 1.0, act, act_alpha
        ConvMainUnitTest.implicit_gemm2(p)
        ref, _ = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=tile[0],
                                                dtype_in=dtype, dtype_w=dtype, dtype_out=dtype, bias=bias, beta=1.0,
                                                act=act.value, act_alpha=act_alpha)
        got, want = H.as_f32(H.host(p.output), dtype), H.as_f32(ref, dtype)
        assert H.rel_err(got, want) < TOL
        if act == Activation.Sigmoid:
            assert 0.0 <= got.min() and got.max() <= 1.0 and 0.3 < got.mean() < 0.7
        elif act_alpha == 0.1:
            assert got.min() < 0.0       # negative values pass, scaled


@pytest.mark.parametrize("act_alpha", [0.1, 0.25])
def test_int8_inference_leaky_relu_bit_exact(act_alpha):
    print("case int8 leaky relu", act_alpha, flush=True)
    c_in, k_out = 64, 128
    rng, coords, pt, feat, w, n_in, n_out = _case(43, 3000, c_in, k_out, "s8", strided=True)
    scale = rng.uniform(0.001, 0.01, size=(k_out,)).astype(np.float32)
    bias = rng.normal(0, 1, size=(k_out,)).astype(np.float32)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = np.zeros((n_out, k_out), np.int8)
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp("s8", ConvOpType.Forward, 64, 128, int8_inference=True)
    p.input, p.weight, p.output = H.dev(feat, "s8"), H.dev(w, "s8"), H.dev(out0, "s8")
    p.scale, p.bias = H.dev(scale, "f32"), H.dev(bias, "f32")
    p.act_type, p.act_alpha = Activation.LeakyReLU, act_alpha
    p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_fwd, "i32"), H.dev(ms, "u32"), H.dev(order, "i32")
    ConvMainUnitTest.implicit_gemm2(p)
    ref, _ = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=64, dtype_in="s8",
                                            dtype_w="s8", dtype_out="s8", scale=scale, bias=bias,
                                            act=Activation.LeakyReLU.value, act_alpha=act_alpha, int8_inference=True)
    got = H.host(p.output)
    np.testing.assert_array_equal(got, ref)
    assert (got < 0).any() and (got > 0).any()


@pytest.mark.parametrize("tile", [(64, 64), (128, 64), (64, 128), (128, 128)])
@pytest.mark.parametrize("strided", [False, True])
def test_s8_forward_s32_accumulators_bit_exact(tile, strided):
    """The "s8,s8,s32,s32,s32" kind: the raw s32 accumulators, and the integer linear combination
    with a source and ReLU, bit for bit against the oracle's exact integer sums."""
    print("case s8 -> s32", tile, strided, flush=True)
    c_in, k_out = 64, 128
    rng, coords, pt, feat, w, n_in, n_out = _case(25, 3000, c_in, k_out, "s8", strided=strided)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    src = rng.integers(-100000, 100000, size=(n_out, k_out)).astype(np.int32)
    desp = H.find_conv_desp("s8", ConvOpType.Forward, *tile, dtype_out="s32")
    _, mo, acc = conv_ref.implicit_gemm_fwd_ref(
        feat, w, src, pt.indices_fwd, ms, order, tile_m=tile[0], dtype_in="s8", dtype_w="s8",
        dtype_out="s32", return_acc=True)
    for alpha, beta, act in ((1.0, 0.0, Activation.None_), (2.0, -1.0, Activation.ReLU)):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = desp
        p.input, p.weight, p.output = H.dev(feat, "s8"), H.dev(w, "s8"), H.dev(src, "s32")
        p.indices = H.dev(pt.indices_fwd, "i32")
        p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
        p.mask_output = tv.zeros([(n_out + tile[0] - 1) // tile[0]], tv.uint32, 0)
        p.alpha, p.beta, p.act_type = alpha, beta, act
        ConvMainUnitTest.implicit_gemm2(p)
        ref, _ = conv_ref.implicit_gemm_fwd_ref(
            feat, w, src, pt.indices_fwd, ms, order, tile_m=tile[0], dtype_in="s8", dtype_w="s8",
            dtype_out="s32", alpha=alpha, beta=beta, act=act.value)
        got = H.host(p.output)
        np.testing.assert_array_equal(got, ref)
        np.testing.assert_array_equal(H.host(p.mask_output), mo)
        if beta == 0.0:
            np.testing.assert_array_equal(got, acc)     # alpha = 1: the accumulators themselves
        else:                                           # the closed form on the exact sums
            want = np.maximum(2 * acc.astype(np.int64) - src.astype(np.int64), 0)
            np.testing.assert_array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("tile", [(64, 64), (128, 128)])
def test_f32_output_forward_and_backward_input(dtype, tile):
    """f16 / bf16 operands with the fp32 accumulators as the output (no rounding to 16 bits)."""
    print("case f32 out", dtype, tile, flush=True)
    c_in, k_out = 64, 96
    rng, coords, pt, feat, w, n_in, n_out = _case(26, 2500, c_in, k_out, dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32)
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, *tile, dtype_out="f32")
    p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, "f32")
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
    p.alpha, p.beta = 0.5, 1.0
    ConvMainUnitTest.implicit_gemm2(p)
    ref, _ = conv_ref.implicit_gemm_fwd_ref(
        feat, w, out0, pt.indices_fwd, ms, order, tile_m=tile[0], dtype_in=dtype, dtype_w=dtype,
        dtype_out="f32", alpha=0.5, beta=1.0)
    assert H.rel_err(H.host(p.output), ref) < 2e-3
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    din0 = np.zeros((n_in, c_in), np.float32)
    q = ConvParams(3, ConvOpType.BackwardInput)
    # (the input gradient is the GEMM's C operand: dtype_c f32; dtype_output names the conv output, dOut)
    q.conv_algo_desp = [d for d in ConvMainUnitTest.get_all_conv_algo_desp()
                        if d.dtype_a == H.TV_DTYPE[dtype] and d.dtype_c == tv.float32 and
                        ConvOpType(d.op_type) == ConvOpType.BackwardInput and list(d.tile_shape[:2]) == list(tile)][0]
    q.input, q.weight, q.output = H.dev(din0, "f32"), H.dev(w, dtype), H.dev(dout, dtype)
    q.indices = H.dev(pt.indices_bwd, "i32")
    q.mask, q.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
    q.reverse_mask = True
    ConvMainUnitTest.implicit_gemm2(q)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(
        dout, w, din0, pt.indices_bwd, ms, order, tile_m=tile[0], dtype_in=dtype, dtype_w=dtype,
        dtype_out="f32", reverse_mask=True)
    assert H.rel_err(H.host(q.input), ref_d) < 2e-3


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_long_contraction_forward_and_backward_input(dtype):
    """640 channels on the contraction side: more than eight stage rows, which the chunked
    register-gather kernel serves (forward: C = 640; backward-input: K = 640)."""
    print("case long contraction", dtype, flush=True)
    c_in, k_out = 640, 64
    rng, coords, pt, feat, w, n_in, n_out = _case(27, 600, c_in, k_out, dtype)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = H.to_storage(np.zeros((n_out, k_out), np.float32), dtype)
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, 64, 64)
    p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
    ConvMainUnitTest.implicit_gemm2(p)
    ref, _ = conv_ref.implicit_gemm_fwd_ref(
        feat, w, out0, pt.indices_fwd, ms, order, tile_m=64, dtype_in=dtype, dtype_w=dtype, dtype_out=dtype)
    assert H.rel_err(H.as_f32(H.host(p.output), dtype), H.as_f32(ref, dtype)) < TOL
    # backward-input with the roles swapped: K = 640 is the contraction
    w2 = H.to_storage(rng.normal(0, 0.05, size=(640, 27, 64)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, 640)).astype(np.float32), dtype)
    din0 = H.to_storage(np.zeros((n_in, 64), np.float32), dtype)
    q = ConvParams(3, ConvOpType.BackwardInput)
    q.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, 64, 64)
    q.input, q.weight, q.output = H.dev(din0, dtype), H.dev(w2, dtype), H.dev(dout, dtype)
    q.indices = H.dev(pt.indices_bwd, "i32")
    q.mask, q.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
    q.reverse_mask = True
    ConvMainUnitTest.implicit_gemm2(q)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(
        dout, w2, din0, pt.indices_bwd, ms, order, tile_m=64, dtype_in=dtype, dtype_w=dtype,
        dtype_out=dtype, reverse_mask=True)
    assert H.rel_err(H.as_f32(H.host(q.input), dtype), H.as_f32(ref_d, dtype)) < TOL


def _desps_128(dtype, op):
    """Both descriptors of the 128 x 128 tile: three stages of 64-byte chunks, two of 128-byte chunks."""
    found = {}
    for d in ConvMainUnitTest.get_all_conv_algo_desp():
        if (d.dtype_a == H.TV_DTYPE[dtype] and d.dtype_output == H.TV_DTYPE[dtype] and
                d.dtype_input == H.TV_DTYPE[dtype] and ConvOpType(d.op_type) == op and
                tuple(d.tile_shape[:2]) == (128, 128) and not d.dynamic_mask and not d.is_int8_inference):
            found[d.num_stage] = d
    assert sorted(found) == [2, 3]
    return found


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("c_in,k_out", [(128, 128), (96, 256), (160, 72), (256, 128)])
def test_both_stage_counts_of_the_128_tile(dtype, c_in, k_out):
    """Contractions of more than 128 bytes through both descriptors of the 128 x 128 tile, forward
    and backward-input (strided table, so the two passes differ): each against the oracle, and
    the same bits from both (the products are added in the same order, chunk by chunk)."""
    print("case both stage counts", dtype, c_in, k_out, flush=True)
    rng, coords, pt, feat, w, n_in, n_out = _case(31, 2500, c_in, k_out, dtype, strided=True)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=128, dtype_in=dtype,
                                                 dtype_w=dtype, dtype_out=dtype, beta=1.0)
    got = {}
    for stages, desp in _desps_128(dtype, ConvOpType.Forward).items():
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = desp
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
        p.indices = H.dev(pt.indices_fwd, "i32")
        p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
        p.mask_output = tv.zeros([(n_out + 127) // 128], tv.uint32, 0)
        p.mask_width = 128
        p.beta = 1.0
        ConvMainUnitTest.implicit_gemm2(p)
        got[stages] = H.host(p.output)
        assert H.rel_err_rows(H.as_f32(got[stages], dtype), H.as_f32(ref, dtype)) < TOL, stages
        np.testing.assert_array_equal(H.host(p.mask_output), ref_mo)
    np.testing.assert_array_equal(got[2], got[3])
    msb, orderb = pairs.sort_by_mask(pt.mask_bwd)
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    din0 = H.to_storage(np.zeros((n_in, c_in), np.float32), dtype)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, din0, pt.indices_bwd, msb, orderb, tile_m=128, dtype_in=dtype,
                                             dtype_w=dtype, dtype_out=dtype)
    got = {}
    for stages, desp in _desps_128(dtype, ConvOpType.BackwardInput).items():
        q = ConvParams(3, ConvOpType.BackwardInput)
        q.conv_algo_desp = desp
        q.input, q.weight, q.output = H.dev(din0, dtype), H.dev(w, dtype), H.dev(dout, dtype)
        q.indices = H.dev(pt.indices_bwd, "i32")
        q.mask, q.mask_argsort = H.dev(msb, "u32"), H.dev(orderb, "i32")
        ConvMainUnitTest.implicit_gemm2(q)
        got[stages] = H.host(q.input)
        assert H.rel_err_rows(H.as_f32(got[stages], dtype), H.as_f32(ref_d, dtype)) < TOL, stages
    np.testing.assert_array_equal(got[2], got[3])


@pytest.mark.parametrize("dtype,tile", [("f16", (64, 64)), ("bf16", (128, 128)), ("s8", (64, 128))])
def test_mask_bit_clear_over_a_valid_entry(dtype, tile):
    """Where this library narrows the reference's mask contract, as a tested fact.  The reference
    walks the kernel offsets of a tile's OR-ed mask and gates each row by its pair-table entry
    alone (cumm/conv/sparse_iters.py:629-631); the oracle does the same.  The LDS-streaming
    kernels here let a position take part in offset k only if its OWN mask word has bit k.  For
    masks made from the pair table (bit k wherever the entry is valid) the two rules are the
    same thing.  This test clears bits over valid entries in a third of the words:
      * default: the result is the oracle's on a pair table whose entries under a cleared bit
        are removed (and it differs from the oracle on the table as given);
      * ``ungated_rows``: the result is the oracle's on the table as given (the reference's
        rule), with the same ``mask_output``."""
    print("case cleared mask bits", dtype, tile, flush=True)
    c_in, k_out = (64, 128) if dtype == "s8" else (64, 64)
    rng, coords, pt, feat, w, n_in, n_out = _case(31, 3000, c_in, k_out, dtype)
    mask = pt.mask_fwd.copy()
    victims = rng.permutation(n_out)[:n_out // 3]
    for o in victims:
        bits = [k for k in range(27) if k != 13 and (mask[o] >> k) & 1]
        if bits:
            mask[o] &= ~np.uint32(1 << int(rng.choice(bits)))
    assert (mask != pt.mask_fwd).sum() > 100
    ms, order = pairs.sort_by_mask(mask)
    # the table with the entries under a cleared bit removed
    gated = pt.indices_fwd.copy()
    for k in range(27):
        gated[k][((mask >> np.uint32(k)) & 1) == 0] = -1
    kw = dict(tile_m=tile[0], dtype_in=dtype, dtype_w=dtype, dtype_out=dtype)
    scale = bias = None
    if dtype == "s8":
        scale = rng.uniform(0.001, 0.01, size=(k_out,)).astype(np.float32)
        bias = rng.normal(0, 1, size=(k_out,)).astype(np.float32)
        kw.update(scale=scale, bias=bias, int8_inference=True)
    out0 = np.zeros((n_out, k_out), np.int8) if dtype == "s8" else H.to_storage(np.zeros((n_out, k_out), np.float32), dtype)
    ref_given, mo_given = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, **kw)
    ref_gated, mo_gated = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, gated, ms, order, **kw)
    np.testing.assert_array_equal(mo_given, mo_gated)
    assert (np.asarray(ref_given) != np.asarray(ref_gated)).any(), "the case must tell the two rules apart"

    def run(ungated):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, *tile, int8_inference=dtype == "s8")
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
        if dtype == "s8":
            p.scale, p.bias = H.dev(scale, "f32"), H.dev(bias, "f32")
        p.indices = H.dev(pt.indices_fwd, "i32")
        p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
        p.mask_output = tv.zeros([(n_out + tile[0] - 1) // tile[0]], tv.uint32, 0)
        p.ungated_rows = ungated
        p.light_prefix = pairs.light_prefix(ms)     # (ignored with ungated_rows)
        ConvMainUnitTest.implicit_gemm2(p)
        return H.host(p.output), H.host(p.mask_output)

    got, mo = run(False)
    got_u, mo_u = run(True)
    np.testing.assert_array_equal(mo, mo_gated)
    np.testing.assert_array_equal(mo_u, mo_given)
    if dtype == "s8":
        np.testing.assert_array_equal(got, ref_gated)
        np.testing.assert_array_equal(got_u, ref_given)
    else:
        assert H.rel_err(H.as_f32(got, dtype), H.as_f32(ref_gated, dtype)) < TOL
        assert H.rel_err(H.as_f32(got_u, dtype), H.as_f32(ref_given, dtype)) < TOL
        assert H.rel_err(H.as_f32(got, dtype), H.as_f32(ref_given, dtype)) > TOL     # the divergence is real


@pytest.mark.parametrize("dtype,tile,c_in,k_out", [("f16", (64, 64), 64, 64), ("f16", (128, 64), 32, 96),
                                                    ("bf16", (128, 128), 128, 128), ("bf16", (64, 128), 200, 72),
                                                    ("s8", (64, 128), 64, 128), ("s8", (128, 128), 128, 64)])
@pytest.mark.parametrize("strided", [False, True])
def test_pair_table_by_position(dtype, tile, c_in, k_out, strided):
    """``indices_by_position``: the pair table permuted into the order of the sorted positions
    (pairs.pairs_by_position_device, bit-exact against the host's fancy indexing) gives the same
    output bits and tile masks as the table by row, forward and backward-input, with and without
    the light_prefix hint - and the table by row is checked against the oracle."""
    print("case pair table by position", dtype, tile, c_in, k_out, strided, flush=True)
    rng, coords, pt, feat, w, n_in, n_out = _case(33, 3000, c_in, k_out, dtype, strided=strided)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    d_ind, d_order = H.dev(pt.indices_fwd, "i32"), H.dev(order, "i32")
    d_pos = pairs.pairs_by_position_device(d_ind, d_order)
    np.testing.assert_array_equal(H.host(d_pos), pairs.pairs_by_position(pt.indices_fwd, order))
    int8 = dtype == "s8"
    scale = bias = None
    kw = dict(tile_m=tile[0], dtype_in=dtype, dtype_w=dtype, dtype_out=dtype)
    if int8:
        scale = rng.uniform(0.001, 0.01, size=(k_out,)).astype(np.float32)
        bias = rng.normal(0, 1, size=(k_out,)).astype(np.float32)
        kw.update(scale=scale, bias=bias, int8_inference=True)
    out0 = np.zeros((n_out, k_out), np.int8) if int8 else H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    beta = 0.0 if int8 else 1.0
    ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, beta=beta, **kw)

    def forward(by_pos, hint):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, *tile, int8_inference=int8)
        p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
        if int8:
            p.scale, p.bias = H.dev(scale, "f32"), H.dev(bias, "f32")
        p.indices = d_pos if by_pos else d_ind
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort = H.dev(ms, "u32"), d_order
        p.mask_output = tv.zeros([(n_out + tile[0] - 1) // tile[0]], tv.uint32, 0)
        p.beta = beta
        p.light_prefix = hint
        ConvMainUnitTest.implicit_gemm2(p)
        return H.host(p.output), H.host(p.mask_output)

    base, base_mo = forward(False, 0)
    np.testing.assert_array_equal(base_mo, ref_mo)
    if int8:
        np.testing.assert_array_equal(base, ref)
    else:
        assert H.rel_err(H.as_f32(base, dtype), H.as_f32(ref, dtype)) < TOL
    for hint in (0, pairs.light_prefix(ms)):
        got, got_mo = forward(True, hint)
        np.testing.assert_array_equal(got.view(np.uint8), base.view(np.uint8))
        np.testing.assert_array_equal(got_mo, base_mo)

    if int8:
        return
    # backward-input: the backward table by position of the sort the launch uses
    if strided:
        msb, orderb = pairs.sort_by_mask(pt.mask_bwd)
        reverse = False
    else:
        msb, orderb = ms, order
        reverse = True
    dout = H.to_storage(rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32), dtype)
    d_indb, d_orderb = H.dev(pt.indices_bwd, "i32"), H.dev(orderb, "i32")
    d_posb = pairs.pairs_by_position_device(d_indb, d_orderb)

    def backward_input(by_pos):
        p = ConvParams(3, ConvOpType.BackwardInput)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, *tile)
        din = H.dev(H.to_storage(np.zeros((n_in, c_in), np.float32), dtype), dtype)
        p.input, p.weight, p.output = din, H.dev(w, dtype), H.dev(dout, dtype)
        p.indices = d_posb if by_pos else d_indb
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort = H.dev(msb, "u32"), d_orderb
        p.reverse_mask = reverse
        ConvMainUnitTest.implicit_gemm2(p)
        return H.host(din)

    base = backward_input(False)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, np.zeros((n_in, c_in), base.dtype), pt.indices_bwd, msb, orderb,
                                             tile_m=tile[0], dtype_in=dtype, dtype_w=dtype, dtype_out=dtype,
                                             reverse_mask=reverse)
    assert H.rel_err(H.as_f32(base, dtype), H.as_f32(ref_d, dtype)) < TOL
    np.testing.assert_array_equal(backward_input(True).view(np.uint16), base.view(np.uint16))


@pytest.mark.parametrize("dtype,c_in,k_out", [("f16", 64, 64), ("bf16", 48, 40), ("f16", 32, 32)])
@pytest.mark.parametrize("n_target", [12000, 2100])
def test_order_by_offset_count_and_half_tiles(dtype, c_in, k_out, n_target):
    """The launch that finds its hints on the device, on masks in the GPU sort's order by offset
    count: the light end in 128-row tiles, the heavy end - the last few tiles, ten offsets or more -
    in halves of 32 rows (contractions of more than 64 bytes).  Forward (bias + ReLU) and
    backward-input give the same output bits as 64-row tiles throughout (light_prefix = -1: no
    hints) and as the same layer on masks sorted by value, the tile masks are the oracle's, and the
    results are within tolerance of the oracle."""
    print("case order by count", dtype, c_in, k_out, n_target, flush=True)
    rng = np.random.default_rng(21)
    grid = (41, 400, 400)
    coords = synth.clustered_voxels(rng, n_target, grid, 6, sigma=15.0, noise_frac=0.1)
    pt = pairs.subm_pairs(coords, grid)
    n = coords.shape[0]
    filt = 0x07FFFFFF
    d_mask = H.dev(pt.mask_fwd, "u32")
    feat = H.to_storage(rng.normal(0, 1, size=(n, c_in)).astype(np.float32), dtype)
    w = H.to_storage(rng.normal(0, 0.05, size=(k_out, 27, c_in)).astype(np.float32), dtype)
    bias = H.to_storage(rng.normal(0, 1, size=(k_out,)).astype(np.float32), dtype)
    dout = H.to_storage(rng.normal(0, 1, size=(n, k_out)).astype(np.float32), dtype)
    out0 = H.to_storage(np.zeros((n, k_out), np.float32), dtype)
    din0 = H.to_storage(np.full((n, c_in), 3.0, np.float32), dtype)
    d_feat, d_w, d_bias, d_dout = H.dev(feat, dtype), H.dev(w, dtype), H.dev(bias, dtype), H.dev(dout, dtype)
    d_ind, d_indb = H.dev(pt.indices_fwd, "i32"), H.dev(pt.indices_bwd, "i32")
    tiles = (n + 63) // 64
    results = {}
    for by_count in (False, True):
        ms, order = pairs.sort_by_mask_device(d_mask, filt, by_offset_count=by_count)
        ms_h, order_h = H.host(ms), H.host(order)
        light, heavy = pairs.hints_device(ms, filt)
        if by_count and n_target == 12000:
            assert light >= 256 and heavy < n and (tiles - heavy // 64) * 8 <= tiles, "the case should have pairs and halves"
        for hint in (-1, 0):
            p = ConvParams(3, ConvOpType.Forward)
            p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, 64, 64)
            p.input, p.weight, p.output, p.bias = d_feat, d_w, H.dev(out0, dtype), d_bias
            p.beta, p.act_type = 1.0, Activation.ReLU
            p.indices, p.mask, p.mask_argsort, p.mask_filter = d_ind, ms, order, filt
            p.mask_output = tv.zeros([tiles], tv.uint32, 0)
            p.light_prefix = hint
            ConvMainUnitTest.implicit_gemm2(p)
            pd = ConvParams(3, ConvOpType.BackwardInput)
            pd.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, 64, 64)
            pd.input, pd.weight, pd.output = H.dev(din0, dtype), d_w, d_dout
            pd.indices, pd.mask, pd.mask_argsort, pd.mask_filter, pd.reverse_mask = d_indb, ms, order, filt, True
            pd.light_prefix = hint
            ConvMainUnitTest.implicit_gemm2(pd)
            results[(by_count, hint)] = (H.host(p.output), H.host(pd.input))
            np.testing.assert_array_equal(H.host(p.mask_output), conv_ref.tile_masks(ms_h, 64, filt))
        if by_count:
            ref, _ = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms_h, order_h, tile_m=64, dtype_in=dtype,
                                                    dtype_w=dtype, dtype_out=dtype, mask_filter=filt, beta=1.0, bias=bias,
                                                    act=onm.ACT_RELU)
            ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, din0, pt.indices_bwd, ms_h, order_h, tile_m=64, dtype_in=dtype,
                                                     dtype_w=dtype, dtype_out=dtype, mask_filter=filt, reverse_mask=True)
            assert H.rel_err(H.as_f32(results[(True, 0)][0], dtype), H.as_f32(ref, dtype)) < TOL
            assert H.rel_err(H.as_f32(results[(True, 0)][1], dtype), H.as_f32(ref_d, dtype)) < TOL
    base = results[(False, -1)]
    for key, (out, din) in results.items():
        np.testing.assert_array_equal(out.view(np.uint16), base[0].view(np.uint16), err_msg=str(key))
        np.testing.assert_array_equal(din.view(np.uint16), base[1].view(np.uint16), err_msg=str(key))
