"""Parity at the benchmark configurations' full sizes (thousands of tiles, many
more than the device holds workgroups at once), against the CPU oracle on the
same seeded inputs, plus a size-independent property (linearity in the
features) for the f16 forward."""
import numpy as np
import pytest

import helpers as H
from cumm_amd import pairs, synth
from cumm_amd import tensorview as tv
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.gemm.main import GemmMainUnitTest
from cumm_amd.tensorview.gemm import ConvOpType, ConvParams, GemmParams, ShuffleStrideType
from oracle import conv_ref, gemm_ref

pytestmark = pytest.mark.gpu

TOL = 1e-2          # max |got - ref| / max |ref| for f16 / bf16 outputs
GRID = (41, 1600, 1408)


def _subm_case(seed, n_target, dtype, c, k):
    rng = np.random.default_rng(seed)
    coords = synth.clustered_voxels(rng, n_target, GRID, 60, sigma=15.0, noise_frac=0.10)
    pt = pairs.subm_pairs(coords, GRID)
    n = coords.shape[0]
    feat = H.to_storage(rng.normal(0, 1, size=(n, c)).astype(np.float32), dtype)
    w = H.to_storage(rng.normal(0, 0.05, size=(k, 27, c)).astype(np.float32), dtype)
    return rng, pt, feat, w, n


@pytest.mark.parametrize("tile_m", [64, 128])
def test_subm_f16_c64_forward_dgrad_full_size(tile_m):
    print("case full size subm f16", tile_m, flush=True)
    dtype = "f16"
    rng, pt, feat, w, n = _subm_case(20240607, 120000, dtype, 64, 64)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = np.zeros((n, 64), np.float16)
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, tile_m, 64)
    p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(w, dtype), H.dev(out0, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
    p.mask_output = tv.zeros([(n + tile_m - 1) // tile_m], tv.uint32, 0)
    ConvMainUnitTest.implicit_gemm2(p)
    ref, mask_out = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=tile_m,
                                                   dtype_in=dtype, dtype_w=dtype, dtype_out=dtype)
    got = H.as_f32(H.host(p.output), dtype)
    assert H.rel_err(got, H.as_f32(ref, dtype)) < TOL
    assert H.rel_err_rows(got, H.as_f32(ref, dtype)) < TOL           # every row by its own scale
    np.testing.assert_array_equal(H.host(p.mask_output), mask_out)   # integer work: bit-exact

    # linearity: conv(2 x) == 2 conv(x); scaling by two is exact in f32 and in normal f16 (no
    # overflow here), only subnormal f16 results may round differently (one subnormal ulp, 2^-24)
    p2 = ConvParams(3, ConvOpType.Forward)
    p2.conv_algo_desp = p.conv_algo_desp
    p2.input = H.dev((feat.astype(np.float32) * 2).astype(np.float16), dtype)
    p2.weight, p2.output = p.weight, H.dev(out0, dtype)
    p2.indices, p2.mask, p2.mask_argsort = p.indices, p.mask, p.mask_argsort
    ConvMainUnitTest.implicit_gemm2(p2)
    got2 = H.as_f32(H.host(p2.output), dtype)
    normal = np.abs(got) >= 2.0 ** -14
    np.testing.assert_array_equal(got2[normal], 2 * got[normal])
    assert np.max(np.abs(got2 - 2 * got)) <= 2.0 ** -23

    # backward-input on the same pair table
    dout = H.to_storage(rng.normal(0, 1, size=(n, 64)).astype(np.float32), dtype)
    din0 = np.zeros((n, 64), np.float16)
    pd = ConvParams(3, ConvOpType.BackwardInput)
    pd.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, tile_m, 64)
    pd.input, pd.weight, pd.output = H.dev(din0, dtype), p.weight, H.dev(dout, dtype)
    pd.indices = H.dev(pt.indices_bwd, "i32")
    pd.mask, pd.mask_argsort = p.mask, p.mask_argsort
    pd.reverse_mask = True
    ConvMainUnitTest.implicit_gemm2(pd)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, din0, pt.indices_bwd, ms, order, tile_m=tile_m,
                                             dtype_in=dtype, dtype_w=dtype, dtype_out=dtype, reverse_mask=True)
    assert H.rel_err(H.as_f32(H.host(pd.input), dtype), H.as_f32(ref_d, dtype)) < TOL
    assert H.rel_err_rows(H.as_f32(H.host(pd.input), dtype), H.as_f32(ref_d, dtype)) < TOL


def test_subm_f16_c64_two_tile_shapes_full_size():
    """The launch the benchmark times: the headline voxel set with the light end of the sorted
    order in 128-row tiles (``light_prefix`` as input preparation counts it; several hundred
    128-row tiles next to several hundred 64-row tiles in one launch).  Forward and
    backward-input: the same output bits and the same ``mask_output`` as the launch without the
    hint, and within tolerance of the oracle, over the whole tensor and row by row."""
    print("case full size subm f16, two tile shapes", flush=True)
    dtype, tile_m = "f16", 64
    rng, pt, feat, w, n = _subm_case(20240607, 120000, dtype, 64, 64)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    light = pairs.light_prefix(ms)
    assert light >= 256 and light % 128 == 0 and n - light >= 64 * 100   # both shapes, hundreds of each
    out0 = np.zeros((n, 64), np.float16)
    tiles = (n + tile_m - 1) // tile_m
    d_feat, d_w = H.dev(feat, dtype), H.dev(w, dtype)
    d_ind, d_ms, d_order = H.dev(pt.indices_fwd, "i32"), H.dev(ms, "u32"), H.dev(order, "i32")
    d_ms_check = H.dev(ms, "u32")
    assert pairs.light_prefix_device(d_ms_check) == light
    outs, mask_outs = [], []
    for hint in (0, light):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, tile_m, 64)
        p.input, p.weight, p.output = d_feat, d_w, H.dev(out0, dtype)
        p.indices, p.mask, p.mask_argsort = d_ind, d_ms, d_order
        p.mask_output = tv.zeros([tiles], tv.uint32, 0)
        p.light_prefix = hint
        ConvMainUnitTest.implicit_gemm2(p)
        outs.append(H.host(p.output))
        mask_outs.append(H.host(p.mask_output))
    ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=tile_m,
                                                 dtype_in=dtype, dtype_w=dtype, dtype_out=dtype)
    np.testing.assert_array_equal(outs[1].view(np.uint16), outs[0].view(np.uint16))
    np.testing.assert_array_equal(mask_outs[1], mask_outs[0])
    np.testing.assert_array_equal(mask_outs[1], ref_mo)
    got = H.as_f32(outs[1], dtype)
    assert H.rel_err(got, H.as_f32(ref, dtype)) < TOL
    assert H.rel_err_rows(got, H.as_f32(ref, dtype)) < TOL

    dout = H.to_storage(rng.normal(0, 1, size=(n, 64)).astype(np.float32), dtype)
    din0 = np.zeros((n, 64), np.float16)
    d_dout, d_indb = H.dev(dout, dtype), H.dev(pt.indices_bwd, "i32")
    dins = []
    for hint in (0, light):
        pd = ConvParams(3, ConvOpType.BackwardInput)
        pd.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardInput, tile_m, 64)
        pd.input, pd.weight, pd.output = H.dev(din0, dtype), d_w, d_dout
        pd.indices, pd.mask, pd.mask_argsort = d_indb, d_ms, d_order
        pd.reverse_mask = True
        pd.light_prefix = hint
        ConvMainUnitTest.implicit_gemm2(pd)
        dins.append(H.host(pd.input))
    ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, din0, pt.indices_bwd, ms, order, tile_m=tile_m,
                                             dtype_in=dtype, dtype_w=dtype, dtype_out=dtype, reverse_mask=True)
    np.testing.assert_array_equal(dins[1].view(np.uint16), dins[0].view(np.uint16))
    assert H.rel_err(H.as_f32(dins[1], dtype), H.as_f32(ref_d, dtype)) < TOL
    assert H.rel_err_rows(H.as_f32(dins[1], dtype), H.as_f32(ref_d, dtype)) < TOL


def test_subm_f16_c64_order_by_offset_count_full_size():
    """The headline voxel set with input preparation as the benchmark does it: the GPU sort in its
    order by offset count, the hints found on the device (pairs for the light end, halves for
    the heavy end), the pair table by row and by position.  Same output bits as the launch on
    masks sorted by value without hints; tile masks and values against the oracle."""
    print("case full size subm f16, order by offset count", flush=True)
    dtype, tile_m, filt = "f16", 64, 0x07FFFFFF
    rng, pt, feat, w, n = _subm_case(20240607, 120000, dtype, 64, 64)
    d_mask = H.dev(pt.mask_fwd, "u32")
    d_feat, d_w, d_ind = H.dev(feat, dtype), H.dev(w, dtype), H.dev(pt.indices_fwd, "i32")
    out0 = np.zeros((n, 64), np.float16)
    tiles = (n + tile_m - 1) // tile_m

    def run(ms, order, hint, by_pos):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.Forward, tile_m, 64)
        p.input, p.weight, p.output = d_feat, d_w, H.dev(out0, dtype)
        p.indices = pairs.pairs_by_position_device(d_ind, order) if by_pos else d_ind
        p.indices_by_position = by_pos
        p.mask, p.mask_argsort, p.mask_filter = ms, order, filt
        p.mask_output = tv.zeros([tiles], tv.uint32, 0)
        p.light_prefix = hint
        ConvMainUnitTest.implicit_gemm2(p)
        return H.host(p.output), H.host(p.mask_output)

    ms_v, order_v = pairs.sort_by_mask_device(d_mask, filt)
    base, _ = run(ms_v, order_v, -1, False)
    ms_c, order_c = pairs.sort_by_mask_device(d_mask, filt, by_offset_count=True)
    ms_h, order_h = pairs.sort_by_mask(pt.mask_fwd, filt, by_offset_count=True)
    np.testing.assert_array_equal(H.host(ms_c), ms_h)
    np.testing.assert_array_equal(H.host(order_c), order_h)
    light, heavy = pairs.hints_device(ms_c, filt)
    assert light == pairs.light_prefix(ms_h, light_offsets=3) and heavy == pairs.heavy_from(ms_h)
    assert light >= 64 * 1000 and 0 < (n - heavy) // 64 <= tiles // 8            # hundreds of pairs, some halves
    ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms_h, order_h, tile_m=tile_m, dtype_in=dtype,
                                                 dtype_w=dtype, dtype_out=dtype, mask_filter=filt)
    for by_pos in (False, True):
        got, mo = run(ms_c, order_c, 0, by_pos)
        np.testing.assert_array_equal(got.view(np.uint16), base.view(np.uint16))
        np.testing.assert_array_equal(mo, ref_mo)
    assert H.rel_err(H.as_f32(got, dtype), H.as_f32(ref, dtype)) < TOL
    assert H.rel_err_rows(H.as_f32(got, dtype), H.as_f32(ref, dtype)) < TOL


def test_subm_f16_c64_wgrad_full_size():
    """Backward-weight at the benchmark size with the balanced descriptor and split_k_slices = 32
    (eight fp32 images), on the reduced masks that the forward pass writes."""
    print("case full size subm f16 wgrad", flush=True)
    dtype, tile_m = "f16", 64
    rng, pt, feat, w, n = _subm_case(20240607, 120000, dtype, 64, 64)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    red = conv_ref.tile_masks(ms, tile_m)
    dout = H.to_storage(rng.normal(0, 1, size=(n, 64)).astype(np.float32), dtype)
    dw0 = np.zeros((64, 27, 64), np.float16)
    p = ConvParams(3, ConvOpType.BackwardWeight)
    p.conv_algo_desp = H.find_conv_desp(dtype, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)
    p.input, p.weight, p.output = H.dev(feat, dtype), H.dev(dw0, dtype), H.dev(dout, dtype)
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(red, "u32"), H.dev(order, "i32")
    p.mask_width = tile_m
    p.split_k_slices = 32
    for _ in range(2):   # the second call finds the workspace of the first
        ConvMainUnitTest.implicit_gemm2(p)
    ref = conv_ref.implicit_gemm_wgrad_ref(
        dout, feat, dw0, pt.indices_fwd, red, order, mask_width=tile_m, dtype_dout=dtype,
        dtype_in=dtype, dtype_w=dtype, split_k_slices=1)
    assert H.rel_err(H.as_f32(H.host(p.weight), dtype), H.as_f32(ref, dtype)) < TOL
    # per (output channel, kernel offset) row of the gradient
    assert H.rel_err_rows(H.as_f32(H.host(p.weight), dtype).reshape(64 * 27, 64),
                          H.as_f32(ref, dtype).reshape(64 * 27, 64)) < TOL


def test_s8_stride2_full_size_bit_exact():
    print("case full size s8 stride 2", flush=True)
    rng = np.random.default_rng(20240611)
    coords = synth.clustered_voxels(rng, 300000, GRID, 60, sigma=15.0, noise_frac=0.10)
    pt = pairs.sparse_conv_pairs(coords, GRID)
    n_in, n_out = coords.shape[0], pt.indices_fwd.shape[1]
    feat = rng.integers(-127, 128, size=(n_in, 64)).astype(np.int8)
    w = rng.integers(-127, 128, size=(128, 27, 64)).astype(np.int8)
    scale = rng.uniform(0.001, 0.01, size=(128,)).astype(np.float32)
    bias = rng.normal(0, 1, size=(128,)).astype(np.float32)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = np.zeros((n_out, 128), np.int8)
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp("s8", ConvOpType.Forward, 64, 128, int8_inference=True)
    p.input, p.weight, p.output = H.dev(feat, "s8"), H.dev(w, "s8"), H.dev(out0, "s8")
    p.scale, p.bias = H.dev(scale, "f32"), H.dev(bias, "f32")
    p.indices = H.dev(pt.indices_fwd, "i32")
    p.mask, p.mask_argsort = H.dev(ms, "u32"), H.dev(order, "i32")
    ConvMainUnitTest.implicit_gemm2(p)
    ref, _, acc = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=64, dtype_in="s8",
                                                 dtype_w="s8", dtype_out="s8", scale=scale, bias=bias,
                                                 int8_inference=True, return_acc=True)
    np.testing.assert_array_equal(H.host(p.output), ref)

    # the same launch on the pair table in the order of the sorted positions: the same bits
    p.output = H.dev(out0, "s8")
    p.indices = pairs.pairs_by_position_device(p.indices, p.mask_argsort)
    p.indices_by_position = True
    ConvMainUnitTest.implicit_gemm2(p)
    np.testing.assert_array_equal(H.host(p.output), ref)
    p.indices, p.indices_by_position = H.dev(pt.indices_fwd, "i32"), False

    # the s32 accumulators themselves ("s8,s8,s32,s32,s32"): bit-exact against the oracle's
    # exact integer sums, and through the integer linear combination with a source
    src = rng.integers(-1000, 1000, size=(n_out, 128)).astype(np.int32)
    q = ConvParams(3, ConvOpType.Forward)
    q.conv_algo_desp = H.find_conv_desp("s8", ConvOpType.Forward, 64, 128, dtype_out="s32")
    q.input, q.weight, q.output = p.input, p.weight, H.dev(src, "s32")
    q.indices, q.mask, q.mask_argsort = p.indices, p.mask, p.mask_argsort
    ConvMainUnitTest.implicit_gemm2(q)
    np.testing.assert_array_equal(H.host(q.output), acc)
    q.output = H.dev(src, "s32")
    q.alpha, q.beta = 3.0, -2.0
    ConvMainUnitTest.implicit_gemm2(q)
    np.testing.assert_array_equal(H.host(q.output).astype(np.int64), 3 * acc.astype(np.int64) - 2 * src.astype(np.int64))


def test_gather_gemm_scatter_full_size():
    """One kernel offset: F[200000,64] f16, W[64,64], 150000 (in, out) pairs, alpha = beta = 1."""
    print("case full size gather-gemm-scatter", flush=True)
    dtype = "f16"
    rng = np.random.default_rng(20240609)
    rows, m, n, k = 200000, 150000, 64, 64
    a = H.to_storage(rng.normal(0, 1, size=(rows, k)).astype(np.float32), dtype)
    b = H.to_storage(rng.normal(0, 0.1, size=(k, n)).astype(np.float32), dtype)
    a_inds = rng.permutation(rows)[:m].astype(np.int32)
    c_inds = rng.permutation(rows)[:m].astype(np.int32)
    c0 = H.to_storage(rng.normal(0, 1, size=(rows, n)).astype(np.float32), dtype)
    p = GemmParams()
    p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.ShuffleAC, 64, 64, False, False)
    p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(c0, dtype)
    p.a_inds, p.c_inds = H.dev(a_inds, "i32"), H.dev(c_inds, "i32")
    p.alpha, p.beta = 1.0, 1.0
    GemmMainUnitTest.matmul2(p)
    ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype,
                               shuffle=gemm_ref.SHUFFLE_AC, a_inds=a_inds, c_inds=c_inds, alpha=1.0, beta=1.0)
    got = H.as_f32(H.host(p.c), dtype)
    assert H.rel_err(got, H.as_f32(ref, dtype)) < TOL
    assert H.rel_err_rows(got, H.as_f32(ref, dtype)) < TOL
    untouched = np.setdiff1d(np.arange(rows), c_inds)
    np.testing.assert_array_equal(H.host(p.c)[untouched], c0[untouched])   # rows not in c_inds stay as they were


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(2000, 1544, 512, 0.0), (2048, 2048, 1024, 1.0), (3000, 1000, 192, 0.5),
                                   (4100, 4104, 128, 1.0)])
def test_dense_gemm_large(dtype, shape):
    """Plain matmul2 with A [m, k] and B [n, k] at sizes that select the LDS-ring GEMM kernel:
    ragged m and n, accumulation into C, against a float32 matrix product of the stored values
    (the last shape has a 256 x 256 tile per CU and takes the 8-wave variant)."""
    m, n, k, beta = shape
    print("case dense gemm", dtype, shape, flush=True)
    rng = np.random.default_rng(20240613)
    a = H.to_storage(rng.normal(0, 1, size=(m, k)).astype(np.float32), dtype)
    b = H.to_storage(rng.normal(0, 0.1, size=(n, k)).astype(np.float32), dtype)
    c0 = H.to_storage(rng.normal(0, 1, size=(m, n)).astype(np.float32), dtype)
    p = GemmParams()
    p.algo_desp = H.find_gemm_desp(dtype, ShuffleStrideType.NoShuffle, 128, 128, False, True)
    p.a, p.b, p.c = H.dev(a, dtype), H.dev(b, dtype), H.dev(c0, dtype)
    p.alpha, p.beta = 1.0, beta
    GemmMainUnitTest.matmul2(p)
    ref = gemm_ref.matmul2_ref(a, b, c0, dtype_a=dtype, dtype_b=dtype, dtype_c=dtype, trans_b=True,
                               alpha=1.0, beta=beta)
    assert H.rel_err(H.as_f32(H.host(p.c), dtype), H.as_f32(ref, dtype)) < TOL
