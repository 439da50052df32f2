"""The bf16 sparse stack at its full size: 1 M active voxels (200 clusters on a 64 x 2048 x 2048
grid), SubMConv3d 3x3x3 layers at C = 128 with the folded-batch-norm bias and ReLU in the epilogue,
one stride-2 SparseConv3d from C = 128 to C = 256, forward and backward, backward-weight with
split-k.  Pair tables, masks and sorts come from the GPU input preparation and are compared
bit-exactly with the host builder; layer outputs are compared with the CPU oracle on the same
inputs (max relative error 1e-2, fp32 accumulation on both sides)."""
import numpy as np
import pytest

import helpers as H
from cumm_amd import pairs, synth
from cumm_amd import tensorview as tv
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.tensorview.gemm import Activation, ConvOpType, ConvParams
from oracle import conv_ref

pytestmark = pytest.mark.gpu

TOL = 1e-2
GRID = (64, 2048, 2048)
DT = "bf16"
C = 128


def _voxels():
    rng = np.random.default_rng(404)
    coords = synth.clustered_voxels(rng, 1_000_000, GRID, 200, sigma=15.0, noise_frac=0.10)
    return rng, coords


def _values(rng, shape, scale):
    """bf16-exact values (small integers times a power of two): cheap to make at this size."""
    v = rng.integers(-127, 128, size=shape, dtype=np.int8).astype(np.float32) * np.float32(scale)
    return H.to_storage(v, DT)


def _forward(x_tv, w_tv, bias_tv, out_tv, ind, ms, order, tile=(128, 128)):
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = H.find_conv_desp(DT, ConvOpType.Forward, *tile)
    p.input, p.weight, p.output, p.bias = x_tv, w_tv, out_tv, bias_tv
    p.indices, p.mask, p.mask_argsort = ind, ms, order
    p.beta, p.act_type = 1.0, Activation.ReLU
    ConvMainUnitTest.implicit_gemm2(p)


def test_stack_submanifold_layers_forward():
    print("case stack forward", flush=True)
    rng, coords = _voxels()
    n = coords.shape[0]
    table = pairs.subm_pairs_device(H.dev(coords, "i32"), GRID)
    ms_tv, order_tv = pairs.sort_by_mask_device(table.mask_fwd)
    ind, ms, order = H.host(table.indices_fwd), H.host(ms_tv), H.host(order_tv)
    ref_table = pairs.subm_pairs(coords, GRID)
    np.testing.assert_array_equal(ind, ref_table.indices_fwd)          # integer work: bit-exact
    np.testing.assert_array_equal(H.host(table.mask_fwd), ref_table.mask_fwd)
    ref_ms, ref_order = pairs.sort_by_mask(ref_table.mask_fwd)
    np.testing.assert_array_equal(ms, ref_ms)
    np.testing.assert_array_equal(order, ref_order)

    x = [_values(rng, (n, C), 1.0 / 64)]
    ws = [_values(rng, (C, 27, C), 1.0 / 2048) for _ in range(4)]
    bs = [_values(rng, (C,), 1.0 / 512) for _ in range(4)]
    acts = [H.dev(x[0], DT)]
    for l in range(4):
        out = tv.zeros([n, C], tv.bfloat16, 0)
        _forward(acts[-1], H.dev(ws[l], DT), H.dev(bs[l], DT), out, table.indices_fwd, ms_tv, order_tv)
        acts.append(out)
        x.append(H.host(out))
    zero = np.zeros((n, C), np.uint16)
    for l in (0, 3):      # first and last layer against the oracle, each on the input the GPU layer had
        print("  oracle layer", l, flush=True)
        ref, _ = conv_ref.implicit_gemm_fwd_ref(x[l], ws[l], zero, ind, ms, order, tile_m=128, dtype_in=DT,
                                                dtype_w=DT, dtype_out=DT, bias=bs[l], beta=1.0,
                                                act=Activation.ReLU.value)
        got, want = H.as_f32(x[l + 1], DT), H.as_f32(ref, DT)
        assert np.count_nonzero(want) > want.size // 4      # ReLU leaves a good part alive
        assert H.rel_err(got, want) < TOL
    # every layer: ReLU outputs are non-negative and not all zero
    for l in range(1, 5):
        f = H.as_f32(x[l], DT)
        assert f.min() >= 0.0 and f.max() > 0.0


def test_stack_downsample_layer_forward_and_backward():
    print("case stack stride 2", flush=True)
    rng, coords = _voxels()
    n_in = coords.shape[0]
    table = pairs.sparse_conv_pairs_device(H.dev(coords, "i32"), GRID, batch_size=1)
    ref_table = pairs.sparse_conv_pairs(coords, GRID)
    ind_f, ind_b = H.host(table.indices_fwd), H.host(table.indices_bwd)
    np.testing.assert_array_equal(ind_f, ref_table.indices_fwd)
    np.testing.assert_array_equal(ind_b, ref_table.indices_bwd)
    np.testing.assert_array_equal(H.host(table.out_coords), ref_table.out_coords)
    np.testing.assert_array_equal(H.host(table.mask_fwd), ref_table.mask_fwd)
    np.testing.assert_array_equal(H.host(table.mask_bwd), ref_table.mask_bwd)
    n_out = ind_f.shape[1]
    K = 256
    ms_tv, order_tv = pairs.sort_by_mask_device(table.mask_fwd)
    ms, order = H.host(ms_tv), H.host(order_tv)
    x = _values(rng, (n_in, C), 1.0 / 64)
    w = _values(rng, (K, 27, C), 1.0 / 2048)
    b = _values(rng, (K,), 1.0 / 512)
    x_tv, w_tv = H.dev(x, DT), H.dev(w, DT)
    out = tv.zeros([n_out, K], tv.bfloat16, 0)
    _forward(x_tv, w_tv, H.dev(b, DT), out, table.indices_fwd, ms_tv, order_tv)
    print("  oracle forward", flush=True)
    ref, _ = conv_ref.implicit_gemm_fwd_ref(x, w, np.zeros((n_out, K), np.uint16), ind_f, ms, order, tile_m=128,
                                            dtype_in=DT, dtype_w=DT, dtype_out=DT, bias=b, beta=1.0,
                                            act=Activation.ReLU.value)
    assert H.rel_err(H.as_f32(H.host(out), DT), H.as_f32(ref, DT)) < TOL

    # backward-input: the input-side masks, sorted on their own
    dout = _values(rng, (n_out, K), 1.0 / 64)
    dout_tv = H.dev(dout, DT)
    msb_tv, orderb_tv = pairs.sort_by_mask_device(table.mask_bwd)
    pd = ConvParams(3, ConvOpType.BackwardInput)
    pd.conv_algo_desp = H.find_conv_desp(DT, ConvOpType.BackwardInput, 128, 128)
    pd.input, pd.weight, pd.output = tv.zeros([n_in, C], tv.bfloat16, 0), w_tv, dout_tv
    pd.indices, pd.mask, pd.mask_argsort = table.indices_bwd, msb_tv, orderb_tv
    ConvMainUnitTest.implicit_gemm2(pd)
    print("  oracle backward-input", flush=True)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, np.zeros((n_in, C), np.uint16), ind_b, H.host(msb_tv),
                                             H.host(orderb_tv), tile_m=128, dtype_in=DT, dtype_w=DT,
                                             dtype_out=DT, reverse_mask=False)
    assert H.rel_err(H.as_f32(H.host(pd.input), DT), H.as_f32(ref_d, DT)) < TOL

    # backward-weight, balanced split-k
    red = conv_ref.tile_masks(ms, 64)
    pw = ConvParams(3, ConvOpType.BackwardWeight)
    pw.conv_algo_desp = H.find_conv_desp(DT, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=True)
    pw.input, pw.weight, pw.output = x_tv, tv.zeros([K, 27, C], tv.bfloat16, 0), dout_tv
    pw.indices, pw.mask, pw.mask_argsort = table.indices_fwd, H.dev(red, "u32"), order_tv
    pw.mask_width, pw.split_k_slices = 64, 32
    ConvMainUnitTest.implicit_gemm2(pw)
    print("  oracle backward-weight", flush=True)
    ref_w = conv_ref.implicit_gemm_wgrad_ref(dout, x, np.zeros((K, 27, C), np.uint16), ind_f, red, order,
                                             mask_width=64, dtype_dout=DT, dtype_in=DT, dtype_w=DT, split_k_slices=1)
    assert H.rel_err(H.as_f32(H.host(pw.weight), DT), H.as_f32(ref_w, DT)) < TOL


def test_stack_submanifold_layer_backward():
    print("case stack backward", flush=True)
    rng, coords = _voxels()
    n = coords.shape[0]
    table = pairs.subm_pairs_device(H.dev(coords, "i32"), GRID)
    ms_tv, order_tv = pairs.sort_by_mask_device(table.mask_fwd)
    ind_f, ind_b, ms, order = (H.host(t) for t in (table.indices_fwd, table.indices_bwd, ms_tv, order_tv))
    x = _values(rng, (n, C), 1.0 / 64)
    w = _values(rng, (C, 27, C), 1.0 / 2048)
    dout = _values(rng, (n, C), 1.0 / 64)
    x_tv, w_tv, dout_tv = H.dev(x, DT), H.dev(w, DT), H.dev(dout, DT)

    pd = ConvParams(3, ConvOpType.BackwardInput)
    pd.conv_algo_desp = H.find_conv_desp(DT, ConvOpType.BackwardInput, 128, 128)
    pd.input, pd.weight, pd.output = tv.zeros([n, C], tv.bfloat16, 0), w_tv, dout_tv
    pd.indices, pd.mask, pd.mask_argsort = table.indices_bwd, ms_tv, order_tv
    pd.reverse_mask = True
    ConvMainUnitTest.implicit_gemm2(pd)
    print("  oracle backward-input", flush=True)
    ref_d = conv_ref.implicit_gemm_dgrad_ref(dout, w, np.zeros((n, C), np.uint16), ind_b, ms, order, tile_m=128,
                                             dtype_in=DT, dtype_w=DT, dtype_out=DT, reverse_mask=True)
    assert H.rel_err(H.as_f32(H.host(pd.input), DT), H.as_f32(ref_d, DT)) < TOL

    red = conv_ref.tile_masks(ms, 64)
    red_tv = H.dev(red, "u32")
    # balanced atomic variant (one rounding at the end), then serial split-k (the partial sums
    # round to bf16 between the slices, which the oracle follows)
    for parallel, slices, ref_slices in ((True, 32, 1), (False, 8, 8)):
        pw = ConvParams(3, ConvOpType.BackwardWeight)
        pw.conv_algo_desp = H.find_conv_desp(DT, ConvOpType.BackwardWeight, 64, 64, split_k_parallel=parallel)
        pw.input, pw.weight, pw.output = x_tv, tv.zeros([C, 27, C], tv.bfloat16, 0), dout_tv
        pw.indices, pw.mask, pw.mask_argsort = table.indices_fwd, red_tv, order_tv
        pw.mask_width, pw.split_k_slices = 64, slices
        ConvMainUnitTest.implicit_gemm2(pw)
        print("  oracle backward-weight", parallel, flush=True)
        ref_w = conv_ref.implicit_gemm_wgrad_ref(dout, x, np.zeros((C, 27, C), np.uint16), ind_f, red, order,
                                                 mask_width=64, dtype_dout=DT, dtype_in=DT, dtype_w=DT,
                                                 split_k_slices=ref_slices, tile_k=32)
        assert H.rel_err(H.as_f32(H.host(pw.weight), DT), H.as_f32(ref_w, DT)) < TOL
