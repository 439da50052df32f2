"""Pins for the sparse-convolution oracle: the densified problem run through torch's dense
conv3d (cross-correlation) and autograd on small grids, plus integer closed forms for the
tile masks.  A wrong offset order, a transposed weight, a swapped pair table or a dropped
offset fails these."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import conv_ref, pairs_ref
from oracle import numerics as nm

from cumm_amd import pairs, synth


def _dense_problem(seed, grid, n, c_in, k_out, stride):
    rng = np.random.default_rng(seed)
    coords = synth.clustered_voxels(rng, n, grid, 3, sigma=2.0)
    feat = rng.normal(0, 1, size=(coords.shape[0], c_in)).astype(np.float32)
    w_ref = rng.normal(0, 0.2, size=(27, k_out, c_in)).astype(np.float32)   # [kv, K, C]
    weight = np.ascontiguousarray(w_ref.transpose(1, 0, 2))                 # [K, kv, C]
    if stride == 1:
        pt = pairs.subm_pairs(coords, grid)
    else:
        pt = pairs.sparse_conv_pairs(coords, grid, stride=(stride,) * 3)
    dense = torch.zeros(1, c_in, *grid, dtype=torch.float64)
    dense[0, :, coords[:, 1], coords[:, 2], coords[:, 3]] = torch.from_numpy(feat.T.astype(np.float64))
    # torch weight [K, C, kz, ky, kx]; offset index k = (kz*3+ky)*3+kx
    wt = torch.from_numpy(w_ref.astype(np.float64)).reshape(3, 3, 3, k_out, c_in).permute(3, 4, 0, 1, 2)
    return coords, pt, feat, weight, dense, wt.contiguous()


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("tile_m", [32, 64])
def test_forward_dgrad_wgrad_against_dense_conv3d(stride, tile_m):
    grid = (7, 9, 8)
    c_in, k_out = 8, 16
    coords, pt, feat, weight, dense, wt = _dense_problem(11 + stride, grid, 120, c_in, k_out, stride)
    dense.requires_grad_(True)
    wt.requires_grad_(True)
    out_dense = F.conv3d(dense, wt, padding=1, stride=stride)
    oc = pt.out_coords
    n_out = oc.shape[0]
    want_out = out_dense[0, :, oc[:, 1], oc[:, 2], oc[:, 3]].T.detach().numpy()

    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = np.zeros((n_out, k_out), np.float32)
    got, mask_out = conv_ref.implicit_gemm_fwd_ref(feat, weight, out0, pt.indices_fwd, ms, order,
                                                   tile_m=tile_m, dtype_in="f32", dtype_w="f32",
                                                   dtype_out="f32")
    np.testing.assert_allclose(got, want_out, rtol=1e-4, atol=1e-4)
    if stride == 2:
        # every active output of the strided conv is a non-zero site of the dense result's support
        assert n_out == len({tuple(c) for c in oc.tolist()})

    # backward: gradient of sum(out * dout) restricted to the active sites
    rng = np.random.default_rng(5)
    dout = rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32)
    gdense = torch.zeros_like(out_dense)
    gdense[0, :, oc[:, 1], oc[:, 2], oc[:, 3]] = torch.from_numpy(dout.T.astype(np.float64))
    out_dense.backward(gdense)
    want_din = dense.grad[0, :, coords[:, 1], coords[:, 2], coords[:, 3]].T.numpy()
    want_dw = wt.grad.permute(2, 3, 4, 0, 1).reshape(27, k_out, c_in).numpy()   # [kv, K, C]

    if stride == 1:
        msb, orderb, table, reverse = ms, order, pt.indices_bwd, True   # forward mask, reversed
    else:
        msb, orderb = pairs.sort_by_mask(pt.mask_bwd)
        table, reverse = pt.indices_bwd, False
    din = conv_ref.implicit_gemm_dgrad_ref(dout, weight, np.zeros_like(feat), table, msb, orderb,
                                           tile_m=tile_m, dtype_in="f32", dtype_w="f32",
                                           dtype_out="f32", reverse_mask=reverse)
    np.testing.assert_allclose(din, want_din, rtol=1e-4, atol=1e-4)

    red = conv_ref.tile_masks(ms, tile_m)
    np.testing.assert_array_equal(red, mask_out)
    for split in (1, 3):
        dw = conv_ref.implicit_gemm_wgrad_ref(dout, feat, np.zeros_like(weight), pt.indices_fwd, red,
                                              order, mask_width=tile_m, dtype_dout="f32",
                                              dtype_in="f32", dtype_w="f32", split_k_slices=split,
                                              tile_k=32)
        np.testing.assert_allclose(dw.transpose(1, 0, 2), want_dw, rtol=1e-4, atol=1e-4)


def test_tile_mask_closed_forms_and_reverse():
    rng = np.random.default_rng(0)
    m = rng.integers(0, 1 << 27, size=1000, dtype=np.uint32)
    for tile_m in (32, 64, 128):
        km = conv_ref.tile_masks(m, tile_m, 0x07FFFFFF)
        for t in range(len(km)):
            want = 0
            for v in m[t * tile_m:(t + 1) * tile_m]:
                want |= int(v)
            assert km[t] == want
        km2 = conv_ref.tile_masks(m, tile_m, 0x3FFF)
        np.testing.assert_array_equal(km2, km & 0x3FFF)
    x = np.array([1, 1 << 26, 0b101, 0x07FFFFFF], np.uint32)
    rev = conv_ref.bitrev32(x) >> np.uint32(32 - 27)
    np.testing.assert_array_equal(rev, np.array([1 << 26, 1, 0b101 << 24, 0x07FFFFFF], np.uint32))


def test_subm_backward_table_is_the_reversed_forward_table():
    rng = np.random.default_rng(3)
    grid = (6, 12, 10)
    coords = synth.clustered_voxels(rng, 200, grid, 3, sigma=2.0)
    pt = pairs.subm_pairs(coords, grid)
    np.testing.assert_array_equal(pt.indices_bwd, pt.indices_fwd[::-1])
    np.testing.assert_array_equal(pt.mask_bwd, conv_ref.bitrev32(pt.mask_fwd) >> np.uint32(5))
    np.testing.assert_array_equal(pt.indices_fwd[13], np.arange(coords.shape[0]))
    # a pair (k: i -> o) appears in both tables
    for k in range(27):
        o = np.nonzero(pt.indices_fwd[k] >= 0)[0]
        i = pt.indices_fwd[k][o]
        np.testing.assert_array_equal(pt.indices_bwd[k][i], o)


def test_forward_skipped_tile_still_runs_the_epilogue_and_dgrad_does_not():
    """cumm/conv/kernel.py:875-921: forward writes act(beta*src) for a tile whose mask is empty,
    backward-input returns before writing."""
    rng = np.random.default_rng(9)
    grid = (6, 10, 10)
    coords = synth.clustered_voxels(rng, 150, grid, 2, sigma=2.0)
    pt = pairs.subm_pairs(coords, grid)
    n = coords.shape[0]
    feat = rng.normal(0, 1, (n, 8)).astype(np.float32)
    w = rng.normal(0, 1, (8, 27, 8)).astype(np.float32)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    out0 = rng.normal(0, 1, (n, 8)).astype(np.float32)
    out, mo = conv_ref.implicit_gemm_fwd_ref(feat, w, out0, pt.indices_fwd, ms, order, tile_m=32,
                                             dtype_in="f32", dtype_w="f32", dtype_out="f32",
                                             mask_filter=0, beta=0.0)
    assert not out.any() and not mo.any()
    din0 = rng.normal(0, 1, (n, 8)).astype(np.float32)
    din = conv_ref.implicit_gemm_dgrad_ref(feat, w, din0, pt.indices_bwd, ms, order, tile_m=32,
                                           dtype_in="f32", dtype_w="f32", dtype_out="f32",
                                           mask_filter=0, reverse_mask=True)
    np.testing.assert_array_equal(din, din0)


def test_wgrad_serial_split_k_rounds_between_slices():
    """With f16 weights the serial split-K result is the slice-ordered chain of roundings
    (cumm/gemm/output_op/linear.py:90-99), not the once-rounded float32 sum."""
    rng = np.random.default_rng(10)
    grid = (8, 16, 16)
    coords = synth.clustered_voxels(rng, 600, grid, 3, sigma=3.0)
    pt = pairs.subm_pairs(coords, grid)
    n = coords.shape[0]
    feat = rng.normal(0, 1, (n, 8)).astype(np.float16)
    dout = rng.normal(0, 1, (n, 8)).astype(np.float16)
    ms, order = pairs.sort_by_mask(pt.mask_fwd)
    red = conv_ref.tile_masks(ms, 64)
    kw = dict(mask_width=64, dtype_dout="f16", dtype_in="f16", dtype_w="f16", tile_k=32)
    dw0 = np.zeros((8, 27, 8), np.float16)
    one = conv_ref.implicit_gemm_wgrad_ref(dout, feat, dw0, pt.indices_fwd, red, order, split_k_slices=1, **kw)
    ser = conv_ref.implicit_gemm_wgrad_ref(dout, feat, dw0, pt.indices_fwd, red, order, split_k_slices=8, **kw)
    par = conv_ref.implicit_gemm_wgrad_ref(dout, feat, dw0, pt.indices_fwd, red, order, split_k_slices=8,
                                           serial_rounding=False, **kw)
    np.testing.assert_allclose(ser.astype(np.float32), one.astype(np.float32), rtol=2e-2, atol=2e-2)
    assert np.max(np.abs(par.astype(np.float32) - one.astype(np.float32))) <= \
        np.max(np.abs(ser.astype(np.float32) - one.astype(np.float32))) + 1e-3
    # manual chain for the centre offset
    r = 13
    pos = np.arange(n)
    cur = np.zeros((8, 8), np.float32)
    for z in range(8):
        sel = ((pos // 32) % 8 == z) & (((red[pos // 64] >> np.uint32(r)) & 1) == 1)
        o = order[sel]
        i = pt.indices_fwd[r][o]
        o, i = o[i >= 0], i[i >= 0]
        part = dout[o].astype(np.float32).T @ feat[i].astype(np.float32)
        cur = (part + (cur if z else 0 * cur)).astype(np.float16).astype(np.float32)
    np.testing.assert_array_equal(ser[:, r, :].astype(np.float32), cur)
