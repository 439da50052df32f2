"""Pins for the per-offset ("native") convolution oracle and for the host pair builders at kernel
volumes above 32: torch's dense conv3d (cross-correlation) and autograd on small grids with a
5 x 5 x 5 submanifold kernel and a strided 3 x 3 x 5 one, and brute-force pair tables."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import native_ref, pairs_ref

from cumm_amd import pairs, synth


@pytest.mark.parametrize("case", ["subm555", "strided335"])
def test_native_oracle_against_dense_conv3d(case):
    rng = np.random.default_rng(41)
    grid = (9, 10, 11)
    c_in, k_out = 8, 16
    coords = synth.clustered_voxels(rng, 150, grid, 3, sigma=2.0)
    if case == "subm555":
        ksize, stride, padding = (5, 5, 5), (1, 1, 1), (2, 2, 2)
        pt = pairs.subm_pairs(coords, grid, ksize=ksize)
        np.testing.assert_array_equal(pt.indices_fwd, pairs_ref.subm_pairs_ref(coords, grid, ksize))
    else:
        ksize, stride, padding = (3, 3, 5), (2, 2, 2), (1, 1, 2)
        pt = pairs.sparse_conv_pairs(coords, grid, ksize=ksize, stride=stride, padding=padding)
        f, b, oc = pairs_ref.sparse_conv_pairs_ref(coords, grid, ksize, stride, padding, (1, 1, 1))
        np.testing.assert_array_equal(pt.indices_fwd, f)
        np.testing.assert_array_equal(pt.indices_bwd, b)
        np.testing.assert_array_equal(pt.out_coords, oc)
    kv = ksize[0] * ksize[1] * ksize[2]
    assert pt.mask_fwd is None and kv > 32
    lists = pairs.pair_lists(pt.indices_fwd)
    assert int(lists.counts.sum()) == int((pt.indices_fwd >= 0).sum())
    n_in, n_out = coords.shape[0], pt.indices_fwd.shape[1]
    feat = rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32)
    w_ref = rng.normal(0, 0.2, size=(kv, k_out, c_in)).astype(np.float32)
    weight = np.ascontiguousarray(w_ref.transpose(1, 0, 2))
    bias = rng.normal(0, 1, size=(k_out,)).astype(np.float32)
    dense = torch.zeros(1, c_in, *grid, dtype=torch.float64)
    dense[0, :, coords[:, 1], coords[:, 2], coords[:, 3]] = torch.from_numpy(feat.T.astype(np.float64))
    wt = torch.from_numpy(w_ref.astype(np.float64)).reshape(*ksize, k_out, c_in).permute(3, 4, 0, 1, 2).contiguous()
    dense.requires_grad_(True)
    wt.requires_grad_(True)
    out_dense = F.conv3d(dense, wt, padding=padding, stride=stride)
    oc = pt.out_coords
    want = out_dense[0, :, oc[:, 1], oc[:, 2], oc[:, 3]].T.detach().numpy()
    got = native_ref.native_fwd_ref(feat, weight, lists.pair_in, lists.pair_out, lists.counts, n_out, dtype="f32")
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    got_b = native_ref.native_fwd_ref(feat, weight, lists.pair_in, lists.pair_out, lists.counts, n_out, dtype="f32",
                                      bias=bias, act=1)
    np.testing.assert_allclose(got_b, np.maximum(want + bias[None, :], 0), rtol=1e-4, atol=1e-4)
    dout = rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32)
    gdense = torch.zeros_like(out_dense)
    gdense[0, :, oc[:, 1], oc[:, 2], oc[:, 3]] = torch.from_numpy(dout.T.astype(np.float64))
    out_dense.backward(gdense)
    want_din = dense.grad[0, :, coords[:, 1], coords[:, 2], coords[:, 3]].T.numpy()
    want_dw = wt.grad.permute(2, 3, 4, 0, 1).reshape(kv, k_out, c_in).numpy()
    din = native_ref.native_dgrad_ref(dout, weight, lists.pair_in, lists.pair_out, lists.counts, n_in, dtype="f32")
    np.testing.assert_allclose(din, want_din, rtol=1e-4, atol=1e-4)
    dw = native_ref.native_wgrad_ref(dout, feat, lists.pair_in, lists.pair_out, lists.counts, kv, dtype="f32")
    np.testing.assert_allclose(dw.transpose(1, 0, 2), want_dw, rtol=1e-4, atol=1e-4)


def test_pair_lists_are_the_table_packed_in_ascending_output_order():
    rng = np.random.default_rng(42)
    grid = (6, 9, 9)
    coords = synth.clustered_voxels(rng, 120, grid, 2, sigma=2.0)
    pt = pairs.subm_pairs(coords, grid)
    lists = pairs.pair_lists(pt.indices_fwd)
    for k in range(27):
        n = int(lists.counts[k])
        o = lists.pair_out[k][:n]
        assert np.all(np.diff(o) > 0)
        np.testing.assert_array_equal(pt.indices_fwd[k][o], lists.pair_in[k][:n])
        assert n == int((pt.indices_fwd[k] >= 0).sum())
