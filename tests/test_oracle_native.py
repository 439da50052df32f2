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


@pytest.mark.parametrize("case", ["subm555", "strided335"])
def test_dynamic_mask_oracle_against_the_per_offset_oracle(case):
    """The mask-based oracle with several mask words per position (kernel volumes above 32, the
    layout of the reference's dynamic-mask loader) pinned by the per-offset oracle, which the
    test above pins by torch's dense conv3d: forward, backward-input with the backward masks,
    and backward-input with the forward masks reversed end for end (SubM only, where the backward
    table is the forward one reversed).  The multi-word masks are pinned by the tables
    themselves, the reversal by the invariant mask_bwd == reverse(mask_fwd)."""
    from oracle import conv_ref
    rng = np.random.default_rng(43)
    grid = (9, 10, 11)
    c_in, k_out = 8, 16
    coords = synth.clustered_voxels(rng, 150, grid, 3, sigma=2.0)
    if case == "subm555":
        pt = pairs.subm_pairs(coords, grid, ksize=(5, 5, 5))
    else:
        pt = pairs.sparse_conv_pairs(coords, grid, ksize=(3, 3, 5), stride=(2, 2, 2), padding=(1, 1, 2))
    kv, n_out = pt.indices_fwd.shape
    n_in = coords.shape[0]
    words = (kv + 31) // 32
    mf, mb = pairs.masks_from_pairs(pt.indices_fwd), pairs.masks_from_pairs(pt.indices_bwd)
    assert mf.shape == (n_out, words) and mb.shape == (n_in, words)
    for k in range(kv):       # bit by bit against the table
        np.testing.assert_array_equal((mf[:, k // 32] >> np.uint32(k % 32)) & 1, (pt.indices_fwd[k] >= 0).astype(np.uint32))
    assert not (mf[:, -1] >> np.uint32(kv - 32 * (words - 1))).any()      # no bits past the kernel volume
    if case == "subm555":
        np.testing.assert_array_equal(conv_ref.reverse_mask_words(mf, kv), mb)
        np.testing.assert_array_equal(conv_ref.reverse_mask_words(mb, kv), mf)
    lists = pairs.pair_lists(pt.indices_fwd)
    feat = rng.normal(0, 1, size=(n_in, c_in)).astype(np.float32)
    weight = rng.normal(0, 0.2, size=(k_out, kv, c_in)).astype(np.float32)
    dout = rng.normal(0, 1, size=(n_out, k_out)).astype(np.float32)
    ms, order = pairs.sort_by_mask_words(mf)
    np.testing.assert_array_equal(ms, mf[order])
    assert sorted(order.tolist()) == list(range(n_out))
    want = native_ref.native_fwd_ref(feat, weight, lists.pair_in, lists.pair_out, lists.counts, n_out, dtype="f32")
    for tile_m in (64, 128):
        got, mo = conv_ref.implicit_gemm_fwd_ref(feat, weight, np.zeros((n_out, k_out), np.float32), pt.indices_fwd, ms, order,
                                                 tile_m=tile_m, dtype_in="f32", dtype_w="f32", dtype_out="f32")
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
        assert mo.shape == ((n_out + tile_m - 1) // tile_m, words)
    want_d = native_ref.native_dgrad_ref(dout, weight, lists.pair_in, lists.pair_out, lists.counts, n_in, dtype="f32")
    msb, orderb = pairs.sort_by_mask_words(mb)
    got_d = conv_ref.implicit_gemm_dgrad_ref(dout, weight, np.zeros((n_in, c_in), np.float32), pt.indices_bwd, msb, orderb,
                                             tile_m=64, dtype_in="f32", dtype_w="f32", dtype_out="f32")
    np.testing.assert_allclose(got_d, want_d, rtol=1e-4, atol=1e-4)
    if case == "subm555":
        got_r = conv_ref.implicit_gemm_dgrad_ref(dout, weight, np.zeros((n_in, c_in), np.float32), pt.indices_bwd, ms, order,
                                                 tile_m=64, dtype_in="f32", dtype_w="f32", dtype_out="f32", reverse_mask=True)
        np.testing.assert_allclose(got_r, want_d, rtol=1e-4, atol=1e-4)


def test_masks_from_pairs_agree_with_the_builders_below_33_offsets():
    rng = np.random.default_rng(44)
    grid = (6, 9, 9)
    coords = synth.clustered_voxels(rng, 120, grid, 2, sigma=2.0)
    pt = pairs.subm_pairs(coords, grid)
    np.testing.assert_array_equal(pairs.masks_from_pairs(pt.indices_fwd)[:, 0], pt.mask_fwd)
    np.testing.assert_array_equal(pairs.masks_from_pairs(pt.indices_bwd)[:, 0], pt.mask_bwd)
    keys = pairs.mask_words_keys(pairs.masks_from_pairs(pt.indices_fwd))
    pc = np.array([bin(int(m)).count("1") for m in pt.mask_fwd])
    np.testing.assert_array_equal(keys >> np.uint32(26), np.minimum(pc, 63))
    same = pt.mask_fwd[:, None] == pt.mask_fwd[None, :]
    assert ((keys[:, None] == keys[None, :]) >= same).all()          # equal masks, equal keys
