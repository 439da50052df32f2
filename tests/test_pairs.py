"""The host pair-table builder against the oracle's brute-force dictionary search
(bit-exact), on SubM and strided problems, with ragged / tiny / dilated cases."""
import numpy as np
import pytest

from oracle import pairs_ref

from cumm_amd import pairs, synth


@pytest.mark.parametrize("seed,n,grid,dil", [(0, 300, (8, 20, 18), (1, 1, 1)), (1, 1, (3, 3, 3), (1, 1, 1)),
                                             (2, 500, (5, 30, 30), (2, 1, 2)), (3, 64, (4, 4, 4), (1, 1, 1))])
def test_subm_pairs_bit_exact(seed, n, grid, dil):
    rng = np.random.default_rng(seed)
    coords = synth.clustered_voxels(rng, n, grid, 3, sigma=2.5)
    pt = pairs.subm_pairs(coords, grid, dilation=dil)
    ref = pairs_ref.subm_pairs_ref(coords, grid, dilation=dil)
    np.testing.assert_array_equal(pt.indices_fwd, ref)
    np.testing.assert_array_equal(pt.mask_fwd, pairs_ref.masks_ref(ref))
    assert pt.indices_fwd.dtype == np.int32 and pt.mask_fwd.dtype == np.uint32


@pytest.mark.parametrize("seed,n,grid,stride,pad", [(0, 300, (9, 21, 18), (2, 2, 2), (1, 1, 1)),
                                                    (1, 2, (4, 4, 4), (2, 2, 2), (1, 1, 1)),
                                                    (2, 400, (8, 16, 17), (1, 2, 2), (1, 1, 1)),
                                                    (3, 200, (10, 10, 10), (2, 2, 2), (0, 0, 0))])
def test_strided_pairs_bit_exact(seed, n, grid, stride, pad):
    rng = np.random.default_rng(seed)
    coords = synth.clustered_voxels(rng, n, grid, 3, sigma=2.5)
    pt = pairs.sparse_conv_pairs(coords, grid, stride=stride, padding=pad)
    f, b, oc = pairs_ref.sparse_conv_pairs_ref(coords, grid, (3, 3, 3), stride, pad, (1, 1, 1))
    np.testing.assert_array_equal(pt.out_coords, oc)
    np.testing.assert_array_equal(pt.indices_fwd, f)
    np.testing.assert_array_equal(pt.indices_bwd, b)
    np.testing.assert_array_equal(pt.mask_fwd, pairs_ref.masks_ref(f))
    np.testing.assert_array_equal(pt.mask_bwd, pairs_ref.masks_ref(b))
    assert pt.out_shape == pairs_ref.calc_output_dims(grid, (3, 3, 3), pad, stride, (1, 1, 1))
    assert (pt.indices_fwd >= 0).sum() == (pt.indices_bwd >= 0).sum()


def test_sort_by_mask_is_stable_and_filtered():
    m = np.array([5, 1, 5, 0, 1, 8 | 5], np.uint32)
    ms, order = pairs.sort_by_mask(m)
    np.testing.assert_array_equal(order, [3, 1, 4, 0, 2, 5])
    np.testing.assert_array_equal(ms, m[order])
    ms2, order2 = pairs.sort_by_mask(m, 0x4)
    np.testing.assert_array_equal(ms2, (m & 4)[order2])
    np.testing.assert_array_equal(order2, [1, 3, 4, 0, 2, 5])


def test_light_prefix_counts_whole_runs_of_light_halves():
    c = np.uint32(1 << 13)
    m = np.full(700, c, np.uint32)
    assert pairs.light_prefix(m) == 640                 # five whole runs of 128; the rest is not counted
    assert pairs.light_prefix(m[:127]) == 0
    m[300] |= 1                                         # two offsets in a half are still light
    assert pairs.light_prefix(m) == 640
    m[310] |= 2                                         # a third offset in the same half of run 2
    assert pairs.light_prefix(m) == 256
    assert pairs.light_prefix(m, mask_filter=0xFFFFFFFD) == 640
    m[5] = 7
    assert pairs.light_prefix(m) == 0
    assert pairs.light_prefix(np.zeros(0, np.uint32)) == 0


def test_synthetic_cloud_is_unique_in_grid_and_seeded():
    grid = (41, 200, 176)
    a = synth.clustered_voxels(np.random.default_rng(7), 5000, grid, 8)
    b = synth.clustered_voxels(np.random.default_rng(7), 5000, grid, 8)
    np.testing.assert_array_equal(a, b)
    assert len({tuple(r) for r in a.tolist()}) == a.shape[0]
    assert (a[:, 1:] >= 0).all() and (a[:, 1:] < np.array(grid)).all()
    assert abs(a.shape[0] - 5000) < 100


def test_subm_backward_table_is_the_inverse_relation_and_even_sizes_are_rejected():
    """indices_bwd must be the inverse relation of indices_fwd (input i feeds output o through
    offset k iff o gathers i through k); for odd kernel sizes that is the forward table reversed.
    Even sizes have asymmetric offsets, for which the reversal is wrong: rejected."""
    rng = np.random.default_rng(5)
    grid = (6, 12, 11)
    coords = synth.clustered_voxels(rng, 250, grid, 3, sigma=2.0)
    for ksize in ((3, 3, 3), (1, 3, 5), (3, 1, 1)):
        pt = pairs.subm_pairs(coords, grid, ksize=ksize)
        kv, n = pt.indices_fwd.shape
        inv = np.full((kv, n), -1, np.int32)
        for k in range(kv):
            o = np.nonzero(pt.indices_fwd[k] >= 0)[0]
            inv[k, pt.indices_fwd[k, o]] = o
        np.testing.assert_array_equal(pt.indices_bwd, inv)
        np.testing.assert_array_equal(pt.mask_bwd, pairs_ref.masks_ref(inv))
    for ksize in ((1, 1, 2), (2, 2, 2), (3, 4, 3)):
        with pytest.raises(ValueError, match="odd"):
            pairs.subm_pairs(coords, grid, ksize=ksize)
