"""Pair tables and mask sort built on the GPU against the host builder (integer work: bit-exact)."""
import numpy as np
import pytest

import helpers as H
from cumm_amd import _capi, pairs, synth
from cumm_amd import tensorview as tv

pytestmark = pytest.mark.gpu


def _check_case(coords, shape, ksize=(3, 3, 3), dilation=(1, 1, 1)):
    ref = pairs.subm_pairs(coords, shape, ksize, dilation)
    got = pairs.subm_pairs_device(H.dev(np.ascontiguousarray(coords, np.int32), "i32"), shape, ksize, dilation)
    np.testing.assert_array_equal(H.host(got.indices_fwd), ref.indices_fwd)
    np.testing.assert_array_equal(H.host(got.indices_bwd), ref.indices_bwd)
    np.testing.assert_array_equal(H.host(got.mask_fwd), ref.mask_fwd)
    np.testing.assert_array_equal(H.host(got.mask_bwd), ref.mask_bwd)
    return ref, got


@pytest.mark.parametrize("n,shape", [(1, (4, 4, 4)), (65, (6, 10, 10)), (3000, (12, 40, 40)), (5000, (9, 17, 33))])
def test_subm_pairs_small(n, shape):
    print("case subm pairs", n, shape, flush=True)
    rng = np.random.default_rng(100 + n)
    total = 2 * shape[0] * shape[1] * shape[2]     # two batches
    cells = rng.choice(total, size=min(n, total), replace=False)
    coords = np.stack(np.unravel_index(cells, (2,) + tuple(shape)), axis=1).astype(np.int32)
    _check_case(coords, shape)


def test_subm_pairs_dense_block_and_kernel_shapes():
    """Every voxel of a block (all 27 neighbours inside), then 1x3x3 and dilation 2."""
    g = np.stack(np.meshgrid(np.arange(8), np.arange(9), np.arange(10), indexing="ij"), -1).reshape(-1, 3)
    coords = np.zeros((g.shape[0], 4), np.int32)
    coords[:, 1:] = g
    rng = np.random.default_rng(5)
    coords = coords[rng.permutation(coords.shape[0])]
    _check_case(coords, (8, 9, 10))
    _check_case(coords, (8, 9, 10), ksize=(1, 3, 3))
    _check_case(coords, (8, 9, 10), ksize=(3, 3, 3), dilation=(2, 2, 2))


def test_subm_pairs_and_sort_full_size():
    """The benchmark's voxel set (120 k voxels in 41 x 1600 x 1408): tables, masks, sorted masks and
    argsort, bit-exact; then a split filter."""
    print("case subm pairs full size", flush=True)
    rng = np.random.default_rng(20240607)
    grid = (41, 1600, 1408)
    coords = synth.clustered_voxels(rng, 120000, grid, 60, sigma=15.0, noise_frac=0.10)
    ref, got = _check_case(coords, grid)
    for filt in (0xFFFFFFFF, 0x3FFF, 0x1FFF << 14):
        ms_ref, order_ref = pairs.sort_by_mask(ref.mask_fwd, filt)
        ms, order = pairs.sort_by_mask_device(got.mask_fwd, filt)
        np.testing.assert_array_equal(H.host(ms), ms_ref)
        np.testing.assert_array_equal(H.host(order), order_ref)


def test_pairs_argument_errors():
    lib = _capi.lib()
    assert lib.cumm_hip_subm_pairs_workspace(1000) >= 2 * 1000 * 16
    c = tv.zeros([8, 4], tv.int32, 0)
    with pytest.raises(ValueError):
        pairs.subm_pairs_device(c, (4, 4, 4), ksize=(3, 3, 5))        # kernel volume 45 > 32
    with pytest.raises(RuntimeError):
        pairs.subm_pairs_device(c, (4, 4, 4), workspace=tv.zeros([64], tv.uint8, 0))   # too small
