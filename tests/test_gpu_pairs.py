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
        pairs.subm_pairs_device(c, (4, 4, 4), ksize=(5, 5, 7))        # kernel volume 175 > 128
    with pytest.raises(ValueError):
        pairs.subm_pairs_device(c, (4, 4, 4), ksize=(3, 2, 3))        # even kernel size
    # kernel volume 45: tables without masks; asking for masks is an error
    big = pairs.subm_pairs_device(c, (4, 4, 4), ksize=(3, 3, 5))
    assert big.mask_fwd is None and big.indices_fwd.shape == [45, 8]
    import ctypes as C
    arr3 = C.c_int32 * 3
    ws = tv.zeros([int(lib.cumm_hip_subm_pairs_workspace(8))], tv.uint8, 0)
    m = tv.zeros([8], tv.uint32, 0)
    assert lib.cumm_hip_subm_pairs(c.byte_pointer(), 8, arr3(4, 4, 4), arr3(3, 3, 5), arr3(1, 1, 1),
                                   big.indices_fwd.byte_pointer(), None, m.byte_pointer(), None,
                                   ws.byte_pointer(), ws.nbytes, 0) == _capi.EINVAL
    with pytest.raises(RuntimeError):
        pairs.subm_pairs_device(c, (4, 4, 4), workspace=tv.zeros([64], tv.uint8, 0))   # too small


# ---- regular (strided) sparse convolution -------------------------------------------------------

def _check_conv_case(coords, shape, ksize=(3, 3, 3), stride=(2, 2, 2), padding=(1, 1, 1), dilation=(1, 1, 1),
                     batch_size=2):
    ref = pairs.sparse_conv_pairs(coords, shape, ksize, stride, padding, dilation)
    got = pairs.sparse_conv_pairs_device(H.dev(np.ascontiguousarray(coords, np.int32), "i32"), shape, ksize,
                                         stride, padding, dilation, batch_size=batch_size)
    assert tuple(got.out_shape) == tuple(ref.out_shape)
    np.testing.assert_array_equal(H.host(got.out_coords), ref.out_coords)
    np.testing.assert_array_equal(H.host(got.indices_fwd), ref.indices_fwd)
    np.testing.assert_array_equal(H.host(got.indices_bwd), ref.indices_bwd)
    np.testing.assert_array_equal(H.host(got.mask_fwd), ref.mask_fwd)
    np.testing.assert_array_equal(H.host(got.mask_bwd), ref.mask_bwd)
    return ref, got


def _random_coords(rng, n, shape, batches=2):
    total = batches * shape[0] * shape[1] * shape[2]
    cells = rng.choice(total, size=min(n, total), replace=False)
    return np.stack(np.unravel_index(cells, (batches,) + tuple(shape)), axis=1).astype(np.int32)


@pytest.mark.parametrize("n,shape", [(1, (4, 4, 4)), (65, (6, 10, 10)), (3000, (12, 40, 40)), (5000, (9, 17, 33))])
def test_sparse_conv_pairs_small(n, shape):
    print("case sparse conv pairs", n, shape, flush=True)
    _check_conv_case(_random_coords(np.random.default_rng(200 + n), n, shape), shape)


def test_sparse_conv_pairs_geometries():
    """Strides, paddings, dilations and kernel shapes other than 3x3x3 / 2 / 1 / 1, also a stride
    that shares a factor with the dilation and a stride-1 convolution (every offset reaches)."""
    rng = np.random.default_rng(7)
    shape = (10, 21, 18)
    coords = _random_coords(rng, 2500, shape)
    for ksize, stride, padding, dilation in [
            ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
            ((3, 3, 3), (2, 2, 2), (0, 0, 0), (1, 1, 1)),
            ((2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)),
            ((3, 3, 3), (2, 2, 2), (2, 2, 2), (2, 2, 2)),
            ((1, 3, 3), (1, 2, 3), (0, 1, 2), (1, 1, 2)),
            ((3, 2, 4), (3, 1, 2), (1, 0, 1), (1, 2, 1))]:
        print("case sparse conv geometry", ksize, stride, padding, dilation, flush=True)
        _check_conv_case(coords, shape, ksize, stride, padding, dilation)


def test_sparse_conv_pairs_dense_block():
    """Every voxel of a block: every output site has all of its in-range inputs."""
    g = np.stack(np.meshgrid(np.arange(8), np.arange(9), np.arange(10), indexing="ij"), -1).reshape(-1, 3)
    coords = np.zeros((g.shape[0], 4), np.int32)
    coords[:, 1:] = g
    coords = coords[np.random.default_rng(5).permutation(coords.shape[0])]
    _check_conv_case(coords, (8, 9, 10))


def test_sparse_conv_pairs_huge_grid_hash_path():
    """An output grid of 2 x 2048^3 = 2^34 sites is beyond the bitmap: hash set and sort.  Clusters
    of neighbours so that output sites are shared; also a 3-batch case with a kernel that every
    input reaches 27 times."""
    print("case sparse conv pairs hash path", flush=True)
    rng = np.random.default_rng(11)
    shape = (4096, 4096, 4096)
    centres = rng.integers(8, 4088, size=(400, 3))
    pts = (centres[:, None, :] + rng.integers(-3, 4, size=(400, 40, 3))).reshape(-1, 3)
    b = rng.integers(0, 2, size=(pts.shape[0], 1))
    coords = np.unique(np.concatenate([b, pts], axis=1), axis=0).astype(np.int32)
    coords = coords[rng.permutation(coords.shape[0])]
    _check_conv_case(coords, shape)
    _check_conv_case(coords, shape, stride=(1, 1, 1), batch_size=3)


def test_sparse_conv_pairs_full_size():
    """The stride-2 benchmark geometry (300 k voxels in 41 x 1600 x 1408, about 650 k outputs)."""
    print("case sparse conv pairs full size", flush=True)
    rng = np.random.default_rng(20240607 + 1)
    grid = (41, 1600, 1408)
    coords = synth.clustered_voxels(rng, 300000, grid, 60, sigma=15.0, noise_frac=0.10)
    ref, got = _check_conv_case(coords, grid, batch_size=1)
    assert ref.out_coords.shape[0] > coords.shape[0]


def test_sparse_conv_pairs_empty_and_errors():
    got = pairs.sparse_conv_pairs_device(tv.zeros([0, 4], tv.int32, 0), (8, 8, 8))
    assert got.out_coords.shape[0] == 0 and tuple(got.out_shape) == (4, 4, 4)
    c = tv.zeros([8, 4], tv.int32, 0)
    with pytest.raises(ValueError):
        pairs.sparse_conv_pairs_device(c, (8, 8, 8), ksize=(5, 5, 7))        # kernel volume 175 > 128
    with pytest.raises(ValueError):
        pairs.sparse_conv_pairs_device(c, (2, 2, 2), ksize=(3, 3, 3), padding=(0, 0, 0))   # no output
    with pytest.raises(RuntimeError):
        pairs.sparse_conv_pairs_device(c, (4, 4, 4), workspace=tv.zeros([256], tv.uint8, 0))   # too small


@pytest.mark.parametrize("n", [1, 63, 4096, 4097, 50000, 300001])
@pytest.mark.parametrize("kind", ["random27", "few", "all_equal", "random32", "sorted", "reverse"])
def test_sort_by_mask_against_stable_argsort(n, kind):
    """The hand-written radix sort against numpy's stable argsort: random 27- and 32-bit keys, a
    handful of distinct keys (long runs of ties across chunk borders), one key only, keys already
    in order and in reverse; with a filter that drops bits; outputs and workspace reused."""
    print("case sort", n, kind, flush=True)
    rng = np.random.default_rng(n + len(kind))
    if kind == "random27":
        mask = rng.integers(0, 1 << 27, size=n, dtype=np.uint32)
    elif kind == "random32":
        mask = rng.integers(0, 1 << 32, size=n, dtype=np.uint64).astype(np.uint32)
    elif kind == "few":
        mask = rng.choice(np.array([0x2000, 0x6000, 0x7FFFFFF, 0x2001, 0x4002000], np.uint32), size=n)
    elif kind == "all_equal":
        mask = np.full(n, 0x2000, np.uint32)
    elif kind == "sorted":
        mask = np.sort(rng.integers(0, 1 << 27, size=n, dtype=np.uint32))
    else:
        mask = np.sort(rng.integers(0, 1 << 27, size=n, dtype=np.uint32))[::-1].copy()
    d_mask = H.dev(mask, "u32")
    lib = _capi.lib()
    ws = tv.empty([int(lib.cumm_hip_sort_by_mask_workspace(n))], tv.uint8, 0)
    out = (tv.empty([n], tv.uint32, 0), tv.empty([n], tv.int32, 0))
    for filt in (0xFFFFFFFF, 0x07FFFFFF, 0x3FFF, 0x1FFF << 14, 0x1):
        ms_ref, order_ref = pairs.sort_by_mask(mask, filt)
        ms, order = pairs.sort_by_mask_device(d_mask, filt, workspace=ws, out=out)
        np.testing.assert_array_equal(H.host(ms), ms_ref)
        np.testing.assert_array_equal(H.host(order), order_ref)
    from cumm_amd.gemm.main import GemmMainUnitTest
    GemmMainUnitTest.device_synchronize()      # (would raise if a look-back had given up)


@pytest.mark.parametrize("n", [1, 127, 128, 1000, 4096, 50001])
def test_light_prefix_against_the_host_count(n):
    """cumm_hip_light_prefix against pairs.light_prefix: sorted arrays whose light end has a random
    length (centre-only words, a few with one more offset), followed by words of many offsets;
    with filters that turn heavy words light."""
    print("case light prefix", n, flush=True)
    rng = np.random.default_rng(n)
    for light_len in (0, n // 3, n - n // 7, n):
        light = np.full(light_len, 1 << 13, np.uint32)
        light[rng.random(light_len) < 0.05] |= np.uint32(1 << 14)
        heavy = (rng.integers(1, 1 << 13, size=n - light_len, dtype=np.uint32) | np.uint32(1 << 13) | np.uint32(7 << 20))
        mask = np.sort(np.concatenate([light, heavy]))
        d = H.dev(mask, "u32")
        for filt in (0xFFFFFFFF, 0x6000, 1 << 13, 0x1FFF):
            assert pairs.light_prefix_device(d, mask_filter=filt) == pairs.light_prefix(mask, filt), (light_len, hex(filt))


def test_sort_leaves_the_light_prefix_for_the_launch():
    """The GPU sort counts the light prefix of its result and leaves it in the library's
    device-side table under the result's address, where a forward launch with no hint of its own
    looks: the table holds what the host count says, per filter; an array nobody prepared has no
    entry; cumm_hip_light_prefix registers an array that another sort made; and the launch gives
    the same bits whether it is told the count, finds it, or is told to use none."""
    from cumm_amd.conv.main import ConvMainUnitTest
    from cumm_amd.tensorview.gemm import ConvOpType, ConvParams
    print("case light hint table", flush=True)
    rng = np.random.default_rng(77)
    grid = (16, 200, 200)
    coords = synth.clustered_voxels(rng, 9000, grid, 8, sigma=4.0, noise_frac=0.6)
    pt = pairs.subm_pairs(coords, grid)
    n = coords.shape[0]
    d_mask = H.dev(pt.mask_fwd, "u32")
    for filt in (0xFFFFFFFF, 0x07FFFFFF, 0x3FFF):
        ms_ref, order_ref = pairs.sort_by_mask(pt.mask_fwd, filt)
        ms, order = pairs.sort_by_mask_device(d_mask, filt)
        np.testing.assert_array_equal(H.host(ms), ms_ref)
        assert pairs.light_hint_device(ms, filt) == pairs.light_prefix(ms_ref, filt)
        assert pairs.light_hint_device(ms, filt ^ 0x10) == -1          # another filter: no entry
    ms_ref, order_ref = pairs.sort_by_mask(pt.mask_fwd)
    exact = pairs.light_prefix(ms_ref)
    assert 256 <= exact <= n - 256
    foreign = H.dev(ms_ref, "u32")                  # sorted elsewhere: nothing known about it
    # (the slot of this address may hold an older array's entry, never this one's)
    assert pairs.light_hint_device(foreign) in (-1, exact)
    assert pairs.light_prefix_device(foreign) == exact
    assert pairs.light_hint_device(foreign) == exact
    ms, order = pairs.sort_by_mask_device(d_mask)
    feat = H.to_storage(rng.normal(0, 1, size=(n, 64)).astype(np.float32), "f16")
    w = H.to_storage(rng.normal(0, 0.05, size=(64, 27, 64)).astype(np.float32), "f16")
    outs = []
    for hint in (-1, 0, exact):
        p = ConvParams(3, ConvOpType.Forward)
        p.conv_algo_desp = H.find_conv_desp("f16", ConvOpType.Forward, 64, 64)
        p.input, p.weight, p.output = H.dev(feat, "f16"), H.dev(w, "f16"), tv.zeros([n, 64], tv.float16, 0)
        p.indices, p.mask, p.mask_argsort = H.dev(pt.indices_fwd, "i32"), ms, order
        p.mask_output = tv.zeros([(n + 63) // 64], tv.uint32, 0)
        p.light_prefix = hint
        ConvMainUnitTest.implicit_gemm2(p)
        outs.append((H.host(p.output), H.host(p.mask_output)))
    from oracle import conv_ref
    ref, ref_mo = conv_ref.implicit_gemm_fwd_ref(feat, w, np.zeros((n, 64), np.float16), pt.indices_fwd, ms_ref, order_ref,
                                                 tile_m=64, dtype_in="f16", dtype_w="f16", dtype_out="f16")
    assert H.rel_err(H.as_f32(outs[0][0], "f16"), H.as_f32(ref, "f16")) < 1e-2
    for got, mo in outs:
        np.testing.assert_array_equal(got.view(np.uint16), outs[0][0].view(np.uint16))
        np.testing.assert_array_equal(mo, ref_mo)


@pytest.mark.parametrize("n", [1, 127, 4097, 50000, 300001])
@pytest.mark.parametrize("kind", ["cloud", "random27", "few", "all_equal"])
def test_sort_by_offset_count_against_the_host(n, kind):
    """cumm_hip_sort_by_mask_ordered, order 1 (ascending number of kernel offsets, then value)
    against the host's stable argsort of the same key, and what the sort leaves in the hint table
    for its result - the light prefix (counted with three offsets for this order) and the start
    of the heavy end - against the host counts; a filter of more than 27 bits is refused."""
    print("case sort by count", n, kind, flush=True)
    rng = np.random.default_rng(n + len(kind))
    if kind == "cloud":
        # masks as a sparse cloud has them: most positions the centre alone, some with a few neighbours
        mask = np.full(n, 1 << 13, np.uint32)
        extra = rng.random(n)
        for frac, bits in ((0.35, 1), (0.12, 2), (0.04, 4), (0.01, 7)):
            sel = extra < frac
            for _ in range(bits):
                mask[sel] |= (np.uint32(1) << rng.integers(0, 27, size=int(sel.sum())).astype(np.uint32))
    elif kind == "random27":
        mask = rng.integers(0, 1 << 27, size=n, dtype=np.uint32)
    elif kind == "few":
        mask = rng.choice(np.array([0x2000, 0x6000, 0x7FFFFFF, 0x2001, 0x4002000], np.uint32), size=n)
    else:
        mask = np.full(n, 0x2000, np.uint32)
    d_mask = H.dev(mask, "u32")
    for filt in (0x07FFFFFF, 0x3FFF, 0x1FFF << 14):
        ms_ref, order_ref = pairs.sort_by_mask(mask, filt, by_offset_count=True)
        ms, order = pairs.sort_by_mask_device(d_mask, filt, by_offset_count=True)
        np.testing.assert_array_equal(H.host(ms), ms_ref)
        np.testing.assert_array_equal(H.host(order), order_ref)
        assert pairs.hints_device(ms, filt) == (pairs.light_prefix(ms_ref, light_offsets=3), pairs.heavy_from(ms_ref))
        ms_v, _ = pairs.sort_by_mask_device(d_mask, filt)
        ms_vref, _ = pairs.sort_by_mask(mask, filt)
        assert pairs.hints_device(ms_v, filt) == (pairs.light_prefix(ms_vref), pairs.heavy_from(ms_vref))
    with pytest.raises(ValueError):
        pairs.sort_by_mask_device(d_mask, 0xFFFFFFFF, by_offset_count=True)
    from cumm_amd.gemm.main import GemmMainUnitTest
    GemmMainUnitTest.device_synchronize()
