"""Random geometries through the GPU input preparation, against the host builders: bit-exact.

Submanifold tables (kernel sizes 1, 3, 5 per axis, dilation) and strided tables (kernel sizes 1 to
5, strides 1 to 3, padding 0 to 2, dilation, several batches) of clouds from one voxel to a few
thousand; on each: the masks of any width made from the table, their sort, the table in the order
of the sorted positions, the per-offset pair lists, and for kernel volumes up to 32 the mask sort in
both orders with the hints it leaves in the device table.  Each case prints its parameters first.
"""
import json

import numpy as np
import pytest

import helpers as H
from cumm_amd import pairs, synth

pytestmark = pytest.mark.gpu


def one_case(seed):
    rng = np.random.default_rng(seed)
    batch = int(rng.choice([1, 1, 2, 3]))
    grid = (int(rng.integers(3, 20)), int(rng.integers(4, 50)), int(rng.integers(4, 50)))
    n = int(rng.choice([1, 5, 64, 200, 1500, 6000]))
    parts = []
    for b in range(batch):
        c = synth.clustered_voxels(rng, max(1, n // batch), grid, int(rng.integers(1, 5)), sigma=float(rng.uniform(1.0, 5.0)), batch=b)
        parts.append(c)
    coords = np.concatenate(parts).astype(np.int32)
    strided = bool(rng.integers(0, 2))
    dil = tuple(int(x) for x in rng.choice([1, 1, 2], size=3))
    desc = dict(seed=seed, batch=batch, grid=grid, n=int(coords.shape[0]), strided=strided, dil=dil)
    if strided:
        ksize = tuple(int(x) for x in rng.choice([1, 2, 3, 4, 5], size=3))
        while ksize[0] * ksize[1] * ksize[2] > 128:
            ksize = tuple(int(x) for x in rng.choice([1, 2, 3], size=3))
        stride = tuple(int(x) for x in rng.choice([1, 2, 3], size=3))
        padding = tuple(int(x) for x in rng.choice([0, 1, 2], size=3))
        desc.update(ksize=ksize, stride=stride, padding=padding)
        print("case", json.dumps(desc), flush=True)
        try:
            host = pairs.sparse_conv_pairs(coords, grid, ksize, stride, padding, dil)
        except Exception as e:
            return True, "host refused: %r" % (e,), desc
        if min(host.out_shape) <= 0:
            return True, "empty output grid", desc
        # host builder ignores batch in out_shape linearisation? it linearises (batch, z, y, x) through coords[:, 0]
        dev = pairs.sparse_conv_pairs_device(H.dev(coords, "i32"), grid, ksize, stride, padding, dil, batch_size=batch)
        ok = (tuple(dev.out_shape) == tuple(host.out_shape) and np.array_equal(H.host(dev.out_coords), host.out_coords)
              and np.array_equal(H.host(dev.indices_fwd), host.indices_fwd) and np.array_equal(H.host(dev.indices_bwd), host.indices_bwd))
        kv = ksize[0] * ksize[1] * ksize[2]
        if ok and kv <= 32:
            ok = np.array_equal(H.host(dev.mask_fwd), host.mask_fwd) and np.array_equal(H.host(dev.mask_bwd), host.mask_bwd)
        ind_d, mask_h = dev.indices_fwd, host.mask_fwd
    else:
        ksize = tuple(int(x) for x in rng.choice([1, 3, 5], size=3))
        desc.update(ksize=ksize)
        print("case", json.dumps(desc), flush=True)
        host = pairs.subm_pairs(coords, grid, ksize, dil)
        dev = pairs.subm_pairs_device(H.dev(coords, "i32"), grid, ksize, dil)
        ok = np.array_equal(H.host(dev.indices_fwd), host.indices_fwd) and np.array_equal(H.host(dev.indices_bwd), host.indices_bwd)
        kv = ksize[0] * ksize[1] * ksize[2]
        if ok and kv <= 32:
            ok = np.array_equal(H.host(dev.mask_fwd), host.mask_fwd) and np.array_equal(H.host(dev.mask_bwd), host.mask_bwd)
        ind_d, mask_h = dev.indices_fwd, host.mask_fwd
    if not ok:
        return False, "tables differ", desc
    n_out = host.indices_fwd.shape[1]
    if n_out == 0:
        return True, "", desc
    # masks of any width, their sorts, the table by position, the per-offset lists
    mw_h = pairs.masks_from_pairs(host.indices_fwd)
    mw_d = pairs.masks_from_pairs_device(ind_d)
    if not np.array_equal(H.host(mw_d), mw_h):
        return False, "masks_from_pairs", desc
    sm_h, so_h = pairs.sort_by_mask_words(mw_h)
    sm_d, so_d = pairs.sort_by_mask_words_device(mw_d)
    if not (np.array_equal(H.host(sm_d), sm_h) and np.array_equal(H.host(so_d), so_h)):
        return False, "sort_by_mask_words", desc
    if not np.array_equal(H.host(pairs.pairs_by_position_device(ind_d, so_d)), pairs.pairs_by_position(host.indices_fwd, so_h)):
        return False, "pairs_by_position", desc
    l_h, l_d = pairs.pair_lists(host.indices_fwd), pairs.pair_lists_device(ind_d)
    if not np.array_equal(np.asarray(l_d.counts), l_h.counts):
        return False, "pair list counts", desc
    pi, po = H.host(l_d.pair_in), H.host(l_d.pair_out)
    for k in range(kv):
        c = int(l_h.counts[k])
        if not (np.array_equal(pi[k, :c], l_h.pair_in[k, :c]) and np.array_equal(po[k, :c], l_h.pair_out[k, :c])):
            return False, "pair lists offset %d" % k, desc
    if kv <= 32:
        for by_count in (False, True):
            if by_count and kv > 27:
                continue
            filt = int(rng.choice([0xFFFFFFFF, (1 << kv) - 1, 0x5555555])) & (0x7FFFFFF if by_count else 0xFFFFFFFF)
            m_h, o_h = pairs.sort_by_mask(mask_h, filt, by_offset_count=by_count)
            m_d, o_d = pairs.sort_by_mask_device(H.dev(mask_h, "u32"), filt, by_offset_count=by_count)
            if not (np.array_equal(H.host(m_d), m_h) and np.array_equal(H.host(o_d), o_h)):
                return False, "sort_by_mask count=%s filt=%x" % (by_count, filt), desc
            lp = pairs.hints_device(m_d, filt)
            want = (pairs.light_prefix(m_h, filt, light_offsets=3 if by_count else 2), pairs.heavy_from(m_h, filt))
            if tuple(lp) != tuple(want):
                return False, "hints %s != %s" % (lp, want), desc
    return True, "", desc


@pytest.mark.parametrize("block", range(4))
def test_random_geometries_against_the_host_builders(block):
    bad = []
    for it in range(60):
        ok, err, desc = one_case(8000000 + block * 1000 + it)
        if not ok:
            bad.append((desc, err))
    assert not bad, bad
