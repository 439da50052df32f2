"""Brute-force pair tables for the oracle (dictionary lookups, pure Python).

Test infrastructure only (see oracle/__init__.py).  PARITY UNPINNED against
spconv (which builds these tables for the reference's callers and is not part
of the reference tree); geometry follows the call sites
cumm/conv/main_real_spconv.py:91-105 and ConvProblem.calc_output_dims
(cumm/conv/params.py:268-292).  Use on small inputs only.
"""
import numpy as np


def calc_output_dims(in_shape, ksize, padding, stride, dilation):
    return tuple((i + 2 * p - d * (k - 1) - 1) // s + 1
                 for i, k, p, s, d in zip(in_shape, ksize, padding, stride, dilation))


def subm_pairs_ref(coords, spatial_shape, ksize=(3, 3, 3), dilation=(1, 1, 1)):
    """indices[k][i] = j  iff  coord[j] == coord[i] + (k_zyx - ksize//2) * dilation."""
    n = len(coords)
    table = {tuple(int(v) for v in c): i for i, c in enumerate(coords)}
    kv = ksize[0] * ksize[1] * ksize[2]
    ind = np.full((kv, n), -1, dtype=np.int32)
    for i, c in enumerate(coords):
        b, z, y, x = (int(v) for v in c)
        k = 0
        for kz in range(ksize[0]):
            for ky in range(ksize[1]):
                for kx in range(ksize[2]):
                    q = (b, z + (kz - ksize[0] // 2) * dilation[0],
                         y + (ky - ksize[1] // 2) * dilation[1],
                         x + (kx - ksize[2] // 2) * dilation[2])
                    ind[k, i] = table.get(q, -1)
                    k += 1
    return ind


def sparse_conv_pairs_ref(coords, spatial_shape, ksize, stride, padding, dilation):
    """Returns (indices_fwd [kv, N_out], indices_bwd [kv, N_in], out_coords).

    Output o (coordinate p) gathers input at p*stride - padding + k*dilation;
    outputs are the sites reached by at least one input, ordered by ascending
    (batch, z, y, x) -- this build's convention."""
    out_shape = calc_output_dims(spatial_shape, ksize, padding, stride, dilation)
    outs = set()
    for c in coords:
        b, z, y, x = (int(v) for v in c)
        for kz in range(ksize[0]):
            for ky in range(ksize[1]):
                for kx in range(ksize[2]):
                    num = (z + padding[0] - kz * dilation[0], y + padding[1] - ky * dilation[1],
                           x + padding[2] - kx * dilation[2])
                    if any(v % s for v, s in zip(num, stride)):
                        continue
                    o = tuple(v // s for v, s in zip(num, stride))
                    if all(0 <= v < e for v, e in zip(o, out_shape)):
                        outs.add((b,) + o)
    out_list = sorted(outs)
    in_table = {tuple(int(v) for v in c): i for i, c in enumerate(coords)}
    kv = ksize[0] * ksize[1] * ksize[2]
    ind_f = np.full((kv, len(out_list)), -1, dtype=np.int32)
    ind_b = np.full((kv, len(coords)), -1, dtype=np.int32)
    for o, p in enumerate(out_list):
        k = 0
        for kz in range(ksize[0]):
            for ky in range(ksize[1]):
                for kx in range(ksize[2]):
                    q = (p[0], p[1] * stride[0] - padding[0] + kz * dilation[0],
                         p[2] * stride[1] - padding[1] + ky * dilation[1],
                         p[3] * stride[2] - padding[2] + kx * dilation[2])
                    i = in_table.get(q, -1)
                    ind_f[k, o] = i
                    if i >= 0:
                        ind_b[k, i] = o
                    k += 1
    return ind_f, ind_b, np.array(out_list, dtype=np.int32).reshape(-1, 4)


def masks_ref(indices):
    kv, n = indices.shape
    m = np.zeros(n, dtype=np.uint32)
    for k in range(kv):
        m |= np.where(indices[k] >= 0, np.uint32(1 << k), np.uint32(0)).astype(np.uint32)
    return m
