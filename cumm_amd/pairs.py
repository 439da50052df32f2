"""Host-side pair-table builder for mask-based sparse convolution.

The reference does not build pair tables itself: its callers get them from
spconv (``SpconvOps.generate_subm_conv_inds`` / ``generate_conv_inds_mask_stage1/2``
/ ``sort_1d_by_key``; call sites cumm/conv/main_real_spconv.py:91-145).  This
module is the host (numpy) stand-in that prepares operator inputs: sorted-key
lookups, O(kv * N log N).

Conventions of this build (spconv's own are not part of the reference tree):
kernel offset index k = (kz*KY + ky)*KX + kx; cross-correlation, i.e. output o
gathers the input at ``coord[o]*stride - padding + k_zyx*dilation``; rows of a
strided convolution's output are ordered by ascending (batch, z, y, x); the
mask sort is a stable ascending argsort.
"""
from typing import NamedTuple, Sequence, Tuple

import numpy as np


class PairTable(NamedTuple):
    indices_fwd: np.ndarray   # [kv, N_out] int32: output row -> input row, -1 = none
    indices_bwd: np.ndarray   # [kv, N_in]  int32: input row -> output row, -1 = none
    mask_fwd: np.ndarray      # [N_out] uint32, bit k set iff indices_fwd[k][o] >= 0 (None if kv > 32)
    mask_bwd: np.ndarray      # [N_in]  uint32, bit k set iff indices_bwd[k][i] >= 0 (None if kv > 32)
    out_coords: np.ndarray    # [N_out, 4] int32 (batch, z, y, x)
    out_shape: Tuple[int, int, int]


def _linear(coords: np.ndarray, shape: Sequence[int]) -> np.ndarray:
    c = coords.astype(np.int64)
    return ((c[:, 0] * shape[0] + c[:, 1]) * shape[1] + c[:, 2]) * shape[2] + c[:, 3]


def _offsets(ksize: Sequence[int]) -> np.ndarray:
    kz, ky, kx = np.meshgrid(np.arange(ksize[0]), np.arange(ksize[1]), np.arange(ksize[2]),
                             indexing="ij")
    return np.stack([kz.ravel(), ky.ravel(), kx.ravel()], axis=1).astype(np.int64)


def _masks(indices: np.ndarray):
    """One bit per kernel offset; kernel volumes above 32 have no 32-bit masks (None): their
    tables feed the per-offset convolution (:func:`pair_lists`), not the mask-based kernels."""
    kv = indices.shape[0]
    if kv > 32:
        return None
    bits = (np.uint32(1) << np.arange(kv, dtype=np.uint32))[:, None]
    return np.bitwise_or.reduce(np.where(indices >= 0, bits, np.uint32(0)), axis=0).astype(np.uint32)


def _lookup(sorted_keys, order, query_keys, valid):
    pos = np.searchsorted(sorted_keys, query_keys)
    pos = np.minimum(pos, len(sorted_keys) - 1)
    hit = valid & (sorted_keys[pos] == query_keys)
    return np.where(hit, order[pos], -1).astype(np.int32)


def calc_output_dims(in_shape, ksize, padding, stride, dilation):
    """cumm/conv/params.py:268-292 of the reference (ConvProblem.calc_output_dims)."""
    return tuple((int(i) + 2 * int(p) - int(d) * (int(k) - 1) - 1) // int(s) + 1
                 for i, k, p, s, d in zip(in_shape, ksize, padding, stride, dilation))


def _check_odd_ksize(ksize):
    if any(int(k) < 1 or int(k) % 2 == 0 for k in ksize):
        raise ValueError("submanifold convolution needs odd kernel sizes, got %s" % (list(ksize),))


def subm_pairs(coords: np.ndarray, spatial_shape: Sequence[int], ksize=(3, 3, 3),
               dilation=(1, 1, 1)) -> PairTable:
    """Submanifold convolution: outputs sit on the input sites.  Kernel sizes must be odd: only
    then is offset kv-1-k the negative of offset k, which the backward table (the forward one
    reversed) and the bit-reversed backward masks rely on."""
    _check_odd_ksize(ksize)
    coords = np.ascontiguousarray(coords, dtype=np.int32)
    n = coords.shape[0]
    offs = _offsets(ksize)
    kv = offs.shape[0]
    center = np.array([k // 2 for k in ksize], dtype=np.int64)
    keys = _linear(coords, spatial_shape)
    order = np.argsort(keys, kind="stable")
    skeys = keys[order]
    assert n == 0 or np.all(skeys[1:] != skeys[:-1]), "duplicate voxel coordinates"
    ind = np.full((kv, n), -1, dtype=np.int32)
    sp = np.asarray(spatial_shape, dtype=np.int64)
    c64 = coords.astype(np.int64)
    for k in range(kv):
        q = c64.copy()
        q[:, 1:] += (offs[k] - center) * np.asarray(dilation, dtype=np.int64)
        valid = np.all((q[:, 1:] >= 0) & (q[:, 1:] < sp), axis=1)
        if n:
            ind[k] = _lookup(skeys, order, _linear(np.where(valid[:, None], q, 0), spatial_shape), valid)
    ind_b = ind[::-1].copy()  # input i feeds output o through offset k iff o sees i through kv-1-k
    return PairTable(ind, ind_b, _masks(ind), _masks(ind_b), coords, tuple(int(s) for s in spatial_shape))


def sparse_conv_pairs(coords: np.ndarray, spatial_shape: Sequence[int], ksize=(3, 3, 3),
                      stride=(2, 2, 2), padding=(1, 1, 1), dilation=(1, 1, 1)) -> PairTable:
    """Regular (strided) sparse convolution: an output site is active iff any
    input falls in its receptive field."""
    coords = np.ascontiguousarray(coords, dtype=np.int32)
    n_in = coords.shape[0]
    offs = _offsets(ksize)
    kv = offs.shape[0]
    out_shape = calc_output_dims(spatial_shape, ksize, padding, stride, dilation)
    st = np.asarray(stride, dtype=np.int64)
    pd = np.asarray(padding, dtype=np.int64)
    dl = np.asarray(dilation, dtype=np.int64)
    osz = np.asarray(out_shape, dtype=np.int64)
    c64 = coords.astype(np.int64)
    cand_keys = []
    per_k = []
    for k in range(kv):
        num = c64[:, 1:] + pd - offs[k] * dl
        o = num // st
        valid = np.all((num % st == 0) & (o >= 0) & (o < osz), axis=1)
        oc = np.concatenate([c64[:, :1], o], axis=1)
        okey = _linear(np.where(valid[:, None], oc, 0), out_shape)
        per_k.append((valid, okey))
        cand_keys.append(okey[valid])
    all_keys = np.unique(np.concatenate(cand_keys)) if n_in else np.zeros(0, np.int64)
    n_out = all_keys.shape[0]
    out_coords = np.zeros((n_out, 4), dtype=np.int32)
    rem = all_keys.copy()
    for d, s in zip((3, 2, 1), out_shape[::-1]):
        out_coords[:, d] = rem % s
        rem //= s
    out_coords[:, 0] = rem
    ind_f = np.full((kv, n_out), -1, dtype=np.int32)
    ind_b = np.full((kv, n_in), -1, dtype=np.int32)
    for k in range(kv):
        valid, okey = per_k[k]
        rows_in = np.nonzero(valid)[0]
        rows_out = np.searchsorted(all_keys, okey[valid])
        ind_f[k, rows_out] = rows_in
        ind_b[k, rows_in] = rows_out
    return PairTable(ind_f, ind_b, _masks(ind_f), _masks(ind_b), out_coords, out_shape)


def sort_by_mask(mask: np.ndarray, mask_filter: int = 0xFFFFFFFF, by_offset_count: bool = False):
    """(sorted mask, argsort): stable ascending sort of ``mask & mask_filter``
    (spconv's sort_1d_by_key[_split]; the kernel reads the mask by sorted position
    and the pair table by real row, cumm/conv/kernel.py:853-855,
    cumm/conv/sparse_iters.py:349-352 of the reference).  ``by_offset_count``: ascending number
    of kernel offsets first, then value (filters of at most 27 bits) - an order of this build's
    own that keeps the many-offset positions in a short run at the end."""
    key = mask & np.uint32(mask_filter)
    if by_offset_count:
        if int(mask_filter) >> 27:
            raise ValueError("the order by offset count takes filters of at most 27 bits")
        count = np.zeros(key.shape, np.uint32)
        for b in range(27):
            count += (key >> np.uint32(b)) & np.uint32(1)
        order = np.argsort((count << np.uint32(27)) | key, kind="stable").astype(np.int32)
    else:
        order = np.argsort(key, kind="stable").astype(np.int32)
    return np.ascontiguousarray(key[order]), order


def light_prefix(sorted_mask: np.ndarray, mask_filter: int = 0xFFFFFFFF, light_offsets: int = 2) -> int:
    """How far the light end of a sorted mask array reaches: the number of leading positions (a
    multiple of 128) in runs of 128 whose two halves of 64 each OR to at most ``light_offsets``
    kernel offsets (two; the GPU sort counts with three for its order by offset count).
    The value of ``ConvParams.light_prefix`` (a submanifold layer's centre-only positions lead the
    ascending order); the reference has no such hint."""
    key = np.asarray(sorted_mask, np.uint32) & np.uint32(mask_filter)
    runs = key.shape[0] // 128
    if runs == 0:
        return 0
    words = np.bitwise_or.reduce(key[:runs * 128].reshape(runs * 2, 64), axis=1)
    bits = np.zeros(runs * 2, np.int64)
    for b in range(32):
        bits += (words >> np.uint32(b)) & np.uint32(1)
    heavy = np.nonzero(bits.reshape(runs, 2).max(axis=1) > light_offsets)[0]
    return int(heavy[0] if heavy.size else runs) * 128


def heavy_from(sorted_mask: np.ndarray, mask_filter: int = 0xFFFFFFFF, heavy_offsets: int = 10) -> int:
    """Where the heavy end of a sorted mask array begins: the first position of the first tile of 64
    positions whose masks OR to ``heavy_offsets`` or more kernel offsets; the length rounded up
    to 64 when there is none.  What the GPU sort leaves next to the light prefix."""
    key = np.asarray(sorted_mask, np.uint32) & np.uint32(mask_filter)
    n = key.shape[0]
    tiles = (n + 63) // 64
    pad = np.zeros(tiles * 64, np.uint32)
    pad[:n] = key
    words = np.bitwise_or.reduce(pad.reshape(tiles, 64), axis=1)
    bits = np.zeros(tiles, np.int64)
    for b in range(32):
        bits += (words >> np.uint32(b)) & np.uint32(1)
    heavy = np.nonzero(bits >= heavy_offsets)[0]
    return int(heavy[0] if heavy.size else tiles) * 64


def masks_from_pairs(indices: np.ndarray) -> np.ndarray:
    """Masks of a pair table [kv, N] of any kernel volume: [N, ceil(kv / 32)] uint32, bit b of word w
    set wherever ``indices[32 w + b][o] >= 0`` - the layout the reference's dynamic-mask kernels read
    (``mask_ptr[mask_int_count * pos + word]``, cumm/gemm/blockmma/mma.py:176-190)."""
    kv, n = indices.shape
    words = (kv + 31) // 32
    out = np.zeros((n, words), np.uint32)
    for k in range(kv):
        out[:, k // 32] |= np.where(indices[k] >= 0, np.uint32(1 << (k % 32)), np.uint32(0)).astype(np.uint32)
    return out


def mask_words_keys(mask: np.ndarray) -> np.ndarray:
    """Sort key of positions with several mask words [N, words]: the number of offsets (at most
    63) in the upper six bits, a 26-bit hash of the words below - few offsets first, equal masks
    together."""
    mask = np.asarray(mask, np.uint32)
    pc = np.zeros(mask.shape[0], np.uint32)
    h = np.zeros(mask.shape[0], np.uint32)
    for i in range(mask.shape[1]):
        w = mask[:, i]
        for b in range(32):
            pc += (w >> np.uint32(b)) & np.uint32(1)
        r = (7 * i) & 31
        h ^= ((w << np.uint32(r)) | (w >> np.uint32(32 - r))).astype(np.uint32) if r else w
    h = ((h.astype(np.uint64) * np.uint64(0x9E3779B1)) & np.uint64(0xFFFFFFFF)).astype(np.uint32) >> np.uint32(6)
    return ((np.minimum(pc, 63).astype(np.uint32) << np.uint32(26)) | h).astype(np.uint32)


def sort_by_mask_words(mask: np.ndarray):
    """(sorted masks [N, words], argsort): stable ascending sort by :func:`mask_words_keys`."""
    order = np.argsort(mask_words_keys(mask), kind="stable").astype(np.int32)
    return np.ascontiguousarray(np.asarray(mask, np.uint32)[order]), order


def pairs_by_position(indices: np.ndarray, mask_argsort: np.ndarray) -> np.ndarray:
    """The pair table in the order of the sorted positions: ``out[k][pos] = indices[k][mask_argsort[pos]]``
    (what ``ConvParams.indices_by_position`` takes; the reference's iterator forms this index per
    access, cumm/conv/sparse_iters.py:280-357)."""
    return np.ascontiguousarray(np.asarray(indices)[:, np.asarray(mask_argsort, np.int64)])


class PairLists(NamedTuple):
    pair_in: np.ndarray    # [kv, N] int32: input rows of offset k's pairs, packed to the front
    pair_out: np.ndarray   # [kv, N] int32: their output rows (ascending)
    counts: np.ndarray     # [kv] int32: pairs per offset


def pair_lists(indices_fwd: np.ndarray) -> PairLists:
    """Per-offset (input row, output row) lists of a forward pair table, ascending output row:
    what the per-offset ("native") convolution walks (spconv's indice_pairs / indice_num_per_loc,
    rebuilt the same way in cumm/conv/main_real_spconv.py:300-326 of the reference)."""
    kv, n = indices_fwd.shape
    pin = np.full((kv, n), -1, np.int32)
    pout = np.full((kv, n), -1, np.int32)
    counts = np.zeros(kv, np.int32)
    for k in range(kv):
        o = np.nonzero(indices_fwd[k] >= 0)[0]
        counts[k] = o.size
        pin[k, :o.size] = indices_fwd[k, o]
        pout[k, :o.size] = o
    return PairLists(pin, pout, counts)


# ---- the same tables built on the GPU (cumm_hip_subm_pairs / cumm_hip_sort_by_mask) ----------

class DevicePairTable(NamedTuple):
    indices_fwd: "object"   # tv.Tensor [kv, N] int32 on the device
    indices_bwd: "object"   # tv.Tensor [kv, N] int32
    mask_fwd: "object"      # tv.Tensor [N] uint32
    mask_bwd: "object"      # tv.Tensor [N] uint32


def subm_pairs_device(coords, spatial_shape: Sequence[int], ksize=(3, 3, 3), dilation=(1, 1, 1),
                      workspace=None, stream: int = 0, out: "DevicePairTable" = None) -> DevicePairTable:
    """GPU counterpart of :func:`subm_pairs`: ``coords`` is a device ``tv.Tensor`` [N, 4] int32 of
    unique (batch, z, y, x); the tables stay on the device.  What the reference's callers take from
    ``SpconvOps.generate_subm_conv_inds`` (cumm/conv/main_real_spconv.py:91-105 of the reference).
    With ``workspace`` (``cumm_hip_subm_pairs_workspace(n)`` bytes) and ``out`` (a DevicePairTable
    of the right shapes, e.g. the previous call's result) the call allocates nothing.  Kernel
    volumes above 32 (up to 128) come without masks."""
    import ctypes as C

    from . import _capi
    from . import tensorview as tv
    if coords.device < 0 or coords.dtype != tv.int32 or coords.ndim != 2 or coords.shape[1] != 4:
        raise ValueError("coords must be a device int32 tensor of shape [N, 4]")
    _check_odd_ksize(ksize)
    n = int(coords.shape[0])
    kv = int(ksize[0]) * int(ksize[1]) * int(ksize[2])
    lib = _capi.lib()
    need = int(lib.cumm_hip_subm_pairs_workspace(n))
    if workspace is None or workspace.empty():
        workspace = tv.empty([max(need, 16)], tv.uint8, 0)
    if out is not None:     # the caller's tensors, reused from call to call: nothing is allocated
        ind_f, ind_b, mask_f, mask_b = out
        if (ind_f.shape != [kv, n] or ind_b.shape != [kv, n] or ind_f.dtype != tv.int32 or ind_b.dtype != tv.int32):
            raise ValueError("out must hold int32 tables of shape [kv, N]")
        for m in (mask_f, mask_b):
            if kv > 32:
                if m is not None:
                    raise ValueError("kernel volumes above 32 have no 32-bit masks: out must hold None for them")
            elif m is None or m.shape != [n] or m.dtype != tv.uint32 or m.device < 0:
                raise ValueError("out must hold uint32 device masks of shape [N]")
    else:
        ind_f = tv.empty([kv, n], tv.int32, 0)
        ind_b = tv.empty([kv, n], tv.int32, 0)
        mask_f = tv.empty([n], tv.uint32, 0) if kv <= 32 else None
        mask_b = tv.empty([n], tv.uint32, 0) if kv <= 32 else None
    arr3 = C.c_int32 * 3
    _capi.check(lib.cumm_hip_subm_pairs(
        coords.byte_pointer(), n, arr3(*[int(v) for v in spatial_shape]), arr3(*[int(v) for v in ksize]),
        arr3(*[int(v) for v in dilation]), ind_f.byte_pointer(), ind_b.byte_pointer(),
        mask_f.byte_pointer() if mask_f is not None else None,
        mask_b.byte_pointer() if mask_b is not None else None, workspace.byte_pointer(), workspace.nbytes, stream))
    return DevicePairTable(ind_f, ind_b, mask_f, mask_b)


class DeviceConvPairTable(NamedTuple):
    indices_fwd: "object"   # tv.Tensor [kv, N_out] int32 on the device
    indices_bwd: "object"   # tv.Tensor [kv, N_in] int32
    mask_fwd: "object"      # tv.Tensor [N_out] uint32
    mask_bwd: "object"      # tv.Tensor [N_in] uint32
    out_coords: "object"    # tv.Tensor [N_out, 4] int32
    out_shape: Tuple[int, ...]


def sparse_conv_pairs_device(coords, spatial_shape: Sequence[int], ksize=(3, 3, 3), stride=(2, 2, 2),
                             padding=(1, 1, 1), dilation=(1, 1, 1), batch_size: int = 1, workspace=None,
                             stream: int = 0, out=None) -> DeviceConvPairTable:
    """GPU counterpart of :func:`sparse_conv_pairs`: ``coords`` is a device ``tv.Tensor`` [N, 4]
    int32 of unique (batch, z, y, x); the tables stay on the device.  Two library calls with one
    stream synchronisation between them (the number of active output sites sizes the tables), as
    with spconv's generate_conv_inds_mask_stage1 / stage2.  Batch indices are 0 .. batch_size-1.
    ``out``: the table of an earlier call; its tensors are written again when the number of output
    sites is the same (with ``workspace`` the call then allocates nothing)."""
    import ctypes as C

    from . import _capi
    from . import tensorview as tv
    if coords.device < 0 or coords.dtype != tv.int32 or coords.ndim != 2 or coords.shape[1] != 4:
        raise ValueError("coords must be a device int32 tensor of shape [N, 4]")
    n_in = int(coords.shape[0])
    kv = int(ksize[0]) * int(ksize[1]) * int(ksize[2])
    lib = _capi.lib()
    arr3 = C.c_int32 * 3
    geo = [arr3(*[int(v) for v in a]) for a in (spatial_shape, ksize, stride, padding, dilation)]
    need = int(lib.cumm_hip_conv_pairs_workspace(n_in, int(batch_size), *geo))
    if need == 0:
        raise ValueError("bad geometry (kernel volume 1..128, non-empty output grid) or too many voxels")
    if workspace is None or workspace.empty():
        workspace = tv.empty([max(need, 256)], tv.uint8, 0)
    out_shape = arr3()
    n_out = C.c_int32(0)
    _capi.check(lib.cumm_hip_conv_pairs_sites(coords.byte_pointer(), n_in, int(batch_size), *geo, out_shape, C.byref(n_out),
                                              workspace.byte_pointer(), workspace.nbytes, stream))
    n = int(n_out.value)
    if out is not None and out.indices_fwd.shape == [kv, n] and out.indices_bwd.shape == [kv, n_in] and \
            out.out_coords.shape == [n, 4] and (out.mask_fwd is None) == (kv > 32) and (out.mask_bwd is None) == (kv > 32) and \
            (kv > 32 or (out.mask_fwd.shape == [n] and out.mask_bwd.shape == [n_in] and
                         out.mask_fwd.dtype == tv.uint32 and out.mask_bwd.dtype == tv.uint32)):
        out_coords, ind_f, ind_b, mask_f, mask_b = out.out_coords, out.indices_fwd, out.indices_bwd, out.mask_fwd, out.mask_bwd
    else:
        out_coords = tv.empty([n, 4], tv.int32, 0)
        ind_f = tv.empty([kv, n], tv.int32, 0)
        ind_b = tv.empty([kv, n_in], tv.int32, 0)
        mask_f = tv.empty([n], tv.uint32, 0) if kv <= 32 else None
        mask_b = tv.empty([n_in], tv.uint32, 0) if kv <= 32 else None
    _capi.check(lib.cumm_hip_conv_pairs_fill(
        coords.byte_pointer(), n_in, int(batch_size), *geo, n, out_coords.byte_pointer(), ind_f.byte_pointer(),
        ind_b.byte_pointer(), mask_f.byte_pointer() if mask_f is not None else None,
        mask_b.byte_pointer() if mask_b is not None else None, workspace.byte_pointer(),
        workspace.nbytes, stream))
    return DeviceConvPairTable(ind_f, ind_b, mask_f, mask_b, out_coords, tuple(int(v) for v in out_shape))


def sort_by_mask_device(mask, mask_filter: int = 0xFFFFFFFF, workspace=None, stream: int = 0, out=None,
                        by_offset_count: bool = False):
    """GPU counterpart of :func:`sort_by_mask` on a device ``tv.Tensor`` [N] uint32: returns
    (sorted mask, argsort) device tensors (spconv's sort_1d_by_key[_split], call site
    cumm/conv/main_real_spconv.py:118-145 of the reference).  With ``workspace`` and ``out`` =
    (sorted mask, argsort) tensors of a previous call the call allocates nothing.
    ``by_offset_count``: the order of :func:`sort_by_mask` with the same switch."""
    from . import _capi
    from . import tensorview as tv
    if mask.device < 0 or mask.dtype != tv.uint32 or mask.ndim != 1:
        raise ValueError("mask must be a device uint32 vector")
    n = int(mask.shape[0])
    lib = _capi.lib()
    need = int(lib.cumm_hip_sort_by_mask_workspace(n))
    if workspace is None or workspace.empty():
        workspace = tv.empty([max(need, 256)], tv.uint8, 0)
    if out is not None:
        out_mask, order = out
        if out_mask.shape != [n] or order.shape != [n] or out_mask.dtype != tv.uint32 or order.dtype != tv.int32:
            raise ValueError("out must be (uint32 [N], int32 [N]) device tensors")
    else:
        out_mask = tv.empty([n], tv.uint32, 0)
        order = tv.empty([n], tv.int32, 0)
    _capi.check(lib.cumm_hip_sort_by_mask_ordered(mask.byte_pointer(), n, int(mask_filter) & 0xFFFFFFFF,
                                                  1 if by_offset_count else 0,
                                                  out_mask.byte_pointer(), order.byte_pointer(),
                                                  workspace.byte_pointer(), workspace.nbytes, stream))
    return out_mask, order


def light_prefix_device(sorted_mask, mask_filter: int = 0xFFFFFFFF, stream: int = 0) -> int:
    """:func:`light_prefix` of a device ``tv.Tensor`` [N] uint32, counted on the GPU; the one
    number comes back to the host (the call waits for the stream)."""
    from . import _capi
    from . import tensorview as tv
    if sorted_mask.device < 0 or sorted_mask.dtype != tv.uint32 or sorted_mask.ndim != 1:
        raise ValueError("sorted_mask must be a device uint32 vector")
    lib = _capi.lib()
    res = tv.empty([1], tv.int32, 0)
    _capi.check(lib.cumm_hip_light_prefix(sorted_mask.byte_pointer(), int(sorted_mask.shape[0]),
                                          int(mask_filter) & 0xFFFFFFFF, res.byte_pointer(), stream))
    _capi.check(lib.cumm_hip_stream_synchronize(stream))
    return int(res.cpu().numpy()[0])


def light_hint_device(sorted_mask, mask_filter: int = 0xFFFFFFFF, stream: int = 0) -> int:
    """The light prefix that the library's device-side table holds for this sorted mask tensor
    (left there by :func:`sort_by_mask_device` or :func:`light_prefix_device`), -1 if none: what a
    forward / backward-input launch with ``light_prefix == 0`` on this tensor will use."""
    return hints_device(sorted_mask, mask_filter, stream)[0]


def hints_device(sorted_mask, mask_filter: int = 0xFFFFFFFF, stream: int = 0):
    """(light prefix, first position of the heavy end) as the library's device-side table holds
    them for this sorted mask tensor; (-1, -1) if it holds nothing for it."""
    import ctypes
    from . import _capi
    out, heavy = ctypes.c_int32(-1), ctypes.c_int32(-1)
    _capi.check(_capi.lib().cumm_hip_query_light_hint(sorted_mask.byte_pointer(), int(sorted_mask.shape[0]),
                                                      int(mask_filter) & 0xFFFFFFFF, ctypes.byref(out), ctypes.byref(heavy),
                                                      stream))
    return int(out.value), int(heavy.value)


def masks_from_pairs_device(indices, stream: int = 0):
    """:func:`masks_from_pairs` of a device table [kv, N]: a device tensor [N, ceil(kv / 32)] uint32."""
    from . import _capi
    from . import tensorview as tv
    if indices.device < 0 or indices.dtype != tv.int32 or indices.ndim != 2:
        raise ValueError("indices must be a device int32 tensor [kv, N]")
    kv, n = int(indices.shape[0]), int(indices.shape[1])
    out = tv.empty([n, (kv + 31) // 32], tv.uint32, 0)
    _capi.check(_capi.lib().cumm_hip_masks_from_pairs(indices.byte_pointer(), kv, n, out.byte_pointer(), stream))
    return out


def sort_by_mask_words_device(mask, workspace=None, stream: int = 0):
    """:func:`sort_by_mask_words` of a device tensor [N, words] uint32 (1 to 4 words)."""
    from . import _capi
    from . import tensorview as tv
    if mask.device < 0 or mask.dtype != tv.uint32 or mask.ndim != 2 or not 1 <= int(mask.shape[1]) <= 4:
        raise ValueError("mask must be a device uint32 tensor [N, 1..4]")
    n, words = int(mask.shape[0]), int(mask.shape[1])
    lib = _capi.lib()
    need = int(lib.cumm_hip_sort_by_mask_words_workspace(n))
    if workspace is None or workspace.empty():
        workspace = tv.empty([max(need, 256)], tv.uint8, 0)
    out_mask = tv.empty([n, words], tv.uint32, 0)
    order = tv.empty([n], tv.int32, 0)
    _capi.check(lib.cumm_hip_sort_by_mask_words(mask.byte_pointer(), n, words, out_mask.byte_pointer(), order.byte_pointer(),
                                                workspace.byte_pointer(), workspace.nbytes, stream))
    return out_mask, order


def pairs_by_position_device(indices, mask_argsort, out=None, stream: int = 0):
    """:func:`pairs_by_position` of device tensors ``indices`` [kv, N] int32 and ``mask_argsort``
    [N] int32, in stream order; ``out`` ([kv, N] int32) is filled when given."""
    from . import _capi
    from . import tensorview as tv
    if indices.device < 0 or indices.dtype != tv.int32 or indices.ndim != 2:
        raise ValueError("indices must be a device int32 tensor [kv, N]")
    kv, n = int(indices.shape[0]), int(indices.shape[1])
    if mask_argsort.device < 0 or mask_argsort.dtype != tv.int32 or list(mask_argsort.shape) != [n]:
        raise ValueError("mask_argsort must be a device int32 vector [N]")
    if out is None:
        out = tv.empty([kv, n], tv.int32, 0)
    elif out.device < 0 or out.dtype != tv.int32 or list(out.shape) != [kv, n]:
        raise ValueError("out must be a device int32 tensor [kv, N]")
    _capi.check(_capi.lib().cumm_hip_pairs_by_position(indices.byte_pointer(), mask_argsort.byte_pointer(), kv, n,
                                                       out.byte_pointer(), stream))
    return out


class DevicePairLists(NamedTuple):
    pair_in: "object"    # tv.Tensor [kv, N] int32 on the device
    pair_out: "object"   # tv.Tensor [kv, N] int32
    counts: np.ndarray   # [kv] int32 on the host (the launches of the per-offset convolution are sized by them)


def pair_lists_device(indices_fwd, workspace=None, stream: int = 0) -> DevicePairLists:
    """GPU counterpart of :func:`pair_lists` on a device table [kv, N]; the counts come back to
    the host (one stream synchronisation): the per-offset launches are sized by them."""
    from . import _capi
    from . import tensorview as tv
    if indices_fwd.device < 0 or indices_fwd.dtype != tv.int32 or indices_fwd.ndim != 2:
        raise ValueError("indices_fwd must be a device int32 tensor [kv, N]")
    kv, n = int(indices_fwd.shape[0]), int(indices_fwd.shape[1])
    lib = _capi.lib()
    need = int(lib.cumm_hip_pair_lists_workspace(kv, n))
    if workspace is None or workspace.empty():
        workspace = tv.empty([max(need, 4)], tv.uint8, 0)
    pin = tv.empty([kv, n], tv.int32, 0)
    pout = tv.empty([kv, n], tv.int32, 0)
    counts = tv.empty([kv], tv.int32, 0)
    _capi.check(lib.cumm_hip_pair_lists(indices_fwd.byte_pointer(), kv, n, pin.byte_pointer(), pout.byte_pointer(),
                                        counts.byte_pointer(), workspace.byte_pointer(), workspace.nbytes, stream))
    ctx = tv.Context()
    ctx.set_cuda_stream(stream)
    return DevicePairLists(pin, pout, counts.cpu(ctx).numpy())
