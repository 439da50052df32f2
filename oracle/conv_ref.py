"""CPU oracle for ``ConvMainUnitTest.implicit_gemm2`` (mask-based sparse conv).

Test infrastructure only (see oracle/__init__.py).

Tensors use the reference's layouts: input [N_in, C], weight [K, kv, C],
output [N_out, K], indices [kv, N] (row of the gathered operand, -1 = none),
mask [N] u32 *in sorted order*, mask_argsort [N] (sorted position -> real row).
"""
import numpy as np

from . import numerics as nm
from .gemm_ref import _is_int, _matmul_acc, _src_f32, linear_combination


def bitrev32(x):
    x = np.asarray(x, dtype=np.uint32).copy()
    x = ((x >> 1) & 0x55555555) | ((x & 0x55555555) << 1)
    x = ((x >> 2) & 0x33333333) | ((x & 0x33333333) << 2)
    x = ((x >> 4) & 0x0F0F0F0F) | ((x & 0x0F0F0F0F) << 4)
    x = ((x >> 8) & 0x00FF00FF) | ((x & 0x00FF00FF) << 8)
    x = (x >> 16) | (x << 16)
    return x.astype(np.uint32)


def tile_masks(mask_sorted, tile_m, mask_filter=0xFFFFFFFF):
    """kmask per tile of ``tile_m`` consecutive sorted positions:
    OR of the tile's mask words, AND mask_filter
    (cumm/conv/kernel.py:844-864 of the reference).

    ``mask_sorted`` [N, words] (the dynamic-mask layout for kernel volumes above 32: word w of
    a position holds offsets 32 w .. 32 w + 31) gives [tiles, words]: every word is reduced and
    filtered by itself (``load_mask``, cumm/gemm/blockmma/mma.py:176-204 of the reference)."""
    if mask_sorted.ndim == 2:
        return np.stack([tile_masks(np.ascontiguousarray(mask_sorted[:, w]), tile_m, mask_filter)
                         for w in range(mask_sorted.shape[1])], axis=1)
    n = mask_sorted.shape[0]
    nt = (n + tile_m - 1) // tile_m
    padded = np.zeros(nt * tile_m, dtype=np.uint32)
    padded[:n] = mask_sorted
    red = np.bitwise_or.reduce(padded.reshape(nt, tile_m), axis=1)
    return (red & np.uint32(mask_filter)).astype(np.uint32)


def _tile_has_offset(kmask_tiles, k):
    """Per tile: does the (possibly several-word) tile mask name kernel offset k?"""
    if kmask_tiles.ndim == 2:
        return ((kmask_tiles[:, k // 32] >> np.uint32(k % 32)) & 1).astype(bool)
    return ((kmask_tiles >> np.uint32(k)) & 1).astype(bool)


def reverse_mask_words(words, kv):
    """The kv-bit string held in 32-bit words (bit j of the string = bit j % 32 of word j // 32)
    reversed end for end: what the reference's loader walks with ``reverse``
    (cumm/gemm/blockmma/mma.py:141-147, 196-215: words from the last to the first, each
    bit-reversed, starting ``words * 32 - kv`` bits in).  Written bit by bit on purpose."""
    words = np.asarray(words, dtype=np.uint32)
    out = np.zeros_like(words)
    for j in range(kv):
        src = kv - 1 - j
        bit = (words[..., src // 32] >> np.uint32(src % 32)) & np.uint32(1)
        out[..., j // 32] |= (bit << np.uint32(j % 32)).astype(np.uint32)
    return out


def _epilogue(acc, src, alpha, beta, act, act_alpha, act_beta, dtype_out):
    return linear_combination(acc, src, alpha, beta, act, act_alpha, act_beta, dtype_out)


def implicit_gemm_fwd_ref(inp, weight, output, indices, mask_sorted, mask_argsort, *, tile_m,
                          dtype_in, dtype_w, dtype_out, mask_filter=0xFFFFFFFF, alpha=1.0,
                          beta=0.0, bias=None, act=nm.ACT_NONE, act_alpha=0.0, act_beta=0.0,
                          scale=None, output_add=None, int8_inference=False,
                          return_acc=False):
    """Forward.  Returns (output_after, mask_output).

    cumm/conv/kernel.py:844-921 (tile mask, mask_output, the mma call is
    skipped for an all-zero tile mask but the epilogue still runs),
    cumm/gemm/blockmma/mma.py:445-578 (loop over the set bits of the tile
    mask), cumm/conv/sparse_iters.py:871-944, 1138-1175 (row o = mask_argsort[pos]
    gathers input row indices[k][o]; a negative index contributes zeros),
    check pattern cumm/conv/main_real_spconv.py:309-326 of the reference.
    Source operand: bias (stride 0) when given, else the output itself
    (cumm/conv/nvrtc_code.py:78-92).
    """
    n = indices.shape[1]
    kv = indices.shape[0]
    k_out = weight.shape[0]
    assert weight.shape[1] == kv and mask_sorted.shape[0] >= n and mask_argsort.shape[0] >= n
    kmask_tiles = tile_masks(mask_sorted[:n], tile_m, mask_filter)
    tile_of_pos = np.arange(n) // tile_m
    rows = mask_argsort[:n].astype(np.int64)
    acc_dtype = np.int32 if _is_int(dtype_in) else np.float32
    acc = np.zeros((n, k_out), dtype=np.float64 if _is_int(dtype_in) else np.float32)
    for k in range(kv):
        active = _tile_has_offset(kmask_tiles, k)[tile_of_pos]
        o = rows[active]
        i = indices[k][o]
        valid = i >= 0
        o, i = o[valid], i[valid]
        if o.size == 0:
            continue
        wk = weight[:, k, :]
        if _is_int(dtype_in):
            contrib = inp[i].astype(np.float64) @ wk.astype(np.float64).T
        else:
            contrib = nm.to_f32(inp[i], dtype_in) @ nm.to_f32(wk, dtype_w).T
        # each output row appears once per k, so a plain indexed add is exact
        acc[o] += contrib
    if _is_int(dtype_in):
        assert np.all(np.abs(acc) < 2 ** 31)
    acc = acc.astype(acc_dtype)
    out = np.array(output, copy=True)
    touched = rows  # every position of every tile runs the epilogue in forward
    if int8_inference:
        src = None
        if output_add is not None:
            src = output_add[touched]
        res = nm.int8_epilogue(acc[touched], scale, bias, src, beta, act, act_alpha)
    else:
        if bias is not None:
            src = _src_f32(bias, dtype_out)[None, :]
        else:
            src = _src_f32(out[touched], dtype_out)
        res = _epilogue(acc[touched], src, alpha, beta, act, act_alpha, act_beta, dtype_out)
    out[touched] = res
    if return_acc:
        return out, kmask_tiles, acc
    return out, kmask_tiles


def implicit_gemm_dgrad_ref(dout, weight, dinp, indices_bwd, mask_sorted, mask_argsort, *,
                            tile_m, dtype_in, dtype_w, dtype_out, mask_filter=0xFFFFFFFF,
                            reverse_mask=False, alpha=1.0, beta=0.0, act=nm.ACT_NONE,
                            act_alpha=0.0, act_beta=0.0):
    """BackwardInput.  Returns dinp_after.

    As forward with A = dOut [N,K], the weight viewed as (k,K)->C and the
    backward pair table; a tile whose mask is zero returns before the
    epilogue (its rows are NOT written); with reverse_mask the tile mask is
    bit-reversed over kv bits (cumm/conv/kernel.py:875-889), check pattern
    cumm/conv/main_real_spconv.py:347-365 of the reference.
    """
    n = indices_bwd.shape[1]
    kv = indices_bwd.shape[0]
    c_in = weight.shape[2]
    kmask_tiles = tile_masks(mask_sorted[:n], tile_m, mask_filter)
    live_tile = kmask_tiles != 0 if kmask_tiles.ndim == 1 else np.any(kmask_tiles != 0, axis=1)
    if reverse_mask:
        if kmask_tiles.ndim == 2:
            kmask_tiles = reverse_mask_words(kmask_tiles, kv)
        else:
            kmask_tiles = (bitrev32(kmask_tiles) >> np.uint32(32 - kv)).astype(np.uint32)
    tile_of_pos = np.arange(n) // tile_m
    rows = mask_argsort[:n].astype(np.int64)
    acc = np.zeros((n, c_in), dtype=np.float32)
    for k in range(kv):
        active = _tile_has_offset(kmask_tiles, k)[tile_of_pos]
        o = rows[active]
        i = indices_bwd[k][o]
        valid = i >= 0
        o, i = o[valid], i[valid]
        if o.size == 0:
            continue
        acc[o] += nm.to_f32(dout[i], dtype_in) @ nm.to_f32(weight[:, k, :], dtype_w)
    out = np.array(dinp, copy=True)
    touched = rows[live_tile[tile_of_pos]]
    src = _src_f32(out[touched], dtype_out)
    out[touched] = _epilogue(acc[touched], src, alpha, beta, act, act_alpha, act_beta, dtype_out)
    return out


def implicit_gemm_wgrad_ref(dout, inp, dweight, indices, reduced_mask, mask_argsort, *,
                            mask_width, dtype_dout, dtype_in, dtype_w,
                            mask_filter=0xFFFFFFFF, alpha=1.0, beta=0.0, split_k_slices=1,
                            tile_k=32, serial_rounding=True):
    """BackwardWeight.  Returns dweight_after ([K, kv, C]).

    dW[:, r, :] = sum over sorted positions pos with
    reduced_mask[pos // mask_width] bit r set and i = indices[r][o] >= 0 of
    dOut[o]^T (x) In[i], o = mask_argsort[pos]
    (cumm/gemm/blockmma/mma.py:580-765, cumm/conv/kernel.py:891-897,969-974;
    check pattern cumm/conv/main_real_spconv.py:375-403 of the reference).
    Offsets r whose bit is clear in mask_filter are not written.

    split_k_slices > 1 with ``serial_rounding``: slice z owns the position
    tiles z, z+S, z+2S, ... of width tile_k; slice 0 writes
    cvt(alpha*acc0 + beta*dW), slice z>0 then writes cvt(alpha*acc_z + dW) in
    slice order, i.e. partial sums are rounded to the weight dtype between
    slices (cumm/conv/kernel.py:960-968,1004-1014,1068-1083 and
    cumm/gemm/output_op/linear.py:90-99 of the reference).
    Without it the slices are summed in float32 and rounded once.
    """
    kv, n = indices.shape
    k_out = dout.shape[1]
    c_in = inp.shape[1]
    rows = mask_argsort[:n].astype(np.int64)
    pos = np.arange(n)
    red = reduced_mask[pos // mask_width]
    out = np.array(dweight, copy=True)
    s = max(1, int(split_k_slices))
    slice_of_pos = (pos // tile_k) % s
    dout_f = nm.to_f32(dout, dtype_dout)
    inp_f = nm.to_f32(inp, dtype_in)
    for r in range(kv):
        if not (int(mask_filter) >> r) & 1:
            continue
        live = ((red >> np.uint32(r)) & 1).astype(bool)
        cur = _src_f32(out[:, r, :], dtype_w)
        parts = []
        for z in range(s):
            sel = live & (slice_of_pos == z)
            o = rows[sel]
            i = indices[r][o]
            valid = i >= 0
            o, i = o[valid], i[valid]
            if o.size:
                parts.append(dout_f[o].T @ inp_f[i])
            else:
                parts.append(np.zeros((k_out, c_in), dtype=np.float32))
        if serial_rounding:
            for z in range(s):
                b = beta if z == 0 else 1.0
                res = linear_combination(parts[z], cur, alpha, b, nm.ACT_NONE, 0.0, 0.0, dtype_w)
                cur = _src_f32(res, dtype_w)
            out[:, r, :] = res
        else:
            tot = parts[0].copy()
            for z in range(1, s):
                tot += parts[z]
            out[:, r, :] = linear_combination(tot, cur, alpha, beta, nm.ACT_NONE, 0.0, 0.0,
                                              dtype_w)
    return out
