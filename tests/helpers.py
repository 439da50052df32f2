"""Shared builders for the parity tests: seeded inputs, descriptor lookup and
calls through the operator API (which goes through the C ABI)."""
import numpy as np

from cumm_amd import pairs, synth
from cumm_amd import tensorview as tv
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.gemm.main import GemmMainUnitTest
from cumm_amd.tensorview.gemm import (Activation, ConvOpType, ConvParams, GemmParams,
                                      ShuffleStrideType)

TV_DTYPE = {"f16": tv.float16, "bf16": tv.bfloat16, "s8": tv.int8, "f32": tv.float32, "s32": tv.int32}


def to_storage(x_f32, dtype):
    """float32 values -> array in the storage dtype (bf16 as uint16 bits)."""
    if dtype == "f16":
        return x_f32.astype(np.float16)
    if dtype == "bf16":
        return synth.f32_to_bf16_bits(x_f32)
    if dtype == "s8":
        return x_f32.astype(np.int8)
    if dtype == "s32":
        return x_f32.astype(np.int32)
    return x_f32.astype(np.float32)


def as_f32(x, dtype):
    if dtype == "bf16":
        return synth.bf16_bits_to_f32(x)
    return np.asarray(x).astype(np.float32)


def dev(arr, dtype):
    """numpy array in storage dtype -> device tv.Tensor."""
    t = tv.from_numpy(np.ascontiguousarray(arr))
    if dtype == "bf16":
        t = t.type_view(tv.bfloat16)
    return t.cuda()


def host(t):
    return t.cpu().numpy()


def rel_err(got_f32, ref_f32):
    """The larger of two figures: max |got-ref| / max |ref| over the whole tensor - the reference's
    own criterion (cumm/gemm/main_real.py:672-677) - and the same per row (:func:`rel_err_rows`),
    so that a wrong row of small magnitude cannot hide under the tensor's largest value."""
    got_f32, ref_f32 = np.asarray(got_f32), np.asarray(ref_f32)
    denom = max(float(np.max(np.abs(ref_f32))), 1e-6) if ref_f32.size else 1.0
    if ref_f32.size == 0:
        return 0.0
    whole = float(np.max(np.abs(got_f32.astype(np.float64) - ref_f32.astype(np.float64)))) / denom
    if ref_f32.ndim == 0:
        return whole
    return max(whole, rel_err_rows(got_f32, ref_f32))


def rel_err_rows(got_f32, ref_f32, floor_frac=1e-2):
    """The same, normalised per row: max over rows of max |got-ref| over the row / max |ref| over
    the row, so that a wrong row of small magnitude cannot hide under the tensor's largest
    value.  Rows whose own maximum is below ``floor_frac`` of the tensor's are measured against
    that floor (rounding noise of a near-zero row is not a relative error)."""
    g = got_f32.astype(np.float64).reshape(got_f32.shape[0], -1)
    r = ref_f32.astype(np.float64).reshape(ref_f32.shape[0], -1)
    floor = max(float(np.max(np.abs(r))) * floor_frac, 1e-6)
    denom = np.maximum(np.max(np.abs(r), axis=1), floor)
    return float(np.max(np.max(np.abs(g - r), axis=1) / denom))


def find_conv_desp(dtype, op, tile_m, tile_n, int8_inference=False, split_k_parallel=False, dtype_out=None,
                   dynamic_mask=False):
    """``dtype_out``: element type of the result when it differs from the operands' ("s32", "f32");
    ``dynamic_mask``: the descriptors for kernel volumes above 32 (several mask words per position)."""
    for d in ConvMainUnitTest.get_all_conv_algo_desp():
        if (d.dtype_a == TV_DTYPE[dtype] and d.dtype_output == TV_DTYPE[dtype_out or dtype] and
                d.dtype_input == TV_DTYPE[dtype] and ConvOpType(d.op_type) == op and
                d.tile_shape[0] == tile_m and d.tile_shape[1] == tile_n and
                d.is_int8_inference == int8_inference and d.split_k_parallel == split_k_parallel and
                bool(d.dynamic_mask) == dynamic_mask):
            return d
    raise KeyError((dtype, op, tile_m, tile_n, int8_inference, split_k_parallel, dynamic_mask))


def find_gemm_desp(dtype, shuffle, tile_m, tile_n, trans_a, trans_b, trans_c=False, dtype_c=None):
    for d in GemmMainUnitTest.get_all_algo_desp():
        if (d.dtype_a == TV_DTYPE[dtype] and d.dtype_c == TV_DTYPE[dtype_c or dtype] and d.shuffle_type == shuffle and
                d.tile_shape[0] == tile_m and d.tile_shape[1] == tile_n and
                d.trans_a == trans_a and d.trans_b == trans_b and d.trans_c == trans_c):
            return d
    raise KeyError((dtype, shuffle, tile_m, tile_n, trans_a, trans_b, trans_c))


def small_cloud(seed, n, grid=(12, 40, 36), clusters=6, sigma=3.0):
    rng = np.random.default_rng(seed)
    return synth.clustered_voxels(rng, n, grid, clusters, sigma=sigma), grid
