"""ctypes binding of libcummhip.so (the C ABI declared in include/cumm_hip.h).

The library is loaded from ``cumm_amd/libcummhip.so``; if it has not been built
it is built once with hipcc (``cumm_amd.build``).  There is no CPU fallback:
every operator raises if the library cannot be loaded.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcummhip.so")

OK, EINVAL, ERUNTIME, ENOALGO = 0, 1, 2, 3
STATIC_WORKSPACE_BYTES = 8 << 20   # CUMM_HIP_STATIC_WORKSPACE_BYTES


class GemmDesc(C.Structure):
    _fields_ = [("dtype_a", C.c_int32), ("dtype_b", C.c_int32), ("dtype_c", C.c_int32),
                ("dacc", C.c_int32), ("dcomp", C.c_int32),
                ("trans_a", C.c_int32), ("trans_b", C.c_int32), ("trans_c", C.c_int32),
                ("tile_shape", C.c_int32 * 3), ("warp_tile_shape", C.c_int32 * 3),
                ("num_stage", C.c_int32), ("shuffle_type", C.c_int32),
                ("split_k_serial", C.c_int32), ("split_k_parallel", C.c_int32)]


class ConvDesc(C.Structure):
    _fields_ = [("gemm", GemmDesc), ("ndim", C.c_int32), ("op_type", C.c_int32),
                ("mask_sparse", C.c_int32), ("increment_k_first", C.c_int32),
                ("dynamic_mask", C.c_int32), ("is_int8_inference", C.c_int32)]


class GemmArgs(C.Structure):
    _fields_ = [("m", C.c_int32), ("n", C.c_int32), ("k", C.c_int32),
                ("ptr_A", C.c_void_p), ("ptr_B", C.c_void_p), ("ptr_D", C.c_void_p),
                ("ptr_C", C.c_void_p),
                ("stride_A", C.c_int64), ("stride_B", C.c_int64), ("stride_C", C.c_int64),
                ("stride_D", C.c_int64),
                ("indiceA", C.c_void_p), ("indiceBorC", C.c_void_p), ("indiceD", C.c_void_p),
                ("alpha", C.c_float), ("beta", C.c_float), ("act_alpha", C.c_float),
                ("act_beta", C.c_float), ("act_type", C.c_int32), ("split_k_slices", C.c_int32),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
                ("rows_A", C.c_int32), ("rows_B", C.c_int32), ("rows_C", C.c_int32)]


class SparseConvArgs(C.Structure):
    _fields_ = [("ptr_A", C.c_void_p), ("ptr_B", C.c_void_p), ("ptr_D", C.c_void_p),
                ("ptr_C", C.c_void_p),
                ("alpha", C.c_float), ("beta", C.c_float), ("act_alpha", C.c_float),
                ("act_beta", C.c_float), ("act_type", C.c_int32), ("split_k_slices", C.c_int32),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
                ("mask_ptr", C.c_void_p), ("mask_out_ptr", C.c_void_p),
                ("indice_ptr", C.c_void_p), ("mask_argsort_ptr", C.c_void_p),
                ("mask_filter", C.c_uint32), ("reverse_mask", C.c_int32),
                ("mask_width", C.c_int32),
                ("ndim", C.c_int32), ("N", C.c_int32), ("C", C.c_int32), ("K", C.c_int32),
                ("kernel_volume", C.c_int32), ("mode", C.c_int32), ("groups", C.c_int32),
                ("d_is_bias", C.c_int32), ("deterministic", C.c_int32),
                ("bias_pointer", C.c_void_p), ("scale_pointer", C.c_void_p),
                ("rows_in", C.c_int32), ("rows_out", C.c_int32), ("light_prefix", C.c_int32),
                ("ungated_rows", C.c_int32), ("indices_by_position", C.c_int32), ("mask_int_count", C.c_int32)]


# every symbol include/cumm_hip.h declares: name -> (restype, argtypes)
_VP, _PVP = C.c_void_p, C.POINTER(C.c_void_p)
SYMBOLS = {
    "cumm_hip_gemm": (C.c_int, [C.POINTER(GemmDesc), C.POINTER(GemmArgs), _VP]),
    "cumm_hip_sparse_conv": (C.c_int, [C.POINTER(ConvDesc), C.POINTER(SparseConvArgs), _VP]),
    "cumm_hip_sparse_conv_static_ws": (C.c_int, [C.POINTER(ConvDesc), C.POINTER(SparseConvArgs), _VP]),
    "cumm_hip_query_gemm_workspace": (C.c_int64, [C.POINTER(GemmDesc), C.c_int, C.c_int, C.c_int, C.c_int]),
    "cumm_hip_query_conv_workspace": (C.c_int64, [C.POINTER(ConvDesc), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "cumm_hip_query_wgrad_ordered_workspace": (C.c_int64, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "cumm_hip_list_gemm_algos": (C.c_int, [C.POINTER(GemmDesc), C.c_int]),
    "cumm_hip_list_conv_algos": (C.c_int, [C.POINTER(ConvDesc), C.c_int]),
    "cumm_hip_gemm_supported": (C.c_int, [C.POINTER(GemmDesc)]),
    "cumm_hip_conv_supported": (C.c_int, [C.POINTER(ConvDesc)]),
    "cumm_hip_last_error": (C.c_char_p, []),
    "cumm_hip_last_wgrad_path": (C.c_int, []),
    "cumm_hip_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "cumm_hip_malloc": (C.c_int, [_PVP, C.c_size_t]),
    "cumm_hip_free": (C.c_int, [_VP]),
    "cumm_hip_host_malloc": (C.c_int, [_PVP, C.c_size_t]),
    "cumm_hip_host_free": (C.c_int, [_VP]),
    "cumm_hip_memcpy_h2d": (C.c_int, [_VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_memcpy_d2h": (C.c_int, [_VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_memcpy_d2d": (C.c_int, [_VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_memset": (C.c_int, [_VP, C.c_int, C.c_size_t, _VP]),
    "cumm_hip_stream_create": (C.c_int, [_PVP]),
    "cumm_hip_stream_destroy": (C.c_int, [_VP]),
    "cumm_hip_stream_synchronize": (C.c_int, [_VP]),
    "cumm_hip_device_synchronize": (C.c_int, []),
    "cumm_hip_take_async_errors": (C.c_int, [C.POINTER(C.c_int32)]),
    "cumm_hip_set_split_k_spin_limit": (C.c_int, [C.c_int]),
    "cumm_hip_event_create": (C.c_int, [_PVP]),
    "cumm_hip_event_destroy": (C.c_int, [_VP]),
    "cumm_hip_event_record": (C.c_int, [_VP, _VP]),
    "cumm_hip_event_synchronize": (C.c_int, [_VP]),
    "cumm_hip_event_elapsed_ms": (C.c_int, [_VP, _VP, C.POINTER(C.c_float)]),
    "cumm_hip_copy_kernel": (C.c_int, [_VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_subm_pairs_workspace": (C.c_size_t, [C.c_int]),
    "cumm_hip_subm_pairs": (C.c_int, [_VP, C.c_int, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                      _VP, _VP, _VP, _VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_sort_by_mask_workspace": (C.c_size_t, [C.c_int]),
    "cumm_hip_sort_by_mask": (C.c_int, [_VP, C.c_int, C.c_uint32, _VP, _VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_masks_from_pairs": (C.c_int, [_VP, C.c_int, C.c_int, _VP, _VP]),
    "cumm_hip_sort_by_mask_words_workspace": (C.c_size_t, [C.c_int]),
    "cumm_hip_sort_by_mask_words": (C.c_int, [_VP, C.c_int, C.c_int, _VP, _VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_sort_by_mask_ordered": (C.c_int, [_VP, C.c_int, C.c_uint32, C.c_int, _VP, _VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_pairs_by_position": (C.c_int, [_VP, _VP, C.c_int, C.c_int, _VP, _VP]),
    "cumm_hip_query_light_hint": (C.c_int, [_VP, C.c_int, C.c_uint32, C.POINTER(C.c_int32), C.POINTER(C.c_int32), _VP]),
    "cumm_hip_light_prefix": (C.c_int, [_VP, C.c_int, C.c_uint32, _VP, _VP]),
    "cumm_hip_conv_pairs_workspace": (C.c_size_t, [C.c_int, C.c_int] + [C.POINTER(C.c_int32)] * 5),
    "cumm_hip_conv_pairs_sites": (C.c_int, [_VP, C.c_int, C.c_int] + [C.POINTER(C.c_int32)] * 5 +
                                  [C.POINTER(C.c_int32), C.POINTER(C.c_int32), _VP, C.c_size_t, _VP]),
    "cumm_hip_conv_pairs_fill": (C.c_int, [_VP, C.c_int, C.c_int] + [C.POINTER(C.c_int32)] * 5 +
                                 [C.c_int, _VP, _VP, _VP, _VP, _VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_pair_lists_workspace": (C.c_size_t, [C.c_int, C.c_int]),
    "cumm_hip_pair_lists": (C.c_int, [_VP, C.c_int, C.c_int, _VP, _VP, _VP, _VP, C.c_size_t, _VP]),
    "cumm_hip_finish_rows": (C.c_int, [_VP, C.c_int, _VP, _VP, C.c_int64, C.c_int, C.c_float, C.c_float, C.c_int,
                                       C.c_float, _VP]),
    "cumm_hip_relu_backward": (C.c_int, [_VP, _VP, _VP, C.c_size_t, C.c_int, _VP]),
    "cumm_hip_column_sum_workspace": (C.c_size_t, [C.c_int64, C.c_int]),
    "cumm_hip_column_sum": (C.c_int, [_VP, _VP, C.c_int64, C.c_int, C.c_int, _VP, C.c_size_t, _VP]),
    "cumm_hip_gather_rows": (C.c_int, [_VP, _VP, _VP, C.c_int, C.c_int, C.c_size_t, _VP]),
    "cumm_hip_scatter_add_rows": (C.c_int, [_VP, _VP, _VP, C.c_int, C.c_int, C.c_int, C.c_int, _VP]),
}

_lib = None


def lib():
    """The loaded library; builds it first if no built library is present."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            from . import build as _build
            _build.build()
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def last_error():
    msg = lib().cumm_hip_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(status):
    """Raise the exception class the reference raises for this kind of failure
    (include/tensorview/core/common.h:102-142: TV_ASSERT_RT_ERR -> RuntimeError,
    TV_ASSERT_INVALID_ARG -> ValueError)."""
    if status == OK:
        return
    msg = last_error()
    if status == EINVAL:
        raise ValueError(msg)
    raise RuntimeError(msg)
