"""Scalar numerics shared by the oracle: rounding, activations, dtype names.

Test infrastructure only (see oracle/__init__.py).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

# activation ids: include/tensorview/gemm/core/constants.h:38-54 of the reference
ACT_NONE, ACT_RELU, ACT_SIGMOID, ACT_LEAKY_RELU = 0, 1, 2, 3


def f32_to_bf16_bits(x):
    """float32 -> bfloat16 bit pattern, round-to-nearest-even.

    Follows include/tensorview/gemm/dtypes/bfloat16.h:86-111 of the reference
    (round bit 15, sticky bits 0-14, ties to even on bit 16, NaN -> 0x7FFF).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    lsb = (bits >> 16) & 1
    rounded = (bits + 0x7FFF + lsb) >> 16
    out = rounded.astype(np.uint16)
    out[np.isnan(x)] = 0x7FFF
    return out


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def to_f32(x, dtype):
    """Widen an array of the named storage dtype to float32 (exact)."""
    if dtype == "bf16":
        return bf16_bits_to_f32(x)
    return np.asarray(x).astype(np.float32)


def from_f32(x, dtype):
    """Round float32 to the named storage dtype (RNE), as NumericConverter does
    (include/tensorview/gemm/math/numeric_convert.h of the reference)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == "f32":
        return x.copy()
    if dtype == "f16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16)
    if dtype == "bf16":
        return f32_to_bf16_bits(x)
    raise ValueError(dtype)


def activation(x, act, act_alpha=0.0, act_beta=0.0):
    """UnaryActivation, cumm/gemm/gemmmath/__init__.py:181-214 of the reference."""
    x = np.asarray(x, dtype=np.float32)
    if act == ACT_NONE:
        return x
    if act == ACT_RELU:
        return np.maximum(x, np.float32(0))
    if act == ACT_LEAKY_RELU:
        return np.where(x >= 0, x, x * np.float32(act_alpha)).astype(np.float32)
    if act == ACT_SIGMOID:
        return (np.float32(1) / (np.float32(1) + np.exp(-x))).astype(np.float32)
    raise ValueError(act)


# ---------------------------------------------------------------------------
# C helper (fused multiply-add with a single rounding, nearbyint + saturate)
# ---------------------------------------------------------------------------
_LIB = None


def build_c(force=False):
    so = os.path.join(_HERE, "liboracle.so")
    src = os.path.join(_HERE, "epilogue.c")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    return so


def _lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(build_c())
        f = _LIB.oracle_int8_epilogue
        f.restype = None
        f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                      ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_float,
                      ctypes.c_int, ctypes.c_float]
        g = _LIB.oracle_linear_combination
        g.restype = None
        g.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                      ctypes.c_float, ctypes.c_float]
    return _LIB


def linear_combination_f32(acc, src, alpha, beta):
    """alpha*acc + beta*src in float32 with the reference's operation order
    (see oracle_linear_combination in epilogue.c); ``src`` None or beta == 0
    means the source is not read."""
    acc = np.ascontiguousarray(acc, dtype=np.float32)
    out = np.empty_like(acc)
    src_p = None
    if src is not None and beta != 0.0:
        src = np.ascontiguousarray(np.broadcast_to(np.asarray(src, dtype=np.float32), acc.shape))
        src_p = src.ctypes.data
    _lib().oracle_linear_combination(out.ctypes.data, acc.ctypes.data, src_p, acc.size,
                                     float(alpha), float(beta))
    return out


def int8_epilogue(acc_i32, scale, bias, output_add=None, beta=0.0, act=ACT_NONE, act_alpha=0.0):
    """s32 accumulators -> s8 output rows.

    Int8Inference, cumm/gemm/output_op/linear.py:279-360 of the reference:
    ``t = scale[n]*float(acc) + bias[n]`` (multiply_add, one fused rounding as
    nvcc contracts ``a*b+c``), ``t = beta*float(output_add) + t`` when a source
    is given and beta != 0, activation, clamp to [-128,127], round half to even.
    Conversion: include/tensorview/gemm/math/numeric_convert.h:171-192,262-285.
    """
    acc = np.ascontiguousarray(acc_i32, dtype=np.int32)
    rows, cols = acc.shape
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    assert scale.shape == (cols,) and bias.shape == (cols,)
    out = np.empty((rows, cols), dtype=np.int8)
    src_p = None
    if output_add is not None and beta != 0.0:
        src = np.ascontiguousarray(output_add, dtype=np.int8)
        assert src.shape == acc.shape
        src_p = src.ctypes.data
    _lib().oracle_int8_epilogue(out.ctypes.data, acc.ctypes.data, scale.ctypes.data,
                                bias.ctypes.data, src_p, rows, cols, float(beta), int(act),
                                float(act_alpha))
    return out
