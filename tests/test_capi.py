"""The C-ABI library loads and exports every symbol include/cumm_hip.h declares; the
algorithm tables and the argument checks that need no GPU behave as documented."""
import ctypes
import os
import re

import numpy as np
import pytest

from cumm_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "cumm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cumm_hip_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared_symbols()
    assert len(names) >= 20
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_capi.SYMBOLS) == names   # the ctypes table covers exactly the header


def test_struct_layouts_match_the_header():
    """sizeof() of the ctypes mirrors against the C compiler's view of include/cumm_hip.h
    (a silent drift would corrupt arguments); the literal sizes guard machines without gcc."""
    sizes = [ctypes.sizeof(c) for c in (_capi.GemmDesc, _capi.ConvDesc, _capi.GemmArgs, _capi.SparseConvArgs)]
    assert sizes == [72, 96, 160, 168]
    import shutil
    import subprocess
    import tempfile
    if shutil.which("gcc"):
        with tempfile.TemporaryDirectory() as d:
            src = os.path.join(d, "sz.c")
            open(src, "w").write(
                '#include <stdio.h>\n#include "cumm_hip.h"\nint main(){printf("%zu %zu %zu %zu", '
                "sizeof(CummHipGemmDesc), sizeof(CummHipConvDesc), sizeof(CummHipGemmArgs), "
                "sizeof(CummHipSparseConvArgs));}\n")
            exe = os.path.join(d, "sz")
            subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), src, "-o", exe])
            assert [int(x) for x in subprocess.check_output([exe]).split()] == sizes


def test_algorithm_tables():
    lib = _capi.lib()
    n = lib.cumm_hip_list_gemm_algos(None, 0)
    arr = (_capi.GemmDesc * n)()
    assert lib.cumm_hip_list_gemm_algos(arr, n) == n and n > 0
    for d in arr:
        assert lib.cumm_hip_gemm_supported(ctypes.byref(d)) == 1
    bad = _capi.GemmDesc()
    ctypes.memmove(ctypes.byref(bad), ctypes.byref(arr[0]), ctypes.sizeof(bad))
    bad.tile_shape[0] = 48
    assert lib.cumm_hip_gemm_supported(ctypes.byref(bad)) == 0
    m = lib.cumm_hip_list_conv_algos(None, 0)
    carr = (_capi.ConvDesc * m)()
    lib.cumm_hip_list_conv_algos(carr, m)
    for c in carr:
        assert lib.cumm_hip_conv_supported(ctypes.byref(c)) == 1
    ops = {c.op_type for c in carr}
    assert ops == {0, 1, 2}


def test_argument_errors_without_a_gpu():
    lib = _capi.lib()
    assert lib.cumm_hip_gemm(None, None, None) == _capi.EINVAL
    assert b"null" in lib.cumm_hip_last_error()
    n = lib.cumm_hip_list_gemm_algos(None, 0)
    arr = (_capi.GemmDesc * n)()
    lib.cumm_hip_list_gemm_algos(arr, n)
    bad = _capi.GemmDesc()
    ctypes.memmove(ctypes.byref(bad), ctypes.byref(arr[0]), ctypes.sizeof(bad))
    bad.dtype_b = 0
    args = _capi.GemmArgs()
    assert lib.cumm_hip_gemm(ctypes.byref(bad), ctypes.byref(args), None) == _capi.ENOALGO
    with pytest.raises(RuntimeError, match="suitable algo"):
        _capi.check(_capi.ENOALGO)
    # a supported descriptor with empty operands: the reference's "a,b,c must not empty"
    args.m, args.n, args.k = 64, 64, 64
    assert lib.cumm_hip_gemm(ctypes.byref(arr[0]), ctypes.byref(args), None) == _capi.ERUNTIME
    assert b"must not empty" in lib.cumm_hip_last_error()
    # misaligned pointer
    args.ptr_A, args.ptr_B, args.ptr_C = 8, 16, 16
    assert lib.cumm_hip_gemm(ctypes.byref(arr[0]), ctypes.byref(args), None) == _capi.EINVAL
    # sparse conv: kernel volume above 32 has no kernel
    m = lib.cumm_hip_list_conv_algos(None, 0)
    carr = (_capi.ConvDesc * m)()
    lib.cumm_hip_list_conv_algos(carr, m)
    sargs = _capi.SparseConvArgs()
    sargs.N, sargs.C, sargs.K, sargs.kernel_volume = 10, 64, 64, 125
    assert lib.cumm_hip_sparse_conv(ctypes.byref(carr[0]), ctypes.byref(sargs), None) == _capi.EINVAL
    assert lib.cumm_hip_copy_kernel(8, 16, 32, None) == _capi.EINVAL
