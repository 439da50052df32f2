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
    assert sizes == [72, 96, 160, 192]
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
    sargs.mode, sargs.groups = 1, 1
    assert lib.cumm_hip_sparse_conv(ctypes.byref(carr[0]), ctypes.byref(sargs), None) == _capi.EINVAL
    assert b"kernel volume" in lib.cumm_hip_last_error()
    # true convolution (flipped kernel) and grouped convolution have no kernel
    sargs.kernel_volume, sargs.mode = 27, 0
    assert lib.cumm_hip_sparse_conv(ctypes.byref(carr[0]), ctypes.byref(sargs), None) == _capi.EINVAL
    assert b"cross-correlation" in lib.cumm_hip_last_error()
    sargs.mode, sargs.groups = 1, 2
    assert lib.cumm_hip_sparse_conv(ctypes.byref(carr[0]), ctypes.byref(sargs), None) == _capi.EINVAL
    assert b"groups" in lib.cumm_hip_last_error()
    assert lib.cumm_hip_copy_kernel(8, 16, 32, None) == _capi.EINVAL


def test_workspace_queries_follow_the_descriptors():
    """cumm_hip_query_*_workspace against the Python mirrors of GemmAlgoDesp.query_workspace_size /
    ConvAlgoDesp.query_conv_workspace_size (which the golden cases pin against the reference's headers)."""
    from cumm_amd.conv.main import ConvMainUnitTest, conv_desp_to_c
    from cumm_amd.gemm.main import GemmMainUnitTest, desp_to_c
    lib = _capi.lib()
    for d in GemmMainUnitTest.get_all_algo_desp():
        cd = desp_to_c(d)
        for m, n, k, s in ((1000, 136, 64, 1), (1000, 136, 640, 4), (64, 64, 64, 2)):
            if s > 1 and not (d.split_k_serial or d.split_k_parallel):
                assert lib.cumm_hip_query_gemm_workspace(ctypes.byref(cd), m, n, k, s) == -1
            else:
                assert lib.cumm_hip_query_gemm_workspace(ctypes.byref(cd), m, n, k, s) == d.query_workspace_size(m, n, k, s)
    for d in ConvMainUnitTest.get_all_conv_algo_desp():
        cd = conv_desp_to_c(d)
        for m, n, k, s, kv in ((64, 27 * 64, 120000, 1, 27), (128, 27 * 128, 5000, 32, 27), (64, 8 * 72, 999, 2, 8)):
            if s > 1 and not (d.split_k_serial or d.split_k_parallel):
                assert lib.cumm_hip_query_conv_workspace(ctypes.byref(cd), m, n, k, s, kv) == -1
            else:
                assert lib.cumm_hip_query_conv_workspace(ctypes.byref(cd), m, n, k, s, kv) == \
                    d.query_conv_workspace_size(m, n, k, s, kv)


def test_fixed_order_backward_weight_workspace_query():
    """cumm_hip_query_wgrad_ordered_workspace: 256-byte aligned pieces (live-tile counts, the table of
    workgroups per (offset, channel block), the live-tile lists) in front of one slot of 64 x 64
    (or 128 x 128) floats per workgroup and per (offset, channel block); -1 for sizes it does not take."""
    lib = _capi.lib()
    q = lib.cumm_hip_query_wgrad_ordered_workspace
    # 3000 positions, 64-position mask words: 47 tiles, 16 per unit at most -> (3 + 1) * 27 = 108 units
    n, c, k, kv, mw = 3000, 64, 64, 27, 64
    lists = 128 + 256 + ((4 * kv * 47 + 255) // 256) * 256
    assert q(n, c, k, kv, mw) == lists + (108 + 27) * 64 * 64 * 4
    # both channel counts above 64: slots of 128 x 128; many tiles: 512 workgroups at most
    n = 1000000
    tiles = (n + 63) // 64
    lists = 128 + 256 + ((4 * kv * tiles + 255) // 256) * 256
    assert q(n, 128, 128, kv, 64) == lists + (512 + 27) * 128 * 128 * 4
    assert q(n, 128, 256, kv, 64) == 128 + 512 + ((4 * kv * tiles + 255) // 256) * 256 + (512 + 54) * 128 * 128 * 4
    for bad in ((-1, 64, 64, 27, 64), (10, 0, 64, 27, 64), (10, 64, 64, 33, 64), (10, 64, 64, 27, 2048), (10, 64, 64, 27, 0)):
        assert q(*bad) == -1
    args = _capi.SparseConvArgs()
    args.deterministic = 1     # the field exists (it fills former padding)
    args.light_prefix = 128
    assert ctypes.sizeof(args) == 192
