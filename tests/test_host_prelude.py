"""Host logic of the operator surface that needs no GPU: m/n/k extraction, tile selection,
validation errors (same exception classes as the reference), tv.Tensor host behaviour and the
cache of validated arguments."""
import numpy as np
import pytest

from cumm_amd import tensorview as tv
from cumm_amd.conv.main import ConvMainUnitTest
from cumm_amd.gemm.main import GemmMainUnitTest
from cumm_amd.tensorview.gemm import (Activation, ConvOpType, ConvParams, GemmAlgoDesp, GemmParams,
                                      ShuffleStrideType)


def blob(shape, dtype):
    """A tensor that claims to live on device 0 (never dereferenced in these tests)."""
    return tv.from_blob(0x7F0000000000, shape, dtype, 0)


def test_extract_mnk_follows_the_reference():
    f = GemmMainUnitTest.extract_mnk
    assert f([100, 32], [32, 48], False, False, False) == (100, 48, 32)
    assert f([32, 100], [48, 32], True, True, False) == (100, 48, 32)
    assert f([100, 32], [32, 48], False, False, True) == (48, 100, 32)          # swapped problem
    assert f([1000, 64], [64, 64], False, True, False, 1, [700], [], [700]) == (700, 64, 64)
    assert f([1000, 64], [1000, 32], True, False, False, 2, [555], [555]) == (64, 32, 555)
    with pytest.raises(RuntimeError):
        f([64, 1000], [64, 64], True, True, False, 1, [700], [], [700])       # A must be row major
    with pytest.raises(RuntimeError):
        f([1000, 64], [1000, 32], False, False, False, 2, [555], [555])       # ShuffleAB must be nt
    assert ConvMainUnitTest.extract_mnk(ConvOpType.BackwardWeight, 1000, 64, 64, 27, -1, -1, True) == (64, 1728, 1000)


def test_align_to_power2_and_tile_selection():
    a = GemmMainUnitTest.align_to_power2
    assert [a(v) for v in (1, 2, 3, 5, 64, 65, 1000)] == [1, 2, 4, 8, 64, 128, 1024]
    algos = {64 | (64 << 20) | (32 << 40): [1], 128 | (64 << 20) | (32 << 40): [2],
             128 | (128 << 20) | (32 << 40): [3]}
    sel = GemmMainUnitTest.simple_select_tile_shape
    assert sel(100, 64, 64, [64, 128], [64, 128], [32], algos, False) == [2]
    assert sel(30, 30, 8, [64, 128], [64, 128], [32], algos, False) == [1]
    assert sel(5000, 5000, 64, [64, 128], [64, 128], [32], algos, True) == [3]
    assert sel(10, 10, 10, [32], [32], [32], algos, False) == []


def _fwd_params():
    n = 1000
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = [d for d in ConvMainUnitTest.get_all_conv_algo_desp()
                        if d.dtype_a == tv.float16 and d.dtype_c == tv.float16 and
                        ConvOpType(d.op_type) == ConvOpType.Forward][0]
    p.input, p.weight, p.output = blob([n, 64], tv.float16), blob([64, 27, 64], tv.float16), blob([n, 64], tv.float16)
    p.indices, p.mask, p.mask_argsort = blob([27, n], tv.int32), blob([n], tv.uint32), blob([n], tv.int32)
    return p


def test_conv_prelude_errors():
    p = _fwd_params()
    p.output_add = blob([1000, 64], tv.float16)
    with pytest.raises(ValueError, match="only int8 inference"):
        ConvMainUnitTest.implicit_gemm2(p)
    p = _fwd_params()
    p.split_k_slices = 4
    with pytest.raises(RuntimeError, match="splitk"):
        ConvMainUnitTest.implicit_gemm2(p)
    p = _fwd_params()
    p.mask_int_count = 2                               # several mask words per position: not built
    with pytest.raises(RuntimeError, match="mask_int_count"):
        ConvMainUnitTest.implicit_gemm2(p)
    p = _fwd_params()
    p.indices = tv.Tensor()
    with pytest.raises(RuntimeError):
        ConvMainUnitTest.implicit_gemm2(p)
    p = _fwd_params()
    p.input = blob([1000, 60], tv.float16)            # C not a multiple of the access width
    p.weight = blob([64, 27, 60], tv.float16)
    with pytest.raises(RuntimeError):
        ConvMainUnitTest.implicit_gemm2(p)
    p = _fwd_params()
    p.output = blob([999, 64], tv.float16)            # N must equal output rows
    with pytest.raises(RuntimeError):
        ConvMainUnitTest.implicit_gemm2(p)
    p = _fwd_params()
    p.input = tv.from_numpy(np.zeros((1000, 64), np.float16))   # host tensor
    with pytest.raises((RuntimeError, ValueError)):
        ConvMainUnitTest.implicit_gemm2(p)
    # backward weight: mask_width must be a positive multiple of tile k
    pw = ConvParams(3, ConvOpType.BackwardWeight)
    pw.conv_algo_desp = [d for d in ConvMainUnitTest.get_all_conv_algo_desp()
                         if d.dtype_a == tv.float16 and ConvOpType(d.op_type) == ConvOpType.BackwardWeight][0]
    pw.input, pw.weight, pw.output = blob([1000, 64], tv.float16), blob([64, 27, 64], tv.float16), blob([1000, 64], tv.float16)
    pw.indices, pw.mask, pw.mask_argsort = blob([27, 1000], tv.int32), blob([16], tv.uint32), blob([1000], tv.int32)
    pw.mask_width = 48
    with pytest.raises(RuntimeError):
        ConvMainUnitTest.implicit_gemm2(pw)


def test_gemm_prelude_errors():
    d = [x for x in GemmMainUnitTest.get_all_algo_desp()
         if x.dtype_a == tv.float16 and x.dtype_c == tv.float16 and
         x.shuffle_type == ShuffleStrideType.ShuffleAC and x.trans_b][0]
    p = GemmParams()
    p.algo_desp = d
    with pytest.raises(RuntimeError, match="a,b,c must not empty"):
        GemmMainUnitTest.matmul2(p)
    p.a, p.b, p.c = blob([100, 64], tv.float16), blob([64, 64], tv.float16), blob([100, 64], tv.float16)
    with pytest.raises(RuntimeError, match="c_inds"):
        GemmMainUnitTest.matmul2(p)
    p.c_inds = blob([100], tv.int32)
    p.b = blob([64, 72], tv.float16)                 # k mismatch
    with pytest.raises(ValueError):
        GemmMainUnitTest.matmul2(p)
    p.b = blob([64, 64], tv.float16)
    p.a = blob([100, 60], tv.float16)                # misaligned contiguous dim
    p.b = blob([64, 60], tv.float16)
    with pytest.raises(ValueError, match="misaligned"):
        GemmMainUnitTest.matmul2(p)
    p.a, p.b = blob([100, 64], tv.float16), blob([64, 64], tv.float16)
    p.split_k_slices = 2
    with pytest.raises(RuntimeError, match="splitk"):
        GemmMainUnitTest.matmul2(p)


def test_tensor_host_semantics():
    a = np.arange(24, dtype=np.float32).reshape(4, 6)
    t = tv.from_numpy(a)
    assert t.shape == [4, 6] and t.stride == [6, 1] and t.dtype == tv.float32 and t.device == -1
    assert t.dim(1) == 6 and t.ndim == 2 and t.size == 24 and t.itemsize == 4 and not t.empty()
    np.testing.assert_array_equal(t[1:3].numpy(), a[1:3])
    np.testing.assert_array_equal(t[2].numpy(), a[2])
    np.testing.assert_array_equal(t[:, 1:5:2].numpy(), a[:, 1:5:2])
    np.testing.assert_array_equal(t.T.numpy(), a.T)
    np.testing.assert_array_equal(t.view([2, 12]).numpy(), a.reshape(2, 12))
    np.testing.assert_array_equal(t.slice_first_axis(1, 3).numpy(), a[1:3])
    assert not t.T.is_contiguous() and t[1:3].is_contiguous()
    z = tv.zeros([3, 2], tv.int32)
    assert not z.numpy().any()
    z.fill_int_(7)
    assert (z.numpy() == 7).all()
    c = t.clone()
    c.zero_()
    assert t.numpy().any() and not c.numpy().any()
    assert tv.Tensor().empty()
    with pytest.raises(ValueError):
        t.view([2, 12]).T.T.view([4, 6]).T.T[0].T   # .T only on 2-D tensors
    b = tv.from_numpy(np.zeros(4, np.uint16)).type_view(tv.bfloat16)
    assert b.dtype == tv.bfloat16 and b.numpy().dtype == np.uint16


def test_validated_argument_cache_is_invalidated_by_any_assignment():
    calls = []
    from cumm_amd import _capi
    real = _capi.lib()

    class Spy:
        def __getattr__(self, n):
            if n == "cumm_hip_sparse_conv":
                def f(desc, args, stream):
                    calls.append((args._obj.beta, args._obj.mask_filter, desc._obj.gemm.tile_shape[0]))
                    return 0
                return f
            return getattr(real, n)
    _capi._lib = Spy()
    try:
        p = _fwd_params()
        ConvMainUnitTest.implicit_gemm2(p)
        ConvMainUnitTest.implicit_gemm2(p)          # cached path
        p.beta = 1.0
        ConvMainUnitTest.implicit_gemm2(p)
        p.mask_filter = 0x3FFF
        ConvMainUnitTest.implicit_gemm2(p)
        d = p.conv_algo_desp
        d.tile_shape[0] = 128                       # in-place edit of the descriptor
        d.warp_tile_shape[0] = 32
        ConvMainUnitTest.implicit_gemm2(p)
        assert calls == [(0.0, 0xFFFFFFFF, 64), (0.0, 0xFFFFFFFF, 64), (1.0, 0xFFFFFFFF, 64),
                         (1.0, 0x3FFF, 64), (1.0, 0x3FFF, 128)]
    finally:
        _capi._lib = real


def test_conv_prelude_rejects_wrong_element_types():
    """Every operand must have the descriptor's element type (the reference's data_ptr<T>()
    check): the kernels size their buffer descriptors from the descriptor, so a narrower tensor
    would be read past its end."""
    cases = [("input", blob([1000, 64], tv.int8)), ("input", blob([1000, 64], tv.float32)),
             ("weight", blob([64, 27, 64], tv.bfloat16)), ("output", blob([1000, 64], tv.int8)),
             ("indices", blob([27, 1000], tv.int64)), ("mask_argsort", blob([1000], tv.int64)),
             ("mask", blob([1000], tv.int32)), ("mask_output", blob([16], tv.int32)),
             ("bias", blob([64], tv.float32))]
    for name, bad in cases:
        p = _fwd_params()
        setattr(p, name, bad)
        with pytest.raises(RuntimeError, match="dtype"):
            ConvMainUnitTest.implicit_gemm2(p)
    # int8 inference: scale and bias are float32
    d = [x for x in ConvMainUnitTest.get_all_conv_algo_desp() if x.is_int8_inference and x.dtype_c == tv.int8][0]
    p = ConvParams(3, ConvOpType.Forward)
    p.conv_algo_desp = d
    p.input, p.weight, p.output = blob([1000, 64], tv.int8), blob([128, 27, 64], tv.int8), blob([1000, 128], tv.int8)
    p.indices, p.mask, p.mask_argsort = blob([27, 1000], tv.int32), blob([1000], tv.uint32), blob([1000], tv.int32)
    p.scale, p.bias = blob([128], tv.float16), blob([128], tv.float32)
    with pytest.raises(RuntimeError, match="dtype"):
        ConvMainUnitTest.implicit_gemm2(p)


def test_gemm_prelude_rejects_wrong_index_types():
    d = [x for x in GemmMainUnitTest.get_all_algo_desp()
         if x.dtype_a == tv.float16 and x.dtype_c == tv.float16 and
         x.shuffle_type == ShuffleStrideType.ShuffleAC and x.trans_b][0]
    p = GemmParams()
    p.algo_desp = d
    p.a, p.b, p.c = blob([100, 64], tv.float16), blob([64, 64], tv.float16), blob([100, 64], tv.float16)
    p.c_inds = blob([100], tv.int64)
    with pytest.raises(RuntimeError, match="dtype"):
        GemmMainUnitTest.matmul2(p)
    p.c_inds = blob([100], tv.int32)
    p.a_inds = blob([100], tv.int64)
    with pytest.raises(RuntimeError, match="dtype"):
        GemmMainUnitTest.matmul2(p)


def test_full_and_fill_on_bfloat16():
    """tv.full / fill_float_ on bf16 write bf16 bit patterns (round to nearest even), not the
    value truncated to an integer."""
    from cumm_amd import synth
    for val in (1.0, -2.5, 0.1, 3.0e38, 1.00390625):   # the last one is a tie: rounds to even
        t = tv.full([3, 4], val, tv.bfloat16)
        assert t.dtype == tv.bfloat16
        bits = t.numpy_view()
        want = synth.f32_to_bf16_bits(np.full((3, 4), val, np.float32))
        np.testing.assert_array_equal(bits, want)
    t = tv.zeros([5], tv.bfloat16)
    t.fill_int_(7)
    np.testing.assert_array_equal(synth.bf16_bits_to_f32(t.numpy_view()), np.full(5, 7.0, np.float32))
