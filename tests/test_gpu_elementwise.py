"""Row-wise helper kernels (cumm_hip_finish_rows / relu_backward / column_sum) through the C ABI
against their closed forms in numpy: elementwise work is bit-exact, the fp32 column sum is
compared with a float64 sum within fp32 rounding and must repeat bit for bit."""
import numpy as np
import pytest

import helpers as H
from cumm_amd import _capi
from cumm_amd import tensorview as tv
from oracle import numerics as onm

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("rows,channels", [(1000, 64), (37, 8), (5000, 136)])
def test_finish_rows(dtype, rows, channels):
    rng = np.random.default_rng(3)
    acc = rng.normal(0, 2, size=(rows, channels)).astype(np.float32)
    bias = H.to_storage(rng.normal(0, 1, size=(channels,)).astype(np.float32), dtype)
    lib = _capi.lib()
    for alpha, beta, act, use_bias in ((1.0, 0.0, onm.ACT_NONE, False), (0.5, 1.0, onm.ACT_RELU, True),
                                       (1.0, 2.0, onm.ACT_LEAKY_RELU, True)):
        out = tv.zeros([rows, channels], H.TV_DTYPE[dtype], 0)
        d_acc, d_bias = H.dev(acc, "f32"), H.dev(bias, dtype)
        _capi.check(lib.cumm_hip_finish_rows(out.byte_pointer(), H.TV_DTYPE[dtype], d_acc.byte_pointer(),
                                             d_bias.byte_pointer() if use_bias else None, rows, channels,
                                             alpha, beta, act, 0.1, 0))
        t = onm.linear_combination_f32(acc, H.as_f32(bias, dtype)[None, :] if use_bias else None, alpha,
                                       beta if use_bias else 0.0)
        want = onm.from_f32(onm.activation(t, act, 0.1), dtype)
        np.testing.assert_array_equal(H.host(out), want)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_relu_backward(dtype):
    rng = np.random.default_rng(4)
    n = 4096 * 3 + 8
    out = H.to_storage(np.maximum(rng.normal(0, 1, size=n), 0).astype(np.float32), dtype)
    grad = H.to_storage(rng.normal(0, 1, size=n).astype(np.float32), dtype)
    dst = tv.zeros([n], H.TV_DTYPE[dtype], 0)
    d_g, d_o = H.dev(grad, dtype), H.dev(out, dtype)
    _capi.check(_capi.lib().cumm_hip_relu_backward(dst.byte_pointer(), d_g.byte_pointer(), d_o.byte_pointer(), n,
                                                   H.TV_DTYPE[dtype], 0))
    want = np.where(H.as_f32(out, dtype) > 0, grad, np.zeros_like(grad))
    np.testing.assert_array_equal(H.host(dst), want)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("rows,channels", [(100000, 128), (777, 64), (3, 256), (50000, 8)])
def test_column_sum(dtype, rows, channels):
    rng = np.random.default_rng(5)
    src = H.to_storage(rng.normal(0.1, 1, size=(rows, channels)).astype(np.float32), dtype)
    lib = _capi.lib()
    need = int(lib.cumm_hip_column_sum_workspace(rows, channels))
    ws = tv.empty([need], tv.uint8, 0)
    d_src = H.dev(src, dtype)
    results = []
    for _ in range(2):
        dst = tv.zeros([channels], H.TV_DTYPE[dtype], 0)
        _capi.check(lib.cumm_hip_column_sum(dst.byte_pointer(), d_src.byte_pointer(), rows, channels,
                                            H.TV_DTYPE[dtype], ws.byte_pointer(), need, 0))
        results.append(H.host(dst))
    np.testing.assert_array_equal(results[0], results[1])        # fixed order of the sums
    exact = H.as_f32(src, dtype).astype(np.float64).sum(axis=0)
    got = H.as_f32(results[0], dtype).astype(np.float64)
    # fp32 partial sums + one rounding to 16 bits
    scale = np.abs(H.as_f32(src, dtype)).astype(np.float64).sum(axis=0) + 1e-6
    ulp16 = 2.0 ** (-10 if dtype == "f16" else -7)
    assert np.all(np.abs(got - exact) <= 1e-5 * scale + ulp16 * np.abs(exact))
