"""Pins for the oracle's scalar numerics: bf16 rounding against torch, the int8 epilogue
against exhaustive closed forms (round half to even, saturation, fused multiply-add)."""
import numpy as np
import torch

from oracle import numerics as nm


def test_bf16_rounding_matches_torch_including_ties():
    rng = np.random.default_rng(0)
    x = rng.normal(0, 100, size=20000).astype(np.float32)
    # exact ties: mantissa tail 0x8000 after a kept bit of 0 and of 1, plus specials
    ties = np.array([0x3F808000, 0x3F818000, 0xBF808000, 0xBF818000, 0x7F7F8000, 0x00008000,
                     0x7F800000, 0xFF800000, 0x00000000, 0x80000000], dtype=np.uint32).view(np.float32)
    x = np.concatenate([x, ties])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = nm.f32_to_bf16_bits(x)
    np.testing.assert_array_equal(got, want)
    back = nm.bf16_bits_to_f32(got)
    np.testing.assert_array_equal(back, torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    assert nm.f32_to_bf16_bits(np.array([np.nan], np.float32))[0] == 0x7FFF


def test_int8_epilogue_round_half_even_and_saturation():
    # scale 0.5, bias 0: acc = 2t+1 lands on exact .5 ties for every t
    acc = np.arange(-600, 601, dtype=np.int32)[None, :]
    n = acc.shape[1]
    out = nm.int8_epilogue(acc, np.full(n, 0.5, np.float32), np.zeros(n, np.float32))
    exact = acc[0] / 2.0
    want = np.clip(np.round(exact), -128, 127)   # numpy round = half to even
    np.testing.assert_array_equal(out[0].astype(np.int64), want.astype(np.int64))
    assert out[0][acc[0] == 5][0] == 2 and out[0][acc[0] == 7][0] == 4 and out[0][acc[0] == -5][0] == -2
    assert out.min() == -128 and out.max() == 127


def test_int8_epilogue_is_a_fused_multiply_add():
    # 16777217 is not a float32; (float)acc rounds to 16777216 first, as the device converter does.
    # scale*acc + bias with ONE rounding differs from two roundings for these operands:
    scale = np.float32(1.0 + 2.0 ** -23)
    accv = np.int32(2 ** 23 + 1)
    bias = np.float32(-(2.0 ** 23))
    fused = float(np.float64(scale) * np.float64(np.float32(accv)) + np.float64(bias))
    two_step = float(np.float32(np.float32(scale) * np.float32(accv)) + bias)
    assert fused != two_step
    out = nm.int8_epilogue(np.array([[accv]], np.int32), np.array([scale]), np.array([bias]))
    assert out[0, 0] == int(np.clip(np.rint(np.float32(fused)), -128, 127))


def test_int8_epilogue_source_activation_order():
    rng = np.random.default_rng(1)
    acc = rng.integers(-20000, 20000, size=(64, 32)).astype(np.int32)
    scale = rng.uniform(0.001, 0.01, 32).astype(np.float32)
    bias = rng.normal(0, 1, 32).astype(np.float32)
    add = rng.integers(-127, 128, size=(64, 32)).astype(np.int8)
    out = nm.int8_epilogue(acc, scale, bias, add, beta=0.5, act=nm.ACT_RELU)
    t = acc.astype(np.float64) * scale.astype(np.float64) + bias.astype(np.float64)
    t = 0.5 * add.astype(np.float64) + t
    want = np.clip(np.rint(np.maximum(t, 0)), -128, 127)
    # float64 evaluation agrees except within float32 rounding of a .5 tie
    assert np.mean(out.astype(np.int64) == want.astype(np.int64)) > 0.999
    assert out.min() >= 0
    # beta == 0 must not read the source at all
    out0 = nm.int8_epilogue(acc, scale, bias, add, beta=0.0)
    np.testing.assert_array_equal(out0, nm.int8_epilogue(acc, scale, bias))


def test_activations():
    x = np.array([-2.0, -0.5, 0.0, 0.5, 3.0], np.float32)
    np.testing.assert_array_equal(nm.activation(x, nm.ACT_RELU), np.array([0, 0, 0, 0.5, 3], np.float32))
    np.testing.assert_allclose(nm.activation(x, nm.ACT_LEAKY_RELU, 0.1), np.where(x >= 0, x, 0.1 * x), rtol=1e-7)
    np.testing.assert_allclose(nm.activation(x, nm.ACT_SIGMOID), torch.sigmoid(torch.from_numpy(x)).numpy(), rtol=1e-6)
