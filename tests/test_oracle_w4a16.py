"""Pins the CPU oracle's W4A16 functions (restating lib/cpu.ml:128-170,226,239)
against the reference's golden vectors and against exact rational arithmetic."""
from fractions import Fraction

import numpy as np
import pytest

import oracle


def _bits_to_f16(bits):
    return np.array(bits, dtype=np.uint16).view(np.float16)


def test_f16_conversion_matches_ieee_on_every_half_and_random_floats():
    every = np.arange(65536, dtype=np.uint16)
    as_f32 = every.view(np.float16).astype(np.float32)
    ours = np.array([oracle.f16_bits_to_f32(int(b)) for b in every[::7]], dtype=np.float32)
    finite = ~np.isnan(as_f32[::7])  # NaN payloads do not survive a float return value
    np.testing.assert_array_equal(ours.view(np.uint32)[finite], as_f32[::7].view(np.uint32)[finite])
    assert np.all(np.isnan(ours[~finite]))
    rng = np.random.default_rng(0)
    samples = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * 100,
        (rng.standard_normal(2000) * 1e-6).astype(np.float32),
        np.array([65504, 65519.99, 65520, 1e9, 2**-25, np.nextafter(np.float32(2**-25), 1),
                  2**-24, 1.5 * 2**-24, 2.5 * 2**-24, 0.0, -0.0, 1 + 2**-11, 1 + 3 * 2**-11,
                  6.1e-5, 6.0975e-5], dtype=np.float32)])
    with np.errstate(over="ignore"):
        expected = samples.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16_bits(float(v)) for v in samples], dtype=np.uint16)
    np.testing.assert_array_equal(got, expected)


def test_nibble_order_and_sign(golden):
    case = golden["w4a16_nibble_order"]
    packed = np.zeros((1, 32), dtype=np.uint8)
    packed[0, 0] = case["byte"]
    scale = np.ones((1, 1), dtype=np.float16)
    weight = oracle.w4_dequant(packed, scale)
    assert weight[0, 0] == case["k0"] and weight[0, 1] == case["k1"]
    assert np.all(weight[0, 2:] == 0)


def test_every_byte_unpacks_to_twos_complement_pairs():
    packed = np.arange(256, dtype=np.uint8).reshape(8, 32)
    weight = oracle.w4_dequant(packed, np.ones((8, 1), dtype=np.float16)).reshape(-1)
    for byte in range(256):
        low, high = byte & 15, byte >> 4
        assert weight[2 * byte] == (low if low < 8 else low - 16)
        assert weight[2 * byte + 1] == (high if high < 8 else high - 16)


def test_reference_fixture_golden_bits(golden):
    case = golden["w4a16_linear_fixture"]
    packed = np.arange(96, dtype=np.uint8).reshape(3, 32)
    packed[0, 0] = 0x78
    scale = np.array(case["scale"], dtype=np.float16).reshape(3, 1)
    bias = np.array(case["bias"], dtype=np.float16)
    x = _bits_to_f16([case["input_bits"]] * 128).reshape(2, 64)
    out = oracle.w4a16_linear(x, packed, scale, bias)
    assert out.astype(np.float16).view(np.uint16).reshape(-1).tolist() == case["expected_output_bits"]
    # the values are exact: 0.375, 17, 63
    np.testing.assert_array_equal(out[0], np.array([0.375, 17.0, 63.0], dtype=np.float32))


@pytest.mark.parametrize("with_bias", [True, False])
def test_runtime_smoke_closed_form(golden, with_bias):
    case = golden["w4a16_runtime_smoke"]
    m, n, k = case["m"], case["n"], case["k"]
    packed = np.empty((n, k // 2), dtype=np.uint8)
    packed[0::2] = case["even_row_byte"]
    packed[1::2] = case["odd_row_byte"]
    scale = np.full((n, 1), case["scale"], dtype=np.float16)
    bias = np.arange(n, dtype=np.float16) if with_bias else None
    x = np.ones((m, k), dtype=np.float16)
    out = oracle.w4a16_linear(x, packed, scale, bias)
    expected = np.where(np.arange(n) % 2 == 0, 32.0, -32.0)
    if with_bias:
        expected = expected + np.arange(n)
    np.testing.assert_array_equal(out, np.tile(expected.astype(np.float32), (m, 1)))


def _random_case(rng, m, n, k):
    packed = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    scale = rng.uniform(0.005, 0.02, size=(n, k // 64)).astype(np.float16)
    x = rng.standard_normal((m, k)).astype(np.float16)
    bias = rng.standard_normal(n).astype(np.float16)
    return x, packed, scale, bias


def test_exact_rational_brute_force_on_tiny_shapes():
    """Independent arithmetic: python Fractions over explicitly decoded nibbles.
    Every term x*q*s is exact in binary64 and the sum of <= 128 such terms is
    correct to ~1e-16 relative, so the oracle's float32 result must equal the
    correctly rounded rational sum (up to one double rounding in 1e9 cases)."""
    rng = np.random.default_rng(11)
    x, packed, scale, bias = _random_case(rng, 3, 5, 128)
    out = oracle.w4a16_linear(x, packed, scale, bias)
    for row in range(3):
        for col in range(5):
            total = Fraction(0)
            for inner in range(128):
                byte = int(packed[col, inner // 2])
                nibble = (byte & 15) if inner % 2 == 0 else (byte >> 4)
                q = nibble - 16 if nibble >= 8 else nibble
                total += (Fraction(float(x[row, inner])) * q
                          * Fraction(float(scale[col, inner // 64])))
            total += Fraction(float(bias[col]))
            assert out[row, col] == np.float32(float(total))


@pytest.mark.parametrize("m,n,k", [(1, 1536, 576), (4, 96, 4096), (8, 40, 1024)])
def test_vectorised_fp64_cross_check(m, n, k):
    """A differently-structured computation (dequantise, then BLAS matmul in
    fp64) agrees to 1e-12 relative: catches a wrong group index, a transposed
    operand or a dropped bias."""
    rng = np.random.default_rng(5)
    x, packed, scale, bias = _random_case(rng, m, n, k)
    low = (packed & 15).astype(np.int16)
    high = (packed >> 4).astype(np.int16)
    q = np.stack([low, high], axis=-1).reshape(n, k)
    q = np.where(q >= 8, q - 16, q).astype(np.float64)
    w = q * np.repeat(scale.astype(np.float64), 64, axis=1)
    expected = x.astype(np.float64) @ w.T + bias.astype(np.float64)
    out = oracle.w4a16_linear(x, packed, scale, bias)
    np.testing.assert_allclose(out, expected, rtol=2e-7, atol=1e-7)
    np.testing.assert_array_equal(oracle.w4_dequant(packed, scale), w.astype(np.float32))
    no_bias = oracle.w4a16_linear(x, packed, scale, None)
    np.testing.assert_allclose(no_bias, expected - bias.astype(np.float64), rtol=2e-7, atol=1e-7)


def test_linearity_in_the_activation():
    rng = np.random.default_rng(2)
    x, packed, scale, _ = _random_case(rng, 2, 16, 256)
    doubled = oracle.w4a16_linear((x.astype(np.float32) * 2).astype(np.float16), packed, scale)
    np.testing.assert_array_equal(doubled, 2 * oracle.w4a16_linear(x, packed, scale))


def test_add_and_pointwise():
    left = np.array([[1.0, 2.0], [3.0, 4.0]], dtype=np.float32)
    row = np.array([[10.0, 20.0]], dtype=np.float32)
    np.testing.assert_array_equal(oracle.add(left, row), left + row)
    np.testing.assert_array_equal(oracle.add(left, left), 2 * left)
    x = np.array([-20.0, -1.0, 0.0, 0.5, 3.0, 30.0], dtype=np.float32)
    expected = x.astype(np.float64) / (1.0 + np.exp(-x.astype(np.float64)))
    np.testing.assert_array_equal(oracle.silu(x), expected.astype(np.float32))
    assert oracle.silu(np.zeros(1))[0] == 0.0
    other = np.array([2.0, -3.0, 5.0, 4.0, 0.25, -1.0], dtype=np.float32)
    np.testing.assert_array_equal(oracle.silu_mul(x, other),
                                  (expected * other.astype(np.float64)).astype(np.float32))
    # silu(x) - silu(-x) = x
    np.testing.assert_allclose(oracle.silu(x) - oracle.silu(-x), x, rtol=1e-6, atol=1e-7)
