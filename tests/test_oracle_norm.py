"""Pins the oracle's FP32 row operations (oracle/norm_oracle.c) before any GPU result is compared with them."""
import math

import numpy as np
import pytest

import oracle


def bits(a):
    return np.asarray(a, dtype=np.float32).view(np.uint32)


def test_reference_vector_of_rms_norm_per_head():
    # Qwen35MathTests.cs:10-12: RmsNorm([3,4,-3,-4],[2,.5], eps 0, head width 2) and the zero row
    expected = np.array([1.6970562748, 0.5656854249, -1.6970562748, -0.5656854249])
    for fn in (oracle.rms_norm_serial, oracle.rms_norm, oracle.np_rms_norm):
        got = fn([3, 4, -3, -4], [2, 0.5], 2, 2, 0.0).ravel()
        assert np.abs(got - expected).max() < 1e-6
        assert fn([0, 0], [1, 1], 1, 2, 1e-6).tolist() == [[0.0, 0.0]]


def test_closed_forms():
    # a constant row c: sum/width = c^2 exactly for powers of two, inverse = 1/sqrt(c^2 + eps)
    for width in (1, 17, 128, 129, 4096):
        x = np.full(width, 4.0, dtype=np.float32)
        w = np.arange(width, dtype=np.float32)
        out = oracle.rms_norm(x, w, 1, width, 0.0)[0]
        assert np.array_equal(out, w)                       # 4 * (1/4) * w
    x = np.full(256, 0.5, dtype=np.float32)
    inv = np.float32(1.0) / np.sqrt(np.float32(0.25) + np.float32(0.75))
    assert np.array_equal(oracle.rms_norm(x, np.ones(256, np.float32), 1, 256, 0.75)[0], np.full(256, 0.5 * inv, np.float32))


@pytest.mark.parametrize("width", [1, 17, 127, 128, 129, 255, 257, 513, 5121])
def test_tree_order_matches_the_separate_statement_bit_for_bit(width):
    rng = np.random.default_rng(width)
    # magnitudes spread over 2^-48 .. 2^48 make the sum depend on the order of the additions
    x = (rng.uniform(-1, 1, width) * np.exp2((np.arange(width) % 9 - 4) * 12.0)).astype(np.float32)
    w = rng.uniform(-2, 2, width).astype(np.float32)
    a = oracle.rms_norm(x, w, 1, width, 1e-6)
    b = oracle.np_rms_norm(x, w, 1, width, 1e-6)
    assert np.array_equal(bits(a), bits(b))
    if width == 5121:
        # and the order matters on these inputs: the serial sum gives different bits somewhere
        assert not np.array_equal(bits(a), bits(oracle.rms_norm_serial(x, w, 1, width, 1e-6)))


def test_stride_rows_and_float64():
    rng = np.random.default_rng(5)
    rows, width, stride = 5, 273, 290
    x = rng.uniform(-2, 2, rows * stride).astype(np.float32)
    w = rng.uniform(-2, 2, width).astype(np.float32)
    got = oracle.rms_norm(x, w, rows, width, 1e-5, stride)
    assert np.array_equal(bits(got), bits(oracle.np_rms_norm(x, w, rows, width, 1e-5, stride)))
    xr = x.reshape(rows, stride)[:, :width].astype(np.float64)
    want = xr / np.sqrt((xr * xr).mean(axis=1, keepdims=True) + 1e-5) * w
    assert np.abs(got - want).max() < 2e-5                  # the reference's GPU-vs-CPU bound


def test_add_rms_norm_is_add_then_norm():
    rng = np.random.default_rng(6)
    width = 5120
    h = rng.standard_normal(width).astype(np.float32)
    r = rng.standard_normal(width).astype(np.float32)
    w = rng.uniform(-2, 2, width).astype(np.float32)
    summed, normed = oracle.add_rms_norm(h, r, w, 1, width, 1e-6)
    assert np.array_equal(bits(summed), bits(h + r))
    assert np.array_equal(bits(normed), bits(oracle.rms_norm(h + r, w, 1, width, 1e-6)))
    assert np.array_equal(bits(oracle.add_in_place(h, r)), bits(h + r))


def test_silu_limits_and_float64():
    # Qwen35MathTests.cs:29-37: sigmoid(100) == 1, sigmoid(-100) in (0, 1e-40], silu(0) == 0
    one = np.ones(3, dtype=np.float32)
    out = oracle.silu_multiply(np.array([100.0, -100.0, 0.0], np.float32), one)
    assert out[0] == np.float32(100.0)
    assert -1e-38 <= out[1] <= 0.0 and math.isfinite(out[1])
    assert out[2] == 0.0
    rng = np.random.default_rng(7)
    g = rng.uniform(-30, 30, 4096).astype(np.float32)
    u = rng.uniform(-2, 2, 4096).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    got = oracle.silu_multiply(g, u)
    assert np.abs(got - want).max() <= 2e-5
    assert (np.abs(got - want) / np.maximum(np.abs(want), 1e-30)).max() < 1e-6


def _round_to_f32(q):
    """Correctly rounded (nearest, ties to even) float32 of a fractions.Fraction, via integer arithmetic only."""
    from fractions import Fraction
    if q == 0:
        return np.float32(0.0)
    sign = -1 if q < 0 else 1
    q = abs(q)
    e = q.numerator.bit_length() - q.denominator.bit_length()
    if Fraction(2) ** e > q:
        e -= 1                                        # 2^e <= q < 2^(e+1)
    e = max(e, -126)                                  # subnormal range keeps the exponent of 2^-126
    scaled = q / Fraction(2) ** (e - 23)              # mantissa units
    n, rem = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * rem
    if twice > scaled.denominator or (twice == scaled.denominator and n % 2 == 1):
        n += 1
    return np.float32(sign * float(Fraction(n) * Fraction(2) ** (e - 23)))


def _fma32(a, b, c):
    from fractions import Fraction
    return _round_to_f32(Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c)))


def test_lora_halves_against_exact_rational_arithmetic():
    rng = np.random.default_rng(12)
    rows, width, rank, output = 2, 300, 3, 5
    x = rng.uniform(-0.4, 0.4, rows * width).astype(np.float32)
    a = rng.uniform(-0.4, 0.4, rank * width).astype(np.float32)
    z = oracle.lora_a(x, a, rows, width, rank)
    for t in range(rows):
        for r in range(rank):
            partial = []
            for lane in range(128):
                s = np.float32(0.0)
                for j in range(lane, width, 128):
                    s = _fma32(x[t * width + j], a[r * width + j], s)
                partial.append(s)
            stride = 64
            while stride:
                for lane in range(stride):
                    partial[lane] = np.float32(partial[lane] + partial[lane + stride])
                stride >>= 1
            assert bits(z[t, r]) == bits(partial[0])
    b = rng.uniform(-0.4, 0.4, output * rank).astype(np.float32)
    y = rng.uniform(-1, 1, rows * output).astype(np.float32)
    for scale in (2.0, -0.75, 0.0):
        got = oracle.lora_b(z, b, y, rows, output, rank, scale)
        for t in range(rows):
            for o in range(output):
                s = np.float32(0.0)
                for r in range(rank):
                    s = _fma32(z[t, r], b[o * rank + r], s)
                want = np.float32(y[t * output + o] + np.float32(np.float32(scale) * s))
                assert bits(got[t, o]) == bits(want)
    # and against float64
    z64 = x.reshape(rows, width).astype(np.float64) @ a.reshape(rank, width).astype(np.float64).T
    assert np.abs(z - z64).max() < 1e-5
