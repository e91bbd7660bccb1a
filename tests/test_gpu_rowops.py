"""GPU parity of the FP32 row operations around the mat-vec (RMSNorm, add + RMSNorm, SiLU * up, add), through the
C ABI, against the CPU oracle.

Bars: RMSNorm and add + RMSNorm bit-exact (same summation order, IEEE division and square root), on the widths,
strides and row counts of the reference's own exactness test (NNtrain.Core.Tests/Qwen35ExactRmsNormTests.cs:16-19)
with its input recipe (zero rows of both signs, magnitudes 2^-48 .. 2^48, subnormals, negative-zero weights, NaN
guards past the end).  SiLU * up within 2e-5 absolute (the reference's bound, Qwen35GpuAttentionTests.cs:26-28) and
1e-6 relative: exp is a library routine on both sides.
"""
import numpy as np
import pytest

import oracle
from nntrain_amd import HipExecutionLane, NnHipError, qwen35_gpu

pytestmark = pytest.mark.gpu

GUARD = 13


@pytest.fixture(scope="module")
def lane():
    with HipExecutionLane(0) as ln:
        yield ln


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _exactness_inputs(width, stride, rows):
    rng = np.random.default_rng(width * 31 + rows * 17 + stride)
    x = np.full(rows * stride + GUARD, np.nan, dtype=np.float32)
    for r in range(rows):
        col = np.arange(width)
        if r == 1:
            v = np.where(col % 2 == 0, np.float32(0.0), np.float32(-0.0)).astype(np.float32)
        else:
            v = (rng.uniform(-1, 1, width) * np.exp2((col % 9 - 4) * 12.0)).astype(np.float32)
            tiny = np.where(col % 2 == 0, np.float32(1e-45), np.float32(-1e-45)).astype(np.float32)
            v = np.where(col % 31 == 0, tiny, v)
        x[r * stride:r * stride + width] = v
    w = rng.uniform(-2, 2, width).astype(np.float32)
    w[::17] = np.float32(-0.0)
    return x, w


@pytest.mark.parametrize("width", [1, 17, 127, 128, 129, 255, 256, 257, 513, 4096, 5120, 5121, 6144, 17408])
def test_rms_norm_bits_for_model_widths_heads_and_odd_tails(lane, width):
    for padding in (0, 17):
        for rows in (1, 5):
            stride = width + padding
            eps = 1e-6 if width % 2 == 0 else 1e-5
            x, w = _exactness_inputs(width, stride, rows)
            xb, wb = lane.upload_raw(x), lane.upload_raw(w)
            h2d, d2h = lane.counters()["h2d_bytes"], lane.counters()["d2h_bytes"]
            ob = qwen35_gpu.rms_norm(lane, xb, wb, rows, width, eps, stride)
            assert (lane.counters()["h2d_bytes"], lane.counters()["d2h_bytes"]) == (h2d, d2h)
            got = lane.read(ob, count=rows * width)
            want = oracle.rms_norm(x, w, rows, width, eps, stride).ravel()
            assert np.all(np.isfinite(got))
            assert np.array_equal(_bits(got), _bits(want)), f"width={width} stride={stride} rows={rows}"
            assert np.array_equal(_bits(lane.read(xb, count=x.size)), _bits(x))       # the input is not touched
            assert np.array_equal(_bits(lane.read(wb, count=w.size)), _bits(w))
            for b in (xb, wb, ob):
                b.dispose()


@pytest.mark.parametrize("width", [1, 129, 2048, 5120, 5376])
def test_add_rms_norm_updates_the_residual_stream_and_normalizes(lane, width):
    rng = np.random.default_rng(width)
    hidden = rng.standard_normal(width).astype(np.float32) * np.float32(3)
    residual = rng.standard_normal(width).astype(np.float32)
    weight = rng.uniform(-2, 2, width).astype(np.float32)
    hb, rb, wb = lane.upload_raw(hidden), lane.upload_raw(residual), lane.upload_raw(weight)
    ob = qwen35_gpu.add_residual_and_rms_norm(lane, hb, rb, wb, width, 1e-6)
    want_hidden, want_norm = oracle.add_rms_norm(hidden, residual, weight, 1, width, 1e-6)
    assert np.array_equal(_bits(lane.read(hb, count=width)), _bits(want_hidden))
    assert np.array_equal(_bits(lane.read(ob, count=width)), _bits(want_norm.ravel()))
    assert np.array_equal(_bits(lane.read(rb, count=width)), _bits(residual))
    for b in (hb, rb, wb, ob):
        b.dispose()


def test_norm_activation_and_residual_match_cpu_without_host_transfers(lane):
    # the composition of Qwen35GpuAttentionTests.cs:10-30: rows 3, width 273, gate values that overflow a naive sigmoid
    rows, width = 3, 273
    rng = np.random.default_rng(1)
    x = rng.uniform(-2, 2, rows * width).astype(np.float32)
    w = rng.uniform(-2, 2, width).astype(np.float32)
    up = rng.uniform(-2, 2, rows * width).astype(np.float32)
    x[0], x[1] = -100.0, 100.0
    xb, wb, ub = lane.upload_raw(x), lane.upload_raw(w), lane.upload_raw(up)
    before = lane.counters()
    normalized = qwen35_gpu.rms_norm(lane, xb, wb, rows, width, 1e-5)
    activated = qwen35_gpu.silu_multiply(lane, xb, ub, x.size)
    qwen35_gpu.add_in_place(lane, activated, normalized, x.size)
    after = lane.counters()
    assert (after["h2d_bytes"], after["d2h_bytes"]) == (before["h2d_bytes"], before["d2h_bytes"])
    got = lane.read(activated, count=x.size)
    x64 = x.astype(np.float64).reshape(rows, width)
    norm64 = (x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + 1e-5) * w).ravel()
    silu64 = x.astype(np.float64) / (1 + np.exp(-x.astype(np.float64))) * up
    assert np.all(np.isfinite(got))
    assert np.abs(got - (norm64 + silu64)).max() <= 2e-5
    want = oracle.rms_norm(x, w, rows, width, 1e-5).ravel() + oracle.silu_multiply(x, up)
    assert np.abs(got - want).max() <= 2e-5
    assert np.array_equal(_bits(lane.read(xb, count=x.size)), _bits(x))
    for b in (xb, wb, ub, normalized, activated):
        b.dispose()


def test_silu_multiply_and_add_in_place_large(lane):
    rng = np.random.default_rng(9)
    n = 17408
    g = rng.uniform(-30, 30, n).astype(np.float32)
    g[:4] = [100.0, -100.0, 0.0, -0.0]
    u = rng.uniform(-2, 2, n).astype(np.float32)
    gb, ub = lane.upload_raw(g), lane.upload_raw(u)
    ob = qwen35_gpu.silu_multiply(lane, gb, ub, n)
    got = lane.read(ob, count=n)
    want = oracle.silu_multiply(g, u)
    assert np.abs(got - want).max() <= 2e-5
    assert (np.abs(got - want) / np.maximum(np.abs(want), 1e-30)).max() < 1e-6
    assert got[0] == np.float32(100.0) * u[0] and got[2] == 0.0
    qwen35_gpu.add_in_place(lane, ob, gb, n)
    assert np.array_equal(_bits(lane.read(ob, count=n)), _bits(got + g))       # one FP32 addition: exact parity
    for b in (gb, ub, ob):
        b.dispose()


def test_argument_checks(lane):
    b = lane.allocate(16)
    with pytest.raises(ValueError):
        qwen35_gpu.rms_norm(lane, b, b, 0, 16, 1e-6)
    with pytest.raises(ValueError):
        qwen35_gpu.rms_norm(lane, b, b, 1, 16, float("nan"))
    with pytest.raises(ValueError):
        qwen35_gpu.rms_norm(lane, b, b, 1, 16, -1e-6)
    with pytest.raises(ValueError):
        qwen35_gpu.rms_norm(lane, b, b, 2, 16, 1e-6)                  # input too small for two rows
    with pytest.raises(ValueError):
        qwen35_gpu.silu_multiply(lane, b, b, 17)
    with pytest.raises(NnHipError):
        from ctypes import c_void_p
        from nntrain_amd.native import check
        check(lane._lib.nnhip_rms_norm(lane._handle, c_void_p(b.ptr), c_void_p(b.ptr), c_void_p(b.ptr), 1, 16, 8, 1e-6),
              "rms_norm")                                             # stride smaller than width
    b.dispose()
