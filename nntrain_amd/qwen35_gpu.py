"""Resident FP32 row operations of the decode path, shaped like the reference's Qwen35Gpu helpers
(NNtrain.Core/Modules/Qwen35Gpu.Attention.cs:11-58) and AddResidualAndRmsNorm
(NNtrain.Core/Modules/Qwen35QuantizedModel.cs:527-546).  Callers own returned buffers; nothing crosses to the host.
"""
from __future__ import annotations

import math
from ctypes import c_void_p

from .lane import HipBuffer, HipExecutionLane
from .native import check


def _positive(value: int, name: str) -> None:
    if value <= 0:
        raise ValueError(f"{name} must be positive (ArgumentOutOfRangeException in the reference).")


def _validate_epsilon(eps: float) -> None:
    if not math.isfinite(eps) or eps < 0.0:
        raise ValueError("eps must be finite and not negative.")


def _validate_buffer(buffer: HipBuffer, elements: int, name: str) -> None:
    if buffer is None:
        raise TypeError(f"{name} is null.")
    if buffer.disposed or buffer.nbytes < elements * 4:
        raise ValueError(f"The buffer '{name}' is disposed or too small for its declared dimensions.")


def _output(lane: HipExecutionLane, out: HipBuffer | None, elements: int) -> HipBuffer:
    if out is None:
        return lane.allocate(elements)
    _validate_buffer(out, elements, "out")
    return out


def rms_norm(lane: HipExecutionLane, input: HipBuffer, weight: HipBuffer, rows: int, width: int, eps: float,
             input_stride: int | None = None, out: HipBuffer | None = None) -> HipBuffer:
    """Qwen35Gpu.RmsNorm: output[r] = input[r] * inverse_rms(input[r]) * weight."""
    _positive(rows, "rows")
    _positive(width, "width")
    _validate_epsilon(eps)
    stride = width if input_stride is None else input_stride
    if stride < width:
        raise ValueError("input_stride must be at least width.")
    _validate_buffer(input, (rows - 1) * stride + width, "input")
    _validate_buffer(weight, width, "weight")
    output = _output(lane, out, rows * width)
    try:
        with lane.kernel("rms_norm"):
            check(lane._lib.nnhip_rms_norm(lane._handle, c_void_p(input._require()), c_void_p(weight._require()),
                                           c_void_p(output._require()), rows, width, stride, eps), "rms_norm")
        return output
    except BaseException:
        if out is None:
            output.dispose()
        raise


def add_residual_and_rms_norm(lane: HipExecutionLane, hidden: HipBuffer, residual: HipBuffer, weight: HipBuffer,
                              width: int, eps: float, out: HipBuffer | None = None) -> HipBuffer:
    """AddResidualAndRmsNorm (fused form): hidden += residual in place, returns RMSNorm(hidden) * weight."""
    _positive(width, "width")
    _validate_epsilon(eps)
    _validate_buffer(hidden, width, "hidden")
    _validate_buffer(residual, width, "residual")
    _validate_buffer(weight, width, "weight")
    output = _output(lane, out, width)
    try:
        with lane.kernel("add_rms_norm"):
            check(lane._lib.nnhip_add_rms_norm(lane._handle, c_void_p(hidden._require()), c_void_p(residual._require()),
                                               c_void_p(weight._require()), c_void_p(output._require()), 1, width, width,
                                               eps), "add_rms_norm")
        return output
    except BaseException:
        if out is None:
            output.dispose()
        raise


def silu_multiply(lane: HipExecutionLane, gate: HipBuffer, up: HipBuffer, length: int,
                  out: HipBuffer | None = None) -> HipBuffer:
    """Qwen35Gpu.SiluMultiply: gate * sigmoid(gate) * up."""
    _positive(length, "length")
    _validate_buffer(gate, length, "gate")
    _validate_buffer(up, length, "up")
    output = _output(lane, out, length)
    try:
        with lane.kernel("silu_multiply"):
            check(lane._lib.nnhip_silu_multiply(lane._handle, c_void_p(gate._require()), c_void_p(up._require()),
                                                c_void_p(output._require()), length), "silu_multiply")
        return output
    except BaseException:
        if out is None:
            output.dispose()
        raise


def add_in_place(lane: HipExecutionLane, destination: HipBuffer, source: HipBuffer, length: int) -> None:
    """Qwen35Gpu.AddInPlace: destination += source."""
    _positive(length, "length")
    _validate_buffer(destination, length, "destination")
    _validate_buffer(source, length, "source")
    with lane.kernel("add_in_place"):
        check(lane._lib.nnhip_add_in_place(lane._handle, c_void_p(destination._require()), c_void_p(source._require()),
                                           length), "add_in_place")


def lora_project_a(lane: HipExecutionLane, x: HipBuffer, a: HipBuffer, rows: int, width: int, rank: int) -> HipBuffer:
    """z[rows, rank] = x . a^T, the first half of a low-rank adapter (q35l_lora_a_coop)."""
    _positive(rows, "rows")
    _positive(width, "width")
    _positive(rank, "rank")
    _validate_buffer(x, rows * width, "x")
    _validate_buffer(a, rank * width, "a")
    z = lane.allocate(rows * rank)
    try:
        with lane.kernel("lora_a"):
            check(lane._lib.nnhip_lora_a(lane._handle, c_void_p(x._require()), c_void_p(a._require()), c_void_p(z._require()),
                                         rows, width, rank), "lora_a")
        return z
    except BaseException:
        z.dispose()
        raise


def lora_apply_b(lane: HipExecutionLane, z: HipBuffer, b: HipBuffer, y: HipBuffer, rows: int, output: int, rank: int,
                 scale: float) -> None:
    """y[rows, output] += scale * z . b^T, the second half (q35l_lora_b)."""
    _positive(rows, "rows")
    _positive(output, "output")
    _positive(rank, "rank")
    _validate_buffer(z, rows * rank, "z")
    _validate_buffer(b, output * rank, "b")
    _validate_buffer(y, rows * output, "y")
    with lane.kernel("lora_b"):
        check(lane._lib.nnhip_lora_b(lane._handle, c_void_p(z._require()), c_void_p(b._require()), c_void_p(y._require()),
                                     rows, output, rank, scale), "lora_b")


def first_token_attention(lane: HipExecutionLane, value: HipBuffer, heads: int, kv_heads: int, head_width: int,
                          out: HipBuffer | None = None) -> HipBuffer:
    """Causal grouped-query attention for the first token of a sequence: every query head receives its group's value
    head (the single key has softmax weight 1).  The general attention step (Qwen35Gpu.AttentionStep) is not part of
    this library."""
    _positive(heads, "heads")
    _positive(kv_heads, "kv_heads")
    _positive(head_width, "head_width")
    if heads % kv_heads != 0:
        raise ValueError("heads must be a multiple of kv_heads.")
    _validate_buffer(value, kv_heads * head_width, "value")
    output = _output(lane, out, heads * head_width)
    try:
        with lane.kernel("first_token_attention"):
            check(lane._lib.nnhip_first_token_attention(lane._handle, c_void_p(value._require()), c_void_p(output._require()),
                                                        heads, kv_heads, head_width), "first_token_attention")
        return output
    except BaseException:
        if out is None:
            output.dispose()
        raise
