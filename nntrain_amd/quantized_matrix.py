"""HipQuantizedMatrix: an immutable GGUF block-quantized matrix that stays encoded in HBM.

Constructor checks, error kinds and `forward` semantics follow ArcQuantizedMatrix
(NNtrain.Core/Serialization/ArcQuantizedMatrix.cs:16-60) and Qwen35QuantizedModel.Matrix.Forward
(NNtrain.Core/Modules/Qwen35QuantizedModel.cs:1210-1369), extended from Q4_K/Q6_K to the seven storage types of this path (six block formats and bfloat16).
Exceptions map as: NotSupportedException -> NotImplementedError, ArgumentOutOfRangeException/ArgumentException ->
ValueError, InvalidDataException -> ValueError("... payload ...").
"""
from __future__ import annotations

import ctypes
from ctypes import c_void_p

import numpy as np

from . import native
from .lane import HipBuffer, HipExecutionLane
from .native import PRE_NONE, PRE_RMS_NORM, PRE_SILU_MULTIPLY, FusedMatvecDesc, check  # noqa: F401

GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_IQ3_S, GGML_IQ2_S, GGML_BF16 = 8, 12, 13, 14, 21, 22, 30
BLOCK_ELEMS = {GGML_Q8_0: 32, GGML_Q4_K: 256, GGML_Q5_K: 256, GGML_Q6_K: 256, GGML_IQ3_S: 256, GGML_IQ2_S: 256,
               GGML_BF16: 1}
BLOCK_BYTES = {GGML_Q8_0: 34, GGML_Q4_K: 144, GGML_Q5_K: 176, GGML_Q6_K: 210, GGML_IQ3_S: 110, GGML_IQ2_S: 82,
               GGML_BF16: 2}

# rows at or above which forward() uses the bf16 MFMA mat-mul when asked to (Qwen35QuantizedModel.cs:1249: rows >= 16)
PREFILL_MIN_ROWS = 16


class HipQuantizedMatrix:
    def __init__(self, payload, ggml_type: int, output_width: int, input_width: int,
                 inference_matmul_prefill: "bool | str" = False):
        if payload is None:
            raise TypeError("payload is null")
        if ggml_type not in BLOCK_ELEMS:
            raise NotImplementedError(f"GGML type {ggml_type} is not a supported quantized matrix type.")
        if output_width <= 0 or input_width <= 0:
            raise ValueError("outputWidth and inputWidth must be positive.")
        elems = BLOCK_ELEMS[ggml_type]
        if input_width % elems != 0:
            raise NotImplementedError(f"Quantized rows must contain complete {elems}-value blocks.")
        data = np.ascontiguousarray(np.frombuffer(payload, dtype=np.uint8) if isinstance(payload, (bytes, bytearray, memoryview))
                                    else payload)
        if data.dtype != np.uint8:
            raise TypeError("payload must be raw bytes")
        expected = output_width * (input_width // elems) * BLOCK_BYTES[ggml_type]
        if data.size != expected:
            raise ValueError(f"Quantized matrix payload has {data.size} bytes; expected {expected}.")
        self._payload = data
        self.ggml_type = ggml_type
        self.output_width = output_width
        self.input_width = input_width
        # Matrix takes inferenceXmxPrefill from the execution options (Qwen35QuantizedModel.cs:252); off unless asked for
        # (Qwen35ExecutionOptions.InferenceXmxPrefill, Qwen35ExecutionOptions.cs:50), because that route rounds to bfloat16.
        # "split": the three-product form (both operands as two bfloat16 parts), which meets the 5e-5 the reference tests its
        # XMX prefill at (Qwen35XmxPrefillLinearTests.cs:87-89); True: one bfloat16 rounding of each operand (2e-3), a third
        # of the cost.
        if inference_matmul_prefill not in (False, True, "split"):
            raise ValueError("inference_matmul_prefill must be False, True or 'split'.")
        self.inference_matmul_prefill = inference_matmul_prefill
        self._lane: HipExecutionLane | None = None
        self._device_payload: HipBuffer | None = None

    @classmethod
    def from_device(cls, lane: HipExecutionLane, buffer: HipBuffer, ggml_type: int, output_width: int,
                    input_width: int) -> "HipQuantizedMatrix":
        """A matrix whose raw blocks are already in `buffer` on `lane` (streamed there piece by piece); the matrix
        takes ownership of the buffer and is bound to that lane, like one whose host payload was dropped."""
        if ggml_type not in BLOCK_ELEMS:
            raise NotImplementedError(f"GGML type {ggml_type} is not a supported quantized matrix type.")
        if output_width <= 0 or input_width <= 0:
            raise ValueError("outputWidth and inputWidth must be positive.")
        elems = BLOCK_ELEMS[ggml_type]
        if input_width % elems != 0:
            raise NotImplementedError(f"Quantized rows must contain complete {elems}-value blocks.")
        expected = output_width * (input_width // elems) * BLOCK_BYTES[ggml_type]
        if buffer.nbytes < expected:
            raise ValueError(f"Quantized matrix payload has {buffer.nbytes} bytes; expected {expected}.")
        self = cls.__new__(cls)
        self._payload = None
        self._storage_bytes = expected
        self.ggml_type = ggml_type
        self.output_width = output_width
        self.input_width = input_width
        self.inference_matmul_prefill = False
        self._lane = lane
        self._device_payload = buffer
        return self

    @classmethod
    def stacked(cls, lane: HipExecutionLane, matrices) -> "HipQuantizedMatrix":
        """One device matrix holding the rows of `matrices` one after the other (same storage type and input width):
        projections that consume the same vector, such as the gate and up matrices of a feed-forward block
        (Qwen35QuantizedModel.cs:488-489), then cost one launch, and row i of matrix k is output row offset_k + i with
        the bits it has alone.  Raw blocks are copied device to device; the inputs stay usable."""
        matrices = list(matrices)
        if not matrices:
            raise ValueError("no matrices to stack")
        first = matrices[0]
        if any(m.ggml_type != first.ggml_type or m.input_width != first.input_width for m in matrices):
            raise ValueError("stacked matrices must share the storage type and the input width")
        total = sum(m.storage_bytes for m in matrices)
        buffer = lane.allocate_bytes(total)
        try:
            offset = 0
            for m in matrices:
                lane.copy(buffer, m.device_payload(lane), m.storage_bytes, dst_offset=offset)
                offset += m.storage_bytes
        except BaseException:
            buffer.dispose()
            raise
        return cls.from_device(lane, buffer, first.ggml_type, sum(m.output_width for m in matrices), first.input_width)

    @property
    def storage_bytes(self) -> int:
        return int(self._payload.size) if self._payload is not None else self._storage_bytes

    def device_payload(self, lane: HipExecutionLane) -> HipBuffer:
        """Lazy one-time upload of the raw blocks (ArcQuantizedMatrix.DevicePayload, :80-88)."""
        if self._device_payload is not None and self._lane is lane:
            return self._device_payload
        if self._payload is None:
            raise ValueError("host payload was dropped; the matrix is bound to its first lane")
        if self._device_payload is not None:
            self._device_payload.dispose()
        self._device_payload = lane.upload_raw(self._payload)
        self._lane = lane
        return self._device_payload

    def drop_host_payload(self) -> None:
        """Keep only the device copy, as Qwen35QuantizedModel.LoadTensor does (Qwen35QuantizedModel.cs:239-241)."""
        if self._device_payload is None:
            raise ValueError("upload first")
        self._storage_bytes = int(self._payload.size)
        self._payload = None

    def uses_prefill(self, rows: int) -> bool:
        """Whether forward() sends `rows` input rows to the bfloat16 matrix-core mat-mul: only when the matrix was
        given inference_matmul_prefill (the reference's opt-in InferenceXmxPrefill), for rows >= 16 as in Matrix.Forward
        (Qwen35QuantizedModel.cs:1249) and rows of whole 256-weight blocks; the FP32-grade mat-vec kernels otherwise."""
        return bool(self.inference_matmul_prefill) and rows >= PREFILL_MIN_ROWS and self.input_width % 256 == 0

    def forward(self, lane: HipExecutionLane, x: HipBuffer, bias: HipBuffer | None, rows: int = 1,
                out: HipBuffer | None = None) -> HipBuffer:
        """y[rows, out] = bias + x[rows, in] . W^T on the device; x is FP32.  The caller disposes the result.
        Every row count goes to the dequantization-fused mat-vec (FP32 accumulation, 1e-5 of the float64 product; up to
        four input rows share a pass over the weights on the large matrices).  With inference_matmul_prefill set, rows
        >= 16 go to the bfloat16 matrix-core mat-mul instead (activations and weights rounded to bfloat16 once: 2e-3),
        the counterpart of the reference's opt-in XMX prefill (Qwen35QuantizedModel.cs:1249-1317); that path's own bound is
        5e-5 because it splits its operands into two f16 parts, which inference_matmul_prefill="split" does with bfloat16
        parts (three products, about 3e-6)."""
        if rows < 1:
            raise ValueError("rows must be positive.")
        if x.nbytes < 4 * rows * self.input_width:
            raise ValueError("Quantized linear input width mismatch.")
        if bias is not None and bias.nbytes < 4 * self.output_width:
            raise ValueError("Quantized linear bias width mismatch.")
        w = self.device_payload(lane)
        if out is not None and out.nbytes < 4 * rows * self.output_width:
            raise ValueError("output buffer too small")
        y = out if out is not None else lane.allocate(rows * self.output_width)
        if not self.uses_prefill(rows):
            entry, fn = "quant_matvec", lane._lib.nnhip_quant_matvec
        elif self.inference_matmul_prefill == "split":
            entry, fn = "quant_matmul_split", lane._lib.nnhip_quant_matmul_split
        else:
            entry, fn = "quant_matmul", lane._lib.nnhip_quant_matmul
        try:
            with lane.kernel(entry):
                check(fn(lane._handle, self.ggml_type, c_void_p(x._require()), c_void_p(w._require()),
                         c_void_p(bias._require()) if bias is not None else None, c_void_p(y._require()), rows,
                         self.input_width, self.output_width), entry)
        except BaseException:
            if out is None:
                y.dispose()
            raise
        return y

    def fused_descriptor(self, lane: HipExecutionLane, x: HipBuffer, *, pre_op: int = PRE_NONE, x2: HipBuffer | None = None,
                         norm_weight: HipBuffer | None = None, epsilon: float = 0.0, x_out: HipBuffer | None = None,
                         sum_out: HipBuffer | None = None, bias: HipBuffer | None = None, addend: HipBuffer | None = None,
                         out: HipBuffer, lora_z: HipBuffer | None = None, lora_b: HipBuffer | None = None,
                         lora_rank: int = 0, lora_scale: float = 0.0, x_head_width: int = 0,
                         x_head_group: int = 0, post_op: int = 0) -> FusedMatvecDesc:
        """The native descriptor of forward_fused with these arguments."""
        if lora_rank < 0:
            raise ValueError("lora_rank must not be negative.")
        if lora_rank > 0 and (lora_z is None or lora_b is None or lora_z.nbytes < 4 * lora_rank
                              or lora_b.nbytes < 4 * lora_rank * self.output_width):
            raise ValueError("LoRA buffers do not match lora_rank.")
        n_in, n_out = 4 * self.input_width, 4 * self.output_width
        n_y = n_out // 2 if post_op else n_out
        n_x = n_in // x_head_group if x_head_group > 0 else n_in
        for name, buf, need in (("x", x, n_x), ("x2", x2, n_in), ("norm_weight", norm_weight, n_in), ("x_out", x_out, n_in),
                                ("sum_out", sum_out, n_in), ("bias", bias, n_out), ("addend", addend, n_out), ("out", out, n_y)):
            if buf is not None and buf.nbytes < need:
                raise ValueError(f"Quantized linear '{name}' width mismatch.")
        w = self.device_payload(lane)
        ptr = lambda b: c_void_p(b._require()) if b is not None else None   # noqa: E731
        return FusedMatvecDesc(struct_size=ctypes.sizeof(FusedMatvecDesc), ggml_type=self.ggml_type, pre_op=pre_op,
                               epsilon=epsilon, x=ptr(x), x2=ptr(x2), norm_weight=ptr(norm_weight), x_out=ptr(x_out),
                               sum_out=ptr(sum_out), w=ptr(w), bias=ptr(bias), addend=ptr(addend), y=ptr(out),
                               in_w=self.input_width, out_w=self.output_width, lora_z=ptr(lora_z), lora_b=ptr(lora_b),
                               lora_rank=lora_rank, lora_scale=lora_scale, x_head_width=x_head_width,
                               x_head_group=x_head_group, post_op=post_op)

    def forward_fused(self, lane: HipExecutionLane, x: HipBuffer, *, pre_op: int = PRE_NONE, x2: HipBuffer | None = None,
                      norm_weight: HipBuffer | None = None, epsilon: float = 0.0, x_out: HipBuffer | None = None,
                      sum_out: HipBuffer | None = None, bias: HipBuffer | None = None, addend: HipBuffer | None = None,
                      out: HipBuffer | None = None, lora_z: HipBuffer | None = None, lora_b: HipBuffer | None = None,
                      lora_rank: int = 0, lora_scale: float = 0.0, x_head_width: int = 0, x_head_group: int = 0,
                      post_op: int = 0) -> HipBuffer:
        """One decode mat-vec with its neighbours fused into the launch: v = RMSNorm(x + x2) * norm_weight
        (PRE_RMS_NORM; x2 optional) or SiLU(x) * x2 (PRE_SILU_MULTIPLY) or x, then y = addend + bias + W v.
        x_out / sum_out receive v and x + x2 when given.  `out` may be `addend` (the residual stream updated in place).
        lora_z [rank] and lora_b [out, rank] add the low-rank adapter branch lora_scale * z . b^T before the addend
        (Matrix.ForwardFusedLora, Qwen35QuantizedModel.cs:1387).  x_head_width / x_head_group: x holds key/value heads and
        is gathered first, v[h * width + j] = x[(h // group) * width + j] (what first-token attention hands the o
        projection).  post_op POST_SILU_PAIR: the matrix stacks gate | up and `out` receives output_width / 2 values,
        SiLU(gate) * up."""
        n_y = self.output_width // 2 if post_op else self.output_width
        if out is not None and out.nbytes < 4 * n_y:
            raise ValueError("Quantized linear 'out' width mismatch.")
        y = out if out is not None else lane.allocate(n_y)
        try:
            desc = self.fused_descriptor(lane, x, pre_op=pre_op, x2=x2, norm_weight=norm_weight, epsilon=epsilon, x_out=x_out,
                                         sum_out=sum_out, bias=bias, addend=addend, out=y, lora_z=lora_z, lora_b=lora_b,
                                         lora_rank=lora_rank, lora_scale=lora_scale, x_head_width=x_head_width,
                                         x_head_group=x_head_group, post_op=post_op)
            with lane.kernel("quant_matvec_fused"):
                check(lane._lib.nnhip_quant_matvec_fused(lane._handle, ctypes.byref(desc)), "quant_matvec_fused")
        except BaseException:
            if out is None:
                y.dispose()
            raise
        return y

    def forward_bf16(self, lane: HipExecutionLane, x_bf16: HipBuffer, bias: HipBuffer | None, rows: int,
                     out: HipBuffer | None = None) -> HipBuffer:
        """Prefill: x holds bfloat16 bit patterns [rows, in]; bf16 MFMA with FP32 accumulation.  Every storage
        type with in_w a multiple of 256."""
        if rows < 1:
            raise ValueError("rows must be positive.")
        if x_bf16.nbytes < 2 * rows * self.input_width:
            raise ValueError("Quantized linear input width mismatch.")
        if bias is not None and bias.nbytes < 4 * self.output_width:
            raise ValueError("Quantized linear bias width mismatch.")
        w = self.device_payload(lane)
        if out is not None and out.nbytes < 4 * rows * self.output_width:
            raise ValueError("output buffer too small")
        y = out if out is not None else lane.allocate(rows * self.output_width)
        try:
            with lane.kernel("quant_matmul_bf16"):
                check(lane._lib.nnhip_quant_matmul_bf16(lane._handle, self.ggml_type, c_void_p(x_bf16._require()),
                                                        c_void_p(w._require()),
                                                        c_void_p(bias._require()) if bias is not None else None,
                                                        c_void_p(y._require()), rows, self.input_width, self.output_width),
                      "quant_matmul_bf16")
        except BaseException:
            if out is None:
                y.dispose()
            raise
        return y

    def dequantize(self, lane: HipExecutionLane, row: int | None = None, out: HipBuffer | None = None) -> HipBuffer:
        """Decode the whole matrix, or one row (the embedding lookup of Matrix.Embedding,
        Qwen35QuantizedModel.cs:1497-1521), to FP32 on the device."""
        w = self.device_payload(lane)
        row_bytes = self.input_width // BLOCK_ELEMS[self.ggml_type] * BLOCK_BYTES[self.ggml_type]
        if row is None:
            elements, offset = self.output_width * self.input_width, 0
        else:
            if not 0 <= row < self.output_width:
                raise IndexError(f"Embedding index {row} is outside the vocabulary.")
            elements, offset = self.input_width, row * row_bytes
        out = lane.allocate(elements) if out is None else out
        if out.nbytes < 4 * elements:
            raise ValueError("output buffer too small")
        with lane.kernel("dequantize"):
            check(lane._lib.nnhip_dequantize(lane._handle, self.ggml_type, c_void_p(w._require() + offset),
                                             c_void_p(out._require()), elements), "dequantize")
        return out

    def dispose(self) -> None:
        if self._device_payload is not None:
            self._device_payload.dispose()
        self._device_payload = None
        self._lane = None
