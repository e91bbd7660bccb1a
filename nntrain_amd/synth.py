"""Seeded synthetic GGUF block payloads and activations for the benchmark configurations.

Shapes, distributions and seeds are those the benchmark is quoted on: Q8_0 from w ~ N(0, 0.02) quantised the way
ggml's quantize_row_q8_0 does (d = max|w|/127 stored as fp16, q = round(w/d)); K-quant and IQ2_S super-blocks with
fp16 scales from |N(0, 0.01)| and uniformly random packed fields.  NumPy PCG64 only, so every run and every machine
sees the same bytes.
"""
from __future__ import annotations

import ctypes
from ctypes import c_void_p
from pathlib import Path

import numpy as np

from .quantized_matrix import (BLOCK_BYTES, BLOCK_ELEMS, GGML_BF16, GGML_IQ2_S, GGML_IQ3_S, GGML_Q4_K, GGML_Q5_K,
                               GGML_Q6_K, GGML_Q8_0)


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def quantize_q8_0(w: np.ndarray) -> np.ndarray:
    """FP32 [..., 32k] -> raw Q8_0 bytes (34 per 32 values)."""
    w = np.ascontiguousarray(w, dtype=np.float32).reshape(-1, 32)
    amax = np.max(np.abs(w), axis=1)
    d = (amax / np.float32(127)).astype(np.float32)
    inv = np.where(d > 0, np.float32(1) / np.where(d > 0, d, np.float32(1)), np.float32(0)).astype(np.float32)
    v = w * inv[:, None]
    q = np.trunc(v + np.copysign(np.float32(0.5), v)).astype(np.int32)  # roundf: halves away from zero
    q = np.clip(q, -127, 127).astype(np.int8)
    out = np.empty((w.shape[0], 34), dtype=np.uint8)
    out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


def q8_0_matrix(out_w: int, in_w: int, seed: int, sigma: float = 0.02, chunk_rows: int = 2048) -> np.ndarray:
    rng = _rng(seed)
    parts = []
    for r0 in range(0, out_w, chunk_rows):
        n = min(chunk_rows, out_w - r0)
        w = rng.standard_normal((n, in_w), dtype=np.float32) * np.float32(sigma)
        parts.append(quantize_q8_0(w))
    return np.concatenate(parts)


def _half_abs_normal(rng, n: int, sigma: float) -> np.ndarray:
    return np.abs(rng.standard_normal(n, dtype=np.float32) * np.float32(sigma)).astype(np.float16).view(np.uint8).reshape(n, 2)


def k_quant_matrix(ggml_type: int, out_w: int, in_w: int, seed: int, sigma: float = 0.01) -> np.ndarray:
    """Random Q4_K / Q5_K / Q6_K / IQ2_S / IQ3_S payload: fp16 scales from |N(0, sigma)|, every packed field uniform."""
    rng = _rng(seed)
    bb = BLOCK_BYTES[ggml_type]
    n = out_w * (in_w // BLOCK_ELEMS[ggml_type])
    blocks = rng.integers(0, 256, size=(n, bb), dtype=np.uint8)
    if ggml_type in (GGML_Q4_K, GGML_Q5_K):
        blocks[:, 0:2] = _half_abs_normal(rng, n, sigma)
        blocks[:, 2:4] = _half_abs_normal(rng, n, sigma)
    elif ggml_type == GGML_Q6_K:
        blocks[:, 208:210] = _half_abs_normal(rng, n, sigma)
    elif ggml_type in (GGML_IQ2_S, GGML_IQ3_S):
        blocks[:, 0:2] = _half_abs_normal(rng, n, sigma)
    else:
        raise ValueError("not a super-block type")
    return blocks.reshape(-1)


def bf16_matrix(out_w: int, in_w: int, seed: int, sigma: float = 0.02) -> np.ndarray:
    """bfloat16 weights N(0, sigma), as raw bytes."""
    w = _rng(seed).standard_normal((out_w, in_w), dtype=np.float32) * np.float32(sigma)
    return to_bf16_bits(w).reshape(-1).view(np.uint8)


def matrix(ggml_type: int, out_w: int, in_w: int, seed: int) -> np.ndarray:
    if ggml_type == GGML_BF16:
        return bf16_matrix(out_w, in_w, seed)
    if ggml_type == GGML_Q8_0:
        return q8_0_matrix(out_w, in_w, seed)
    return k_quant_matrix(ggml_type, out_w, in_w, seed)


def activations(rows: int, in_w: int, seed: int) -> np.ndarray:
    return _rng(seed).standard_normal((rows, in_w), dtype=np.float32)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + np.uint32(0x7FFF)
    return ((u + r) >> 16).astype(np.uint16)


class DeviceSynth:
    """Draws synthetic Q8_0 blocks and N(0, 1) activations on the device (libnnhip_synth.so): the 27B-shape decode set
    is 28.7 GB of random-init weights, far quicker to generate in HBM than to upload."""

    def __init__(self):
        path = Path(__file__).resolve().parent / "csrc" / "libnnhip_synth.so"
        if not path.exists():
            raise FileNotFoundError(f"{path} is missing: build it with `make -C nntrain_amd/csrc`")
        self.lib = ctypes.CDLL(str(path))
        self.lib.nnhip_synth_q8_0.argtypes = [c_void_p, c_void_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_float]
        self.lib.nnhip_synth_normal_f32.argtypes = [c_void_p, c_void_p, ctypes.c_uint64, ctypes.c_uint64]

    @staticmethod
    def _stream(lane) -> c_void_p:
        s = c_void_p()
        lane._lib.nnhip_lane_stream(lane._handle, ctypes.byref(s))
        return s

    def q8_0(self, lane, buf, blocks: int, seed: int, sigma: float = 0.02) -> None:
        rc = self.lib.nnhip_synth_q8_0(self._stream(lane), c_void_p(buf.ptr), blocks, seed, sigma)
        if rc:
            raise RuntimeError(f"nnhip_synth_q8_0 failed ({rc})")

    def normal(self, lane, buf, count: int, seed: int) -> None:
        rc = self.lib.nnhip_synth_normal_f32(self._stream(lane), c_void_p(buf.ptr), count, seed)
        if rc:
            raise RuntimeError(f"nnhip_synth_normal_f32 failed ({rc})")


def decode27b_tensors():
    """(name, out_w, in_w) of every mat-vec of one token of a Gemma-3-27B-shaped stack: hidden 5376, 32 query and 16
    key/value heads of 128, feed-forward 21504, vocabulary 262144, 62 layers: 435 matrices, 28,695,625,728 Q8_0 bytes."""
    hidden, q_out, kv_out, ffn, vocab, layers = 5376, 32 * 128, 16 * 128, 21504, 262144, 62
    per_layer = [("attn_q", q_out, hidden), ("attn_k", kv_out, hidden), ("attn_v", kv_out, hidden),
                 ("attn_o", hidden, q_out), ("ffn_gate", ffn, hidden), ("ffn_up", ffn, hidden),
                 ("ffn_down", hidden, ffn)]
    out = []
    for layer in range(layers):
        out += [(f"blk.{layer}.{n}", o, i) for n, o, i in per_layer]
    out.append(("output", vocab, hidden))
    return out
