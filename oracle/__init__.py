"""CPU oracle for the GGUF block-quantized linear path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the
product (nntrain_amd and the HIP library) never does.

Two independent statements of the same algorithms live here:
  * libquant_oracle.so (quant_oracle.c) - scalar C, loaded through ctypes; cites the reference per function.
  * the np_dequantize_* functions below - vectorised numpy, written separately from the C so that a slip
    in one (a wrong index, nibble or rounding order) shows up as a disagreement between them as well as
    against the golden vectors.
FP32 rounding order follows the reference's managed decoders (NNtrain.Core/Serialization/GgufQ4K.cs:34-41,
GgufQ6K.cs:45-48) and the device formulas for the fixture-pinned types (NNtrain.Arc/Kernels/qwen35_iq.cl:398-429).
"""
from __future__ import annotations

import ctypes
import re
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent

Q8_0, Q4_K, Q5_K, Q6_K, IQ3_S, IQ2_S, BF16 = 8, 12, 13, 14, 21, 22, 30
BLOCK_ELEMS = {Q8_0: 32, Q4_K: 256, Q5_K: 256, Q6_K: 256, IQ3_S: 256, IQ2_S: 256, BF16: 1}
BLOCK_BYTES = {Q8_0: 34, Q4_K: 144, Q5_K: 176, Q6_K: 210, IQ3_S: 110, IQ2_S: 82, BF16: 2}

_lib = None


def build() -> Path:
    """Compile libquant_oracle.so with the committed Makefile."""
    subprocess.run(["make", "-C", str(HERE), "-B"], check=True, capture_output=True)
    return HERE / "libquant_oracle.so"


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = HERE / "libquant_oracle.so"
        if not path.exists():
            build()
        L = ctypes.CDLL(str(path))
        c_u8p = ctypes.c_void_p
        L.oracle_block_elems.argtypes = [ctypes.c_uint32]
        L.oracle_block_bytes.argtypes = [ctypes.c_uint32]
        L.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_half_to_float.restype = ctypes.c_float
        L.oracle_dequantize.argtypes = [ctypes.c_uint32, c_u8p, ctypes.c_void_p, ctypes.c_int64]
        L.oracle_cpu_linear.argtypes = [ctypes.c_uint32, c_u8p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.oracle_linear_f64.argtypes = [ctypes.c_uint32, c_u8p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_int]
        L.oracle_max_threads.restype = ctypes.c_int
        vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L.oracle_rms_norm.argtypes = [vp, vp, vp, ci, ci, ci, cf]
        L.oracle_add_rms_norm.argtypes = [vp, vp, vp, vp, ci, ci, ci, cf]
        L.oracle_rms_norm_serial.argtypes = [vp, vp, vp, ci, ci, cf]
        L.oracle_silu_multiply.argtypes = [vp, vp, vp, ci]
        L.oracle_add_in_place.argtypes = [vp, vp, ci]
        L.oracle_lora_a.argtypes = [vp, vp, vp, ci, ci, ci]
        L.oracle_lora_b.argtypes = [vp, vp, vp, ci, ci, ci, cf]
        _lib = L
    return _lib


_native = None


def native_lib():
    """The same sources compiled for the host this process runs on (-march=native), for timing the CPU path where it
    runs; the committed library is built for x86-64-v3 so that it loads anywhere.  Returns (library, build flags);
    falls back to the committed library when no compiler is at hand."""
    global _native
    if _native is None:
        import tempfile
        flags = "-O3 -march=native -ffp-contract=off -fno-fast-math -fopenmp -fPIC"
        out = Path(tempfile.gettempdir()) / f"libquant_oracle_native_{os.getpid()}.so"
        try:
            subprocess.run(["gcc", *flags.split(), "-shared", "-o", str(out), str(HERE / "quant_oracle.c"),
                            str(HERE / "norm_oracle.c"), "-lm"], check=True, capture_output=True)
            L = ctypes.CDLL(str(out))
            L.oracle_cpu_linear.argtypes = lib().oracle_cpu_linear.argtypes
            _native = (L, "gcc " + flags)
        except (OSError, subprocess.CalledProcessError):
            _native = (lib(), "committed build (x86-64-v3)")
        finally:
            if out.exists():
                out.unlink()
    return _native


def cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _raw(w) -> np.ndarray:
    a = np.ascontiguousarray(np.frombuffer(w, dtype=np.uint8) if isinstance(w, (bytes, bytearray, memoryview)) else w)
    assert a.dtype == np.uint8
    return a


def max_threads() -> int:
    return int(lib().oracle_max_threads())


def dequantize(ggml_type: int, raw, elements: int | None = None) -> np.ndarray:
    """C oracle: decode `elements` weights (default: all blocks in `raw`)."""
    raw = _raw(raw)
    if elements is None:
        elements = raw.size // BLOCK_BYTES[ggml_type] * BLOCK_ELEMS[ggml_type]
    need = elements // BLOCK_ELEMS[ggml_type] * BLOCK_BYTES[ggml_type]
    if raw.size < need:
        raise ValueError("payload shorter than required")
    out = np.empty(elements, dtype=np.float32)
    if lib().oracle_dequantize(ggml_type, _ptr(raw), _ptr(out), elements) != 0:
        raise ValueError("bad type or element count")
    return out


def cpu_linear(ggml_type: int, raw, x: np.ndarray, bias, rows: int, in_w: int, out_w: int,
               threads: int = 0, native: bool = False) -> np.ndarray:
    """C oracle: the reference's CpuLinear (FP32 sequential FMA from bias).  native=True runs the build made for this
    host (native_lib), for timing."""
    raw = _raw(raw)
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.size == rows * in_w
    assert raw.size == out_w * (in_w // BLOCK_ELEMS[ggml_type]) * BLOCK_BYTES[ggml_type]
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    y = np.empty((rows, out_w), dtype=np.float32)
    L = native_lib()[0] if native else lib()
    rc = L.oracle_cpu_linear(ggml_type, _ptr(raw), _ptr(x), _ptr(b), _ptr(y), rows, in_w, out_w, threads)
    if rc != 0:
        raise ValueError(f"oracle_cpu_linear failed ({rc})")
    return y


def linear_f64(ggml_type: int, raw, x: np.ndarray, bias, rows: int, in_w: int, out_w: int,
               threads: int = 0, x_is_bf16: bool = False):
    """C oracle: float64 dot over FP32-decoded weights. Returns (y[rows,out_w] f64, abs_sum f64)."""
    raw = _raw(raw)
    x = np.ascontiguousarray(x, dtype=np.uint16 if x_is_bf16 else np.float32)
    assert x.size == rows * in_w
    assert raw.size == out_w * (in_w // BLOCK_ELEMS[ggml_type]) * BLOCK_BYTES[ggml_type]
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    y = np.empty((rows, out_w), dtype=np.float64)
    a = np.empty((rows, out_w), dtype=np.float64)
    rc = lib().oracle_linear_f64(ggml_type, _ptr(raw), _ptr(x), int(x_is_bf16), _ptr(b), _ptr(y), _ptr(a),
                                 rows, in_w, out_w, threads)
    if rc != 0:
        raise ValueError(f"oracle_linear_f64 failed ({rc})")
    return y, a


def rel_l2(actual, expected) -> float:
    """sqrt(sum (a-b)^2 / sum b^2): NNtrain.Core.Tests/Qwen35XmxPrefillLinearTests.cs:80-89."""
    a = np.asarray(actual, dtype=np.float64).ravel()
    b = np.asarray(expected, dtype=np.float64).ravel()
    den = float(np.sum(b * b))
    return float(np.sqrt(np.sum((a - b) ** 2) / max(den, 1e-300)))


# ---------------------------------------------------------------- numpy restatements (independent of the C)

def _grids():
    text = (HERE / "iq_grids.inc").read_text()
    g2 = np.array([int(v, 16) for v in re.findall(r"0x([0-9a-f]{16})ull", text)], dtype=np.uint64)
    g3 = np.array([int(v, 16) for v in re.findall(r"0x([0-9a-f]{8})u\b", text)], dtype=np.uint32)
    assert g2.size == 1024 and g3.size == 512
    return g2.view(np.uint8).reshape(1024, 8), g3.view(np.uint8).reshape(512, 4)


_GRID_CACHE = None


def grids():
    global _GRID_CACHE
    if _GRID_CACHE is None:
        _GRID_CACHE = _grids()
    return _GRID_CACHE


def _half(b: np.ndarray) -> np.ndarray:
    """[n,2] uint8 -> float32 via numpy's IEEE float16."""
    return np.ascontiguousarray(b).view("<f2").astype(np.float32).reshape(-1)


def _k4_scales(sc: np.ndarray):
    sc = sc.astype(np.uint8)
    s = np.empty((sc.shape[0], 8), np.uint8)
    m = np.empty((sc.shape[0], 8), np.uint8)
    s[:, :4] = sc[:, 0:4] & 63
    m[:, :4] = sc[:, 4:8] & 63
    s[:, 4:] = (sc[:, 8:12] & 15) | ((sc[:, 0:4] >> 6) << 4)
    m[:, 4:] = (sc[:, 8:12] >> 4) | ((sc[:, 4:8] >> 6) << 4)
    return s, m


def np_dequantize(ggml_type: int, raw) -> np.ndarray:
    raw = _raw(raw)
    bb = BLOCK_BYTES[ggml_type]
    assert raw.size % bb == 0
    b = raw.reshape(-1, bb)
    n = b.shape[0]
    f32 = np.float32
    if ggml_type == BF16:
        return (b.reshape(-1).view('<u2').astype(np.uint32) << 16).view(f32)
    if ggml_type == Q8_0:
        d = _half(b[:, 0:2])
        q = b[:, 2:34].view(np.int8).astype(f32)
        return (d[:, None] * q).astype(f32).reshape(-1)
    if ggml_type in (Q4_K, Q5_K):
        d = _half(b[:, 0:2])
        dmin = _half(b[:, 2:4])
        s, m = _k4_scales(b[:, 4:16])
        if ggml_type == Q4_K:
            qs = b[:, 16:144].reshape(n, 4, 32)
            hi = None
        else:
            qs = b[:, 48:176].reshape(n, 4, 32)
            hi = b[:, 16:48]
        q = np.empty((n, 8, 32), np.uint8)
        q[:, 0::2] = qs & 15
        q[:, 1::2] = qs >> 4
        if hi is not None:
            for g in range(8):
                q[:, g] |= ((hi >> g) & 1) << 4
        scale = (d[:, None] * s.astype(f32)).astype(f32)
        mn = (dmin[:, None] * m.astype(f32)).astype(f32)
        prod = (scale[:, :, None] * q.astype(f32)).astype(f32)
        return (prod - mn[:, :, None]).astype(f32).reshape(-1)
    if ggml_type == Q6_K:
        ql = b[:, 0:128].reshape(n, 2, 2, 32)      # [block, half, which 32-run, l]
        qh = b[:, 128:192].reshape(n, 2, 32)
        sc = b[:, 192:208].view(np.int8).reshape(n, 2, 8).astype(f32)
        d = _half(b[:, 208:210])
        q = np.empty((n, 2, 4, 32), np.int32)
        q[:, :, 0] = (ql[:, :, 0] & 15) | (((qh >> 0) & 3) << 4)
        q[:, :, 1] = (ql[:, :, 1] & 15) | (((qh >> 2) & 3) << 4)
        q[:, :, 2] = (ql[:, :, 0] >> 4) | (((qh >> 4) & 3) << 4)
        q[:, :, 3] = (ql[:, :, 1] >> 4) | (((qh >> 6) & 3) << 4)
        q -= 32
        ds = (d[:, None, None] * sc).astype(f32)                  # [n,2,8]; sub-scale index = 2*j + l//16
        ds = ds.reshape(n, 2, 4, 2)
        ds = np.repeat(ds, 16, axis=3)                            # [n,2,4,32]
        return (ds * q.astype(f32)).astype(f32).reshape(-1)
    if ggml_type == IQ2_S:
        g2, _ = grids()
        d = _half(b[:, 0:2])
        qs = b[:, 2:34].reshape(n, 8, 4).astype(np.int32)
        signs = b[:, 34:66].reshape(n, 8, 4)
        qh = b[:, 66:74].astype(np.int32)
        sc = b[:, 74:82].astype(np.int32)
        o = np.arange(4)
        idx = qs | (((qh[:, :, None] >> (2 * o)) & 3) << 8)
        mag = g2[idx].astype(f32)                                  # [n,8,4,8]
        s4 = (sc[:, :, None] >> (4 * (o >> 1))) & 15               # [n,8,4]
        db = (d[:, None, None] * (f32(0.5) + s4.astype(f32)).astype(f32)).astype(f32)
        db = (db * f32(0.25)).astype(f32)
        neg = (signs[:, :, :, None] >> np.arange(8)) & 1
        sign = np.where(neg != 0, f32(-1), f32(1)).astype(f32)
        return ((db[:, :, :, None] * mag).astype(f32) * sign).astype(f32).reshape(-1)
    if ggml_type == IQ3_S:
        _, g3 = grids()
        d = _half(b[:, 0:2])
        qs = b[:, 2:66].reshape(n, 8, 8).astype(np.int32)
        qh = b[:, 66:74].astype(np.int32)
        signs = b[:, 74:106].reshape(n, 32)
        sc = b[:, 106:110].astype(np.int32)
        qi = np.arange(8)
        idx = qs | (((qh[:, :, None] >> qi) & 1) << 8)             # [n,8,8]
        mag = g3[idx].astype(f32)                                  # [n,8,8,4]
        g = np.arange(8)
        s4 = (sc[:, g >> 1] >> ((g & 1) * 4)) & 15                 # [n,8]
        db = (d[:, None] * (1 + 2 * s4).astype(f32)).astype(f32)
        neg = ((signs[:, :, None] >> np.arange(8)) & 1).reshape(n, 8, 8, 4)
        sign = np.where(neg != 0, f32(-1), f32(1)).astype(f32)
        return ((db[:, :, None, None] * mag).astype(f32) * sign).astype(f32).reshape(-1)
    raise ValueError(f"unsupported ggml type {ggml_type}")


def np_linear_f64(ggml_type: int, raw, x: np.ndarray, bias, rows: int, in_w: int, out_w: int) -> np.ndarray:
    w = np_dequantize(ggml_type, raw).reshape(out_w, in_w).astype(np.float64)
    y = np.asarray(x, np.float32).reshape(rows, in_w).astype(np.float64) @ w.T
    if bias is not None:
        y = y + np.asarray(bias, np.float32).astype(np.float64)[None, :]
    return y


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even; NaN kept quiet."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + np.uint32(0x7FFF)
    out = ((u + r) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if np.any(nan):
        out = np.where(nan, np.uint16(0x7FC0), out)
    return out


def bf16_widen(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ------------------------------------------------------------------ FP32 row operations around the mat-vec
# C statements in norm_oracle.c (which cites the reference kernels); the np_* functions are written separately.

def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def rms_norm(x, weight, rows: int, width: int, eps: float, input_stride: int | None = None) -> np.ndarray:
    """q35a_rms_norm: x holds `rows` rows `input_stride` apart; returns [rows, width]."""
    stride = width if input_stride is None else input_stride
    x, weight = _f32(x), _f32(weight)
    assert x.size >= (rows - 1) * stride + width and weight.size == width
    out = np.empty(rows * width, dtype=np.float32)
    lib().oracle_rms_norm(_ptr(x), _ptr(weight), _ptr(out), rows, width, stride, eps)
    return out.reshape(rows, width)


def add_rms_norm(destination, residual, weight, rows: int, width: int, eps: float,
                 input_stride: int | None = None):
    """q35a_add_rms_norm: returns (destination + residual, normalized [rows, width])."""
    stride = width if input_stride is None else input_stride
    dest = _f32(destination).copy()
    residual, weight = _f32(residual), _f32(weight)
    out = np.empty(rows * width, dtype=np.float32)
    lib().oracle_add_rms_norm(_ptr(dest), _ptr(residual), _ptr(weight), _ptr(out), rows, width, stride, eps)
    return dest, out.reshape(rows, width)


def rms_norm_serial(x, weight, rows: int, width: int, eps: float) -> np.ndarray:
    """Qwen35Math.RmsNorm: one running sum per row."""
    x, weight = _f32(x), _f32(weight)
    out = np.empty(rows * width, dtype=np.float32)
    lib().oracle_rms_norm_serial(_ptr(x), _ptr(weight), _ptr(out), rows, width, eps)
    return out.reshape(rows, width)


def silu_multiply(gate, up) -> np.ndarray:
    gate, up = _f32(gate), _f32(up)
    out = np.empty(gate.size, dtype=np.float32)
    lib().oracle_silu_multiply(_ptr(gate), _ptr(up), _ptr(out), gate.size)
    return out


def add_in_place(destination, source) -> np.ndarray:
    dest, source = _f32(destination).copy(), _f32(source)
    lib().oracle_add_in_place(_ptr(dest), _ptr(source), dest.size)
    return dest


def lora_a(x, a, rows: int, width: int, rank: int) -> np.ndarray:
    """q35l_lora_a_coop: z[rows, rank] = x[rows, width] . a[rank, width]^T."""
    x, a = _f32(x), _f32(a)
    assert x.size == rows * width and a.size == rank * width
    z = np.empty(rows * rank, dtype=np.float32)
    lib().oracle_lora_a(_ptr(x), _ptr(a), _ptr(z), rows, width, rank)
    return z.reshape(rows, rank)


def lora_b(z, b, y, rows: int, output: int, rank: int, scale: float) -> np.ndarray:
    """q35l_lora_b: returns y[rows, output] + scale * z[rows, rank] . b[output, rank]^T."""
    z, b, out = _f32(z), _f32(b), _f32(y).copy()
    assert z.size == rows * rank and b.size == output * rank and out.size == rows * output
    lib().oracle_lora_b(_ptr(z), _ptr(b), _ptr(out), rows, output, rank, scale)
    return out.reshape(rows, output)


def np_tree_sum_of_squares(x: np.ndarray) -> np.float32:
    """The 128-lane strided partial sums and the halving tree, with numpy float32 scalars (separate from the C)."""
    x = np.asarray(x, dtype=np.float32)
    sums = np.zeros(128, dtype=np.float32)
    for j in range(x.size):                      # lane j % 128 meets its elements in increasing j
        sums[j % 128] = np.float32(sums[j % 128] + np.float32(x[j] * x[j]))
    stride = 64
    while stride > 0:
        sums[:stride] = sums[:stride] + sums[stride:2 * stride]
        stride >>= 1
    return sums[0]


def np_rms_norm(x, weight, rows: int, width: int, eps: float, input_stride: int | None = None) -> np.ndarray:
    stride = width if input_stride is None else input_stride
    x, weight = np.asarray(x, dtype=np.float32), np.asarray(weight, dtype=np.float32)
    out = np.empty((rows, width), dtype=np.float32)
    for r in range(rows):
        row = x[r * stride:r * stride + width]
        mean = np.float32(np_tree_sum_of_squares(row) / np.float32(width))
        inverse = np.float32(np.float32(1.0) / np.sqrt(np.float32(mean + np.float32(eps))))
        out[r] = (row * inverse) * weight
    return out
