"""Pins the CPU oracle (C and numpy statements) to the reference's golden vectors and to closed forms.

Vectors: tests/golden/qwen_gguf_expected.json (gguf-py, NNtrain.Core.Tests/QwenGgufIndependentReferenceTests.cs:18-97)
and tests/golden/iq_quant_blocks.json (native ggml, NNtrain.Core.Tests/Qwen35GpuIqTests.cs:25-45).
"""
import base64
import hashlib
import json
import struct

import numpy as np
import pytest

import oracle
from oracle import IQ2_S, IQ3_S, Q4_K, Q5_K, Q6_K, Q8_0


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _same_bits_mod_zero_sign(a, b):
    """Bit equality, treating +0 and -0 as equal (the fixture README allows exactly that)."""
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    return bool(np.all((_bits(a) == _bits(b)) | ((a == 0) & (b == 0))))


@pytest.fixture(scope="module")
def qwen_expected(golden_dir):
    return json.loads((golden_dir / "qwen_gguf_expected.json").read_text())


@pytest.fixture(scope="module")
def iq_blocks(golden_dir):
    return json.loads((golden_dir / "iq_quant_blocks.json").read_text())["cases"]


def _gguf_payloads(golden_dir):
    """Tiny structural GGUF walk (independent of the product's reader) -> {name: (type, shape, bytes)}."""
    blob = (golden_dir / "qwen_gguf_reference.gguf").read_bytes()
    pos = 0

    def rd(fmt):
        nonlocal pos
        v = struct.unpack_from("<" + fmt, blob, pos)
        pos += struct.calcsize("<" + fmt)
        return v[0] if len(v) == 1 else v

    def rstr():
        nonlocal pos
        n = rd("Q")
        s = blob[pos:pos + n].decode()
        pos += n
        return s

    sizes = {0: 1, 1: 1, 2: 2, 3: 2, 4: 4, 5: 4, 6: 4, 7: 1, 10: 8, 11: 8, 12: 8}

    def rval(t):
        nonlocal pos
        if t == 8:
            return rstr()
        if t == 9:
            et, n = rd("I"), rd("Q")
            return [rval(et) for _ in range(n)]
        v = blob[pos:pos + sizes[t]]
        pos += sizes[t]
        return v

    assert rd("I") == 0x46554747
    assert rd("I") in (2, 3)
    nt, nkv = rd("Q"), rd("Q")
    align = 32
    for _ in range(nkv):
        k = rstr()
        t = rd("I")
        v = rval(t)
        if k == "general.alignment":
            align = int.from_bytes(v, "little")
    infos = []
    for _ in range(nt):
        name = rstr()
        nd = rd("I")
        shape = [rd("Q") for _ in range(nd)]
        typ, off = rd("I"), rd("Q")
        infos.append((name, typ, shape, off))
    data = (pos + align - 1) // align * align
    out = {}
    for name, typ, shape, off in infos:
        out[name] = (typ, shape, blob, data + off)
    return out


@pytest.mark.parametrize("impl", ["c", "numpy"])
def test_q4k_q6k_dequant_bit_exact_vs_gguf_py(golden_dir, qwen_expected, impl):
    payloads = _gguf_payloads(golden_dir)
    seen = 0
    for t in qwen_expected["tensors"]:
        if t["type"] not in (Q4_K, Q6_K):
            continue
        typ, shape, blob, off = payloads[t["name"]]
        assert typ == t["type"] and list(shape) == list(t["shape"])
        raw = np.frombuffer(blob, np.uint8, t["payloadBytes"], off)
        expect = np.frombuffer(base64.b64decode(t["decodedFloat32Base64"]), "<f4")
        got = oracle.dequantize(typ, raw) if impl == "c" else oracle.np_dequantize(typ, raw)
        assert got.size == expect.size == 7 * 512
        assert np.array_equal(_bits(got), _bits(expect)), t["name"]
        seen += 1
    assert seen == 4


@pytest.mark.parametrize("impl", ["c", "numpy"])
@pytest.mark.parametrize("typ,count", [(Q5_K, 25), (IQ2_S, 69), (IQ3_S, 45)])
def test_q5k_iq_dequant_bit_exact_vs_native_ggml(iq_blocks, typ, count, impl):
    n = 0
    for case in iq_blocks:
        if case["type"] != typ:
            continue
        raw = np.frombuffer(base64.b64decode(case["encoded"]), np.uint8)
        expect = np.frombuffer(base64.b64decode(case["decodedFloat32Base64"]), "<f4")
        got = oracle.dequantize(typ, raw) if impl == "c" else oracle.np_dequantize(typ, raw)
        assert _same_bits_mod_zero_sign(got, expect), case["id"]
        if np.array_equal(_bits(got), _bits(expect)):
            assert hashlib.sha256(got.astype("<f4").tobytes()).hexdigest() == case["decodedFloat32LittleEndianSha256"]
        n += 1
    assert n == count


def test_q5k_all_ff_closed_form():
    # d = 0.5 (0x3800), dmin = 0.25 (0x3400), every other byte 0xFF -> 0.5*63*31 - 0.25*63 = 960.75
    raw = np.full(176, 0xFF, np.uint8)
    raw[0:2] = (0x00, 0x38)
    raw[2:4] = (0x00, 0x34)
    for got in (oracle.dequantize(Q5_K, raw), oracle.np_dequantize(Q5_K, raw)):
        assert np.all(got == np.float32(960.75))


def test_known_single_weight_answers():
    # NNtrain.Core.Tests/QwenArcKernelTests.cs:104-131: Q4_K d=0x0001 (2^-24), sc=63, q=15 -> 945 * 2^-24
    raw = np.zeros(144, np.uint8)
    raw[0] = 1
    raw[4] = 63
    raw[16] = 0x0F
    got = oracle.dequantize(Q4_K, raw)
    assert got[0] == np.float32(945 * 2.0 ** -24) and np.all(got[1:] == 0)
    # Q6_K d=0x03ff (largest subnormal), scale=127, q=31 (ql nibble 15, qh bits 3 -> 63-32)
    raw = np.zeros(210, np.uint8)
    raw[208:210] = (0xFF, 0x03)
    raw[192] = 127
    raw[0] = 0x0F
    raw[128] = 0x03
    got = oracle.dequantize(Q6_K, raw)
    d = np.float32(1023 * 2.0 ** -24)
    assert got[0] == np.float32(np.float32(d * np.float32(127)) * np.float32(31))
    # every other value has q = -32 with scale 0 or 127
    assert got[1] == np.float32(np.float32(d * np.float32(127)) * np.float32(-32))
    # all-zero blocks decode to zero for every type (NNtrain.Core.Tests/QwenPrimitiveTests.cs:30-37); Q6_K gives -0*32
    for typ in (Q8_0, Q4_K, Q5_K, IQ2_S, IQ3_S, Q6_K):
        z = oracle.dequantize(typ, np.zeros(oracle.BLOCK_BYTES[typ], np.uint8))
        assert np.all(z == 0)


def test_half_to_float_all_65536_patterns():
    h = np.arange(65536, dtype=np.uint16)
    expect = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib().oracle_half_to_float(int(v)) for v in h], dtype=np.float32)
    same = (_bits(got) == _bits(expect)) | (np.isnan(got) & np.isnan(expect))
    assert np.all(same)


def test_q8_0_closed_form_vs_numpy_and_brute_force():
    rng = np.random.default_rng(7)
    raw = rng.integers(0, 256, size=(4096, 34), dtype=np.uint8)
    # keep scales finite: clear the top exponent bit pattern 0x7c00
    d16 = raw[:, 0:2].copy().view("<u2")
    d16[(d16 & 0x7C00) == 0x7C00] &= 0x3FFF
    raw[:, 0:2] = d16.view(np.uint8)
    got = oracle.dequantize(Q8_0, raw.reshape(-1))
    textbook = (raw[:, 0:2].copy().view("<f2").astype(np.float32) * raw[:, 2:].view(np.int8).astype(np.float32))
    assert np.array_equal(_bits(got), _bits(textbook.reshape(-1)))
    # brute force in Python floats: d*q is exact in binary64 and representable in binary32
    for blk in (0, 17, 4095):
        d = float(np.frombuffer(raw[blk, 0:2].tobytes(), "<f2")[0])
        for i in (0, 5, 31):
            q = int(np.int8(raw[blk, 2 + i]))
            assert float(got[blk * 32 + i]) == d * q


@pytest.mark.parametrize("typ", [Q8_0, Q4_K, Q5_K, Q6_K, IQ2_S, IQ3_S])
def test_c_and_numpy_statements_agree_on_random_blocks(typ):
    rng = np.random.default_rng(100 + typ)
    bb = oracle.BLOCK_BYTES[typ]
    raw = rng.integers(0, 256, size=(512, bb), dtype=np.uint8)
    for off in ((0, 2) if typ in (Q4_K, Q5_K) else (208,) if typ == Q6_K else (0,)):
        raw[:, off + 1] &= 0x7B  # finite, positive-or-negative handled by low byte; keeps exponent < 31
    a = oracle.dequantize(typ, raw.reshape(-1))
    b = oracle.np_dequantize(typ, raw.reshape(-1))
    assert np.array_equal(_bits(a), _bits(b))


def test_linear_f64_vs_reference_vectors(golden_dir, qwen_expected):
    payloads = _gguf_payloads(golden_dir)
    K, N = qwen_expected["inputWidth"], qwen_expected["outputWidth"]
    x_all = np.frombuffer(base64.b64decode(qwen_expected["inputFloat32Base64"]), "<f4").reshape(
        qwen_expected["inputRows"], K)
    n = 0
    for t in qwen_expected["tensors"]:
        if t["type"] not in (Q4_K, Q6_K):
            continue
        typ, shape, blob, off = payloads[t["name"]]
        raw = np.frombuffer(blob, np.uint8, t["payloadBytes"], off)
        bias = np.frombuffer(base64.b64decode(t["biasFloat32Base64"]), "<f4")
        expect = np.frombuffer(base64.b64decode(t["linearFloat64Base64"]), "<f8").reshape(-1, N)
        rows = expect.shape[0]
        y, asum = oracle.linear_f64(typ, raw, x_all[:rows], bias, rows, K, N)
        assert np.max(np.abs(y - expect)) <= 1e-12 * max(1.0, np.max(np.abs(expect)))
        ynp = oracle.np_linear_f64(typ, raw, x_all[:rows], bias, rows, K, N)
        assert np.max(np.abs(ynp - expect)) <= 1e-12 * max(1.0, np.max(np.abs(expect)))
        # the reference's tolerance for FP32 kernels applies to the FP32 CpuLinear statement too
        y32 = oracle.cpu_linear(typ, raw, x_all[:rows], bias, rows, K, N)
        assert np.max(np.abs(y32 - expect)) <= np.max(np.abs(expect)) * 5e-6 + 1e-9
        assert np.all(asum >= np.abs(y) - 1e-12)
        n += 1
    assert n == 4


def test_cpu_linear_brute_force_and_invariants():
    rng = np.random.default_rng(11)
    typ, K, N, rows = Q4_K, 512, 5, 3
    raw = rng.integers(0, 256, size=N * 2 * 144, dtype=np.uint8)
    raw.reshape(-1, 144)[:, 1] &= 0x3B
    raw.reshape(-1, 144)[:, 3] &= 0x3B
    x = rng.standard_normal((rows, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    w = oracle.dequantize(typ, raw).reshape(N, K)
    y = oracle.cpu_linear(typ, raw, x, bias, rows, K, N, threads=1)
    # brute force: the same sequential fused multiply-add written with exact rationals rounded once per step
    import math
    for r in range(rows):
        for o in range(N):
            s = np.float32(bias[o])
            for k in range(K):
                s = np.float32(math.fma(float(x[r, k]), float(w[o, k]), float(s))) if hasattr(math, "fma") \
                    else np.float32(np.float64(x[r, k]) * np.float64(w[o, k]) + np.float64(s))
            assert abs(float(s) - float(y[r, o])) <= 1e-6 * max(1.0, abs(float(y[r, o])))
    # threads do not change the result (rows are independent)
    assert np.array_equal(_bits(y), _bits(oracle.cpu_linear(typ, raw, x, bias, rows, K, N, threads=4)))
    # rows > 1 equals stacked single rows, bitwise
    for r in range(rows):
        assert np.array_equal(_bits(y[r]), _bits(oracle.cpu_linear(typ, raw, x[r], bias, 1, K, N)[0]))
    # linearity in x for the float64 statement, and bias is a pure add
    y0, _ = oracle.linear_f64(typ, raw, x, None, rows, K, N)
    yb, _ = oracle.linear_f64(typ, raw, x, bias, rows, K, N)
    assert np.allclose(yb - y0, bias.astype(np.float64)[None, :], rtol=0, atol=1e-9)
    y2, _ = oracle.linear_f64(typ, raw, (2 * x).astype(np.float32), None, rows, K, N)
    assert np.allclose(y2, 2 * y0, rtol=1e-13, atol=0)
    # a transposed-operand mistake would fail this: one-hot x picks a single weight column
    e = np.zeros((1, K), np.float32)
    e[0, 37] = 1
    yk, _ = oracle.linear_f64(typ, raw, e, None, 1, K, N)
    assert np.array_equal(yk[0], w[:, 37].astype(np.float64))


def test_bf16_helpers():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.14159, 0.0, 65504.0, 1e-40], np.float32)
    b = oracle.bf16_round(x)
    w = oracle.bf16_widen(b)
    assert w[0] == 1.0 and w[1] == 1.0 and w[2] == np.float32(1.015625)  # ties to even, then round up
    assert np.all(np.abs(w - x) <= np.abs(x) * 2.0 ** -8 + 1e-38)
    y, _ = oracle.linear_f64(Q8_0, np.zeros(34, np.uint8), b[:1].repeat(32), None, 1, 32, 1, x_is_bf16=True)
    assert y[0, 0] == 0.0
