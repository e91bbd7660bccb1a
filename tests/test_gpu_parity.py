"""GPU parity: the HIP path (through the C ABI) against the CPU oracle and the reference's golden vectors.

Bars: dequantized weights bit-exact (+0/-0 equal); mat-vec relative L2 <= 1e-5 against the float64 oracle, plus the
reference's per-element bound 2e-6 + 3e-6 * sum|x*w| (NNtrain.Core.Tests/Qwen35GpuLinearTests.cs:66-84).
"""
import base64
import json

import numpy as np
import pytest

import oracle
from nntrain_amd import (BLOCK_BYTES, BLOCK_ELEMS, GGML_IQ2_S, GGML_IQ3_S, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_Q8_0,
                         GgufReader, HipExecutionLane, HipQuantizedMatrix, NnHipError, synth)

pytestmark = pytest.mark.gpu

ALL_TYPES = [GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_IQ3_S, GGML_IQ2_S]
NAN_BITS = 0x7FC00000
REL_L2_BAR = 1e-5


@pytest.fixture(scope="module")
def lane():
    with HipExecutionLane(0) as ln:
        yield ln


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _same_mod_zero(a, b):
    return bool(np.all((_bits(a) == _bits(b)) | ((a == 0) & (b == 0))))


def _random_payload(typ, out_w, in_w, seed):
    if typ == GGML_Q8_0:
        rng = np.random.default_rng(seed)
        w = rng.standard_normal((out_w, in_w), dtype=np.float32) * np.float32(0.02)
        return synth.quantize_q8_0(w)
    return synth.k_quant_matrix(typ, out_w, in_w, seed)


def _run_matvec(lane, typ, payload, x, bias, rows, in_w, out_w):
    """Returns y[rows, out_w]; checks NaN guards past the output and that the launch moved no bytes."""
    mat = HipQuantizedMatrix(payload, typ, out_w, in_w)
    mat.device_payload(lane)
    xb = lane.upload_raw(np.ascontiguousarray(x, np.float32))
    bb = lane.upload_raw(np.ascontiguousarray(bias, np.float32)) if bias is not None else None
    yb = lane.allocate(rows * out_w + 2)
    lane.fill_u32(yb, NAN_BITS, rows * out_w + 2)
    lane.synchronize()
    before = lane.counters()
    mat.forward(lane, xb, bb, rows, out=yb)
    lane.synchronize()
    after = lane.counters()
    assert after["h2d_bytes"] == before["h2d_bytes"] and after["d2h_bytes"] == before["d2h_bytes"]
    assert after["allocated_bytes"] == before["allocated_bytes"]
    y = lane.read(yb)
    assert np.isnan(y[-1]) and np.isnan(y[-2]), "guard elements past the output were overwritten"
    for b in (xb, bb, yb):
        if b is not None:
            b.dispose()
    mat.dispose()
    assert np.all(np.isfinite(y[:-2]))
    return y[:-2].reshape(rows, out_w)


def _check_against_f64(y, ref, asum):
    assert oracle.rel_l2(y, ref) <= REL_L2_BAR
    assert np.all(np.abs(y.astype(np.float64) - ref) <= 2e-6 + 3e-6 * asum)


# ----------------------------------------------------------------------------------------------- dequantize

def test_dequantize_q4k_q6k_bit_exact_vs_gguf_py(lane, golden_dir):
    expected = json.loads((golden_dir / "qwen_gguf_expected.json").read_text())
    with GgufReader(str(golden_dir / "qwen_gguf_reference.gguf")) as reader:
        seen = 0
        for t in expected["tensors"]:
            if t["type"] not in (GGML_Q4_K, GGML_Q6_K):
                continue
            info = reader.get_tensor(t["name"])
            in_w, out_w = reader.matrix_dims(info)
            mat = HipQuantizedMatrix(reader.read_tensor_bytes(info), info.type, out_w, in_w)
            got = lane.read(mat.dequantize(lane))
            want = np.frombuffer(base64.b64decode(t["decodedFloat32Base64"]), "<f4")
            assert np.array_equal(_bits(got), _bits(want)), t["name"]
            row = lane.read(mat.dequantize(lane, row=out_w - 1))
            assert np.array_equal(_bits(row), _bits(want[-in_w:]))
            mat.dispose()
            seen += 1
        assert seen == 4


@pytest.mark.parametrize("typ", [GGML_Q5_K, GGML_IQ2_S, GGML_IQ3_S])
def test_dequantize_bit_exact_vs_native_ggml_blocks(lane, golden_dir, typ):
    cases = [c for c in json.loads((golden_dir / "iq_quant_blocks.json").read_text())["cases"] if c["type"] == typ]
    assert len(cases) == {GGML_Q5_K: 25, GGML_IQ2_S: 69, GGML_IQ3_S: 45}[typ]
    raw = np.concatenate([np.frombuffer(base64.b64decode(c["encoded"]), np.uint8) for c in cases])
    want = np.concatenate([np.frombuffer(base64.b64decode(c["decodedFloat32Base64"]), "<f4") for c in cases])
    mat = HipQuantizedMatrix(raw, typ, len(cases), 256)
    got = lane.read(mat.dequantize(lane))
    mat.dispose()
    for i, c in enumerate(cases):
        assert _same_mod_zero(got[256 * i:256 * i + 256], want[256 * i:256 * i + 256]), c["id"]


@pytest.mark.parametrize("typ", ALL_TYPES)
def test_dequantize_bit_exact_vs_oracle_random_blocks(lane, typ):
    rng = np.random.default_rng(500 + typ)
    n_blocks = 4096 + 7
    raw = rng.integers(0, 256, size=(n_blocks, BLOCK_BYTES[typ]), dtype=np.uint8)
    for off in ((0, 2) if typ in (GGML_Q4_K, GGML_Q5_K) else (208,) if typ == GGML_Q6_K else (0,)):
        raw[:, off + 1] &= 0x7B          # keep fp16 scales finite (any sign, normal and subnormal)
    raw[:64, 0 if typ != GGML_Q6_K else 208] = rng.integers(0, 256, 64)
    raw[:64, 1 if typ != GGML_Q6_K else 209] &= 0x83  # subnormal-only scales in the first blocks
    mat = HipQuantizedMatrix(raw.reshape(-1), typ, n_blocks, BLOCK_ELEMS[typ])
    got = lane.read(mat.dequantize(lane))
    mat.dispose()
    want = oracle.dequantize(typ, raw.reshape(-1))
    assert np.array_equal(_bits(got), _bits(want))


def test_dequantize_rejects_bad_arguments(lane):
    buf = lane.allocate(256)
    from ctypes import c_void_p
    lib, h = lane._lib, lane._handle
    assert lib.nnhip_dequantize(h, 99, c_void_p(buf.ptr), c_void_p(buf.ptr), 256) == 2     # unsupported type
    assert lib.nnhip_dequantize(h, GGML_Q4_K, c_void_p(buf.ptr), c_void_p(buf.ptr), 255) == 3  # incomplete block
    assert lib.nnhip_dequantize(h, GGML_Q4_K, None, c_void_p(buf.ptr), 256) == 1
    assert lib.nnhip_dequantize(h, GGML_Q4_K, c_void_p(buf.ptr), c_void_p(buf.ptr), 0) == 0
    buf.dispose()


# ----------------------------------------------------------------------------------------------- mat-vec

def test_matvec_reference_float64_vectors(lane, golden_dir):
    """Rows 1/3/5, K=512, N=7, with bias; tolerance of QwenGgufIndependentReferenceTests.cs:76-97."""
    expected = json.loads((golden_dir / "qwen_gguf_expected.json").read_text())
    K, N = expected["inputWidth"], expected["outputWidth"]
    x_all = np.frombuffer(base64.b64decode(expected["inputFloat32Base64"]), "<f4").reshape(expected["inputRows"], K)
    with GgufReader(str(golden_dir / "qwen_gguf_reference.gguf")) as reader:
        for t in expected["tensors"]:
            if t["type"] not in (GGML_Q4_K, GGML_Q6_K):
                continue
            payload = np.frombuffer(reader.read_tensor_bytes(reader.get_tensor(t["name"])), np.uint8)
            bias = np.frombuffer(base64.b64decode(t["biasFloat32Base64"]), "<f4")
            want = np.frombuffer(base64.b64decode(t["linearFloat64Base64"]), "<f8").reshape(-1, N)
            rows = want.shape[0]
            for r in (1, 3, rows):
                y = _run_matvec(lane, t["type"], payload, x_all[:r], bias, r, K, N)
                bound = np.max(np.abs(want[:r])) * 5e-6 + 1e-9
                assert np.max(np.abs(y - want[:r])) <= bound, (t["name"], r)


@pytest.mark.parametrize("typ", ALL_TYPES)
@pytest.mark.parametrize("in_w,out_w", [(256, 1), (512, 7), (1024, 67), (5120, 131), (17408, 33)])
def test_matvec_vs_oracle_shapes(lane, typ, in_w, out_w):
    payload = _random_payload(typ, out_w, in_w, seed=1000 * typ + in_w + out_w)
    x = synth.activations(1, in_w, seed=7 + in_w)
    bias = np.random.default_rng(3).standard_normal(out_w).astype(np.float32)
    y = _run_matvec(lane, typ, payload, x, bias, 1, in_w, out_w)
    ref, asum = oracle.linear_f64(typ, payload, x, bias, 1, in_w, out_w)
    _check_against_f64(y, ref, asum)
    # FP32 sequential CPU statement of the operator agrees to the same bar
    assert oracle.rel_l2(oracle.cpu_linear(typ, payload, x, bias, 1, in_w, out_w), y) <= REL_L2_BAR


@pytest.mark.parametrize("typ", ALL_TYPES)
def test_matvec_rows_equal_stacked_single_rows_bitwise(lane, typ):
    in_w, out_w, rows = 1024, 45, 5
    payload = _random_payload(typ, out_w, in_w, seed=42 + typ)
    x = synth.activations(rows, in_w, seed=9)
    y = _run_matvec(lane, typ, payload, x, None, rows, in_w, out_w)
    for r in range(rows):
        y1 = _run_matvec(lane, typ, payload, x[r:r + 1], None, 1, in_w, out_w)
        assert np.array_equal(_bits(y[r]), _bits(y1[0]))
    ref, asum = oracle.linear_f64(typ, payload, x, None, rows, in_w, out_w)
    _check_against_f64(y, ref, asum)


@pytest.mark.parametrize("in_w,out_w", [(5376, 70), (21504, 11), (7168, 33)])
@pytest.mark.parametrize("rows", [2, 3, 4, 7])
def test_matvec_row_tiles_equal_single_rows_bitwise(lane, rows, in_w, out_w):
    """Q8_0 and bfloat16 launches with several input rows share one pass over the weights between up to four rows (two
    when only two staging areas fit LDS, one for the widest vectors); a row's bits must not depend on the grouping."""
    from nntrain_amd import GGML_BF16
    x = synth.activations(rows, in_w, seed=rows + in_w)
    bias = np.random.default_rng(8).standard_normal(out_w).astype(np.float32)
    rng = np.random.default_rng(in_w + out_w)
    bf16 = synth.to_bf16_bits(rng.standard_normal((out_w, in_w), dtype=np.float32) * np.float32(0.02)).view(np.uint8).reshape(-1)
    for typ, payload in ((GGML_Q8_0, _random_payload(GGML_Q8_0, out_w, in_w, seed=31)), (GGML_BF16, bf16)):
        y = _run_matvec(lane, typ, payload, x, bias, rows, in_w, out_w)
        for r in range(rows):
            y1 = _run_matvec(lane, typ, payload, x[r:r + 1], bias, 1, in_w, out_w)
            assert np.array_equal(_bits(y[r]), _bits(y1[0])), (typ, r)
    ref, asum = oracle.linear_f64(GGML_Q8_0, _random_payload(GGML_Q8_0, out_w, in_w, seed=31), x, bias, rows, in_w, out_w)
    _check_against_f64(_run_matvec(lane, GGML_Q8_0, _random_payload(GGML_Q8_0, out_w, in_w, seed=31), x, bias, rows, in_w, out_w), ref, asum)


@pytest.mark.parametrize("in_w", [64, 128, 192, 256])
@pytest.mark.parametrize("out_w", [300, 1000, 5000])
def test_matvec_narrow_rows_several_input_rows(lane, in_w, out_w):
    """Rows of one to four units with several input rows: a workgroup then holds hundreds of matrix rows per step, and
    the results of a whole ring turn (times the input rows of the tile) must still fit its LDS result buffer.  Compared
    with the oracle and, bit for bit, with single-row launches (NaN guards past the output checked by the helper).
    Odd shapes and guard elements follow NNtrain.Core.Tests/Qwen35GpuLinearTests.cs:24-86."""
    from nntrain_amd import GGML_BF16
    rng = np.random.default_rng(in_w * 7 + out_w)
    bias = rng.standard_normal(out_w).astype(np.float32)
    bf16 = synth.to_bf16_bits(rng.standard_normal((out_w, in_w), dtype=np.float32) * np.float32(0.02)).view(np.uint8).reshape(-1)
    q8 = _random_payload(GGML_Q8_0, out_w, in_w, seed=in_w + out_w)
    singles = {}
    for rows in (1, 2, 3, 4, 7):
        x = synth.activations(7, in_w, seed=in_w)[:rows]
        for typ, payload in ((GGML_Q8_0, q8), (GGML_BF16, bf16)):
            y = _run_matvec(lane, typ, payload, x, bias, rows, in_w, out_w)
            if rows == 1:
                for r in range(7):
                    xr = synth.activations(7, in_w, seed=in_w)[r:r + 1]
                    singles[(typ, r)] = _run_matvec(lane, typ, payload, xr, bias, 1, in_w, out_w)[0]
            for r in range(rows):
                assert np.array_equal(_bits(y[r]), _bits(singles[(typ, r)])), (typ, rows, r)
            if typ == GGML_Q8_0:
                ref, asum = oracle.linear_f64(typ, payload, x, bias, rows, in_w, out_w)
                _check_against_f64(y, ref, asum)


def test_matvec_narrow_rows_very_tall_matrix(lane):
    """in_w = 64 with more rows than one ring turn of every workgroup holds: the flush in the middle of the loop."""
    in_w, out_w = 64, 400_000
    payload = _random_payload(GGML_Q8_0, out_w, in_w, seed=5)
    x = synth.activations(1, in_w, seed=6)
    y = _run_matvec(lane, GGML_Q8_0, payload, x, None, 1, in_w, out_w)
    ref, asum = oracle.linear_f64(GGML_Q8_0, payload, x, None, 1, in_w, out_w)
    _check_against_f64(y, ref, asum)


def test_matvec_q8_0_odd_block_count_rows(lane):
    in_w, out_w = 32 * 5, 19
    payload = _random_payload(GGML_Q8_0, out_w, in_w, seed=77)
    x = synth.activations(2, in_w, seed=78)
    y = _run_matvec(lane, GGML_Q8_0, payload, x, None, 2, in_w, out_w)
    ref, asum = oracle.linear_f64(GGML_Q8_0, payload, x, None, 2, in_w, out_w)
    _check_against_f64(y, ref, asum)


@pytest.mark.parametrize("typ", [GGML_Q4_K, GGML_Q6_K])
def test_matvec_subnormal_only_scales_zero_bias(lane, typ):
    """All fp16 scales subnormal (QwenQuantizedLinearFastTests.cs:99-123): lost subnormals would zero the output."""
    in_w, out_w = 512, 9
    rng = np.random.default_rng(typ)
    raw = rng.integers(0, 256, size=(out_w * 2, BLOCK_BYTES[typ]), dtype=np.uint8)
    for off in ((0, 2) if typ == GGML_Q4_K else (208,)):
        raw[:, off + 1] &= 0x03
        raw[:, off] |= 0x01
    x = synth.activations(1, in_w, seed=5)
    y = _run_matvec(lane, typ, raw.reshape(-1), x, None, 1, in_w, out_w)
    ref, asum = oracle.linear_f64(typ, raw.reshape(-1), x, None, 1, in_w, out_w)
    assert np.all(ref != 0)
    _check_against_f64(y, ref, asum)


def test_matvec_linearity_and_one_hot(lane):
    typ, in_w, out_w = GGML_Q5_K, 768, 21
    payload = _random_payload(typ, out_w, in_w, seed=8)
    e = np.zeros((1, in_w), np.float32)
    e[0, 517] = 1.0
    y = _run_matvec(lane, typ, payload, e, None, 1, in_w, out_w)
    w = oracle.dequantize(typ, payload).reshape(out_w, in_w)
    assert np.array_equal(_bits(y[0]), _bits(w[:, 517]))     # a one-hot activation reads one weight column exactly
    x = synth.activations(1, in_w, seed=1)
    y1 = _run_matvec(lane, typ, payload, x, None, 1, in_w, out_w)
    y2 = _run_matvec(lane, typ, payload, 2 * x, None, 1, in_w, out_w)
    assert np.array_equal(_bits(2 * y1), _bits(y2))           # scaling by 2 is exact in binary FP


def test_operator_argument_errors(lane):
    with pytest.raises(NotImplementedError):
        HipQuantizedMatrix(np.zeros(144, np.uint8), 2, 1, 256)
    with pytest.raises(NotImplementedError):
        HipQuantizedMatrix(np.zeros(144, np.uint8), GGML_Q4_K, 1, 255)
    with pytest.raises(ValueError):
        HipQuantizedMatrix(np.zeros(143, np.uint8), GGML_Q4_K, 1, 256)
    mat = HipQuantizedMatrix(np.zeros(144, np.uint8), GGML_Q4_K, 1, 256)
    x = lane.allocate(128)
    with pytest.raises(ValueError):
        mat.forward(lane, x, None)
    x.dispose()
    from ctypes import c_void_p
    buf = lane.allocate(1024)
    rc = lane._lib.nnhip_quant_matvec(lane._handle, GGML_Q4_K, c_void_p(buf.ptr), c_void_p(buf.ptr), None, c_void_p(buf.ptr),
                                      0, 256, 1)
    assert rc == 1
    with pytest.raises(NnHipError):
        from nntrain_amd.native import check
        check(rc, "quant_matvec")
    buf.dispose()
    mat.dispose()


# ----------------------------------------------------------------------------------------------- full-size configs

FULL = [
    ("cfg1_q8_0", GGML_Q8_0, 5376, 21504, 1001, 1002),
    ("cfg2_q4_k", GGML_Q4_K, 5120, 17408, 2001, 2000),
    ("cfg2_q5_k", GGML_Q5_K, 5120, 17408, 2002, 2000),
    ("cfg2_q6_k", GGML_Q6_K, 5120, 17408, 2003, 2000),
    ("cfg5_iq2_s", GGML_IQ2_S, 17408, 5120, 5001, 5002),
]


@pytest.mark.parametrize("name,typ,in_w,out_w,wseed,xseed", FULL, ids=[f[0] for f in FULL])
def test_matvec_full_size_configs(lane, name, typ, in_w, out_w, wseed, xseed):
    payload = synth.matrix(typ, out_w, in_w, wseed)
    x = synth.activations(1, in_w, xseed)
    y = _run_matvec(lane, typ, payload, x, None, 1, in_w, out_w)
    ref, asum = oracle.linear_f64(typ, payload, x, None, 1, in_w, out_w)
    _check_against_f64(y, ref, asum)
    print(f"{name}: rel_l2 vs f64 = {oracle.rel_l2(y, ref):.3e}")


# ----------------------------------------------------------------------------------------------- batched launch

def test_matvec_batch_equals_single_launches_bitwise(lane):
    """A batch (mixed formats, tiny and long matrices, rows > 1, bias) must reproduce per-matrix launches bit for bit."""
    from ctypes import c_void_p
    from nntrain_amd.native import MatvecDesc, check
    rng = np.random.default_rng(2024)
    shapes = [(GGML_Q8_0, 5376, 300, 1), (GGML_Q8_0, 4096, 37, 1), (GGML_Q8_0, 21504, 90, 1), (GGML_Q8_0, 64, 5, 2),
              (GGML_Q4_K, 5120, 260, 1), (GGML_Q4_K, 256, 3, 3), (GGML_Q6_K, 1024, 130, 1), (GGML_Q5_K, 2048, 77, 1),
              (GGML_IQ2_S, 17408, 40, 1), (GGML_Q8_0, 5376, 4100, 1), (GGML_Q8_0, 160, 9, 1), (GGML_Q4_K, 5120, 1, 1)]
    items = []
    for i, (typ, in_w, out_w, rows) in enumerate(shapes):
        payload = _random_payload(typ, out_w, in_w, seed=900 + i)
        x = rng.standard_normal((rows, in_w)).astype(np.float32)
        bias = rng.standard_normal(out_w).astype(np.float32) if i % 2 else None
        wb = lane.upload_raw(payload)
        xb = lane.upload_raw(x)
        bb = lane.upload_raw(bias) if bias is not None else None
        y1 = lane.allocate(rows * out_w + 2)
        y2 = lane.allocate(rows * out_w + 2)
        lane.fill_u32(y1, NAN_BITS, rows * out_w + 2)
        lane.fill_u32(y2, NAN_BITS, rows * out_w + 2)
        items.append((typ, in_w, out_w, rows, payload, x, bias, wb, xb, bb, y1, y2))
    lib, h = lane._lib, lane._handle
    for typ, in_w, out_w, rows, payload, x, bias, wb, xb, bb, y1, y2 in items:
        check(lib.nnhip_quant_matvec(h, typ, c_void_p(xb.ptr), c_void_p(wb.ptr), c_void_p(bb.ptr) if bb else None,
                                     c_void_p(y1.ptr), rows, in_w, out_w), "quant_matvec")
    descs = (MatvecDesc * len(items))()
    for i, (typ, in_w, out_w, rows, payload, x, bias, wb, xb, bb, y1, y2) in enumerate(items):
        descs[i] = MatvecDesc(xb.ptr, wb.ptr, bb.ptr if bb else None, y2.ptr, typ, rows, in_w, out_w)
    for _ in range(2):      # the second call reuses the device table
        check(lib.nnhip_quant_matvec_batch(h, descs, len(items)), "quant_matvec_batch")
    lane.synchronize()
    for typ, in_w, out_w, rows, payload, x, bias, wb, xb, bb, y1, y2 in items:
        a, b = lane.read(y1), lane.read(y2)
        assert np.isnan(b[-1]) and np.isnan(b[-2])
        assert np.array_equal(_bits(a[:-2]), _bits(b[:-2])), (typ, in_w, out_w, rows)
        ref, asum = oracle.linear_f64(typ, payload, x, bias, rows, in_w, out_w)
        _check_against_f64(b[:-2].reshape(rows, out_w), ref, asum)
    assert lib.nnhip_quant_matvec_batch(h, descs, 0) == 0
    assert lib.nnhip_quant_matvec_batch(h, None, 3) == 1
    for it in items:
        for b in it[7:]:
            if b is not None:
                b.dispose()


# ----------------------------------------------------------------------------------------------- prefill mat-mul

PREFILL_BAR = 2e-3      # relative L2 against the float64 oracle fed the same bf16 activation bits
# The kernel multiplies weights rounded once to bfloat16 (8 significant bits: 1.6e-3 rms), which is all of that error:
# against the same float64 product taken with the oracle's weights rounded to bfloat16 it must agree to FP32
# accumulation accuracy.  That tighter bar is applied everywhere; the 2e-3 one only where the matrix is large enough
# for the rounding errors to average (a 16 x 256 matrix can land at 2.2e-3).
PREFILL_TIGHT_BAR = 5e-6


def _bf16_weight_product(typ, payload, xb, bias, rows, in_w, out_w):
    w = oracle.bf16_widen(oracle.bf16_round(oracle.dequantize(typ, payload).reshape(out_w, in_w))).astype(np.float64)
    x = oracle.bf16_widen(np.asarray(xb).reshape(rows, in_w)).astype(np.float64)
    y = x @ w.T
    return y if bias is None else y + np.asarray(bias, dtype=np.float64)


PREFILL_TYPES = [GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_Q8_0, GGML_IQ2_S, GGML_IQ3_S]


@pytest.mark.parametrize("typ", PREFILL_TYPES)
@pytest.mark.parametrize("rows,in_w,out_w", [(16, 256, 16), (33, 512, 100), (128, 1024, 81), (200, 768, 160),
                                             (512, 1024, 300), (700, 512, 75), (300, 2304, 130)])
def test_prefill_matmul_vs_oracle(lane, typ, rows, in_w, out_w):
    payload = _random_payload(typ, out_w, in_w, seed=rows + in_w + out_w)
    xb = synth.to_bf16_bits(synth.activations(rows, in_w, seed=17))
    bias = np.random.default_rng(5).standard_normal(out_w).astype(np.float32) * np.float32(0.01)
    mat = HipQuantizedMatrix(payload, typ, out_w, in_w)
    x = lane.upload_raw(xb)
    b = lane.upload_raw(bias)
    y = lane.allocate(rows * out_w + 2)
    lane.fill_u32(y, NAN_BITS, rows * out_w + 2)
    mat.forward_bf16(lane, x, b, rows, out=y)
    lane.synchronize()
    got = lane.read(y)
    assert np.isnan(got[-1]) and np.isnan(got[-2])
    got = got[:-2].reshape(rows, out_w)
    assert np.all(np.isfinite(got))
    assert oracle.rel_l2(got, _bf16_weight_product(typ, payload, xb, bias, rows, in_w, out_w)) <= PREFILL_TIGHT_BAR
    if in_w * out_w >= 32768:
        ref, _ = oracle.linear_f64(typ, payload, xb, bias, rows, in_w, out_w, x_is_bf16=True)
        rel = oracle.rel_l2(got, ref)
        assert rel <= PREFILL_BAR, rel
    for buf in (x, b, y):
        buf.dispose()
    mat.dispose()


def test_prefill_matmul_rejects_other_types_and_widths(lane):
    from ctypes import c_void_p
    x = lane.allocate(256)
    w = lane.allocate(256)
    y = lane.allocate(4)
    # GGML type 2 (Q4_0) is no matrix storage of the reference (Qwen35Gguf.cs:12-13)
    status = lane._lib.nnhip_quant_matmul_bf16(lane._handle, 2, c_void_p(x.ptr), c_void_p(w.ptr), None, c_void_p(y.ptr), 1, 256, 1)
    assert status == 2
    w.dispose()
    y.dispose()
    mat = HipQuantizedMatrix(np.zeros(34 * 4, np.uint8), GGML_Q8_0, 1, 128)
    with pytest.raises(NnHipError) as e:
        mat.forward_bf16(lane, x, None, 1)
    assert e.value.status == 3                      # Q8_0 rows must hold a multiple of 256 weights here
    x.dispose()
    mat.dispose()


@pytest.mark.parametrize("typ", [GGML_Q5_K, GGML_Q6_K, GGML_Q8_0, GGML_IQ2_S, GGML_IQ3_S])
def test_prefill_matmul_model_width_sample(lane, typ):
    """A 5120-wide strip at M = 512 (the 256-row tiles, nine column tiles) for the other formats."""
    in_w, out_w, rows = 5120, 1500, 512
    payload = _random_payload(typ, out_w, in_w, 77)
    xb = synth.to_bf16_bits(synth.activations(rows, in_w, 4001))
    mat = HipQuantizedMatrix(payload, typ, out_w, in_w)
    x = lane.upload_raw(xb)
    got = lane.read(mat.forward_bf16(lane, x, None, rows)).reshape(rows, out_w)
    pick = np.arange(0, rows, 16)
    ref, _ = oracle.linear_f64(typ, payload, xb[pick], None, len(pick), in_w, out_w, x_is_bf16=True)
    assert oracle.rel_l2(got[pick], ref) <= PREFILL_BAR
    assert oracle.rel_l2(got[pick], _bf16_weight_product(typ, payload, xb[pick], None, len(pick), in_w, out_w)) <= PREFILL_TIGHT_BAR
    x.dispose()
    mat.dispose()


def test_prefill_matmul_full_width_sample(lane):
    """The benchmark prefill shape (Q4_K 17408 x 5120) at M = 128: every output of 16 sampled rows against the oracle."""
    in_w, out_w, rows = 5120, 17408, 128
    payload = synth.matrix(GGML_Q4_K, out_w, in_w, 2001)
    xb = synth.to_bf16_bits(synth.activations(rows, in_w, 4000))
    mat = HipQuantizedMatrix(payload, GGML_Q4_K, out_w, in_w)
    x = lane.upload_raw(xb)
    got = lane.read(mat.forward_bf16(lane, x, None, rows)).reshape(rows, out_w)
    pick = np.arange(0, rows, 8)
    ref, _ = oracle.linear_f64(GGML_Q4_K, payload, xb[pick], None, len(pick), in_w, out_w, x_is_bf16=True)
    rel = oracle.rel_l2(got[pick], ref)
    print(f"prefill 128x5120x17408 rel-L2 = {rel:.3e}")
    assert rel <= PREFILL_BAR
    x.dispose()
    mat.dispose()


# ----------------------------------------------------------------------------------------------- bfloat16 storage

def test_prefill_matmul_bf16_weights(lane):
    """Unquantized bfloat16 matrices through the prefill mat-mul: the weights are exact, so the product agrees with
    float64 to FP32 accumulation accuracy."""
    from nntrain_amd import GGML_BF16
    for rows, in_w, out_w in [(16, 256, 16), (200, 768, 160), (512, 1024, 300), (300, 2304, 130)]:
        rng = np.random.default_rng(rows + in_w)
        wb = synth.to_bf16_bits(rng.standard_normal((out_w, in_w), dtype=np.float32) * np.float32(0.02))
        xb = synth.to_bf16_bits(synth.activations(rows, in_w, seed=29))
        bias = rng.standard_normal(out_w).astype(np.float32) * np.float32(0.01)
        mat = HipQuantizedMatrix(wb.view(np.uint8).reshape(-1), GGML_BF16, out_w, in_w)
        x, b = lane.upload_raw(xb), lane.upload_raw(bias)
        got = lane.read(mat.forward_bf16(lane, x, b, rows)).reshape(rows, out_w)
        ref = oracle.bf16_widen(xb).astype(np.float64) @ oracle.bf16_widen(wb).astype(np.float64).T + bias.astype(np.float64)
        assert oracle.rel_l2(got, ref) <= PREFILL_TIGHT_BAR
        x.dispose()
        b.dispose()
        mat.dispose()


def test_bf16_matrix_storage(lane):
    """Unquantized bfloat16 matrices (the reference's "bf16" matrix storage, Qwen35Gguf.cs:12-13): widening is exact,
    the mat-vec meets the same bar as the block formats, rows are independent, the batched entry is bit-identical."""
    from nntrain_amd import GGML_BF16
    from nntrain_amd.native import MatvecDesc
    from ctypes import c_void_p
    for in_w, out_w, rows in [(64, 1, 1), (512, 7, 3), (5376, 131, 1), (21504, 33, 2)]:
        payload = synth.matrix(GGML_BF16, out_w, in_w, 40 + out_w)
        want = oracle.dequantize(GGML_BF16, payload)
        assert np.array_equal(_bits(want), payload.view("<u2").astype(np.uint32) << 16)
        mat = HipQuantizedMatrix(payload, GGML_BF16, out_w, in_w)
        assert np.array_equal(_bits(lane.read(mat.dequantize(lane))), _bits(want))
        assert np.array_equal(_bits(lane.read(mat.dequantize(lane, row=out_w - 1))), _bits(want[-in_w:]))
        x = synth.activations(rows, in_w, 6)
        bias = np.random.default_rng(3).standard_normal(out_w).astype(np.float32)
        y = _run_matvec(lane, GGML_BF16, payload, x, bias, rows, in_w, out_w)
        ref, asum = oracle.linear_f64(GGML_BF16, payload, x, bias, rows, in_w, out_w)
        _check_against_f64(y, ref, asum)
        y1 = np.stack([_run_matvec(lane, GGML_BF16, payload, x[r:r + 1], bias, 1, in_w, out_w)[0] for r in range(rows)])
        assert np.array_equal(_bits(y), _bits(y1))
        xb, bb, yb = lane.upload_raw(x), lane.upload_raw(bias), lane.allocate(rows * out_w)
        desc = (MatvecDesc * 1)(MatvecDesc(xb.ptr, mat.device_payload(lane).ptr, bb.ptr, yb.ptr, GGML_BF16, rows, in_w, out_w))
        assert lane._lib.nnhip_quant_matvec_batch(lane._handle, desc, 1) == 0
        assert np.array_equal(_bits(lane.read(yb)), _bits(y.reshape(-1)))
        for b in (xb, bb, yb):
            b.dispose()
        mat.dispose()
    lib, h = lane._lib, lane._handle
    buf = lane.allocate(4096)
    assert lib.nnhip_quant_matvec(h, GGML_BF16, c_void_p(buf.ptr), c_void_p(buf.ptr), None, c_void_p(buf.ptr), 1, 96, 2) == 3
    assert lib.nnhip_dequantize(h, GGML_BF16, c_void_p(buf.ptr), c_void_p(buf.ptr), 6) == 3
    assert lib.nnhip_dequantize(h, GGML_BF16, c_void_p(buf.ptr), c_void_p(buf.ptr), 8) == 0
    buf.dispose()
