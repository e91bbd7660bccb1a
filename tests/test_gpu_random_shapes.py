"""Seeded random sweeps over shapes, row counts, scales and groupings of the mat-vec entry points against the float64
oracle: the fixed cases of the other files pin the known corners, these pin "nothing in between is special".  Every
output buffer carries two NaN guard words behind its end; the bars are the ones of the parity tests (relative L2 1e-5
and the reference's per-element bound 2e-6 + 3e-6 * sum|x w|, QwenQuantizedLinearFastTests.cs:45-62)."""
from ctypes import c_void_p

import numpy as np
import pytest

import oracle
from nntrain_amd import (GGML_IQ2_S, GGML_IQ3_S, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_Q8_0, HipExecutionLane, synth)
from nntrain_amd.native import MatvecDesc, check

pytestmark = pytest.mark.gpu

TYPES = {"Q8_0": GGML_Q8_0, "Q4_K": GGML_Q4_K, "Q5_K": GGML_Q5_K, "Q6_K": GGML_Q6_K, "IQ2_S": GGML_IQ2_S, "IQ3_S": GGML_IQ3_S}
NAN_BITS = 0x7FC00000


@pytest.fixture(scope="module")
def lane():
    with HipExecutionLane(0) as ln:
        yield ln


def _check(name, y_all, rows, out_w, typ, payload, x, bias, in_w):
    assert np.isnan(y_all[-1]) and np.isnan(y_all[-2]), f"{name}: a write behind the end of y"
    y = y_all[:-2].reshape(rows, out_w)
    ref, asum = oracle.linear_f64(typ, payload, x, bias, rows, in_w, out_w)
    assert np.all(np.isfinite(y)), name
    assert np.all(np.abs(y.astype(np.float64) - ref) <= 2e-6 + 3e-6 * asum), name
    if y.size >= 256:           # (a relative norm over a handful of values says nothing)
        assert oracle.rel_l2(y, ref) <= 1e-5, name


def test_random_batches(lane):
    """Batches of one block format and row length with one to eight matrices of unrelated heights (one of them large
    enough, now and then, to send the group to the matrix cores), one to five input rows each, shared or own
    activations of very different magnitudes, with and without bias."""
    rng = np.random.default_rng(20240611)
    lib, h = lane._lib, lane._handle
    widths = [1024, 1280, 2048, 2560, 3072, 4096, 5120, 5376, 6144, 8192]
    for case in range(48):
        tname = str(rng.choice(list(TYPES)))
        typ = TYPES[tname]
        in_w = int(rng.choice(widths))
        if tname in ("Q6_K", "IQ2_S", "IQ3_S") and (in_w // 256) % 2:
            in_w += 256
        n = int(rng.integers(1, 9))
        share = bool(rng.integers(0, 2))
        big = int(rng.choice([1, 7, 17, 300, 4000, 20000, 40000]))
        items, shared = [], None
        for i in range(n):
            out_w = big if i == 0 else int(rng.choice([1, 5, 16, 33, 250, 1000, 3000, 12000]))
            rows = int(rng.choice([1, 1, 1, 2, 3, 4, 5]))
            payload = synth.matrix(typ, out_w, in_w, seed=77000 + case * 10 + i)
            if share and shared is not None and shared[0].shape[0] == rows:
                x, xd = shared
            else:
                x = rng.standard_normal((rows, in_w)).astype(np.float32) * float(rng.choice([1e-3, 1.0, 50.0]))
                xd = lane.upload_raw(x)
                if share:
                    shared = (x, xd)
            bias = rng.standard_normal(out_w).astype(np.float32) if rng.integers(0, 2) else None
            items.append(dict(out_w=out_w, rows=rows, payload=payload, x=x, xd=xd, bias=bias, wd=lane.upload_raw(payload),
                              bd=lane.upload_raw(bias) if bias is not None else None, yd=lane.allocate(rows * out_w + 2)))
        descs = (MatvecDesc * n)()
        for i, it in enumerate(items):
            descs[i] = MatvecDesc(it["xd"].ptr, it["wd"].ptr, it["bd"].ptr if it["bd"] else None, it["yd"].ptr, typ, it["rows"],
                                  in_w, it["out_w"])
            lane.fill_u32(it["yd"], NAN_BITS, it["rows"] * it["out_w"] + 2)
        check(lib.nnhip_quant_matvec_batch(h, descs, n), "batch")
        lane.synchronize()
        for i, it in enumerate(items):
            name = f"case {case} {tname} in_w={in_w} matrix {i} of {[(t['out_w'], t['rows']) for t in items]} shared={share}"
            _check(name, lane.read(it["yd"]), it["rows"], it["out_w"], typ, it["payload"], it["x"], it["bias"], in_w)
        seen = set()
        for it in items:
            for key in ("xd", "wd", "bd", "yd"):
                b = it[key]
                if b is not None and id(b) not in seen:
                    seen.add(id(b))
                    b.dispose()
        lane.trim()


def test_random_single_calls_with_one_to_sixteen_rows(lane):
    """nnhip_quant_matvec over heights on both sides of the tile-count rules and every row count up to sixteen (row-step
    passes, row-tiled passes and shared passes on the matrix cores), rows scaled differently from each other."""
    rng = np.random.default_rng(20240612)
    widths = [1024, 2048, 2560, 4096, 5120, 5376]
    for case in range(40):
        tname = str(rng.choice(list(TYPES)))
        typ = TYPES[tname]
        in_w = int(rng.choice(widths))
        if tname in ("Q6_K", "IQ2_S", "IQ3_S") and (in_w // 256) % 2:
            in_w += 256
        rows = int(rng.integers(1, 17))
        out_w = int(rng.choice([100, 2049, 4100, 9000, 17408, 33000]))
        payload = synth.matrix(typ, out_w, in_w, seed=88000 + case)
        x = rng.standard_normal((rows, in_w)).astype(np.float32)
        x *= rng.choice([1e-2, 1.0, 30.0], size=(rows, 1)).astype(np.float32)
        bias = rng.standard_normal(out_w).astype(np.float32) if rng.integers(0, 2) else None
        xd, wd = lane.upload_raw(x), lane.upload_raw(payload)
        bd = lane.upload_raw(bias) if bias is not None else None
        yd = lane.allocate(rows * out_w + 2)
        lane.fill_u32(yd, NAN_BITS, rows * out_w + 2)
        check(lane._lib.nnhip_quant_matvec(lane._handle, typ, c_void_p(xd.ptr), c_void_p(wd.ptr), c_void_p(bd.ptr) if bd else None,
                                           c_void_p(yd.ptr), rows, in_w, out_w), "matvec")
        lane.synchronize()
        _check(f"case {case} {tname} in_w={in_w} out_w={out_w} rows={rows}", lane.read(yd), rows, out_w, typ, payload, x, bias, in_w)
        for b in (xd, wd, bd, yd):
            if b is not None:
                b.dispose()
        lane.trim()


def test_random_single_calls_on_long_rows(lane):
    """The same over rows of 6656 - 28672 values, where the planes of four input rows (and, from 24000 values on, of one)
    do not fit LDS beside the stage buffers: shared passes in the split form, a pass per input row, row-tiled and
    row-step passes, as the tile counts decide."""
    rng = np.random.default_rng(20240613)
    widths = [6656, 7168, 8192, 11264, 14336, 17408, 21504, 24576, 28672]
    for case in range(36):
        tname = str(rng.choice(list(TYPES)))
        typ = TYPES[tname]
        in_w = int(rng.choice(widths))
        if tname in ("Q6_K", "IQ2_S", "IQ3_S") and (in_w // 256) % 2:
            in_w += 256
        rows = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 12, 13, 16, 19]))
        out_w = int(rng.choice([37, 1030, 2049, 4100, 5120, 9000]))
        payload = synth.matrix(typ, out_w, in_w, seed=99000 + case)
        x = rng.standard_normal((rows, in_w)).astype(np.float32)
        x *= rng.choice([1e-2, 1.0, 30.0], size=(rows, 1)).astype(np.float32)
        bias = rng.standard_normal(out_w).astype(np.float32) if rng.integers(0, 2) else None
        xd, wd = lane.upload_raw(x), lane.upload_raw(payload)
        bd = lane.upload_raw(bias) if bias is not None else None
        yd = lane.allocate(rows * out_w + 2)
        lane.fill_u32(yd, NAN_BITS, rows * out_w + 2)
        check(lane._lib.nnhip_quant_matvec(lane._handle, typ, c_void_p(xd.ptr), c_void_p(wd.ptr), c_void_p(bd.ptr) if bd else None,
                                           c_void_p(yd.ptr), rows, in_w, out_w), "matvec")
        lane.synchronize()
        _check(f"case {case} {tname} in_w={in_w} out_w={out_w} rows={rows}", lane.read(yd), rows, out_w, typ, payload, x, bias, in_w)
        for b in (xd, wd, bd, yd):
            if b is not None:
                b.dispose()
        lane.trim()


def test_random_prefill_shapes(lane):
    """The bf16 matrix-core mat-mul over row counts around its tile sizes (16 .. 600), heights that do not fill a strip,
    every storage format, with the activations handed over as FP32 (rounded to bfloat16 on the device) or as bfloat16
    bits; against the oracle fed the same bfloat16 values, within the 2e-3 the bf16 path is held to."""
    from nntrain_amd import GGML_BF16, HipQuantizedMatrix
    rng = np.random.default_rng(20240613)
    types = dict(TYPES, BF16=GGML_BF16)
    for case in range(24):
        tname = str(rng.choice(list(types)))
        typ = types[tname]
        in_w = int(rng.choice([256, 512, 1024, 2560, 5120]))
        out_w = int(rng.choice([1, 17, 68, 136, 137, 500, 3000]))
        rows = int(rng.choice([16, 17, 100, 128, 129, 256, 300, 513, 600]))
        payload = synth.matrix(typ, out_w, in_w, seed=99000 + case)
        x = rng.standard_normal((rows, in_w)).astype(np.float32)
        bias = rng.standard_normal(out_w).astype(np.float32) if rng.integers(0, 2) else None
        bits = synth.to_bf16_bits(x)
        mat = HipQuantizedMatrix(payload, typ, out_w, in_w)
        bd = lane.upload_raw(bias) if bias is not None else None
        yd = lane.allocate(rows * out_w + 2)
        lane.fill_u32(yd, NAN_BITS, rows * out_w + 2)
        as_bits = bool(rng.integers(0, 2))
        xd = lane.upload_raw(bits if as_bits else x)
        if as_bits:
            mat.forward_bf16(lane, xd, bd, rows, out=yd)
        else:
            mat.forward(lane, xd, bd, rows, out=yd)             # rows >= 16: the same kernel behind the FP32 entry
        lane.synchronize()
        y_all = lane.read(yd)
        name = f"case {case} {tname} in_w={in_w} out_w={out_w} rows={rows} bf16 input={as_bits}"
        assert np.isnan(y_all[-1]) and np.isnan(y_all[-2]), f"{name}: a write behind the end of y"
        y = y_all[:-2].reshape(rows, out_w)
        ref, _ = oracle.linear_f64(typ, payload, bits, bias, rows, in_w, out_w, x_is_bf16=True)
        assert np.all(np.isfinite(y)), name
        assert oracle.rel_l2(y, ref) <= 2e-3, (name, oracle.rel_l2(y, ref))
        for b in (xd, bd, yd):
            if b is not None:
                b.dispose()
        mat.dispose()
        lane.trim()
