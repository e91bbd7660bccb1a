"""nnhip_quant_matvec_batch_static: the batched mat-vec whose descriptor table lives in the library's fixed device
workspace, for callers that cannot allocate.  Checked through the C ABI against nnhip_quant_matvec_batch (bit for bit)
and the CPU oracle, on two calls in a row, the second with a smaller batch; sizes beyond the workspace are rejected.
"""
from ctypes import c_void_p

import numpy as np
import pytest

import oracle
from nntrain_amd import GGML_IQ2_S, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_Q8_0, HipExecutionLane, synth
from nntrain_amd.native import MatvecDesc, check, last_error

pytestmark = pytest.mark.gpu

NAN_BITS = 0x7FC00000
STATIC_MAX_ENTRIES = 1024


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _batch(lane, shapes, seed):
    rng = np.random.default_rng(seed)
    items = []
    for i, (typ, in_w, out_w, rows) in enumerate(shapes):
        payload = synth.matrix(typ, out_w, in_w, seed=seed + i)
        x = rng.standard_normal((rows, in_w)).astype(np.float32)
        bias = rng.standard_normal(out_w).astype(np.float32) if i % 2 else None
        items.append(dict(typ=typ, in_w=in_w, out_w=out_w, rows=rows, payload=payload, x=x, bias=bias,
                          w=lane.upload_raw(payload), xd=lane.upload_raw(x),
                          bd=lane.upload_raw(bias) if bias is not None else None,
                          y_ref=lane.allocate(rows * out_w + 2), y_new=lane.allocate(rows * out_w + 2)))
    return items


def _descs(items, key):
    descs = (MatvecDesc * len(items))()
    for i, it in enumerate(items):
        descs[i] = MatvecDesc(it["xd"].ptr, it["w"].ptr, it["bd"].ptr if it["bd"] else None, it[key].ptr, it["typ"],
                              it["rows"], it["in_w"], it["out_w"])
    return descs


def _compare(lane, items):
    for it in items:
        n = it["rows"] * it["out_w"]
        a, b = lane.read(it["y_ref"]), lane.read(it["y_new"])
        assert np.isnan(b[-1]) and np.isnan(b[-2]), "guard elements past the output were overwritten"
        assert np.all(np.isfinite(b[:n]))
        assert np.array_equal(_bits(a[:n]), _bits(b[:n])), (it["typ"], it["in_w"], it["out_w"], it["rows"])
        ref, asum = oracle.linear_f64(it["typ"], it["payload"], it["x"], it["bias"], it["rows"], it["in_w"], it["out_w"])
        got = b[:n].reshape(it["rows"], it["out_w"])
        assert oracle.rel_l2(got, ref) <= 1e-5
        assert np.all(np.abs(got.astype(np.float64) - ref) <= 2e-6 + 3e-6 * asum)


def test_static_workspace_batch_matches_the_allocating_entry_point():
    with HipExecutionLane(0) as lane:
        lib, h = lane._lib, lane._handle
        first = _batch(lane, [(GGML_Q8_0, 5376, 300, 1), (GGML_Q4_K, 5120, 260, 1), (GGML_Q8_0, 64, 5, 2),
                              (GGML_Q6_K, 1024, 130, 3), (GGML_IQ2_S, 2048, 40, 1), (GGML_Q8_0, 160, 9, 1),
                              (GGML_Q8_0, 21504, 90, 1), (GGML_Q4_K, 256, 3, 60),
                              (GGML_Q5_K, 2560, 33000, 1)], seed=400)         # the last one: a matrix-core group
        second = _batch(lane, [(GGML_Q4_K, 1024, 70, 1), (GGML_Q8_0, 512, 64, 2)], seed=500)
        for items in (first, second):           # the second call is smaller: stale entries of the first stay behind it
            for it in items:
                for key in ("y_ref", "y_new"):
                    lane.fill_u32(it[key], NAN_BITS, it["rows"] * it["out_w"] + 2)
            check(lib.nnhip_quant_matvec_batch(h, _descs(items, "y_ref"), len(items)), "quant_matvec_batch")
            lane.synchronize()
            before = lane.counters()
            check(lib.nnhip_quant_matvec_batch_static(h, _descs(items, "y_new"), len(items)), "quant_matvec_batch_static")
            lane.synchronize()
            after = lane.counters()
            # driver_allocations counts every device or pinned-host allocation the library makes for the lane (buffers,
            # descriptor tables, staging): the static entry point must leave it alone
            for key in ("h2d_bytes", "d2h_bytes", "allocated_bytes", "peak_allocated_bytes", "driver_allocations"):
                assert after[key] == before[key], key
            _compare(lane, items)
        # exactly the workspace's capacity is accepted, one row more is refused and nothing is enqueued
        wide = lane.upload_raw(synth.matrix(GGML_Q8_0, 3, 256, seed=9))
        xs = np.random.default_rng(1).standard_normal((STATIC_MAX_ENTRIES + 1, 256)).astype(np.float32)
        xd = lane.upload_raw(xs)
        y_ref, y_new = lane.allocate((STATIC_MAX_ENTRIES + 1) * 3), lane.allocate((STATIC_MAX_ENTRIES + 1) * 3)
        full = (MatvecDesc * 1)()
        for y, fn in ((y_ref, lib.nnhip_quant_matvec_batch), (y_new, lib.nnhip_quant_matvec_batch_static)):
            full[0] = MatvecDesc(xd.ptr, wide.ptr, None, y.ptr, GGML_Q8_0, STATIC_MAX_ENTRIES, 256, 3)
            check(fn(h, full, 1), "batch at capacity")
        lane.synchronize()
        n = STATIC_MAX_ENTRIES * 3
        assert np.array_equal(_bits(lane.read(y_ref)[:n]), _bits(lane.read(y_new)[:n]))
        launches = lane.counters()["kernel_launches"]
        full[0] = MatvecDesc(xd.ptr, wide.ptr, None, y_new.ptr, GGML_Q8_0, STATIC_MAX_ENTRIES + 1, 256, 3)
        assert lib.nnhip_quant_matvec_batch_static(h, full, 1) == 8          # NNHIP_ERR_TOO_LARGE
        info, message = last_error()
        assert info.status == 8 and "1025" in message and "1024" in message
        assert lane.counters()["kernel_launches"] == launches
        assert lib.nnhip_quant_matvec_batch_static(h, full, 0) == 0
        assert lib.nnhip_quant_matvec_batch_static(h, None, 2) == 1
        # the first batch once more after all that: the workspace is rewritten by every call
        for it in first:
            lane.fill_u32(it["y_new"], NAN_BITS, it["rows"] * it["out_w"] + 2)
        check(lib.nnhip_quant_matvec_batch_static(h, _descs(first, "y_new"), len(first)), "quant_matvec_batch_static")
        lane.synchronize()
        _compare(lane, first)


def test_static_workspace_batch_inside_a_captured_graph():
    """The caller this entry point is for: a graph captured without any allocation, replayed between eager work."""
    with HipExecutionLane(0) as lane:
        lib, h = lane._lib, lane._handle
        items = _batch(lane, [(GGML_Q8_0, 1024, 200, 1), (GGML_Q4_K, 512, 90, 1), (GGML_Q4_K, 2560, 33000, 1)], seed=600)
        other = _batch(lane, [(GGML_Q6_K, 256, 31, 1)], seed=700)
        check(lib.nnhip_quant_matvec_batch(h, _descs(items, "y_ref"), len(items)), "quant_matvec_batch")
        lane.synchronize()
        before = lane.counters()["driver_allocations"]
        lane.graph_begin()
        check(lib.nnhip_quant_matvec_batch_static(h, _descs(items, "y_new"), len(items)), "quant_matvec_batch_static")
        assert lane.counters()["driver_allocations"] == before
        graph = lane.graph_end()
        for _ in range(3):
            for it in items:
                lane.fill_u32(it["y_new"], NAN_BITS, it["rows"] * it["out_w"] + 2)
            check(lib.nnhip_quant_matvec_batch_static(h, _descs(other, "y_new"), len(other)), "quant_matvec_batch_static")
            lane.synchronize()
            lane.graph_launch(graph)
            lane.synchronize()
            for it in items:
                n = it["rows"] * it["out_w"]
                assert np.array_equal(_bits(lane.read(it["y_ref"])[:n]), _bits(lane.read(it["y_new"])[:n]))
        lane.graph_destroy(graph)


def test_two_lanes_of_a_device_use_their_own_slices_of_the_workspace():
    """Each lane takes one slice of the device's fixed workspace at creation, so two lanes may run this entry point at
    the same time: both are left unsynchronized here while the other one enqueues."""
    with HipExecutionLane(0) as one, HipExecutionLane(0) as two:
        a = _batch(one, [(GGML_Q8_0, 5376, 3000, 1), (GGML_Q4_K, 5120, 2600, 1), (GGML_Q6_K, 1024, 130, 3)], seed=800)
        b = _batch(two, [(GGML_Q5_K, 2560, 2100, 1), (GGML_Q8_0, 512, 64, 2), (GGML_IQ2_S, 2048, 400, 1)], seed=900)
        for lane, items in ((one, a), (two, b)):
            for it in items:
                for key in ("y_ref", "y_new"):
                    lane.fill_u32(it[key], NAN_BITS, it["rows"] * it["out_w"] + 2)
            check(lane._lib.nnhip_quant_matvec_batch(lane._handle, _descs(items, "y_ref"), len(items)), "quant_matvec_batch")
            lane.synchronize()
        for _ in range(8):
            for lane, items in ((one, a), (two, b)):
                check(lane._lib.nnhip_quant_matvec_batch_static(lane._handle, _descs(items, "y_new"), len(items)),
                      "quant_matvec_batch_static")
        one.synchronize()
        two.synchronize()
        _compare(one, a)
        _compare(two, b)
