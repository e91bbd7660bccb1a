"""HipExecutionLane: one device, one in-order HIP stream, and the buffers it owns.

Mirrors the part of ArcExecutionLane the quantized operator uses (NNtrain.Arc/ArcExecutionLane.cs): UploadRaw :322,
Allocate :241, AllocateBytes :271, Read :334, Synchronize :658, the byte counters :71-91 and ArcBuffer :917-931.
"""
from __future__ import annotations

import contextlib
import ctypes
from ctypes import byref, c_float, c_int, c_uint64, c_void_p

import numpy as np

from . import native
from .native import check


class HipBuffer:
    """Device allocation owned by a lane (the reference's ArcBuffer).  Dispose frees it; the lane frees leaks."""

    def __init__(self, lane: "HipExecutionLane", ptr: int, nbytes: int):
        self.lane = lane
        self.ptr = ptr
        self.nbytes = nbytes

    @property
    def disposed(self) -> bool:
        return self.ptr == 0

    def dispose(self) -> None:
        if self.ptr and not self.lane.disposed:
            check(self.lane._lib.nnhip_free(self.lane._handle, c_void_p(self.ptr)), "free")
        self.ptr = 0

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.dispose()

    def _require(self) -> int:
        if not self.ptr:
            raise ValueError("buffer has been disposed")
        return self.ptr

    def view(self, offset_bytes: int, nbytes: int) -> "HipBuffer":
        """A window of this allocation that does not own it (disposing the view frees nothing)."""
        if offset_bytes < 0 or nbytes <= 0 or offset_bytes + nbytes > self.nbytes:
            raise ValueError("view exceeds the buffer")
        return _HipBufferView(self.lane, self._require() + offset_bytes, nbytes)


class _HipBufferView(HipBuffer):
    def dispose(self) -> None:
        self.ptr = 0


class HipEvent:
    def __init__(self, lane: "HipExecutionLane"):
        self.lane = lane
        h = c_void_p()
        check(lane._lib.nnhip_event_create(lane._handle, byref(h)), "event_create")
        self.handle = h

    def record(self) -> "HipEvent":
        check(self.lane._lib.nnhip_event_record(self.lane._handle, self.handle), "event_record")
        return self

    def dispose(self) -> None:
        if self.handle:
            check(self.lane._lib.nnhip_event_destroy(self.lane._handle, self.handle), "event_destroy")
            self.handle = None


class HipExecutionLane:
    def __init__(self, device: int = 0):
        self._lib = native.load_library()
        h = c_void_p()
        check(self._lib.nnhip_lane_create(device, byref(h)), "lane_create")
        self._handle = h
        self.device = device
        cu, mem = c_int(), c_uint64()
        check(self._lib.nnhip_device_info(device, byref(cu), byref(mem)), "device_info")
        self.compute_units = cu.value
        self.total_memory_bytes = mem.value
        # per-kernel device timing (ArcExecutionLane.KernelMilliseconds / KernelTimings, ArcExecutionLane.cs:87-92):
        # off by default; when on, every operation is bracketed by two events that synchronize() turns into times
        self.collect_kernel_events = False
        self.kernel_milliseconds = 0.0
        self.kernel_timings: dict[str, float] = {}
        self._pending_events: list = []
        self._event_pool: list = []
        self._capturing = False

    # ---- enumeration (ArcDevices.Enumerate) ----
    @staticmethod
    def device_count() -> int:
        lib = native.load_library()
        n = c_int()
        check(lib.nnhip_device_count(byref(n)), "device_count")
        return n.value

    @staticmethod
    def device_name(device: int = 0) -> str:
        lib = native.load_library()
        buf = ctypes.create_string_buffer(256)
        check(lib.nnhip_device_name(device, buf, len(buf)), "device_name")
        return buf.value.decode()

    @property
    def disposed(self) -> bool:
        return self._handle is None

    def dispose(self) -> None:
        if self._handle is not None:
            for _, start, stop in self._pending_events:
                self._event_pool += [start, stop]
            self._pending_events.clear()
            for e in self._event_pool:
                e.dispose()
            self._event_pool.clear()
            h, self._handle = self._handle, None
            check(self._lib.nnhip_lane_destroy(h), "lane_destroy")

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.dispose()

    # ---- memory ----
    def allocate_bytes(self, nbytes: int) -> HipBuffer:
        p = c_void_p()
        check(self._lib.nnhip_alloc(self._handle, nbytes, byref(p)), "alloc")
        return HipBuffer(self, p.value, nbytes)

    def trim(self) -> None:
        """Drain the stream and return the blocks kept for reuse to the driver."""
        check(self._lib.nnhip_lane_trim(self._handle), "lane_trim")

    def allocate(self, elements: int) -> HipBuffer:
        """FP32 elements, as ArcExecutionLane.Allocate."""
        return self.allocate_bytes(4 * elements)

    def upload_raw(self, values) -> HipBuffer:
        """Upload a host array byte for byte (ArcExecutionLane.UploadRaw)."""
        a = np.ascontiguousarray(values)
        buf = self.allocate_bytes(max(a.nbytes, 4))
        self.write(buf, a)
        return buf

    def write(self, buf: HipBuffer, values, offset: int = 0) -> None:
        a = np.ascontiguousarray(values)
        if offset + a.nbytes > buf.nbytes:
            raise ValueError("write exceeds the buffer")
        check(self._lib.nnhip_upload(self._handle, c_void_p(buf._require()), offset, a.ctypes.data_as(c_void_p), a.nbytes),
              "upload")

    def write_from_file(self, buf: HipBuffer, fd: int, file_offset: int, nbytes: int, offset: int = 0) -> None:
        """`nbytes` bytes at `file_offset` of the open file `fd` into the buffer at `offset`: read and copied by the
        library through its pinned staging buffers, a piece travelling while the next is read."""
        if nbytes < 0 or offset < 0 or offset + nbytes > buf.nbytes:
            raise ValueError("write exceeds the buffer")
        check(self._lib.nnhip_upload_from_file(self._handle, c_void_p(buf._require()), offset, fd, file_offset, nbytes), "upload")

    def read(self, buf: HipBuffer, dtype=np.float32, count: int | None = None, offset: int = 0) -> np.ndarray:
        itemsize = np.dtype(dtype).itemsize
        if count is None:
            count = (buf.nbytes - offset) // itemsize
        out = np.empty(count, dtype=dtype)
        if offset + out.nbytes > buf.nbytes:
            raise ValueError("read exceeds the buffer")
        check(self._lib.nnhip_download(self._handle, c_void_p(buf._require()), offset, out.ctypes.data_as(c_void_p),
                                       out.nbytes), "download")
        return out

    def copy(self, dst: HipBuffer, src: HipBuffer, nbytes: int, dst_offset: int = 0, src_offset: int = 0) -> None:
        if dst_offset + nbytes > dst.nbytes or src_offset + nbytes > src.nbytes:
            raise ValueError("copy exceeds a buffer")
        check(self._lib.nnhip_copy(self._handle, c_void_p(dst._require()), dst_offset, c_void_p(src._require()), src_offset,
                                   nbytes), "copy")

    def fill_u32(self, buf: HipBuffer, value: int, count: int, offset: int = 0) -> None:
        if offset + 4 * count > buf.nbytes:
            raise ValueError("fill exceeds the buffer")
        check(self._lib.nnhip_fill_u32(self._handle, c_void_p(buf._require()), offset, value & 0xFFFFFFFF, count), "fill")

    def synchronize(self) -> None:
        check(self._lib.nnhip_synchronize(self._handle), "synchronize")
        self._drain_events()

    # ---- per-kernel timing (ArcExecutionLane.RecordKernelTime, ArcExecutionLane.cs:727-742) ----
    @contextlib.contextmanager
    def kernel(self, name: str):
        """Brackets one operation with device events when collect_kernel_events is set (not while a graph is captured)."""
        if not self.collect_kernel_events or self._capturing:
            yield
            return
        start = self._event_pool.pop() if self._event_pool else HipEvent(self)
        stop = self._event_pool.pop() if self._event_pool else HipEvent(self)
        start.record()
        try:
            yield
        finally:
            stop.record()
            self._pending_events.append((name, start, stop))

    def _drain_events(self) -> None:
        for name, start, stop in self._pending_events:
            ms = self.elapsed_ms(start, stop)
            self.kernel_milliseconds += ms
            self.kernel_timings[name] = self.kernel_timings.get(name, 0.0) + ms
            self._event_pool += [start, stop]
        self._pending_events.clear()

    def reset_profile(self) -> None:
        """ArcExecutionLane.ResetProfile (ArcExecutionLane.cs:56-65): only with nothing pending."""
        if self._pending_events:
            raise RuntimeError("Synchronize before resetting the profile.")
        self.kernel_milliseconds = 0.0
        self.kernel_timings.clear()

    # ---- counters (ArcExecutionLane.H2DBytes etc.) ----
    def counters(self) -> dict:
        c = native.LaneCounters()
        check(self._lib.nnhip_lane_get_counters(self._handle, byref(c), ctypes.sizeof(c)), "counters")
        return {"h2d_bytes": c.h2d_bytes, "d2h_bytes": c.d2h_bytes, "allocated_bytes": c.allocated_bytes,
                "peak_allocated_bytes": c.peak_allocated_bytes, "kernel_launches": c.kernel_launches,
                "driver_allocations": c.driver_allocations}

    # ---- options ----
    @property
    def row_step_only(self) -> bool:
        """Whether every mat-vec of this lane stays on the FP32 row-step kernels, so that a call with several input rows
        equals stacked single-row calls bit for bit (the property of Qwen35InferencePrefillLinearTests.cs:64-77), at the
        price of the shared matrix-core passes.  Off when a lane is created."""
        v = ctypes.c_int64()
        check(self._lib.nnhip_lane_get_option(self._handle, native.OPTION_ROW_STEP_ONLY, byref(v)), "lane_get_option")
        return bool(v.value)

    @row_step_only.setter
    def row_step_only(self, on: bool) -> None:
        check(self._lib.nnhip_lane_set_option(self._handle, native.OPTION_ROW_STEP_ONLY, 1 if on else 0), "lane_set_option")

    # ---- timing / replay ----
    def event(self) -> HipEvent:
        return HipEvent(self)

    def elapsed_ms(self, start: HipEvent, stop: HipEvent) -> float:
        ms = c_float()
        check(self._lib.nnhip_event_elapsed_ms(self._handle, start.handle, stop.handle, byref(ms)), "event_elapsed")
        return ms.value

    def graph_begin(self) -> None:
        check(self._lib.nnhip_graph_begin(self._handle), "graph_begin")
        self._capturing = True

    def graph_end(self):
        g = c_void_p()
        self._capturing = False
        check(self._lib.nnhip_graph_end(self._handle, byref(g)), "graph_end")
        return g

    def graph_launch(self, graph) -> None:
        check(self._lib.nnhip_graph_launch(self._handle, graph), "graph_launch")

    def graph_destroy(self, graph) -> None:
        check(self._lib.nnhip_graph_destroy(self._handle, graph), "graph_destroy")
