"""ctypes binding of libnnhip.so - one declaration per entry point of include/nnhip.h.

This is the Python counterpart of the LibraryImport class a C# maintainer adds to NNtrain (bindings/csharp/NnHipNative.cs);
it declares argument types only and converts non-zero statuses to exceptions the way OpenClNative.Check does
(NNtrain.Arc/OpenClNative.cs:37-41).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, byref, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint16, c_uint32, \
    c_uint64, c_void_p
from pathlib import Path

ABI_MAJOR = 1
OPTION_ROW_STEP_ONLY = 1   # nnhip_lane_set_option: every mat-vec on the FP32 row-step kernels

STATUS_NAMES = {
    0: "OK", 1: "INVALID_ARGUMENT", 2: "UNSUPPORTED_TYPE", 3: "INCOMPLETE_BLOCKS", 4: "OUT_OF_MEMORY", 5: "HIP",
    6: "NO_DEVICE", 7: "BAD_HANDLE", 8: "TOO_LARGE",
}


class NnHipError(RuntimeError):
    def __init__(self, status: int, operation: str, message: str):
        super().__init__(f"nnhip {operation} failed ({STATUS_NAMES.get(status, status)}): {message}")
        self.status = status
        self.operation = operation
        self.native_message = message


class ErrorInfo(Structure):
    _fields_ = [("struct_size", c_uint32), ("abi_version", c_uint32), ("sequence", c_uint64), ("status", c_int32),
                ("device_index", c_int32), ("operation", c_uint32), ("reserved", c_uint32)]


class LaneCounters(Structure):
    _fields_ = [("struct_size", c_uint32), ("driver_allocations", c_uint32), ("h2d_bytes", c_uint64), ("d2h_bytes", c_uint64),
                ("allocated_bytes", c_uint64), ("peak_allocated_bytes", c_uint64), ("kernel_launches", c_uint64)]


class MatvecDesc(Structure):
    _fields_ = [("x", c_void_p), ("w", c_void_p), ("bias", c_void_p), ("y", c_void_p), ("ggml_type", c_uint32),
                ("rows", c_int32), ("in_w", c_int32), ("out_w", c_int32)]


class FusedMatvecDesc(Structure):
    _fields_ = [("struct_size", c_uint32), ("ggml_type", c_uint32), ("pre_op", c_uint32), ("epsilon", c_float),
                ("x", c_void_p), ("x2", c_void_p), ("norm_weight", c_void_p), ("x_out", c_void_p), ("sum_out", c_void_p),
                ("w", c_void_p), ("bias", c_void_p), ("addend", c_void_p), ("y", c_void_p), ("in_w", c_int32),
                ("out_w", c_int32), ("lora_z", c_void_p), ("lora_b", c_void_p), ("lora_rank", c_int32),
                ("lora_scale", c_float), ("x_head_width", c_int32), ("x_head_group", c_int32), ("post_op", c_uint32),
                ("reserved", c_uint32)]


class MatvecPlanInfo(Structure):
    _fields_ = [("struct_size", c_uint32), ("kernel", c_int32), ("threads", c_int32), ("rows_per_step", c_int32),
                ("steps", c_int32), ("groups", c_int32), ("row_tile", c_int32), ("ring_depth", c_int32),
                ("result_buffer_floats", c_int32), ("dynamic_lds_bytes", c_int32)]


class BatchLaunchInfo(Structure):
    _fields_ = [("struct_size", c_uint32), ("ggml_type", c_uint32), ("kernel", c_int32), ("in_w", c_int32),
                ("entries", c_int32), ("units", c_int32), ("groups", c_int32), ("threads", c_int32),
                ("rows_per_pass", c_int32), ("consecutive_runs", c_int32), ("stage_buffers", c_int32),
                ("activations_in_lds", c_int32), ("dynamic_lds_bytes", c_int32)]


PRE_NONE, PRE_RMS_NORM, PRE_SILU_MULTIPLY = 0, 1, 2
POST_NONE, POST_SILU_PAIR = 0, 1

# name -> (restype, argtypes); exactly the prototypes of include/nnhip.h
PROTOTYPES = {
    "nnhip_abi_version": (c_uint32, []),
    "nnhip_last_error": (c_int, [POINTER(ErrorInfo), c_size_t]),
    "nnhip_last_error_message": (c_int, [c_char_p, c_int]),
    "nnhip_device_count": (c_int, [POINTER(c_int)]),
    "nnhip_device_name": (c_int, [c_int, c_char_p, c_int]),
    "nnhip_device_info": (c_int, [c_int, POINTER(c_int), POINTER(c_uint64)]),
    "nnhip_type_block": (c_int, [c_uint32, POINTER(c_int), POINTER(c_int)]),
    "nnhip_matrix_bytes": (c_int, [c_uint32, c_int, c_int, POINTER(c_uint64)]),
    "nnhip_lane_create": (c_int, [c_int, POINTER(c_void_p)]),
    "nnhip_lane_destroy": (c_int, [c_void_p]),
    "nnhip_alloc": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "nnhip_free": (c_int, [c_void_p, c_void_p]),
    "nnhip_lane_trim": (c_int, [c_void_p]),
    "nnhip_upload": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p, c_size_t]),
    "nnhip_upload_from_file": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_uint64, c_size_t]),
    "nnhip_download": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p, c_size_t]),
    "nnhip_copy": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p, c_size_t, c_size_t]),
    "nnhip_fill_u32": (c_int, [c_void_p, c_void_p, c_size_t, c_uint32, c_size_t]),
    "nnhip_synchronize": (c_int, [c_void_p]),
    "nnhip_lane_get_counters": (c_int, [c_void_p, POINTER(LaneCounters), c_size_t]),
    "nnhip_lane_stream": (c_int, [c_void_p, POINTER(c_void_p)]),
    "nnhip_lane_set_option": (c_int, [c_void_p, c_uint32, c_int64]),
    "nnhip_lane_get_option": (c_int, [c_void_p, c_uint32, POINTER(c_int64)]),
    "nnhip_dequantize": (c_int, [c_void_p, c_uint32, c_void_p, c_void_p, c_int64]),
    "nnhip_quant_matvec": (c_int, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]),
    "nnhip_matvec_plan": (c_int, [c_uint32, c_int, c_int, c_int, c_int, POINTER(MatvecPlanInfo)]),
    "nnhip_matvec_batch_plan": (c_int, [POINTER(MatvecDesc), c_int, c_int, POINTER(BatchLaunchInfo), c_int, POINTER(c_int)]),
    "nnhip_quant_matvec_batch": (c_int, [c_void_p, POINTER(MatvecDesc), c_int]),
    "nnhip_quant_matvec_batch_static": (c_int, [c_void_p, POINTER(MatvecDesc), c_int]),
    "nnhip_quant_matvec_fused": (c_int, [c_void_p, POINTER(FusedMatvecDesc)]),
    "nnhip_quant_matmul": (c_int, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]),
    "nnhip_quant_matmul_split": (c_int, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]),
    "nnhip_quant_matmul_bf16": (c_int, [c_void_p, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]),
    "nnhip_rms_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float]),
    "nnhip_add_rms_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float]),
    "nnhip_silu_multiply": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int]),
    "nnhip_add_in_place": (c_int, [c_void_p, c_void_p, c_void_p, c_int]),
    "nnhip_first_token_attention": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]),
    "nnhip_lora_a": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]),
    "nnhip_lora_b": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float]),
    "nnhip_event_create": (c_int, [c_void_p, POINTER(c_void_p)]),
    "nnhip_event_destroy": (c_int, [c_void_p, c_void_p]),
    "nnhip_event_record": (c_int, [c_void_p, c_void_p]),
    "nnhip_event_elapsed_ms": (c_int, [c_void_p, c_void_p, c_void_p, POINTER(c_float)]),
    "nnhip_graph_begin": (c_int, [c_void_p]),
    "nnhip_graph_end": (c_int, [c_void_p, POINTER(c_void_p)]),
    "nnhip_graph_launch": (c_int, [c_void_p, c_void_p]),
    "nnhip_graph_destroy": (c_int, [c_void_p, c_void_p]),
}

_lib = None


def library_path() -> Path:
    override = os.environ.get("NNHIP_LIBRARY")
    return Path(override) if override else Path(__file__).resolve().parent / "csrc" / "libnnhip.so"


def load_library() -> ctypes.CDLL:
    """Load libnnhip.so and check the ABI major version.  Raises if the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not path.exists():
        raise FileNotFoundError(
            f"{path} is missing: build it with `make -C nntrain_amd/csrc` (or __graft_entry__.build()); "
            "there is no CPU fallback for the quantized linear path")
    lib = ctypes.CDLL(str(path))
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    packed = lib.nnhip_abi_version()
    if (packed >> 16) != ABI_MAJOR:
        raise RuntimeError(f"libnnhip.so reports ABI {packed >> 16}.{packed & 0xffff}; this host layer needs major {ABI_MAJOR}")
    _lib = lib
    return lib


def abi_version() -> tuple[int, int]:
    packed = load_library().nnhip_abi_version()
    return packed >> 16, packed & 0xFFFF


def last_error() -> tuple[ErrorInfo, str]:
    lib = load_library()
    info = ErrorInfo()
    lib.nnhip_last_error(byref(info), ctypes.sizeof(info))
    buf = ctypes.create_string_buffer(256)
    lib.nnhip_last_error_message(buf, len(buf))
    return info, buf.value.decode("utf-8", "replace")


def check(status: int, operation: str) -> None:
    if status != 0:
        _, message = last_error()
        raise NnHipError(status, operation, message)
