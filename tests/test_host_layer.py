"""CPU-side tests: the C ABI loads and exports what include/nnhip.h declares, host-layer validation, GGUF reader."""
import ctypes
import json
import re
import struct
from ctypes import byref, c_int, c_uint64, c_void_p

import numpy as np
import pytest

import nntrain_amd as nn
from nntrain_amd import native
from nntrain_amd.gguf import GgufReader, GgufReadLimits, InvalidDataError


def test_library_exports_every_declared_symbol():
    header = (native.library_path().parent.parent.parent / "include" / "nnhip.h").read_text()
    declared = set(re.findall(r"NNHIP_API\s+[\w\s\*]+?\b(nnhip_\w+)\s*\(", header))
    assert len(declared) >= 30
    lib = ctypes.CDLL(str(native.library_path()))
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in nnhip.h but not exported"
    assert declared == set(native.PROTOTYPES), declared ^ set(native.PROTOTYPES)


def _c_prototypes(header: str) -> dict:
    """name -> list of argument classes from nnhip.h: 'p' (pointer, size_t, uint64_t: one unsigned 64-bit register),
    'i32', 'u32', 'i64', 'f32'."""
    protos = {}
    for m in re.finditer(r"NNHIP_API\s+(?:int|uint32_t)\s+(nnhip_\w+)\s*\(([^;]*?)\)\s*;", header, re.S):
        args = []
        body = " ".join(m.group(2).split())
        if body != "void":
            for a in body.split(","):
                a = a.strip()
                if "*" in a or a.startswith("size_t"):
                    args.append("p")
                elif a.startswith("uint32_t"):
                    args.append("u32")
                elif a.startswith("int64_t"):
                    args.append("i64")
                elif a.startswith("uint64_t"):
                    args.append("p")
                elif a.startswith("float"):
                    args.append("f32")
                elif a.startswith("int"):
                    args.append("i32")
                else:
                    raise AssertionError(f"unclassified C argument {a!r} of {m.group(1)}")
        protos[m.group(1)] = args
    return protos


def test_csharp_declarations_match_the_header():
    """bindings/csharp/NnHipNative.cs is not compiled here, so every LibraryImport is checked against include/nnhip.h
    mechanically: same set of names, same arity, same 32/64-bit width and kind per argument, and the structures both
    bindings pass by pointer have the sizes the C compiler gives them."""
    root = native.library_path().parent.parent.parent
    protos = _c_prototypes((root / "include" / "nnhip.h").read_text())
    assert set(protos) == set(native.PROTOTYPES)
    cs = (root / "bindings" / "csharp" / "NnHipNative.cs").read_text()
    width = {"nint": "p", "nuint": "p", "int": "i32", "uint": "u32", "long": "i64", "ulong": "p", "float": "f32"}
    seen = {}
    for m in re.finditer(r"\[LibraryImport\(Library\)\]\s+internal static partial (\w+) (nnhip_\w+)\(([^)]*)\);", cs):
        ret, name, body = m.groups()
        args = []
        for a in filter(None, (x.strip() for x in body.split(","))):
            parts = a.split()
            if parts[0] == "out" or parts[-2].endswith("*"):
                args.append("p")
            else:
                args.append(width[parts[-2]])
        seen[name] = args
        assert ret == ("uint" if name == "nnhip_abi_version" else "int"), name
    assert set(seen) == set(protos), set(seen) ^ set(protos)
    for name, args in protos.items():
        assert seen[name] == args, (name, seen[name], args)
    # ctypes prototypes agree with the header as well
    kinds = {ctypes.c_int: "i32", ctypes.c_uint32: "u32", ctypes.c_int64: "i64", ctypes.c_float: "f32"}
    for name, (_, argtypes) in native.PROTOTYPES.items():
        got = [kinds.get(t, "p") for t in argtypes]
        assert got == protos[name], (name, got, protos[name])
    # structure sizes: C# field lists (4-byte scalars, 8-byte nint / ulong) against the ctypes structures
    sizes = {"uint": 4, "int": 4, "float": 4, "nint": 8, "ulong": 8}
    for cs_name, ct in (("ErrorInfo", native.ErrorInfo), ("LaneCounters", native.LaneCounters), ("MatvecDesc", native.MatvecDesc),
                        ("FusedMatvecDesc", native.FusedMatvecDesc), ("MatvecPlanInfo", native.MatvecPlanInfo),
                        ("BatchLaunchInfo", native.BatchLaunchInfo)):
        body = re.search(r"internal struct %s\s*\{(.*?)\n    \}" % cs_name, cs, re.S).group(1)
        fields = re.findall(r"internal (\w+) \w+;", body)
        offset = 0
        for f in fields:
            offset = (offset + sizes[f] - 1) // sizes[f] * sizes[f] + sizes[f]
        align = max(sizes[f] for f in fields)
        assert (offset + align - 1) // align * align == ctypes.sizeof(ct), (cs_name, offset, ctypes.sizeof(ct))
        assert len(fields) == len(ct._fields_), cs_name
    assert ctypes.sizeof(native.FusedMatvecDesc) == 136


def test_abi_version_and_struct_layouts():
    assert native.abi_version() == (1, 0)
    assert ctypes.sizeof(native.ErrorInfo) == 32      # the reference's NativeErrorInfo layout
    assert ctypes.sizeof(native.MatvecDesc) == 48
    assert ctypes.sizeof(native.LaneCounters) == 48
    assert ctypes.sizeof(native.MatvecPlanInfo) == 40
    assert ctypes.sizeof(native.FusedMatvecDesc) == 136


def test_geometry_queries_without_a_gpu():
    lib = native.load_library()
    e, b = c_int(), c_int()
    for typ, (elems, nbytes) in {8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210), 21: (256, 110), 22: (256, 82)}.items():
        assert lib.nnhip_type_block(typ, byref(e), byref(b)) == 0
        assert (e.value, b.value) == (elems, nbytes)
    assert lib.nnhip_type_block(2, byref(e), byref(b)) == 2
    n = c_uint64()
    assert lib.nnhip_matrix_bytes(8, 5376, 21504, byref(n)) == 0 and n.value == 122_830_848
    assert lib.nnhip_matrix_bytes(12, 5120, 17408, byref(n)) == 0 and n.value == 50_135_040
    assert lib.nnhip_matrix_bytes(13, 5120, 17408, byref(n)) == 0 and n.value == 61_276_160
    assert lib.nnhip_matrix_bytes(14, 5120, 17408, byref(n)) == 0 and n.value == 73_113_600
    assert lib.nnhip_matrix_bytes(22, 17408, 5120, byref(n)) == 0 and n.value == 28_549_120
    assert lib.nnhip_matrix_bytes(12, 5000, 10, byref(n)) == 3
    info, msg = native.last_error()
    assert info.status == 3 and "256" in msg and info.struct_size == 32


def test_matvec_plan_keeps_a_ring_turn_inside_the_result_buffer():
    """A workgroup of the row-step kernel parks ring_depth * rows_per_step * row_tile results in LDS before it can
    flush; the plan must keep that inside the buffer for every accepted shape (narrow rows with several input rows are
    the ones that would overrun)."""
    lib = native.load_library()
    info = native.MatvecPlanInfo(struct_size=ctypes.sizeof(native.MatvecPlanInfo))
    seen_tiles = set()
    for typ, widths in ((8, (64, 128, 192, 256, 320, 640, 1024, 5376, 21504)), (30, (64, 128, 256, 4096)),
                        (12, (256, 512, 5120, 17408)), (13, (256, 5120)), (14, (256, 5120)), (21, (256, 5120)),
                        (22, (256, 17408))):
        for in_w in widths:
            for out_w in (1, 2, 63, 300, 1000, 5000, 200_000, 1_000_000):
                for rows in (1, 2, 3, 4, 7, 16, 37):
                    assert lib.nnhip_matvec_plan(typ, rows, in_w, out_w, 256, byref(info)) == 0, (typ, in_w, out_w, rows)
                    if info.kernel == 2:
                        # several input rows of a K-quant / IQ2_S / IQ3_S / Q8_0 matrix on the matrix cores: 16-row tiles, four
                        # rows a pass and sixteen a launch (Q8_0 from three rows on: two stay with its row-tiled kernel); the
                        # floor is 2048 tiles x rows, 768 from three rows on except for Q8_0
                        assert (3 if typ == 8 else 2) <= rows and typ in (8, 12, 13, 14, 21, 22)
                        assert typ != 8 or in_w in (1024, 5376)         # (21504-wide planes of four rows do not fit LDS)
                        assert info.rows_per_step == 16 and info.threads % 128 == 0
                        if in_w == 17408 and info.row_tile == 1:
                            # four sets of planes do not fit LDS: a pass per input row, four rows a launch, from 1024 tiles x rows (IQ2_S: 512)
                            assert typ in (12, 22) and rows * -(-out_w // 16) >= (512 if typ == 22 else 1024)
                            assert info.steps == -(-out_w // 16) * min(rows, 4)
                            assert info.dynamic_lds_bytes + 2048 + (10240 if typ == 22 else 0) <= 160 * 1024
                        elif in_w == 17408:
                            # ... or shared passes in the split form (the planes of one group of block columns at a time) where
                            # the groups of four input rows make 3.5 rounds of tiles over the workgroups (IQ2_S: 2.5)
                            tiles = -(-out_w // 16)
                            assert typ in (12, 22) and info.row_tile == min(rows, 4)
                            assert 2 * -(-rows // 4) * tiles >= (5 if typ == 22 else 7) * 256
                            assert info.steps == tiles * -(-min(rows, 16) // 4)
                            # (the sums of a run's tiles take what the planes and the stage buffers leave)
                            assert info.dynamic_lds_bytes + 8192 + (10240 if typ == 22 else 0) <= 160 * 1024
                            seen_tiles.add((typ, "split"))
                        else:
                            assert rows * -(-out_w // 16) >= (768 if rows >= 3 and typ != 8 else 2048)
                            assert info.row_tile == min(rows, 4)
                            assert info.steps == -(-out_w // 16) * -(-min(rows, 16) // 4)
                            assert info.dynamic_lds_bytes + 8192 <= 160 * 1024
                        assert info.groups == min(info.steps, 256)
                        seen_tiles.add((typ, "matrix core"))
                        continue
                    if info.kernel != 0:
                        continue
                    assert info.ring_depth * info.rows_per_step * info.row_tile <= info.result_buffer_floats, \
                        (typ, in_w, out_w, rows, info.rows_per_step, info.row_tile)
                    assert info.rows_per_step * (in_w // 64) <= info.threads <= 1024
                    assert info.threads % 64 == 0 and 1 <= info.rows_per_step <= out_w
                    assert info.steps == -(-out_w // info.rows_per_step) and info.groups == min(info.steps, 256)
                    assert info.dynamic_lds_bytes <= 140 * 1024
                    seen_tiles.add((typ, info.row_tile))
    assert {(8, 1), (8, 2), (8, 4), (30, 4), (12, 1), (8, "matrix core"), (12, "matrix core"), (14, "matrix core"),
            (21, "matrix core"), (12, "split"), (22, "split")} <= seen_tiles
    # three rows reach the matrix cores at 768 tiles x rows, two rows at 2048
    assert lib.nnhip_matvec_plan(12, 3, 5120, 4096, 256, byref(info)) == 0 and info.kernel == 2
    assert lib.nnhip_matvec_plan(12, 3, 5120, 4000, 256, byref(info)) == 0 and info.kernel == 0
    assert lib.nnhip_matvec_plan(12, 2, 5120, 4096, 256, byref(info)) == 0 and info.kernel == 0
    assert lib.nnhip_matvec_plan(8, 4, 5376, 4096, 256, byref(info)) == 0 and info.kernel == 0
    assert lib.nnhip_matvec_plan(8, 1, 32 * 5, 19, 256, byref(info)) == 0 and info.kernel == 1   # odd block count
    assert lib.nnhip_matvec_plan(12, 1, 255, 19, 256, byref(info)) == 3
    assert lib.nnhip_matvec_plan(12, 1, 256 * 300, 19, 256, byref(info)) == 8
    assert lib.nnhip_matvec_plan(99, 1, 256, 19, 256, byref(info)) == 2
    info.struct_size = 8
    assert lib.nnhip_matvec_plan(12, 1, 256, 19, 256, byref(info)) == 1


def _batch_plan(lib, descs, compute_units=256, capacity=16):
    arr = (native.MatvecDesc * max(len(descs), 1))(*descs)
    out = (native.BatchLaunchInfo * max(capacity, 1))()
    for o in out:
        o.struct_size = ctypes.sizeof(native.BatchLaunchInfo)
    n = c_int(-1)
    rc = lib.nnhip_matvec_batch_plan(arr, len(descs), compute_units, out if capacity else None, capacity, byref(n))
    assert rc == 0, native.last_error()[1]
    return [out[i] for i in range(min(n.value, capacity))], n.value


def _desc(typ, rows, in_w, out_w, x=0x1000, w=0x100000, y=0x2000):
    # (addresses are compared and checked for alignment, never followed: no device is needed)
    return native.MatvecDesc(x=x, w=w, bias=None, y=y, ggml_type=typ, rows=rows, in_w=in_w, out_w=out_w)


def test_batch_plan_groups_a_models_projections_by_type_and_row_length():
    """The decode batch of a Q8_0 model: one matrix-core launch per row length, every 16-row tile counted once, runs of
    consecutive tiles per workgroup, and whole tiles in one stage buffer where rows are not a multiple of 128 bytes
    (5376 weights = 5712 bytes)."""
    lib = native.load_library()
    descs = []
    for layer in range(48):
        descs += [_desc(8, 1, 5376, 21504, x=0x1000 + layer * 0x10000), _desc(8, 1, 5376, 21504, x=0x1000 + layer * 0x10000),
                  _desc(8, 1, 21504, 5376, x=0x8000 + layer * 0x10000), _desc(8, 1, 4096, 5376, x=0xc000 + layer * 0x10000)]
    launches, n = _batch_plan(lib, descs)
    assert n == 3 and [(l.ggml_type, l.kernel, l.in_w) for l in launches] == [(8, 2, 5376), (8, 2, 21504), (8, 2, 4096)]
    assert [l.entries for l in launches] == [96, 48, 48]
    assert [l.units for l in launches] == [96 * 1344, 48 * 336, 48 * 336]
    for l in launches:
        assert l.groups == 256 and l.rows_per_pass == 1 and l.consecutive_runs == 1 and l.activations_in_lds == 1
        assert l.threads % 128 == 0 and 512 <= l.threads <= 768
        assert l.dynamic_lds_bytes + 2048 <= 160 * 1024
    assert [l.stage_buffers for l in launches] == [1, 2, 2]
    # a stage buffer of the 5376-wide launch holds a whole tile (16 rows of 5712 bytes) beside the four digit planes
    assert launches[0].dynamic_lds_bytes >= 16 * 5712 + 4 * 5376
    # fewer compute units than tiles or more: one workgroup per unit at most
    launches, _ = _batch_plan(lib, [_desc(8, 1, 4096, 16 * 2100)], compute_units=4096)
    assert launches[0].kernel == 2 and launches[0].groups == 2100


def test_batch_plan_threshold_counts_tiles_once_per_input_row():
    lib = native.load_library()
    # 2047 tiles: the row-step kernel; one more tile from a second matrix of the same type and row length: the matrix cores
    launches, n = _batch_plan(lib, [_desc(12, 1, 4096, 16 * 2047)])
    assert n == 1 and launches[0].kernel == 0 and launches[0].stage_buffers == 0
    launches, n = _batch_plan(lib, [_desc(12, 1, 4096, 16 * 2047), _desc(12, 1, 4096, 9)])
    assert n == 1 and launches[0].kernel == 2 and launches[0].units == 2048 and launches[0].entries == 2
    # a different row length or type does not count towards the group
    launches, n = _batch_plan(lib, [_desc(12, 1, 4096, 16 * 2047), _desc(12, 1, 5120, 16), _desc(13, 1, 4096, 16)])
    assert n == 2 and all(l.kernel == 0 for l in launches) and [l.ggml_type for l in launches] == [12, 13]
    assert launches[0].entries == 2 and launches[0].in_w == 5120
    # input rows count: 4 rows x 512 tiles
    launches, n = _batch_plan(lib, [_desc(12, 4, 4096, 16 * 512)])
    assert n == 1 and launches[0].kernel == 2 and launches[0].rows_per_pass == 4 and launches[0].units == 512
    launches, n = _batch_plan(lib, [_desc(12, 4, 4096, 16 * 511)])
    assert n == 1 and launches[0].kernel == 0 and launches[0].entries == 4
    # a weight pointer the 16-byte loads cannot take keeps a Q6_K matrix with the row-step kernel (4-byte alignment is its rule)
    launches, n = _batch_plan(lib, [_desc(14, 1, 4096, 16 * 3000, w=0x100004)])
    assert n == 1 and launches[0].kernel == 0
    # Q6_K, IQ2_S and IQ3_S rows must hold an even number of 256-blocks for the matrix cores
    for typ in (14, 22, 21):
        assert _batch_plan(lib, [_desc(typ, 1, 256 * 17, 16 * 3000)])[0][0].kernel == 0
        assert _batch_plan(lib, [_desc(typ, 1, 256 * 18, 16 * 3000)])[0][0].kernel == 2
    # below 1024 weights a row: never
    assert _batch_plan(lib, [_desc(12, 1, 768, 16 * 5000)])[0][0].kernel == 0


def test_batch_plan_shared_passes_and_tile_order():
    lib = native.load_library()
    # twenty matrices on one activation vector: every groups-th tile; a vector per matrix: runs of consecutive tiles
    shared, _ = _batch_plan(lib, [_desc(12, 1, 5120, 17408)] * 20)
    own, _ = _batch_plan(lib, [_desc(12, 1, 5120, 17408, x=0x1000 + i * 0x10000) for i in range(20)])
    assert shared[0].kernel == own[0].kernel == 2 and shared[0].units == own[0].units == 20 * 1088
    assert (shared[0].consecutive_runs, own[0].consecutive_runs) == (0, 1)
    assert shared[0].activations_in_lds == 0                  # (5120 = 20 blocks fit the register form)
    # two vectors (one change along the table) still deal every groups-th tile
    two, _ = _batch_plan(lib, [_desc(12, 1, 5120, 17408)] * 10 + [_desc(12, 1, 5120, 17408, x=0x9000)] * 10)
    assert two[0].consecutive_runs == 0
    # input rows of a descriptor share passes four at a time; K-quants from two rows on, Q8_0 from three
    for typ, rows, entries, per_pass in ((12, 2, 1, 2), (12, 4, 1, 4), (12, 6, 2, 4), (13, 9, 3, 4), (14, 16, 4, 4), (22, 5, 2, 4), (21, 5, 2, 4),
                                         (8, 2, 2, 1), (8, 3, 1, 3), (8, 7, 2, 4)):
        in_w = 5376 if typ == 8 else 5120 if typ != 22 else 4096
        launches, n = _batch_plan(lib, [_desc(typ, rows, in_w, 17408)])
        l = launches[0]
        assert n == 1 and l.kernel == 2 and (l.entries, l.rows_per_pass) == (entries, per_pass), (typ, rows, l.entries, l.rows_per_pass)
        assert l.units == entries * 1088 and l.activations_in_lds == 1
        assert l.dynamic_lds_bytes + (8192 if per_pass > 1 else 2048) + (2048 if typ in (21, 22) else 0) <= 160 * 1024
    # 21504-wide planes of four rows do not fit LDS: those rows get an entry each
    launches, _ = _batch_plan(lib, [_desc(8, 4, 21504, 16384)])
    assert launches[0].kernel == 2 and (launches[0].entries, launches[0].rows_per_pass) == (4, 1)
    # descriptors with and without shared passes of one type and row length make two launches
    launches, n = _batch_plan(lib, [_desc(12, 1, 4096, 16 * 2048), _desc(12, 3, 4096, 16 * 2048)])
    assert n == 2 and sorted(l.rows_per_pass for l in launches) == [1, 3]


def test_batch_plan_mixed_types_and_errors():
    lib = native.load_library()
    descs = [_desc(12, 1, 4096, 16 * 3000), _desc(14, 1, 4096, 16 * 3000), _desc(21, 1, 4096, 100), _desc(8, 1, 160, 19),
             _desc(22, 1, 4096, 16 * 3000), _desc(30, 2, 4096, 77), _desc(8, 1, 64, 5)]
    launches, n = _batch_plan(lib, descs)
    kinds = [(l.ggml_type, l.kernel) for l in launches]
    # matrix-core groups first, then the row-step launches in type order, then Q8_0 rows with an odd number of blocks
    assert n == 7 and kinds == [(12, 2), (14, 2), (22, 2), (8, 0), (21, 0), (30, 0), (8, 1)]
    assert launches[5].entries == 2 and launches[6].in_w == 160 and launches[6].entries == 1
    # a small capacity still reports the count and fills what fits
    few, n = _batch_plan(lib, descs, capacity=2)
    assert n == 7 and [(l.ggml_type, l.kernel) for l in few] == kinds[:2]
    none, n = _batch_plan(lib, descs, capacity=0)
    assert n == 7 and none == []
    assert _batch_plan(lib, [])[1] == 0
    # the descriptor checks of the batch itself
    n = c_int()
    out = (native.BatchLaunchInfo * 1)()
    out[0].struct_size = ctypes.sizeof(native.BatchLaunchInfo)
    one = (native.MatvecDesc * 1)

    def status(d, cus=256):
        return lib.nnhip_matvec_batch_plan(one(d), 1, cus, out, 1, byref(n))

    assert status(_desc(12, 1, 4096, 16, w=0x100004)) == 1 and "16-byte" in native.last_error()[1]
    assert status(_desc(12, 1, 4000, 16)) == 3
    assert status(_desc(99, 1, 4096, 16)) == 2
    assert status(_desc(12, 0, 4096, 16)) == 1
    assert status(_desc(12, 1, 256 * 300, 16)) == 8
    assert status(_desc(12, 1, 4096, 16, x=0)) == 1
    assert status(_desc(12, 1, 4096, 16), cus=0) == 1
    assert lib.nnhip_matvec_batch_plan(one(_desc(12, 1, 4096, 16)), 1, 256, out, 1, None) == 1
    # size limits of a batched call: 65535 input rows a descriptor, 2^20 mat-vec rows a call
    assert status(_desc(12, 65535, 256, 16)) == 0
    assert status(_desc(12, 65536, 256, 16)) == 8 and "65535" in native.last_error()[1]
    many = (native.MatvecDesc * 17)(*[_desc(12, 65535, 256, 16)] * 17)
    assert lib.nnhip_matvec_batch_plan(many, 16, 256, out, 1, byref(n)) == 0
    assert lib.nnhip_matvec_batch_plan(many, 17, 256, out, 1, byref(n)) == 8 and "split the batch" in native.last_error()[1]
    out[0].struct_size = 8
    assert status(_desc(12, 1, 4096, 16)) == 1 and "struct_size" in native.last_error()[1]


def test_bad_handles_are_reported_not_dereferenced():
    lib = native.load_library()
    assert lib.nnhip_synchronize(None) == 7
    assert lib.nnhip_upload_from_file(None, None, 0, 0, 0, 16) == 7
    p = c_void_p()
    assert lib.nnhip_alloc(None, 16, byref(p)) == 7
    assert lib.nnhip_quant_matvec(None, 8, None, None, None, None, 1, 32, 1) == 7


def test_quantized_matrix_constructor_validation():
    """Mirrors ArcQuantizedMatrix's constructor checks (NNtrain.Core/Serialization/ArcQuantizedMatrix.cs:20-32)."""
    with pytest.raises(TypeError):
        nn.HipQuantizedMatrix(None, nn.GGML_Q4_K, 1, 256)
    with pytest.raises(NotImplementedError):
        nn.HipQuantizedMatrix(b"\0" * 144, 0, 1, 256)              # F32 is not a quantized matrix type
    with pytest.raises(ValueError):
        nn.HipQuantizedMatrix(b"\0" * 144, nn.GGML_Q4_K, 0, 256)
    with pytest.raises(NotImplementedError):
        nn.HipQuantizedMatrix(b"\0" * 144, nn.GGML_Q4_K, 1, 128)   # incomplete 256-value block
    with pytest.raises(ValueError, match="expected 144"):
        nn.HipQuantizedMatrix(b"\0" * 145, nn.GGML_Q4_K, 1, 256)
    m = nn.HipQuantizedMatrix(b"\0" * (34 * 4), nn.GGML_Q8_0, 2, 64)
    assert (m.ggml_type, m.output_width, m.input_width, m.storage_bytes) == (8, 2, 64, 136)
    for typ in (8, 12, 13, 14, 21, 22):
        nn.HipQuantizedMatrix(np.zeros(nn.BLOCK_BYTES[typ] * 3, np.uint8), typ, 3, nn.BLOCK_ELEMS[typ])


# ------------------------------------------------------------------------------------------------ GGUF reader

def test_gguf_reader_reference_fixture(golden_dir):
    expected = json.loads((golden_dir / "qwen_gguf_expected.json").read_text())
    with GgufReader(str(golden_dir / "qwen_gguf_reference.gguf")) as r:
        assert r.version == 3 and r.data_offset == 480
        assert r.metadata["general.architecture"] == "qwen2"
        assert [t.name for t in r.tensors] == [t["name"] for t in expected["tensors"]]
        for want in expected["tensors"]:
            info = r.get_tensor(want["name"])
            assert info.type == want["type"] and list(info.shape) == list(want["shape"])
            assert info.byte_count() == want["payloadBytes"]
            assert len(r.read_tensor_bytes(info)) == want["payloadBytes"]
        q = r.get_tensor("q4_k_mixed.weight")
        assert r.matrix_dims(q) == (512, 7)           # GGUF shape is [input_width, output_width]
        with pytest.raises(KeyError):
            r.get_tensor("missing")
        with pytest.raises(EOFError):
            r.read_tensor_bytes(r.tensors[-1], 10_000)


def _gguf(tmp_path, *, magic=0x46554747, version=3, kvs=(), tensors=(), name="t.gguf", tail=b""):
    def s(x):
        b = x.encode()
        return struct.pack("<Q", len(b)) + b
    blob = struct.pack("<IIQQ", magic, version, len(tensors), len(kvs))
    for k, t, v in kvs:
        blob += s(k) + struct.pack("<I", t) + v
    for n, shape, typ, off in tensors:
        blob += s(n) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape)
        blob += struct.pack("<IQ", typ, off)
    p = tmp_path / name
    p.write_bytes(blob + tail)
    return str(p)


def test_gguf_reader_rejects_what_the_reference_rejects(tmp_path):
    with pytest.raises(InvalidDataError, match="Not a GGUF"):
        GgufReader(_gguf(tmp_path, magic=0x12345678))
    with pytest.raises(NotImplementedError, match="version 4"):
        GgufReader(_gguf(tmp_path, version=4))
    with pytest.raises(NotImplementedError, match="version 1"):
        GgufReader(_gguf(tmp_path, version=1))
    with pytest.raises(InvalidDataError, match="rank"):
        GgufReader(_gguf(tmp_path, tensors=[("w", (), 12, 0)], tail=b"\0" * 64))
    with pytest.raises(InvalidDataError, match="rank"):
        GgufReader(_gguf(tmp_path, tensors=[("w", (1, 2, 3, 4, 5), 12, 0)], tail=b"\0" * 64))
    with pytest.raises(InvalidDataError, match="alignment"):
        GgufReader(_gguf(tmp_path, kvs=[("general.alignment", 4, struct.pack("<I", 24))]))
    with pytest.raises(InvalidDataError, match="bool"):
        GgufReader(_gguf(tmp_path, kvs=[("flag", 7, b"\x02")]))
    with pytest.raises(NotImplementedError, match="metadata type"):
        GgufReader(_gguf(tmp_path, kvs=[("k", 13, b"\0" * 8)]))
    with pytest.raises(EOFError):
        GgufReader(_gguf(tmp_path, kvs=[("k", 8, struct.pack("<Q", 1000) + b"abc")]))
    with pytest.raises(EOFError):                      # the table cannot fit in the bytes that remain
        GgufReader(_gguf(tmp_path, tensors=[("w", (), 12, 0)]))
    with pytest.raises(InvalidDataError, match="too large"):
        GgufReader(_gguf(tmp_path, kvs=[("k", 9, struct.pack("<IQ", 4, 5) + b"\0" * 20)]),
                   GgufReadLimits(maximum_array_elements=4))
    with pytest.raises(InvalidDataError, match="table"):
        GgufReader(_gguf(tmp_path, tensors=[("a", (256,), 12, 0), ("b", (256,), 12, 0)]), GgufReadLimits(maximum_tensors=1))


def test_gguf_reader_alignment_metadata_and_payload(tmp_path):
    kvs = [("general.alignment", 4, struct.pack("<I", 64)), ("x.count", 10, struct.pack("<Q", 7)),
           ("x.names", 9, struct.pack("<IQ", 8, 2) + struct.pack("<Q", 1) + b"a" + struct.pack("<Q", 2) + b"bc"),
           ("x.f", 6, struct.pack("<f", 1.5)), ("x.ok", 7, b"\x01")]
    path = _gguf(tmp_path, version=2, kvs=kvs, tensors=[("w", (256, 3), 12, 64)], tail=b"\0" * 64 + bytes(range(256)) * 4)
    with GgufReader(path) as r:
        assert r.version == 2 and r.data_offset % 64 == 0
        assert r.metadata["x.count"] == 7 and r.metadata["x.names"] == ["a", "bc"] and r.metadata["x.ok"] is True
        t = r.get_tensor("w")
        assert t.byte_count() == 3 * 144 and r.matrix_dims(t) == (256, 3)
        with pytest.raises(InvalidDataError):
            nn.GgufTensorInfo("bad", (100, 3), 12, 0).byte_count()


def test_synthetic_payload_generators():
    from nntrain_amd import synth
    import oracle
    w = np.random.default_rng(0).standard_normal((4, 64)).astype(np.float32) * 0.02
    raw = synth.quantize_q8_0(w)
    assert raw.size == 4 * 2 * 34
    back = oracle.dequantize(8, raw).reshape(4, 64)
    d = raw.reshape(-1, 34)[:, :2].copy().view(np.float16).astype(np.float32).reshape(4, 2)
    # half a quantisation step, plus up to 127 steps of the fp16 rounding of the scale (2^-11 relative)
    assert np.all(np.abs(back - w).reshape(4, 2, 32) <= 0.57 * d[:, :, None] + 1e-9)
    for typ in (12, 13, 14, 21, 22):
        p = synth.k_quant_matrix(typ, 5, 512, 3)
        assert p.size == 5 * 2 * nn.BLOCK_BYTES[typ]
        assert np.all(np.isfinite(oracle.dequantize(typ, p)))
    assert np.array_equal(synth.to_bf16_bits(np.array([1.0, -2.0], np.float32)), np.array([0x3F80, 0xC000], np.uint16))


# ------------------------------------------------------------------------------------------------ tensor directory

def test_tensor_directory_checks_follow_the_reference(tmp_path):
    """Qwen35Gguf.ValidateDirectory (NNtrain.Core/Serialization/Qwen35Gguf.cs:110-193): the same cases, same kinds."""
    from nntrain_amd import GgufTensorDirectory, NotSupportedError
    tail = b"\0" * 4096
    path = _gguf(tmp_path, tensors=[("a.weight", (512, 7), 12, 0), ("n.weight", (512,), 0, 2048), ("h.weight", (16,), 1, 4000)],
                 tail=tail)
    with GgufReader(path) as r:
        d = GgufTensorDirectory(r)
        assert d.matrix("a.weight", 512, 7).type == 12
        assert d.dense("n.weight", 512).type == 0
        with pytest.raises(InvalidDataError, match="missing"):
            d.matrix("b.weight", 512, 7)
        with pytest.raises(InvalidDataError, match=r"shape \[512,7\] does not match expected \[7,512\]"):
            d.matrix("a.weight", 7, 512)                      # GGUF order is [input_width, output_width]
        with pytest.raises(NotSupportedError, match="F32/F16/BF16"):
            d.dense("a.weight", 512, 7)
        with pytest.raises(NotSupportedError, match="storage; got type 0"):
            nn.loader.check_matrix_storage(nn.GgufTensorInfo("f32.weight", (512, 1), 0, 0))
        with pytest.raises(NotSupportedError, match="Unexpected tensor 'h.weight'"):
            d.reject_unexpected()
        d.dense("h.weight", 16)
        d.reject_unexpected()
    with GgufReader(_gguf(tmp_path, tensors=[("w", (256, 1), 12, 0), ("w", (256, 1), 12, 256)], tail=tail)) as r:
        with pytest.raises(InvalidDataError, match="Duplicate GGUF tensor 'w'"):
            GgufTensorDirectory(r)
    with pytest.raises(InvalidDataError, match="divisible by 256"):
        nn.loader.check_matrix_storage(nn.GgufTensorInfo("short", (128, 3), 12, 0))
    with pytest.raises(InvalidDataError, match="divisible by 32"):
        nn.loader.check_matrix_storage(nn.GgufTensorInfo("short", (48, 3), 8, 0))
    with pytest.raises(NotSupportedError, match="payload limit"):
        nn.loader.check_matrix_storage(nn.GgufTensorInfo("huge", (256, 1 << 24), 12, 0))     # 144 * 2^24 > 2^31 - 1
    assert nn.loader.check_matrix_storage(nn.GgufTensorInfo("lm_head", (5376, 262144), 8, 0)) == 1_497_366_528
    with pytest.raises(NotSupportedError, match="payload limit"):
        nn.loader.check_dense_storage(nn.GgufTensorInfo("big", (1 << 30,), 0, 0))


def test_dense_widening_is_exact():
    from nntrain_amd.loader import widen_dense
    f16 = np.array([0x0001, 0x03ff, 0x0400, 0x3c00, 0xbc00, 0x7bff, 0x8000, 0x7c00], np.uint16)
    got = widen_dense(1, f16.tobytes())
    assert np.array_equal(got.view(np.uint32), f16.view(np.float16).astype(np.float32).view(np.uint32))
    assert got[0] == np.float32(2.0 ** -24) and np.isinf(got[-1])
    bf16 = np.array([0x3f80, 0xc000, 0x0001, 0x7f80], np.uint16)
    assert np.array_equal(widen_dense(30, bf16.tobytes()).view(np.uint32), bf16.astype(np.uint32) << 16)
    f32 = np.array([1.5, -0.0, 3e-45], np.float32)
    assert np.array_equal(widen_dense(0, f32.tobytes()).view(np.uint32), f32.view(np.uint32))


def test_gguf_ranged_reads(tmp_path):
    from gguf_writer import write_gguf
    payload = bytes(range(256)) * 9                       # 16 Q4_K blocks = 2304 bytes
    path = write_gguf(tmp_path / "r.gguf", [("pad", (32,), 8, b"\x11" * 34), ("w", (256, 16), 12, payload)])
    with GgufReader(path) as r:
        t = r.get_tensor("w")
        assert r.read_tensor_bytes(t) == payload
        assert r.read_tensor_range(t, 0, 10) == payload[:10]
        assert r.read_tensor_range(t, 1000, 1304) == payload[1000:]
        assert r.read_tensor_range(t, 2304, 0) == b""
        with pytest.raises(ValueError):
            r.read_tensor_range(t, 2300, 5)


def test_headers_compile_as_c_and_cpp(tmp_path):
    """The ABI headers are what a binding is written from: they must be plain C (and valid C++) on their own."""
    import shutil
    import subprocess
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    src = tmp_path / "use_headers.c"
    src.write_text('#include "nnhip.h"\n#include "nnhip_synth.h"\n'
                   'int main(void) { nnhip_error_info e; nnhip_fused_matvec_desc d; (void)e; (void)d; return (int)sizeof(nnhip_matvec_desc) == 0; }\n')
    for compiler, std in (("gcc", "-std=c99"), ("g++", "-std=c++17")):
        if shutil.which(compiler) is None:
            pytest.skip(f"{compiler} not installed")
        lang = ["-x", "c++"] if compiler == "g++" else []
        res = subprocess.run([compiler, std, "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", f"-I{root / 'include'}", *lang, str(src)],
                             capture_output=True, text=True)
        assert res.returncode == 0, res.stderr
