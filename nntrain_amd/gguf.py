"""GGUF v2/v3 container reader: header, key/value metadata, tensor directory, positional payload reads.

Follows NNtrain.Core/Serialization/GgufReader.cs (structure :28-92, limits GgufReadLimits.cs:6-13, payload read
:107-123) so the same files open, the same files are rejected, and tensor payloads come back as the raw bytes that
are uploaded unchanged.  Matrix shape rules follow Qwen35Gguf.cs:170-182 (GGUF shape is [input_width, output_width]).
"""
from __future__ import annotations

import os
import struct
from dataclasses import dataclass, field

MAGIC = 0x46554747  # "GGUF" little-endian

# GgufValueType
UINT8, INT8, UINT16, INT16, UINT32, INT32, FLOAT32, BOOL, STRING, ARRAY, UINT64, INT64, FLOAT64 = range(13)
_SCALAR = {UINT8: "B", INT8: "b", UINT16: "H", INT16: "h", UINT32: "I", INT32: "i", FLOAT32: "f", UINT64: "Q",
           INT64: "q", FLOAT64: "d"}
_MIN_SIZE = {UINT8: 1, INT8: 1, BOOL: 1, UINT16: 2, INT16: 2, UINT32: 4, INT32: 4, FLOAT32: 4, UINT64: 8, INT64: 8,
             FLOAT64: 8, STRING: 8, ARRAY: 12}

# ggml type id -> (elements per block, bytes per block) for the tensor types this path reads
TYPE_BLOCKS = {0: (1, 4), 1: (1, 2), 30: (1, 2), 8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210),
               21: (256, 110), 22: (256, 82)}


class InvalidDataError(ValueError):
    """The reference's InvalidDataException."""


@dataclass
class GgufReadLimits:
    maximum_array_elements: int = 4 * 1024 * 1024
    maximum_string_bytes: int = 16 * 1024 * 1024
    maximum_metadata_entries: int = 100_000
    maximum_tensors: int = 1_000_000
    maximum_nesting_depth: int = 32
    maximum_decoded_bytes: int = 512 * 1024 * 1024

    def validate(self) -> None:
        for name, value in vars(self).items():
            if value <= 0:
                raise ValueError(f"{name} must be positive")


@dataclass(frozen=True)
class GgufTensorInfo:
    name: str
    shape: tuple
    type: int
    offset: int

    @property
    def element_count(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n

    def byte_count(self) -> int:
        """Payload bytes; rows (shape[0]) must hold whole blocks (Qwen2Gguf.cs:199-208)."""
        if self.type not in TYPE_BLOCKS:
            raise NotImplementedError(f"GGML tensor type {self.type} is unsupported.")
        elems, nbytes = TYPE_BLOCKS[self.type]
        if self.shape[0] % elems != 0:
            raise InvalidDataError(f"Tensor '{self.name}' has incomplete {elems}-value blocks.")
        return self.element_count // elems * nbytes


@dataclass
class _Cursor:
    fd: int
    size: int
    pos: int = 0
    buf: bytes = b""
    buf_pos: int = 0
    decoded: int = 0
    limits: GgufReadLimits = field(default_factory=GgufReadLimits)

    def remaining(self) -> int:
        return self.size - self.pos

    def ensure(self, n: int) -> None:
        if n > self.remaining():
            raise EOFError("GGUF header value exceeds remaining file bytes.")

    def reserve(self, n: int) -> None:
        if n > self.limits.maximum_decoded_bytes - self.decoded:
            raise InvalidDataError("GGUF decoded metadata budget exceeded.")
        self.decoded += n

    def read(self, n: int) -> bytes:
        self.ensure(n)
        lo = self.pos - self.buf_pos
        if lo < 0 or lo + n > len(self.buf):
            self.buf = os.pread(self.fd, max(n, 1 << 20), self.pos)
            self.buf_pos = self.pos
            lo = 0
            if len(self.buf) < n:
                raise EOFError("unexpected end of GGUF file")
        self.pos += n
        return self.buf[lo:lo + n]

    def unpack(self, fmt: str):
        return struct.unpack("<" + fmt, self.read(struct.calcsize("<" + fmt)))[0]

    def string(self) -> str:
        n = self.unpack("Q")
        if n > self.limits.maximum_string_bytes:
            raise InvalidDataError("GGUF string is too large.")
        self.ensure(n)
        self.reserve(32 + n * 3)
        return self.read(n).decode("utf-8")


class GgufReader:
    def __init__(self, path: str, limits: GgufReadLimits | None = None):
        if not path or not str(path).strip():
            raise ValueError("path is empty")
        limits = limits or GgufReadLimits()
        limits.validate()
        self.file_path = os.path.abspath(path)
        self._fd = os.open(self.file_path, os.O_RDONLY)
        try:
            size = os.fstat(self._fd).st_size
            c = _Cursor(self._fd, size, limits=limits)
            if size < 4 or c.unpack("I") != MAGIC:
                raise InvalidDataError("Not a GGUF file.")
            self.version = c.unpack("I")
            if not 2 <= self.version <= 3:
                raise NotImplementedError(f"GGUF version {self.version} is not supported.")
            tensor_count = c.unpack("Q")
            metadata_count = c.unpack("Q")
            if tensor_count > limits.maximum_tensors or metadata_count > limits.maximum_metadata_entries:
                raise InvalidDataError("GGUF table is too large.")
            c.ensure(metadata_count * 13 + tensor_count * 32)
            c.reserve(metadata_count * 128 + tensor_count * 160)
            self.metadata: dict = {}
            for _ in range(metadata_count):
                key = c.string()
                vtype = c.unpack("I")
                if key in self.metadata:
                    raise InvalidDataError(f"duplicate GGUF metadata key '{key}'")
                self.metadata[key] = self._value(c, vtype, 0, False)
            self.tensors: list[GgufTensorInfo] = []
            for _ in range(tensor_count):
                name = c.string()
                dims = c.unpack("I")
                if dims == 0 or dims > 4:
                    raise InvalidDataError(f"Tensor '{name}' has unsupported rank {dims}.")
                shape = tuple(c.unpack("Q") for _ in range(dims))
                ttype = c.unpack("I")
                offset = c.unpack("Q")
                self.tensors.append(GgufTensorInfo(name, shape, ttype, offset))
            alignment = 32
            if "general.alignment" in self.metadata:
                alignment = int(self.metadata["general.alignment"])
            if alignment <= 0 or alignment & (alignment - 1):
                raise InvalidDataError(f"Invalid GGUF alignment {alignment}.")
            self._data_offset = (c.pos + alignment - 1) // alignment * alignment
            self._size = size
        except BaseException:
            self.dispose()
            raise

    def _value(self, c: _Cursor, vtype: int, depth: int, reserved: bool):
        if vtype not in _MIN_SIZE:
            raise NotImplementedError(f"GGUF metadata type {vtype} is unsupported.")
        c.ensure(_MIN_SIZE[vtype])
        if not reserved:
            c.reserve(32)
        if vtype in _SCALAR:
            return c.unpack(_SCALAR[vtype])
        if vtype == BOOL:
            b = c.unpack("B")
            if b > 1:
                raise InvalidDataError("Invalid GGUF bool.")
            return bool(b)
        if vtype == STRING:
            return c.string()
        # ARRAY
        depth += 1
        if depth > c.limits.maximum_nesting_depth:
            raise InvalidDataError("GGUF metadata nesting limit exceeded.")
        etype = c.unpack("I")
        count = c.unpack("Q")
        if etype not in _MIN_SIZE:
            raise NotImplementedError(f"GGUF metadata type {etype} is unsupported.")
        if count > c.limits.maximum_array_elements:
            raise InvalidDataError("GGUF metadata array is too large.")
        c.ensure(count * _MIN_SIZE[etype])
        c.reserve(32 + count * 40)
        return [self._value(c, etype, depth, True) for _ in range(count)]

    # ---- tensor access ----
    @property
    def data_offset(self) -> int:
        return self._data_offset

    def get_tensor(self, name: str) -> GgufTensorInfo:
        for t in self.tensors:
            if t.name == name:
                return t
        raise KeyError(f"GGUF tensor '{name}' was not found.")

    def read_tensor_bytes(self, tensor: GgufTensorInfo, byte_count: int | None = None) -> bytes:
        """Exact byte range, positional (os.pread), safe to call from several threads at once."""
        if byte_count is None:
            byte_count = tensor.byte_count()
        if byte_count < 0:
            raise ValueError("byteCount is negative")
        offset = self._data_offset + tensor.offset
        if offset > self._size or byte_count > self._size - offset:
            raise EOFError("tensor payload exceeds the file")
        chunks = []
        done = 0
        while done < byte_count:
            piece = os.pread(self._fd, min(byte_count - done, 1 << 28), offset + done)
            if not piece:
                raise EOFError("tensor payload exceeds the file")
            chunks.append(piece)
            done += len(piece)
        return chunks[0] if len(chunks) == 1 else b"".join(chunks)

    def read_tensor_range(self, tensor: GgufTensorInfo, start: int, byte_count: int) -> bytes:
        """Bytes [start, start + byte_count) of a tensor's payload (positional, for streaming uploads)."""
        total = tensor.byte_count()
        if start < 0 or byte_count < 0 or start + byte_count > total:
            raise ValueError("range is outside the tensor payload")
        offset = self._data_offset + tensor.offset + start
        if offset > self._size or byte_count > self._size - offset:
            raise EOFError("tensor payload exceeds the file")
        chunks = []
        done = 0
        while done < byte_count:
            piece = os.pread(self._fd, min(byte_count - done, 1 << 28), offset + done)
            if not piece:
                raise EOFError("tensor payload exceeds the file")
            chunks.append(piece)
            done += len(piece)
        return chunks[0] if len(chunks) == 1 else b"".join(chunks)

    def tensor_file_range(self, tensor: GgufTensorInfo, start: int, byte_count: int) -> tuple[int, int]:
        """(file descriptor, absolute file offset) of bytes [start, start + byte_count) of a tensor's payload, after the
        same checks as read_tensor_range: for uploads that read the file themselves (positional reads: the descriptor's
        own position is neither used nor moved)."""
        total = tensor.byte_count()
        if start < 0 or byte_count < 0 or start + byte_count > total:
            raise ValueError("range is outside the tensor payload")
        offset = self._data_offset + tensor.offset + start
        if offset > self._size or byte_count > self._size - offset:
            raise EOFError("tensor payload exceeds the file")
        return self._fd, offset

    def matrix_dims(self, tensor: GgufTensorInfo) -> tuple[int, int]:
        """(input_width, output_width) of a 2-D weight: GGUF stores ne0 = K first (Qwen35Gguf.cs:170-182)."""
        if len(tensor.shape) != 2:
            raise InvalidDataError(f"Tensor '{tensor.name}' is not a matrix.")
        return int(tensor.shape[0]), int(tensor.shape[1])

    def dispose(self) -> None:
        if getattr(self, "_fd", None) is not None:
            os.close(self._fd)
            self._fd = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.dispose()
