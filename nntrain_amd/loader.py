"""GGUF file -> device-resident tensors: directory checks, then a streaming upload of the raw blocks.

The directory checks are those of Qwen35Gguf.ValidateDirectory (NNtrain.Core/Serialization/Qwen35Gguf.cs:110-193):
duplicate names, required tensors and exact shapes (GGUF shape of a matrix is [input_width, output_width]), the
storage types a matrix or a dense tensor may have, whole blocks per row, the 2^31-1 byte payload limit, and "no
tensor that nobody asked for".  The upload is that of Qwen35QuantizedModel.LoadTensor
(NNtrain.Core/Modules/Qwen35QuantizedModel.cs:234-282): quantized matrices go to the device as the file's bytes,
unchanged, through positional reads, and no model-sized host copy is kept; dense tensors are widened to FP32 as
Qwen2Gguf.ReadTensor does (NNtrain.Core/Serialization/Qwen2Gguf.cs:308-357).

Which tensors a model needs is the model's business (the reference derives the list from its metadata); this module
offers the checks as calls (`matrix`, `dense`, `reject_unexpected`) and a loader that works on any GGUF file.
"""
from __future__ import annotations

import numpy as np

from .gguf import TYPE_BLOCKS, GgufReader, GgufTensorInfo, InvalidDataError
from .lane import HipBuffer, HipExecutionLane
from .quantized_matrix import BLOCK_BYTES, BLOCK_ELEMS, HipQuantizedMatrix

F32_TYPE, F16_TYPE, BF16_TYPE = 0, 1, 30
DENSE_STORAGE_TYPES = (F32_TYPE, F16_TYPE, BF16_TYPE)
MANAGED_PAYLOAD_LIMIT = 2**31 - 1           # int.MaxValue: the reference holds a payload in one managed array


class NotSupportedError(NotImplementedError):
    """The reference's NotSupportedException."""


def is_quantized_matrix(tensor: GgufTensorInfo) -> bool:
    """A 2-D tensor stored in one of the formats the mat-vec kernels read (block formats and bfloat16; a 2-D F16 or
    F32 tensor is a dense tensor, as in Qwen35Gguf.IsSupportedMatrixStorage)."""
    return len(tensor.shape) == 2 and tensor.type in BLOCK_ELEMS


class GgufTensorDirectory:
    """Name-indexed tensor table with the reference's per-tensor checks."""

    def __init__(self, reader: GgufReader):
        self.reader = reader
        self._tensors: dict[str, GgufTensorInfo] = {}
        for tensor in reader.tensors:
            if tensor.name in self._tensors:
                raise InvalidDataError(f"Duplicate GGUF tensor '{tensor.name}'.")
            self._tensors[tensor.name] = tensor
        self._expected: set[str] = set()

    def __contains__(self, name: str) -> bool:
        return name in self._tensors

    def __iter__(self):
        return iter(self._tensors.values())

    def shape(self, name: str, shape) -> GgufTensorInfo:
        self._expected.add(name)
        tensor = self._tensors.get(name)
        if tensor is None:
            raise InvalidDataError(f"Required GGUF tensor '{name}' is missing.")
        if tuple(int(d) for d in tensor.shape) != tuple(int(d) for d in shape):
            raise InvalidDataError(f"GGUF tensor '{name}' shape [{','.join(str(d) for d in tensor.shape)}] does not "
                                   f"match expected [{','.join(str(d) for d in shape)}].")
        return tensor

    def matrix(self, name: str, input_width: int, output_width: int) -> GgufTensorInfo:
        tensor = self.shape(name, (input_width, output_width))
        check_matrix_storage(tensor)
        return tensor

    def dense(self, name: str, *shape: int) -> GgufTensorInfo:
        tensor = self.shape(name, shape)
        check_dense_storage(tensor)
        return tensor

    def reject_unexpected(self) -> None:
        """Every tensor in the file must have been asked for through shape/matrix/dense."""
        for name in self._tensors:
            if name not in self._expected:
                raise NotSupportedError(f"Unexpected tensor '{name}'; only the declared tensor directory is supported.")


def check_matrix_storage(tensor: GgufTensorInfo) -> int:
    """Storage checks of a quantized matrix; returns its payload size in bytes."""
    if len(tensor.shape) != 2:
        raise InvalidDataError(f"GGUF tensor '{tensor.name}' is not a matrix.")
    if tensor.type not in BLOCK_ELEMS:
        raise NotSupportedError(f"Matrix '{tensor.name}' requires Q8_0/Q4_K/Q5_K/Q6_K/IQ3_S/IQ2_S/BF16 storage; got type "
                                f"{tensor.type}.")
    input_width, output_width = int(tensor.shape[0]), int(tensor.shape[1])
    elems = BLOCK_ELEMS[tensor.type]
    if input_width % elems != 0:
        raise InvalidDataError(f"Matrix '{tensor.name}' requires a row width divisible by {elems}.")
    nbytes = output_width * (input_width // elems) * BLOCK_BYTES[tensor.type]
    if nbytes > MANAGED_PAYLOAD_LIMIT:
        raise NotSupportedError(f"Matrix '{tensor.name}' exceeds the managed payload limit.")
    return nbytes


def check_dense_storage(tensor: GgufTensorInfo) -> int:
    """Storage checks of a dense tensor; returns its element count."""
    if tensor.type not in DENSE_STORAGE_TYPES:
        raise NotSupportedError(f"Tensor '{tensor.name}' requires F32/F16/BF16 storage; got type {tensor.type}.")
    elements = tensor.element_count
    if elements > MANAGED_PAYLOAD_LIMIT // (4 if tensor.type == F32_TYPE else 2):
        raise NotSupportedError(f"Tensor '{tensor.name}' exceeds the managed payload limit.")
    return elements


def widen_dense(tensor_type: int, payload: bytes) -> np.ndarray:
    """F32 / F16 / BF16 little-endian payload -> float32, exactly (every F16 and BF16 value is an FP32 value)."""
    if tensor_type == F32_TYPE:
        return np.frombuffer(payload, dtype="<f4").astype(np.float32, copy=True)
    if tensor_type == F16_TYPE:
        return np.frombuffer(payload, dtype="<f2").astype(np.float32)
    if tensor_type == BF16_TYPE:
        return (np.frombuffer(payload, dtype="<u2").astype(np.uint32) << 16).view(np.float32)
    raise NotSupportedError(f"GGML tensor type {tensor_type} is not a dense storage type.")


class HipGgufLoader:
    """Uploads tensors of one GGUF file to one lane.

    A quantized matrix goes from the file to the device inside the library (`staged`, the default: positional reads
    into two pinned buffers, one travelling while the other is filled), or is read here and uploaded in pieces of
    `chunk_bytes`; either way the host never holds more than a piece of it, and the reads are positional, so several
    loaders (one per lane, one thread each) may share a reader.
    """

    def __init__(self, lane: HipExecutionLane, reader: GgufReader, chunk_bytes: int = 64 << 20, staged: bool = True):
        if chunk_bytes <= 0:
            raise ValueError("chunk_bytes must be positive")
        self.lane = lane
        self.reader = reader
        self.chunk_bytes = chunk_bytes
        self.staged = staged
        self.quantized_bytes = 0
        self.dense_bytes = 0

    def _info(self, tensor) -> GgufTensorInfo:
        return tensor if isinstance(tensor, GgufTensorInfo) else self.reader.get_tensor(tensor)

    def load_matrix(self, tensor) -> HipQuantizedMatrix:
        info = self._info(tensor)
        nbytes = check_matrix_storage(info)
        if TYPE_BLOCKS[info.type] != (BLOCK_ELEMS[info.type], BLOCK_BYTES[info.type]) or info.byte_count() != nbytes:
            raise InvalidDataError(f"Matrix '{info.name}' has an inconsistent block geometry.")
        buffer = self.lane.allocate_bytes(nbytes)
        try:
            if self.staged:
                fd, file_offset = self.reader.tensor_file_range(info, 0, nbytes)
                self.lane.write_from_file(buffer, fd, file_offset, nbytes)
            else:
                done = 0
                while done < nbytes:
                    piece = self.reader.read_tensor_range(info, done, min(self.chunk_bytes, nbytes - done))
                    self.lane.write(buffer, np.frombuffer(piece, dtype=np.uint8), offset=done)
                    done += len(piece)
        except BaseException:
            buffer.dispose()
            raise
        self.quantized_bytes += nbytes
        return HipQuantizedMatrix.from_device(self.lane, buffer, info.type, int(info.shape[1]), int(info.shape[0]))

    def load_dense(self, tensor) -> HipBuffer:
        info = self._info(tensor)
        elements = check_dense_storage(info)
        values = widen_dense(info.type, self.reader.read_tensor_bytes(info, elements * (4 if info.type == F32_TYPE else 2)))
        self.dense_bytes += 4 * elements
        return self.lane.upload_raw(values)

    def load_all(self, progress=None):
        """Every quantized matrix (in file order of their payloads) and every dense tensor of the file.
        Returns (matrices by name, dense FP32 buffers by name); tensors of other kinds raise NotSupportedError."""
        directory = GgufTensorDirectory(self.reader)
        matrices: dict[str, HipQuantizedMatrix] = {}
        dense: dict[str, HipBuffer] = {}
        loaded = 0
        total = len(self.reader.tensors)
        try:
            for info in sorted(directory, key=lambda t: t.offset):
                if is_quantized_matrix(info):
                    matrices[info.name] = self.load_matrix(info)
                else:
                    dense[info.name] = self.load_dense(info)
                loaded += 1
                if progress is not None and loaded % 100 == 0:
                    progress(f"Loading tensors: {loaded}/{total}")
        except BaseException:
            for m in matrices.values():
                m.dispose()
            for b in dense.values():
                b.dispose()
            raise
        return matrices, dense
