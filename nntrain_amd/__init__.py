"""MI355X-native GGUF block-quantized linear path (host layer over libnnhip.so).

The package mirrors, above the C ABI in include/nnhip.h, the three reference objects the path is reached through:
  GgufReader / GgufTensorInfo      NNtrain.Core/Serialization/GgufReader.cs
  HipExecutionLane / HipBuffer     NNtrain.Arc/ArcExecutionLane.cs (the subset the operator uses)
  GgufTensorDirectory/HipGgufLoader Qwen35Gguf.ValidateDirectory and Qwen35QuantizedModel.LoadTensor
  HipQuantizedMatrix               NNtrain.Core/Serialization/ArcQuantizedMatrix.cs and
                                   Qwen35QuantizedModel.Matrix (NNtrain.Core/Modules/Qwen35QuantizedModel.cs:1069-1369)
Nothing here computes on the CPU: every operator call goes to the HIP library and raises if it is missing.
"""
from .native import NnHipError, abi_version, library_path, load_library  # noqa: F401
from .lane import HipBuffer, HipExecutionLane  # noqa: F401
from .quantized_matrix import (BLOCK_BYTES, BLOCK_ELEMS, GGML_BF16, GGML_IQ2_S, GGML_IQ3_S, GGML_Q4_K,  # noqa: F401
                               GGML_Q5_K, GGML_Q6_K, GGML_Q8_0, HipQuantizedMatrix)
from .gguf import GgufReader, GgufReadLimits, GgufTensorInfo, InvalidDataError  # noqa: F401
from .loader import GgufTensorDirectory, HipGgufLoader, NotSupportedError  # noqa: F401
from . import qwen35_gpu  # noqa: F401
from .decoder import DecoderDescriptor, GenerationTiming, QuantizedDecoder  # noqa: F401
