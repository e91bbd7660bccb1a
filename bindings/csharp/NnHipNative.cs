// Source-generated P/Invoke (LibraryImport) declarations for libnnhip.so - one per entry point of include/nnhip.h.
// Drop into an NNtrain project that may reference NNtrain.Runtime (same layer as NNtrain.Arc / NNtrain.Cuda).
// Not compiled in this repository (no .NET toolchain in the build image); the C header is the source of truth and
// tests/test_host_layer.py checks that every symbol declared there is exported and that every declaration below
// matches it in name, arity and argument widths (and the structure sizes).
using System.Runtime.InteropServices;

namespace NNtrain.Hip;

internal static unsafe partial class NnHipNative
{
    private const string Library = "nnhip";   // resolves to libnnhip.so / nnhip.dll

    internal const uint SupportedAbiMajor = 1;
    internal const uint TypeQ8_0 = 8, TypeQ4K = 12, TypeQ5K = 13, TypeQ6K = 14, TypeIQ3S = 21, TypeIQ2S = 22, TypeBF16 = 30;

    [StructLayout(LayoutKind.Sequential)]
    internal struct ErrorInfo
    {
        internal uint StructSize; internal uint AbiVersion; internal ulong Sequence;
        internal int Status; internal int DeviceIndex; internal uint Operation; internal uint Reserved;
    }

    [StructLayout(LayoutKind.Sequential)]
    internal struct LaneCounters
    {
        internal uint StructSize; internal uint DriverAllocations; internal ulong H2DBytes; internal ulong D2HBytes;
        internal ulong AllocatedBytes; internal ulong PeakAllocatedBytes; internal ulong KernelLaunches;
    }

    [StructLayout(LayoutKind.Sequential)]
    internal struct MatvecDesc
    {
        internal nint X; internal nint W; internal nint Bias; internal nint Y;
        internal uint GgmlType; internal int Rows; internal int InW; internal int OutW;
    }

    [StructLayout(LayoutKind.Sequential)]
    internal struct MatvecPlanInfo
    {
        internal uint StructSize; internal int Kernel; internal int Threads; internal int RowsPerStep; internal int Steps;
        internal int Groups; internal int RowTile; internal int RingDepth; internal int ResultBufferFloats;
        internal int DynamicLdsBytes;
    }

    [StructLayout(LayoutKind.Sequential)]
    internal struct BatchLaunchInfo
    {
        internal uint StructSize; internal uint GgmlType; internal int Kernel; internal int InW; internal int Entries;
        internal int Units; internal int Groups; internal int Threads; internal int RowsPerPass; internal int ConsecutiveRuns;
        internal int StageBuffers; internal int ActivationsInLds; internal int DynamicLdsBytes;
    }

    internal const uint PreNone = 0, PreRmsNorm = 1, PreSiluMultiply = 2;
    internal const uint PostNone = 0, PostSiluPair = 1;

    [StructLayout(LayoutKind.Sequential)]
    internal struct FusedMatvecDesc
    {
        internal uint StructSize; internal uint GgmlType; internal uint PreOp; internal float Epsilon;
        internal nint X; internal nint X2; internal nint NormWeight; internal nint XOut; internal nint SumOut;
        internal nint W; internal nint Bias; internal nint Addend; internal nint Y;
        internal int InW; internal int OutW;
        internal nint LoraZ; internal nint LoraB; internal int LoraRank; internal float LoraScale;
        internal int XHeadWidth; internal int XHeadGroup; internal uint PostOp; internal uint Reserved;
    }

    [LibraryImport(Library)] internal static partial uint nnhip_abi_version();
    [LibraryImport(Library)] internal static partial int nnhip_last_error(out ErrorInfo info, nuint size);
    [LibraryImport(Library)] internal static partial int nnhip_last_error_message(byte* buffer, int capacity);
    [LibraryImport(Library)] internal static partial int nnhip_device_count(out int count);
    [LibraryImport(Library)] internal static partial int nnhip_device_name(int device, byte* buffer, int capacity);
    [LibraryImport(Library)] internal static partial int nnhip_device_info(int device, out int computeUnits, out ulong totalMemoryBytes);
    [LibraryImport(Library)] internal static partial int nnhip_type_block(uint ggmlType, out int blockElems, out int blockBytes);
    [LibraryImport(Library)] internal static partial int nnhip_matrix_bytes(uint ggmlType, int inW, int outW, out ulong bytes);
    [LibraryImport(Library)] internal static partial int nnhip_lane_create(int device, out nint lane);
    [LibraryImport(Library)] internal static partial int nnhip_lane_destroy(nint lane);
    [LibraryImport(Library)] internal static partial int nnhip_alloc(nint lane, nuint bytes, out nint dptr);
    [LibraryImport(Library)] internal static partial int nnhip_free(nint lane, nint dptr);
    [LibraryImport(Library)] internal static partial int nnhip_lane_trim(nint lane);
    [LibraryImport(Library)] internal static partial int nnhip_upload(nint lane, nint dptr, nuint offset, void* host, nuint bytes);
    [LibraryImport(Library)] internal static partial int nnhip_upload_from_file(nint lane, nint dptr, nuint offset, int fd, ulong fileOffset, nuint bytes);
    [LibraryImport(Library)] internal static partial int nnhip_download(nint lane, nint dptr, nuint offset, void* host, nuint bytes);
    [LibraryImport(Library)] internal static partial int nnhip_copy(nint lane, nint dst, nuint dstOffset, nint src, nuint srcOffset, nuint bytes);
    [LibraryImport(Library)] internal static partial int nnhip_fill_u32(nint lane, nint dptr, nuint offset, uint value, nuint count);
    [LibraryImport(Library)] internal static partial int nnhip_synchronize(nint lane);
    [LibraryImport(Library)] internal static partial int nnhip_lane_get_counters(nint lane, out LaneCounters counters, nuint size);
    [LibraryImport(Library)] internal static partial int nnhip_lane_stream(nint lane, out nint stream);
    internal const uint OptionRowStepOnly = 1;
    [LibraryImport(Library)] internal static partial int nnhip_lane_set_option(nint lane, uint option, long value);
    [LibraryImport(Library)] internal static partial int nnhip_lane_get_option(nint lane, uint option, out long value);
    [LibraryImport(Library)] internal static partial int nnhip_dequantize(nint lane, uint ggmlType, nint w, nint output, long elements);
    [LibraryImport(Library)] internal static partial int nnhip_quant_matvec(nint lane, uint ggmlType, nint x, nint w, nint bias, nint y, int rows, int inW, int outW);
    [LibraryImport(Library)] internal static partial int nnhip_matvec_plan(uint ggmlType, int rows, int inW, int outW, int computeUnits, MatvecPlanInfo* info);
    [LibraryImport(Library)] internal static partial int nnhip_matvec_batch_plan(MatvecDesc* descs, int count, int computeUnits, BatchLaunchInfo* launches, int capacity, out int launchCount);
    [LibraryImport(Library)] internal static partial int nnhip_quant_matvec_batch(nint lane, MatvecDesc* descs, int count);
    [LibraryImport(Library)] internal static partial int nnhip_quant_matvec_batch_static(nint lane, MatvecDesc* descs, int count);
    [LibraryImport(Library)] internal static partial int nnhip_quant_matvec_fused(nint lane, FusedMatvecDesc* desc);
    [LibraryImport(Library)] internal static partial int nnhip_quant_matmul(nint lane, uint ggmlType, nint x, nint w, nint bias, nint y, int rows, int inW, int outW);
    [LibraryImport(Library)] internal static partial int nnhip_quant_matmul_split(nint lane, uint ggmlType, nint x, nint w, nint bias, nint y, int rows, int inW, int outW);
    [LibraryImport(Library)] internal static partial int nnhip_quant_matmul_bf16(nint lane, uint ggmlType, nint xBf16, nint w, nint bias, nint y, int rows, int inW, int outW);
    [LibraryImport(Library)] internal static partial int nnhip_rms_norm(nint lane, nint input, nint weight, nint output, int rows, int width, int inputStride, float epsilon);
    [LibraryImport(Library)] internal static partial int nnhip_add_rms_norm(nint lane, nint destination, nint residual, nint weight, nint output, int rows, int width, int inputStride, float epsilon);
    [LibraryImport(Library)] internal static partial int nnhip_silu_multiply(nint lane, nint gate, nint up, nint output, int length);
    [LibraryImport(Library)] internal static partial int nnhip_add_in_place(nint lane, nint destination, nint source, int length);
    [LibraryImport(Library)] internal static partial int nnhip_first_token_attention(nint lane, nint v, nint output, int heads, int kvHeads, int headWidth);
    [LibraryImport(Library)] internal static partial int nnhip_lora_a(nint lane, nint x, nint a, nint z, int rows, int width, int rank);
    [LibraryImport(Library)] internal static partial int nnhip_lora_b(nint lane, nint z, nint b, nint y, int rows, int output, int rank, float scale);
    [LibraryImport(Library)] internal static partial int nnhip_event_create(nint lane, out nint evt);
    [LibraryImport(Library)] internal static partial int nnhip_event_destroy(nint lane, nint evt);
    [LibraryImport(Library)] internal static partial int nnhip_event_record(nint lane, nint evt);
    [LibraryImport(Library)] internal static partial int nnhip_event_elapsed_ms(nint lane, nint start, nint stop, out float milliseconds);
    [LibraryImport(Library)] internal static partial int nnhip_graph_begin(nint lane);
    [LibraryImport(Library)] internal static partial int nnhip_graph_end(nint lane, out nint graph);
    [LibraryImport(Library)] internal static partial int nnhip_graph_launch(nint lane, nint graph);
    [LibraryImport(Library)] internal static partial int nnhip_graph_destroy(nint lane, nint graph);

    /// <summary>Non-zero status -> exception carrying the native message, as OpenClNative.Check does.</summary>
    internal static void Check(int status, string operation)
    {
        if (status == 0) return;
        byte* text = stackalloc byte[256];
        nnhip_last_error_message(text, 256);
        string message = Marshal.PtrToStringUTF8((nint)text) ?? string.Empty;
        throw status switch
        {
            2 => new NotSupportedException($"HIP {operation}: {message}"),
            1 or 3 => new ArgumentException($"HIP {operation}: {message}"),
            4 => new OutOfMemoryException($"HIP {operation}: {message}"),
            _ => new InvalidOperationException($"HIP {operation} failed ({status}): {message}"),
        };
    }

    /// <summary>Checked once, lazily: the native major version must match (CudaNativeGateway.cs:1320-1358).</summary>
    internal static void EnsureAbi()
    {
        uint packed = nnhip_abi_version();
        if (packed >> 16 != SupportedAbiMajor)
            throw new InvalidOperationException($"nnhip reports ABI {packed >> 16}.{packed & 0xffff}; expected major {SupportedAbiMajor}.");
    }
}
