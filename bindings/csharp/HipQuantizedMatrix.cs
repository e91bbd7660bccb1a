// Immutable GGUF block-quantized matrix resident in HBM.  Same constructor checks, exceptions and Forward contract as
// ArcQuantizedMatrix (NNtrain.Core/Serialization/ArcQuantizedMatrix.cs:16-60) and Qwen35QuantizedModel.Matrix.Forward
// (NNtrain.Core/Modules/Qwen35QuantizedModel.cs:1210-1369), extended to GGML types 8, 12, 13, 14, 21, 22 and 30 (bfloat16).
namespace NNtrain.Hip;

public sealed class HipQuantizedMatrix : IDisposable
{
    private byte[]? _payload;
    private HipExecutionLane? _lane;
    private HipBuffer? _devicePayload;

    public HipQuantizedMatrix(byte[] payload, uint ggmlType, int outputWidth, int inputWidth)
    {
        ArgumentNullException.ThrowIfNull(payload);
        if (NnHipNative.nnhip_type_block(ggmlType, out int elems, out int blockBytes) != 0)
            throw new NotSupportedException($"GGML type {ggmlType} is not a supported quantized matrix type.");
        if (outputWidth <= 0 || inputWidth <= 0)
            throw new ArgumentOutOfRangeException(nameof(outputWidth));
        if (inputWidth % elems != 0)
            throw new NotSupportedException($"Quantized rows must contain complete {elems}-value blocks.");
        long expected = checked((long)outputWidth * (inputWidth / elems) * blockBytes);
        if (payload.Length != expected)
            throw new InvalidDataException($"Quantized matrix payload has {payload.Length} bytes; expected {expected}.");
        _payload = payload;
        GgmlType = ggmlType;
        OutputWidth = outputWidth;
        InputWidth = inputWidth;
        StorageBytes = payload.Length;
    }

    public uint GgmlType { get; }
    public int OutputWidth { get; }
    public int InputWidth { get; }
    public long StorageBytes { get; }

    /// <summary>Rows at or above which Forward uses the matrix-core mat-mul (Qwen35QuantizedModel.cs:1249).</summary>
    public const int PrefillMinRows = 16;

    /// <summary>Opt-in, like Qwen35ExecutionOptions.InferenceXmxPrefill (Qwen35ExecutionOptions.cs:50): rows >= 16 go to
    /// the bfloat16 matrix-core mat-mul (2e-3 of the exact product) instead of the FP32-grade mat-vec (1e-5).</summary>
    public bool InferenceMatmulPrefill { get; init; }

    /// <summary>With InferenceMatmulPrefill: both operands as two bfloat16 parts and three products (about 3e-6 of the
    /// exact product, inside the 5e-5 the reference tests its XMX prefill at, Qwen35XmxPrefillLinearTests.cs:87-89) at
    /// three times the cost.</summary>
    public bool InferenceMatmulPrefillSplit { get; init; }

    /// <summary>Whether Forward sends this many input rows to the matrix-core mat-mul.</summary>
    public bool UsesPrefill(int rows) => InferenceMatmulPrefill && rows >= PrefillMinRows && InputWidth % 256 == 0;

    /// <summary>y[rows, out] = bias + x[rows, in] . W^T, FP32 activations; the caller disposes the result.
    /// Every row count goes to the dequantization-fused mat-vec unless InferenceMatmulPrefill is set, in which case rows
    /// >= 16 go to the bf16 matrix-core mat-mul (activations rounded to bfloat16 on the device), the counterpart of the
    /// reference's opt-in XMX prefill (Qwen35QuantizedModel.cs:1249-1317).  Allocating the
    /// output per call is cheap: the lane hands out the block a previous Dispose returned.</summary>
    public HipBuffer Forward(HipExecutionLane lane, HipBuffer input, HipBuffer? bias, int rows = 1)
    {
        ArgumentNullException.ThrowIfNull(lane);
        ArgumentNullException.ThrowIfNull(input);
        if (rows < 1) throw new ArgumentOutOfRangeException(nameof(rows));
        if (input.Bytes < (long)rows * InputWidth * sizeof(float))
            throw new ArgumentException("Quantized linear input width mismatch.", nameof(input));
        if (bias is not null && bias.Bytes < (long)OutputWidth * sizeof(float))
            throw new ArgumentException("Quantized linear bias width mismatch.", nameof(bias));
        HipBuffer encoded = DevicePayload(lane);
        HipBuffer output = lane.Allocate(checked(rows * OutputWidth));
        bool prefill = UsesPrefill(rows);
        int status = lane.Locked(h => prefill
            ? (InferenceMatmulPrefillSplit
                ? NnHipNative.nnhip_quant_matmul_split(h, GgmlType, input.Pointer, encoded.Pointer, bias?.Pointer ?? 0, output.Pointer,
                    rows, InputWidth, OutputWidth)
                : NnHipNative.nnhip_quant_matmul(h, GgmlType, input.Pointer, encoded.Pointer, bias?.Pointer ?? 0, output.Pointer,
                    rows, InputWidth, OutputWidth))
            : NnHipNative.nnhip_quant_matvec(h, GgmlType, input.Pointer, encoded.Pointer, bias?.Pointer ?? 0, output.Pointer,
                rows, InputWidth, OutputWidth));
        if (status != 0) { output.Dispose(); NnHipNative.Check(status, prefill ? "quantized mat-mul" : "quantized mat-vec"); }
        return output;
    }

    /// <summary>Prefill: bf16 activations, bf16 MFMA, FP32 accumulate (rows >= 16 in the reference's routing).</summary>
    public HipBuffer ForwardBFloat16(HipExecutionLane lane, HipBuffer inputBf16, HipBuffer? bias, int rows)
    {
        if (inputBf16.Bytes < (long)rows * InputWidth * sizeof(ushort))
            throw new ArgumentException("Quantized linear input width mismatch.", nameof(inputBf16));
        HipBuffer encoded = DevicePayload(lane);
        HipBuffer output = lane.Allocate(checked(rows * OutputWidth));
        int status = lane.Locked(h => NnHipNative.nnhip_quant_matmul_bf16(h, GgmlType, inputBf16.Pointer, encoded.Pointer,
            bias?.Pointer ?? 0, output.Pointer, rows, InputWidth, OutputWidth));
        if (status != 0) { output.Dispose(); NnHipNative.Check(status, "quantized mat-mul"); }
        return output;
    }

    /// <summary>Lazy one-time upload of the raw blocks (ArcQuantizedMatrix.DevicePayload).</summary>
    private HipBuffer DevicePayload(HipExecutionLane lane)
    {
        if (_devicePayload is not null && ReferenceEquals(_lane, lane)) return _devicePayload;
        if (_payload is null) throw new InvalidOperationException("The host payload was dropped; the matrix is bound to its first lane.");
        _devicePayload?.Dispose();
        _devicePayload = lane.UploadRaw(_payload);
        _lane = lane;
        return _devicePayload;
    }

    /// <summary>Keep only the device copy, as Qwen35QuantizedModel.LoadTensor does after upload.</summary>
    public void DropHostPayload()
    {
        if (_devicePayload is null) throw new InvalidOperationException("Upload first.");
        _payload = null;
    }

    public void Dispose()
    {
        _devicePayload?.Dispose();
        _devicePayload = null;
        _lane = null;
    }
}
