// Managed lane over libnnhip.so: the subset of ArcExecutionLane (NNtrain.Arc/ArcExecutionLane.cs) that the quantized
// linear operator uses - UploadRaw / Allocate / AllocateBytes / Read / Synchronize and the byte counters.
namespace NNtrain.Hip;

public sealed unsafe class HipExecutionLane : IDisposable
{
    private readonly object _sync = new();
    private nint _lane;

    public HipExecutionLane(int deviceIndex = 0)
    {
        NnHipNative.EnsureAbi();
        NnHipNative.Check(NnHipNative.nnhip_lane_create(deviceIndex, out _lane), "lane create");
        DeviceIndex = deviceIndex;
    }

    public int DeviceIndex { get; }
    internal nint Handle => _lane != 0 ? _lane : throw new ObjectDisposedException(nameof(HipExecutionLane));

    public static int DeviceCount()
    {
        NnHipNative.Check(NnHipNative.nnhip_device_count(out int count), "device count");
        return count;
    }

    public long H2DBytes => (long)Counters().H2DBytes;
    public long D2HBytes => (long)Counters().D2HBytes;
    public long AllocatedBytes => (long)Counters().AllocatedBytes;
    public long PeakAllocatedBytes => (long)Counters().PeakAllocatedBytes;

    /// <summary>Keeps every mat-vec of the lane on the FP32 row-step kernels: calls with several input rows then equal
    /// stacked single-row calls bit for bit (Qwen35InferencePrefillLinearTests.cs:64-77), without the shared
    /// matrix-core passes.</summary>
    public bool RowStepOnly
    {
        get
        {
            NnHipNative.Check(NnHipNative.nnhip_lane_get_option(Handle, NnHipNative.OptionRowStepOnly, out long value), "lane option");
            return value != 0;
        }
        set => NnHipNative.Check(NnHipNative.nnhip_lane_set_option(Handle, NnHipNative.OptionRowStepOnly, value ? 1 : 0), "lane option");
    }

    public HipBuffer Allocate(int elements) => AllocateBytes(checked(elements * sizeof(float)));

    public HipBuffer AllocateBytes(long bytes)
    {
        lock (_sync)
        {
            NnHipNative.Check(NnHipNative.nnhip_alloc(Handle, (nuint)bytes, out nint dptr), "alloc");
            return new HipBuffer(this, dptr, bytes);
        }
    }

    /// <summary>Uploads the array byte for byte (raw GGUF blocks stay encoded).</summary>
    public HipBuffer UploadRaw(ReadOnlySpan<byte> values)
    {
        HipBuffer buffer = AllocateBytes(Math.Max(values.Length, 4));
        lock (_sync)
            fixed (byte* host = values)
                NnHipNative.Check(NnHipNative.nnhip_upload(Handle, buffer.Pointer, 0, host, (nuint)values.Length), "upload");
        return buffer;
    }

    /// <summary>Uploads <paramref name="bytes"/> bytes that sit at <paramref name="fileOffset"/> of an open file: the
    /// library reads the range through two pinned buffers of its own, one travelling while the other is filled, so no
    /// managed array of the tensor's size exists (the pair ReadTensorBytes + UploadRaw of
    /// Qwen35QuantizedModel.LoadTensor in one call).  On Linux a SafeFileHandle's handle is the descriptor.</summary>
    public HipBuffer UploadFromFile(Microsoft.Win32.SafeHandles.SafeFileHandle file, long fileOffset, long bytes)
    {
        HipBuffer buffer = AllocateBytes(Math.Max(bytes, 4));
        bool held = false;
        try
        {
            file.DangerousAddRef(ref held);
            lock (_sync)
                NnHipNative.Check(NnHipNative.nnhip_upload_from_file(Handle, buffer.Pointer, 0, (int)file.DangerousGetHandle(),
                                                                     (ulong)fileOffset, (nuint)bytes), "upload");
        }
        catch
        {
            buffer.Dispose();
            throw;
        }
        finally
        {
            if (held) file.DangerousRelease();
        }
        return buffer;
    }

    public void Read(HipBuffer buffer, Span<float> values)
    {
        lock (_sync)
            fixed (float* host = values)
                NnHipNative.Check(NnHipNative.nnhip_download(Handle, buffer.Pointer, 0, host, (nuint)(values.Length * sizeof(float))), "download");
    }

    public void Synchronize()
    {
        lock (_sync) NnHipNative.Check(NnHipNative.nnhip_synchronize(Handle), "synchronize");
    }

    internal void Free(nint dptr)
    {
        lock (_sync) if (_lane != 0) NnHipNative.Check(NnHipNative.nnhip_free(_lane, dptr), "free");
    }

    internal T Locked<T>(Func<nint, T> call)
    {
        lock (_sync) return call(Handle);
    }

    private NnHipNative.LaneCounters Counters()
    {
        lock (_sync)
        {
            NnHipNative.Check(NnHipNative.nnhip_lane_get_counters(Handle, out var c, (nuint)sizeof(NnHipNative.LaneCounters)), "counters");
            return c;
        }
    }

    public void Dispose()
    {
        lock (_sync)
        {
            if (_lane == 0) return;
            nint lane = _lane;
            _lane = 0;
            NnHipNative.Check(NnHipNative.nnhip_lane_destroy(lane), "lane destroy");
        }
    }
}

/// <summary>Device allocation owned by a lane (the reference's ArcBuffer, ArcExecutionLane.cs:917-931).</summary>
public sealed class HipBuffer : IDisposable
{
    private readonly HipExecutionLane _lane;
    private nint _pointer;

    internal HipBuffer(HipExecutionLane lane, nint pointer, long bytes)
    {
        _lane = lane;
        _pointer = pointer;
        Bytes = bytes;
    }

    public long Bytes { get; }
    internal nint Pointer => _pointer != 0 ? _pointer : throw new ObjectDisposedException(nameof(HipBuffer));

    public void Dispose()
    {
        if (_pointer == 0) return;
        nint p = _pointer;
        _pointer = 0;
        _lane.Free(p);
    }
}
