// C ABI of libnnhip.so: lanes, device memory, transfers, error record, and validated dispatch to the kernels.
#include <cerrno>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>

#include <unistd.h>

#include "nnhip_internal.h"

namespace nnhip {

namespace {

std::mutex g_error_mutex;
nnhip_error_info g_last_error{sizeof(nnhip_error_info), (NNHIP_ABI_MAJOR << 16) | NNHIP_ABI_MINOR, 0, 0, -1, 0, 0};
char g_last_message[256] = "";

Lane* as_lane(void* h)
{
    Lane* l = static_cast<Lane*>(h);
    return (l && l->magic == kLaneMagic) ? l : nullptr;
}

int hip_fail(hipError_t e, uint32_t op, int device, const char* what)
{
    return fail(NNHIP_ERR_HIP, op, device, static_cast<uint32_t>(e), "%s failed: %s (%d)", what, hipGetErrorString(e),
                static_cast<int>(e));
}

#define NNHIP_LANE(handle, op)                                                                     \
    Lane* lane = as_lane(handle);                                                                  \
    if (!lane) return fail(NNHIP_ERR_BAD_HANDLE, op, -1, 0, "lane handle is null or not a lane");   \
    {                                                                                              \
        hipError_t e_ = hipSetDevice(lane->device);                                                \
        if (e_ != hipSuccess) return hip_fail(e_, op, lane->device, "hipSetDevice");               \
    }

// Shape checks shared by the compute entries; mirror ArcQuantizedMatrix's constructor and Forward
// (NNtrain.Core/Serialization/ArcQuantizedMatrix.cs:20-32,49-54).
int check_linear(uint32_t op, Lane* lane, uint32_t type, const void* x, const void* w, const void* y, int rows, int in_w,
                 int out_w)
{
    int elems = 0, bytes = 0;
    if (!type_block(type, &elems, &bytes))
        return fail(NNHIP_ERR_UNSUPPORTED_TYPE, op, lane->device, 0, "GGML type %u is not a supported quantized matrix type", type);
    if (!x || !w || !y) return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "x, w and y must be non-null");
    if (rows < 1 || in_w < 1 || out_w < 1)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "rows, in_w and out_w must be positive (got %d, %d, %d)", rows, in_w, out_w);
    if (in_w % elems != 0)
        return fail(NNHIP_ERR_INCOMPLETE_BLOCKS, op, lane->device, 0, "quantized rows must contain complete %d-value blocks (in_w = %d)", elems, in_w);
    if ((reinterpret_cast<uintptr_t>(x) & 15u) || (reinterpret_cast<uintptr_t>(y) & 3u))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "x must be 16-byte aligned and y 4-byte aligned");
    if (type == NNHIP_TYPE_BF16 && op != NNHIP_OP_DEQUANTIZE && in_w % 64 != 0)
        return fail(NNHIP_ERR_INCOMPLETE_BLOCKS, op, lane->device, 0, "bfloat16 rows must hold a multiple of 64 weights (in_w = %d)", in_w);
    const uintptr_t wa = (type == NNHIP_TYPE_Q4_K || type == NNHIP_TYPE_Q5_K || type == NNHIP_TYPE_BF16) ? 15u : 3u;
    if (reinterpret_cast<uintptr_t>(w) & wa)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "weight pointer must be %u-byte aligned", static_cast<unsigned>(wa + 1));
    return NNHIP_OK;
}

// Moves `bytes` bytes to the device through the lane's two pinned staging buffers: `fill(dst, done, want)` puts bytes
// [done, done + want) of the source into `dst` (returning a status), and piece i is filled into buffer i % 2 while
// piece i - 1 travels from the other one; a buffer is reused once the copy that last read it has completed.  On any
// failure the stream is drained before returning: no copy may still read a buffer that the next call fills.
template <class Fill>
int staged_upload(nnhip::Lane* lane, void* dptr, size_t offset, size_t bytes, Fill&& fill)
{
    for (int i = 0; i < 2; ++i) {
        if (!lane->staging[i]) {
            const hipError_t e = hipHostMalloc(&lane->staging[i], kStagingBytes, hipHostMallocDefault);
            if (e == hipSuccess) ++lane->counters.driver_allocations;
            if (e != hipSuccess) {
                lane->staging[i] = nullptr;
                return hip_fail(e, NNHIP_OP_UPLOAD, lane->device, "pinned staging buffer");
            }
        }
        if (!lane->staging_done[i]) {
            const hipError_t e = hipEventCreateWithFlags(&lane->staging_done[i], hipEventDisableTiming);
            if (e != hipSuccess) {
                lane->staging_done[i] = nullptr;
                return hip_fail(e, NNHIP_OP_UPLOAD, lane->device, "staging event");
            }
        }
    }
    size_t done = 0;
    int status = NNHIP_OK;
    for (int piece = 0; done < bytes; ++piece) {
        const int slot = piece & 1;
        if (piece >= 2) {
            const hipError_t e = hipEventSynchronize(lane->staging_done[slot]);
            if (e != hipSuccess) {
                status = hip_fail(e, NNHIP_OP_UPLOAD, lane->device, "waiting for a staging buffer");
                break;
            }
        }
        const size_t want = bytes - done < kStagingBytes ? bytes - done : kStagingBytes;
        status = fill(lane->staging[slot], done, want);
        if (status != NNHIP_OK) break;
        hipError_t e = hipMemcpyAsync(static_cast<char*>(dptr) + offset + done, lane->staging[slot], want, hipMemcpyHostToDevice, lane->stream);
        if (e == hipSuccess) e = hipEventRecord(lane->staging_done[slot], lane->stream);
        if (e != hipSuccess) {
            status = hip_fail(e, NNHIP_OP_UPLOAD, lane->device, "host-to-device copy");
            break;
        }
        done += want;
    }
    const hipError_t e = hipStreamSynchronize(lane->stream);
    if (status == NNHIP_OK && e != hipSuccess) status = hip_fail(e, NNHIP_OP_UPLOAD, lane->device, "host-to-device copy");
    std::lock_guard<std::mutex> guard(lane->mutex);
    lane->counters.h2d_bytes += done;
    return status;
}

}  // namespace

bool type_block(uint32_t type, int* elems, int* bytes)
{
    int e = 0, b = 0;
    switch (type) {
    case NNHIP_TYPE_Q8_0: e = 32; b = 34; break;
    case NNHIP_TYPE_Q4_K: e = 256; b = 144; break;
    case NNHIP_TYPE_Q5_K: e = 256; b = 176; break;
    case NNHIP_TYPE_Q6_K: e = 256; b = 210; break;
    case NNHIP_TYPE_IQ3_S: e = 256; b = 110; break;
    case NNHIP_TYPE_IQ2_S: e = 256; b = 82; break;
    case NNHIP_TYPE_BF16: e = 1; b = 2; break;
    default: return false;
    }
    if (elems) *elems = e;
    if (bytes) *bytes = b;
    return true;
}

int fail(int status, uint32_t op, int device, uint32_t hip_error, const char* fmt, ...)
{
    std::lock_guard<std::mutex> guard(g_error_mutex);
    g_last_error.sequence += 1;
    g_last_error.status = status;
    g_last_error.device_index = device;
    g_last_error.operation = op;
    g_last_error.reserved = hip_error;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_message, sizeof(g_last_message), fmt, ap);
    va_end(ap);
    return status;
}

}  // namespace nnhip

using namespace nnhip;

extern "C" {

uint32_t nnhip_abi_version(void) { return (NNHIP_ABI_MAJOR << 16) | NNHIP_ABI_MINOR; }

int nnhip_last_error(nnhip_error_info* out, size_t out_size)
{
    if (!out || out_size < sizeof(nnhip_error_info)) return NNHIP_ERR_INVALID_ARGUMENT;
    std::lock_guard<std::mutex> guard(g_error_mutex);
    *out = g_last_error;
    return NNHIP_OK;
}

int nnhip_last_error_message(char* buf, int cap)
{
    if (!buf || cap < 1) return NNHIP_ERR_INVALID_ARGUMENT;
    std::lock_guard<std::mutex> guard(g_error_mutex);
    snprintf(buf, static_cast<size_t>(cap), "%s", g_last_message);
    return NNHIP_OK;
}

int nnhip_device_count(int* count)
{
    if (!count) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_DEVICE_QUERY, -1, 0, "count is null");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e == hipErrorNoDevice) {
        *count = 0;
        return NNHIP_OK;
    }
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_DEVICE_QUERY, -1, "hipGetDeviceCount");
    *count = n;
    return NNHIP_OK;
}

int nnhip_device_name(int device, char* buf, int cap)
{
    if (!buf || cap < 1) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_DEVICE_QUERY, device, 0, "buffer is null or empty");
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_DEVICE_QUERY, device, "hipGetDeviceProperties");
    snprintf(buf, static_cast<size_t>(cap), "%s (%s)", prop.name, prop.gcnArchName);
    return NNHIP_OK;
}

int nnhip_device_info(int device, int* compute_units, uint64_t* total_memory_bytes)
{
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_DEVICE_QUERY, device, "hipGetDeviceProperties");
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_memory_bytes) *total_memory_bytes = prop.totalGlobalMem;
    return NNHIP_OK;
}

int nnhip_type_block(uint32_t ggml_type, int* block_elems, int* block_bytes)
{
    if (!type_block(ggml_type, block_elems, block_bytes))
        return fail(NNHIP_ERR_UNSUPPORTED_TYPE, NNHIP_OP_NONE, -1, 0, "GGML type %u is not a supported quantized matrix type", ggml_type);
    return NNHIP_OK;
}

int nnhip_matrix_bytes(uint32_t ggml_type, int in_w, int out_w, uint64_t* bytes)
{
    int elems = 0, bb = 0;
    if (!type_block(ggml_type, &elems, &bb))
        return fail(NNHIP_ERR_UNSUPPORTED_TYPE, NNHIP_OP_NONE, -1, 0, "GGML type %u is not a supported quantized matrix type", ggml_type);
    if (!bytes || in_w < 1 || out_w < 1)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_NONE, -1, 0, "widths must be positive and bytes non-null");
    if (in_w % elems != 0)
        return fail(NNHIP_ERR_INCOMPLETE_BLOCKS, NNHIP_OP_NONE, -1, 0, "quantized rows must contain complete %d-value blocks", elems);
    *bytes = static_cast<uint64_t>(out_w) * static_cast<uint64_t>(in_w / elems) * static_cast<uint64_t>(bb);
    return NNHIP_OK;
}

int nnhip_lane_create(int device, void** out)
{
    if (!out) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_LANE_CREATE, device, 0, "lane output pointer is null");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) return fail(NNHIP_ERR_NO_DEVICE, NNHIP_OP_LANE_CREATE, device, static_cast<uint32_t>(e), "no HIP device is available");
    if (device < 0 || device >= n)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_LANE_CREATE, device, 0, "device index %d is outside 0..%d", device, n - 1);
    e = hipSetDevice(device);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_LANE_CREATE, device, "hipSetDevice");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_LANE_CREATE, device, "hipGetDeviceProperties");
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(NNHIP_ERR_NO_DEVICE, NNHIP_OP_LANE_CREATE, device, 0, "device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
    Lane* lane = new (std::nothrow) Lane();
    if (!lane) return fail(NNHIP_ERR_OUT_OF_MEMORY, NNHIP_OP_LANE_CREATE, device, 0, "host allocation failed");
    lane->device = device;
    lane->compute_units = prop.multiProcessorCount;
    lane->counters.struct_size = sizeof(nnhip_lane_counters);
    e = hipStreamCreateWithFlags(&lane->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete lane;
        return hip_fail(e, NNHIP_OP_LANE_CREATE, device, "hipStreamCreateWithFlags");
    }
    // the fixed batch workspace: every device has its own copy of the array, at its own address; the lanes of a device
    // take its slices in rotation
    static std::atomic<unsigned> lane_serial[64];
    e = static_table_address(&lane->static_table, lane_serial[device & 63].fetch_add(1u));
    if (e != hipSuccess || !lane->static_table) {
        (void)hipStreamDestroy(lane->stream);
        delete lane;
        return hip_fail(e, NNHIP_OP_LANE_CREATE, device, "hipGetSymbolAddress of the fixed batch workspace");
    }
    // the descriptor table of batched launches starts with room for 819 mat-vec rows, so that small batches (and calls
    // with a few input rows, which use it) never have to grow it inside a graph capture
    e = hipMalloc(&lane->batch_table, 65536);
    if (e == hipSuccess) ++lane->counters.driver_allocations;
    if (e != hipSuccess) {
        (void)hipStreamDestroy(lane->stream);
        delete lane;
        return hip_fail(e, NNHIP_OP_LANE_CREATE, device, "hipMalloc of the batch descriptor table");
    }
    lane->batch_table_bytes = 65536;
    *out = lane;
    return NNHIP_OK;
}

int nnhip_lane_destroy(void* handle)
{
    NNHIP_LANE(handle, NNHIP_OP_LANE_DESTROY)
    hipError_t first = hipStreamSynchronize(lane->stream);
    for (auto& kv : lane->buffers) {
        hipError_t e = hipFree(kv.first);
        if (first == hipSuccess) first = e;
    }
    lane->buffers.clear();
    for (auto& kv : lane->free_blocks)
        for (void* p : kv.second) {
            hipError_t e = hipFree(p);
            if (first == hipSuccess) first = e;
        }
    lane->free_blocks.clear();
    for (const auto& b : lane->capture_pinned) (void)hipFree(b.first);
    lane->capture_pinned.clear();
    for (Graph* gr : lane->graphs) {            // graphs the caller never destroyed: their scratch blocks go with the lane
        for (const auto& b : gr->pinned) (void)hipFree(b.first);
        gr->pinned.clear();
    }
    lane->graphs.clear();
    if (lane->batch_table) (void)hipFree(lane->batch_table);
    for (void* t : lane->retired_tables) (void)hipFree(t);
    for (int i = 0; i < 2; ++i) {
        if (lane->staging[i]) (void)hipHostFree(lane->staging[i]);
        if (lane->staging_done[i]) (void)hipEventDestroy(lane->staging_done[i]);
    }
    hipError_t e = hipStreamDestroy(lane->stream);
    if (first == hipSuccess) first = e;
    const int device = lane->device;
    lane->magic = 0;
    delete lane;
    if (first != hipSuccess) return hip_fail(first, NNHIP_OP_LANE_DESTROY, device, "lane teardown");
    return NNHIP_OK;
}

// Allocation sizes are rounded up to 256 bytes and freed blocks of up to kCacheBlockMax are kept by the lane for the
// next request of that size: the operator pattern of the reference allocates the output of every projection and
// disposes it after use (Qwen35QuantizedModel.cs:488-491), which must not cost a device synchronisation per call.
int nnhip_alloc(void* handle, size_t bytes, void** dptr)
{
    NNHIP_LANE(handle, NNHIP_OP_ALLOC)
    if (!dptr || bytes == 0) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_ALLOC, lane->device, 0, "allocation size must be positive and dptr non-null");
    const size_t capacity = (bytes + 255u) & ~static_cast<size_t>(255u);
    void* p = nullptr;
    {
        std::lock_guard<std::mutex> guard(lane->mutex);
        auto it = lane->free_blocks.find(capacity);
        if (it != lane->free_blocks.end() && !it->second.empty()) {
            p = it->second.back();
            it->second.pop_back();
            lane->cached_bytes -= capacity;
        }
    }
    if (!p) {
        if (lane->capturing) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_ALLOC, lane->device, 0, "no new device allocation while a graph is being captured (only blocks freed earlier can be handed out)");
        hipError_t e = hipMalloc(&p, capacity);
        if (e == hipErrorOutOfMemory) {
            (void)hipGetLastError();
            // give the cached blocks back and try once more
            if (nnhip_lane_trim(handle) == NNHIP_OK) e = hipMalloc(&p, capacity);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return fail(NNHIP_ERR_OUT_OF_MEMORY, NNHIP_OP_ALLOC, lane->device, static_cast<uint32_t>(e), "device allocation of %zu bytes failed", bytes);
            }
        }
        if (e != hipSuccess) return hip_fail(e, NNHIP_OP_ALLOC, lane->device, "hipMalloc");
        std::lock_guard<std::mutex> guard(lane->mutex);
        ++lane->counters.driver_allocations;
    }
    std::lock_guard<std::mutex> guard(lane->mutex);
    lane->buffers.emplace(p, Lane::Block{bytes, capacity});
    lane->counters.allocated_bytes += bytes;
    if (lane->counters.allocated_bytes > lane->counters.peak_allocated_bytes)
        lane->counters.peak_allocated_bytes = lane->counters.allocated_bytes;
    *dptr = p;
    return NNHIP_OK;
}

int nnhip_free(void* handle, void* dptr)
{
    NNHIP_LANE(handle, NNHIP_OP_FREE)
    if (!dptr) return NNHIP_OK;
    size_t capacity = 0;
    {
        std::lock_guard<std::mutex> guard(lane->mutex);
        auto it = lane->buffers.find(dptr);
        if (it == lane->buffers.end())
            return fail(NNHIP_ERR_BAD_HANDLE, NNHIP_OP_FREE, lane->device, 0, "pointer was not allocated by this lane");
        capacity = it->second.capacity;
        const bool keep = capacity <= kCacheBlockMax && lane->cached_bytes + capacity <= kCacheTotalMax;
        if (!keep && lane->capturing)
            return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_FREE, lane->device, 0, "a block this large cannot be freed while a graph is being captured");
        lane->counters.allocated_bytes -= it->second.bytes;
        lane->buffers.erase(it);
        if (keep && lane->capturing) {
            // the work being recorded names this block: it stays out of circulation until the graph is destroyed
            lane->capture_pinned.emplace_back(dptr, capacity);
            return NNHIP_OK;
        }
        if (keep) {
            lane->free_blocks[capacity].push_back(dptr);
            lane->cached_bytes += capacity;
            return NNHIP_OK;
        }
    }
    // Returned to the driver.  Work already enqueued may still read the buffer: drain the lane's stream first (hipFree
    // itself only waits for the null stream, which a non-blocking stream does not join).
    hipError_t e = hipStreamSynchronize(lane->stream);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_FREE, lane->device, "hipStreamSynchronize");
    e = hipFree(dptr);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_FREE, lane->device, "hipFree");
    return NNHIP_OK;
}

int nnhip_lane_trim(void* handle)
{
    NNHIP_LANE(handle, NNHIP_OP_FREE)
    if (lane->capturing) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_FREE, lane->device, 0, "no trim while a graph is being captured");
    std::unordered_map<size_t, std::vector<void*>> blocks;
    {
        std::lock_guard<std::mutex> guard(lane->mutex);
        blocks.swap(lane->free_blocks);
        lane->cached_bytes = 0;
    }
    hipError_t first = hipStreamSynchronize(lane->stream);
    for (auto& kv : blocks)
        for (void* p : kv.second) {
            const hipError_t e = hipFree(p);
            if (first == hipSuccess) first = e;
        }
    if (first != hipSuccess) return hip_fail(first, NNHIP_OP_FREE, lane->device, "trim");
    return NNHIP_OK;
}

int nnhip_upload(void* handle, void* dptr, size_t offset, const void* host, size_t bytes)
{
    NNHIP_LANE(handle, NNHIP_OP_UPLOAD)
    if (bytes == 0) return NNHIP_OK;
    if (!dptr || !host) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_UPLOAD, lane->device, 0, "null pointer");
    if (lane->capturing) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_UPLOAD, lane->device, 0, "no transfer while a graph is being captured");
    hipError_t e = hipMemcpyAsync(static_cast<char*>(dptr) + offset, host, bytes, hipMemcpyHostToDevice, lane->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(lane->stream);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_UPLOAD, lane->device, "host-to-device copy");
    std::lock_guard<std::mutex> guard(lane->mutex);
    lane->counters.h2d_bytes += bytes;
    return NNHIP_OK;
}

int nnhip_upload_from_file(void* handle, void* dptr, size_t offset, int fd, uint64_t file_offset, size_t bytes)
{
    NNHIP_LANE(handle, NNHIP_OP_UPLOAD)
    if (bytes == 0) return NNHIP_OK;
    if (!dptr || fd < 0) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_UPLOAD, lane->device, 0, "null device pointer or negative file descriptor");
    if (lane->capturing) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_UPLOAD, lane->device, 0, "no transfer while a graph is being captured");
    const int device = lane->device;
    return staged_upload(lane, dptr, offset, bytes, [&](void* dst, size_t done, size_t want) {
        size_t got = 0;
        while (got < want) {
            const ssize_t n = pread(fd, static_cast<char*>(dst) + got, want - got, static_cast<off_t>(file_offset + done + got));
            if (n > 0) {
                got += static_cast<size_t>(n);
            } else if (n == 0) {
                return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_UPLOAD, device, 0,
                            "the file ends %zu bytes before the end of the range", bytes - done - got);
            } else if (errno != EINTR) {
                return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_UPLOAD, device, 0, "reading the file failed: %s", strerror(errno));
            }
        }
        return static_cast<int>(NNHIP_OK);
    });
}

int nnhip_download(void* handle, const void* dptr, size_t offset, void* host, size_t bytes)
{
    NNHIP_LANE(handle, NNHIP_OP_DOWNLOAD)
    if (bytes == 0) return NNHIP_OK;
    if (!dptr || !host) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_DOWNLOAD, lane->device, 0, "null pointer");
    if (lane->capturing) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_DOWNLOAD, lane->device, 0, "no transfer while a graph is being captured");
    hipError_t e = hipMemcpyAsync(host, static_cast<const char*>(dptr) + offset, bytes, hipMemcpyDeviceToHost, lane->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(lane->stream);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_DOWNLOAD, lane->device, "device-to-host copy");
    std::lock_guard<std::mutex> guard(lane->mutex);
    lane->counters.d2h_bytes += bytes;
    return NNHIP_OK;
}

int nnhip_copy(void* handle, void* dst, size_t dst_offset, const void* src, size_t src_offset, size_t bytes)
{
    NNHIP_LANE(handle, NNHIP_OP_COPY)
    if (bytes == 0) return NNHIP_OK;
    if (!dst || !src) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_COPY, lane->device, 0, "null pointer");
    hipError_t e = hipMemcpyAsync(static_cast<char*>(dst) + dst_offset, static_cast<const char*>(src) + src_offset, bytes,
                                  hipMemcpyDeviceToDevice, lane->stream);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_COPY, lane->device, "device-to-device copy");
    return NNHIP_OK;
}

int nnhip_fill_u32(void* handle, void* dptr, size_t offset, uint32_t value, size_t count)
{
    NNHIP_LANE(handle, NNHIP_OP_FILL)
    if (!dptr || (offset & 3u)) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_FILL, lane->device, 0, "null pointer or offset not a multiple of 4");
    hipError_t e = launch_fill_u32(lane, reinterpret_cast<uint32_t*>(static_cast<char*>(dptr) + offset), value, count);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_FILL, lane->device, "fill launch");
    return NNHIP_OK;
}

int nnhip_synchronize(void* handle)
{
    NNHIP_LANE(handle, NNHIP_OP_SYNCHRONIZE)
    if (lane->capturing) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_SYNCHRONIZE, lane->device, 0, "no synchronise while a graph is being captured");
    hipError_t e = hipStreamSynchronize(lane->stream);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_SYNCHRONIZE, lane->device, "hipStreamSynchronize");
    return NNHIP_OK;
}

int nnhip_lane_get_counters(void* handle, nnhip_lane_counters* out, size_t out_size)
{
    Lane* lane = as_lane(handle);
    if (!lane) return fail(NNHIP_ERR_BAD_HANDLE, NNHIP_OP_NONE, -1, 0, "lane handle is null or not a lane");
    if (!out || out_size < sizeof(nnhip_lane_counters)) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_NONE, lane->device, 0, "counter buffer too small");
    std::lock_guard<std::mutex> guard(lane->mutex);
    *out = lane->counters;
    return NNHIP_OK;
}

int nnhip_lane_stream(void* handle, void** stream)
{
    Lane* lane = as_lane(handle);
    if (!lane || !stream) return fail(NNHIP_ERR_BAD_HANDLE, NNHIP_OP_NONE, -1, 0, "lane handle is null or not a lane");
    *stream = lane->stream;
    return NNHIP_OK;
}

int nnhip_lane_set_option(void* handle, uint32_t option, int64_t value)
{
    NNHIP_LANE(handle, NNHIP_OP_NONE)
    if (option != NNHIP_OPTION_ROW_STEP_ONLY)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_NONE, lane->device, 0, "unknown lane option %u", option);
    std::lock_guard<std::mutex> guard(lane->mutex);
    lane->row_step_only = value != 0;
    return NNHIP_OK;
}

int nnhip_lane_get_option(void* handle, uint32_t option, int64_t* value)
{
    NNHIP_LANE(handle, NNHIP_OP_NONE)
    if (option != NNHIP_OPTION_ROW_STEP_ONLY || !value)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_NONE, lane->device, 0, "unknown lane option %u, or value is null", option);
    *value = lane->row_step_only ? 1 : 0;
    return NNHIP_OK;
}

int nnhip_dequantize(void* handle, uint32_t ggml_type, const void* w, float* out, int64_t elements)
{
    NNHIP_LANE(handle, NNHIP_OP_DEQUANTIZE)
    int elems = 0, bytes = 0;
    if (!type_block(ggml_type, &elems, &bytes))
        return fail(NNHIP_ERR_UNSUPPORTED_TYPE, NNHIP_OP_DEQUANTIZE, lane->device, 0, "GGML type %u is not a supported quantized matrix type", ggml_type);
    if (elements < 0) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_DEQUANTIZE, lane->device, 0, "element count must be non-negative");
    if (ggml_type == NNHIP_TYPE_BF16) elems = 4;     // decoded four at a time
    if (elements % elems != 0)
        return fail(NNHIP_ERR_INCOMPLETE_BLOCKS, NNHIP_OP_DEQUANTIZE, lane->device, 0, "element count must be a multiple of %d", elems);
    if (elements == 0) return NNHIP_OK;
    if (!w || !out) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_DEQUANTIZE, lane->device, 0, "null pointer");
    const uintptr_t wa = (ggml_type == NNHIP_TYPE_Q4_K || ggml_type == NNHIP_TYPE_Q5_K) ? 3u : 1u;
    if ((reinterpret_cast<uintptr_t>(out) & 15u) || (reinterpret_cast<uintptr_t>(w) & wa))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_DEQUANTIZE, lane->device, 0, "out must be 16-byte aligned and w %u-byte aligned", static_cast<unsigned>(wa + 1));
    hipError_t e = launch_dequantize(lane, ggml_type, w, out, elements);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_DEQUANTIZE, lane->device, "dequantize launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_quant_matvec(void* handle, uint32_t ggml_type, const float* x, const void* w, const float* bias, float* y,
                       int rows, int in_w, int out_w)
{
    NNHIP_LANE(handle, NNHIP_OP_MATVEC)
    int rc = check_linear(NNHIP_OP_MATVEC, lane, ggml_type, x, w, y, rows, in_w, out_w);
    if (rc != NNHIP_OK) return rc;
    if (in_w > matvec_max_in_w(ggml_type))
        return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_MATVEC, lane->device, 0, "in_w %d exceeds the %d values one workgroup can stage", in_w, matvec_max_in_w(ggml_type));
    if (rows > 65535) return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_MATVEC, lane->device, 0, "rows %d exceeds 65535", rows);
    if (const int per_pass = lane->row_step_only ? 0 : matvec_rows_per_pass(ggml_type, rows, in_w, out_w, w, lane->compute_units)) {
        // two or more input rows of a large matrix: up to four rows share a pass over the weights on the matrix cores,
        // sixteen rows go into a launch (the reference routes such calls to row-tiled kernels,
        // Qwen35QuantizedModel.cs:1335-1344)
        int launches = 0;
        const hipError_t e = launch_matvec_rows_shared(lane, ggml_type, x, w, bias, y, rows, in_w, out_w, per_pass, &launches);
        lane->counters.kernel_launches += static_cast<uint64_t>(launches);
        if (e != hipSuccess) return hip_fail(e, NNHIP_OP_MATVEC, lane->device, "mat-vec launch");
        return NNHIP_OK;
    }
    hipError_t e = launch_matvec(lane, ggml_type, x, w, bias, y, rows, in_w, out_w);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_MATVEC, lane->device, "mat-vec launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_matvec_plan(uint32_t ggml_type, int rows, int in_w, int out_w, int compute_units, nnhip_matvec_plan_info* info)
{
    int elems = 0;
    if (!type_block(ggml_type, &elems, nullptr))
        return fail(NNHIP_ERR_UNSUPPORTED_TYPE, NNHIP_OP_MATVEC, -1, 0, "GGML type %u is not a supported quantized matrix type", ggml_type);
    if (!info || info->struct_size != sizeof(nnhip_matvec_plan_info))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_MATVEC, -1, 0, "info is null or has the wrong struct_size");
    if (rows < 1 || in_w < 1 || out_w < 1 || compute_units < 1)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_MATVEC, -1, 0, "rows, in_w, out_w and compute_units must be positive");
    if (in_w % elems != 0 || (ggml_type == NNHIP_TYPE_BF16 && in_w % 64 != 0))
        return fail(NNHIP_ERR_INCOMPLETE_BLOCKS, NNHIP_OP_MATVEC, -1, 0, "quantized rows must contain complete blocks (in_w = %d)", in_w);
    if (in_w > matvec_max_in_w(ggml_type) || !describe_matvec(ggml_type, rows, in_w, out_w, compute_units, info))
        return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_MATVEC, -1, 0, "in_w %d exceeds the %d values one workgroup can stage", in_w, matvec_max_in_w(ggml_type));
    return NNHIP_OK;
}

static int check_norm(uint32_t op, nnhip::Lane* lane, const void* input, const void* weight, const void* output, int rows,
                      int width, int input_stride, float epsilon)
{
    using namespace nnhip;
    if (!input || !weight || !output)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "input, weight and output must be non-null");
    if (rows < 1 || width < 1 || input_stride < width)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "rows and width must be positive and input_stride >= width");
    if (!(epsilon >= 0.0f) || !std::isfinite(epsilon))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "epsilon must be finite and not negative");
    if (rows > 65535) return fail(NNHIP_ERR_TOO_LARGE, op, lane->device, 0, "rows %d exceeds 65535", rows);
    return NNHIP_OK;
}

int nnhip_rms_norm(void* handle, const float* input, const float* weight, float* output, int rows, int width,
                   int input_stride, float epsilon)
{
    NNHIP_LANE(handle, NNHIP_OP_RMS_NORM)
    int rc = check_norm(NNHIP_OP_RMS_NORM, lane, input, weight, output, rows, width, input_stride, epsilon);
    if (rc != NNHIP_OK) return rc;
    hipError_t e = launch_rms_norm(lane, const_cast<float*>(input), nullptr, weight, output, rows, width, input_stride, epsilon);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_RMS_NORM, lane->device, "RMSNorm launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_add_rms_norm(void* handle, float* destination, const float* residual, const float* weight, float* output,
                       int rows, int width, int input_stride, float epsilon)
{
    NNHIP_LANE(handle, NNHIP_OP_RMS_NORM)
    int rc = check_norm(NNHIP_OP_RMS_NORM, lane, destination, weight, output, rows, width, input_stride, epsilon);
    if (rc != NNHIP_OK) return rc;
    if (!residual) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_RMS_NORM, lane->device, 0, "residual must be non-null");
    hipError_t e = launch_rms_norm(lane, destination, residual, weight, output, rows, width, input_stride, epsilon);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_RMS_NORM, lane->device, "add + RMSNorm launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_silu_multiply(void* handle, const float* gate, const float* up, float* output, int length)
{
    NNHIP_LANE(handle, NNHIP_OP_SILU_MULTIPLY)
    if (!gate || !up || !output || length < 1)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_SILU_MULTIPLY, lane->device, 0, "pointers must be non-null and length positive");
    hipError_t e = launch_silu_multiply(lane, gate, up, output, length);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_SILU_MULTIPLY, lane->device, "SiLU multiply launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_add_in_place(void* handle, float* destination, const float* source, int length)
{
    NNHIP_LANE(handle, NNHIP_OP_ADD_IN_PLACE)
    if (!destination || !source || length < 1)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_ADD_IN_PLACE, lane->device, 0, "pointers must be non-null and length positive");
    hipError_t e = launch_add_in_place(lane, destination, source, length);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_ADD_IN_PLACE, lane->device, "add launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_quant_matvec_fused(void* handle, const nnhip_fused_matvec_desc* d)
{
    NNHIP_LANE(handle, NNHIP_OP_MATVEC_FUSED)
    const uint32_t op = NNHIP_OP_MATVEC_FUSED;
    if (!d || d->struct_size != sizeof(nnhip_fused_matvec_desc))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "descriptor is null or has the wrong struct_size");
    int rc = check_linear(op, lane, d->ggml_type, d->x, d->w, d->y, 1, d->in_w, d->out_w);
    if (rc != NNHIP_OK) return rc;
    if (d->in_w > matvec_max_in_w(d->ggml_type))
        return fail(NNHIP_ERR_TOO_LARGE, op, lane->device, 0, "in_w %d exceeds the %d values one workgroup can stage", d->in_w, matvec_max_in_w(d->ggml_type));
    if (!matvec_fused_supported(d->ggml_type, d->in_w))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "Q8_0 rows with an odd number of blocks are not covered by the fused mat-vec");
    auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    if (!aligned(d->x2) || !aligned(d->norm_weight) || !aligned(d->x_out) || !aligned(d->sum_out))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "x2, norm_weight, x_out and sum_out must be 16-byte aligned");
    switch (d->pre_op) {
    case NNHIP_PRE_NONE:
        if (d->x2 || d->norm_weight || d->x_out || d->sum_out)
            return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "x2, norm_weight, x_out and sum_out must be null without a pre-op");
        break;
    case NNHIP_PRE_RMS_NORM:
        if (!d->norm_weight) return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "norm_weight is null");
        if (!(d->epsilon >= 0.0f) || !std::isfinite(d->epsilon))
            return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "epsilon must be finite and not negative");
        if (d->sum_out && !d->x2) return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "sum_out needs a residual (x2)");
        break;
    case NNHIP_PRE_SILU_MULTIPLY:
        if (!d->x2) return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "the up vector (x2) is null");
        if (d->norm_weight || d->sum_out)
            return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "norm_weight and sum_out must be null for SiLU * up");
        break;
    default:
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "unknown pre_op %u", d->pre_op);
    }
    if (d->reserved != 0) return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "reserved must be 0");
    if (d->x_head_width < 0 || d->x_head_group < 0 || (d->x_head_width > 0) != (d->x_head_group > 0))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "x_head_width and x_head_group must both be positive or both be zero");
    if (d->x_head_width > 0 && (d->x_head_width % 4 != 0 || d->in_w % (d->x_head_width * d->x_head_group) != 0 || d->pre_op != NNHIP_PRE_NONE))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0,
                    "x_head_width must be a multiple of 4, in_w a whole number of head groups, and pre_op NNHIP_PRE_NONE");
    if (d->post_op != NNHIP_POST_NONE) {
        if (d->post_op != NNHIP_POST_SILU_PAIR) return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "unknown post_op %u", d->post_op);
        if (d->out_w % 2 != 0 || d->addend || d->lora_rank != 0 || d->pre_op == NNHIP_PRE_SILU_MULTIPLY || d->x_head_width > 0)
            return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0,
                        "NNHIP_POST_SILU_PAIR needs an even out_w, no addend, no low-rank branch, and pre_op NNHIP_PRE_NONE or NNHIP_PRE_RMS_NORM");
    }
    if (d->lora_rank < 0 || (d->lora_rank > 0 && (!d->lora_z || !d->lora_b)) || (d->lora_rank == 0 && (d->lora_z || d->lora_b)))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "lora_z and lora_b go with a positive lora_rank, and only with one");
    if (d->lora_rank > 0 && !std::isfinite(d->lora_scale))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "lora_scale must be finite");
    const size_t xbytes = static_cast<size_t>(d->in_w) * sizeof(float);
    auto overlaps = [&](const float* out, const float* in) {
        if (!out || !in) return false;
        const char* a = reinterpret_cast<const char*>(out);
        const char* b = reinterpret_cast<const char*>(in);
        return a < b + xbytes && b < a + xbytes;
    };
    if (overlaps(d->x_out, d->x) || overlaps(d->x_out, d->x2) || overlaps(d->sum_out, d->x) || overlaps(d->sum_out, d->x2) ||
        overlaps(d->x_out, d->sum_out))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, op, lane->device, 0, "x_out and sum_out must not overlap the inputs or each other");
    hipError_t e = launch_matvec_fused(lane, *d);
    if (e != hipSuccess) return hip_fail(e, op, lane->device, "fused mat-vec launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_first_token_attention(void* handle, const float* v, float* out, int heads, int kv_heads, int head_width)
{
    NNHIP_LANE(handle, NNHIP_OP_ATTENTION)
    if (!v || !out || heads < 1 || kv_heads < 1 || head_width < 1 || heads % kv_heads != 0)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_ATTENTION, lane->device, 0, "pointers must be non-null, counts positive and heads a multiple of kv_heads");
    if (static_cast<int64_t>(heads) * head_width > 0x7fffffff)
        return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_ATTENTION, lane->device, 0, "heads * head_width exceeds one launch");
    hipError_t e = launch_first_token_attention(lane, v, out, heads, kv_heads, head_width);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_ATTENTION, lane->device, "first-token attention launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_lora_a(void* handle, const float* x, const float* a, float* z, int rows, int width, int rank)
{
    NNHIP_LANE(handle, NNHIP_OP_LORA)
    if (!x || !a || !z || rows < 1 || width < 1 || rank < 1)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_LORA, lane->device, 0, "pointers must be non-null and rows, width, rank positive");
    if (static_cast<int64_t>(rows) * rank > 0x7fffffff)
        return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_LORA, lane->device, 0, "rows * rank exceeds one launch");
    hipError_t e = launch_lora_a(lane, x, a, z, rows, width, rank);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_LORA, lane->device, "adapter A launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_lora_b(void* handle, const float* z, const float* b, float* y, int rows, int output, int rank, float scale)
{
    NNHIP_LANE(handle, NNHIP_OP_LORA)
    if (!z || !b || !y || rows < 1 || output < 1 || rank < 1)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_LORA, lane->device, 0, "pointers must be non-null and rows, output, rank positive");
    if (static_cast<int64_t>(rows) * output > 0x7fffffff)
        return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_LORA, lane->device, 0, "rows * output exceeds one launch");
    hipError_t e = launch_lora_b(lane, z, b, y, rows, output, rank, scale);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_LORA, lane->device, "adapter B launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

// The checks every entry point that takes a descriptor array makes; *entries receives the mat-vec rows of the batch.
static int check_batch(nnhip::Lane* lane, const nnhip_matvec_desc* descs, int count, long* entries)
{
    using namespace nnhip;
    if (count < 0 || (count > 0 && !descs))
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_MATVEC_BATCH, lane->device, 0, "descriptor array is null or count negative");
    long total = 0;
    for (int i = 0; i < count; ++i) {
        const nnhip_matvec_desc& d = descs[i];
        int rc = check_linear(NNHIP_OP_MATVEC_BATCH, lane, d.ggml_type, d.x, d.w, d.y, d.rows, d.in_w, d.out_w);
        if (rc != NNHIP_OK) return rc;
        if (d.in_w > matvec_max_in_w(d.ggml_type))
            return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_MATVEC_BATCH, lane->device, 0, "descriptor %d: in_w %d exceeds the %d values one workgroup can stage", i, d.in_w, matvec_max_in_w(d.ggml_type));
        if (d.rows > 65535)
            return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_MATVEC_BATCH, lane->device, 0, "descriptor %d: rows %d exceeds 65535", i, d.rows);
        total += d.rows;
    }
    if (total > NNHIP_BATCH_MAX_ENTRIES)
        return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_MATVEC_BATCH, lane->device, 0,
                    "the batch has %ld mat-vec rows; a call takes at most %d (split the batch)", total, NNHIP_BATCH_MAX_ENTRIES);
    *entries = total;
    return NNHIP_OK;
}

int nnhip_quant_matvec_batch(void* handle, const nnhip_matvec_desc* descs, int count)
{
    NNHIP_LANE(handle, NNHIP_OP_MATVEC_BATCH)
    long entries = 0;
    const int rc = check_batch(lane, descs, count, &entries);
    if (rc != NNHIP_OK) return rc;
    if (count == 0) return NNHIP_OK;
    hipError_t e = hipSuccess;
    try {
        e = launch_matvec_batch(lane, descs, count);
    } catch (const std::bad_alloc&) {       // (the host copy of the table)
        return fail(NNHIP_ERR_OUT_OF_MEMORY, NNHIP_OP_MATVEC_BATCH, lane->device, 0, "host memory for the descriptor table");
    }
    if (e == hipErrorStreamCaptureUnsupported)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_MATVEC_BATCH, lane->device, static_cast<uint32_t>(e),
                    "the batch needs a larger descriptor table than the lane holds, and a table cannot grow while a graph is "
                    "being captured: issue a batch of this size once before the capture");
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_MATVEC_BATCH, lane->device, "batched mat-vec launch");
    return NNHIP_OK;
}

int nnhip_matvec_batch_plan(const nnhip_matvec_desc* descs, int count, int compute_units, nnhip_batch_launch_info* launches,
                            int capacity, int* n_launches)
{
    if (count < 0 || (count > 0 && !descs) || capacity < 0 || (capacity > 0 && !launches) || !n_launches || compute_units < 1)
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_MATVEC_BATCH, -1, 0, "null array, negative count or capacity, or compute_units < 1");
    for (int i = 0; i < capacity; ++i)
        if (launches[i].struct_size != sizeof(nnhip_batch_launch_info))
            return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_MATVEC_BATCH, -1, 0, "launches[%d] has the wrong struct_size", i);
    Lane nowhere;
    nowhere.device = -1;
    long entries = 0;
    const int rc = check_batch(&nowhere, descs, count, &entries);
    if (rc != NNHIP_OK) return rc;
    int n = 0;
    try {
        n = plan_matvec_batch(descs, count, compute_units, launches, capacity);
    } catch (const std::bad_alloc&) {
        return fail(NNHIP_ERR_OUT_OF_MEMORY, NNHIP_OP_MATVEC_BATCH, -1, 0, "host memory for the descriptor table");
    }
    if (n < 0) return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_MATVEC_BATCH, -1, 0, "no kernel takes one of the shapes");
    *n_launches = n;
    return NNHIP_OK;
}

int nnhip_quant_matvec_batch_static(void* handle, const nnhip_matvec_desc* descs, int count)
{
    NNHIP_LANE(handle, NNHIP_OP_MATVEC_BATCH)
    long entries = 0;
    const int rc = check_batch(lane, descs, count, &entries);
    if (rc != NNHIP_OK) return rc;
    if (entries > NNHIP_STATIC_BATCH_MAX_ENTRIES)
        return fail(NNHIP_ERR_TOO_LARGE, NNHIP_OP_MATVEC_BATCH, lane->device, 0,
                    "the batch has %ld mat-vec rows; the fixed workspace holds %d (use nnhip_quant_matvec_batch, or split the batch)",
                    entries, NNHIP_STATIC_BATCH_MAX_ENTRIES);
    if (count == 0) return NNHIP_OK;
    hipError_t e = launch_matvec_batch_static(lane, descs, count);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_MATVEC_BATCH, lane->device, "batched mat-vec launch (fixed workspace)");
    return NNHIP_OK;
}

int nnhip_quant_matmul_bf16(void* handle, uint32_t ggml_type, const uint16_t* x_bf16, const void* w, const float* bias,
                            float* y, int rows, int in_w, int out_w)
{
    NNHIP_LANE(handle, NNHIP_OP_MATMUL_BF16)
    int rc = check_linear(NNHIP_OP_MATMUL_BF16, lane, ggml_type, x_bf16, w, y, rows, in_w, out_w);
    if (rc != NNHIP_OK) return rc;
    if (in_w % 256 != 0 && matmul_bf16_supported(ggml_type, 256))
        return fail(NNHIP_ERR_INCOMPLETE_BLOCKS, NNHIP_OP_MATMUL_BF16, lane->device, 0, "the bf16 prefill mat-mul needs in_w to be a multiple of 256 (got %d)", in_w);
    hipError_t e = launch_matmul_bf16(lane, ggml_type, x_bf16, w, bias, y, rows, in_w, out_w);
    if (e == hipErrorNotSupported)
        return fail(NNHIP_ERR_UNSUPPORTED_TYPE, NNHIP_OP_MATMUL_BF16, lane->device, 0, "bf16 prefill mat-mul does not support GGML type %u", ggml_type);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_MATMUL_BF16, lane->device, "mat-mul launch");
    lane->counters.kernel_launches += 1;
    return NNHIP_OK;
}

int nnhip_quant_matmul(void* handle, uint32_t ggml_type, const float* x, const void* w, const float* bias, float* y,
                       int rows, int in_w, int out_w)
{
    NNHIP_LANE(handle, NNHIP_OP_MATMUL)
    int rc = check_linear(NNHIP_OP_MATMUL, lane, ggml_type, x, w, y, rows, in_w, out_w);
    if (rc != NNHIP_OK) return rc;
    if (in_w % 256 != 0 && matmul_bf16_supported(ggml_type, 256))
        return fail(NNHIP_ERR_INCOMPLETE_BLOCKS, NNHIP_OP_MATMUL, lane->device, 0, "the prefill mat-mul needs in_w to be a multiple of 256 (got %d)", in_w);
    if (!matmul_bf16_supported(ggml_type, in_w))
        return fail(NNHIP_ERR_UNSUPPORTED_TYPE, NNHIP_OP_MATMUL, lane->device, 0, "the prefill mat-mul does not support GGML type %u", ggml_type);
    // the bfloat16 copy of the activations lives in a lane block for the duration of the two launches; freeing it hands
    // it to the next call of the same size without touching the driver
    const size_t count = static_cast<size_t>(rows) * static_cast<size_t>(in_w);
    void* staged = nullptr;
    rc = nnhip_alloc(handle, count * sizeof(uint16_t), &staged);
    if (rc != NNHIP_OK) return rc;
    hipError_t e = launch_to_bf16(lane, x, static_cast<uint16_t*>(staged), count);
    if (e == hipSuccess) e = launch_matmul_bf16(lane, ggml_type, static_cast<const uint16_t*>(staged), w, bias, y, rows, in_w, out_w);
    const int freed = nnhip_free(handle, staged);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_MATMUL, lane->device, "mat-mul launch");
    if (freed != NNHIP_OK) return freed;
    lane->counters.kernel_launches += 2;
    return NNHIP_OK;
}

int nnhip_quant_matmul_split(void* handle, uint32_t ggml_type, const float* x, const void* w, const float* bias, float* y,
                             int rows, int in_w, int out_w)
{
    NNHIP_LANE(handle, NNHIP_OP_MATMUL)
    int rc = check_linear(NNHIP_OP_MATMUL, lane, ggml_type, x, w, y, rows, in_w, out_w);
    if (rc != NNHIP_OK) return rc;
    if (in_w % 256 != 0 && matmul_bf16_supported(ggml_type, 256))
        return fail(NNHIP_ERR_INCOMPLETE_BLOCKS, NNHIP_OP_MATMUL, lane->device, 0, "the prefill mat-mul needs in_w to be a multiple of 256 (got %d)", in_w);
    if (!matmul_bf16_supported(ggml_type, in_w))
        return fail(NNHIP_ERR_UNSUPPORTED_TYPE, NNHIP_OP_MATMUL, lane->device, 0, "the prefill mat-mul does not support GGML type %u", ggml_type);
    // both bfloat16 parts of the activations share one lane block for the duration of the launches
    const size_t count = static_cast<size_t>(rows) * static_cast<size_t>(in_w);
    const size_t part_bytes = (count * sizeof(uint16_t) + 255u) & ~static_cast<size_t>(255u);
    void* staged = nullptr;
    rc = nnhip_alloc(handle, 2 * part_bytes, &staged);
    if (rc != NNHIP_OK) return rc;
    uint16_t* hi = static_cast<uint16_t*>(staged);
    uint16_t* lo = reinterpret_cast<uint16_t*>(static_cast<char*>(staged) + part_bytes);
    int launches = 0;
    hipError_t e = launch_to_bf16_parts(lane, x, hi, lo, count);
    if (e == hipSuccess) e = launch_matmul_parts(lane, ggml_type, hi, lo, w, bias, y, rows, in_w, out_w, &launches);
    const int freed = nnhip_free(handle, staged);
    lane->counters.kernel_launches += static_cast<uint64_t>(launches) + 1;
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_MATMUL, lane->device, "mat-mul launch");
    if (freed != NNHIP_OK) return freed;
    return NNHIP_OK;
}

int nnhip_event_create(void* handle, void** event)
{
    NNHIP_LANE(handle, NNHIP_OP_EVENT)
    if (!event) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_EVENT, lane->device, 0, "event output pointer is null");
    Event* ev = new (std::nothrow) Event();
    if (!ev) return fail(NNHIP_ERR_OUT_OF_MEMORY, NNHIP_OP_EVENT, lane->device, 0, "host allocation failed");
    hipError_t e = hipEventCreate(&ev->event);
    if (e != hipSuccess) {
        delete ev;
        return hip_fail(e, NNHIP_OP_EVENT, lane->device, "hipEventCreate");
    }
    *event = ev;
    return NNHIP_OK;
}

int nnhip_event_destroy(void* handle, void* event)
{
    NNHIP_LANE(handle, NNHIP_OP_EVENT)
    Event* ev = static_cast<Event*>(event);
    if (!ev || ev->magic != kEventMagic) return fail(NNHIP_ERR_BAD_HANDLE, NNHIP_OP_EVENT, lane->device, 0, "not an event handle");
    hipError_t e = hipEventDestroy(ev->event);
    ev->magic = 0;
    delete ev;
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_EVENT, lane->device, "hipEventDestroy");
    return NNHIP_OK;
}

int nnhip_event_record(void* handle, void* event)
{
    NNHIP_LANE(handle, NNHIP_OP_EVENT)
    Event* ev = static_cast<Event*>(event);
    if (!ev || ev->magic != kEventMagic) return fail(NNHIP_ERR_BAD_HANDLE, NNHIP_OP_EVENT, lane->device, 0, "not an event handle");
    hipError_t e = hipEventRecord(ev->event, lane->stream);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_EVENT, lane->device, "hipEventRecord");
    return NNHIP_OK;
}

int nnhip_event_elapsed_ms(void* handle, void* start, void* stop, float* ms)
{
    NNHIP_LANE(handle, NNHIP_OP_EVENT)
    Event* a = static_cast<Event*>(start);
    Event* b = static_cast<Event*>(stop);
    if (!a || !b || a->magic != kEventMagic || b->magic != kEventMagic || !ms)
        return fail(NNHIP_ERR_BAD_HANDLE, NNHIP_OP_EVENT, lane->device, 0, "not an event handle, or ms is null");
    hipError_t e = hipEventSynchronize(b->event);
    if (e == hipSuccess) e = hipEventElapsedTime(ms, a->event, b->event);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_EVENT, lane->device, "hipEventElapsedTime");
    return NNHIP_OK;
}

// Blocks that were pinned to a capture or a graph go back into circulation (or to the driver when the cache is full).
static void release_pinned(nnhip::Lane* lane, std::vector<std::pair<void*, size_t>>& blocks)
{
    std::lock_guard<std::mutex> guard(lane->mutex);
    for (const auto& b : blocks) {
        if (lane->cached_bytes + b.second <= nnhip::kCacheTotalMax) {
            lane->free_blocks[b.second].push_back(b.first);
            lane->cached_bytes += b.second;
        } else {
            (void)hipFree(b.first);
        }
    }
    blocks.clear();
}

int nnhip_graph_begin(void* handle)
{
    NNHIP_LANE(handle, NNHIP_OP_GRAPH)
    if (lane->capturing) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_GRAPH, lane->device, 0, "a capture is already in progress");
    hipError_t e = hipStreamBeginCapture(lane->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_GRAPH, lane->device, "hipStreamBeginCapture");
    lane->capturing = true;
    return NNHIP_OK;
}

int nnhip_graph_end(void* handle, void** graph)
{
    NNHIP_LANE(handle, NNHIP_OP_GRAPH)
    if (!lane->capturing) return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_GRAPH, lane->device, 0, "no capture in progress");
    lane->capturing = false;
    lane->batch_shadow.clear();
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(lane->stream, &g);
    if (e != hipSuccess) {
        release_pinned(lane, lane->capture_pinned);      // (nothing was recorded that could be replayed)
        return hip_fail(e, NNHIP_OP_GRAPH, lane->device, "hipStreamEndCapture");
    }
    if (!graph) {
        (void)hipGraphDestroy(g);
        release_pinned(lane, lane->capture_pinned);
        return fail(NNHIP_ERR_INVALID_ARGUMENT, NNHIP_OP_GRAPH, lane->device, 0, "graph output pointer is null");
    }
    Graph* gr = new (std::nothrow) Graph();
    if (!gr) {
        (void)hipGraphDestroy(g);
        release_pinned(lane, lane->capture_pinned);
        return fail(NNHIP_ERR_OUT_OF_MEMORY, NNHIP_OP_GRAPH, lane->device, 0, "host allocation failed");
    }
    gr->graph = g;
    e = hipGraphInstantiate(&gr->exec, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        delete gr;
        release_pinned(lane, lane->capture_pinned);
        return hip_fail(e, NNHIP_OP_GRAPH, lane->device, "hipGraphInstantiate");
    }
    // the blocks freed during the capture belong to the graph from here on
    gr->pinned.swap(lane->capture_pinned);
    lane->graphs.push_back(gr);
    *graph = gr;
    return NNHIP_OK;
}

int nnhip_graph_launch(void* handle, void* graph)
{
    NNHIP_LANE(handle, NNHIP_OP_GRAPH)
    Graph* gr = static_cast<Graph*>(graph);
    if (!gr || gr->magic != kGraphMagic) return fail(NNHIP_ERR_BAD_HANDLE, NNHIP_OP_GRAPH, lane->device, 0, "not a graph handle");
    hipError_t e = hipGraphLaunch(gr->exec, lane->stream);
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_GRAPH, lane->device, "hipGraphLaunch");
    lane->batch_shadow.clear();         // a replayed batch rewrites the lane's descriptor table
    return NNHIP_OK;
}

int nnhip_graph_destroy(void* handle, void* graph)
{
    NNHIP_LANE(handle, NNHIP_OP_GRAPH)
    Graph* gr = static_cast<Graph*>(graph);
    if (!gr || gr->magic != kGraphMagic) return fail(NNHIP_ERR_BAD_HANDLE, NNHIP_OP_GRAPH, lane->device, 0, "not a graph handle");
    hipError_t e = hipStreamSynchronize(lane->stream);
    hipError_t e2 = hipGraphExecDestroy(gr->exec);
    hipError_t e3 = hipGraphDestroy(gr->graph);
    release_pinned(lane, gr->pinned);
    for (size_t i = 0; i < lane->graphs.size(); ++i)
        if (lane->graphs[i] == gr) {
            lane->graphs.erase(lane->graphs.begin() + static_cast<long>(i));
            break;
        }
    gr->magic = 0;
    delete gr;
    if (e == hipSuccess) e = e2;
    if (e == hipSuccess) e = e3;
    if (e != hipSuccess) return hip_fail(e, NNHIP_OP_GRAPH, lane->device, "graph teardown");
    return NNHIP_OK;
}

}  // extern "C"
