// Internal declarations shared by the translation units of libnnhip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/nnhip.h"

namespace nnhip {

constexpr uint32_t kLaneMagic = 0x4e4c414eu;   // "NLAN"
constexpr uint32_t kEventMagic = 0x4e45564eu;  // "NEVN"
constexpr uint32_t kGraphMagic = 0x4e475248u;  // "NGRH"

constexpr size_t kCacheBlockMax = 64u << 20;   // larger blocks (weights) are returned to the driver when freed
constexpr size_t kCacheTotalMax = 1u << 30;    // most bytes a lane keeps for reuse
constexpr size_t kStagingBytes = 16u << 20;    // one pinned staging buffer of a file upload

struct Lane {
    uint32_t magic = kLaneMagic;
    int device = 0;
    int compute_units = 0;
    hipStream_t stream = nullptr;
    bool capturing = false;
    bool row_step_only = false;                 // NNHIP_OPTION_ROW_STEP_ONLY
    nnhip_lane_counters counters{};
    struct Block { size_t bytes, capacity; };   // bytes asked for; bytes the allocation really has
    std::unordered_map<void*, Block> buffers;   // device allocations handed out and still owned by the lane
    // Freed blocks wait here, by capacity, to be handed out again.  All work of a lane runs on one in-order stream, so
    // a block can be reused at once: whatever still reads it was enqueued before whatever the next owner enqueues.
    std::unordered_map<size_t, std::vector<void*>> free_blocks;
    size_t cached_bytes = 0;
    // Blocks freed while a graph is being captured: the recorded work names them, so they must not be handed out again
    // while that graph can still be replayed.  They pass to the graph when the capture ends and come back to free_blocks
    // when it is destroyed.
    std::vector<std::pair<void*, size_t>> capture_pinned;
    std::vector<struct Graph*> graphs;          // graphs captured on this lane and not destroyed yet
    std::mutex mutex;                           // guards buffers + counters (uploads may come from loader threads)
    void* batch_table = nullptr;                // device table of the batched mat-vec (written by a kernel on the stream)
    size_t batch_table_bytes = 0;               // its capacity
    std::vector<void*> retired_tables;          // outgrown tables: freed with the lane, a captured graph may name them
    std::vector<char> batch_shadow;             // the entries the device table holds now (empty: unknown)
    void* static_table = nullptr;               // this device's address of the library's fixed batch workspace
    // Two pinned host buffers (and an event each) through which nnhip_upload_from_file moves a file range: the next piece
    // is read while the last one travels.  Allocated by the first such upload, freed with the lane.
    void* staging[2] = {nullptr, nullptr};
    hipEvent_t staging_done[2] = {nullptr, nullptr};
};

struct Event {
    uint32_t magic = kEventMagic;
    hipEvent_t event = nullptr;
};

struct Graph {
    uint32_t magic = kGraphMagic;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<std::pair<void*, size_t>> pinned;      // lane blocks (pointer, capacity) the recorded work uses as scratch
};

// Raises the dynamic-LDS limit of one kernel, once per device (the attribute belongs to a function on a device).  Lanes
// of several threads may get here together: setting it twice is harmless, so a lock-free "done" bit per device is enough.
struct LdsLimit {
    std::atomic<uint64_t> done{0};
    hipError_t ensure(int device, const void* kernel, int bytes)
    {
        const uint64_t bit = 1ull << (device & 63);
        if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
        const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
        return e;
    }
};

// Block geometry; returns false for an unsupported type.
bool type_block(uint32_t type, int* elems, int* bytes);

// Failure bookkeeping (nnhip_api.hip).  fail() records and returns `status`.
int fail(int status, uint32_t op, int device, uint32_t hip_error, const char* fmt, ...);

// Kernel launchers.  Shapes are validated by the callers in nnhip_api.hip; these only pick launch geometry.
hipError_t launch_dequantize(Lane* lane, uint32_t type, const void* w, float* out, int64_t elements);
hipError_t launch_matvec(Lane* lane, uint32_t type, const float* x, const void* w, const float* bias, float* y,
                         int rows, int in_w, int out_w);
// Mat-vec with the activation preparation and the residual add fused in (descriptor checked by the caller).
bool matvec_fused_supported(uint32_t type, int in_w);
hipError_t launch_matvec_fused(Lane* lane, const nnhip_fused_matvec_desc& d);
hipError_t launch_matvec_batch(Lane* lane, const nnhip_matvec_desc* descs, int count);
// Matrix-core form of the mat-vec (gemv_mfma_kernels.hip): whether it takes a shape (and with which geometry), and its launch.
struct MfmaPlan {
    int waves, cols, kchunks, stages, stage_bytes, loads_per_wave, lds_bytes;
};
bool matvec_mfma_geometry(uint32_t type, int in_w, int out_w, const void* w, MfmaPlan* plan);
// One matrix (one input row of it) of a table-driven launch of the matrix-core mat-vec: all entries of a launch share
// the storage type and in_w.  80 bytes, the slot size of a lane's descriptor table.
struct MfmaTableEntry {
    const float* x;
    const uint8_t* w;
    const float* bias;
    float* y;
    int out_w;
    uint32_t w_bytes;       // whole matrix (< 2 GB)
    int tiles;              // ceil(out_w / 16)
    int first_tile;         // position of the matrix' first tile in the launch's tile sequence
    int rows;               // input rows that share the pass (wide form: 1 - 4; x, y advance by in_w, out_w per row)
    uint32_t pad_[7];
};
static_assert(sizeof(MfmaTableEntry) == 80, "table slots are 80 bytes");
MfmaTableEntry matvec_mfma_entry(uint32_t type, const float* x, const void* w, const float* bias, float* y, int in_w,
                                 int out_w, int first_tile);
// `runs`: workgroups take runs of consecutive tiles instead of every G-th tile (for tables whose activations change from
// entry to entry: a workgroup then converts two or three vectors instead of all of them; same bits per row).
hipError_t launch_matvec_mfma_table(Lane* lane, uint32_t type, int in_w, const MfmaTableEntry* device_entries, int entries,
                                    int total_tiles, bool runs);
// The wide form of the matrix-core mat-vec (activation planes in LDS): any in_w of at least four super-blocks, and
// entries of up to four input rows that share a pass over the weights (`inputs` = 1: every entry has one row).
// *split (optional) receives whether the launch would take the split form (planes of one group of block columns in LDS
// at a time: rows too long for `inputs` full sets of planes beside useful stage buffers).
bool matvec_mfma_wide_geometry(uint32_t type, int in_w, int out_w, const void* w, int inputs, bool* split = nullptr);
// Whether a single call with `rows` input rows is served by that form rather than by row-step passes: 0 (it is not), 4
// (up to four input rows share a pass over the weights) or 1 (a pass per input row, for rows whose four sets of planes do
// not fit LDS).
int matvec_rows_per_pass(uint32_t type, int rows, int in_w, int out_w, const void* w, int compute_units);
// That call: two or more input rows, `per_pass` of them per table entry and four entries per launch (the descriptors
// travel in the kernel arguments); *launches receives the number of launches made.
bool describe_matvec_rows_shared(uint32_t type, int rows, int in_w, int out_w, int per_pass, int compute_units,
                                 nnhip_matvec_plan_info* info);
hipError_t launch_matvec_rows_shared(Lane* lane, uint32_t type, const float* x, const void* w, const float* bias, float* y,
                                     int rows, int in_w, int out_w, int per_pass, int* launches);
hipError_t launch_matvec_mfma_wide_table(Lane* lane, uint32_t type, int in_w, int inputs, const MfmaTableEntry* device_entries,
                                         int entries, int total_tiles, bool runs);
// Geometry of one matrix-core launch of a batch (`form` 1: operand A in registers, 2: the wide form, 3: the wide form
// with shared passes), and the launches a whole batch splits into; no device needed.  plan_matvec_batch returns the
// number of launches, of which it describes the first `capacity`.
bool describe_matvec_mfma_launch(uint32_t type, int in_w, int form, bool runs, nnhip_batch_launch_info* info);
int plan_matvec_batch(const nnhip_matvec_desc* descs, int count, int compute_units, nnhip_batch_launch_info* launches,
                      int capacity);
// The fixed device workspace: its address on the current device, and the batched launch that uses it.
hipError_t static_table_address(void** address, unsigned serial);
hipError_t launch_matvec_batch_static(Lane* lane, const nnhip_matvec_desc* descs, int count);
hipError_t launch_matmul_bf16(Lane* lane, uint32_t type, const uint16_t* x, const void* w, const float* bias, float* y,
                              int rows, int in_w, int out_w, bool low_weight_part = false, bool accumulate = false);
// The three-product form: both operands as two bfloat16 parts each (see gemm_kernels.hip).
hipError_t launch_to_bf16_parts(Lane* lane, const float* x, uint16_t* hi, uint16_t* lo, size_t count);
hipError_t launch_matmul_parts(Lane* lane, uint32_t type, const uint16_t* x_hi, const uint16_t* x_lo, const void* w, const float* bias,
                               float* y, int rows, int in_w, int out_w, int* launches);
hipError_t launch_to_bf16(Lane* lane, const float* x, uint16_t* out, size_t count);
// FP32 row operations (rowop_kernels.hip).  residual == nullptr: plain RMSNorm of io (not modified).
hipError_t launch_rms_norm(Lane* lane, float* io, const float* residual, const float* weight, float* output, int rows,
                           int width, int input_stride, float epsilon);
hipError_t launch_silu_multiply(Lane* lane, const float* gate, const float* up, float* output, int length);
hipError_t launch_add_in_place(Lane* lane, float* destination, const float* source, int length);
hipError_t launch_first_token_attention(Lane* lane, const float* v, float* out, int heads, int kv_heads, int head_width);
hipError_t launch_lora_a(Lane* lane, const float* x, const float* a, float* z, int rows, int width, int rank);
hipError_t launch_lora_b(Lane* lane, const float* z, const float* b, float* y, int rows, int output, int rank, float scale);
// Storage types and widths the bf16 prefill mat-mul covers.
bool matmul_bf16_supported(uint32_t type, int in_w);
hipError_t launch_fill_u32(Lane* lane, uint32_t* p, uint32_t value, size_t count);

// Launch shape nnhip_quant_matvec would use (no device needed); false if no kernel takes the shape.
bool describe_matvec(uint32_t type, int rows, int in_w, int out_w, int compute_units, nnhip_matvec_plan_info* info);

// Largest in_w the mat-vec kernels can stage in LDS.
int matvec_max_in_w(uint32_t type);

}  // namespace nnhip
