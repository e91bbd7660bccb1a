// Internal declarations shared by the translation units of libnnhip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <unordered_map>

#include "../../include/nnhip.h"

namespace nnhip {

constexpr uint32_t kLaneMagic = 0x4e4c414eu;   // "NLAN"
constexpr uint32_t kEventMagic = 0x4e45564eu;  // "NEVN"
constexpr uint32_t kGraphMagic = 0x4e475248u;  // "NGRH"

struct Lane {
    uint32_t magic = kLaneMagic;
    int device = 0;
    int compute_units = 0;
    hipStream_t stream = nullptr;
    bool capturing = false;
    nnhip_lane_counters counters{};
    std::unordered_map<void*, size_t> buffers;  // device allocations still owned by the lane
    std::mutex mutex;                           // guards buffers + counters (uploads may come from loader threads)
    void* batch_table = nullptr;                // device copy of the descriptor table of the last batch launch
    size_t batch_table_bytes = 0;               // capacity of both copies
    size_t batch_table_used = 0;                // bytes of the table that is on the device now
    void* batch_table_host = nullptr;           // pinned staging for the table
};

struct Event {
    uint32_t magic = kEventMagic;
    hipEvent_t event = nullptr;
};

struct Graph {
    uint32_t magic = kGraphMagic;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
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
hipError_t launch_matmul_bf16(Lane* lane, uint32_t type, const uint16_t* x, const void* w, const float* bias,
                              float* y, int rows, int in_w, int out_w);
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

// Largest in_w the mat-vec kernels can stage in LDS.
int matvec_max_in_w(uint32_t type);

}  // namespace nnhip
