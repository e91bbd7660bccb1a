/*
 * nnhip - C ABI of the MI355X (gfx950) GGUF block-quantized linear library, libnnhip.so.
 *
 * This is the native boundary that replaces, for the quantized-linear path only, what NNtrain's managed
 * operator objects reach through ArcExecutionLane + embedded OpenCL kernels.  Every entry point cites the
 * reference interface it stands in for (paths relative to the NNtrain tree).
 *
 * Conventions (taken from the reference's own native boundary, NNtrain.Cuda/Interop/CudaNativeGateway.cs):
 *   - extern "C", cdecl, default visibility; blittable arguments only (pointers, sizes, ints).
 *   - every entry returns int status, 0 = success (CudaNativeGateway.cs:275-283); details of the most recent
 *     failure are fetched with nnhip_last_error (CudaNativeGateway.cs:1360-1371 record layout).
 *   - packed ABI version (major << 16) | minor, major must match (CudaNativeGateway.cs:7-50).
 *   - device pointers, lanes, events and graphs are opaque handles (void*).
 *   - a lane owns one in-order HIP stream (ArcExecutionLane.cs:156); compute entries enqueue and return,
 *     only transfers and nnhip_synchronize block (ArcExecutionLane.cs:447-474,658).  Calls on one lane must be
 *     serialised by the caller (the managed lane takes lock(_sync), ArcExecutionLane.cs:28).
 *   - weights are raw GGUF blocks, uploaded unchanged; matrix row o is in_w/block_elems consecutive blocks
 *     (NNtrain.Arc/Kernels/qwen.cl:372-373).
 */
#ifndef NNHIP_H
#define NNHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(NNHIP_BUILD)
#define NNHIP_API __attribute__((visibility("default")))
#else
#define NNHIP_API
#endif

#define NNHIP_ABI_MAJOR 1u
#define NNHIP_ABI_MINOR 0u

/* GGML tensor type ids accepted as `ggml_type` (Qwen2Gguf.cs:8-12, Qwen35Gguf.cs:6-7, Gemma3LocalModel.cs:80). */
enum {
    NNHIP_TYPE_Q8_0 = 8,
    NNHIP_TYPE_Q4_K = 12,
    NNHIP_TYPE_Q5_K = 13,
    NNHIP_TYPE_Q6_K = 14,
    NNHIP_TYPE_IQ3_S = 21,
    NNHIP_TYPE_IQ2_S = 22,
    NNHIP_TYPE_BF16 = 30    /* unquantized bfloat16 matrix storage (Qwen35Gguf.cs:12-13); one 2-byte "block" per weight, the
                             * mat-vec needs rows of a multiple of 64 weights */
};

/* Status codes.  Positive values below 1000 are this library's own; HIP runtime errors are reported as
 * NNHIP_ERR_HIP with the hipError_t in nnhip_error_info.reserved. */
enum {
    NNHIP_OK = 0,
    NNHIP_ERR_INVALID_ARGUMENT = 1,   /* null pointer, non-positive width, rows < 1 ...                */
    NNHIP_ERR_UNSUPPORTED_TYPE = 2,   /* ggml_type is not one of the seven above                        */
    NNHIP_ERR_INCOMPLETE_BLOCKS = 3,  /* in_w (or elements) is not a whole number of blocks             */
    NNHIP_ERR_OUT_OF_MEMORY = 4,
    NNHIP_ERR_HIP = 5,                /* a HIP call failed                                               */
    NNHIP_ERR_NO_DEVICE = 6,
    NNHIP_ERR_BAD_HANDLE = 7,         /* lane / event / graph handle not created by this library        */
    NNHIP_ERR_TOO_LARGE = 8           /* a size exceeds what one launch or the fixed workspace can hold  */
};

/* Operation ids recorded with a failure (nnhip_error_info.operation). */
enum {
    NNHIP_OP_NONE = 0, NNHIP_OP_LANE_CREATE, NNHIP_OP_LANE_DESTROY, NNHIP_OP_ALLOC, NNHIP_OP_FREE,
    NNHIP_OP_UPLOAD, NNHIP_OP_DOWNLOAD, NNHIP_OP_COPY, NNHIP_OP_SYNCHRONIZE, NNHIP_OP_DEQUANTIZE,
    NNHIP_OP_MATVEC, NNHIP_OP_MATVEC_BATCH, NNHIP_OP_MATMUL_BF16, NNHIP_OP_EVENT, NNHIP_OP_GRAPH,
    NNHIP_OP_DEVICE_QUERY, NNHIP_OP_FILL, NNHIP_OP_RMS_NORM, NNHIP_OP_SILU_MULTIPLY, NNHIP_OP_ADD_IN_PLACE,
    NNHIP_OP_MATVEC_FUSED, NNHIP_OP_LORA, NNHIP_OP_ATTENTION, NNHIP_OP_MATMUL
};

/* Same field order as the reference's NativeErrorInfo (CudaNativeGateway.cs:1360-1371). */
typedef struct nnhip_error_info {
    uint32_t struct_size;
    uint32_t abi_version;
    uint64_t sequence;      /* increments with every recorded failure */
    int32_t status;
    int32_t device_index;
    uint32_t operation;
    uint32_t reserved;      /* hipError_t when status == NNHIP_ERR_HIP */
} nnhip_error_info;

/* Lane byte counters, the quantities ArcExecutionLane exposes (ArcExecutionLane.cs:71-91). */
typedef struct nnhip_lane_counters {
    uint32_t struct_size;
    uint32_t driver_allocations;   /* device and pinned-host allocations the library has asked the driver for on behalf of
                                    * the lane (buffers, descriptor tables, staging): a call that must not allocate leaves it alone */
    uint64_t h2d_bytes;
    uint64_t d2h_bytes;
    uint64_t allocated_bytes;
    uint64_t peak_allocated_bytes;
    uint64_t kernel_launches;
} nnhip_lane_counters;

/* One quantized mat-vec of a batch (nnhip_quant_matvec_batch).  Same meaning as the arguments of
 * nnhip_quant_matvec; 48 bytes, no padding. */
typedef struct nnhip_matvec_desc {
    const float* x;         /* device, f32 [rows, in_w]       */
    const void* w;          /* device, raw blocks             */
    const float* bias;      /* device, f32 [out_w], nullable  */
    float* y;               /* device, f32 [rows, out_w]      */
    uint32_t ggml_type;
    int32_t rows;
    int32_t in_w;
    int32_t out_w;
} nnhip_matvec_desc;

/* --- library ---------------------------------------------------------------------------------------------- */

/* Packed ABI version.  Replaces nntrain_abi_version (NNtrain.Cuda/native/cuda_runtime_bridge.cu:1436-1438). */
NNHIP_API uint32_t nnhip_abi_version(void);

/* Copies the most recent failure record; returns NNHIP_OK, or NNHIP_ERR_INVALID_ARGUMENT when out is null or
 * out_size < sizeof(nnhip_error_info).  Replaces nntrain_last_error (cuda_runtime_bridge.cu:1440-1481). */
NNHIP_API int nnhip_last_error(nnhip_error_info* out, size_t out_size);

/* Human-readable text of the most recent failure (NUL terminated, truncated to cap).  The managed side turns
 * it into the exception message, as OpenClNative.Check does (NNtrain.Arc/OpenClNative.cs:37-41). */
NNHIP_API int nnhip_last_error_message(char* buf, int cap);

/* Device enumeration.  Replaces ArcDevices.Enumerate (NNtrain.Arc/ArcDevices.cs:18). */
NNHIP_API int nnhip_device_count(int* count);
NNHIP_API int nnhip_device_name(int device, char* buf, int cap);
/* Compute units and bytes of device memory, for reporting. */
NNHIP_API int nnhip_device_info(int device, int* compute_units, uint64_t* total_memory_bytes);

/* Block geometry of a type: elements per block and bytes per block (Qwen35Gguf.cs:15-34). */
NNHIP_API int nnhip_type_block(uint32_t ggml_type, int* block_elems, int* block_bytes);
/* Payload bytes of an [out_w, in_w] matrix, with the same validation as ArcQuantizedMatrix's constructor
 * (NNtrain.Core/Serialization/ArcQuantizedMatrix.cs:20-32). */
NNHIP_API int nnhip_matrix_bytes(uint32_t ggml_type, int in_w, int out_w, uint64_t* bytes);

/* --- lane: one device, one in-order stream ------------------------------------------------------------------ */

/* Replaces ArcExecutionLane construction (ArcExecutionLane.cs:120-209) and Dispose (:872-915).
 * Destroy synchronises, then frees every buffer the lane still owns. */
NNHIP_API int nnhip_lane_create(int device, void** lane);
NNHIP_API int nnhip_lane_destroy(void* lane);

/* Replaces ArcExecutionLane.Allocate / AllocateBytes (:241,:271) and ArcBuffer.Dispose (:917-931).
 * Memory is not cleared.  nnhip_free does not wait for the device: blocks of up to 64 MiB (at most 1 GiB in all) are
 * kept by the lane and handed out again by the next nnhip_alloc of that size (rounded up to 256 bytes) - safe because
 * all work of a lane is ordered on its one stream - so the reference's pattern of allocating each projection's output
 * and disposing it after use (Qwen35QuantizedModel.cs:488-491) costs no synchronisation.  Larger blocks are returned
 * to the driver after the stream has drained.  While a graph is being captured nnhip_alloc can only hand out kept
 * blocks, and a block freed during the capture stays out of circulation until that graph is destroyed (the recorded
 * work names it; a replay must not write into memory that has a new owner).  nnhip_lane_trim drains the stream and returns every kept block to the driver; it has no counterpart in the
 * reference, whose OpenCL runtime defers releases itself. */
NNHIP_API int nnhip_alloc(void* lane, size_t bytes, void** dptr);
NNHIP_API int nnhip_free(void* lane, void* dptr);
NNHIP_API int nnhip_lane_trim(void* lane);

/* Blocking raw transfers.  Replace UploadRaw (:322-327) and Read / ReadRaw (:277,:334).  The bytes are not
 * interpreted: GGUF blocks go up exactly as they sit in the file. */
NNHIP_API int nnhip_upload(void* lane, void* dptr, size_t offset, const void* host, size_t bytes);
NNHIP_API int nnhip_download(void* lane, const void* dptr, size_t offset, void* host, size_t bytes);
/* nnhip_upload of `bytes` bytes that sit at `file_offset` of the open file `fd` (a POSIX descriptor; the file position
 * is not used or moved): the library reads the range piece by piece into two pinned buffers of its own and copies one
 * piece while it reads the next, so the caller holds no copy of the tensor and the copy does not wait for the read.
 * Replaces the pair GgufReader.ReadTensorBytes (GgufReader.cs:107-123) + UploadRaw that
 * Qwen35QuantizedModel.LoadTensor issues per tensor (Qwen35QuantizedModel.cs:234-243).  Blocking; a range that
 * reaches past the end of the file is NNHIP_ERR_INVALID_ARGUMENT (what arrived before it is counted in h2d_bytes).
 * One lane = one thread at a time, as for every call; lanes of several threads may read one descriptor. */
NNHIP_API int nnhip_upload_from_file(void* lane, void* dptr, size_t offset, int fd, uint64_t file_offset, size_t bytes);
/* Device-to-device copy on the lane's stream (asynchronous).  Replaces the lane's CopyBuffer used for KV
 * growth and staging (Qwen35QuantizedModel.cs:1037-1061). */
NNHIP_API int nnhip_copy(void* lane, void* dst, size_t dst_offset, const void* src, size_t src_offset, size_t bytes);
/* Fill `count` 32-bit words with `value` on the lane's stream (asynchronous); used for zero bias and NaN guards. */
NNHIP_API int nnhip_fill_u32(void* lane, void* dptr, size_t offset, uint32_t value, size_t count);

/* Replaces ArcExecutionLane.Synchronize (:658). */
NNHIP_API int nnhip_synchronize(void* lane);

/* Replaces the H2DBytes / D2HBytes / AllocatedBytes / PeakAllocatedBytes properties (:71-91). */
NNHIP_API int nnhip_lane_get_counters(void* lane, nnhip_lane_counters* out, size_t out_size);

/* The lane's hipStream_t, for callers that interoperate with other HIP code. */
NNHIP_API int nnhip_lane_stream(void* lane, void** stream);

/* Lane options (all 0 when a lane is created).
 * NNHIP_OPTION_ROW_STEP_ONLY = 1: nnhip_quant_matvec, nnhip_quant_matvec_batch and nnhip_quant_matvec_batch_static keep
 * every product on the FP32 row-step kernels, whatever the number of input rows or the size of the batch.  With it the
 * property the reference tests for its row-tiled kernels holds without exception: a call with rows > 1 equals stacked
 * rows == 1 calls bit for bit (Qwen35InferencePrefillLinearTests.cs:64-77), and a batch equals its single calls.  The
 * price is the shared matrix-core passes (a call with four input rows on 17408 x 5120 Q4_K: about twice the time).
 * Unknown options: NNHIP_ERR_INVALID_ARGUMENT. */
enum { NNHIP_OPTION_ROW_STEP_ONLY = 1 };
NNHIP_API int nnhip_lane_set_option(void* lane, uint32_t option, int64_t value);
NNHIP_API int nnhip_lane_get_option(void* lane, uint32_t option, int64_t* value);

/* --- compute ------------------------------------------------------------------------------------------------ */

/* out[i] = decoded weight i, FP32, bit-identical to the managed decoders GgufQ4K.Dequantize / GgufQ6K.Dequantize
 * (NNtrain.Core/Serialization/GgufQ4K.cs:9-60, GgufQ6K.cs:9-54) and to native ggml for Q5_K / IQ2_S / IQ3_S / Q8_0
 * (NNtrain.Arc/Kernels/qwen35_iq.cl:398-429).  Also the embedding-row lookup of
 * Matrix.Embedding (Qwen35QuantizedModel.cs:1497-1521) when w points at one row.  `elements` must be a whole
 * number of blocks.  Asynchronous. */
NNHIP_API int nnhip_dequantize(void* lane, uint32_t ggml_type, const void* w, float* out, int64_t elements);

/* y[r, o] = bias[o] + sum_k x[r, k] * w[o, k], FP32 accumulate, dequantization fused.  Argument order is the
 * kernel signature used throughout the reference, (x, weight, bias, y, rows, input_width, output_width)
 * (NNtrain.Arc/Kernels/qwen.cl:374-377; call site Qwen35QuantizedModel.cs:1355-1358).  Replaces the launch made
 * by Qwen35QuantizedModel.Matrix.Forward (Qwen35QuantizedModel.cs:1210-1369) and Tensor.ArcQwenQuantizedLinear
 * (NNtrain.Core/Tensors/Tensor.QwenQuantized.cs:29-96) for decode (rows == 1) and small row counts.  Each
 * output row of y is computed with the same operation order whatever `rows` is, so rows > 1 equals stacked
 * rows == 1 calls bit for bit (Qwen35InferencePrefillLinearTests.cs:64-77), except for calls with two or more input rows
 * on Q4_K / Q5_K / Q6_K / IQ2_S / IQ3_S matrices (three or more on Q8_0) with rows x ceil(out_w / 16) >= 2048, or >= 768
 * from three rows on (Q8_0: 2048): those take the matrix-core path described at nnhip_quant_matvec_batch (up to four
 * input rows per pass over the weights, sixteen per launch; a row's bits do not depend on the rows it travels with; 1e-6
 * from the rows == 1 result).  Rows too long for four sets of activation planes in LDS (in_w above about 8700; never
 * Q8_0) share passes in a split form, with the planes of one group of block columns in LDS at a time, where the groups
 * of four input rows make at least 3.5 rounds of 16-row tiles over the compute units (IQ2_S 2.5; IQ3_S always);
 * otherwise they get one matrix-core pass per input row, four rows a launch, from
 * rows x ceil(out_w / 16) >= 1024 on (IQ3_S 768, IQ2_S 512).  A row's bits depend on which of these forms the call
 * takes, not on the rows it travels with.  nnhip_matvec_plan reports which form a call takes; a lane with NNHIP_OPTION_ROW_STEP_ONLY set takes
 * none of these forms and keeps the bit-for-bit property for every call.  bias may be null (zero).  Asynchronous. */
NNHIP_API int nnhip_quant_matvec(void* lane, uint32_t ggml_type, const float* x, const void* w, const float* bias,
                                 float* y, int rows, int in_w, int out_w);

/* The launch shape nnhip_quant_matvec picks for a call, computed on the host without touching a device: for
 * reporting (the reference prints its kernel choice per matrix, Qwen35QuantizedModel.cs:1335-1344 selects by rows) and
 * for checking the kernels' capacity assumptions in tests.  compute_units is the workgroup count to plan for (256 on
 * MI355X).  The plan assumes a weight pointer on a 16-byte boundary, which every buffer from nnhip_alloc has: a call
 * whose w is less aligned (a view at an odd offset into a stacked payload) always takes the row-step kernels, also where
 * this reports NNHIP_MATVEC_KERNEL_MATRIX_CORE.  Returns NNHIP_ERR_TOO_LARGE when no kernel takes the shape.
 * struct_size = sizeof of the structure. */
enum { NNHIP_MATVEC_KERNEL_ROWSTEP = 0, NNHIP_MATVEC_KERNEL_Q8_0_ODD_BLOCKS = 1,
       NNHIP_MATVEC_KERNEL_MATRIX_CORE = 2 /* 16-row tiles over the workgroups, up to four input rows per pass */ };

typedef struct nnhip_matvec_plan_info {
    uint32_t struct_size;
    int32_t kernel;                 /* NNHIP_MATVEC_KERNEL_*                                                   */
    int32_t threads;                /* lanes per workgroup                                                     */
    int32_t rows_per_step;          /* whole matrix rows a workgroup reduces per step (matrix core: 16 per tile)  */
    int32_t steps;                  /* ceil(out_w / rows_per_step)                                             */
    int32_t groups;                 /* workgroups along the matrix                                             */
    int32_t row_tile;               /* input rows that share one pass over the weights                         */
    int32_t ring_depth;             /* steps whose results are parked in LDS before a flush is possible        */
    int32_t result_buffer_floats;   /* capacity of that LDS buffer: ring_depth * rows_per_step * row_tile fits */
    int32_t dynamic_lds_bytes;
} nnhip_matvec_plan_info;

NNHIP_API int nnhip_matvec_plan(uint32_t ggml_type, int rows, int in_w, int out_w, int compute_units,
                                nnhip_matvec_plan_info* info);

/* Most mat-vec rows (descriptors counted once per input row) one batched call takes: 80 MB of descriptor table. */
#define NNHIP_BATCH_MAX_ENTRIES (1 << 20)

/* `count` independent mat-vecs enqueued as one unit of work (a single launch per group of equal type), for the
 * per-token projection sets that ForwardTokenDevice issues back to back (Qwen35QuantizedModel.cs:451-513).
 * `descs` is a host array, read before the call returns.  Results are identical to `count` nnhip_quant_matvec calls,
 * with one exception: Q8_0, Q4_K, Q5_K, Q6_K, IQ2_S and IQ3_S matrices of one in_w (at least 1024, a multiple of 256; an
 * even number of 256-blocks for Q6_K, IQ2_S and IQ3_S) whose 16-row tiles, counted once per input row, add up to 2048 or more
 * within a call are multiplied on the matrix cores with the activations in 32-bit fixed point; descriptors with two or
 * more input rows (Q8_0: three or more) share one pass over the weights between up to four rows there.
 * Those results are deterministic,
 * depend on the weights, in_w and the activations of the row only (not on out_w, the other matrices or input rows of
 * the call, or the order), agree with the single launch to FP32 summation accuracy (relative L2 difference below 1e-6)
 * and are closer to the exact product than it.  The fixed point is relative to the largest magnitude of the input row,
 * v = rint(x * 2^e) with |v| <= 2^30, products and sums of v and the quants are exact integers, so
 *     |y[o] - exact[o]| <= 2^-31 * max_k |x[k]| * sum_k |w[o, k]|  +  the rounding of the FP32 accumulation;
 * for activations of ordinary dynamic range that is below one FP32 rounding per product.  An input row whose largest
 * magnitude exceeds its other values by a factor of 2^24 or more loses those other values' low bits (by 2^31 or more:
 * all of them), which FP32 arithmetic would keep in the rows whose weight at the large activation is zero; such rows
 * belong in nnhip_quant_matvec with rows == 1, which multiplies FP32 activations.  A NaN or an infinity in an input row
 * makes every output of that row NaN.
 * The descriptors reach the device as a table in lane-owned memory, written by a small kernel on the lane's stream
 * (skipped when the table already holds them), so the call never waits for the device.  Under graph capture the write
 * is recorded with the launch and a replay restores the table it needs; the table cannot grow during a capture
 * (NNHIP_ERR_INVALID_ARGUMENT: issue a batch at least as large once before capturing), and tables a graph may name are
 * kept until the lane is destroyed.  A descriptor takes at most 65535 input rows and a call at most
 * NNHIP_BATCH_MAX_ENTRIES rows in all (NNHIP_ERR_TOO_LARGE).  Asynchronous. */
NNHIP_API int nnhip_quant_matvec_batch(void* lane, const nnhip_matvec_desc* descs, int count);

/* The launches nnhip_quant_matvec_batch would split `count` descriptors into, without a device: one structure per launch,
 * in launch order.  No counterpart in the reference, which issues one kernel per matrix; it exists for reporting and so
 * that the grouping rules above (which matrices reach the matrix cores, which input rows share passes, how tiles are
 * dealt to the workgroups) can be checked in tests on a machine without a GPU.  The descriptors are checked as for the
 * batch itself; their pointers are inspected for alignment and equality only, never followed.  `launches` has room for
 * `capacity` structures, each with struct_size set; *n_launches receives the number of launches, which may exceed
 * `capacity` (then only the first `capacity` are described). */
typedef struct nnhip_batch_launch_info {
    uint32_t struct_size;
    uint32_t ggml_type;
    int32_t kernel;                 /* NNHIP_MATVEC_KERNEL_*                                                          */
    int32_t in_w;                   /* matrix core: the row length all entries share; row-step: the longest           */
    int32_t entries;                /* table entries: one per matrix and input row (or group of up to four rows)      */
    int32_t units;                  /* work items dealt to the workgroups: 16-row tiles, or chunks of row steps       */
    int32_t groups;                 /* workgroups: min(units, compute_units)                                          */
    int32_t threads;                /* lanes per workgroup                                                            */
    int32_t rows_per_pass;          /* most input rows of an entry that share a pass over the weights (1 - 4)         */
    int32_t consecutive_runs;       /* 1: a workgroup takes a run of consecutive tiles; 0: every groups-th tile       */
    int32_t stage_buffers;          /* matrix core: weight stages in LDS (1 = one buffer holding a whole tile)        */
    int32_t activations_in_lds;     /* matrix core: 1 = digit planes in LDS (the wide form), 0 = in registers         */
    int32_t dynamic_lds_bytes;
} nnhip_batch_launch_info;

NNHIP_API int nnhip_matvec_batch_plan(const nnhip_matvec_desc* descs, int count, int compute_units,
                                      nnhip_batch_launch_info* launches, int capacity, int* n_launches);

/* nnhip_quant_matvec_batch for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and bit-identical
 * results to nnhip_quant_matvec_batch; the descriptor table lives in a fixed array inside the library's device image (80 bytes per mat-vec row,
 * NNHIP_STATIC_BATCH_MAX_ENTRIES rows = 80 KiB per lane slice, held on every device the library is loaded on until the process ends)
 * instead of lane-owned memory, and the call makes no device or host allocation.  A batch with more rows (the sum of
 * `rows` over the descriptors) is rejected with NNHIP_ERR_TOO_LARGE.  The array has NNHIP_STATIC_BATCH_LANES slices of that
 * size (640 KiB in all); a lane takes one when it is created, in rotation per device, so up to that many lanes of a
 * device issue static batches (and replay graphs that contain them) independently of each other.  A call rewrites the
 * entries it uses; lanes that share a slice (the ninth lane of a device shares the first one's) must not have static
 * batches in flight at the same time.  Asynchronous. */
#define NNHIP_STATIC_BATCH_MAX_ENTRIES 1024
#define NNHIP_STATIC_BATCH_LANES 8
NNHIP_API int nnhip_quant_matvec_batch_static(void* lane, const nnhip_matvec_desc* descs, int count);

/* Prefill: y[r, o] = bias[o] + sum_k x[r, k] * w[o, k] with x given as bfloat16 bit patterns [rows, in_w];
 * weight tiles are dequantized to bfloat16 in LDS and contracted on MFMA with FP32 accumulators.  Replaces the
 * XMX prefill launch of Matrix.Forward for rows >= 16 (Qwen35QuantizedModel.cs:1249-1317, kernels
 * q35l_prefill_xmx_<format>_f16x2, NNtrain.Arc/Kernels/qwen35_prefill_xmx.cl:112-184).  Storage types Q4_K, Q5_K,
 * Q6_K, Q8_0, IQ2_S, IQ3_S and unquantized bfloat16 with in_w a multiple of 256 (NNHIP_ERR_INCOMPLETE_BLOCKS
 * otherwise).  Asynchronous. */
NNHIP_API int nnhip_quant_matmul_bf16(void* lane, uint32_t ggml_type, const uint16_t* x_bf16, const void* w,
                                      const float* bias, float* y, int rows, int in_w, int out_w);

/* Prefill with FP32 activations, the form Matrix.Forward takes them in: x [rows, in_w] is rounded to bfloat16 on the
 * device (round to nearest even) into a block owned by the lane, then multiplied as nnhip_quant_matmul_bf16 does.
 * Replaces the input conversion + XMX launch pair of Matrix.Forward for rows >= 16 (Qwen35QuantizedModel.cs:1249-1317:
 * q35l_prefill_xmx_input_f16x2 followed by q35l_prefill_xmx_<format>_f16x2, NNtrain.Arc/Kernels/
 * qwen35_prefill_xmx.cl:35-47,112-184).  The result equals nnhip_quant_matmul_bf16 on the rounded activations bit for
 * bit.  Same type and width rules.  The staging block comes from the lane's kept blocks when one of that size was
 * freed before (always, from the second call of a shape on; required while a graph is being captured).  Asynchronous. */
NNHIP_API int nnhip_quant_matmul(void* lane, uint32_t ggml_type, const float* x, const void* w, const float* bias,
                                 float* y, int rows, int in_w, int out_w);

/* Prefill at the accuracy the reference holds its XMX path to: that path splits the activations into a high and a low
 * half-precision part and multiplies both (q35l_prefill_xmx_input_f16x2 and the two-panel loop of
 * q35l_prefill_xmx_<format>_f16x2, NNtrain.Arc/Kernels/qwen35_prefill_xmx.cl:35-47,145-165), and is tested at relative
 * L2 < 5e-5 against the FP32 mat-vec (NNtrain.Core.Tests/Qwen35XmxPrefillLinearTests.cs:87-89).  Here both operands are
 * taken as hi + lo bfloat16 parts (hi = bf16(v), lo = bf16(v - hi): what is left is below 2^-17 of v) and three of the
 * four products are formed on the matrix cores with FP32 accumulation, x_hi w_hi + x_lo w_hi + x_hi w_lo (the fourth is
 * below 2^-16 of the first): three launches of the kernel of nnhip_quant_matmul_bf16 (two for unquantized bfloat16
 * weights, which have no low part), the second and third adding to y.  Relative L2 against the exact product: about
 * 3e-6.  Same type and width rules and the same staging-block behaviour as nnhip_quant_matmul (the block holds both
 * parts).  Asynchronous. */
NNHIP_API int nnhip_quant_matmul_split(void* lane, uint32_t ggml_type, const float* x, const void* w, const float* bias,
                                       float* y, int rows, int in_w, int out_w);

/* --- FP32 row operations around the mat-vec ------------------------------------------------------------------ */

/* output[r, j] = input[r * input_stride + j] * inverse_r * weight[j], inverse_r = 1 / sqrt(sum_j x^2 / width + epsilon),
 * for `rows` rows.  Replaces q35a_rms_norm (NNtrain.Arc/Kernels/qwen35_attention.cl:16-36; host wrapper
 * Qwen35Gpu.RmsNorm, NNtrain.Core/Modules/Qwen35Gpu.Attention.cs:11-36) with the same summation order (128
 * lane-strided partial sums, halving tree), so results have the bits of that kernel evaluated with IEEE arithmetic.
 * epsilon must be finite and >= 0 (ValidateAttentionEpsilon, Qwen35Gpu.Attention.cs:181-184).  Asynchronous. */
NNHIP_API int nnhip_rms_norm(void* lane, const float* input, const float* weight, float* output, int rows, int width,
                             int input_stride, float epsilon);

/* destination[r, j] += residual[r, j] (stored), then output = RMSNorm(destination) * weight as above.  Replaces
 * q35a_add_rms_norm (qwen35_attention.cl:55-78; call site AddResidualAndRmsNorm,
 * NNtrain.Core/Modules/Qwen35QuantizedModel.cs:527-546).  destination and residual rows are input_stride apart.
 * Asynchronous. */
NNHIP_API int nnhip_add_rms_norm(void* lane, float* destination, const float* residual, const float* weight,
                                 float* output, int rows, int width, int input_stride, float epsilon);

/* output[i] = gate[i] * sigmoid(gate[i]) * up[i] with the overflow-free two-sided sigmoid.  Replaces
 * q35a_silu_multiply (qwen35_attention.cl:9-14,38-43; Qwen35Gpu.SiluMultiply, Qwen35Gpu.Attention.cs:38-50).
 * Asynchronous. */
NNHIP_API int nnhip_silu_multiply(void* lane, const float* gate, const float* up, float* output, int length);

/* destination[i] += source[i].  Replaces q35a_add_in_place (qwen35_attention.cl:45-49; Qwen35Gpu.AddInPlace,
 * Qwen35Gpu.Attention.cs:52-58).  Asynchronous. */
NNHIP_API int nnhip_add_in_place(void* lane, float* destination, const float* source, int length);

/* One decode mat-vec with the row operations on either side of it fused into the launch, for the feed-forward half
 * of a layer as ForwardTokenDevice issues it (NNtrain.Core/Modules/Qwen35QuantizedModel.cs:482-498):
 *   pre_op NNHIP_PRE_RMS_NORM       v = RMSNorm(x + x2) * norm_weight   (x2 may be null: plain RMSNorm of x); replaces
 *                                   q35a_add_rms_norm / q35a_rms_norm followed by the projection; sum_out (may be null)
 *                                   receives x + x2, x_out (may be null) the normalized vector, bit-identical to
 *                                   nnhip_add_rms_norm / nnhip_rms_norm;
 *   pre_op NNHIP_PRE_SILU_MULTIPLY  v = x * sigmoid(x) * x2 (gate, up); replaces q35a_silu_multiply followed by the
 *                                   down projection; x_out (may be null) receives v;
 *   pre_op NNHIP_PRE_NONE           v = x;
 *   then  y[o] = addend[o] + ((bias[o] + sum_k v[k] * w[o, k]) + lora_scale * sum_r lora_z[r] * lora_b[o, r]);
 *   the low-rank term is the fused adapter branch of q35l_*_sg16_lora (NNtrain.Arc/Kernels/qwen35_linear_fast.cl:
 *   217-275; Matrix.ForwardFusedLora, Qwen35QuantizedModel.cs:1387) and is bit-identical to nnhip_lora_b applied to
 *   the plain result; addend may be null, and may be y itself (the residual stream: replaces q35a_add_in_place after
 *   the down projection).  bias may be null.
 *   x_head_width / x_head_group > 0 (with NNHIP_PRE_NONE): x holds in_w / x_head_group floats, kv heads of x_head_width
 *   values, and v[h * width + j] = x[(h / group) * width + j]: the launch reads the value heads as
 *   nnhip_first_token_attention would have copied them (replaces that launch in front of the o projection).
 *   post_op NNHIP_POST_SILU_PAIR (out_w even; no addend, no low-rank branch): w stacks two projections of out_w / 2 rows
 *   (gate | up) and y receives out_w / 2 values, y[o] = SiLU(z[o]) * z[out_w / 2 + o] with z = bias + W v and the SiLU of
 *   nnhip_silu_multiply: replaces the two projections and q35a_silu_multiply (Qwen35QuantizedModel.cs:489-496) with one
 *   launch, bit-identical to them.
 * The mat-vec part is bit-identical to nnhip_quant_matvec on the same v.  x, x2, norm_weight hold in_w floats;
 * x_out and sum_out must not overlap x or x2 (every workgroup reads those while workgroup 0 writes).  Q8_0 rows with
 * an odd number of blocks are not covered (NNHIP_ERR_INVALID_ARGUMENT).  struct_size = sizeof of this structure.
 * This fusion has no single counterpart in the reference, which launches the parts one by one.  Asynchronous. */
enum { NNHIP_PRE_NONE = 0, NNHIP_PRE_RMS_NORM = 1, NNHIP_PRE_SILU_MULTIPLY = 2 };
enum { NNHIP_POST_NONE = 0, NNHIP_POST_SILU_PAIR = 1 };

typedef struct nnhip_fused_matvec_desc {
    uint32_t struct_size;
    uint32_t ggml_type;
    uint32_t pre_op;
    float epsilon;              /* RMSNorm only: finite, >= 0 */
    const float* x;
    const float* x2;
    const float* norm_weight;   /* RMSNorm only */
    float* x_out;
    float* sum_out;             /* RMSNorm with x2 only */
    const void* w;
    const float* bias;
    const float* addend;
    float* y;
    int32_t in_w;
    int32_t out_w;
    const float* lora_z;        /* low-rank branch (null / 0 for none): lora_rank floats, z = A x of the adapter       */
    const float* lora_b;        /* [out_w, lora_rank] FP32                                                             */
    int32_t lora_rank;
    float lora_scale;
    int32_t x_head_width;       /* > 0: x is gathered by heads first, v[h * width + j] = x[(h / x_head_group) * width + j]   */
    int32_t x_head_group;       /* (x then holds in_w / x_head_group floats); both 0: x is used as it is                       */
    uint32_t post_op;           /* NNHIP_POST_SILU_PAIR: y[o] = SiLU(z[o]) * z[out_w / 2 + o] for o < out_w / 2, z = bias + W v */
    uint32_t reserved;          /* 0                                                                                           */
} nnhip_fused_matvec_desc;

NNHIP_API int nnhip_quant_matvec_fused(void* lane, const nnhip_fused_matvec_desc* desc);

/* out[h, :] = v[h / (heads / kv_heads), :] for h < heads: the result of causal grouped-query attention for the first
 * token of a sequence (a single key has softmax weight 1 whatever the query), which lets a decode loop exercise every
 * projection of a layer without a key/value cache (the attention core itself, Qwen35Gpu.AttentionStep,
 * NNtrain.Core/Modules/Qwen35Gpu.Attention.cs:60-120, is outside this library).  heads must be a multiple of kv_heads.
 * Asynchronous. */
NNHIP_API int nnhip_first_token_attention(void* lane, const float* v, float* out, int heads, int kv_heads, int head_width);

/* Low-rank adapter halves.  z[t, r] = sum_j x[t, j] * a[r, j] (q35l_lora_a_coop, NNtrain.Arc/Kernels/qwen35_lora.cl:
 * 2-11: 128 lane-strided fused multiply-add chains, halving tree) and y[t, o] += scale * sum_r z[t, r] * b[o, r]
 * (q35l_lora_b, qwen35_lora.cl:68-74).  Asynchronous. */
NNHIP_API int nnhip_lora_a(void* lane, const float* x, const float* a, float* z, int rows, int width, int rank);
NNHIP_API int nnhip_lora_b(void* lane, const float* z, const float* b, float* y, int rows, int output, int rank,
                           float scale);

/* --- timing and replay --------------------------------------------------------------------------------------- */

/* Device events on the lane's stream.  Replace the per-kernel OpenCL event timing of
 * ArcExecutionLane.RecordKernelTime (ArcExecutionLane.cs:727-742). */
NNHIP_API int nnhip_event_create(void* lane, void** event);
NNHIP_API int nnhip_event_destroy(void* lane, void* event);
NNHIP_API int nnhip_event_record(void* lane, void* event);
/* Blocks until `stop` has completed, then returns the milliseconds between the two events. */
NNHIP_API int nnhip_event_elapsed_ms(void* lane, void* start, void* stop, float* ms);

/* Capture the work enqueued on the lane between begin and end into a replayable HIP graph, for launch-bound
 * decode loops (the reference batches dispatches instead: ArcExecutionOptions.BatchDispatch,
 * ArcExecutionLane.cs:318,642).  No allocation, transfer or synchronise call is allowed while capturing. */
NNHIP_API int nnhip_graph_begin(void* lane);
NNHIP_API int nnhip_graph_end(void* lane, void** graph);
NNHIP_API int nnhip_graph_launch(void* lane, void* graph);
NNHIP_API int nnhip_graph_destroy(void* lane, void* graph);

#ifdef __cplusplus
}
#endif
#endif /* NNHIP_H */
