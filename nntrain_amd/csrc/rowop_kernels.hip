// FP32 row operations that sit on either side of the quantized mat-vec in the decode path: RMSNorm, residual add +
// RMSNorm, SiLU(gate) * up, in-place add (NNtrain.Arc/Kernels/qwen35_attention.cl:9-78), and the two halves of a low-rank
// adapter (NNtrain.Arc/Kernels/qwen35_lora.cl:2-11,68-74).
//
// The reductions follow the reference's order, so a result has the bits of a plain CPU restatement: lane t of 128 adds
// x[t]^2, x[t+128]^2, ... in that order, the 128 partial sums meet in a halving tree (64, 32, .. 1), and
// inverse = 1 / sqrt(sum / width + eps) uses IEEE division and square root.  The build keeps multiply and add
// separate (-ffp-contract=off).
#include "nnhip_internal.h"
#include "quant_device.h"

namespace nnhip {

namespace {

constexpr int kNormLanes = 128;

// ADD: destination[row] += residual[row] first (and is stored), as q35a_add_rms_norm does.
template <bool ADD>
__global__ __launch_bounds__(kNormLanes) void rms_norm_kernel(float* io, const float* residual, const float* weight,
                                                              float* output, int width, int input_stride, float epsilon)
{
    __shared__ float sums[kNormLanes];
    const int tid = threadIdx.x;
    float* x = io + static_cast<size_t>(blockIdx.x) * input_stride;
    const float* res = ADD ? residual + static_cast<size_t>(blockIdx.x) * input_stride : nullptr;
    float* out = output + static_cast<size_t>(blockIdx.x) * width;
    float sum = 0.0f;
    // eight loads in flight per lane; the additions keep their order
    constexpr int kAhead = 8;
    int j = tid;
    for (; j + (kAhead - 1) * kNormLanes < width; j += kAhead * kNormLanes) {
        float v[kAhead], r[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            v[u] = x[j + u * kNormLanes];
            r[u] = ADD ? res[j + u * kNormLanes] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            if (ADD) {
                v[u] = v[u] + r[u];
                x[j + u * kNormLanes] = v[u];
            }
            sum += v[u] * v[u];
        }
    }
    for (; j < width; j += kNormLanes) {
        float v = x[j];
        if (ADD) {
            v = v + res[j];
            x[j] = v;
        }
        sum += v * v;
    }
    sums[tid] = sum;
    __syncthreads();
    for (int stride = kNormLanes / 2; stride > 0; stride >>= 1) {
        if (tid < stride) sums[tid] += sums[tid + stride];
        __syncthreads();
    }
    const float inverse = 1.0f / sqrtf(sums[0] / static_cast<float>(width) + epsilon);
    // every lane re-reads the components it wrote itself
#pragma unroll 8
    for (int k = tid; k < width; k += kNormLanes) out[k] = x[k] * inverse * weight[k];
}

// The same arithmetic for wide rows with 1024 lanes: the row (plus residual) is staged in LDS by all lanes at once, lanes
// 0-127 take the strided partial sums from LDS in the same order, and all lanes write the output.  One workgroup of
// 128 lanes spends its time waiting for forty dependent batches of loads; this form needs one.
constexpr int kWideLanes = 1024;
constexpr int kWideMaxWidth = 15360;          // floats staged in LDS (60 KB)

template <bool ADD>
__global__ __launch_bounds__(kWideLanes) void rms_norm_wide_kernel(float* io, const float* residual, const float* weight,
                                                                   float* output, int width, int input_stride, float epsilon)
{
    extern __shared__ float row[];
    __shared__ float sums[kNormLanes];
    const int tid = threadIdx.x;
    float* x = io + static_cast<size_t>(blockIdx.x) * input_stride;
    const float* res = ADD ? residual + static_cast<size_t>(blockIdx.x) * input_stride : nullptr;
    float* out = output + static_cast<size_t>(blockIdx.x) * width;
    for (int j = tid; j < width; j += kWideLanes) {
        float v = x[j];
        if (ADD) {
            v = v + res[j];
            x[j] = v;
        }
        row[j] = v;
    }
    __syncthreads();
    if (tid < kNormLanes) {
        float sum = 0.0f;
        for (int j = tid; j < width; j += kNormLanes) sum += row[j] * row[j];
        sums[tid] = sum;
    }
    __syncthreads();
    for (int stride = kNormLanes / 2; stride > 0; stride >>= 1) {
        if (tid < stride) sums[tid] += sums[tid + stride];
        __syncthreads();
    }
    const float inverse = 1.0f / sqrtf(sums[0] / static_cast<float>(width) + epsilon);
    for (int j = tid; j < width; j += kWideLanes) out[j] = row[j] * inverse * weight[j];
}

// Two-sided form: exp never sees a positive argument, so neither side overflows (qwen35_attention.cl:9-14).
__device__ __forceinline__ float stable_sigmoid(float x)
{
    if (x >= 0.0f) return 1.0f / (1.0f + expf(-x));
    const float e = expf(x);
    return e / (1.0f + e);
}

__global__ __launch_bounds__(256) void silu_multiply_kernel(const float* gate, const float* up, float* output, int length)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < length) {
        const float g = gate[i];
        output[i] = g * stable_sigmoid(g) * up[i];
    }
}

__global__ __launch_bounds__(256) void add_in_place_kernel(float* destination, const float* source, int length)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < length) destination[i] += source[i];
}

// z[t, r] = sum_j x[t, j] * a[r, j]: one workgroup per (t, r); 128 lane-strided fused multiply-add chains, then the
// halving tree (NNtrain.Arc/Kernels/qwen35_lora.cl:2-11).
__global__ __launch_bounds__(kNormLanes) void lora_a_kernel(const float* x, const float* a, float* z, int width, int rank)
{
    __shared__ float partial[kNormLanes];
    const int item = blockIdx.x, tid = threadIdx.x;
    const int t = item / rank, r = item - t * rank;
    const float* xr = x + static_cast<size_t>(t) * width;
    const float* ar = a + static_cast<size_t>(r) * width;
    float sum = 0.0f;
    for (int j = tid; j < width; j += kNormLanes) sum = fmaf(xr[j], ar[j], sum);
    partial[tid] = sum;
    __syncthreads();
    for (int s = kNormLanes / 2; s > 0; s >>= 1) {
        if (tid < s) partial[tid] += partial[tid + s];
        __syncthreads();
    }
    if (tid == 0) z[item] = partial[0];
}

// y[t, o] += scale * sum_r z[t, r] * b[o, r] (qwen35_lora.cl:68-74).
__global__ __launch_bounds__(256) void lora_b_kernel(const float* z, const float* b, float* y, int rows, int output, int rank,
                                                     float scale)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * output) return;
    const int t = i / output, o = i - t * output;
    float sum = 0.0f;
    for (int r = 0; r < rank; ++r) sum = fmaf(z[t * rank + r], b[static_cast<size_t>(o) * rank + r], sum);
    y[i] = y[i] + scale * sum;
}

// out[h, :] = v[h / (heads / kv_heads), :]: what causal grouped-query attention returns for the first token of a
// sequence (one key: the softmax weight is 1, whatever the query), so a decode loop can run without a cache.
__global__ __launch_bounds__(256) void first_token_attention_kernel(const float* v, float* out, int heads, int kv_heads, int head_width)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= heads * head_width) return;
    const int h = i / head_width, c = i - h * head_width;
    out[i] = v[(h / (heads / kv_heads)) * head_width + c];
}

}  // namespace

hipError_t launch_first_token_attention(Lane* lane, const float* v, float* out, int heads, int kv_heads, int head_width)
{
    hipLaunchKernelGGL(first_token_attention_kernel, dim3((heads * head_width + 255) / 256), dim3(256), 0, lane->stream, v, out,
                       heads, kv_heads, head_width);
    return hipGetLastError();
}

hipError_t launch_lora_a(Lane* lane, const float* x, const float* a, float* z, int rows, int width, int rank)
{
    hipLaunchKernelGGL(lora_a_kernel, dim3(rows * rank), dim3(kNormLanes), 0, lane->stream, x, a, z, width, rank);
    return hipGetLastError();
}

hipError_t launch_lora_b(Lane* lane, const float* z, const float* b, float* y, int rows, int output, int rank, float scale)
{
    hipLaunchKernelGGL(lora_b_kernel, dim3((rows * output + 255) / 256), dim3(256), 0, lane->stream, z, b, y, rows, output, rank, scale);
    return hipGetLastError();
}

hipError_t launch_rms_norm(Lane* lane, float* io, const float* residual, const float* weight, float* output, int rows,
                           int width, int input_stride, float epsilon)
{
    if (width >= 2 * kWideLanes && width <= kWideMaxWidth) {
        const size_t lds = static_cast<size_t>(width) * sizeof(float);
        static LdsLimit big_lds_add, big_lds_plain;
        hipError_t e = big_lds_add.ensure(lane->device, reinterpret_cast<const void*>(&rms_norm_wide_kernel<true>),
                                          static_cast<int>(kWideMaxWidth * sizeof(float)));
        if (e == hipSuccess)
            e = big_lds_plain.ensure(lane->device, reinterpret_cast<const void*>(&rms_norm_wide_kernel<false>),
                                     static_cast<int>(kWideMaxWidth * sizeof(float)));
        if (e != hipSuccess) return e;
        if (residual)
            hipLaunchKernelGGL(rms_norm_wide_kernel<true>, dim3(rows), dim3(kWideLanes), lds, lane->stream, io, residual, weight,
                               output, width, input_stride, epsilon);
        else
            hipLaunchKernelGGL(rms_norm_wide_kernel<false>, dim3(rows), dim3(kWideLanes), lds, lane->stream, io, residual, weight,
                               output, width, input_stride, epsilon);
        return hipGetLastError();
    }
    if (residual)
        hipLaunchKernelGGL(rms_norm_kernel<true>, dim3(rows), dim3(kNormLanes), 0, lane->stream, io, residual, weight, output,
                           width, input_stride, epsilon);
    else
        hipLaunchKernelGGL(rms_norm_kernel<false>, dim3(rows), dim3(kNormLanes), 0, lane->stream, io, residual, weight, output,
                           width, input_stride, epsilon);
    return hipGetLastError();
}

hipError_t launch_silu_multiply(Lane* lane, const float* gate, const float* up, float* output, int length)
{
    hipLaunchKernelGGL(silu_multiply_kernel, dim3((length + 255) / 256), dim3(256), 0, lane->stream, gate, up, output, length);
    return hipGetLastError();
}

hipError_t launch_add_in_place(Lane* lane, float* destination, const float* source, int length)
{
    hipLaunchKernelGGL(add_in_place_kernel, dim3((length + 255) / 256), dim3(256), 0, lane->stream, destination, source, length);
    return hipGetLastError();
}

}  // namespace nnhip
