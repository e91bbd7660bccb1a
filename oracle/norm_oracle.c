/*
 * CPU oracle for the FP32 row operations that sit on either side of the quantized mat-vec in the decode path.
 * TEST INFRASTRUCTURE ONLY (see quant_oracle.c).  Plain C, every FP32 operation rounded separately
 * (-ffp-contract=off), IEEE square root and division.
 *
 *   rms_norm         NNtrain.Arc/Kernels/qwen35_attention.cl:16-36 (q35a_rms_norm): 128 lane-strided partial sums of
 *                    x*x, binary tree 64, 32 .. 1, inverse = 1 / sqrt(sum / width + eps), out = x * inverse * weight
 *   add_rms_norm     qwen35_attention.cl:55-78 (q35a_add_rms_norm): destination += residual, stored, then as above
 *   silu_multiply    qwen35_attention.cl:9-14,38-43: gate * sigmoid(gate) * up with the two-sided sigmoid
 *   add_in_place     qwen35_attention.cl:45-49
 *   rms_norm_serial  NNtrain.Core/Modules/Qwen35Math.cs:19-35 (the CPU statement: one running sum per row)
 *   lora_a           NNtrain.Arc/Kernels/qwen35_lora.cl:2-11 (q35l_lora_a_coop): z[t, r] = sum_j x[t, j] a[r, j] as 128
 *                    lane-strided fma chains and the halving tree
 *   lora_b           qwen35_lora.cl:68-74 (q35l_lora_b): y[t, o] += scale * (fma chain over r of z[t, r] b[o, r])
 *
 * Pinning (tests/test_oracle_norm.py): the reference's own vector Qwen35Math.RmsNorm([3,4,-3,-4],[2,.5],0,2) and the
 * zero row (Qwen35MathTests.cs:10-12), the sigmoid limits of Qwen35MathTests.cs:29-37, closed forms (constant rows,
 * powers of two), an independent pure-Python statement of the 128-lane tree on inputs whose sum depends on the order,
 * exact rational arithmetic (fractions) on small low-rank cases,
 * and float64 evaluation within 2e-5 (the reference's GPU-vs-CPU bound, Qwen35GpuAttentionTests.cs:26-28).
 */
#include <math.h>
#include <stdint.h>

#define ORACLE_EXPORT __attribute__((visibility("default")))

static float tree_sum_of_squares(const float* x, int width)
{
    float sums[128];
    for (int t = 0; t < 128; ++t) {
        float sum = 0.0f;
        for (int j = t; j < width; j += 128) sum += x[j] * x[j];
        sums[t] = sum;
    }
    for (int stride = 64; stride > 0; stride >>= 1)
        for (int t = 0; t < stride; ++t) sums[t] += sums[t + stride];
    return sums[0];
}

ORACLE_EXPORT void oracle_rms_norm(const float* input, const float* weight, float* output, int rows, int width,
                                   int input_stride, float epsilon)
{
    for (int r = 0; r < rows; ++r) {
        const float* x = input + (long)r * input_stride;
        const float inverse = 1.0f / sqrtf(tree_sum_of_squares(x, width) / (float)width + epsilon);
        for (int j = 0; j < width; ++j) output[(long)r * width + j] = x[j] * inverse * weight[j];
    }
}

ORACLE_EXPORT void oracle_add_rms_norm(float* destination, const float* residual, const float* weight, float* output,
                                       int rows, int width, int input_stride, float epsilon)
{
    for (int r = 0; r < rows; ++r) {
        float* x = destination + (long)r * input_stride;
        const float* res = residual + (long)r * input_stride;
        for (int j = 0; j < width; ++j) x[j] = x[j] + res[j];
        const float inverse = 1.0f / sqrtf(tree_sum_of_squares(x, width) / (float)width + epsilon);
        for (int j = 0; j < width; ++j) output[(long)r * width + j] = x[j] * inverse * weight[j];
    }
}

ORACLE_EXPORT void oracle_rms_norm_serial(const float* input, const float* weight, float* output, int rows, int width,
                                          float epsilon)
{
    for (int r = 0; r < rows; ++r) {
        const float* x = input + (long)r * width;
        float sum = 0.0f;
        for (int j = 0; j < width; ++j) sum += x[j] * x[j];
        const float inverse = 1.0f / sqrtf(sum / (float)width + epsilon);
        for (int j = 0; j < width; ++j) output[(long)r * width + j] = x[j] * inverse * weight[j];
    }
}

static float sigmoid(float x)
{
    if (x >= 0.0f) return 1.0f / (1.0f + expf(-x));
    const float e = expf(x);
    return e / (1.0f + e);
}

ORACLE_EXPORT void oracle_silu_multiply(const float* gate, const float* up, float* output, int length)
{
    for (int i = 0; i < length; ++i) output[i] = gate[i] * sigmoid(gate[i]) * up[i];
}

ORACLE_EXPORT void oracle_add_in_place(float* destination, const float* source, int length)
{
    for (int i = 0; i < length; ++i) destination[i] += source[i];
}

ORACLE_EXPORT void oracle_lora_a(const float* x, const float* a, float* z, int rows, int width, int rank)
{
    for (int t = 0; t < rows; ++t)
        for (int r = 0; r < rank; ++r) {
            float partial[128];
            for (int lane = 0; lane < 128; ++lane) {
                float sum = 0.0f;
                for (int j = lane; j < width; j += 128) sum = fmaf(x[(long)t * width + j], a[(long)r * width + j], sum);
                partial[lane] = sum;
            }
            for (int s = 64; s > 0; s >>= 1)
                for (int lane = 0; lane < s; ++lane) partial[lane] += partial[lane + s];
            z[t * rank + r] = partial[0];
        }
}

ORACLE_EXPORT void oracle_lora_b(const float* z, const float* b, float* y, int rows, int output, int rank, float scale)
{
    for (int t = 0; t < rows; ++t)
        for (int o = 0; o < output; ++o) {
            float sum = 0.0f;
            for (int r = 0; r < rank; ++r) sum = fmaf(z[t * rank + r], b[(long)o * rank + r], sum);
            y[(long)t * output + o] += scale * sum;
        }
}
