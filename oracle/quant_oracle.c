/*
 * CPU oracle for the GGUF block-quantized linear path.  TEST INFRASTRUCTURE ONLY: it is linked by tests/,
 * by __graft_entry__.smoke() and by bench.py's cpu_baseline leg, never by the HIP library or its host layer.
 *
 * Each function restates, in plain C with every FP32 operation rounded separately (build with
 * -ffp-contract=off), the algorithm of the reference file it cites (paths relative to the NNtrain tree):
 *
 *   Q4_K  dequantize   NNtrain.Core/Serialization/GgufQ4K.cs:9-60
 *   Q6_K  dequantize   NNtrain.Core/Serialization/GgufQ6K.cs:9-54
 *   Q5_K  dequantize   NNtrain.Arc/Kernels/qwen35_iq.cl:398-409  (native ggml dequantize_row_q5_K via fixture)
 *   IQ2_S dequantize   NNtrain.Arc/Kernels/qwen35_iq.cl:411-419, tools/iq2s-production-bench/ReferenceData.cs:33-51
 *   IQ3_S dequantize   NNtrain.Arc/Kernels/qwen35_iq.cl:421-429
 *   Q8_0  dequantize   w = d*q, NNtrain.Gemma/gemma-opencl/patches/ggml-opencl-q8-xmx-f16.patch:150
 *                      (block layout ...-gemv-rowtile-upload-candidate.patch:105-106)
 *   half -> float      NNtrain.Arc/Kernels/qwen35_linear_fast.cl:9-33 (IEEE exact, subnormals kept)
 *   cpu_linear         NNtrain.Core.Tests/QwenQuantizedLinearFastTests.cs:170-193 (sum = bias; sum = fma(x,w,sum))
 *   linear_f64         NNtrain.Core.Tests/Qwen35GpuLinearTests.cs:66-84, ReferenceData.cs:54-80 (double dot + abs sum)
 *
 * Pinning (what proves these restatements, all in tests/test_oracle_*.py):
 *   Q4_K, Q6_K : bit-exact on the gguf-py vectors of tests/golden/qwen_gguf_expected.json (4 x 3584 values,
 *                including all-subnormal scales) and the reference's single-weight known answers.
 *   Q5_K       : bit-exact on 25 native-ggml blocks of tests/golden/iq_quant_blocks.json + the 960.75 closed form.
 *   IQ2_S/IQ3_S: bit-exact on 69 / 45 native-ggml blocks covering every codebook index.
 *   Q8_0       : no reference vector exists; pinned by the closed form d*q against numpy
 *                (int8 view times float16->float32) and brute force.  The llama.cpp CPU Q8_0 mat-vec that
 *                gemma-gguf really executes (activation re-quantisation + integer dot, LLamaSharp 0.27.0 /
 *                llama.cpp 3f7c29d) is NOT restated here: parity unpinned for that third-party routine.
 *   linear     : float64 vectors of qwen_gguf_expected.json (rows 1/3/5, K=512, with bias), numpy float64 dot,
 *                pure-Python brute force on tiny shapes, linearity / row-independence invariants.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_EXPORT __attribute__((visibility("default")))

enum { T_Q8_0 = 8, T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14, T_IQ3_S = 21, T_IQ2_S = 22, T_BF16 = 30 };

#include "iq_grids.inc"
static const uint64_t iq2s_grid[1024] = { NNHIP_IQ2S_GRID_VALUES };
static const uint32_t iq3s_grid[512] = { NNHIP_IQ3S_GRID_VALUES };

ORACLE_EXPORT int oracle_block_elems(uint32_t type)
{
    switch (type) {
    case T_BF16: return 1;
    case T_Q8_0: return 32;
    case T_Q4_K: case T_Q5_K: case T_Q6_K: case T_IQ3_S: case T_IQ2_S: return 256;
    default: return 0;
    }
}

ORACLE_EXPORT int oracle_block_bytes(uint32_t type)
{
    switch (type) {
    case T_BF16: return 2;
    case T_Q8_0: return 34;
    case T_Q4_K: return 144;
    case T_Q5_K: return 176;
    case T_Q6_K: return 210;
    case T_IQ3_S: return 110;
    case T_IQ2_S: return 82;
    default: return 0;
    }
}

/* IEEE binary16 -> binary32 by bit manipulation: exact, subnormals and inf/NaN preserved. */
ORACLE_EXPORT float oracle_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int shift = 0;
            while ((man & 0x400u) == 0) { man <<= 1; ++shift; }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static float rd_half(const uint8_t* p) { return oracle_half_to_float((uint16_t)(p[0] | (p[1] << 8))); }

/* 6-bit scale/min pairs of Q4_K and Q5_K: GgufQ4K.cs:51-60. */
static void k4_scales(const uint8_t* packed, uint8_t* sc, uint8_t* mn)
{
    for (int j = 0; j < 4; ++j) {
        sc[j] = packed[j] & 0x3f;
        mn[j] = packed[j + 4] & 0x3f;
        sc[j + 4] = (uint8_t)((packed[j + 8] & 0x0f) | ((packed[j] >> 6) << 4));
        mn[j + 4] = (uint8_t)((packed[j + 8] >> 4) | ((packed[j + 4] >> 6) << 4));
    }
}

static void deq_q8_0(const uint8_t* b, float* out)
{
    float d = rd_half(b);
    for (int i = 0; i < 32; ++i) out[i] = d * (float)(int8_t)b[2 + i];
}

static void deq_q4_k(const uint8_t* b, float* out)
{
    float d = rd_half(b), dmin = rd_half(b + 2);
    uint8_t sc[8], mn[8];
    k4_scales(b + 4, sc, mn);
    const uint8_t* qs = b + 16;
    for (int g = 0; g < 8; ++g) {
        float scale = d * (float)sc[g];
        float min = dmin * (float)mn[g];
        const uint8_t* q = qs + (g / 2) * 32;
        for (int i = 0; i < 32; ++i) {
            int v = (g & 1) ? (q[i] >> 4) : (q[i] & 0x0f);
            float prod = scale * (float)v;
            out[g * 32 + i] = prod - min;
        }
    }
}

static void deq_q5_k(const uint8_t* b, float* out)
{
    float d = rd_half(b), dmin = rd_half(b + 2);
    uint8_t sc[8], mn[8];
    k4_scales(b + 4, sc, mn);
    const uint8_t* qh = b + 16;
    const uint8_t* ql = b + 48;
    for (int g = 0; g < 8; ++g) {
        float scale = d * (float)sc[g];
        float min = dmin * (float)mn[g];
        const uint8_t* q = ql + (g / 2) * 32;
        for (int i = 0; i < 32; ++i) {
            int nib = (g & 1) ? (q[i] >> 4) : (q[i] & 0x0f);
            int v = nib | (((qh[i] >> g) & 1) << 4);
            float prod = scale * (float)v;
            out[g * 32 + i] = prod - min;
        }
    }
}

static void deq_q6_k(const uint8_t* b, float* out)
{
    const uint8_t* ql = b;
    const uint8_t* qh = b + 128;
    const int8_t* scales = (const int8_t*)(b + 192);
    float d = rd_half(b + 208);
    for (int n = 0; n < 256; n += 128) {
        const uint8_t* l4 = ql + n / 2;
        const uint8_t* h2 = qh + n / 4;
        const int8_t* s = scales + n / 16;
        for (int l = 0; l < 32; ++l) {
            int is = l / 16;
            int q1 = ((l4[l] & 0x0f) | (((h2[l] >> 0) & 3) << 4)) - 32;
            int q2 = ((l4[l + 32] & 0x0f) | (((h2[l] >> 2) & 3) << 4)) - 32;
            int q3 = ((l4[l] >> 4) | (((h2[l] >> 4) & 3) << 4)) - 32;
            int q4 = ((l4[l + 32] >> 4) | (((h2[l] >> 6) & 3) << 4)) - 32;
            float s1 = d * (float)s[is], s2 = d * (float)s[is + 2];
            float s3 = d * (float)s[is + 4], s4 = d * (float)s[is + 6];
            out[n + l] = s1 * (float)q1;
            out[n + l + 32] = s2 * (float)q2;
            out[n + l + 64] = s3 * (float)q3;
            out[n + l + 96] = s4 * (float)q4;
        }
    }
}

static void deq_iq2_s(const uint8_t* b, float* out)
{
    float d = rd_half(b);
    for (int i = 0; i < 256; ++i) {
        int g = i >> 5, o = (i >> 3) & 3, t = i & 7;
        int idx = b[2 + g * 4 + o] | (((b[66 + g] >> (o * 2)) & 3) << 8);
        int mag = (int)((iq2s_grid[idx] >> (t * 8)) & 255u);
        int s = (b[74 + g] >> ((o >> 1) * 4)) & 15;
        int neg = (b[34 + g * 4 + o] >> t) & 1;
        float a = 0.5f + (float)s;
        float db = d * a;
        db = db * 0.25f;
        float v = db * (float)mag;
        out[i] = v * (neg ? -1.0f : 1.0f);
    }
}

static void deq_iq3_s(const uint8_t* b, float* out)
{
    float d = rd_half(b);
    for (int i = 0; i < 256; ++i) {
        int g = i >> 5, quartet = (i >> 2) & 7, t = i & 3;
        int idx = b[2 + g * 8 + quartet] | (((b[66 + g] >> quartet) & 1) << 8);
        int mag = (int)((iq3s_grid[idx] >> (t * 8)) & 255u);
        int s = (b[106 + (g >> 1)] >> ((g & 1) * 4)) & 15;
        int neg = (b[74 + (i >> 3)] >> (i & 7)) & 1;
        float db = d * (float)(1 + 2 * s);
        float v = db * (float)mag;
        out[i] = v * (neg ? -1.0f : 1.0f);
    }
}

static int deq_block(uint32_t type, const uint8_t* b, float* out)
{
    switch (type) {
    case T_BF16: {   /* bfloat16 is the upper half of a binary32 (Qwen2Gguf.cs:349-356) */
        uint32_t bits = ((uint32_t)b[0] | ((uint32_t)b[1] << 8)) << 16;
        memcpy(out, &bits, 4);
        return 0;
    }
    case T_Q8_0: deq_q8_0(b, out); return 0;
    case T_Q4_K: deq_q4_k(b, out); return 0;
    case T_Q5_K: deq_q5_k(b, out); return 0;
    case T_Q6_K: deq_q6_k(b, out); return 0;
    case T_IQ2_S: deq_iq2_s(b, out); return 0;
    case T_IQ3_S: deq_iq3_s(b, out); return 0;
    default: return -1;
    }
}

/* Dequantize `elements` weights (a whole number of blocks). Returns 0, or -1 on bad type / count. */
ORACLE_EXPORT int oracle_dequantize(uint32_t type, const uint8_t* src, float* out, int64_t elements)
{
    int elems = oracle_block_elems(type), bytes = oracle_block_bytes(type);
    if (elems == 0 || elements < 0 || elements % elems != 0) return -1;
    int64_t blocks = elements / elems;
    for (int64_t i = 0; i < blocks; ++i)
        deq_block(type, src + i * bytes, out + i * elems);
    return 0;
}

static int check_shape(uint32_t type, int rows, int in_w, int out_w)
{
    int elems = oracle_block_elems(type);
    if (elems == 0 || rows <= 0 || in_w <= 0 || out_w <= 0 || in_w % elems != 0) return -1;
    return 0;
}

/*
 * The reference's CPU statement of the operator: per output row, dequantize the row, then
 * sum = bias[o]; for k: sum = fmaf(x[r,k], w[k], sum)  (FP32, sequential).  bias may be NULL (zero).
 * threads <= 0 means all OpenMP threads.  Weight row o is in_w/elems consecutive blocks.
 */
ORACLE_EXPORT int oracle_cpu_linear(uint32_t type, const uint8_t* w, const float* x, const float* bias,
                                    float* y, int rows, int in_w, int out_w, int threads)
{
    if (check_shape(type, rows, in_w, out_w)) return -1;
    int elems = oracle_block_elems(type), bytes = oracle_block_bytes(type);
    int64_t row_bytes = (int64_t)(in_w / elems) * bytes;
    int failed = 0;
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
#pragma omp parallel num_threads(threads)
#endif
    {
        float* wrow = (float*)malloc(sizeof(float) * (size_t)in_w);
        if (!wrow) {
            failed = 1;
        } else {
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
            for (int o = 0; o < out_w; ++o) {
                const uint8_t* src = w + (int64_t)o * row_bytes;
                for (int b = 0; b < in_w / elems; ++b) deq_block(type, src + (int64_t)b * bytes, wrow + b * elems);
                for (int r = 0; r < rows; ++r) {
                    const float* xr = x + (int64_t)r * in_w;
                    float sum = bias ? bias[o] : 0.0f;
                    for (int k = 0; k < in_w; ++k) sum = fmaf(xr[k], wrow[k], sum);
                    y[(int64_t)r * out_w + o] = sum;
                }
            }
            free(wrow);
        }
    }
    return failed ? -2 : 0;
}

/*
 * Float64 reference: y = bias + sum_k (double)x*(double)w over FP32-decoded weights, plus the sum of
 * absolute terms (including |bias|) used by the reference's abs-sum tolerance.  abs_sum may be NULL.
 * x_is_bf16 != 0: x points at uint16 bfloat16 bit patterns, widened exactly.
 */
ORACLE_EXPORT int oracle_linear_f64(uint32_t type, const uint8_t* w, const void* x, int x_is_bf16,
                                    const float* bias, double* y, double* abs_sum,
                                    int rows, int in_w, int out_w, int threads)
{
    if (check_shape(type, rows, in_w, out_w)) return -1;
    int elems = oracle_block_elems(type), bytes = oracle_block_bytes(type);
    int64_t row_bytes = (int64_t)(in_w / elems) * bytes;
    int failed = 0;
    float* xf = NULL;
    const float* xs = (const float*)x;
    if (x_is_bf16) {
        int64_t n = (int64_t)rows * in_w;
        xf = (float*)malloc(sizeof(float) * (size_t)n);
        if (!xf) return -2;
        const uint16_t* xb = (const uint16_t*)x;
        for (int64_t i = 0; i < n; ++i) {
            uint32_t bits = (uint32_t)xb[i] << 16;
            memcpy(&xf[i], &bits, 4);
        }
        xs = xf;
    }
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_max_threads();
#pragma omp parallel num_threads(threads)
#endif
    {
        float* wrow = (float*)malloc(sizeof(float) * (size_t)in_w);
        if (!wrow) {
            failed = 1;
        } else {
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
            for (int o = 0; o < out_w; ++o) {
                const uint8_t* src = w + (int64_t)o * row_bytes;
                for (int b = 0; b < in_w / elems; ++b) deq_block(type, src + (int64_t)b * bytes, wrow + b * elems);
                for (int r = 0; r < rows; ++r) {
                    const float* xr = xs + (int64_t)r * in_w;
                    double sum = bias ? (double)bias[o] : 0.0;
                    double asum = fabs(sum);
                    for (int k = 0; k < in_w; ++k) {
                        double term = (double)xr[k] * (double)wrow[k];
                        sum += term;
                        asum += fabs(term);
                    }
                    y[(int64_t)r * out_w + o] = sum;
                    if (abs_sum) abs_sum[(int64_t)r * out_w + o] = asum;
                }
            }
            free(wrow);
        }
    }
    free(xf);
    return failed ? -2 : 0;
}

ORACLE_EXPORT int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
