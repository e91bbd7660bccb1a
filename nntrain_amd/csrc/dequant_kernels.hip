// Block dequantizers: raw GGUF blocks -> FP32, bit-identical to the CPU decoders of the reference.
//
// Every product and difference is rounded to FP32 on its own (__fmul_rn / __fsub_rn, never fused), in the order the
// managed decoders use: Q4_K/Q5_K (d*sc)*q - (dmin*m)   (NNtrain.Core/Serialization/GgufQ4K.cs:34-41),
// Q6_K (d*scale)*q (GgufQ6K.cs:45-48), IQ2_S ((d*(0.5+s))*0.25)*mag*sign (NNtrain.Arc/Kernels/qwen35_iq.cl:411-419),
// IQ3_S (d*(1+2s))*mag*sign (qwen35_iq.cl:421-429), Q8_0 d*q.  One thread decodes four consecutive weights and stores one float4.
#include "nnhip_internal.h"
#include "quant_device.h"

#include "iq_grids.inc"

namespace nnhip {

namespace {

__device__ const uint64_t g_iq2s_grid_dq[1024] = { NNHIP_IQ2S_GRID_VALUES };
__device__ const uint32_t g_iq3s_grid_dq[512] = { NNHIP_IQ3S_GRID_VALUES };

__device__ __forceinline__ void k4_scale_min(const uint8_t* packed, int g, uint32_t& sc, uint32_t& mn)
{
    if (g < 4) {
        sc = packed[g] & 63u;
        mn = packed[g + 4] & 63u;
    } else {
        sc = (packed[g + 4] & 15u) | ((packed[g - 4] >> 6) << 4);
        mn = (packed[g + 4] >> 4) | ((packed[g] >> 6) << 4);
    }
}

__device__ __forceinline__ float4 deq4_q8_0(const uint8_t* w, int64_t e)
{
    const uint8_t* p = w + (e >> 5) * 34;
    const int i = static_cast<int>(e & 31);
    const float d = half_bits_to_float(ld16(p));
    const uint32_t q = ld32(p + 2 + i);
    return make_float4(__fmul_rn(d, sbyte0(q)), __fmul_rn(d, sbyte1(q)), __fmul_rn(d, sbyte2(q)), __fmul_rn(d, sbyte3(q)));
}

template <bool FIVE>
__device__ __forceinline__ float4 deq4_q45_k(const uint8_t* w, int64_t e)
{
    const uint8_t* p = w + (e >> 8) * (FIVE ? 176 : 144);
    const int i = static_cast<int>(e & 255), g = i >> 5, j = i & 31;
    // d, dmin and the twelve bytes of 6-bit scales and minima in one load (blocks are 16-byte aligned); the eight groups
    // of a block lie in one wave, so the bytes are picked with selects rather than with branches and byte loads
    const u32x4 h = *reinterpret_cast<const u32x4*>(p);
    const float d = half_bits_to_float(h[0]), dmin = half_bits_to_float(h[0] >> 16);
    auto packed = [&](int k) {                       // byte k of the twelve
        const uint32_t word = k < 4 ? h[1] : (k < 8 ? h[2] : h[3]);
        return (word >> (8 * (k & 3))) & 0xffu;
    };
    const uint32_t a = packed(g & 3), b = packed((g & 3) + 4), c = packed((g & 3) + 8);
    const uint32_t sc = g < 4 ? a & 63u : (c & 15u) | ((a >> 6) << 4);
    const uint32_t mn = g < 4 ? b & 63u : (c >> 4) | ((b >> 6) << 4);
    uint32_t q = *reinterpret_cast<const uint32_t*>(p + (FIVE ? 48 : 16) + (g >> 1) * 32 + j);
    q = (g & 1) ? (q >> 4) & 0x0f0f0f0fu : q & 0x0f0f0f0fu;
    if (FIVE) {
        const uint32_t hb = *reinterpret_cast<const uint32_t*>(p + 16 + j);
        q |= ((hb >> g) & 0x01010101u) << 4;
    }
    const float scale = __fmul_rn(d, static_cast<float>(sc));
    const float min = __fmul_rn(dmin, static_cast<float>(mn));
    return make_float4(__fsub_rn(__fmul_rn(scale, ubyte0(q)), min), __fsub_rn(__fmul_rn(scale, ubyte1(q)), min),
                       __fsub_rn(__fmul_rn(scale, ubyte2(q)), min), __fsub_rn(__fmul_rn(scale, ubyte3(q)), min));
}

__device__ __forceinline__ float4 deq4_q6_k(const uint8_t* w, int64_t e)
{
    const uint8_t* p = w + (e >> 8) * 210;
    const int i = static_cast<int>(e & 255), h = i >> 7, r = i & 127, run = r >> 5, l = r & 31;
    const float d = half_bits_to_float(ld16(p + 208));
    uint32_t lo = ld32(p + 64 * h + (run & 1) * 32 + l);
    lo = (run & 2) ? (lo >> 4) & 0x0f0f0f0fu : lo & 0x0f0f0f0fu;
    const uint32_t hi = (ld32(p + 128 + 32 * h + l) >> (2 * run)) & 0x03030303u;
    const uint32_t q = lo | (hi << 4);
    const float scale = __fmul_rn(d, static_cast<float>(static_cast<int8_t>(p[192 + 8 * h + 2 * run + (l >> 4)])));
    return make_float4(__fmul_rn(scale, static_cast<float>(static_cast<int>(q & 0xffu) - 32)),
                       __fmul_rn(scale, static_cast<float>(static_cast<int>((q >> 8) & 0xffu) - 32)),
                       __fmul_rn(scale, static_cast<float>(static_cast<int>((q >> 16) & 0xffu) - 32)),
                       __fmul_rn(scale, static_cast<float>(static_cast<int>(q >> 24) - 32)));
}

__device__ __forceinline__ float4 deq4_iq2_s(const uint8_t* w, int64_t e)
{
    const uint8_t* p = w + (e >> 8) * 82;
    const int i = static_cast<int>(e & 255), g = i >> 5, o = (i >> 3) & 3, t0 = i & 7;  // t0 is 0 or 4
    const float d = half_bits_to_float(ld16(p));
    const uint32_t idx = p[2 + 4 * g + o] | (((p[66 + g] >> (2 * o)) & 3u) << 8);
    const uint32_t mags = static_cast<uint32_t>(g_iq2s_grid_dq[idx] >> (8 * t0));
    const uint32_t signs = p[34 + 4 * g + o] >> t0;
    const float sub = static_cast<float>((p[74 + g] >> (4 * (o >> 1))) & 15u);
    const float db = __fmul_rn(__fmul_rn(d, __fadd_rn(0.5f, sub)), 0.25f);
    float4 v = make_float4(__fmul_rn(db, ubyte0(mags)), __fmul_rn(db, ubyte1(mags)), __fmul_rn(db, ubyte2(mags)),
                           __fmul_rn(db, ubyte3(mags)));
    v.x = __fmul_rn(v.x, (signs & 1u) ? -1.0f : 1.0f);
    v.y = __fmul_rn(v.y, (signs & 2u) ? -1.0f : 1.0f);
    v.z = __fmul_rn(v.z, (signs & 4u) ? -1.0f : 1.0f);
    v.w = __fmul_rn(v.w, (signs & 8u) ? -1.0f : 1.0f);
    return v;
}

// IQ3_S: d @0, qs[64] @2 (low 8 index bits, one per four weights), qh[8] @66 (ninth index bit), signs[32] @74 (one bit
// per weight), scales[4] @106 (a nibble per 32 weights); the four weights of a quartet are the bytes of the 32-bit
// codebook entry.
__device__ __forceinline__ float4 deq4_iq3_s(const uint8_t* w, int64_t e)
{
    const uint8_t* p = w + (e >> 8) * 110;
    const int i = static_cast<int>(e & 255), g = i >> 5, quartet = (i >> 2) & 7;
    const float d = half_bits_to_float(ld16(p));
    const uint32_t idx = p[2 + 8 * g + quartet] | (((p[66 + g] >> quartet) & 1u) << 8);
    const uint32_t mags = g_iq3s_grid_dq[idx];
    const uint32_t signs = p[74 + (i >> 3)] >> (i & 7);          // i & 7 is 0 or 4
    const uint32_t sub = (p[106 + (g >> 1)] >> (4 * (g & 1))) & 15u;
    const float db = __fmul_rn(d, static_cast<float>(1u + 2u * sub));
    float4 v = make_float4(__fmul_rn(db, ubyte0(mags)), __fmul_rn(db, ubyte1(mags)), __fmul_rn(db, ubyte2(mags)),
                           __fmul_rn(db, ubyte3(mags)));
    v.x = __fmul_rn(v.x, (signs & 1u) ? -1.0f : 1.0f);
    v.y = __fmul_rn(v.y, (signs & 2u) ? -1.0f : 1.0f);
    v.z = __fmul_rn(v.z, (signs & 4u) ? -1.0f : 1.0f);
    v.w = __fmul_rn(v.w, (signs & 8u) ? -1.0f : 1.0f);
    return v;
}

__device__ __forceinline__ float4 deq4_bf16(const uint8_t* w, int64_t e)
{
    const u32x2 v = ld64(w + 2 * e);        // four bfloat16: each is the upper half of its FP32 value
    return make_float4(__uint_as_float(v[0] << 16), __uint_as_float(v[0] & 0xffff0000u), __uint_as_float(v[1] << 16),
                       __uint_as_float(v[1] & 0xffff0000u));
}

template <uint32_t TYPE>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ w, float4* __restrict__ out,
                                                         int64_t quads)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < quads; t += stride) {
        const int64_t e = t * 4;
        float4 v;
        if (TYPE == NNHIP_TYPE_Q8_0) v = deq4_q8_0(w, e);
        else if (TYPE == NNHIP_TYPE_Q4_K) v = deq4_q45_k<false>(w, e);
        else if (TYPE == NNHIP_TYPE_Q5_K) v = deq4_q45_k<true>(w, e);
        else if (TYPE == NNHIP_TYPE_Q6_K) v = deq4_q6_k(w, e);
        else if (TYPE == NNHIP_TYPE_IQ3_S) v = deq4_iq3_s(w, e);
        else if (TYPE == NNHIP_TYPE_BF16) v = deq4_bf16(w, e);
        else v = deq4_iq2_s(w, e);
        // (a stream of writes that nothing reads back soon: stored past the caches)
        __builtin_nontemporal_store(v.x, &out[t].x);
        __builtin_nontemporal_store(v.y, &out[t].y);
        __builtin_nontemporal_store(v.z, &out[t].z);
        __builtin_nontemporal_store(v.w, &out[t].w);
    }
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* p, uint32_t value, size_t count)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) p[i] = value;
}

template <uint32_t TYPE>
hipError_t launch_deq(Lane* lane, const void* w, float* out, int64_t elements)
{
    const int64_t quads = elements / 4;
    if (quads == 0) return hipSuccess;
    int64_t blocks = (quads + 255) / 256;
    const int64_t cap = static_cast<int64_t>(lane->compute_units) * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(dequantize_kernel<TYPE>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, lane->stream,
                       static_cast<const uint8_t*>(w), reinterpret_cast<float4*>(out), quads);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_dequantize(Lane* lane, uint32_t type, const void* w, float* out, int64_t elements)
{
    switch (type) {
    case NNHIP_TYPE_Q8_0: return launch_deq<NNHIP_TYPE_Q8_0>(lane, w, out, elements);
    case NNHIP_TYPE_Q4_K: return launch_deq<NNHIP_TYPE_Q4_K>(lane, w, out, elements);
    case NNHIP_TYPE_Q5_K: return launch_deq<NNHIP_TYPE_Q5_K>(lane, w, out, elements);
    case NNHIP_TYPE_Q6_K: return launch_deq<NNHIP_TYPE_Q6_K>(lane, w, out, elements);
    case NNHIP_TYPE_IQ3_S: return launch_deq<NNHIP_TYPE_IQ3_S>(lane, w, out, elements);
    case NNHIP_TYPE_IQ2_S: return launch_deq<NNHIP_TYPE_IQ2_S>(lane, w, out, elements);
    case NNHIP_TYPE_BF16: return launch_deq<NNHIP_TYPE_BF16>(lane, w, out, elements);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_fill_u32(Lane* lane, uint32_t* p, uint32_t value, size_t count)
{
    if (count == 0) return hipSuccess;
    size_t blocks = (count + 255) / 256;
    const size_t cap = static_cast<size_t>(lane->compute_units) * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(fill_u32_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, lane->stream, p, value, count);
    return hipGetLastError();
}

}  // namespace nnhip
