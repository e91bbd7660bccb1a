// Synthetic Q8_0 weights and normal activations drawn on the device (benchmark / test support, see
// include/nnhip_synth.h).  Counter-based: every value is a pure function of (seed, index).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nnhip_synth.h"

namespace {

__device__ __forceinline__ uint64_t mix64(uint64_t z)   // splitmix64 finaliser
{
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ void normal_pair(uint64_t key, float& a, float& b)   // Box-Muller
{
    const uint64_t r = mix64(key);
    const float u1 = (static_cast<float>(static_cast<uint32_t>(r >> 40)) + 0.5f) * (1.0f / 16777216.0f);
    const float u2 = (static_cast<float>(static_cast<uint32_t>(r) >> 8) + 0.5f) * (1.0f / 16777216.0f);
    const float rad = sqrtf(-2.0f * logf(u1));
    float s, c;
    sincosf(6.283185307179586f * u2, &s, &c);
    a = rad * c;
    b = rad * s;
}

// One thread per block: 34 bytes written as 17 halfwords (block starts are 2-byte aligned).
__global__ __launch_bounds__(256) void synth_q8_0_kernel(uint16_t* out, uint64_t blocks, uint64_t seed, float sigma)
{
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    for (uint64_t b = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; b < blocks; b += stride) {
        float w[32];
        float amax = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            normal_pair(seed * 0x100000001b3ull + b * 16 + i, w[2 * i], w[2 * i + 1]);
            w[2 * i] *= sigma;
            w[2 * i + 1] *= sigma;
            amax = fmaxf(amax, fmaxf(fabsf(w[2 * i]), fabsf(w[2 * i + 1])));
        }
        const float d = amax / 127.0f;
        const float inv = d > 0.0f ? 1.0f / d : 0.0f;
        uint16_t* p = out + b * 17;
        p[0] = __builtin_bit_cast(unsigned short, static_cast<_Float16>(d));
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            int q0 = static_cast<int>(roundf(w[2 * i] * inv)), q1 = static_cast<int>(roundf(w[2 * i + 1] * inv));
            q0 = max(-127, min(127, q0));
            q1 = max(-127, min(127, q1));
            p[1 + i] = static_cast<uint16_t>((q0 & 0xff) | ((q1 & 0xff) << 8));
        }
    }
}

__global__ __launch_bounds__(256) void synth_normal_kernel(float* out, uint64_t count, uint64_t seed)
{
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    const uint64_t pairs = (count + 1) / 2;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < pairs; i += stride) {
        float a, b;
        normal_pair(seed * 0x100000001b3ull + i, a, b);
        out[2 * i] = a;
        if (2 * i + 1 < count) out[2 * i + 1] = b;
    }
}

}  // namespace

extern "C" {

__attribute__((visibility("default"))) int nnhip_synth_q8_0(void* stream, void* dptr, uint64_t blocks, uint64_t seed,
                                                           float sigma)
{
    if (!dptr || (reinterpret_cast<uintptr_t>(dptr) & 1u)) return static_cast<int>(hipErrorInvalidValue);
    if (blocks == 0) return 0;
    uint64_t grid = (blocks + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(synth_q8_0_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint16_t*>(dptr), blocks, seed, sigma);
    return static_cast<int>(hipGetLastError());
}

__attribute__((visibility("default"))) int nnhip_synth_normal_f32(void* stream, float* dptr, uint64_t count, uint64_t seed)
{
    if (!dptr) return static_cast<int>(hipErrorInvalidValue);
    if (count == 0) return 0;
    uint64_t grid = ((count + 1) / 2 + 255) / 256;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(synth_normal_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), dptr, count, seed);
    return static_cast<int>(hipGetLastError());
}

}  // extern "C"
