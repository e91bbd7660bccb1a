// Device-side helpers shared by the GGUF kernels: block geometry, half conversion, wave64 reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nnhip {

// GGUF block geometry (bytes per block / elements per block).
constexpr int kQ8_0Bytes = 34, kQ8_0Elems = 32;
constexpr int kQ4KBytes = 144, kQ5KBytes = 176, kQ6KBytes = 210, kIQ2SBytes = 82, kSuperElems = 256;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Global loads whose address is only 2- or 4-byte aligned (34-, 82- and 210-byte blocks).  gfx950 serves them with
// one dwordx4 / dwordx2 / dword instruction in unaligned access mode.
struct __attribute__((packed, aligned(2))) U128a2 { u32x4 v; };
struct __attribute__((packed, aligned(2))) U64a2 { u32x2 v; };
struct __attribute__((packed, aligned(2))) U32a2 { uint32_t v; };

__device__ __forceinline__ u32x4 ld128(const uint8_t* p) { return reinterpret_cast<const U128a2*>(p)->v; }
__device__ __forceinline__ u32x2 ld64(const uint8_t* p) { return reinterpret_cast<const U64a2*>(p)->v; }
__device__ __forceinline__ uint32_t ld32(const uint8_t* p) { return reinterpret_cast<const U32a2*>(p)->v; }
__device__ __forceinline__ uint32_t ld16(const uint8_t* p) { return *reinterpret_cast<const uint16_t*>(p); }

// IEEE binary16 bit pattern (low 16 bits of h) -> binary32, exact: v_cvt_f32_f16 keeps subnormals because HIP
// kernels run with FP16 denormals enabled.
__device__ __forceinline__ float half_bits_to_float(uint32_t h)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(h & 0xffffu)));
}

// Keeps `v` in a VGPR and hides its producer from the optimiser, so a byte mask applied once per dword is not
// folded back into one bit-field extract per byte.
__device__ __forceinline__ uint32_t opaque(uint32_t v)
{
    asm("" : "+v"(v));
    return v;
}

// Byte i of v as float (v_cvt_f32_ubyte{i}).
__device__ __forceinline__ float ubyte0(uint32_t v) { return static_cast<float>(v & 0xffu); }
__device__ __forceinline__ float ubyte1(uint32_t v) { return static_cast<float>((v >> 8) & 0xffu); }
__device__ __forceinline__ float ubyte2(uint32_t v) { return static_cast<float>((v >> 16) & 0xffu); }
__device__ __forceinline__ float ubyte3(uint32_t v) { return static_cast<float>(v >> 24); }
// Signed byte i of v as float (v_cvt_f32_i32 with an SDWA sign-extending byte select).
__device__ __forceinline__ float sbyte0(uint32_t v) { return static_cast<float>(static_cast<int8_t>(v & 0xffu)); }
__device__ __forceinline__ float sbyte1(uint32_t v) { return static_cast<float>(static_cast<int8_t>((v >> 8) & 0xffu)); }
__device__ __forceinline__ float sbyte2(uint32_t v) { return static_cast<float>(static_cast<int8_t>((v >> 16) & 0xffu)); }
__device__ __forceinline__ float sbyte3(uint32_t v) { return static_cast<float>(static_cast<int8_t>(v >> 24)); }

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// Sum over the 64 lanes of a wave in a fixed order; the total is returned in every lane.
__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_mov<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_mov<0x141>(v);   // row_half_mirror
    v += dpp_mov<0x140>(v);   // row_mirror: every lane of a 16-lane row now holds the row total
    float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (a + b) + (c + d);
}

// Sum over aligned groups of 8 lanes (the total lands in every lane of the group).
__device__ __forceinline__ float oct_sum(float v)
{
    v += dpp_mov<0xB1>(v);
    v += dpp_mov<0x4E>(v);
    v += dpp_mov<0x141>(v);
    return v;
}

// 6-bit (scale, min) pairs of Q4_K / Q5_K for sub-blocks 2j and 2j+1, j in 0..3, from the three dwords that hold
// the 12 packed bytes.  Returns scales in bytes 0,1 of `sc` and mins in bytes 0,1 of `mn`.
__device__ __forceinline__ void k4_scale_pair(uint32_t s0, uint32_t s1, uint32_t s2, int j, uint32_t& sc, uint32_t& mn)
{
    const int sh = (j & 1) * 16;
    const uint32_t a = (s0 >> sh) & 0xffffu;  // packed bytes 2(j&1), 2(j&1)+1
    const uint32_t b = (s1 >> sh) & 0xffffu;  // packed bytes 4 + ...
    const uint32_t c = (s2 >> sh) & 0xffffu;  // packed bytes 8 + ...
    const uint32_t lo_sc = a & 0x3f3fu, lo_mn = b & 0x3f3fu;
    const uint32_t hi_sc = (c & 0x0f0fu) | ((a >> 2) & 0x3030u);
    const uint32_t hi_mn = ((c >> 4) & 0x0f0fu) | ((b >> 2) & 0x3030u);
    sc = j < 2 ? lo_sc : hi_sc;
    mn = j < 2 ? lo_mn : hi_mn;
}

}  // namespace nnhip
