// Tasks of the matrix-core mat-vec kernels: what one wave does with 16 matrix rows x one 256-weight block column of a
// storage format (operand B from the raw block bytes, operand A from digit planes of the activations), and the helpers
// around them.  Shared by gemv_mfma_kernels.hip (batched launches, shared passes) and gemv_mfma_stream.hip (single and
// fused calls).  Everything here has internal linkage: each translation unit that includes it gets its own copy.
#pragma once

#include <cstddef>
#include <cstring>
#include <type_traits>

#include "nnhip_internal.h"
#include "quant_device.h"

#include "iq_grids.inc"

namespace nnhip {

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 16;            // matrix rows per stage = the N of the MFMA
constexpr int kMaxWaves = 12;            // three waves per SIMD: 170 vector registers each


constexpr int kLdsBudget = 156 * 1024;   // dynamic LDS a workgroup may take (the static arrays take 2.1 KB of the 160 KB)
constexpr uint32_t kNoPiece = 0x80000000u;       // added to the offset of a piece that is not to be fetched: beyond any matrix

#define NNHIP_LDS_PTR __attribute__((address_space(3)))
// address-space qualifiers only mean something to the device pass
#if defined(__HIP_DEVICE_COMPILE__)
#define NNHIP_CONST_PTR __attribute__((address_space(4)))
#else
#define NNHIP_CONST_PTR
#endif

__device__ __forceinline__ uint32_t umax_u(uint32_t a, uint32_t b) { return a > b ? a : b; }

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov_u(uint32_t v)
{
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, true));
}

__device__ __forceinline__ uint32_t wave_umax(uint32_t v)
{
    v = umax_u(v, dpp_mov_u<0xB1>(v));
    v = umax_u(v, dpp_mov_u<0x4E>(v));
    v = umax_u(v, dpp_mov_u<0x141>(v));
    v = umax_u(v, dpp_mov_u<0x140>(v));
    const uint32_t a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const uint32_t c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return umax_u(umax_u(a, b), umax_u(c, d));
}

// p[l] + p[l+16] + p[l+32] + p[l+48] as (p0 + p1) + (p2 + p3), in every lane (v_permlane16_swap exchanges the odd
// 16-lane rows of its first operand with the even rows of its second, v_permlane32_swap the upper half of the first
// with the lower half of the second).
__device__ __forceinline__ float quarter_sum(float p)
{
    const uint32_t u = __float_as_uint(p);
    auto s16 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float t = __uint_as_float(s16[0]) + __uint_as_float(s16[1]);
    const uint32_t v = __float_as_uint(t);
    auto s32 = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return __uint_as_float(s32[0]) + __uint_as_float(s32[1]);
}

// Four fixed-point values -> the four digit planes of those values (byte i of plane p = digit p of value i).
__device__ __forceinline__ void digit_planes(int v0, int v1, int v2, int v3, uint32_t out[4])
{
    // balanced digits: add 128 to the three low digits with carry, then flip their top bits
    const uint32_t d0 = (static_cast<uint32_t>(v0) + 0x00808080u) ^ 0x00808080u;
    const uint32_t d1 = (static_cast<uint32_t>(v1) + 0x00808080u) ^ 0x00808080u;
    const uint32_t d2 = (static_cast<uint32_t>(v2) + 0x00808080u) ^ 0x00808080u;
    const uint32_t d3 = (static_cast<uint32_t>(v3) + 0x00808080u) ^ 0x00808080u;
    // 4 x 4 byte transpose (v_perm_b32: selector bytes 0-3 pick from the second operand, 4-7 from the first)
    const uint32_t t0 = __builtin_amdgcn_perm(d1, d0, 0x05010400u);   // d0.b0 d1.b0 d0.b1 d1.b1
    const uint32_t t1 = __builtin_amdgcn_perm(d1, d0, 0x07030602u);   // d0.b2 d1.b2 d0.b3 d1.b3
    const uint32_t t2 = __builtin_amdgcn_perm(d3, d2, 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(d3, d2, 0x07030602u);
    out[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    out[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    out[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    out[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

// sum_p 256^p S_p of the four digit-plane sums.  |S_p| <= 32 * 31 * 128 < 2^17, so S_0 + 256 S_1 and S_2 + 256 S_3 are
// exact in int32 and below 2^25... their conversions to FP32 round at most once each (below 2^24: exact), and one fused
// multiply-add joins them.
__device__ __forceinline__ float recombine(i32x4 s)
{
    const int lo = s[0] + (s[1] << 8), hi = s[2] + (s[3] << 8);
    return fmaf(static_cast<float>(hi), 65536.0f, static_cast<float>(lo));
}

// The same for plane sums of up to 2^24 (scale factors already multiplied in): the pairs are joined in FP32, each join
// rounding at 2^-24 of its value.
__device__ __forceinline__ float recombine_wide(i32x4 s)
{
    const float lo = fmaf(static_cast<float>(s[1]), 256.0f, static_cast<float>(s[0]));
    const float hi = fmaf(static_cast<float>(s[3]), 256.0f, static_cast<float>(s[2]));
    return fmaf(hi, 65536.0f, lo);
}

// a * b for operands inside 24 signed bits (v_mul_i32_i24 / v_mad_i32_i24: full rate; the 32-bit multiply is quarter rate)
__device__ __forceinline__ int mul24(int a, int b) { return __mul24(a, b); }

__device__ __forceinline__ i32x4 mfma_i8(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, i32x4 c)
{
    return __builtin_amdgcn_mfma_i32_16x16x32_i8(__builtin_bit_cast(long, u32x2{a0, a1}), __builtin_bit_cast(long, u32x2{b0, b1}),
                                                 c, 0, 0, 0);
}

__device__ __forceinline__ u32x4 lds128(const uint8_t* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ u32x2 lds64(const uint8_t* p) { return *reinterpret_cast<const u32x2*>(p); }

// This lane's part of operand A for one super-block column: 64 bytes (its digit plane of its quarter's 64 activations;
// zeros in the lanes outside the block diagonal) and the FP32 sums of x over the quarter's NS scale groups.
template <int NS>
struct XSet {
    u32x4 a[4];
    float sx[NS];
    float ie[2];      // block fixed point only: 2^-e of the two 32-activation groups behind a[0], a[1] and a[2], a[3]
};

// 2^-e of 32-activation groups g0 and g1 (block fixed point; `exps` is null where one exponent serves the whole vector).
template <class XS>
__device__ __forceinline__ void load_ie(XS& xs, const float* exps, int g0, int g1)
{
    if (exps) {
        xs.ie[0] = exps[g0];
        xs.ie[1] = exps[g1];
    }
}

// One task of a storage format: 16 rows x one super-block.  `blk` is this lane's row of the stage at the task's block
// column (LDS).  Adds this lane's share (quarter lane / 16 of row lane % 16) to accq (the quant part, still in
// fixed-point units) and accm (the minimum part).
struct Q4KTask {
    static constexpr int kBlockBytes = kQ4KBytes;     // 144 = 9 pieces; blocks and rows are 16-byte aligned
    static constexpr int kLdsTableBytes = 0;          // no lookup tables in LDS
    static constexpr int kPieces = 9;                 // 16-byte pieces a block takes in a stage
    static constexpr int kSumRun = 32;                // activations per FP32 sum (one sub-block)
    static constexpr int kWideM = 1;                  // wide form: block columns per wave and stage,
    static constexpr int kWideLpw = 3;                // and 1 KB pieces per wave and stage (W <= 12)
    static constexpr bool kNeedsSums = true;
    static constexpr bool kTightStage = false;
    static constexpr int kSharedM = kWideM, kSharedLpw = kWideLpw;      // the same with four input rows per pass
    static __device__ __forceinline__ void init_tables(uint8_t*, int, int) {}
    using X = XSet<2>;
    struct Raw { u32x4 h, q1, q2; };

    static __device__ __forceinline__ uint32_t piece_src(uint32_t q, bool) { return 16u * q; }

    // plane = this lane's digit plane of the whole vector, sums = the per-sub-block sums of x; b = super-block column;
    // zeros = null in the lanes on the block diagonal of operand A, else 256 zero bytes in LDS (read in place of the
    // plane: no branch, and the compiler may interleave the reads of two tasks)
    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float* sums, int b, int quarter, const uint8_t* zeros,
                                                  const float* exps = nullptr)
    {
        const uint8_t* src = zeros ? zeros : plane + 256 * b + 64 * quarter;
#pragma unroll
        for (int u = 0; u < 4; ++u) xs.a[u] = lds128(src + 16 * u);
        const float2 v = *reinterpret_cast<const float2*>(sums + 8 * b + 2 * quarter);
        xs.sx[0] = v.x;
        xs.sx[1] = v.y;
        load_ie(xs, exps, 8 * b + 2 * quarter, 8 * b + 2 * quarter + 1);
    }

    static __device__ __forceinline__ Raw load(const uint8_t* blk, int quarter, bool)
    {
        Raw r;
        r.q1 = lds128(blk + 16 + 32 * quarter);
        r.q2 = lds128(blk + 32 + 32 * quarter);
        r.h = lds128(blk);
        return r;
    }

    // The form for passes that several input rows share (see the kernel): one MFMA per 32-weight sub-block, operand A = the
    // four digit planes of up to four input rows, K group g = weights 8 g .. 8 g + 7 of the sub-block.  This lane supplies
    // those eight weights of its matrix row (`g` = lane / 16) and receives the plane sums of input row lane / 16.
    static constexpr bool kStacked = true;
    struct RawS { u32x4 h; u32x2 q[4]; };

    static __device__ __forceinline__ RawS load_stacked(const uint8_t* blk, int g, bool)
    {
        RawS r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r.q[j] = lds64(blk + 16 + 32 * j + 8 * g);
        r.h = lds128(blk);
        return r;
    }

    // a_plane = this lane's digit plane (as a supplier of operand A) at the block's first activation + 8 g; sums = the
    // eight sub-block sums of x of the input row this lane receives
    static __device__ __forceinline__ void run_stacked(const RawS& r, const uint8_t* a_plane, const float* sums, const uint8_t*,
                                                       float& accq, float& accm)
    {
        constexpr uint32_t kLow = 0x0f0f0f0fu;
        u32x2 a[8];
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) a[sb] = lds64(a_plane + 32 * sb);
        float2 sx[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) sx[j] = *reinterpret_cast<const float2*>(sums + 2 * j);
        const float d = half_bits_to_float(r.h[0]), dmin = half_bits_to_float(r.h[0] >> 16);
        // the 6-bit scales are multiplied into the integer plane sums (|sum| <= 32 * 15 * 128 < 2^16, eight of them times
        // 63 stay below 2^25) and the block is recombined once; the minima are summed before dmin multiplies them
        i32x4 total = {0, 0, 0, 0};
        float mins = 0.0f;
        i32x4 s_lo[4], s_hi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {           // (all eight products first: their results are not needed one by one)
            const i32x4 zero = {0, 0, 0, 0};
            s_lo[j] = mfma_i8(a[2 * j][0], a[2 * j][1], r.q[j][0] & kLow, r.q[j][1] & kLow, zero);
            s_hi[j] = mfma_i8(a[2 * j + 1][0], a[2 * j + 1][1], (r.q[j][0] >> 4) & kLow, (r.q[j][1] >> 4) & kLow, zero);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t sc, mn;
            k4_scale_pair(r.h[1], r.h[2], r.h[3], j, sc, mn);
            const int f_lo = static_cast<int>(sc & 0xffu), f_hi = static_cast<int>((sc >> 8) & 0xffu);
#pragma unroll
            for (int p = 0; p < 4; ++p) total[p] += mul24(f_lo, s_lo[j][p]) + mul24(f_hi, s_hi[j][p]);      // (24-bit operands: one full-rate instruction each)
            mins = fmaf(ubyte0(mn), sx[j].x, mins);
            mins = fmaf(ubyte1(mn), sx[j].y, mins);
        }
        accq = fmaf(d, recombine_wide(total), accq);
        accm = fmaf(dmin, mins, accm);
    }

    template <bool BX = false>
    static __device__ __forceinline__ void run(const Raw& r, const X& xs, int quarter, const uint8_t*, float& accq, float& accm)
    {
        constexpr uint32_t kLow = 0x0f0f0f0fu;
        const u32x4 q1 = r.q1, q2 = r.q2, h = r.h;
        const u32x4 a0 = xs.a[0], a1 = xs.a[1], a2 = xs.a[2], a3 = xs.a[3];
        i32x4 s_lo = {0, 0, 0, 0}, s_hi = {0, 0, 0, 0};
        // low nibbles: weights 0-31 of the quarter (sub-block 2 * quarter), high nibbles: weights 32-63
        s_lo = mfma_i8(a0[0], a0[1], q1[0] & kLow, q1[1] & kLow, s_lo);
        s_hi = mfma_i8(a2[0], a2[1], (q1[0] >> 4) & kLow, (q1[1] >> 4) & kLow, s_hi);
        s_lo = mfma_i8(a0[2], a0[3], q1[2] & kLow, q1[3] & kLow, s_lo);
        s_hi = mfma_i8(a2[2], a2[3], (q1[2] >> 4) & kLow, (q1[3] >> 4) & kLow, s_hi);
        s_lo = mfma_i8(a1[0], a1[1], q2[0] & kLow, q2[1] & kLow, s_lo);
        s_hi = mfma_i8(a3[0], a3[1], (q2[0] >> 4) & kLow, (q2[1] >> 4) & kLow, s_hi);
        s_lo = mfma_i8(a1[2], a1[3], q2[2] & kLow, q2[3] & kLow, s_lo);
        s_hi = mfma_i8(a3[2], a3[3], (q2[2] >> 4) & kLow, (q2[3] >> 4) & kLow, s_hi);
        const float d = half_bits_to_float(h[0]), dmin = half_bits_to_float(h[0] >> 16);
        uint32_t sc, mn;
        k4_scale_pair(h[1], h[2], h[3], quarter, sc, mn);
        // (block fixed point: the plane sums of a 32-weight sub-block are in units of its own 2^-e)
        const float f_lo = BX ? (d * ubyte0(sc)) * xs.ie[0] : d * ubyte0(sc);
        const float f_hi = BX ? (d * ubyte1(sc)) * xs.ie[1] : d * ubyte1(sc);
        accq = fmaf(f_lo, recombine(s_lo), accq);
        accq = fmaf(f_hi, recombine(s_hi), accq);
        accm = fmaf(dmin * ubyte0(mn), xs.sx[0], accm);
        accm = fmaf(dmin * ubyte1(mn), xs.sx[1], accm);
    }
};

// Q5_K: as Q4_K plus one high bit per weight; bit g of qh[i] belongs to weight i of sub-block g (header, 32 bytes of
// qh, 128 nibble bytes: 176 = 11 pieces).
struct Q5KTask {
    static constexpr int kBlockBytes = kQ5KBytes;
    static constexpr int kLdsTableBytes = 0;          // no lookup tables in LDS
    static constexpr int kPieces = 11;
    static constexpr int kSumRun = 32;
    static constexpr int kWideM = 1;
    static constexpr int kWideLpw = 3;
    static constexpr bool kNeedsSums = true;
    static constexpr bool kTightStage = false;
    static constexpr int kSharedM = kWideM, kSharedLpw = kWideLpw;      // the same with four input rows per pass
    static __device__ __forceinline__ void init_tables(uint8_t*, int, int) {}
    using X = XSet<2>;
    struct Raw { u32x4 h, ha, hb, q1, q2; };

    static __device__ __forceinline__ uint32_t piece_src(uint32_t q, bool) { return 16u * q; }

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float* sums, int b, int quarter, const uint8_t* zeros,
                                                  const float* exps = nullptr)
    {
        Q4KTask::load_x(xs, plane, sums, b, quarter, zeros, exps);
    }

    static __device__ __forceinline__ Raw load(const uint8_t* blk, int quarter, bool)
    {
        Raw r;
        r.q1 = lds128(blk + 48 + 32 * quarter);
        r.ha = lds128(blk + 16);
        r.q2 = lds128(blk + 64 + 32 * quarter);
        r.hb = lds128(blk + 32);
        r.h = lds128(blk);
        return r;
    }

    // shared passes: as Q4KTask::run_stacked, the fifth bits of sub-block s being bit s of the qh bytes 8 g .. 8 g + 7
    static constexpr bool kStacked = true;
    struct RawS { u32x4 h; u32x2 hq; u32x2 q[4]; };

    static __device__ __forceinline__ RawS load_stacked(const uint8_t* blk, int g, bool)
    {
        RawS r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r.q[j] = lds64(blk + 48 + 32 * j + 8 * g);
        r.hq = lds64(blk + 16 + 8 * g);
        r.h = lds128(blk);
        return r;
    }

    static __device__ __forceinline__ void run_stacked(const RawS& r, const uint8_t* a_plane, const float* sums, const uint8_t*,
                                                       float& accq, float& accm)
    {
        constexpr uint32_t kLow = 0x0f0f0f0fu, kBit4 = 0x10101010u;
        u32x2 a[8];
#pragma unroll
        for (int sb = 0; sb < 8; ++sb) a[sb] = lds64(a_plane + 32 * sb);
        float2 sx[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) sx[j] = *reinterpret_cast<const float2*>(sums + 2 * j);
        const float d = half_bits_to_float(r.h[0]), dmin = half_bits_to_float(r.h[0] >> 16);
        i32x4 total = {0, 0, 0, 0};
        float mins = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const i32x4 zero = {0, 0, 0, 0};
            auto lo5 = [&](uint32_t q, uint32_t hq) { return (q & kLow) | (((hq >> (2 * j)) << 4) & kBit4); };
            auto hi5 = [&](uint32_t q, uint32_t hq) { return ((q >> 4) & kLow) | (((hq >> (2 * j)) << 3) & kBit4); };
            const i32x4 s_lo = mfma_i8(a[2 * j][0], a[2 * j][1], lo5(r.q[j][0], r.hq[0]), lo5(r.q[j][1], r.hq[1]), zero);
            const i32x4 s_hi = mfma_i8(a[2 * j + 1][0], a[2 * j + 1][1], hi5(r.q[j][0], r.hq[0]), hi5(r.q[j][1], r.hq[1]), zero);
            uint32_t sc, mn;
            k4_scale_pair(r.h[1], r.h[2], r.h[3], j, sc, mn);
            const int f_lo = static_cast<int>(sc & 0xffu), f_hi = static_cast<int>((sc >> 8) & 0xffu);
#pragma unroll
            for (int p = 0; p < 4; ++p) total[p] += mul24(f_lo, s_lo[p]) + mul24(f_hi, s_hi[p]);      // (|sum| <= 32 * 31 * 128 < 2^17, 24-bit multiplies: below 2^26)
            mins = fmaf(ubyte0(mn), sx[j].x, mins);
            mins = fmaf(ubyte1(mn), sx[j].y, mins);
        }
        accq = fmaf(d, recombine_wide(total), accq);
        accm = fmaf(dmin, mins, accm);
    }

    template <bool BX = false>
    static __device__ __forceinline__ void run(const Raw& r, const X& xs, int quarter, const uint8_t*, float& accq, float& accm)
    {
        constexpr uint32_t kLow = 0x0f0f0f0fu, kBit4 = 0x10101010u;
        const u32x4 h = r.h, ha = r.ha, hb = r.hb, q1 = r.q1, q2 = r.q2;
        const u32x4 a0 = xs.a[0], a1 = xs.a[1], a2 = xs.a[2], a3 = xs.a[3];
        const int sh = 2 * quarter;
        i32x4 s_lo = {0, 0, 0, 0}, s_hi = {0, 0, 0, 0};
        auto lo5 = [&](uint32_t q, uint32_t hq) { return (q & kLow) | (((hq >> sh) << 4) & kBit4); };
        auto hi5 = [&](uint32_t q, uint32_t hq) { return ((q >> 4) & kLow) | (((hq >> sh) << 3) & kBit4); };
        s_lo = mfma_i8(a0[0], a0[1], lo5(q1[0], ha[0]), lo5(q1[1], ha[1]), s_lo);
        s_hi = mfma_i8(a2[0], a2[1], hi5(q1[0], ha[0]), hi5(q1[1], ha[1]), s_hi);
        s_lo = mfma_i8(a0[2], a0[3], lo5(q1[2], ha[2]), lo5(q1[3], ha[3]), s_lo);
        s_hi = mfma_i8(a2[2], a2[3], hi5(q1[2], ha[2]), hi5(q1[3], ha[3]), s_hi);
        s_lo = mfma_i8(a1[0], a1[1], lo5(q2[0], hb[0]), lo5(q2[1], hb[1]), s_lo);
        s_hi = mfma_i8(a3[0], a3[1], hi5(q2[0], hb[0]), hi5(q2[1], hb[1]), s_hi);
        s_lo = mfma_i8(a1[2], a1[3], lo5(q2[2], hb[2]), lo5(q2[3], hb[3]), s_lo);
        s_hi = mfma_i8(a3[2], a3[3], hi5(q2[2], hb[2]), hi5(q2[3], hb[3]), s_hi);
        const float d = half_bits_to_float(h[0]), dmin = half_bits_to_float(h[0] >> 16);
        uint32_t sc, mn;
        k4_scale_pair(h[1], h[2], h[3], quarter, sc, mn);
        // (block fixed point: the plane sums of a 32-weight sub-block are in units of its own 2^-e)
        const float f_lo = BX ? (d * ubyte0(sc)) * xs.ie[0] : d * ubyte0(sc);
        const float f_hi = BX ? (d * ubyte1(sc)) * xs.ie[1] : d * ubyte1(sc);
        accq = fmaf(f_lo, recombine(s_lo), accq);
        accq = fmaf(f_hi, recombine(s_hi), accq);
        accm = fmaf(dmin * ubyte0(mn), xs.sx[0], accm);
        accm = fmaf(dmin * ubyte1(mn), xs.sx[1], accm);
    }
};

// Q6_K (GgufQ6K.cs:9-54): 210 bytes = ql[128] qh[64] scales[16] (int8) d (fp16); w = d * scale * (q - 32).  In half h,
// byte l of ql[64h ..] and ql[64h + 32 ..] carries weights l / l + 64 and l + 32 / l + 96 of the half in its nibbles, byte l
// of qh[32h ..] their four 2-bit tops, and the 16-weight group of weight i has scale 8h + i / 16.  Quarter (h, e) is
// the 32 ql bytes at 64h + 32e: low nibbles = weights 32e + l, high nibbles = weights 64 + 32e + l, four scale groups.
// The -32 is taken through sums of x: sum x s (q - 32) = s sum(q x) - 32 s sum(x).
// A block is 2-byte aligned in memory; a stage gives it 14 pieces (224 bytes) so that it starts 16-byte aligned in LDS.
struct Q6KTask {
    static constexpr int kBlockBytes = kQ6KBytes;
    static constexpr bool kStacked = false;
    static constexpr int kLdsTableBytes = 0;          // no lookup tables in LDS
    static constexpr int kPieces = 14;
    static constexpr int kSumRun = 16;
    static constexpr int kWideM = 1;
    static constexpr int kWideLpw = 4;
    static constexpr bool kNeedsSums = true;
    static constexpr bool kTightStage = false;
    static constexpr int kSharedM = kWideM, kSharedLpw = kWideLpw;      // the same with four input rows per pass
    static __device__ __forceinline__ void init_tables(uint8_t*, int, int) {}
    using X = XSet<4>;
    struct Raw { u32x4 la, lb, ha, hb; u32x2 sc; uint32_t d; };

    // Blocks with an even index start on a 4-byte boundary of their row and are fetched from there; the others start 2
    // bytes past one and are fetched from it, so every 16-byte request is dword-aligned and an odd block sits 2 bytes
    // into its 14 pieces.  (The last two bytes of an even block share a dword with the next block, an odd one: rows hold
    // an even number of blocks here, so that dword never reaches past the matrix.)
    static __device__ __forceinline__ uint32_t piece_src(uint32_t q, bool odd) { return 16u * q - (odd ? 2u : 0u); }

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float* sums, int b, int quarter, const uint8_t* zeros,
                                                  const float* exps = nullptr)
    {
        const int h = quarter >> 1, e = quarter & 1;
        load_ie(xs, exps, 8 * b + 4 * h + e, 8 * b + 4 * h + 2 + e);
        const uint8_t* src = zeros ? zeros : plane + 256 * b + 128 * h + 32 * e;
        xs.a[0] = lds128(src);
        xs.a[1] = lds128(src + 16);
        xs.a[2] = lds128(src + 64);
        xs.a[3] = lds128(src + 80);
        const float* sp = sums + 16 * b + 8 * h + 2 * e;
        const float2 lo = *reinterpret_cast<const float2*>(sp), hi = *reinterpret_cast<const float2*>(sp + 4);
        xs.sx[0] = lo.x;
        xs.sx[1] = lo.y;
        xs.sx[2] = hi.x;
        xs.sx[3] = hi.y;
    }

    // `odd` (uniform over the wave): the block's bytes sit 2 bytes into its pieces; whole dwords are read and shifted
    static __device__ __forceinline__ Raw load(const uint8_t* blk, int quarter, bool odd)
    {
        const int h = quarter >> 1, e = quarter & 1;
        const uint8_t* ql = blk + 64 * h + 32 * e;
        const uint8_t* qh = blk + 128 + 32 * h;
        const uint8_t* sc = blk + 192 + 8 * h;
        Raw r;
        r.la = lds128(ql);
        r.ha = lds128(qh);
        r.lb = lds128(ql + 16);
        r.hb = lds128(qh + 16);
        r.sc = *reinterpret_cast<const u32x2*>(sc);
        const uint32_t dword = *reinterpret_cast<const uint32_t*>(blk + 208);
        r.d = odd ? dword >> 16 : dword & 0xffffu;
        if (odd) {
            const uint32_t lt = *reinterpret_cast<const uint32_t*>(ql + 32), ht = *reinterpret_cast<const uint32_t*>(qh + 32);
            const uint32_t st = *reinterpret_cast<const uint32_t*>(sc + 8);
            auto shift8 = [](u32x4& a, u32x4& b, uint32_t tail) {
                a[0] = __builtin_amdgcn_alignbyte(a[1], a[0], 2);
                a[1] = __builtin_amdgcn_alignbyte(a[2], a[1], 2);
                a[2] = __builtin_amdgcn_alignbyte(a[3], a[2], 2);
                a[3] = __builtin_amdgcn_alignbyte(b[0], a[3], 2);
                b[0] = __builtin_amdgcn_alignbyte(b[1], b[0], 2);
                b[1] = __builtin_amdgcn_alignbyte(b[2], b[1], 2);
                b[2] = __builtin_amdgcn_alignbyte(b[3], b[2], 2);
                b[3] = __builtin_amdgcn_alignbyte(tail, b[3], 2);
            };
            shift8(r.la, r.lb, lt);
            shift8(r.ha, r.hb, ht);
            r.sc[0] = __builtin_amdgcn_alignbyte(r.sc[1], r.sc[0], 2);
            r.sc[1] = __builtin_amdgcn_alignbyte(st, r.sc[1], 2);
        }
        return r;
    }

    // The 6-bit quants of the task as operand B, and the scales: the same for every input row of a shared pass.
    static constexpr bool kSplitLookups = true;
    struct Looked { uint32_t lo[8], hi[8]; float d, c0, c1, c2, c3; };

    static __device__ __forceinline__ void lookup(const Raw& r, int quarter, const uint8_t*, Looked& lk)
    {
        constexpr uint32_t kLow = 0x0f0f0f0fu, kTop = 0x30303030u;
        const int sh = 2 * (quarter & 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lk.lo[i] = (r.la[i] & kLow) | (((r.ha[i] >> sh) << 4) & kTop);
            lk.hi[i] = ((r.la[i] >> 4) & kLow) | ((r.ha[i] >> sh) & kTop);
            lk.lo[4 + i] = (r.lb[i] & kLow) | (((r.hb[i] >> sh) << 4) & kTop);
            lk.hi[4 + i] = ((r.lb[i] >> 4) & kLow) | ((r.hb[i] >> sh) & kTop);
        }
        // scales 8h + 2e + {0, 1} and 8h + 4 + 2e + {0, 1}: bytes 2e, 2e + 1 of the two dwords read for half h
        const uint32_t w0 = r.sc[0] >> (8 * sh), w1 = r.sc[1] >> (8 * sh);
        lk.d = half_bits_to_float(r.d);
        lk.c0 = sbyte0(w0);
        lk.c1 = sbyte1(w0);
        lk.c2 = sbyte0(w1);
        lk.c3 = sbyte1(w1);
    }

    template <bool BX = false>
    static __device__ __forceinline__ void finish(const Raw&, const Looked& lk, const X& xs, float& accq, float& accm)
    {
        const u32x4 a0 = xs.a[0], a1 = xs.a[1], a2 = xs.a[2], a3 = xs.a[3];
        i32x4 s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0}, s2 = {0, 0, 0, 0}, s3 = {0, 0, 0, 0};
        s0 = mfma_i8(a0[0], a0[1], lk.lo[0], lk.lo[1], s0);
        s2 = mfma_i8(a2[0], a2[1], lk.hi[0], lk.hi[1], s2);
        s0 = mfma_i8(a0[2], a0[3], lk.lo[2], lk.lo[3], s0);
        s2 = mfma_i8(a2[2], a2[3], lk.hi[2], lk.hi[3], s2);
        s1 = mfma_i8(a1[0], a1[1], lk.lo[4], lk.lo[5], s1);
        s3 = mfma_i8(a3[0], a3[1], lk.hi[4], lk.hi[5], s3);
        s1 = mfma_i8(a1[2], a1[3], lk.lo[6], lk.lo[7], s1);
        s3 = mfma_i8(a3[2], a3[3], lk.hi[6], lk.hi[7], s3);
        const float d = lk.d, c0 = lk.c0, c1 = lk.c1, c2 = lk.c2, c3 = lk.c3;
        const float d0 = BX ? d * xs.ie[0] : d, d1 = BX ? d * xs.ie[1] : d;      // (block fixed point: powers of two, exact)
        accq = fmaf(d0 * c0, recombine(s0), accq);
        accq = fmaf(d0 * c1, recombine(s1), accq);
        accq = fmaf(d1 * c2, recombine(s2), accq);
        accq = fmaf(d1 * c3, recombine(s3), accq);
        const float t = fmaf(c0, xs.sx[0], fmaf(c1, xs.sx[1], fmaf(c2, xs.sx[2], c3 * xs.sx[3])));
        accm = fmaf(32.0f * d, t, accm);
    }

    template <bool BX = false>
    static __device__ __forceinline__ void run(const Raw& r, const X& xs, int quarter, const uint8_t*, float& accq, float& accm)
    {
        constexpr uint32_t kLow = 0x0f0f0f0fu, kTop = 0x30303030u;
        const int sh = 2 * (quarter & 1);
        const u32x4 a0 = xs.a[0], a1 = xs.a[1], a2 = xs.a[2], a3 = xs.a[3];
        auto lo6 = [&](uint32_t q, uint32_t t) { return (q & kLow) | (((t >> sh) << 4) & kTop); };
        auto hi6 = [&](uint32_t q, uint32_t t) { return ((q >> 4) & kLow) | ((t >> sh) & kTop); };
        i32x4 s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0}, s2 = {0, 0, 0, 0}, s3 = {0, 0, 0, 0};
        s0 = mfma_i8(a0[0], a0[1], lo6(r.la[0], r.ha[0]), lo6(r.la[1], r.ha[1]), s0);
        s2 = mfma_i8(a2[0], a2[1], hi6(r.la[0], r.ha[0]), hi6(r.la[1], r.ha[1]), s2);
        s0 = mfma_i8(a0[2], a0[3], lo6(r.la[2], r.ha[2]), lo6(r.la[3], r.ha[3]), s0);
        s2 = mfma_i8(a2[2], a2[3], hi6(r.la[2], r.ha[2]), hi6(r.la[3], r.ha[3]), s2);
        s1 = mfma_i8(a1[0], a1[1], lo6(r.lb[0], r.hb[0]), lo6(r.lb[1], r.hb[1]), s1);
        s3 = mfma_i8(a3[0], a3[1], hi6(r.lb[0], r.hb[0]), hi6(r.lb[1], r.hb[1]), s3);
        s1 = mfma_i8(a1[2], a1[3], lo6(r.lb[2], r.hb[2]), lo6(r.lb[3], r.hb[3]), s1);
        s3 = mfma_i8(a3[2], a3[3], hi6(r.lb[2], r.hb[2]), hi6(r.lb[3], r.hb[3]), s3);
        // scales 8h + 2e + {0, 1} and 8h + 4 + 2e + {0, 1}: bytes 2e, 2e + 1 of the two dwords read for half h
        const uint32_t w0 = r.sc[0] >> (8 * sh), w1 = r.sc[1] >> (8 * sh);
        const float d = half_bits_to_float(r.d);
        const float c0 = sbyte0(w0), c1 = sbyte1(w0), c2 = sbyte0(w1), c3 = sbyte1(w1);
        const float d0 = BX ? d * xs.ie[0] : d, d1 = BX ? d * xs.ie[1] : d;      // (block fixed point: powers of two, exact)
        accq = fmaf(d0 * c0, recombine(s0), accq);
        accq = fmaf(d0 * c1, recombine(s1), accq);
        accq = fmaf(d1 * c2, recombine(s2), accq);
        accq = fmaf(d1 * c3, recombine(s3), accq);
        const float t = fmaf(c0, xs.sx[0], fmaf(c1, xs.sx[1], fmaf(c2, xs.sx[2], c3 * xs.sx[3])));
        accm = fmaf(32.0f * d, t, accm);
    }
};

// Q8_0: w = d * q with 32 signed bytes q after a half-precision d, 34 bytes per 32 weights.  Eight such blocks are the
// 256 weights of one block column here: 272 bytes = 17 pieces exactly, and rows are whole columns (in_w % 256 == 0), so
// columns, rows and stages start on piece boundaries.  Quarter P = blocks 2P and 2P + 1 = the 68 bytes at 68 P of the
// column: 17 dwords, of which a lane's 16 rows x 4 quarters fall into 64 different LDS banks (row stride 205 or 103
// pieces).  The quants are the bytes of operand B as they are; those of the first block sit two bytes into their dwords
// (v_alignbyte_b32), those of the second on dword boundaries.  No minima, no offset: no sums of x.
struct Q8_0Task {
    static constexpr int kBlockBytes = 8 * kQ8_0Bytes;
    static constexpr int kLdsTableBytes = 0;          // no lookup tables in LDS
    static constexpr int kPieces = 17;
    static constexpr int kSumRun = 32;
    static constexpr int kWideM = 1;
    static constexpr int kWideLpw = 5;
    static constexpr bool kNeedsSums = false;
    static constexpr bool kTightStage = true;
    static constexpr int kSharedM = 1, kSharedLpw = 5;     // the same with four input rows per pass
    static constexpr int kOneM = 2, kOneLpw = 8;           // one stage = a whole tile: two block columns per wave
    static __device__ __forceinline__ void init_tables(uint8_t*, int, int) {}
    using X = XSet<1>;
    struct Raw { uint32_t w[17]; };

    static __device__ __forceinline__ uint32_t piece_src(uint32_t q, bool) { return 16u * q; }

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float*, int b, int quarter, const uint8_t* zeros,
                                                  const float* exps = nullptr)
    {
        load_ie(xs, exps, 8 * b + 2 * quarter, 8 * b + 2 * quarter + 1);
        const uint8_t* src = zeros ? zeros : plane + 256 * b + 64 * quarter;
#pragma unroll
        for (int u = 0; u < 4; ++u) xs.a[u] = lds128(src + 16 * u);
    }

    static __device__ __forceinline__ Raw load(const uint8_t* blk, int quarter, bool)
    {
        Raw r;
        const uint32_t* src = reinterpret_cast<const uint32_t*>(blk + 68 * quarter);
#pragma unroll
        for (int i = 0; i < 17; ++i) r.w[i] = src[i];
        return r;
    }

    // Shared passes (see Q4KTask::run_stacked): one MFMA per 34-byte block, K group g = its quants 8 g .. 8 g + 7, which
    // start two bytes into a dword in the even blocks of a column and on a dword boundary in the odd ones.
    static constexpr bool kStacked = true;
    struct RawS { uint32_t w[8][3]; uint32_t d[8]; };

    static __device__ __forceinline__ RawS load_stacked(const uint8_t* blk, int g, bool)
    {
        RawS r;
#pragma unroll
        for (int bi = 0; bi < 8; ++bi) {
            const uint32_t* src = reinterpret_cast<const uint32_t*>(blk + 34 * bi + ((bi & 1) ? 2 : 0) + 8 * g);
            r.w[bi][0] = src[0];
            r.w[bi][1] = src[1];
            r.w[bi][2] = (bi & 1) ? 0u : src[2];
            r.d[bi] = *reinterpret_cast<const uint16_t*>(blk + 34 * bi);
        }
        return r;
    }

    static __device__ __forceinline__ void run_stacked(const RawS& r, const uint8_t* a_plane, const float*, const uint8_t*,
                                                       float& accq, float&)
    {
        u32x2 a[8];
#pragma unroll
        for (int bi = 0; bi < 8; ++bi) a[bi] = lds64(a_plane + 32 * bi);
#pragma unroll
        for (int bi = 0; bi < 8; ++bi) {
            const uint32_t q_lo = (bi & 1) ? r.w[bi][0] : __builtin_amdgcn_alignbyte(r.w[bi][1], r.w[bi][0], 2);
            const uint32_t q_hi = (bi & 1) ? r.w[bi][1] : __builtin_amdgcn_alignbyte(r.w[bi][2], r.w[bi][1], 2);
            const i32x4 zero = {0, 0, 0, 0};
            const i32x4 sum = mfma_i8(a[bi][0], a[bi][1], q_lo, q_hi, zero);
            accq = fmaf(half_bits_to_float(r.d[bi]), recombine(sum), accq);
        }
    }

    template <bool BX = false>
    static __device__ __forceinline__ void run(const Raw& r, const X& xs, int, const uint8_t*, float& accq, float&)
    {
        const u32x4 a0 = xs.a[0], a1 = xs.a[1], a2 = xs.a[2], a3 = xs.a[3];
        uint32_t q0[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q0[i] = __builtin_amdgcn_alignbyte(r.w[i + 1], r.w[i], 2);
        i32x4 s0 = {0, 0, 0, 0}, s1 = {0, 0, 0, 0};
        s0 = mfma_i8(a0[0], a0[1], q0[0], q0[1], s0);
        s1 = mfma_i8(a2[0], a2[1], r.w[9], r.w[10], s1);
        s0 = mfma_i8(a0[2], a0[3], q0[2], q0[3], s0);
        s1 = mfma_i8(a2[2], a2[3], r.w[11], r.w[12], s1);
        s0 = mfma_i8(a1[0], a1[1], q0[4], q0[5], s0);
        s1 = mfma_i8(a3[0], a3[1], r.w[13], r.w[14], s1);
        s0 = mfma_i8(a1[2], a1[3], q0[6], q0[7], s0);
        s1 = mfma_i8(a3[2], a3[3], r.w[15], r.w[16], s1);
        // |plane sum| <= 32 * 128 * 128 = 2^19: the pair sums of recombine() stay inside int32, each rounds once in FP32
        const float d0 = half_bits_to_float(r.w[0]), d1 = half_bits_to_float(r.w[8] >> 16);
        accq = fmaf(BX ? d0 * xs.ie[0] : d0, recombine(s0), accq);
        accq = fmaf(BX ? d1 * xs.ie[1] : d1, recombine(s1), accq);
    }
};

// IQ2_S (NNtrain.Arc/Kernels/qwen35_iq.cl:411-419): 82 bytes = d (fp16), 32 index bytes, 32 sign bytes, 8 bytes of index
// tops (two bits per eight weights), 8 bytes of 4-bit scales (one per 16 weights).  Eight weights are one entry of a
// 1024-entry codebook of magnitude bytes (8, 25 or 43) with a sign bit each; w = d * (0.5 + scale) * 0.25 * magnitude *
// sign.  A codebook entry is exactly the eight bytes of operand B that a lane supplies for one MFMA; the signs go in as
// (magnitude ^ mask) + (mask & 1) per byte, with the two masks of a sign byte read from a 256-entry table.  Both tables
// sit in LDS (12 KB).  Quarter P = weights 64P .. 64P + 63 = 32-weight groups 2P and 2P + 1; four scale groups.
// Blocks are 2-byte aligned: fetched from the dword boundary at or below their start into six pieces, so an odd block
// sits 2 bytes into its pieces (and its index and sign bytes on dword boundaries, while those of an even block need a
// 2-byte shift).
__device__ const uint64_t g_iq2s_grid_mv[1024] = { NNHIP_IQ2S_GRID_VALUES };

struct IQ2STask {
    static constexpr int kBlockBytes = kIQ2SBytes;
    static constexpr bool kStacked = false;
    static constexpr int kPieces = 6;
    static constexpr int kSumRun = 32;
    static constexpr int kWideM = 2;                  // (the blocks are small: two per wave make a stage worth its barrier;
    static constexpr int kWideLpw = 4;                //  one where four input rows share a pass: registers)
    static constexpr int kSharedM = 1;
    static constexpr int kSharedLpw = 2;
    static constexpr bool kNeedsSums = false;         // no minimum or offset
    static constexpr bool kTightStage = true;         // 17408-wide planes leave no room for whole 1 KB slots per wave
    static constexpr int kGridBytes = 8192;
    static constexpr int kTableBytes = kGridBytes + 2048;     // the codebook and 256 selector pairs
    static constexpr int kLdsTableBytes = kTableBytes;        // (a static LDS array of the kernel)
    using X = XSet<1>;
    struct Raw { uint32_t q[2], s[2], tops, scales, d; };

    static __device__ __forceinline__ uint32_t piece_src(uint32_t q, bool odd) { return 16u * q - (odd ? 2u : 0u); }

    static __device__ __forceinline__ void init_tables(uint8_t* t, int tid, int threads)
    {
        for (int i = tid; i < 1024; i += threads) reinterpret_cast<uint64_t*>(t)[i] = g_iq2s_grid_mv[i];
        for (int i = tid; i < 256; i += threads) {
            // eight sign bits -> two v_perm_b32 selectors: byte k of a result comes from the magnitudes (selector byte k)
            // or from their negation (selector byte 4 + k)
            const uint32_t lo = ((static_cast<uint32_t>(i) & 15u) * 0x00204081u) & 0x01010101u;
            const uint32_t hi = ((static_cast<uint32_t>(i) >> 4) * 0x00204081u) & 0x01010101u;
            reinterpret_cast<u32x2*>(t + kGridBytes)[i] = u32x2{0x03020100u + (lo << 2), 0x03020100u + (hi << 2)};
        }
    }

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float*, int b, int quarter, const uint8_t* zeros,
                                                  const float* exps = nullptr)
    {
        load_ie(xs, exps, 8 * b + 2 * quarter, 8 * b + 2 * quarter + 1);
        const uint8_t* src = zeros ? zeros : plane + 256 * b + 64 * quarter;
#pragma unroll
        for (int u = 0; u < 4; ++u) xs.a[u] = lds128(src + 16 * u);
        xs.sx[0] = 0.0f;
    }

    static __device__ __forceinline__ Raw load(const uint8_t* blk, int quarter, bool odd)
    {
        // the block's byte k is at blk + k (+ 2 when odd); its index bytes 8P .. 8P + 7 start at 2 + 8P, the sign bytes 32 later
        const uint32_t* base = reinterpret_cast<const uint32_t*>(blk + 8 * quarter + (odd ? 4 : 0));
        const uint32_t sh = odd ? 0u : 2u;
        const uint8_t* b0 = blk + (odd ? 2 : 0);
        Raw r;
        const uint32_t q0 = base[0], q1 = base[1], q2 = base[2];
        const uint32_t s0 = base[8], s1 = base[9], s2 = base[10];
        r.q[0] = __builtin_amdgcn_alignbyte(q1, q0, sh);
        r.q[1] = __builtin_amdgcn_alignbyte(q2, q1, sh);
        r.s[0] = __builtin_amdgcn_alignbyte(s1, s0, sh);
        r.s[1] = __builtin_amdgcn_alignbyte(s2, s1, sh);
        r.tops = *reinterpret_cast<const uint16_t*>(b0 + 66 + 2 * quarter);
        r.scales = *reinterpret_cast<const uint16_t*>(b0 + 74 + 2 * quarter);
        r.d = *reinterpret_cast<const uint16_t*>(b0);
        return r;
    }

    // The sixteen lookups of a task and the products that use them are separate steps: with several input rows sharing
    // a pass the lookups are made once and every row multiplies with them.
    static constexpr bool kSplitLookups = true;
    struct Looked { u32x2 mag[8], sel[8]; };

    static __device__ __forceinline__ void lookup(const Raw& r, int, const uint8_t* tables, Looked& lk)
    {
        u32x2 (&mag)[8] = lk.mag;
        u32x2 (&sel)[8] = lk.sel;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            // the two top bits of entry o of the group as byte o, then index bytes and tops interleaved into 16-bit indices
            const uint32_t t8 = (r.tops >> (8 * g)) & 0xffu;
            const uint32_t tops = (t8 | (t8 << 6) | (t8 << 12) | (t8 << 18)) & 0x03030303u;
            const uint32_t pair[2] = {__builtin_amdgcn_perm(tops, r.q[g], 0x05010400u), __builtin_amdgcn_perm(tops, r.q[g], 0x07030602u)};
#pragma unroll
            for (int o = 0; o < 4; ++o) {
                const uint32_t index = (pair[o >> 1] >> (16 * (o & 1))) & 0xffffu;
                const uint32_t sign = (r.s[g] >> (8 * o)) & 0xffu;
                mag[4 * g + o] = *reinterpret_cast<const u32x2*>(tables + 8u * index);
                sel[4 * g + o] = *reinterpret_cast<const u32x2*>(tables + kGridBytes + 8u * sign);
            }
        }
    }

    template <bool BX = false>
    static __device__ __forceinline__ void finish(const Raw& r, const Looked& lk, const X& xs, float& accq, float&)
    {
        const u32x2 (&mag)[8] = lk.mag;
        const u32x2 (&sel)[8] = lk.sel;
        i32x4 acc[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            // -m per byte = (m ^ 0xff) + 1: no carry leaves a byte because no magnitude is zero
            const uint32_t neg0 = (mag[e][0] ^ 0xffffffffu) + 0x01010101u, neg1 = (mag[e][1] ^ 0xffffffffu) + 0x01010101u;
            const uint32_t b0 = __builtin_amdgcn_perm(neg0, mag[e][0], sel[e][0]), b1 = __builtin_amdgcn_perm(neg1, mag[e][1], sel[e][1]);
            const u32x4 av = xs.a[e >> 1];
            acc[e >> 1] = mfma_i8(av[2 * (e & 1)], av[2 * (e & 1) + 1], b0, b1, acc[e >> 1]);
        }
        // d (0.5 + s) 0.25 = d / 8 * (2 s + 1): the plane sums of the four scale groups are added up with the integer
        // factors 2 s + 1 (|sum| < 4 * 31 * 2^17 < 2^24: exact) and recombined once
        if constexpr (BX) {
            // block fixed point: the two 32-weight halves of the quarter carry exponents of their own
            i32x4 half_total[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int factor = static_cast<int>(2u * ((r.scales >> (4 * k)) & 15u) + 1u);
#pragma unroll
                for (int p = 0; p < 4; ++p) half_total[k >> 1][p] += mul24(factor, acc[k][p]);
            }
            const float dd = half_bits_to_float(r.d) * 0.125f;
            accq = fmaf(dd * xs.ie[0], recombine_wide(half_total[0]), accq);
            accq = fmaf(dd * xs.ie[1], recombine_wide(half_total[1]), accq);
            return;
        }
        i32x4 total = {0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int factor = static_cast<int>(2u * ((r.scales >> (4 * k)) & 15u) + 1u);    // nibble k & 1 of scale byte k >> 1
#pragma unroll
            for (int p = 0; p < 4; ++p) total[p] += mul24(factor, acc[k][p]);     // (24-bit operands: v_mad_i32_i24, not the quarter-rate 32-bit multiply)
        }
        accq = fmaf(half_bits_to_float(r.d) * 0.125f, recombine_wide(total), accq);
    }

    template <bool BX = false>
    static __device__ __forceinline__ void run(const Raw& r, const X& xs, int, const uint8_t* tables, float& accq, float&)
    {
        // every lookup of the task is requested before the first result is used (the scheduling barrier keeps the
        // compiler from folding the reads back into a chain of eight round trips to LDS)
        Looked lk;
        float unused = 0.0f;
        lookup(r, 0, tables, lk);
        __builtin_amdgcn_sched_barrier(0);
        finish<BX>(r, lk, xs, accq, unused);
    }
};

// Loads of the weight stream: 16 bytes per lane through a buffer descriptor that spans the matrix, non-temporal.  An
// offset beyond the buffer returns zeros without touching memory.
__device__ __forceinline__ u32x4 stream16(__amdgpu_buffer_rsrc_t matrix, uint32_t off)
{
    return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(matrix, static_cast<int>(off), 0, 2));
}

}  // namespace

}  // namespace nnhip
