// Decode mat-vec on the matrix cores: for the super-block formats whose unpacking is too much vector-ALU work for the
// lane-per-unit kernels (gemv_kernels.hip), Q4_K, Q5_K, Q6_K, IQ2_S and IQ3_S, and for Q8_0, whose signed bytes are operand B
// as they lie in memory and whose lane-per-unit kernel is held back by its cached, strided loads.  Used for the large
// groups of a batched launch and for calls with 2 - 16 input rows, where it streams faster than the row-step kernels;
// it takes longer to start, so single-row launches stay with those.  Two kernels share the tasks of the formats: matvec_mfma_kernel keeps
// operand A in registers (rows of one or two whole stages), matvec_mfma_wide_kernel keeps the digit planes in LDS (any
// row length, up to four input rows per pass over the weights); the text below describes the first, the second has its
// own paragraph further down.
//
// y[r, o] = bias[o] + sum_k x[r, k] * w[o, k]     (NNtrain.Arc/Kernels/qwen.cl:374-406 defines the operator)
//
// Arithmetic.  The activation vector is turned into 32-bit fixed point relative to its largest magnitude
// (v = rint(x * 2^e), |v| <= 2^30) and split into four balanced base-256 digits (each in [-128, 127]).
// v_mfma_i32_16x16x32_i8 then takes the exact integer sums sum_k digit_p(x_k) * q_k of one 32-weight sub-block for 16
// matrix rows at a time (operand B = the sub-block's quants as bytes, a few masks away from the raw block; operand A =
// digit planes).  The four K groups of an instruction carry four different 64-weight quarters of a super-block and operand A is
// block-diagonal to match (rows 4P .. 4P+3 = the four digit planes of quarter P in K group P, zeros elsewhere), so the 64
// lanes of the result hold the plane sums of (quarter lane / 16, matrix row lane % 16).  They are recombined
// (sum_p 256^p S_p), scaled by d * scale and accumulated per lane in FP32; minima use FP32 sums of x per sub-block:
// sum x (s q - m) = s sum(q x) - m sum(x).  The error of the fixed-point form is at most 2^-31 of the largest |x| per
// element, below the rounding of one FP32 product.
//
// Data movement.  A stage is 16 matrix rows x C super-blocks, copied block by block in 16-byte pieces (verbatim for the
// formats whose blocks are whole pieces; a 210-byte Q6_K block takes 14 pieces so that it starts on a piece boundary in
// LDS, the last piece overlapping the one before it): every wave requests its 1 KB pieces of a
// stage (consecutive memory, non-temporal 16-byte buffer loads) into one of two register sets and parks the set in one of
// two LDS stage buffers a whole stage later, so up to two stages are on their way while one is multiplied; one
// workgroup barrier per stage publishes the parked stage and frees the other buffer.  The LDS row stride is an odd
// number of 16-byte pieces, so the 16 rows an operand read touches fall into different bank groups.
//
// Work split.  Wave w of W owns super-block columns w (+ W) of every stage (a task = 16 rows x one super-block: eight
// MFMAs) and keeps its part of operand A for those columns in registers for as long as the activations stay the same;
// when they change, the digit planes pass once through the free stage buffer.  At the end of a 16-row tile the four
// quarters are added across lanes, the W wave partials go through LDS and 16 lanes add them in wave order.  W and C depend
// on the storage type and in_w only, and a launch is a table of matrices that share both, worked through as one sequence
// of tiles dealt round-robin to the workgroups: a row's bits depend on its weights, in_w and the activation vector, never
// on out_w, on the other matrices of the launch or on its place in it.
#include <cmath>
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

// Launch geometry of the matrix-core mat-vec: a function of the storage type and in_w alone.
struct MfmaGeom {
    int waves;            // W
    int cols;             // C: super-block columns per stage (a multiple of W)
    int kchunks;          // stages per 16-row tile = ceil(nblocks / C)
    int row_pieces;       // LDS row stride of a stage in 16-byte pieces (odd)
    int stage_bytes;      // bytes of one stage (multiple of 1 KB)
    int stage_loads;      // 1 KB load instructions that fill a stage
    int loads_per_wave;   // ceil(stage_loads / W)
    int stages;           // LDS stage buffers (2)
    int tasks;            // M: super-block columns a wave owns per stage
    int one_set;          // 1: one register set on its way instead of two (stages of whole rows, see the kernel)
    size_t lds_bytes;     // the stage buffers
};

using MfmaEntry = MfmaTableEntry;     // one matrix of a launch (nnhip_internal.h)

struct MfmaArgs {
    const MfmaEntry* table;        // device table, one entry per matrix and input row
    int entries;
    int total_tiles;
    int in_w;
    int nblocks;                   // super-blocks per row
    uint32_t row_bytes;
    uint32_t row_pieces_magic;     // ceil(2^32 / row_pieces)
    uint32_t used_pieces_magic;    // ceil(2^32 / (cols * pieces per block)): the pieces of a stage row that are blocks
    int chunked;                   // 1: a workgroup takes a run of consecutive tiles, 0: every G-th tile
    MfmaGeom g;
};

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
};

// One task of a storage format: 16 rows x one super-block.  `blk` is this lane's row of the stage at the task's block
// column (LDS).  Adds this lane's share (quarter lane / 16 of row lane % 16) to accq (the quant part, still in
// fixed-point units) and accm (the minimum part).
struct Q4KTask {
    static constexpr int kBlockBytes = kQ4KBytes;     // 144 = 9 pieces; blocks and rows are 16-byte aligned
    static constexpr int kLdsTableBytes = 0;          // no lookup tables in LDS
    static constexpr int kPieces = 9;                 // 16-byte pieces a block takes in a stage
    static constexpr bool kWholePieces = true;        // a row of blocks is a row of pieces, nothing else
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
    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float* sums, int b, int quarter, const uint8_t* zeros)
    {
        const uint8_t* src = zeros ? zeros : plane + 256 * b + 64 * quarter;
#pragma unroll
        for (int u = 0; u < 4; ++u) xs.a[u] = lds128(src + 16 * u);
        const float2 v = *reinterpret_cast<const float2*>(sums + 8 * b + 2 * quarter);
        xs.sx[0] = v.x;
        xs.sx[1] = v.y;
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
        accq = fmaf(d * ubyte0(sc), recombine(s_lo), accq);
        accq = fmaf(d * ubyte1(sc), recombine(s_hi), accq);
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
    static constexpr bool kWholePieces = true;
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

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float* sums, int b, int quarter, const uint8_t* zeros)
    {
        Q4KTask::load_x(xs, plane, sums, b, quarter, zeros);
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
        accq = fmaf(d * ubyte0(sc), recombine(s_lo), accq);
        accq = fmaf(d * ubyte1(sc), recombine(s_hi), accq);
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

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float* sums, int b, int quarter, const uint8_t* zeros)
    {
        const int h = quarter >> 1, e = quarter & 1;
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
        accq = fmaf(d * c0, recombine(s0), accq);
        accq = fmaf(d * c1, recombine(s1), accq);
        accq = fmaf(d * c2, recombine(s2), accq);
        accq = fmaf(d * c3, recombine(s3), accq);
        const float t = fmaf(c0, xs.sx[0], fmaf(c1, xs.sx[1], fmaf(c2, xs.sx[2], c3 * xs.sx[3])));
        accm = fmaf(32.0f * d, t, accm);
    }

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
        accq = fmaf(d * c0, recombine(s0), accq);
        accq = fmaf(d * c1, recombine(s1), accq);
        accq = fmaf(d * c2, recombine(s2), accq);
        accq = fmaf(d * c3, recombine(s3), accq);
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

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float*, int b, int quarter, const uint8_t* zeros)
    {
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
        accq = fmaf(half_bits_to_float(r.w[0]), recombine(s0), accq);
        accq = fmaf(half_bits_to_float(r.w[8] >> 16), recombine(s1), accq);
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

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float*, int b, int quarter, const uint8_t* zeros)
    {
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
        i32x4 total = {0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int factor = static_cast<int>(2u * ((r.scales >> (4 * k)) & 15u) + 1u);    // nibble k & 1 of scale byte k >> 1
#pragma unroll
            for (int p = 0; p < 4; ++p) total[p] += mul24(factor, acc[k][p]);     // (24-bit operands: v_mad_i32_i24, not the quarter-rate 32-bit multiply)
        }
        accq = fmaf(half_bits_to_float(r.d) * 0.125f, recombine_wide(total), accq);
    }

    static __device__ __forceinline__ void run(const Raw& r, const X& xs, int, const uint8_t* tables, float& accq, float&)
    {
        // every lookup of the task is requested before the first result is used (the scheduling barrier keeps the
        // compiler from folding the reads back into a chain of eight round trips to LDS)
        Looked lk;
        float unused = 0.0f;
        lookup(r, 0, tables, lk);
        __builtin_amdgcn_sched_barrier(0);
        finish(r, lk, xs, accq, unused);
    }
};

// IQ3_S (NNtrain.Arc/Kernels/qwen35_iq.cl:421-429): 110 bytes = d (fp16), 64 index bytes, 8 bytes of ninth index bits (one
// per four weights), 32 sign bytes, 4 bytes of 4-bit scales (one per 32 weights).  Four weights are one entry of a
// 512-entry codebook of magnitude bytes (odd, 1 .. 15); w = d * (1 + 2 scale) * magnitude * sign.  Two entries are the
// eight bytes of operand B that a lane supplies for one MFMA, and one sign byte covers them: the signs go in as for IQ2_S
// (IQ2STask), with the same 256-entry selector table.  Both tables sit in LDS (4 KB).  Quarter P = 32-weight groups 2P and
// 2P + 1: sixteen index bytes, two bytes of ninth bits, eight sign bytes, one scale byte.  Blocks are 2-byte aligned and
// fetched like IQ2_S blocks, from the dword boundary at or below their start, into seven pieces.
__device__ const uint32_t g_iq3s_grid_mv[512] = { NNHIP_IQ3S_GRID_VALUES };

struct IQ3STask {
    static constexpr int kBlockBytes = 110;
    static constexpr bool kStacked = false;
    static constexpr int kPieces = 7;
    static constexpr int kSumRun = 32;
    static constexpr int kWideM = 2;
    static constexpr int kWideLpw = 4;
    static constexpr int kSharedM = 1;
    static constexpr int kSharedLpw = 2;
    static constexpr bool kNeedsSums = false;         // no minimum or offset
    static constexpr bool kTightStage = true;
    static constexpr int kGridBytes = 2048;
    static constexpr int kTableBytes = kGridBytes + 2048;     // the codebook and 256 selector pairs
    static constexpr int kLdsTableBytes = kTableBytes;
    using X = XSet<1>;
    struct Raw { uint32_t q[4], s[2], tops, scales, d; };

    static __device__ __forceinline__ uint32_t piece_src(uint32_t q, bool odd) { return 16u * q - (odd ? 2u : 0u); }

    static __device__ __forceinline__ void init_tables(uint8_t* t, int tid, int threads)
    {
        for (int i = tid; i < 512; i += threads) reinterpret_cast<uint32_t*>(t)[i] = g_iq3s_grid_mv[i];
        for (int i = tid; i < 256; i += threads) {
            const uint32_t lo = ((static_cast<uint32_t>(i) & 15u) * 0x00204081u) & 0x01010101u;
            const uint32_t hi = ((static_cast<uint32_t>(i) >> 4) * 0x00204081u) & 0x01010101u;
            reinterpret_cast<u32x2*>(t + kGridBytes)[i] = u32x2{0x03020100u + (lo << 2), 0x03020100u + (hi << 2)};
        }
    }

    static __device__ __forceinline__ void load_x(X& xs, const uint8_t* plane, const float*, int b, int quarter, const uint8_t* zeros)
    {
        const uint8_t* src = zeros ? zeros : plane + 256 * b + 64 * quarter;
#pragma unroll
        for (int u = 0; u < 4; ++u) xs.a[u] = lds128(src + 16 * u);
        xs.sx[0] = 0.0f;
    }

    static __device__ __forceinline__ Raw load(const uint8_t* blk, int quarter, bool odd)
    {
        // the block's byte k is at blk + k (+ 2 when odd); its index bytes 16P .. 16P + 15 start at 2 + 16P, the sign bytes
        // 8P .. 8P + 7 at 74 + 8P: on dword boundaries in an odd block, two bytes past one in an even block
        const uint32_t* qi = reinterpret_cast<const uint32_t*>(blk + 16 * quarter + (odd ? 4 : 0));
        const uint32_t* si = reinterpret_cast<const uint32_t*>(blk + 8 * quarter + (odd ? 76 : 72));
        const uint32_t sh = odd ? 0u : 2u;
        const uint8_t* b0 = blk + (odd ? 2 : 0);
        Raw r;
        const uint32_t q0 = qi[0], q1 = qi[1], q2 = qi[2], q3 = qi[3], q4 = qi[4];
        const uint32_t s0 = si[0], s1 = si[1], s2 = si[2];
        r.q[0] = __builtin_amdgcn_alignbyte(q1, q0, sh);
        r.q[1] = __builtin_amdgcn_alignbyte(q2, q1, sh);
        r.q[2] = __builtin_amdgcn_alignbyte(q3, q2, sh);
        r.q[3] = __builtin_amdgcn_alignbyte(q4, q3, sh);
        r.s[0] = __builtin_amdgcn_alignbyte(s1, s0, sh);
        r.s[1] = __builtin_amdgcn_alignbyte(s2, s1, sh);
        r.tops = *reinterpret_cast<const uint16_t*>(b0 + 66 + 2 * quarter);
        r.scales = b0[106 + quarter];
        r.d = *reinterpret_cast<const uint16_t*>(b0);
        return r;
    }

    // As for IQ2_S: the lookups of a task are made once and every input row of a shared pass multiplies with them.
    static constexpr bool kSplitLookups = true;
    struct Looked { u32x2 mag[8], sel[8]; };

    static __device__ __forceinline__ void lookup(const Raw& r, int, const uint8_t* tables, Looked& lk)
    {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            // MFMA e of the quarter: codebook entries 2e and 2e + 1 (index byte + its ninth bit, bit 2e / 2e + 1 of the tops)
            const uint32_t word = r.q[e >> 1];
            const uint32_t i0 = ((word >> (16 * (e & 1))) & 0xffu) | (((r.tops >> (2 * e)) & 1u) << 8);
            const uint32_t i1 = ((word >> (16 * (e & 1) + 8)) & 0xffu) | (((r.tops >> (2 * e + 1)) & 1u) << 8);
            const uint32_t sign = (r.s[e >> 2] >> (8 * (e & 3))) & 0xffu;
            lk.mag[e] = u32x2{*reinterpret_cast<const uint32_t*>(tables + 4u * i0), *reinterpret_cast<const uint32_t*>(tables + 4u * i1)};
            lk.sel[e] = *reinterpret_cast<const u32x2*>(tables + kGridBytes + 8u * sign);
        }
    }

    static __device__ __forceinline__ void finish(const Raw& r, const Looked& lk, const X& xs, float& accq, float&)
    {
        i32x4 acc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            // -m per byte = (m ^ 0xff) + 1: no carry leaves a byte because no magnitude is zero
            const uint32_t neg0 = (lk.mag[e][0] ^ 0xffffffffu) + 0x01010101u, neg1 = (lk.mag[e][1] ^ 0xffffffffu) + 0x01010101u;
            const uint32_t b0 = __builtin_amdgcn_perm(neg0, lk.mag[e][0], lk.sel[e][0]);
            const uint32_t b1 = __builtin_amdgcn_perm(neg1, lk.mag[e][1], lk.sel[e][1]);
            const u32x4 av = xs.a[e >> 1];
            acc[e >> 2] = mfma_i8(av[2 * (e & 1)], av[2 * (e & 1) + 1], b0, b1, acc[e >> 2]);
        }
        // the plane sums of the two scale groups are added up with the integer factors 1 + 2 s (|sum| < 2 * 31 * 32 * 15 *
        // 128 < 2^22: exact) and recombined once
        const int f0 = static_cast<int>(1u + 2u * (r.scales & 15u)), f1 = static_cast<int>(1u + 2u * ((r.scales >> 4) & 15u));
        i32x4 total;
#pragma unroll
        for (int p = 0; p < 4; ++p) total[p] = mul24(f0, acc[0][p]) + mul24(f1, acc[1][p]);
        accq = fmaf(half_bits_to_float(r.d), recombine_wide(total), accq);
    }

    static __device__ __forceinline__ void run(const Raw& r, const X& xs, int, const uint8_t* tables, float& accq, float&)
    {
        Looked lk;
        float unused = 0.0f;
        lookup(r, 0, tables, lk);
        __builtin_amdgcn_sched_barrier(0);
        finish(r, lk, xs, accq, unused);
    }
};

template <class F, class = void> struct WholePieces { static constexpr bool value = false; };
template <class F> struct WholePieces<F, std::enable_if_t<F::kWholePieces>> { static constexpr bool value = true; };

// Loads of the weight stream: 16 bytes per lane through a buffer descriptor that spans the matrix, non-temporal.  An
// offset beyond the buffer returns zeros without touching memory.
__device__ __forceinline__ u32x4 stream16(__amdgpu_buffer_rsrc_t matrix, uint32_t off)
{
    return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(matrix, static_cast<int>(off), 0, 2));
}

// grid.x = workgroups striding over the launch's 16-row tiles, blockDim.x = 64 * W.  KC = stages per tile (1 or 2),
// M = super-block columns a wave owns per stage, LPW = 1 KB pieces of a stage a wave moves.  A lane keeps operand A of its KC * M columns in registers for as long as the activations stay
// the same.
// ONESET (stages of whole rows, two columns per wave, for the formats whose unpacking leaves no registers for two sets):
// a wave has one set of pieces on its way.  It parks the set at the end of a stage and asks for the stage after next
// into the same registers, so one stage (as many bytes as two half-row stages) travels while one is multiplied.
template <class F, int KC, int M, int LPW, bool ONESET = false>
__global__ __launch_bounds__(64 * kMaxWaves) void matvec_mfma_kernel(MfmaArgs a)
{
    static_assert(KC == 1 || KC == 2, "a turn of the two register sets is one or two tiles");
    static_assert(!ONESET || KC == 1, "one register set is for stages of whole rows");
    // A stage of whole rows of whole pieces is one run of memory: the wave's 1 KB requests are then cut on 1 KB
    // boundaries of the tile (whole 128-byte lines, each asked for once; cut by the padded LDS rows instead, one request
    // in ten shares a line with its neighbour's and 1 % of the lines came in twice), and each lane parks its piece at
    // the padded place.
    constexpr bool kLinear = KC == 1 && WholePieces<F>::value;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    __shared__ float part[2][kMaxWaves][kTileRows];
    __shared__ uint32_t red[kMaxWaves];
    __shared__ __attribute__((aligned(16))) uint8_t zero_area[256];       // operand A outside the block diagonal

    const MfmaGeom& g = a.g;
    const int tid = threadIdx.x, lane = tid & 63, T = blockDim.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int W = g.waves;
    const int row_l = lane & 15, quarter = lane >> 4;

    // The table is read-only for the whole launch and indexed with workgroup-uniform values: through the constant
    // address space those reads are scalar loads, which do not touch the vector-memory counter.
    const NNHIP_CONST_PTR MfmaEntry* table = (const NNHIP_CONST_PTR MfmaEntry*)a.table;
    auto entry_at = [&](int m) {
        const NNHIP_CONST_PTR MfmaEntry& t = table[m];
        MfmaEntry e;
        e.x = t.x;
        e.w = t.w;
        e.bias = t.bias;
        e.y = t.y;
        e.out_w = t.out_w;
        e.w_bytes = t.w_bytes;
        e.tiles = t.tiles;
        e.first_tile = t.first_tile;
        return e;
    };

    // ---- this lane's pieces of a stage: piece I = wave + W * i is slots 64 I .. 64 I + 63 of the stage; slot s is
    // 16-byte piece s % row_pieces of stage row s / row_pieces: piece q % kPieces of block q / kPieces (the last piece of
    // a row is padding when the blocks take an even number of pieces).  rel[i] is the piece's byte offset from the stage's first byte in the matrix; pieces that do
    // not exist get an offset beyond any matrix and read as zeros.
    const int pieces_used = g.cols * F::kPieces;
    uint32_t rel[LPW];
    uint32_t lds_at[kLinear ? LPW : 1];      // kLinear: where the piece is parked (kNoPiece: nowhere)
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const uint32_t slot = static_cast<uint32_t>(64 * (wave + W * i) + lane);
        if constexpr (kLinear) {
            const uint32_t r = __umulhi(slot, a.used_pieces_magic);
            const uint32_t q = slot - r * static_cast<uint32_t>(pieces_used);
            const bool real = r < static_cast<uint32_t>(kTileRows);
            rel[i] = real ? 16u * slot : kNoPiece;
            lds_at[i] = real ? 16u * (r * static_cast<uint32_t>(g.row_pieces) + q) : kNoPiece;
        } else {
            const uint32_t r = __umulhi(slot, a.row_pieces_magic);
            const uint32_t q = slot - r * static_cast<uint32_t>(g.row_pieces);
            const uint32_t c = q / static_cast<uint32_t>(F::kPieces);
            const bool real = r < static_cast<uint32_t>(kTileRows) && q < static_cast<uint32_t>(pieces_used);
            rel[i] = real ? r * a.row_bytes + c * F::kBlockBytes + F::piece_src(q - c * F::kPieces, c & 1u) : kNoPiece;
        }
    }

    // ---- the stage sequence of this workgroup: tiles blockIdx.x, blockIdx.x + G, ... of the launch's tile sequence,
    // KC stages per tile
    const int G = gridDim.x, bid = blockIdx.x;
    int my_tiles, t_first, t_step;
    if (a.chunked) {
        const int per = a.total_tiles / G, rem = a.total_tiles - per * G;
        my_tiles = per + (bid < rem ? 1 : 0);
        t_first = bid * per + (bid < rem ? bid : rem);
        t_step = 1;
    } else {
        my_tiles = (a.total_tiles - bid + G - 1) / G;
        t_first = bid;
        t_step = G;
    }
    const int t_end = a.chunked ? t_first + my_tiles : a.total_tiles;       // no requests from here on
    const int total = my_tiles * KC;
    const uint32_t chunk_bytes = static_cast<uint32_t>(g.cols) * F::kBlockBytes;
    const int n4 = a.in_w >> 2;

    // ---- prefetch side: the stage it requests next, the matrix that stage belongs to
    // float4 per lane that hold the next matrix' activations on their way in: in_w = KC * M * W * 256 floats over 64 W lanes
    constexpr int kXRegs = KC * M;
    float4 xv[kXRegs];
    int xv_m = -1;                         // the table entry whose activations are in xv (or on their way)
    int f_t = t_first, f_k = 0, f_m = 0;
    if (a.chunked && my_tiles > 0) {       // the entry that holds the run's first tile
        int lo = 0, hi = a.entries - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (table[mid].first_tile <= t_first) lo = mid;
            else hi = mid - 1;
        }
        f_m = lo;
    }
    const int m_first = f_m;
    MfmaEntry fe = entry_at(f_m);
    const float* f_x = nullptr;            // vector of the matrix the prefetch side was in last
    __amdgpu_buffer_rsrc_t f_matrix;
    auto request_x = [&](const float* x, int m) {
        const float4* x4 = reinterpret_cast<const float4*>(x);
#pragma unroll
        for (int j = 0; j < kXRegs; ++j) {
            const int i = tid + j * T;
            xv[j] = x4[i < n4 ? i : 0];
        }
        xv_m = m;
    };
    auto fetch_enter = [&]() {             // f_t moved: find its matrix; ask for its activations if they are new
        while (f_t >= fe.first_tile + fe.tiles && f_m + 1 < a.entries) fe = entry_at(++f_m);
        f_matrix = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(fe.w), 0, static_cast<int>(fe.w_bytes), 0x00020000);
        if (fe.x != f_x) {
            // only one vector can be on its way; a second change before the first was consumed is fetched at the switch
            if (xv_m < 0) request_x(fe.x, f_m);
            f_x = fe.x;
        }
    };
    // Requests this wave's pieces of the next stage into a register set.  Pieces that are padding, rows past the matrix
    // and stages past the end lie beyond the buffer: zeros, no memory traffic.
    auto fetch = [&](u32x4 (&set)[LPW]) {
        const uint32_t base = f_t < t_end
            ? static_cast<uint32_t>(f_t - fe.first_tile) * kTileRows * a.row_bytes + static_cast<uint32_t>(f_k) * chunk_bytes
            : kNoPiece;
#pragma unroll
        for (int i = 0; i < LPW; ++i) set[i] = stream16(f_matrix, base + rel[i]);
        if (++f_k == KC) {
            f_k = 0;
            f_t += t_step;
            if (f_t < t_end && f_t >= fe.first_tile + fe.tiles) fetch_enter();
        }
    };
    // Copies a register set to its place in an LDS stage buffer.
    auto park = [&](uint8_t* buf, const u32x4 (&set)[LPW]) {
        // (a buffer has room for all W * LPW pieces; those past the stage's last are zeros nobody reads)
        uint8_t* dst = buf + wave * 1024 + lane * 16;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            if constexpr (kLinear) {
                if (lds_at[i] != kNoPiece) *reinterpret_cast<u32x4*>(buf + lds_at[i]) = set[i];
            } else {
                // (ONESET: the buffers end with the stage's last piece)
                if (!ONESET || wave + W * i < g.stage_loads) *reinterpret_cast<u32x4*>(dst + W * i * 1024) = set[i];
            }
        }
    };

    // ---- consume side
    int c_t = t_first, c_m = m_first - 1;
    MfmaEntry ce{};
    float inv = 0.0f;
    const float* regs_x = nullptr;         // the vector operand A in the registers below was made from
    typename F::X xs[KC * M];
    // Operand A of this lane: A row lane % 16 = plane (lane % 4) of quarter (lane % 16) / 4, K group lane / 16; it is
    // non-zero only where the K group carries that quarter.
    const bool diag = (row_l >> 2) == quarter;
    if (tid < 64) reinterpret_cast<uint32_t*>(zero_area)[tid] = 0u;      // (published by the barrier after the first parking)
    const uint8_t* const a_zeros = diag ? nullptr : zero_area;

    // Turns matrix c_m's activations into this lane's operand-A registers (all waves; three barriers inside).  The digit
    // planes and sub-block sums pass through the stage buffer `scratch`, which is free at that point.  The vector is in xv
    // when the prefetch side asked for it; otherwise it is fetched here.
    auto prepare_x = [&](uint8_t* scratch) {
        if (xv_m != c_m) request_x(ce.x, c_m);
        xv_m = -1;
        constexpr float4 kZero4 = {0.0f, 0.0f, 0.0f, 0.0f};
        const int plane_stride = a.in_w + 16;
        float* sumx = reinterpret_cast<float*>(scratch + 4 * plane_stride);
        auto umax4 = [](uint32_t m, const float4& v) {
            m = umax_u(m, __float_as_uint(v.x) & 0x7fffffffu);
            m = umax_u(m, __float_as_uint(v.y) & 0x7fffffffu);
            m = umax_u(m, __float_as_uint(v.z) & 0x7fffffffu);
            return umax_u(m, __float_as_uint(v.w) & 0x7fffffffu);
        };
        uint32_t mx = 0;
#pragma unroll
        for (int j = 0; j < kXRegs; ++j) {
            if (tid + j * T >= n4) xv[j] = kZero4;
            mx = umax4(mx, xv[j]);
        }
        mx = wave_umax(mx);
        if (lane == 0) red[wave] = mx;
        __syncthreads();
        mx = 0;
        for (int i = 0; i < W; ++i) mx = umax_u(mx, red[i]);
        // |x| < 2^(E - 126) for the biased exponent E of the largest magnitude; e = 156 - E puts it below 2^30
        const int E = static_cast<int>(mx >> 23);
        int e = 156 - E;
        e = e > 126 ? 126 : e;
        const float scale = __uint_as_float(static_cast<uint32_t>(e + 127) << 23);
        // a NaN or an infinity among the activations makes every output NaN
        inv = E == 255 ? __uint_as_float(0x7fc00000u) : __uint_as_float(static_cast<uint32_t>(127 - e) << 23);
        auto to_planes = [&](int i, const float4& v) {
            uint32_t pl[4];
            digit_planes(__float2int_rn(v.x * scale), __float2int_rn(v.y * scale), __float2int_rn(v.z * scale),
                         __float2int_rn(v.w * scale), pl);
#pragma unroll
            for (int p = 0; p < 4; ++p) *reinterpret_cast<uint32_t*>(scratch + p * plane_stride + 4 * i) = pl[p];
            float s = (v.x + v.y) + (v.z + v.w);
            if (F::kSumRun == 32) {                                  // 32 consecutive activations: one sub-block
                s = oct_sum(s);
                if ((i & 7) == 0) sumx[i >> 3] = s;
            } else {                                                 // 16 consecutive activations
                s += dpp_mov<0xB1>(s);
                s += dpp_mov<0x4E>(s);
                if ((i & 3) == 0) sumx[i >> 2] = s;
            }
        };
#pragma unroll
        for (int j = 0; j < kXRegs; ++j) {
            const int i = tid + j * T;                               // (whole groups of eight lanes are in or out: n4 % 8 == 0)
            if (i < n4) to_planes(i, xv[j]);
        }
        __syncthreads();
        // set k * M + t = super-block column k * cols + t * W + wave of a row
#pragma unroll
        for (int k = 0; k < KC; ++k) {
#pragma unroll
            for (int t = 0; t < M; ++t) {
                const int b = k * g.cols + t * W + wave;
                F::load_x(xs[k * M + t], scratch + (row_l & 3) * plane_stride, sumx, b, quarter, a_zeros);
            }
        }
        regs_x = ce.x;
        __syncthreads();
    };

    // ---- start: the first matrix' activations are requested ahead of the weight stream, then two stages
    uint8_t* const buf0 = smem;
    uint8_t* const buf1 = smem + g.stage_bytes;
    // (a third register set, three stages on their way, was measured without gain)
    u32x4 regs[ONESET ? 1 : 2][LPW];
    fetch_enter();
    fetch(regs[0]);
    if constexpr (!ONESET) fetch(regs[1]);

    const uint32_t row_off = static_cast<uint32_t>(row_l) * (static_cast<uint32_t>(g.row_pieces) * 16u) +
                             static_cast<uint32_t>(wave) * (16u * F::kPieces);
    int pbuf = 0;
    // the tile whose wave partials sit in part[pbuf ^ 1]: added up and stored after the next barrier
    bool done = false;
    float* done_y = nullptr;
    const float* done_bias = nullptr;
    int done_row0 = 0, done_rows = 0;
    auto finalize = [&]() {
        if (tid < kTileRows) {
            float t = 0.0f;
            for (int w2 = 0; w2 < W; ++w2) t += part[pbuf ^ 1][w2][tid];
            if (done_bias) {
                // the 16 bias values come through the scalar cache (wave-uniform addresses) and are dealt to the lanes
                const NNHIP_CONST_PTR float* cb = (const NNHIP_CONST_PTR float*)done_bias + done_row0;
                float bv = 0.0f;
#pragma unroll
                for (int j = 0; j < kTileRows; ++j) {
                    const float v = cb[j < done_rows ? j : 0];
                    bv = tid == j ? v : bv;
                }
                t += bv;
            }
            if (tid < done_rows) done_y[done_row0 + tid] = t;
        }
        done = false;
    };

    float accq = 0.0f, accm = 0.0f;
    // One stage: buffer `cur` holds it; `nxt` receives the stage after it from `landing`, whose loads have been in
    // flight for a whole stage; `refill` (free since it was parked a stage ago) takes the requests of the stage after that.
    auto stage_step = [&](auto k_tag, uint8_t* cur, uint8_t* nxt, u32x4 (&refill)[LPW], const u32x4 (&landing)[LPW]) {
        constexpr int k = decltype(k_tag)::value;
        bool new_x = false;
        if (k == 0) {
            if (c_t >= ce.first_tile + ce.tiles) {              // (always at the first tile: ce.tiles == 0)
                while (c_t >= ce.first_tile + ce.tiles) ce = entry_at(++c_m);
                new_x = ce.x != regs_x;
            }
        }
        if constexpr (!ONESET) fetch(refill);      // (before the activations are dealt with: the stream must not pause for them)
        if (k == 0 && new_x) prepare_x(nxt);
        if (done) finalize();
        const uint8_t* stage = cur + row_off;
        typename F::Raw raw[M];
#pragma unroll
        for (int t = 0; t < M; ++t) raw[t] = F::load(stage + t * W * (16 * F::kPieces), quarter, (wave & 1) != 0);
#pragma unroll
        for (int t = 0; t < M; ++t) F::run(raw[t], xs[k * M + t], quarter, nullptr, accq, accm);
        if (k == KC - 1) {
            float p = fmaf(accq, inv, -accm);
            p = quarter_sum(p);
            if (lane < kTileRows) part[pbuf][wave][lane] = p;
            accq = 0.0f;
            accm = 0.0f;
            done = true;
            done_y = ce.y;
            done_bias = ce.bias;
            done_row0 = (c_t - ce.first_tile) * kTileRows;
            done_rows = ce.out_w - done_row0 < kTileRows ? ce.out_w - done_row0 : kTileRows;
            pbuf ^= 1;
            c_t += t_step;
        }
        park(nxt, landing);
        if constexpr (ONESET) fetch(refill);
        __syncthreads();                // publishes `nxt`, frees `cur`
    };

    park(buf0, regs[0]);
    if constexpr (ONESET) fetch(regs[0]);
    __syncthreads();
    using std::integral_constant;
    for (int n = 0; n < total; n += 2) {
        stage_step(integral_constant<int, 0>{}, buf0, buf1, regs[0], regs[ONESET ? 0 : 1]);
        if (n + 1 < total) stage_step(integral_constant<int, KC - 1>{}, buf1, buf0, regs[ONESET ? 0 : 1], regs[0]);
    }
    if (done) finalize();
}


// ---------------------------------------------------------------------------------------------------- the wide form
// The same mat-vec for rows that do not split into one or two whole stages (17408 = 68 super-blocks) and for calls
// with 2 - 4 input rows that share one pass over the weights: the digit planes of the activations stay in LDS for as
// long as the vector is the same and a lane reads its 64 bytes of operand A for every task (instead of keeping them in
// registers), a tile takes ceil(nblocks / W) stages of W block columns, the last one partly empty, and a task multiplies
// the unpacked quants with the operand A of every input row of the entry.  Rows, planes and results of input row r of
// an entry are x + r * in_w, the r-th plane set and y + r * out_w.
template <class F, class = void> struct SplitLookups { static constexpr bool value = false; };
template <class F> struct SplitLookups<F, std::enable_if_t<F::kSplitLookups>> { static constexpr bool value = true; };

struct WideGeom {
    int waves;            // W (even: block parity is wave parity)
    int cols;             // block columns per stage = W * M
    int kchunks;          // stages per tile = ceil(nblocks / cols)
    int tail_cols;        // block columns of a tile's last stage
    int row_pieces;       // LDS row stride of a stage in 16-byte pieces (odd)
    int stage_bytes;
    int plane_stride;     // bytes of one digit plane (in_w + 16)
    int set_bytes;        // four planes and the sums of one input row
    int single;           // 1: one stage buffer that holds whole tiles (kchunks == 1, cols == nblocks)
    size_t lds_bytes;     // the stage buffers and R plane sets
};

struct WideArgs {
    const MfmaEntry* table;        // device table, or null: the entries are `inline_entries` below
    int entries;
    int total_tiles;
    int in_w;
    int nblocks;
    uint32_t row_bytes;
    uint32_t row_pieces_magic;
    int chunked;                   // 1: a workgroup takes consecutive tiles (few changes of activations), 0: every G-th
    int parts, part_stages;        // SPLIT: a row's stages are taken in `parts` groups of `part_stages` (see the kernel)
    int run_tiles;                 // SPLIT: most tiles of a run (their sums wait in LDS from part to part, behind the planes)
    WideGeom g;
    MfmaEntry inline_entries[4];   // a call with up to 16 input rows needs no table in device memory
};

// SPLIT: a run is as long as the LDS the geometry leaves over holds sums for, up to this many tiles
constexpr int kSplitRunMax = 64;

// SPLIT (rows too long for R full sets of planes in LDS): the stages of a tile are taken in `parts`
// groups of `part_stages`, and LDS holds the planes of one group of block columns at a time.  A workgroup works through
// a run of its tiles of a table entry (at most run_tiles of them) once per part: planes of part 0, that part of
// every tile, planes of part 1, ...; the sums of a tile wait in LDS (bias + part 0, + part 1, ...: one order, so the
// bits of a row depend on its weights, its activations and the launch geometry only) and are stored after the last part.
// Every stage of every tile is still requested and multiplied once; what is paid is a conversion of the activations
// per entry and workgroup, as before, now in `parts` pieces.
template <class F, int M, int LPW, int R, bool ONE = false, bool SPLIT = false>
__global__ __launch_bounds__(64 * kMaxWaves) void matvec_mfma_wide_kernel(WideArgs a)
{
    static_assert(!SPLIT || !ONE, "parts are for the form with two stage buffers");
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    __shared__ float part[2][R][kMaxWaves][kTileRows];
    __shared__ uint32_t red[R][kMaxWaves];
    __shared__ float inv_of_row[R];                                       // 2^-e of each input row's fixed-point scale
    __shared__ __attribute__((aligned(16))) uint8_t zero_area[256];       // operand A outside the block diagonal

    const WideGeom& g = a.g;
    const int tid = threadIdx.x, lane = tid & 63, T = blockDim.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int W = g.waves, KC = g.kchunks;
    const int row_l = lane & 15, quarter = lane >> 4;

    // (the kernel's only argument starts the kernel-argument segment, which is constant memory like the table)
    const NNHIP_CONST_PTR MfmaEntry* table =
        a.table ? (const NNHIP_CONST_PTR MfmaEntry*)a.table
                : (const NNHIP_CONST_PTR MfmaEntry*)((const NNHIP_CONST_PTR char*)__builtin_amdgcn_kernarg_segment_ptr() +
                                                     offsetof(WideArgs, inline_entries));
    auto entry_at = [&](int m) {
        const NNHIP_CONST_PTR MfmaEntry& t = table[m];
        MfmaEntry e;
        e.x = t.x;
        e.w = t.w;
        e.bias = t.bias;
        e.y = t.y;
        e.out_w = t.out_w;
        e.w_bytes = t.w_bytes;
        e.tiles = t.tiles;
        e.first_tile = t.first_tile;
        e.rows = t.rows;
        return e;
    };

    // this lane's pieces of a stage, as in the kernel above; in a tile's last stage the block columns past the row's
    // end fetch nothing
    uint32_t rel[LPW];
    uint32_t in_tail = 0;                  // bit i: this lane's piece i exists in a tile's last stage
    uint32_t in_stage = 0;                 // bit i: this lane's piece i lies inside the stage buffer
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const uint32_t slot = static_cast<uint32_t>(64 * (wave + W * i) + lane);
        const uint32_t r = __umulhi(slot, a.row_pieces_magic);
        const uint32_t q = slot - r * static_cast<uint32_t>(g.row_pieces);
        const uint32_t c = q / static_cast<uint32_t>(F::kPieces);
        const bool real = r < static_cast<uint32_t>(kTileRows) && c < static_cast<uint32_t>(g.cols);
        rel[i] = real ? r * a.row_bytes + c * F::kBlockBytes + F::piece_src(q - c * F::kPieces, c & 1u) : kNoPiece;
        in_tail |= (real && c < static_cast<uint32_t>(g.tail_cols) ? 1u : 0u) << i;
        in_stage |= (r < static_cast<uint32_t>(kTileRows) ? 1u : 0u) << i;
    }

    // ---- this workgroup's tiles of the launch's tile sequence: every G-th, or a run of consecutive ones.  Runs are for
    // launches whose matrices all have activations of their own (a workgroup then meets two or three vectors instead
    // of all of them); the bits of a row are the same either way.
    const int G = gridDim.x, bid = blockIdx.x;
    int my_tiles, t_first, t_step;
    if (a.chunked) {
        const int per = a.total_tiles / G, rem = a.total_tiles - per * G;
        my_tiles = per + (bid < rem ? 1 : 0);
        t_first = bid * per + (bid < rem ? bid : rem);
        t_step = 1;
    } else {
        my_tiles = (a.total_tiles - bid + G - 1) / G;
        t_first = bid;
        t_step = G;
    }
    const int t_end = a.chunked ? t_first + my_tiles : a.total_tiles;       // no requests from here on
    const int total = my_tiles * KC;
    const uint32_t chunk_bytes = static_cast<uint32_t>(g.cols) * F::kBlockBytes;

    // SPLIT: a run of this workgroup's tiles that starts at tile `first` ends with the entry, with the workgroup's tiles,
    // or after run_tiles tiles
    auto run_end = [&](int first, int entry_end) {
        int e = entry_end < t_end ? entry_end : t_end;
        const int cap = first + a.run_tiles * t_step;
        return e < cap ? e : cap;
    };
    // ---- prefetch side
    int f_t = t_first, f_k = 0, f_m = 0;
    int f_p = 0, f_first = t_first;                      // SPLIT: part and first tile of the run of tiles of one entry
    if (a.chunked && my_tiles > 0) {
        // the entry that holds this workgroup's first tile: the last one whose first_tile is not beyond it (a run may
        // start hundreds of entries into the table, and walking there costs a trip to memory per entry)
        int lo = 0, hi = a.entries - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (table[mid].first_tile <= t_first) lo = mid;
            else hi = mid - 1;
        }
        f_m = lo;
    }
    const int m_first = f_m;
    MfmaEntry fe = entry_at(f_m);
    __amdgpu_buffer_rsrc_t f_matrix;
    auto fetch_enter = [&]() {
        while (f_t >= fe.first_tile + fe.tiles && f_m + 1 < a.entries) fe = entry_at(++f_m);
        f_matrix = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(fe.w), 0, static_cast<int>(fe.w_bytes), 0x00020000);
    };
    auto fetch = [&](u32x4 (&set)[LPW]) {
        const uint32_t base = f_t < t_end
            ? static_cast<uint32_t>(f_t - fe.first_tile) * kTileRows * a.row_bytes + static_cast<uint32_t>(f_k) * chunk_bytes
            : kNoPiece;
        const bool tail = f_k == KC - 1;
#pragma unroll
        for (int i = 0; i < LPW; ++i) set[i] = stream16(f_matrix, tail && !((in_tail >> i) & 1u) ? kNoPiece : base + rel[i]);
        if constexpr (SPLIT) {
            const int part_end = (f_p + 1) * a.part_stages < KC ? (f_p + 1) * a.part_stages : KC;
            if (++f_k == part_end) {
                f_t += t_step;
                if (f_t < run_end(f_first, fe.first_tile + fe.tiles)) {      // the same part of the entry's next tile
                    f_k = f_p * a.part_stages;
                } else if (f_p + 1 < a.parts) {          // the next part, from the run's first tile again
                    ++f_p;
                    f_t = f_first;
                    f_k = f_p * a.part_stages;
                } else {                                 // the next entry
                    f_p = 0;
                    f_first = f_t;
                    f_k = 0;
                    if (f_t < t_end) fetch_enter();
                }
            }
        } else if (++f_k == KC) {
            f_k = 0;
            f_t += t_step;
            if (f_t < t_end && f_t >= fe.first_tile + fe.tiles) fetch_enter();
        }
    };
    auto park = [&](uint8_t* buf, const u32x4 (&set)[LPW]) {
        // (where LDS is tight a stage buffer ends with the stage's last row and the slots behind it are not stored)
        uint8_t* dst = buf + wave * 1024 + lane * 16;
#pragma unroll
        for (int i = 0; i < LPW; ++i)
            if (!F::kTightStage || ((in_stage >> i) & 1u)) *reinterpret_cast<u32x4*>(dst + W * i * 1024) = set[i];
    };

    // ---- consume side
    // The format's lookup tables are a static array: its address is a constant of the program, so a table read takes its
    // base from the instruction's offset field instead of an addition per lookup (sixteen per IQ2_S task).
    __shared__ __attribute__((aligned(16))) uint8_t table_area[F::kLdsTableBytes > 0 ? F::kLdsTableBytes : 16];
    uint8_t* const tables = table_area;                    // (published by the first barrier)
    uint8_t* const buf0 = smem;
    uint8_t* const buf1 = smem + g.stage_bytes;            // (not with ONE: a single stage buffer)
    uint8_t* const planes = smem + (ONE ? 1 : 2) * g.stage_bytes;
    F::init_tables(tables, tid, T);
    int c_t = t_first, c_k = 0, c_m = m_first - 1;      // (ce.tiles == 0: the first stage enters entry m_first)
    // SPLIT: part, first tile and end of the run of this workgroup's tiles of one entry, the tile's number in the run
    // (the first stage of tile 0 of a part is where the part's planes have to be made)
    int c_p = 0, c_first = t_first, c_u = 0;
    MfmaEntry ce{};
    float inv[R] = {};
    const float* planes_x = nullptr;       // the vector(s) the planes in LDS were made from
    int planes_rows = 0;
    const bool diag = (row_l >> 2) == quarter;
    if (tid < 64) reinterpret_cast<uint32_t*>(zero_area)[tid] = 0u;      // (published by the barrier after the first parking)
    const uint8_t* const a_zeros = diag ? nullptr : zero_area;

    // Turns the activations of matrix c_m (its `rows` input rows) into digit planes and sums in LDS; two barriers.
    // Every wave has left the stage that last read the planes when this runs.  (Requesting the whole vector at once into
    // registers, one trip to memory instead of two, made the compiler wait for every outstanding load before each
    // parking write of the main loop in the one-row form: 12.6 instead of 8.6 us per 17408-wide Q4_K mat-vec.)
    // (SPLIT: of the block columns of part c_p only, x_first values into every input row)
    const int part_values = SPLIT ? a.part_stages * g.cols * 256 : 0;
    auto prepare_x = [&]() {
        const int x_first = SPLIT ? c_p * part_values : 0;
        const int n4 = SPLIT ? ((a.in_w - x_first < part_values ? a.in_w - x_first : part_values) >> 2) : (a.in_w >> 2);
        auto umax4 = [](uint32_t m, const float4& v) {
            m = umax_u(m, __float_as_uint(v.x) & 0x7fffffffu);
            m = umax_u(m, __float_as_uint(v.y) & 0x7fffffffu);
            m = umax_u(m, __float_as_uint(v.z) & 0x7fffffffu);
            return umax_u(m, __float_as_uint(v.w) & 0x7fffffffu);
        };
        const int rows = ce.rows;
        // With shared passes the rows are requested together when they fit kPrep float4 per lane (one trip to memory
        // instead of two per row: 1.5 us of a 30 us call); the one-row form keeps the loops (see above).
        // (Not with four tiles in flight per wave: the registers do not hold both.)
        constexpr int kPrep = R > 1 && LPW <= 3 && !SPLIT ? 8 : 0;      // (SPLIT: measured 8 % slower with it)
        if (kPrep > 0 && rows * n4 <= kPrep * T) {
            float4 xr[kPrep > 0 ? kPrep : 1];
            const float4* x4 = reinterpret_cast<const float4*>(ce.x);      // the rows are consecutive: x4[r * n4 + i]
            auto row_of = [&](int j) {                                      // wave-uniform (n4 % 64 == 0); -1 past the last row
                const int f0 = (tid & ~63) + j * T;
                const int r = (f0 >= n4) + (f0 >= 2 * n4) + (f0 >= 3 * n4);
                return f0 >= rows * n4 ? -1 : __builtin_amdgcn_readfirstlane(r);
            };
#pragma unroll
            for (int j = 0; j < kPrep; ++j) xr[j] = x4[row_of(j) >= 0 ? tid + j * T : 0];
            uint32_t mx[R] = {};
#pragma unroll
            for (int j = 0; j < kPrep; ++j) {
                const int rj = row_of(j);
                const uint32_t m = umax4(0u, xr[j]);
#pragma unroll
                for (int r = 0; r < R; ++r) mx[r] = rj == r ? umax_u(mx[r], m) : mx[r];
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r < rows) {
                    const uint32_t m = wave_umax(mx[r]);
                    if (lane == 0) red[r][wave] = m;
                }
            }
            __syncthreads();
            float scale[R] = {};
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r < rows) {
                    uint32_t m = 0;
                    for (int i = 0; i < W; ++i) m = umax_u(m, red[r][i]);
                    const int E = static_cast<int>(m >> 23);
                    int e = 156 - E;
                    e = e > 126 ? 126 : e;
                    scale[r] = __uint_as_float(static_cast<uint32_t>(e + 127) << 23);
                    inv[r] = E == 255 ? __uint_as_float(0x7fc00000u) : __uint_as_float(static_cast<uint32_t>(127 - e) << 23);
                    if (tid == 0) inv_of_row[r] = inv[r];
                }
            }
#pragma unroll
            for (int j = 0; j < kPrep; ++j) {
                const int rj = row_of(j);
                if (rj >= 0) {
                    float sc = scale[0];
#pragma unroll
                    for (int r = 1; r < R; ++r) sc = rj == r ? scale[r] : sc;
                    const int i = tid + j * T - rj * n4;
                    const float4 v = xr[j];
                    uint8_t* set = planes + rj * g.set_bytes;
                    float* sumx = reinterpret_cast<float*>(set + 4 * g.plane_stride);
                    uint32_t pl[4];
                    digit_planes(__float2int_rn(v.x * sc), __float2int_rn(v.y * sc), __float2int_rn(v.z * sc), __float2int_rn(v.w * sc), pl);
#pragma unroll
                    for (int p = 0; p < 4; ++p) *reinterpret_cast<uint32_t*>(set + p * g.plane_stride + 4 * i) = pl[p];
                    float s = (v.x + v.y) + (v.z + v.w);
                    if (!F::kNeedsSums) {
                    } else if (F::kSumRun == 32) {
                        s = oct_sum(s);
                        if ((i & 7) == 0) sumx[i >> 3] = s;
                    } else {
                        s += dpp_mov<0xB1>(s);
                        s += dpp_mov<0x4E>(s);
                        if ((i & 3) == 0) sumx[i >> 2] = s;
                    }
                }
            }
            planes_x = ce.x;
            planes_rows = rows;
            __syncthreads();
            return;
        }
        // (SPLIT: the largest magnitudes are those of the whole rows, taken where a run begins and kept in `red` for its
        // other parts: one trip to memory per part instead of two, and one fixed-point scale per input row)
        if (!SPLIT || c_p == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r < rows) {
                    const float4* x4 = reinterpret_cast<const float4*>(ce.x + static_cast<size_t>(r) * a.in_w);
                    const int n4_max = SPLIT ? a.in_w >> 2 : n4;
                    uint32_t mx = 0;
                    for (int i = tid; i < n4_max; i += T) mx = umax4(mx, x4[i]);
                    mx = wave_umax(mx);
                    if (lane == 0) red[r][wave] = mx;
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r < rows) {
                uint32_t mx = 0;
                for (int i = 0; i < W; ++i) mx = umax_u(mx, red[r][i]);
                // |x| < 2^(E - 126) for the biased exponent E of the largest magnitude; e = 156 - E puts it below 2^30
                const int E = static_cast<int>(mx >> 23);
                int e = 156 - E;
                e = e > 126 ? 126 : e;
                const float scale = __uint_as_float(static_cast<uint32_t>(e + 127) << 23);
                // a NaN or an infinity among the activations makes every output of the row NaN
                inv[r] = E == 255 ? __uint_as_float(0x7fc00000u) : __uint_as_float(static_cast<uint32_t>(127 - e) << 23);
                if (tid == 0) inv_of_row[r] = inv[r];
                uint8_t* set = planes + r * g.set_bytes;
                float* sumx = reinterpret_cast<float*>(set + 4 * g.plane_stride);
                const float4* x4 = reinterpret_cast<const float4*>(ce.x + static_cast<size_t>(r) * a.in_w + x_first);
                for (int i = tid; i < n4; i += T) {       // (whole groups of eight lanes are in or out: n4 % 64 == 0)
                    const float4 v = x4[i];
                    uint32_t pl[4];
                    digit_planes(__float2int_rn(v.x * scale), __float2int_rn(v.y * scale), __float2int_rn(v.z * scale),
                                 __float2int_rn(v.w * scale), pl);
#pragma unroll
                    for (int p = 0; p < 4; ++p) *reinterpret_cast<uint32_t*>(set + p * g.plane_stride + 4 * i) = pl[p];
                    float s = (v.x + v.y) + (v.z + v.w);
                    if (!F::kNeedsSums) {
                        // (the format has neither minima nor an offset: no room is kept for the sums)
                    } else if (F::kSumRun == 32) {
                        s = oct_sum(s);
                        if ((i & 7) == 0) sumx[i >> 3] = s;
                    } else {
                        s += dpp_mov<0xB1>(s);
                        s += dpp_mov<0x4E>(s);
                        if ((i & 3) == 0) sumx[i >> 2] = s;
                    }
                }
            }
        }
        planes_x = ce.x;
        planes_rows = rows;
        __syncthreads();
    };

    u32x4 regs[2][LPW];
    fetch_enter();
    fetch(regs[0]);
    fetch(regs[1]);

    const uint32_t row_off = static_cast<uint32_t>(row_l) * (static_cast<uint32_t>(g.row_pieces) * 16u) +
                             static_cast<uint32_t>(wave) * (16u * F::kPieces);
    int pbuf = 0;
    bool done = false;
    int done_row0 = 0;
    int done_up = 0;                       // SPLIT: the finished tile's number in its run times 8, plus the part that was finished
    // Adds up and stores the tile whose wave partials sit in part[pbuf ^ 1].  It runs before the next stage enters its
    // matrix, so the tile's matrix is still `ce` (no copies of its fields: the kernel is short of scalar registers).
    auto finalize = [&]() {
        const int done_rows = ce.out_w - done_row0 < kTileRows ? ce.out_w - done_row0 : kTileRows;
        const int done_out_w = ce.out_w, done_inputs = ce.rows;
        float* const done_y = ce.y;
        const float* const done_bias = ce.bias;
        if (tid < kTileRows * R) {
            const int r = tid >> 4, j0 = tid & 15;
            if (r < done_inputs) {
                float t = 0.0f;
                for (int w2 = 0; w2 < W; ++w2) t += part[pbuf ^ 1][r][w2][j0];
                const int done_p = SPLIT ? done_up & 7 : 0;
                if (done_bias && (!SPLIT || done_p == 0)) {
                    const NNHIP_CONST_PTR float* cb = (const NNHIP_CONST_PTR float*)done_bias + done_row0;
                    float bv = 0.0f;
#pragma unroll
                    for (int j = 0; j < kTileRows; ++j) {
                        const float v = cb[j < done_rows ? j : 0];
                        bv = j0 == j ? v : bv;
                    }
                    t += bv;
                }
                if constexpr (SPLIT) {
                    // (written and read by this lane only: no barrier between the parts)
                    // the sums of the run's tiles between their parts lie behind the planes: [tile of the run][input row][row]
                    float* const kept = reinterpret_cast<float*>(smem + 2 * g.stage_bytes + R * g.set_bytes) + ((done_up >> 3) * R + r) * kTileRows + j0;
                    if (done_p > 0) t = *kept + t;
                    if (done_p + 1 < a.parts) *kept = t;
                    else if (j0 < done_rows) done_y[static_cast<size_t>(r) * done_out_w + done_row0 + j0] = t;
                } else {
                    if (j0 < done_rows) done_y[static_cast<size_t>(r) * done_out_w + done_row0 + j0] = t;
                }
            }
        }
        done = false;
    };
    // SPLIT: the stage just multiplied was the last of its part of tile c_t: where the next stage lies
    auto next_of_part = [&]() {
        done_up = c_u * 8 + c_p;
        c_t += t_step;
        ++c_u;
        if (c_t < run_end(c_first, ce.first_tile + ce.tiles)) {
            c_k = c_p * a.part_stages;
        } else if (c_p + 1 < a.parts) {
            ++c_p;
            c_t = c_first;
            c_u = 0;
            c_k = c_p * a.part_stages;
        } else {
            c_p = 0;
            c_first = c_t;
            c_u = 0;
            c_k = 0;
        }
    };

    float accq[R], accm[R];
#pragma unroll
    for (int r = 0; r < R; ++r) accq[r] = accm[r] = 0.0f;
    // The matrix of the stage about to be multiplied; true when its activations are not the ones in LDS.
    auto enter = [&]() {
        if constexpr (SPLIT) {
            if (c_u != 0 || c_k != c_p * a.part_stages) return false;
            while (c_t >= ce.first_tile + ce.tiles) ce = entry_at(++c_m);      // (only where a run begins)
            return true;
        }
        bool new_x = false;
        if (c_k == 0 && c_t >= ce.first_tile + ce.tiles) {
            while (c_t >= ce.first_tile + ce.tiles) ce = entry_at(++c_m);
            new_x = ce.x != planes_x || ce.rows != planes_rows;
        }
        return new_x;
    };
    // Shared passes of the formats with one scale per 32 weights: one MFMA serves up to four input rows (operand A = their
    // digit planes stacked, lane quarter q' receives input row q'), see run_stacked of the task.
    constexpr bool kStack = R > 1 && F::kStacked;
    float acc_sq = 0.0f, acc_sm = 0.0f;
    auto compute = [&](const uint8_t* cur) {
        if constexpr (kStack) {
            const uint8_t* a_plane = planes + (row_l >> 2) * g.set_bytes + (row_l & 3) * g.plane_stride + 8 * quarter;
            const float* d_sums = reinterpret_cast<const float*>(planes + quarter * g.set_bytes + 4 * g.plane_stride);
            const int b0 = c_k * g.cols + wave;
            const int pb = SPLIT ? c_p * a.part_stages * g.cols : 0;        // the first block column the planes in LDS hold
            const uint8_t* stage = cur + row_off;
            constexpr int kSumsPerBlock = 256 / F::kSumRun;
#pragma unroll
            for (int t = 0; t < M; ++t) {
                const int b = b0 + t * W;
                if (b < a.nblocks)
                    F::run_stacked(F::load_stacked(stage + t * W * (16 * F::kPieces), quarter, (wave & 1) != 0), a_plane + 256 * (b - pb),
                                   d_sums + kSumsPerBlock * (b - pb), tables, acc_sq, acc_sm);
            }
            const int k_end = SPLIT && (c_p + 1) * a.part_stages < KC ? (c_p + 1) * a.part_stages : KC;
            if (++c_k == k_end) {
                const float p = fmaf(acc_sq, inv_of_row[quarter], -acc_sm);     // (from LDS: a register array indexed by the lane would go to scratch memory)
                if (quarter < ce.rows) part[pbuf][quarter][wave][row_l] = p;
                acc_sq = 0.0f;
                acc_sm = 0.0f;
                done = true;
                done_row0 = (c_t - ce.first_tile) * kTileRows;
                pbuf ^= 1;
                if constexpr (SPLIT) {
                    next_of_part();
                } else {
                    c_k = 0;
                    c_t += t_step;
                }
            }
        } else {
        // task t of this wave: block column c_k * cols + t * W + wave of the row (W is even: the block's parity is the
        // wave's).  Stages whose tasks all exist run them as one straight piece of code, so that the lookups and products
        // of one task overlap the other's; a tile's last stage may hold fewer.
        const int pb = SPLIT ? c_p * a.part_stages * g.cols : 0;            // the first block column the planes in LDS hold
        auto task = [&](const typename F::Raw& raw, int b_of_row) {
            const int b = b_of_row - pb;
            if constexpr (SplitLookups<F>::value && R > 1) {
                // what the block's lookups return does not depend on the input row: made once, used by every row
                typename F::Looked lk;
                F::lookup(raw, quarter, tables, lk);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if (r < ce.rows) {
                        const uint8_t* set = planes + r * g.set_bytes;
                        typename F::X xs;
                        F::load_x(xs, set + (row_l & 3) * g.plane_stride, reinterpret_cast<const float*>(set + 4 * g.plane_stride), b,
                                  quarter, a_zeros);
                        F::finish(raw, lk, xs, accq[r], accm[r]);
                    }
                }
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if (r < ce.rows) {
                        const uint8_t* set = planes + r * g.set_bytes;
                        typename F::X xs;
                        F::load_x(xs, set + (row_l & 3) * g.plane_stride, reinterpret_cast<const float*>(set + 4 * g.plane_stride), b,
                                  quarter, a_zeros);
                        F::run(raw, xs, quarter, tables, accq[r], accm[r]);
                    }
                }
            }
        };
        const int b0 = c_k * g.cols + wave;
        const uint8_t* stage = cur + row_off;
        if (b0 + (M - 1) * W < a.nblocks) {
            typename F::Raw raw[M];
#pragma unroll
            for (int t = 0; t < M; ++t) raw[t] = F::load(stage + t * W * (16 * F::kPieces), quarter, (wave & 1) != 0);
#pragma unroll
            for (int t = 0; t < M; ++t) task(raw[t], b0 + t * W);
        } else {
#pragma unroll
            for (int t = 0; t < M - 1; ++t)
                if (b0 + t * W < a.nblocks) task(F::load(stage + t * W * (16 * F::kPieces), quarter, (wave & 1) != 0), b0 + t * W);
        }
        const int k_end = SPLIT && (c_p + 1) * a.part_stages < KC ? (c_p + 1) * a.part_stages : KC;
        if (++c_k == k_end) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float p = fmaf(accq[r], inv[r], -accm[r]);
                p = quarter_sum(p);
                if (lane < kTileRows) part[pbuf][r][wave][lane] = p;
                accq[r] = 0.0f;
                accm[r] = 0.0f;
            }
            done = true;
            done_row0 = (c_t - ce.first_tile) * kTileRows;
            pbuf ^= 1;
            if constexpr (SPLIT) {
                next_of_part();
            } else {
                c_k = 0;
                c_t += t_step;
            }
        }
        }
    };
    if constexpr (ONE) {
        // One stage buffer that holds a whole 16-row tile (a contiguous piece of the matrix: no line of memory is
        // requested by two stages) and two register sets, i.e. up to two tiles on their way: a set is parked when
        // every wave has left the tile before it, and refilled with the tile after the next right away.
        auto one_step = [&](u32x4 (&mine)[LPW]) {
            park(buf0, mine);
            __syncthreads();            // the tile is in LDS
            fetch(mine);
            if (done) finalize();
            if (enter()) prepare_x();
            compute(buf0);
            __syncthreads();            // every wave has read its blocks
        };
        // (an odd last tile is taken after the loop: a conditional second step inside it would make the compiler wait
        // for both register sets before every parking write)
        for (int n = 0; n + 2 <= total; n += 2) {
            one_step(regs[0]);
            one_step(regs[1]);
        }
        if (total & 1) one_step(regs[0]);
    } else {
        auto stage_step = [&](uint8_t* cur, uint8_t* nxt, u32x4 (&refill)[LPW], const u32x4 (&landing)[LPW]) {
            fetch(refill);
            if (done) finalize();
            if (enter()) prepare_x();
            compute(cur);
            park(nxt, landing);
            __syncthreads();
        };
        park(buf0, regs[0]);
        __syncthreads();
        for (int n = 0; n < total; n += 2) {
            stage_step(buf0, buf1, regs[0], regs[1]);
            if (n + 1 < total) stage_step(buf1, buf0, regs[1], regs[0]);
        }
    }
    if (done) finalize();
}

// The (KC, M, LPW) combinations the kernel is instantiated for.
struct Variant { int kc, m, lpw; };
constexpr Variant kVariants[] = {{1, 2, 5}, {1, 2, 6}, {2, 1, 3}, {1, 1, 3}, {1, 1, 2}, {2, 1, 2}, {1, 1, 4}, {2, 1, 4}};
constexpr Variant kOneSetVariants[] = {{1, 2, 6}};

// Picks W and C for (block bytes, in_w).  C = W * M columns per stage must divide the row's super-blocks into KC whole
// stages, two stage buffers must fit LDS (one of them doubles as scratch for the digit planes when the activations
// change), (KC, M, LPW) must be an instantiated variant.  Two columns per wave (`two_columns`) are for stages of whole
// rows only: with two register sets on their way for Q4_K (1), with one set for Q5_K (2), whose unpacking does not leave
// the registers for both a second set of operand A and a second set of pieces (spills cost more than the wide form
// does; Q5_K at 5120 wide streams at 83 - 84 % of the HBM peak so, against 80 % in half rows; Q6_K gained nothing from
// either and stays with one column).  Among the candidates a stage of whole rows comes first (a tile is then one run of whole 128-byte
// lines, where two half-row stages request the line they meet in twice: 3 % of the traffic; Q4_K at 4096 / 5120 / 6144
// wide streams at 82 / 85 / 81 % of the HBM peak so, against 74 / 83 / 79 % in half rows), then one column per wave, the
// larger stage, the waves.
bool plan_mfma(int block_pieces, int in_w, bool even_waves, int two_columns, bool whole_pieces, MfmaGeom* out)
{
    const int nblocks = in_w / 256;
    const int bp = block_pieces;
    if (nblocks < 1 || bp < 1) return false;
    const int planes_bytes = 4 * (in_w + 16) + (in_w / 16) * 4;
    double best_score = -1.0;
    MfmaGeom best{};
    for (int W = 6; W <= kMaxWaves; ++W) {
        for (int m = 1; m <= (two_columns ? 2 : 1); ++m) {
            MfmaGeom g{};
            if (even_waves && (W & 1)) continue;       // block parity must be wave parity (Q6_K)
            g.waves = W;
            g.cols = W * m;
            if (nblocks % g.cols != 0) continue;
            g.kchunks = nblocks / g.cols;
            g.tasks = m;
            g.row_pieces = (g.cols * bp) | 1;
            // (stages of whole rows of whole pieces are requested as the run of memory they are, without the padding)
            const bool linear = whole_pieces && g.kchunks == 1;
            g.stage_loads = (kTileRows * (linear ? g.cols * bp : g.row_pieces) + 63) / 64;
            g.loads_per_wave = (g.stage_loads + W - 1) / W;
            g.one_set = m == 2 && two_columns == 2 ? 1 : 0;
            if (m == 2 && g.kchunks != 1) continue;
            if (g.one_set && W > 10) continue;          // (measured: twelve waves stream faster in half rows with two sets)
            // every wave parks loads_per_wave pieces (one set: only those the stage has)
            g.stage_bytes = linear ? (kTileRows * g.row_pieces * 16 + 1023) / 1024 * 1024
                                   : (g.one_set ? g.stage_loads : g.loads_per_wave * W) * 1024;
            if (g.stage_bytes < planes_bytes || 2 * g.stage_bytes > kLdsBudget) continue;
            bool ok = false;
            if (g.one_set) {
                for (const Variant& v : kOneSetVariants) ok = ok || (v.kc == g.kchunks && v.m == m && v.lpw == g.loads_per_wave);
            } else {
                for (const Variant& v : kVariants) ok = ok || (v.kc == g.kchunks && v.m == m && v.lpw == g.loads_per_wave);
            }
            if (!ok) continue;
            g.stages = 2;
            g.lds_bytes = 2 * static_cast<size_t>(g.stage_bytes);
            const double score = (g.kchunks == 1 ? 2.0 : 0.0) + (m == 1 ? 1.0 : 0.0) +
                                 static_cast<double>(g.stage_bytes) / (256.0 * 1024) + 1e-3 * W;
            if (score > best_score) {
                best_score = score;
                best = g;
            }
        }
    }
    if (best_score < 0) return false;
    *out = best;
    return true;
}

template <class F, int KC, int M, int LPW, bool ONESET = false>
hipError_t launch_mfma_variant(Lane* lane, const MfmaArgs& a, dim3 grid)
{
    static LdsLimit big_lds;
    const hipError_t e = big_lds.ensure(lane->device, reinterpret_cast<const void*>(&matvec_mfma_kernel<F, KC, M, LPW, ONESET>), kLdsBudget);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((matvec_mfma_kernel<F, KC, M, LPW, ONESET>), grid, dim3(64 * a.g.waves), a.g.lds_bytes, lane->stream, a);
    return hipGetLastError();
}

template <class F>
hipError_t launch_mfma(Lane* lane, const MfmaArgs& a)
{
    const int groups = a.total_tiles < lane->compute_units ? a.total_tiles : lane->compute_units;
    const dim3 grid(groups);
    const int kc = a.g.kchunks, m = a.g.tasks, lpw = a.g.loads_per_wave;
#define NNHIP_VARIANT(K, MM, L) if (kc == K && m == MM && lpw == L) return launch_mfma_variant<F, K, MM, L>(lane, a, grid);
    if constexpr (std::is_same_v<F, Q4KTask>) {
        NNHIP_VARIANT(1, 2, 5) NNHIP_VARIANT(1, 2, 6)
    } else if constexpr (std::is_same_v<F, Q5KTask>) {
        if (a.g.one_set && kc == 1 && m == 2 && lpw == 6) return launch_mfma_variant<F, 1, 2, 6, true>(lane, a, grid);
    }
    NNHIP_VARIANT(2, 1, 3) NNHIP_VARIANT(1, 1, 3) NNHIP_VARIANT(1, 1, 2) NNHIP_VARIANT(2, 1, 2) NNHIP_VARIANT(1, 1, 4)
    NNHIP_VARIANT(2, 1, 4)
#undef NNHIP_VARIANT
    return hipErrorInvalidConfiguration;
}

int block_bytes_of(uint32_t type)
{
    switch (type) {
    case NNHIP_TYPE_Q4_K: return Q4KTask::kBlockBytes;
    case NNHIP_TYPE_Q5_K: return Q5KTask::kBlockBytes;
    case NNHIP_TYPE_Q6_K: return Q6KTask::kBlockBytes;
    case NNHIP_TYPE_IQ2_S: return IQ2STask::kBlockBytes;
    case NNHIP_TYPE_IQ3_S: return IQ3STask::kBlockBytes;
    case NNHIP_TYPE_Q8_0: return Q8_0Task::kBlockBytes;
    default: return 0;
    }
}

int block_pieces_of(uint32_t type)
{
    switch (type) {
    case NNHIP_TYPE_Q4_K: return Q4KTask::kPieces;
    case NNHIP_TYPE_Q5_K: return Q5KTask::kPieces;
    case NNHIP_TYPE_Q6_K: return Q6KTask::kPieces;
    case NNHIP_TYPE_IQ2_S: return IQ2STask::kPieces;
    case NNHIP_TYPE_IQ3_S: return IQ3STask::kPieces;
    case NNHIP_TYPE_Q8_0: return Q8_0Task::kPieces;
    default: return 0;
    }
}


struct WideTraits { int pieces, m, lpw, table_bytes; bool sums, tight; int one_m, one_lpw; };

template <class F>
constexpr WideTraits wide_traits_of(bool shared)
{
    return {F::kPieces, shared ? F::kSharedM : F::kWideM, shared ? F::kSharedLpw : F::kWideLpw, 0, F::kNeedsSums, F::kTightStage, 0, 0};
}

WideTraits wide_traits(uint32_t type, bool shared)
{
    switch (type) {
    case NNHIP_TYPE_Q4_K: return wide_traits_of<Q4KTask>(shared);
    case NNHIP_TYPE_Q5_K: return wide_traits_of<Q5KTask>(shared);
    case NNHIP_TYPE_Q6_K: return wide_traits_of<Q6KTask>(shared);
    case NNHIP_TYPE_IQ2_S: {
        WideTraits t = wide_traits_of<IQ2STask>(shared);
        t.table_bytes = IQ2STask::kTableBytes;
        return t;
    }
    case NNHIP_TYPE_IQ3_S: {
        WideTraits t = wide_traits_of<IQ3STask>(shared);
        t.table_bytes = IQ3STask::kTableBytes;
        return t;
    }
    case NNHIP_TYPE_Q8_0: {
        WideTraits t = wide_traits_of<Q8_0Task>(shared);
        if (shared) return t;
        t.one_m = Q8_0Task::kOneM;
        t.one_lpw = Q8_0Task::kOneLpw;
        return t;
    }
    default: return {0, 0, 0, 0, false, false, 0, 0};
    }
}

// room left for the kernel's static arrays (partial sums, maxima, the zero area): 2 KB with one input row per pass,
// 7 KB with four
constexpr int wide_static_lds(int inputs) { return inputs > 1 ? 8 * 1024 : 2 * 1024; }

// W for the wide form: even, as many of the row's blocks per stage as two stage buffers beside the plane sets of
// `inputs` rows leave room for: the most waves, weighted by the share of block slots a tile fills and by an even
// split over the four SIMDs.
bool plan_wide(uint32_t type, int in_w, int inputs, WideGeom* out)
{
    const WideTraits tr = wide_traits(type, inputs > 1);
    const int nblocks = in_w / 256;
    if (!tr.pieces || nblocks < 4) return false;
    WideGeom best{};
    double best_score = -1.0;
    for (int W = 12; W >= 4; W -= 2) {
        WideGeom g{};
        g.waves = W;
        g.cols = W * tr.m;
        if (g.cols > nblocks + tr.m) continue;
        g.kchunks = (nblocks + g.cols - 1) / g.cols;
        g.tail_cols = nblocks - (g.kchunks - 1) * g.cols;
        g.row_pieces = (g.cols * tr.pieces) | 1;
        const int loads = (kTileRows * g.row_pieces + 63) / 64;
        if ((loads + W - 1) / W > tr.lpw) continue;
        g.stage_bytes = (tr.tight ? loads : tr.lpw * W) * 1024;      // to the last row's end, or every wave's slots
        g.plane_stride = in_w + 16;
        g.set_bytes = (4 * g.plane_stride + (tr.sums ? (in_w / 16) * 4 : 0) + 15) / 16 * 16;
        g.lds_bytes = 2 * static_cast<size_t>(g.stage_bytes) + static_cast<size_t>(inputs) * g.set_bytes;
        if (g.lds_bytes + wide_static_lds(inputs) + tr.table_bytes > static_cast<size_t>(160 * 1024)) continue;
        const double fill = static_cast<double>(nblocks) / (g.kchunks * g.cols);
        // (throughput grows with the waves: a stage holds W * M blocks per row and W tasks run side by side)
        // (and of two equal products the fuller stages win: 16 blocks go as 2 x 8 rather than 12 + 4; measured on rows of
        // 28 blocks: three stages of ten columns stream 3 - 6 % faster than three of twelve, the last a third full)
        // (one input row per pass of a K-quant: 1 - 9 % on rows of 17 - 50 blocks; the codebook formats lost 3 - 5 % to it
        // and keep the plain product, as do the shared passes and Q8_0, where it was not measured)
        const bool k_quant = type == NNHIP_TYPE_Q4_K || type == NNHIP_TYPE_Q5_K || type == NNHIP_TYPE_Q6_K;
        const double emptiness = inputs == 1 && k_quant ? fill * std::sqrt(fill) : fill;
        const double score = emptiness * W / 12.0 * (W % 4 == 0 ? 1.0 : 0.95) * (0.9 + 0.1 * fill);
        if (score > best_score) {
            best_score = score;
            best = g;
        }
    }
    const int row_bytes = nblocks * tr.pieces * 16;
    const bool split_lines = row_bytes % 128 != 0 || (best_score >= 0 && best.kchunks > 1 && (best.cols * tr.pieces * 16) % 128 != 0);
    if (tr.one_m && inputs == 1 && split_lines) {
        // Whole tiles in one stage buffer, for rows whose stages would begin or end inside 128-byte lines of memory (5376
        // = 21 blocks: 5712-byte rows): a line shared by two stages is fetched twice by the non-temporal loads (3 % more
        // traffic measured), while a tile of 16 rows is one contiguous, line-aligned piece of the matrix.
        for (int W = 12; W >= 8; W -= 2) {
            WideGeom g{};
            g.waves = W;
            g.cols = nblocks;
            if (nblocks <= W * (tr.one_m - 1) || nblocks > W * tr.one_m) continue;        // (every wave's first task exists)
            g.kchunks = 1;
            g.tail_cols = nblocks;
            g.row_pieces = (g.cols * tr.pieces) | 1;
            const int loads = (kTileRows * g.row_pieces + 63) / 64;
            if ((loads + W - 1) / W > tr.one_lpw) continue;
            g.stage_bytes = loads * 1024;
            g.plane_stride = in_w + 16;
            g.set_bytes = (4 * g.plane_stride + (tr.sums ? (in_w / 16) * 4 : 0) + 15) / 16 * 16;
            g.single = 1;
            g.lds_bytes = static_cast<size_t>(g.stage_bytes) + g.set_bytes;
            if (g.lds_bytes + wide_static_lds(1) + tr.table_bytes > static_cast<size_t>(160 * 1024)) continue;
            *out = g;
            return true;
        }
    }
    if (best_score < 0) return false;
    *out = best;
    return true;
}

// The split form for rows whose sets of planes (one, or four with shared passes) do not fit LDS beside two stage
// buffers of a useful size: W as above, and the fewest parts (groups of whole stages) whose planes do.  Q8_0 has it with
// one input row per entry only: its row-tiled row-step kernel serves calls with several input rows.
bool plan_wide_split(uint32_t type, int in_w, int inputs, WideGeom* out, int* parts, int* part_stages, int* run_tiles)
{
    const WideTraits tr = wide_traits(type, inputs > 1);
    const int nblocks = in_w / 256;
    if (!tr.pieces || nblocks < 4 || (type == NNHIP_TYPE_Q8_0 && inputs > 1)) return false;
    double best_score = -1.0;
    for (int W = 12; W >= 6; W -= 2) {
        WideGeom g{};
        g.waves = W;
        g.cols = W * tr.m;
        if (g.cols > nblocks + tr.m) continue;
        g.kchunks = (nblocks + g.cols - 1) / g.cols;
        g.tail_cols = nblocks - (g.kchunks - 1) * g.cols;
        g.row_pieces = (g.cols * tr.pieces) | 1;
        const int loads = (kTileRows * g.row_pieces + 63) / 64;
        if ((loads + W - 1) / W > tr.lpw) continue;
        g.stage_bytes = (tr.tight ? loads : tr.lpw * W) * 1024;
        for (int P = 2; P <= 6; ++P) {
            const int SP = (g.kchunks + P - 1) / P;
            if ((P - 1) * SP >= g.kchunks) continue;            // (every part holds a stage)
            const int part_w = SP * g.cols * 256;
            g.plane_stride = part_w + 16;
            g.set_bytes = (4 * g.plane_stride + (tr.sums ? (part_w / 16) * 4 : 0) + 15) / 16 * 16;
            g.lds_bytes = 2 * static_cast<size_t>(g.stage_bytes) + static_cast<size_t>(inputs) * g.set_bytes;
            // what is left holds the sums of a run's tiles: at least eight tiles
            const size_t per_tile = static_cast<size_t>(inputs) * kTileRows * sizeof(float);
            const size_t fixed = g.lds_bytes + wide_static_lds(inputs) + tr.table_bytes;
            if (fixed + 8 * per_tile > static_cast<size_t>(160 * 1024)) continue;
            size_t run = (static_cast<size_t>(160 * 1024) - fixed) / per_tile;
            if (run > static_cast<size_t>(kSplitRunMax)) run = kSplitRunMax;
            g.lds_bytes += run * per_tile;
            const double fill = static_cast<double>(nblocks) / (g.kchunks * g.cols);
            const double score = fill * W / 12.0 * (W % 4 == 0 ? 1.0 : 0.95) * (0.9 + 0.1 * fill) * (1.0 - 0.02 * (P - 2));
            if (score > best_score) {
                best_score = score;
                *out = g;
                *parts = P;
                *part_stages = SP;
                *run_tiles = static_cast<int>(run);
            }
            break;
        }
    }
    return best_score >= 0;
}

// The geometry a launch of the wide form takes: the plain form where it gets at least eight waves, else the split form
// where that exists (rows of 28672 values leave the plain one-row form four waves), else whatever the plain form gets.
// *parts = 0: the plain form.
bool plan_wide_any(uint32_t type, int in_w, int inputs, WideGeom* out, int* parts, int* part_stages, int* run_tiles = nullptr)
{
    int run_unused = 0;
    if (!run_tiles) run_tiles = &run_unused;
    WideGeom plain{};
    const bool have_plain = plan_wide(type, in_w, inputs, &plain);
    *parts = 0;
    *part_stages = 0;
    if (have_plain && (plain.waves >= 8 || plain.single)) {
        *out = plain;
        return true;
    }
    if (plan_wide_split(type, in_w, inputs, out, parts, part_stages, run_tiles)) return true;
    *parts = 0;
    *part_stages = 0;
    if (have_plain) *out = plain;
    return have_plain;
}

template <class F, int R>
hipError_t launch_wide_split_of(Lane* lane, const WideArgs& a)
{
    constexpr int M = R == 1 ? F::kWideM : F::kSharedM, LPW = R == 1 ? F::kWideLpw : F::kSharedLpw;
    static LdsLimit big_lds;
    const void* fn = reinterpret_cast<const void*>(&matvec_mfma_wide_kernel<F, M, LPW, R, false, true>);
    const hipError_t e = big_lds.ensure(lane->device, fn, 160 * 1024 - wide_static_lds(R) - F::kLdsTableBytes);
    if (e != hipSuccess) return e;
    const int groups = a.total_tiles < lane->compute_units ? a.total_tiles : lane->compute_units;
    hipLaunchKernelGGL((matvec_mfma_wide_kernel<F, M, LPW, R, false, true>), dim3(groups), dim3(64 * a.g.waves), a.g.lds_bytes,
                       lane->stream, a);
    return hipGetLastError();
}

template <class F, int R>
hipError_t launch_wide_of(Lane* lane, const WideArgs& a)
{
    constexpr int M = R == 1 ? F::kWideM : F::kSharedM, LPW = R == 1 ? F::kWideLpw : F::kSharedLpw;
    static LdsLimit big_lds;
    const void* fn = reinterpret_cast<const void*>(&matvec_mfma_wide_kernel<F, M, LPW, R>);
    const hipError_t e = big_lds.ensure(lane->device, fn, 160 * 1024 - wide_static_lds(R) - F::kLdsTableBytes);
    if (e != hipSuccess) return e;
    const int groups = a.total_tiles < lane->compute_units ? a.total_tiles : lane->compute_units;
    hipLaunchKernelGGL((matvec_mfma_wide_kernel<F, M, LPW, R>), dim3(groups), dim3(64 * a.g.waves), a.g.lds_bytes, lane->stream, a);
    return hipGetLastError();
}

template <class F>
hipError_t launch_wide(Lane* lane, const WideArgs& a, int inputs)
{
    return inputs == 1 ? launch_wide_of<F, 1>(lane, a) : launch_wide_of<F, 4>(lane, a);
}

bool entry_ok(uint32_t type, int in_w, int out_w, const void* w)
{
    const int bb = block_bytes_of(type);
    if (!bb || in_w % 256 != 0 || (reinterpret_cast<uintptr_t>(w) & 15u)) return false;
    if (bb % 16 != 0 && ((in_w / 256) & 1)) return false;      // (Q6_K: a row must end with an odd block, see piece_src)
    const uint64_t bytes = static_cast<uint64_t>(out_w) * (in_w / 256) * bb;
    return bytes < 0x7fffffffull;            // piece offsets are 32-bit and "no piece" is bit 31
}

void fill_args(uint32_t type, int in_w, const MfmaGeom& g, MfmaArgs* a)
{
    a->g = g;
    a->in_w = in_w;
    a->nblocks = in_w / 256;
    a->row_bytes = static_cast<uint32_t>(a->nblocks) * static_cast<uint32_t>(block_bytes_of(type));
    a->row_pieces_magic = static_cast<uint32_t>((0x100000000ull + g.row_pieces - 1) / g.row_pieces);
    const uint32_t used = static_cast<uint32_t>(g.cols) * static_cast<uint32_t>(block_pieces_of(type));
    a->used_pieces_magic = static_cast<uint32_t>((0x100000000ull + used - 1) / used);
}

}  // namespace

MfmaTableEntry matvec_mfma_entry(uint32_t type, const float* x, const void* w, const float* bias, float* y, int in_w,
                                 int out_w, int first_tile)
{
    MfmaTableEntry e{};
    e.x = x;
    e.w = static_cast<const uint8_t*>(w);
    e.bias = bias;
    e.y = y;
    e.out_w = out_w;
    e.w_bytes = static_cast<uint32_t>(out_w) * static_cast<uint32_t>(in_w / 256) * static_cast<uint32_t>(block_bytes_of(type));
    e.tiles = (out_w + kTileRows - 1) / kTileRows;
    e.first_tile = first_tile;
    e.rows = 1;
    return e;
}

bool matvec_mfma_geometry(uint32_t type, int in_w, int out_w, const void* w, MfmaPlan* plan)
{
    if (type == NNHIP_TYPE_IQ2_S || type == NNHIP_TYPE_IQ3_S || type == NNHIP_TYPE_Q8_0) return false;       // (these have the wide form only)

    if (!entry_ok(type, in_w, out_w, w)) return false;
    MfmaGeom g;
    if (!plan_mfma(block_pieces_of(type), in_w, block_bytes_of(type) % 16 != 0, type == NNHIP_TYPE_Q4_K ? 1 : type == NNHIP_TYPE_Q5_K ? 2 : 0,
                   type == NNHIP_TYPE_Q4_K || type == NNHIP_TYPE_Q5_K, &g)) return false;
    if (plan) {
        plan->waves = g.waves;
        plan->cols = g.cols;
        plan->kchunks = g.kchunks;
        plan->stages = g.stages;
        plan->stage_bytes = g.stage_bytes;
        plan->loads_per_wave = g.loads_per_wave;
        plan->lds_bytes = static_cast<int>(g.lds_bytes);
    }
    return true;
}

hipError_t launch_matvec_mfma_table(Lane* lane, uint32_t type, int in_w, const MfmaTableEntry* device_entries, int entries,
                                    int total_tiles, bool runs)
{
    MfmaArgs a{};
    MfmaGeom g;
    if (!plan_mfma(block_pieces_of(type), in_w, block_bytes_of(type) % 16 != 0, type == NNHIP_TYPE_Q4_K ? 1 : type == NNHIP_TYPE_Q5_K ? 2 : 0,
                   type == NNHIP_TYPE_Q4_K || type == NNHIP_TYPE_Q5_K, &g)) return hipErrorInvalidValue;
    fill_args(type, in_w, g, &a);
    a.table = device_entries;
    a.entries = entries;
    a.total_tiles = total_tiles;
    a.chunked = runs ? 1 : 0;
    switch (type) {
    case NNHIP_TYPE_Q4_K: return launch_mfma<Q4KTask>(lane, a);
    case NNHIP_TYPE_Q5_K: return launch_mfma<Q5KTask>(lane, a);
    case NNHIP_TYPE_Q6_K: return launch_mfma<Q6KTask>(lane, a);
    default: return hipErrorInvalidValue;
    }
}

bool matvec_mfma_wide_geometry(uint32_t type, int in_w, int out_w, const void* w, int inputs, bool* split)
{
    WideGeom g;
    int parts = 0, part_stages = 0;
    const bool ok = inputs >= 1 && inputs <= 4 && entry_ok(type, in_w, out_w, w) &&
                    plan_wide_any(type, in_w, inputs == 1 ? 1 : 4, &g, &parts, &part_stages);
    if (split) *split = ok && parts > 0;
    return ok;
}

namespace {

hipError_t launch_wide_args(Lane* lane, uint32_t type, int in_w, int inputs, WideArgs& a)
{
    if (!plan_wide_any(type, in_w, inputs == 1 ? 1 : 4, &a.g, &a.parts, &a.part_stages, &a.run_tiles)) return hipErrorInvalidValue;
    const bool split = a.parts > 0;
    // (the split form: runs of consecutive tiles, so that a workgroup meets few entries, i.e. converts few vectors)
    if (split) a.chunked = 1;
    a.in_w = in_w;
    a.nblocks = in_w / 256;
    a.row_bytes = static_cast<uint32_t>(a.nblocks) * static_cast<uint32_t>(block_bytes_of(type));
    a.row_pieces_magic = static_cast<uint32_t>((0x100000000ull + a.g.row_pieces - 1) / a.g.row_pieces);
    if (split) {
        switch (type) {
        case NNHIP_TYPE_Q4_K: return inputs == 1 ? launch_wide_split_of<Q4KTask, 1>(lane, a) : launch_wide_split_of<Q4KTask, 4>(lane, a);
        case NNHIP_TYPE_Q5_K: return inputs == 1 ? launch_wide_split_of<Q5KTask, 1>(lane, a) : launch_wide_split_of<Q5KTask, 4>(lane, a);
        case NNHIP_TYPE_Q6_K: return inputs == 1 ? launch_wide_split_of<Q6KTask, 1>(lane, a) : launch_wide_split_of<Q6KTask, 4>(lane, a);
        case NNHIP_TYPE_IQ2_S: return inputs == 1 ? launch_wide_split_of<IQ2STask, 1>(lane, a) : launch_wide_split_of<IQ2STask, 4>(lane, a);
        case NNHIP_TYPE_IQ3_S: return inputs == 1 ? launch_wide_split_of<IQ3STask, 1>(lane, a) : launch_wide_split_of<IQ3STask, 4>(lane, a);
        case NNHIP_TYPE_Q8_0: return inputs == 1 ? launch_wide_split_of<Q8_0Task, 1>(lane, a) : hipErrorInvalidValue;
        default: return hipErrorInvalidValue;
        }
    }
    switch (type) {
    case NNHIP_TYPE_Q4_K: return launch_wide<Q4KTask>(lane, a, inputs);
    case NNHIP_TYPE_Q5_K: return launch_wide<Q5KTask>(lane, a, inputs);
    case NNHIP_TYPE_Q6_K: return launch_wide<Q6KTask>(lane, a, inputs);
    case NNHIP_TYPE_IQ2_S: return launch_wide<IQ2STask>(lane, a, inputs);
    case NNHIP_TYPE_IQ3_S: return launch_wide<IQ3STask>(lane, a, inputs);
    case NNHIP_TYPE_Q8_0:
        if (inputs != 1) return launch_wide_of<Q8_0Task, 4>(lane, a);
        a.chunked = 1;          // (always for Q8_0, whose batches are whole models; measured level with every-G-th at one vector)
        if (a.g.single) {
            static LdsLimit big_lds;
            const void* fn = reinterpret_cast<const void*>(&matvec_mfma_wide_kernel<Q8_0Task, Q8_0Task::kOneM, Q8_0Task::kOneLpw, 1, true>);
            const hipError_t e = big_lds.ensure(lane->device, fn, 160 * 1024 - wide_static_lds(1));
            if (e != hipSuccess) return e;
            const int groups = a.total_tiles < lane->compute_units ? a.total_tiles : lane->compute_units;
            hipLaunchKernelGGL((matvec_mfma_wide_kernel<Q8_0Task, Q8_0Task::kOneM, Q8_0Task::kOneLpw, 1, true>), dim3(groups),
                               dim3(64 * a.g.waves), a.g.lds_bytes, lane->stream, a);
            return hipGetLastError();
        }
        return launch_wide_of<Q8_0Task, 1>(lane, a);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

bool describe_matvec_rows_shared(uint32_t type, int rows, int in_w, int out_w, int per_pass, int compute_units,
                                 nnhip_matvec_plan_info* info)
{
    WideGeom g;
    int parts = 0, part_stages = 0;
    if (!plan_wide_any(type, in_w, per_pass, &g, &parts, &part_stages)) return false;
    const int launch_rows = rows < 4 * per_pass ? rows : 4 * per_pass;                 // (four table entries per launch)
    const int tiles = (out_w + kTileRows - 1) / kTileRows * ((launch_rows + per_pass - 1) / per_pass);
    info->kernel = NNHIP_MATVEC_KERNEL_MATRIX_CORE;
    info->threads = 64 * g.waves;
    info->rows_per_step = kTileRows;
    info->steps = tiles;
    info->groups = tiles < compute_units ? tiles : compute_units;
    info->row_tile = rows < per_pass ? rows : per_pass;
    info->ring_depth = 2;                                   // stage buffers
    info->result_buffer_floats = 2 * 4 * kMaxWaves * kTileRows;
    info->dynamic_lds_bytes = static_cast<int32_t>(g.lds_bytes);
    return true;
}

bool describe_matvec_mfma_launch(uint32_t type, int in_w, int form, bool runs, nnhip_batch_launch_info* info)
{
    if (form == 1) {
        MfmaGeom g;
        if (!plan_mfma(block_pieces_of(type), in_w, block_bytes_of(type) % 16 != 0, type == NNHIP_TYPE_Q4_K ? 1 : type == NNHIP_TYPE_Q5_K ? 2 : 0,
                   type == NNHIP_TYPE_Q4_K || type == NNHIP_TYPE_Q5_K, &g)) return false;
        info->threads = 64 * g.waves;
        info->stage_buffers = g.stages;
        info->dynamic_lds_bytes = static_cast<int32_t>(g.lds_bytes);
        info->activations_in_lds = 0;
        info->consecutive_runs = runs ? 1 : 0;
        return true;
    }
    WideGeom g;
    int parts = 0, part_stages = 0;
    if (!plan_wide_any(type, in_w, form == 3 ? 4 : 1, &g, &parts, &part_stages)) return false;
    if (parts > 0) runs = true;
    info->threads = 64 * g.waves;
    info->stage_buffers = g.single ? 1 : 2;
    info->dynamic_lds_bytes = static_cast<int32_t>(g.lds_bytes);
    info->activations_in_lds = 1;
    info->consecutive_runs = (runs || (type == NNHIP_TYPE_Q8_0 && form == 2)) ? 1 : 0;      // (as launch_wide_args)
    return true;
}

hipError_t launch_matvec_mfma_wide_table(Lane* lane, uint32_t type, int in_w, int inputs, const MfmaTableEntry* device_entries,
                                         int entries, int total_tiles, bool runs)
{
    WideArgs a{};
    a.table = device_entries;
    a.entries = entries;
    a.total_tiles = total_tiles;
    a.chunked = runs ? 1 : 0;
    return launch_wide_args(lane, type, in_w, inputs, a);
}

hipError_t launch_matvec_rows_shared(Lane* lane, uint32_t type, const float* x, const void* w, const float* bias, float* y,
                                     int rows, int in_w, int out_w, int per_pass, int* launches)
{
    if (rows < 2 || (per_pass != 1 && per_pass != 4)) return hipErrorInvalidValue;
    // four table entries of `per_pass` input rows per launch (they travel in the kernel arguments); a row's bits do not
    // depend on the rows it shares a pass or a launch with
    *launches = 0;
    const int per_launch = 4 * per_pass;
    for (int r0 = 0; r0 < rows; r0 += per_launch) {
        const int n = rows - r0 < per_launch ? rows - r0 : per_launch;
        WideArgs a{};
        a.table = nullptr;
        for (int r = r0; r < r0 + n; r += per_pass) {
            MfmaTableEntry e = matvec_mfma_entry(type, x + static_cast<size_t>(r) * in_w, w, bias, y + static_cast<size_t>(r) * out_w,
                                                 in_w, out_w, a.total_tiles);
            e.rows = r0 + n - r < per_pass ? r0 + n - r : per_pass;
            a.inline_entries[a.entries++] = e;
            a.total_tiles += e.tiles;
        }
        // (three or four entries, each with planes of its own: runs of consecutive tiles, so that a workgroup converts few vectors)
        a.chunked = a.entries >= 3 || per_pass == 1 ? 1 : 0;
        const hipError_t e = launch_wide_args(lane, type, in_w, per_pass, a);
        if (e != hipSuccess) return e;
        ++*launches;
    }
    return hipSuccess;
}

}  // namespace nnhip
