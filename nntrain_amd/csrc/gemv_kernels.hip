// Dequantization-fused mat-vec kernels for raw GGUF blocks on gfx950 (wave64).
//
// y[r, o] = bias[o] + sum_k x[r, k] * w[o, k]     (NNtrain.Arc/Kernels/qwen.cl:374-406 defines the operator)
//
// Work decomposition (the same for every block format):
//   * a row of the matrix is cut into "units" of 64 weights (two Q8_0 blocks, a quarter of a 256-weight
//     super-block); a unit is the work of one lane: it loads the unit's bytes with 128-bit loads, unpacks scales and
//     nibbles in registers and produces one FP32 partial dot product;
//   * a workgroup of T lanes walks the matrix in "row steps" of RS = floor(T / units_per_row) whole rows: lane t always
//     owns unit t % units_per_row of row t / units_per_row of the step.  Because every step starts on a row boundary
//     a lane meets the same 64 activations in every step, so it loads them ONCE into registers (with their block
//     sums; staged through LDS so the workgroup fetches the vector once) and never recomputes an index for them;
//   * consecutive steps of a workgroup are gridDim.x steps apart (grid-stride), so at any moment all workgroups read
//     one contiguous window of the weight stream, and consecutive lanes read consecutive memory across row ends;
//   * the weight loads of the next DEPTH-1 steps are in flight while a step is reduced (rotating register sets);
//   * unit partials go to LDS (one float per lane, double buffered); after the step's barrier one wave per row adds
//     the row's partials in a fixed order (lane-strided, then a DPP butterfly) and stores y.  The order depends only
//     on in_w, never on the launch geometry, so a row's result is bit-identical for any `rows`, out_w or batching.
#include <cstring>
#include <type_traits>
#include <vector>

#include "nnhip_internal.h"
#include "quant_device.h"

#include "iq_grids.inc"

namespace nnhip {

namespace {

__device__ const uint64_t g_iq2s_grid[1024] = { NNHIP_IQ2S_GRID_VALUES };
__device__ const uint32_t g_iq3s_grid[512] = { NNHIP_IQ3S_GRID_VALUES };

constexpr int kMaxWG = 1024;       // lanes per workgroup (16 waves: 4 per SIMD)
constexpr int kUnitW = 64;         // weights per lane-unit
constexpr int kYBuf = 1024;        // row results a workgroup holds back before storing them
constexpr int kWaitVm0 = 0x0F70;   // s_waitcnt immediate: vmcnt(0), nothing else waited for
constexpr int kMaxDynamicLds = 140 * 1024;   // staged activations; 16 KB of the 160 KB stay for the static arrays

struct MatvecArgs {
    const float* x;
    const uint8_t* w;
    const float* bias;
    float* y;
    int in_w;
    int out_w;
    int units_per_row;     // in_w / 64
    int rows_per_step;     // RS
    int steps;             // ceil(out_w / RS)
    uint32_t row_bytes;
    uint32_t magic;        // ceil(2^32 / units_per_row): t / units_per_row == umulhi(t, magic) for t < 2^32 / upr
    int rows;              // input rows of the call (grid.y covers them MR at a time)
    // fused variants only (null / unused otherwise)
    const float* x2;       // RMSNorm: residual added to x first (or null); SiLU: the `up` vector
    const float* gamma;    // RMSNorm weight
    float* x_out;          // where the vector that was multiplied is stored (or null)
    float* sum_out;        // RMSNorm: where x + residual is stored (or null)
    const float* addend;   // y = addend + (bias + W x) (or null)
    float epsilon;
    const float* lora_z;   // low-rank branch: y += lora_scale * sum_r lora_z[r] * lora_b[o, r] before the addend
    const float* lora_b;
    int lora_rank;         // 0: no low-rank branch
    float lora_scale;
    int head4;             // kPreHeadGather: float4 per head, and the heads that share a source head:
    int head_group;        //   v[h * width + j] = x[(h / group) * width + j] (first-token attention)
    int pair_rows;         // PAIR: out_w / 2; rows o and pair_rows + o leave y[o] = SiLU(z[o]) * z[pair_rows + o]
};

enum : int { kPreNone = 0, kPreRmsNorm = 1, kPreSiluMultiply = 2, kPreHeadGather = 3 };

__device__ __forceinline__ float4 add4(const float4 a, const float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }

// gate * sigmoid(gate) * up with the two-sided sigmoid of the reference (NNtrain.Arc/Kernels/qwen35_attention.cl:9-14,
// 38-43): exp never sees a positive argument.
__device__ __forceinline__ float silu_mul1(float g, float u)
{
    float sig;
    if (g >= 0.0f) {
        sig = 1.0f / (1.0f + expf(-g));
    } else {
        const float e = expf(g);
        sig = e / (1.0f + e);
    }
    return g * sig * u;
}
__device__ __forceinline__ float4 silu_mul4(const float4 g, const float4 u)
{
    return make_float4(silu_mul1(g.x, u.x), silu_mul1(g.y, u.y), silu_mul1(g.z, u.z), silu_mul1(g.w, u.w));
}

__device__ __forceinline__ float dot4s(uint32_t v, const float4 x, float acc)  // 4 signed bytes . x
{
    acc = fmaf(sbyte0(v), x.x, acc);
    acc = fmaf(sbyte1(v), x.y, acc);
    acc = fmaf(sbyte2(v), x.z, acc);
    acc = fmaf(sbyte3(v), x.w, acc);
    return acc;
}

__device__ __forceinline__ float dot4u(uint32_t v, const float4 x, float acc)  // 4 unsigned bytes . x
{
    acc = fmaf(ubyte0(v), x.x, acc);
    acc = fmaf(ubyte1(v), x.y, acc);
    acc = fmaf(ubyte2(v), x.z, acc);
    acc = fmaf(ubyte3(v), x.w, acc);
    return acc;
}

__device__ __forceinline__ float sum4(const float4 v) { return (v.x + v.y) + (v.z + v.w); }

// 64 consecutive activations of unit c, as 16 float4 pieces.
struct XChunk {
    float4 p[16];
};

// The staged activation vector: float4 pieces in natural order with one padding piece after every 16 (a 64-value
// chunk occupies 272 bytes), so lanes that read consecutive chunks hit different LDS banks.
constexpr int kChunkPieces = 17;

__device__ __forceinline__ XChunk load_chunk(const float4* xs, int c)
{
    XChunk r;
    const float4* src = xs + c * kChunkPieces;
#pragma unroll
    for (int i = 0; i < 16; ++i) r.p[i] = src[i];
    return r;
}

// ---------------------------------------------------------------------------------------------------- Q8_0
// Unit = two consecutive 34-byte blocks (68 bytes, 4-byte aligned because a row holds an even number of blocks).
struct Q8_0Unit {
    static constexpr int kGridWords = 0;          // no codebook
    struct X { XChunk c; };
    struct Regs { u32x4 a, b, c, d; uint32_t e; };

    static __device__ __forceinline__ X load_x(const float4* x, int unit)
    {
        X r;
        r.c = load_chunk(x, unit);
        return r;
    }

    static __device__ __forceinline__ Regs load(const uint8_t* row, int unit)
    {
        const uint8_t* p = row + static_cast<uint32_t>(unit) * 68u;
        Regs r;
        r.a = ld128(p); r.b = ld128(p + 16); r.c = ld128(p + 32); r.d = ld128(p + 48);
        r.e = ld32(p + 64);
        return r;
    }

    static __device__ __forceinline__ float dot(const Regs& r, const X& x, int, const uint32_t*)
    {
        const uint32_t w[17] = {r.a[0], r.a[1], r.a[2], r.a[3], r.b[0], r.b[1], r.b[2], r.b[3], r.c[0], r.c[1], r.c[2],
                                r.c[3], r.d[0], r.d[1], r.d[2], r.d[3], r.e};
        const float d0 = half_bits_to_float(w[0]);
        const float d1 = half_bits_to_float(w[8] >> 16);
        float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t q = __builtin_amdgcn_alignbyte(w[i + 1], w[i], 2);  // quants of block 0 start at byte 2
            acc0 = dot4s(q, x.c.p[i], acc0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) acc1 = dot4s(w[9 + i], x.c.p[8 + i], acc1);
        return fmaf(d1, acc1, d0 * acc0);
    }
};

// ---------------------------------------------------------------------------------------------------- Q4_K
// Unit j of a super-block = sub-blocks 2j (low nibbles) and 2j+1 (high nibbles) of qs[32j .. 32j+31].
// sum_k x (s*q - m) = s * sum(q x) - m * sum(x); the two 32-wide sums of x are taken once per lane.
struct Q4KUnit {
    static constexpr int kGridWords = 0;          // no codebook
    struct X { XChunk c; float xs_lo, xs_hi; };
    struct Regs { u32x4 h, qa, qb; };

    static __device__ __forceinline__ X load_x(const float4* x, int unit)
    {
        X r;
        r.c = load_chunk(x, unit);
        float lo = 0.0f, hi = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            lo += sum4(r.c.p[i]);
            hi += sum4(r.c.p[8 + i]);
        }
        r.xs_lo = lo;
        r.xs_hi = hi;
        return r;
    }

    static __device__ __forceinline__ Regs load(const uint8_t* row, int unit)
    {
        const int sb = unit >> 2, j = unit & 3;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 144u;
        Regs r;
        r.h = *reinterpret_cast<const u32x4*>(blk);
        r.qa = *reinterpret_cast<const u32x4*>(blk + 16 + 32 * j);
        r.qb = *reinterpret_cast<const u32x4*>(blk + 32 + 32 * j);
        return r;
    }

    static __device__ __forceinline__ float dot(const Regs& r, const X& x, int unit, const uint32_t*)
    {
        const int j = unit & 3;
        const float d = half_bits_to_float(r.h[0]), dmin = half_bits_to_float(r.h[0] >> 16);
        uint32_t sc, mn;
        k4_scale_pair(r.h[1], r.h[2], r.h[3], j, sc, mn);
        const uint32_t q[8] = {r.qa[0], r.qa[1], r.qa[2], r.qa[3], r.qb[0], r.qb[1], r.qb[2], r.qb[3]};
        float lo = 0.0f, hi = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t l4 = opaque(q[i] & 0x0f0f0f0fu);
            const uint32_t h4 = opaque(q[i] & 0xf0f0f0f0u);   // 16 * high nibble; the 1/16 is folded into the scale
            lo = dot4u(l4, x.c.p[i], lo);
            hi = dot4u(h4, x.c.p[8 + i], hi);
        }
        const float s_lo = d * ubyte0(sc), s_hi = d * ubyte1(sc) * 0.0625f;
        const float m_lo = dmin * ubyte0(mn), m_hi = dmin * ubyte1(mn);
        float acc = s_lo * lo;
        acc = fmaf(s_hi, hi, acc);
        acc = fmaf(-m_lo, x.xs_lo, acc);
        acc = fmaf(-m_hi, x.xs_hi, acc);
        return acc;
    }
};

// ---------------------------------------------------------------------------------------------------- Q5_K
// As Q4_K plus one high bit per weight: bit g of qh[i] belongs to element i of sub-block g.
struct Q5KUnit {
    static constexpr int kGridWords = 0;          // no codebook
    using X = Q4KUnit::X;
    struct Regs { u32x4 h, ha, hb, qa, qb; };

    static __device__ __forceinline__ X load_x(const float4* x, int unit) { return Q4KUnit::load_x(x, unit); }

    static __device__ __forceinline__ Regs load(const uint8_t* row, int unit)
    {
        const int sb = unit >> 2, j = unit & 3;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 176u;
        Regs r;
        r.h = *reinterpret_cast<const u32x4*>(blk);
        r.ha = *reinterpret_cast<const u32x4*>(blk + 16);
        r.hb = *reinterpret_cast<const u32x4*>(blk + 32);
        r.qa = *reinterpret_cast<const u32x4*>(blk + 48 + 32 * j);
        r.qb = *reinterpret_cast<const u32x4*>(blk + 64 + 32 * j);
        return r;
    }

    static __device__ __forceinline__ float dot(const Regs& r, const X& x, int unit, const uint32_t*)
    {
        const int j = unit & 3;
        const float d = half_bits_to_float(r.h[0]), dmin = half_bits_to_float(r.h[0] >> 16);
        uint32_t sc, mn;
        k4_scale_pair(r.h[1], r.h[2], r.h[3], j, sc, mn);
        const uint32_t q[8] = {r.qa[0], r.qa[1], r.qa[2], r.qa[3], r.qb[0], r.qb[1], r.qb[2], r.qb[3]};
        const uint32_t hq[8] = {r.ha[0], r.ha[1], r.ha[2], r.ha[3], r.hb[0], r.hb[1], r.hb[2], r.hb[3]};
        float lo = 0.0f, hi = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t hb2 = hq[i] >> (2 * j);                       // bit 0: sub-block 2j, bit 1: sub-block 2j+1
            const uint32_t l5 = opaque((q[i] & 0x0f0f0f0fu) | ((hb2 << 4) & 0x10101010u));
            const uint32_t h5 = opaque(((q[i] >> 4) & 0x0f0f0f0fu) | ((hb2 << 3) & 0x10101010u));
            lo = dot4u(l5, x.c.p[i], lo);
            hi = dot4u(h5, x.c.p[8 + i], hi);
        }
        const float s_lo = d * ubyte0(sc), s_hi = d * ubyte1(sc);
        const float m_lo = dmin * ubyte0(mn), m_hi = dmin * ubyte1(mn);
        float acc = s_lo * lo;
        acc = fmaf(s_hi, hi, acc);
        acc = fmaf(-m_lo, x.xs_lo, acc);
        acc = fmaf(-m_hi, x.xs_hi, acc);
        return acc;
    }
};

// ---------------------------------------------------------------------------------------------------- Q6_K
// Unit (sb, half h, part p): elements 128h + 32e + 16p + i, i < 16, e < 4 - the four 16-runs that share
// ql[64h+16p ..], ql[64h+32+16p ..] and qh[32h+16p ..].  w = d*scale*(q - 32): sum(q x) - 32 sum16(x).
struct Q6KUnit {
    static constexpr int kGridWords = 0;          // no codebook
    struct X { float4 p[4][4]; float xs[4]; };   // [run e][piece]
    struct Regs { u32x4 la, lb, hh; u32x2 scw; uint32_t d; };

    static __device__ __forceinline__ X load_x(const float4* x, int unit)
    {
        const int sb = unit >> 2, h = (unit >> 1) & 1, p = unit & 1;
        X r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // run e covers pieces 8e + 4p .. +3 of half h: chunk 4 sb + 2 h + (e >> 1), piece 8 (e & 1) + 4 p + i
            const float4* src = x + (4 * sb + 2 * h + (e >> 1)) * kChunkPieces + 8 * (e & 1) + 4 * p;
            float t = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                r.p[e][i] = src[i];
                t += sum4(r.p[e][i]);
            }
            r.xs[e] = t;
        }
        return r;
    }

    static __device__ __forceinline__ Regs load(const uint8_t* row, int unit)
    {
        const int sb = unit >> 2, h = (unit >> 1) & 1, p = unit & 1;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 210u;
        Regs r;
        r.la = ld128(blk + 64 * h + 16 * p);
        r.lb = ld128(blk + 64 * h + 32 + 16 * p);
        r.hh = ld128(blk + 128 + 32 * h + 16 * p);
        r.scw = ld64(blk + 192 + 8 * h);
        r.d = ld16(blk + 208);
        return r;
    }

    static __device__ __forceinline__ float dot(const Regs& r, const X& x, int unit, const uint32_t*)
    {
        const int p = unit & 1;
        const float d = half_bits_to_float(r.d);
        float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t a = r.la[i], b = r.lb[i], q2 = r.hh[i];
            const uint32_t q1 = opaque((a & 0x0f0f0f0fu) | ((q2 << 4) & 0x30303030u));
            const uint32_t q2v = opaque((b & 0x0f0f0f0fu) | ((q2 << 2) & 0x30303030u));
            const uint32_t q3 = opaque(((a >> 4) & 0x0f0f0f0fu) | (q2 & 0x30303030u));
            const uint32_t q4 = opaque(((b >> 4) & 0x0f0f0f0fu) | ((q2 >> 2) & 0x30303030u));
            a0 = dot4u(q1, x.p[0][i], a0);
            a1 = dot4u(q2v, x.p[1][i], a1);
            a2 = dot4u(q3, x.p[2][i], a2);
            a3 = dot4u(q4, x.p[3][i], a3);
        }
        // int8 sub-scales 8h + 2e + p live in byte 2e + p of the 8 bytes loaded for half h
        const uint32_t s01 = r.scw[0] >> (8 * p), s23 = r.scw[1] >> (8 * p);
        const float sc0 = sbyte0(s01), sc1 = sbyte2(s01), sc2 = sbyte0(s23), sc3 = sbyte2(s23);
        float acc = (d * sc0) * fmaf(-32.0f, x.xs[0], a0);
        acc = fmaf(d * sc1, fmaf(-32.0f, x.xs[1], a1), acc);
        acc = fmaf(d * sc2, fmaf(-32.0f, x.xs[2], a2), acc);
        acc = fmaf(d * sc3, fmaf(-32.0f, x.xs[3], a3), acc);
        return acc;
    }
};

// ---------------------------------------------------------------------------------------------------- IQ2_S
// Unit gp of a super-block = 32-groups 2gp and 2gp+1.  Each octet: 10-bit index into the 1024-entry codebook held
// in LDS (8 magnitude bytes), 8 sign bits, 4-bit sub-scale shared by two octets.
struct IQ2SUnit {
    static constexpr int kGridWords = 2048;       // 1024 codebook entries of 8 magnitudes
    static __device__ __forceinline__ const uint32_t* grid_table() { return reinterpret_cast<const uint32_t*>(g_iq2s_grid); }
    struct X { XChunk c; };
    struct Regs { u32x2 qs, sg; uint32_t qh, scl, d; };

    static __device__ __forceinline__ X load_x(const float4* x, int unit)
    {
        X r;
        r.c = load_chunk(x, unit);
        return r;
    }

    static __device__ __forceinline__ Regs load(const uint8_t* row, int unit)
    {
        const int sb = unit >> 2, gp = unit & 3;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 82u;
        Regs r;
        r.qs = ld64(blk + 2 + 8 * gp);
        r.sg = ld64(blk + 34 + 8 * gp);
        r.qh = ld16(blk + 66 + 2 * gp);
        r.scl = ld16(blk + 74 + 2 * gp);
        r.d = ld16(blk);
        return r;
    }

    static __device__ __forceinline__ float signed_mag(float mag, uint32_t signs, int t)
    {
        const uint32_t sign = (signs << (31 - t)) & 0x80000000u;
        return __uint_as_float(__float_as_uint(mag) | sign);
    }

    static __device__ __forceinline__ float dot(const Regs& r, const X& x, int, const uint32_t* grid32)
    {
        const uint64_t* grid = reinterpret_cast<const uint64_t*>(grid32);
        const float d = half_bits_to_float(r.d);
        float acc = 0.0f;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const uint32_t q4 = r.qs[g], s4 = r.sg[g];
            const uint32_t hbits = (r.qh >> (8 * g)) & 0xffu;
            const uint32_t sc = (r.scl >> (8 * g)) & 0xffu;
#pragma unroll
            for (int o = 0; o < 4; ++o) {
                const uint32_t idx = ((q4 >> (8 * o)) & 0xffu) | (((hbits >> (2 * o)) & 3u) << 8);
                const uint64_t gv = grid[idx];
                const uint32_t glo = static_cast<uint32_t>(gv), ghi = static_cast<uint32_t>(gv >> 32);
                const uint32_t signs = (s4 >> (8 * o)) & 0xffu;
                const float4 xa = x.c.p[8 * g + 2 * o], xb = x.c.p[8 * g + 2 * o + 1];
                float t = 0.0f;
                t = fmaf(signed_mag(ubyte0(glo), signs, 0), xa.x, t);
                t = fmaf(signed_mag(ubyte1(glo), signs, 1), xa.y, t);
                t = fmaf(signed_mag(ubyte2(glo), signs, 2), xa.z, t);
                t = fmaf(signed_mag(ubyte3(glo), signs, 3), xa.w, t);
                t = fmaf(signed_mag(ubyte0(ghi), signs, 4), xb.x, t);
                t = fmaf(signed_mag(ubyte1(ghi), signs, 5), xb.y, t);
                t = fmaf(signed_mag(ubyte2(ghi), signs, 6), xb.z, t);
                t = fmaf(signed_mag(ubyte3(ghi), signs, 7), xb.w, t);
                const float sub = static_cast<float>((sc >> (4 * (o >> 1))) & 15u);
                const float db = (d * (0.5f + sub)) * 0.25f;
                acc = fmaf(db, t, acc);
            }
        }
        return acc;
    }
};

// ---------------------------------------------------------------------------------------------------- IQ3_S
// Unit u of a 110-byte super-block = groups 2u and 2u+1 (32 weights each): 16 index bytes, 2 high-bit bytes, 8 sign
// bytes, one byte holding both 4-bit scales.  w = (d * (1 + 2 s)) * magnitude * sign (qwen35_iq.cl:421-429).
struct IQ3SUnit {
    static constexpr int kGridWords = 512;        // 512 codebook entries of 4 magnitudes
    static __device__ __forceinline__ const uint32_t* grid_table() { return g_iq3s_grid; }
    struct X { XChunk c; };
    struct Regs { u32x4 qs; u32x2 sg; uint32_t qh, scl, d; };

    static __device__ __forceinline__ X load_x(const float4* x, int unit)
    {
        X r;
        r.c = load_chunk(x, unit);
        return r;
    }

    static __device__ __forceinline__ Regs load(const uint8_t* row, int unit)
    {
        const int sb = unit >> 2, u = unit & 3;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 110u;
        Regs r;
        r.qs = ld128(blk + 2 + 16 * u);
        r.sg = ld64(blk + 74 + 8 * u);
        r.qh = ld16(blk + 66 + 2 * u);
        r.scl = blk[106 + u];
        r.d = ld16(blk);
        return r;
    }

    static __device__ __forceinline__ float signed_mag(float mag, uint32_t signs, int t)
    {
        const uint32_t sign = (signs << (31 - t)) & 0x80000000u;
        return __uint_as_float(__float_as_uint(mag) | sign);
    }

    static __device__ __forceinline__ float dot(const Regs& r, const X& x, int, const uint32_t* grid)
    {
        const float d = half_bits_to_float(r.d);
        float acc = 0.0f;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const uint32_t hbits = (r.qh >> (8 * g)) & 0xffu;
            const uint32_t s4 = r.sg[g];
            float t = 0.0f;
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const uint32_t word = r.qs[2 * g + (q >> 2)];
                const uint32_t idx = ((word >> (8 * (q & 3))) & 0xffu) | (((hbits >> q) & 1u) << 8);
                const uint32_t gv = grid[idx];
                const uint32_t signs = (s4 >> (8 * (q >> 1) + 4 * (q & 1))) & 0xfu;
                const float4 xa = x.c.p[8 * g + q];
                t = fmaf(signed_mag(ubyte0(gv), signs, 0), xa.x, t);
                t = fmaf(signed_mag(ubyte1(gv), signs, 1), xa.y, t);
                t = fmaf(signed_mag(ubyte2(gv), signs, 2), xa.z, t);
                t = fmaf(signed_mag(ubyte3(gv), signs, 3), xa.w, t);
            }
            const uint32_t sub = (r.scl >> (4 * g)) & 15u;
            acc = fmaf(d * static_cast<float>(1u + 2u * sub), t, acc);
        }
        return acc;
    }
};

// ---------------------------------------------------------------------------------------------------- BF16
// Unquantized bfloat16 rows: a unit is 64 weights = 128 bytes; a bfloat16 is the upper half of its FP32 value.
struct BF16Unit {
    static constexpr int kGridWords = 0;
    struct X { XChunk c; };
    struct Regs { u32x4 v[8]; };

    static __device__ __forceinline__ X load_x(const float4* x, int unit)
    {
        X r;
        r.c = load_chunk(x, unit);
        return r;
    }

    static __device__ __forceinline__ Regs load(const uint8_t* row, int unit)
    {
        const uint8_t* p = row + static_cast<uint32_t>(unit) * 128u;
        Regs r;
#pragma unroll
        for (int i = 0; i < 8; ++i) r.v[i] = *reinterpret_cast<const u32x4*>(p + 16 * i);
        return r;
    }

    static __device__ __forceinline__ float dot(const Regs& r, const X& x, int, const uint32_t*)
    {
        float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const u32x4 w = r.v[i];
            const float4 xa = x.c.p[2 * i], xb = x.c.p[2 * i + 1];
            acc0 = fmaf(__uint_as_float(w[0] << 16), xa.x, acc0);
            acc1 = fmaf(__uint_as_float(w[0] & 0xffff0000u), xa.y, acc1);
            acc0 = fmaf(__uint_as_float(w[1] << 16), xa.z, acc0);
            acc1 = fmaf(__uint_as_float(w[1] & 0xffff0000u), xa.w, acc1);
            acc0 = fmaf(__uint_as_float(w[2] << 16), xb.x, acc0);
            acc1 = fmaf(__uint_as_float(w[2] & 0xffff0000u), xb.y, acc1);
            acc0 = fmaf(__uint_as_float(w[3] << 16), xb.z, acc0);
            acc1 = fmaf(__uint_as_float(w[3] & 0xffff0000u), xb.w, acc1);
        }
        return acc0 + acc1;
    }
};

// ---------------------------------------------------------------------------------------------- the kernel
// Launch shape of one block format: lanes per workgroup, waves per SIMD the register budget is sized for, and the
// number of weight register sets that rotate (DEPTH - 1 row steps are in flight while one is reduced): kDepth for a
// single mat-vec, kBatchDepth for the persistent batched kernel.  More bytes in flight than the memory system needs
// to cover its latency lowers the rate it sustains, so the single launch keeps the ring short.
template <class Q> struct Shape;
template <> struct Shape<Q8_0Unit> { static constexpr int kMaxT = 768, kWavesPerEu = 3, kDepth = 2, kBatchDepth = 3; };
template <> struct Shape<Q4KUnit> { static constexpr int kMaxT = 1024, kWavesPerEu = 4, kDepth = 3, kBatchDepth = 3; };
template <> struct Shape<Q5KUnit> { static constexpr int kMaxT = 768, kWavesPerEu = 3, kDepth = 3, kBatchDepth = 3; };
template <> struct Shape<Q6KUnit> { static constexpr int kMaxT = 768, kWavesPerEu = 3, kDepth = 2, kBatchDepth = 4; };
template <> struct Shape<IQ2SUnit> { static constexpr int kMaxT = 1024, kWavesPerEu = 4, kDepth = 2, kBatchDepth = 4; };
template <> struct Shape<IQ3SUnit> { static constexpr int kMaxT = 1024, kWavesPerEu = 4, kDepth = 2, kBatchDepth = 4; };
template <> struct Shape<BF16Unit> { static constexpr int kMaxT = 512, kWavesPerEu = 2, kDepth = 2, kBatchDepth = 2; };

// grid.x = workgroups striding over row steps, grid.y = input rows, blockDim.x = T (a multiple of 64).
// PRE selects what is done to the activations while they are staged: nothing; (x + residual) -> RMSNorm * gamma in the
// summation order of q35a_add_rms_norm / q35a_rms_norm (NNtrain.Arc/Kernels/qwen35_attention.cl:16-78: 128 lane-strided
// partial sums, halving tree); SiLU(x) * x2 (qwen35_attention.cl:38-43).  Every workgroup prepares the whole vector
// for itself; workgroup 0 also stores it (and the residual sum) where the caller asked.
// MR > 1 (plain launches with several input rows; the reference routes 1 < rows to a row-tiled kernel,
// NNtrain.Core/Modules/Qwen35QuantizedModel.cs:1340-1344): a workgroup multiplies every row step by MR input rows, so the
// weights are streamed once per MR rows.  A lane cannot hold MR x 64 activations in registers: the vectors stay in LDS and
// the lane re-reads its 64 values of a row for every step; the arithmetic and the summation order per input row are
// those of MR = 1, so results do not depend on how the rows were grouped.
// PAIR (a stacked gate | up projection, NNtrain.Core/Modules/Qwen35QuantizedModel.cs:489-496 runs the two and then
// q35a_silu_multiply): a row step is RS / 2 rows of the first half of the matrix and the matching rows of the second, and
// what is stored is SiLU(first) * second, so the product is formed once, by the workgroup that has both sums, instead of
// by every workgroup of the next launch.  Each sum has the bits of the unpaired launch.
template <class Q, int PRE = kPreNone, int MR = 1, bool PAIR = false>
__global__ __launch_bounds__(Shape<Q>::kMaxT) __attribute__((amdgpu_waves_per_eu(Shape<Q>::kWavesPerEu, Shape<Q>::kWavesPerEu)))
void matvec_rowstep_kernel(MatvecArgs a, const float* __restrict__ bias)
{
    static_assert(MR == 1 || PRE == kPreNone, "row tiling is for plain launches");
    static_assert(!PAIR || MR == 1, "paired halves are for single input rows");
    constexpr int kDepth = Shape<Q>::kDepth;
    __shared__ float part[2][MR * kMaxWG];
    __shared__ __attribute__((aligned(8))) uint32_t grid[Q::kGridWords ? Q::kGridWords : 2];

    const int tid = threadIdx.x;
    const int upr = a.units_per_row, rs = a.rows_per_step;
    const int rl = upr == 1 ? tid : static_cast<int>(__umulhi(static_cast<uint32_t>(tid), a.magic));  // row within a step
    const int c = tid - rl * upr;                                                                    // unit within the row
    const bool owner = rl < rs;
    const int row0 = blockIdx.y * MR;                          // first input row of this workgroup
    const float* x = a.x + static_cast<size_t>(row0) * a.in_w;
    float* y = a.y + static_cast<size_t>(row0) * a.out_w;
    const int last_row = a.out_w - 1;
    const int half = rs >> 1;                                  // PAIR: rows of each half per step
    // the matrix row of row `r` of step `st` (PAIR: rows 0 .. half - 1 of a step lie in the first half of the matrix)
    auto row_of = [&](int st, int r) {
        if constexpr (PAIR) return r < half ? st * half + r : a.pair_rows + st * half + (r - half);
        else return st * rs + r;
    };
    auto row_valid = [&](int st, int r) {
        if constexpr (PAIR) return st * half + (r < half ? r : r - half) < a.pair_rows;
        else return st * rs + r < a.out_w;
    };

    // Loads are unconditional: rows past the end re-read the last row, spare lanes re-read row 0 (both stay in L2),
    // and their products are dropped.  That keeps the stream free of branches between loads.
    auto fetch = [&](int step) {
        const int row = owner ? min(row_of(step, rl), last_row) : 0;
        return Q::load(a.w + static_cast<size_t>(row) * a.row_bytes, c);
    };

    // The activations are requested first (they come from L2 and return ahead of the weight stream), staged through
    // LDS so that the workgroup reads them from memory once, and then kept in registers: 64 per lane.
    extern __shared__ float4 xstage[];
    const int pieces = a.in_w >> 2;
    const float4* xg = reinterpret_cast<const float4*>(x);
    const int T = blockDim.x;
    // (a vector gathered by heads is shorter than in_w: its pieces are fetched through the index map further down)
    float4 xv0 = PRE != kPreHeadGather && tid < pieces ? xg[tid] : make_float4(0.f, 0.f, 0.f, 0.f);
    float4 xv1 = PRE != kPreHeadGather && tid + T < pieces ? xg[tid + T] : make_float4(0.f, 0.f, 0.f, 0.f);
    // A plain launch with a long input (a down projection) asks for up to six more pieces per lane here, ahead of the
    // weights: whatever is requested after the weight prefetch comes back behind it, one round trip per piece.
    constexpr int kMorePieces = PRE == kPreNone && MR == 1 ? 6 : 0;
    float4 xw[kMorePieces ? kMorePieces : 1];
    if constexpr (kMorePieces > 0) {
#pragma unroll
        for (int i = 0; i < kMorePieces; ++i)
            xw[i] = tid + (2 + i) * T < pieces ? xg[tid + (2 + i) * T] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    const float4* x2g = reinterpret_cast<const float4*>(a.x2);
    const float4* gg = reinterpret_cast<const float4*>(a.gamma);
    const bool second = PRE == kPreSiluMultiply || (PRE == kPreRmsNorm && a.x2 != nullptr);
    float4 sv0 = make_float4(0.f, 0.f, 0.f, 0.f), sv1 = sv0, gv0 = sv0, gv1 = sv0;
    if constexpr (PRE != kPreNone) {
        if (second && tid < pieces) sv0 = x2g[tid];
        if (second && tid + T < pieces) sv1 = x2g[tid + T];
    }
    if constexpr (PRE == kPreRmsNorm) {
        if (tid < pieces) gv0 = gg[tid];
        if (tid + T < pieces) gv1 = gg[tid + T];
    }
    // The compute unit returns vector-memory data in the order the requests were queued, across waves.  This barrier
    // (no memory wait, just a rendezvous) puts every wave's activation requests ahead of every wave's weight
    // requests, so staging does not wait for the first weight rows to come back from HBM.
    __syncthreads();

    const int stride = gridDim.x;
    int step = blockIdx.x;
    typename Q::Regs regs[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d) regs[d] = fetch(step + d * stride);

    const bool scribe = blockIdx.x == 0;      // the workgroup that stores the prepared vector
    if constexpr (PRE == kPreSiluMultiply) {
        float4* xo = scribe ? reinterpret_cast<float4*>(a.x_out) : nullptr;
        xv0 = silu_mul4(xv0, sv0);
        xv1 = silu_mul4(xv1, sv1);
        if (tid < pieces) { xstage[tid + (tid >> 4)] = xv0; if (xo) xo[tid] = xv0; }
        if (tid + T < pieces) { xstage[tid + T + ((tid + T) >> 4)] = xv1; if (xo) xo[tid + T] = xv1; }
        for (int L = tid + 2 * T; L < pieces; L += T) {
            const float4 v = silu_mul4(xg[L], x2g[L]);
            xstage[L + (L >> 4)] = v;
            if (xo) xo[L] = v;
        }
    } else if constexpr (PRE == kPreRmsNorm) {
        float4* so = scribe ? reinterpret_cast<float4*>(a.sum_out) : nullptr;
        float4* xo = scribe ? reinterpret_cast<float4*>(a.x_out) : nullptr;
        // the residual stream first
        if (second) {                      // (without a residual the input keeps its bits: -0 stays -0)
            xv0 = add4(xv0, sv0);
            xv1 = add4(xv1, sv1);
        }
        if (tid < pieces) { xstage[tid + (tid >> 4)] = xv0; if (so) so[tid] = xv0; }
        if (tid + T < pieces) { xstage[tid + T + ((tid + T) >> 4)] = xv1; if (so) so[tid + T] = xv1; }
        for (int L = tid + 2 * T; L < pieces; L += T) {
            const float4 v = second ? add4(xg[L], x2g[L]) : xg[L];
            xstage[L + (L >> 4)] = v;
            if (so) so[L] = v;
        }
        __syncthreads();
        // 128 lane-strided partial sums of squares ...
        const float* xs = reinterpret_cast<const float*>(xstage);
        float sq = 0.0f;
        if (tid < 128) {
            // (eight reads on their way at a time instead of one dependent read per addition; the additions keep their order)
            auto at = [&](int j) {
                const int L = j >> 2;
                return xs[4 * (L + (L >> 4)) + (j & 3)];
            };
            int j = tid;
            for (; j + 7 * 128 < a.in_w; j += 8 * 128) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = at(j + u * 128);
#pragma unroll
                for (int u = 0; u < 8; ++u) sq += v[u] * v[u];
            }
            for (; j < a.in_w; j += 128) {
                const float v = at(j);
                sq += v * v;
            }
        }
        // ... then the halving tree: 64 through LDS (the two waves that hold the partials), 32 .. 1 inside wave 0
        if (tid >= 64 && tid < 128) part[0][tid - 64] = sq;
        __syncthreads();
        if (tid < 64) {
            sq += part[0][tid];
            const uint32_t u = __float_as_uint(sq);
            auto s32 = __builtin_amdgcn_permlane32_swap(u, u, false, false);
            sq = __uint_as_float(s32[0]) + __uint_as_float(s32[1]);              // lanes 0-31: s[t] + s[t+32]
            const uint32_t v = __float_as_uint(sq);
            auto s16 = __builtin_amdgcn_permlane16_swap(v, v, false, false);
            sq = __uint_as_float(s16[0]) + __uint_as_float(s16[1]);              // lanes 0-15: s[t] + s[t+16]
            sq += dpp_mov<0x108>(sq);                                             // row_shl:8  s[t] + s[t+8]
            sq += dpp_mov<0x104>(sq);                                             // row_shl:4
            sq += dpp_mov<0x102>(sq);                                             // row_shl:2
            sq += dpp_mov<0x101>(sq);                                             // row_shl:1
            if (tid == 0) part[1][0] = sq;
        }
        __syncthreads();
        const float inverse = 1.0f / sqrtf(part[1][0] / static_cast<float>(a.in_w) + a.epsilon);
        auto normalize = [&](float4 h, const float4 g) {
            return make_float4(h.x * inverse * g.x, h.y * inverse * g.y, h.z * inverse * g.z, h.w * inverse * g.w);
        };
        // every lane rewrites the pieces it staged itself
        if (tid < pieces) { xv0 = normalize(xv0, gv0); xstage[tid + (tid >> 4)] = xv0; if (xo) xo[tid] = xv0; }
        if (tid + T < pieces) { xv1 = normalize(xv1, gv1); xstage[tid + T + ((tid + T) >> 4)] = xv1; if (xo) xo[tid + T] = xv1; }
        for (int L = tid + 2 * T; L < pieces; L += T) {
            const float4 v = normalize(xstage[L + (L >> 4)], gg[L]);
            xstage[L + (L >> 4)] = v;
            if (xo) xo[L] = v;
        }
    } else if constexpr (PRE == kPreHeadGather) {
        for (int L = tid; L < pieces; L += T) {
            const int h = L / a.head4;
            xstage[L + (L >> 4)] = xg[(h / a.head_group) * a.head4 + (L - h * a.head4)];
        }
    } else {
        if (tid < pieces) xstage[tid + (tid >> 4)] = xv0;
        if (tid + T < pieces) xstage[tid + T + ((tid + T) >> 4)] = xv1;
        if constexpr (kMorePieces > 0) {
#pragma unroll
            for (int i = 0; i < kMorePieces; ++i) {
                const int L = tid + (2 + i) * T;
                if (L < pieces) xstage[L + (L >> 4)] = xw[i];
            }
        }
        for (int L = tid + (2 + kMorePieces) * T; L < pieces; L += T) xstage[L + (L >> 4)] = xg[L];
        // the other input rows of the tile, each in a staging area of its own (rows past the last one: zeros)
        for (int m = 1; m < MR; ++m) {
            float4* xm = xstage + m * kChunkPieces * upr;
            const bool have = row0 + m < a.rows;
            for (int L = tid; L < pieces; L += T)
                xm[L + (L >> 4)] = have ? xg[m * pieces + L] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    if constexpr (Q::kGridWords > 0)
        for (int i = tid; i < Q::kGridWords; i += T) grid[i] = Q::grid_table()[i];
    __syncthreads();
    typename Q::X xr{};
    if constexpr (MR == 1) xr = Q::load_x(xstage, owner ? c : 0);

    // Row results are collected in LDS and stored to memory in bursts (when the buffer is full, and at the end), so
    // the steady state has no vector-memory traffic besides the weight stream.
    __shared__ float ybuf[kYBuf];
    const int wave = tid >> 6, lane = tid & 63, waves = T >> 6;
    int buf = 0;
    int held = 0;                 // steps whose rows sit in ybuf
    int first_held = step;        // step number of ybuf[0 .. rs)
    auto flush = [&]() {
        __syncthreads();
        if constexpr (PAIR) {
            for (int i = tid; i < held * half; i += T) {
                const int j = i / half, r = i - j * half;
                const int row = (first_held + j * stride) * half + r;
                if (row < a.pair_rows) y[row] = silu_mul1(ybuf[j * rs + r], ybuf[j * rs + half + r]);
            }
            held = 0;
            return;
        }
        for (int i = tid; i < held * rs * MR; i += T) {
            const int j = i / (rs * MR), rem = i - j * rs * MR;
            const int m = MR == 1 ? 0 : rem / rs;
            const int row = (first_held + j * stride) * rs + (rem - m * rs);
            if (row < a.out_w && (MR == 1 || row0 + m < a.rows)) {
                float v = ybuf[i];
                if (a.lora_rank > 0) {      // the branch of q35l_*_sg16_lora (NNtrain.Arc/Kernels/qwen35_linear_fast.cl:262-268)
                    const float* br = a.lora_b + static_cast<size_t>(row) * a.lora_rank;
                    float sum = 0.0f;
                    int r = 0;
                    // (four coefficients a load where the rows of b are 16-byte aligned; the same products in the same order)
                    if ((a.lora_rank & 3) == 0 && (reinterpret_cast<uintptr_t>(a.lora_b) & 15u) == 0) {
                        for (; r < a.lora_rank; r += 4) {
                            const float4 b4 = *reinterpret_cast<const float4*>(br + r);
                            sum = fmaf(a.lora_z[r], b4.x, sum);
                            sum = fmaf(a.lora_z[r + 1], b4.y, sum);
                            sum = fmaf(a.lora_z[r + 2], b4.z, sum);
                            sum = fmaf(a.lora_z[r + 3], b4.w, sum);
                        }
                    }
                    for (; r < a.lora_rank; ++r) sum = fmaf(a.lora_z[r], br[r], sum);
                    v = v + a.lora_scale * sum;
                }
                y[static_cast<size_t>(m) * a.out_w + row] = a.addend ? a.addend[row] + v : v;
            }
        }
        held = 0;
    };
    auto finish = [&](const typename Q::Regs& r, int st) {
        if constexpr (MR == 1) {
            part[buf][tid] = Q::dot(r, xr, c, grid);
        } else {
#pragma unroll 1
            for (int m = 0; m < MR; ++m) {
                if (row0 + m < a.rows) {          // (workgroup-uniform)
                    const typename Q::X xm = Q::load_x(xstage + m * kChunkPieces * upr, owner ? c : 0);
                    part[buf][m * kMaxWG + tid] = Q::dot(r, xm, c, grid);
                }
            }
        }
        __syncthreads();
        for (int rr = wave; rr < rs * MR; rr += waves) {
            const int m = MR == 1 ? 0 : rr / rs, r0 = rr - m * rs;
            const int row = row_of(st, r0);
            if (row_valid(st, r0) && (MR == 1 || row0 + m < a.rows)) {
                float t = 0.0f;
                for (int u = lane; u < upr; u += 64) t += part[buf][m * kMaxWG + r0 * upr + u];
                t = wave_sum(t);
                // the row index is wave-uniform: the bias comes through the scalar cache and does not wait on the
                // vector-memory counter that the prefetched weights are tracked by
                const int urow = __builtin_amdgcn_readfirstlane(row);
                if (lane == 0) ybuf[(held * MR + m) * rs + r0] = (bias ? bias[urow] : 0.0f) + t;
            }
        }
        buf ^= 1;
        ++held;
    };

    // The loop runs whole turns of the register ring and has one exit, at the turn boundary: an exit in the middle of
    // a turn would join the loop's back edge right after a register set was refilled, and the wait for that set at the
    // loop head would then have to be "everything has arrived", which drains the prefetch queue every turn.
    while (step + (kDepth - 1) * stride < a.steps) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            regs[(d + kDepth - 1) % kDepth] = fetch(step + (kDepth - 1) * stride);
            finish(regs[d], step);
            step += stride;
        }
        if ((held + kDepth) * rs * MR > kYBuf) {         // rare: only matrices with very many rows per workgroup get here
            flush();
            __builtin_amdgcn_s_waitcnt(kWaitVm0);
            __syncthreads();
            first_held = step;
        }
    }
    // fewer than kDepth steps are left, and their weights are already in flight
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d) {
        if (step < a.steps) {
            finish(regs[d], step);
            step += stride;
        }
    }
    flush();
}

// ------------------------------------------------------------------------------------------- batched kernel
// One entry of the device table of a batched launch (see matvec_batch_kernel for the chunk sequence).
// Pointers read from a table are generic ("flat") to the device compiler; flat loads tick the LDS counter as well as
// the vector-memory one.  The device pass therefore declares them as global-address-space pointers.
#if defined(__HIP_DEVICE_COMPILE__)
#define NNHIP_GLOBAL_PTR __attribute__((address_space(1)))
#define NNHIP_CONST_PTR __attribute__((address_space(4)))
#else
#define NNHIP_GLOBAL_PTR
#define NNHIP_CONST_PTR
#endif
struct BatchEntry {
    const NNHIP_GLOBAL_PTR float* x;
    const NNHIP_GLOBAL_PTR uint8_t* w;
    const NNHIP_GLOBAL_PTR float* bias;
    NNHIP_GLOBAL_PTR float* y;
    int in_w;
    int out_w;
    int upr;          // units per row
    int rs;           // rows per step
    int steps;
    uint32_t row_bytes;
    uint32_t magic;
    int first_chunk;  // offset of the matrix in the global chunk sequence
    int chunks;       // ceil(steps / DEPTH)
    int pad_[2];
};

// Persistent form of matvec_rowstep_kernel: the weight prefetch runs ahead across matrix boundaries, so the stream
// from HBM never drains between the mat-vecs of a batch.
//
// The steps of a matrix are grouped in chunks of DEPTH consecutive steps (the last chunk of a matrix may be short);
// the chunks of all matrices form one global sequence and chunk j goes to workgroup j % G.  A chunk is exactly one turn
// of the rotating register sets, so a workgroup can only change matrix at the top of a turn, and it stays with a
// matrix for DEPTH steps even when the matrix has few rows (small matrices of a batch are worked on side by side by
// different workgroups).
//
// On entering a matrix a lane re-derives its (row, unit) slot and swaps in that matrix' activations.  Those are
// pumped ahead of time: once the staging area in LDS has been read by everyone, each step requests two float4 per lane
// of the NEXT matrix' vector into a holding register pair and the following step moves them to LDS, so the vector is
// usually complete when the reduction reaches that matrix and the switch costs one barrier and 16 LDS reads.  What the
// pump did not get to is fetched at the switch (the stream stalls once).
template <class Q>
__global__ __launch_bounds__(Shape<Q>::kMaxT) __attribute__((amdgpu_waves_per_eu(Shape<Q>::kWavesPerEu, Shape<Q>::kWavesPerEu)))
void matvec_batch_kernel(const BatchEntry* __restrict__ table_arg, int total_chunks)
{
    constexpr int kDepth = Shape<Q>::kBatchDepth;
    // The table and the bias vectors are read-only for the whole launch and always indexed with workgroup-uniform
    // values: reading them through the constant address space makes those reads scalar loads, which do not tick the
    // vector-memory counter.  A vector load there would make its user wait for every prefetched weight load as well
    // (the counter completes in order), draining the ring once per step.
    const NNHIP_CONST_PTR BatchEntry* table = (const NNHIP_CONST_PTR BatchEntry*)table_arg;
    __shared__ float part[2][kMaxWG];
    __shared__ __attribute__((aligned(8))) uint32_t grid[Q::kGridWords ? Q::kGridWords : 2];
    extern __shared__ float4 xstage[];

    const int tid = threadIdx.x, T = blockDim.x, G = gridDim.x;
    const int wave = tid >> 6, lane = tid & 63, waves = T >> 6;
    if constexpr (Q::kGridWords > 0)
        for (int i = tid; i < Q::kGridWords; i += T) grid[i] = Q::grid_table()[i];

    auto uni = [](int v) { return __builtin_amdgcn_readfirstlane(v); };   // pins workgroup-uniform state to SGPRs
    auto slot = [&](const BatchEntry& e, int& rl, int& c, bool& owner) {
        rl = e.upr == 1 ? tid : static_cast<int>(__umulhi(static_cast<uint32_t>(tid), e.magic));
        c = tid - rl * e.upr;
        owner = rl < e.rs;
    };
    auto find = [&](int m, int chunk) {       // index of the entry that holds global chunk `chunk`, searching from m
        while (chunk >= table[m].first_chunk + table[m].chunks) ++m;
        return uni(m);
    };

    // ---- weight prefetch side: entry `fe`, this lane's slot in it, the chunk being fetched
    int f_m = -1, f_rl = 0, f_c = 0, f_chunk = blockIdx.x;
    bool f_owner = false;
    BatchEntry fe{};
    auto fetch_enter = [&]() {                 // called when f_chunk has moved to a new chunk
        if (f_chunk < total_chunks && (f_m < 0 || f_chunk >= fe.first_chunk + fe.chunks)) {
            f_m = find(f_m < 0 ? 0 : f_m + 1, f_chunk);
            fe = table[f_m];
            slot(fe, f_rl, f_c, f_owner);
        }
    };
    auto fetch = [&](int d) {                  // step d of chunk f_chunk; past the end it re-reads a valid row
        const int s = f_chunk < total_chunks ? (f_chunk - fe.first_chunk) * kDepth + d : 0;
        const int row = f_owner ? min(s * fe.rs + f_rl, fe.out_w - 1) : 0;
        return Q::load((const uint8_t*)(fe.w + static_cast<size_t>(row) * fe.row_bytes), f_c);
    };

    // ---- activation pump: matrix p_m is being staged in rounds of 2T pieces; `held` is the round in the holding pair
    int p_m = -1, p_round = 0, p_rounds = 0, p_pieces = 0, held = -1;
    const NNHIP_GLOBAL_PTR float4* p_x = nullptr;
    float4 xh0 = make_float4(0.f, 0.f, 0.f, 0.f), xh1 = xh0;
    bool staging_free = true;
    auto pump_issue = [&]() {
        const int base = p_round * 2 * T;
        if (base + tid < p_pieces) xh0 = p_x[base + tid];
        if (base + T + tid < p_pieces) xh1 = p_x[base + T + tid];
        held = p_round;
        p_round = uni(p_round + 1);
    };
    auto pump_store = [&]() {
        const int L0 = held * 2 * T + tid, L1 = L0 + T;
        if (L0 < p_pieces) xstage[L0 + (L0 >> 4)] = xh0;
        if (L1 < p_pieces) xstage[L1 + (L1 >> 4)] = xh1;
        held = -1;
    };
    auto pump_target = [&](int m) {
        p_m = m;
        p_x = (const NNHIP_GLOBAL_PTR float4*)table[m].x;
        p_pieces = uni(table[m].in_w >> 2);
        p_rounds = uni((p_pieces + 2 * T - 1) / (2 * T));
        p_round = 0;
        held = -1;
    };
    auto pump_beat = [&]() {
        if (p_m >= 0) {
            if (held >= 0) pump_store();
            if (staging_free && p_round < p_rounds) pump_issue();
        }
    };

    // ---- reduction side
    int c_m = -1, c_rl = 0, c_c = 0, c_chunk = blockIdx.x;
    bool c_owner = false;
    BatchEntry ce{};
    typename Q::X xr{};
    int buf = 0;
    auto enter = [&](int m) {
        if (p_m != m) pump_target(m);        // nothing was pumped for this matrix (first matrix of the workgroup)
        if (held >= 0) pump_store();
        while (p_round < p_rounds) {          // what the pump did not get to: fetched here, the stream stalls
            pump_issue();
            pump_store();
        }
        c_m = m;
        ce = table[m];
        slot(ce, c_rl, c_c, c_owner);
        __syncthreads();
        xr = Q::load_x(xstage, c_owner ? c_c : 0);
        staging_free = false;
        // next matrix this workgroup will meet: its first chunk at or beyond the end of this matrix
        p_m = -1;
        const int end = ce.first_chunk + ce.chunks;
        const int ahead = uni(c_chunk + (end - c_chunk + G - 1) / G * G);
        if (ahead < total_chunks) pump_target(find(m + 1, ahead));
    };
    auto finish = [&](const typename Q::Regs& r, int d) {
        const int st = (c_chunk - ce.first_chunk) * kDepth + d;
        if (st < ce.steps) {                  // the last chunk of a matrix may be short (uniform)
            part[buf][tid] = Q::dot(r, xr, c_c, grid);
            __syncthreads();
            staging_free = true;
            for (int rr = wave; rr < ce.rs; rr += waves) {
                const int row = st * ce.rs + rr;
                if (row < ce.out_w) {
                    float t = 0.0f;
                    for (int u = lane; u < ce.upr; u += 64) t += part[buf][rr * ce.upr + u];
                    t = wave_sum(t);
                    const int urow = __builtin_amdgcn_readfirstlane(row);
                    const NNHIP_CONST_PTR float* cbias = (const NNHIP_CONST_PTR float*)ce.bias;
                    if (lane == 0) ce.y[urow] = (cbias ? cbias[urow] : 0.0f) + t;
                }
            }
            buf ^= 1;
        }
    };

    // One turn = one chunk.  At step d of the reduction the prefetch is kDepth - 1 steps ahead: steps d + kDepth - 1 of
    // this chunk while they exist, then the first steps of the workgroup's next chunk.
    typename Q::Regs regs[kDepth];
    fetch_enter();
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d) regs[d] = fetch(d);
    while (c_chunk < total_chunks) {
        if (c_m < 0 || c_chunk >= ce.first_chunk + ce.chunks) enter(find(c_m < 0 ? 0 : c_m + 1, c_chunk));
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            if (d == 0) {
                regs[kDepth - 1] = fetch(kDepth - 1);
            } else {
                if (d == 1) {
                    f_chunk += G;
                    fetch_enter();
                }
                regs[d - 1] = fetch(d - 1);
            }
            pump_beat();
            finish(regs[d], d);
        }
        c_chunk += G;
    }
}

// Slow path for Q8_0 rows with an odd number of blocks (row starts are then only 2-byte aligned and blocks cannot
// be paired): one wave per output, lanes stride over single blocks.
__global__ __launch_bounds__(256) void matvec_q8_0_oddrow_kernel(MatvecArgs a)
{
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int o = blockIdx.x * 4 + wave;
    const int m = blockIdx.y;
    if (o >= a.out_w) return;
    const uint8_t* row = a.w + static_cast<size_t>(o) * a.row_bytes;
    const float* x = a.x + static_cast<size_t>(m) * a.in_w;
    const int blocks = a.in_w >> 5;
    float t = 0.0f;
    for (int b = lane; b < blocks; b += 64) {
        const uint8_t* p = row + b * 34;
        const float d = half_bits_to_float(ld16(p));
        float acc = 0.0f;
        for (int i = 0; i < 32; ++i) acc = fmaf(static_cast<float>(static_cast<int8_t>(p[2 + i])), x[b * 32 + i], acc);
        t = fmaf(d, acc, t);
    }
    t = wave_sum(t);
    if (lane == 0) a.y[static_cast<size_t>(m) * a.out_w + o] = (a.bias ? a.bias[o] : 0.0f) + t;
}

struct Geometry {
    int threads;        // T
    int rows_per_step;  // RS
    int steps;
    int groups;
};

// Picks RS (whole rows per step) and from it the workgroup size.  Every workgroup runs ceil(steps / groups) rounds of
// RS rows, so the launch lasts about rounds * RS row-times.  The largest RS that fits max_t lanes keeps the most
// bytes in flight; a smaller one is taken only if it saves at least 2 % of rounds * RS.  `rs_cap` bounds RS from above:
// a workgroup parks the results of a whole turn of the register ring (depth steps of RS rows for each of the MR input
// rows of the tile) in its result buffer before it can flush, so depth * RS * MR must fit kYBuf.  The cap only binds
// for rows of one to five units; a row's bits do not depend on RS.
bool plan(int in_w, int out_w, int compute_units, int max_t, int rs_cap, Geometry* g, bool pair = false)
{
    const int upr = in_w / kUnitW;
    if (upr < 1 || upr > max_t || rs_cap < 1) return false;
    int rs_max = max_t / upr;
    if (rs_max > rs_cap) rs_max = rs_cap;
    const int rs_min = (3 * rs_max + 3) / 4;     // never give up more than a quarter of the lanes
    int best_rs = 0;
    long best_cost = 0;
    if (pair) {
        // a step is RS / 2 rows of each half of the matrix
        if (rs_max < 2 || (out_w & 1)) return false;
        rs_max &= ~1;
    }
    for (int rs = rs_max; rs >= rs_min && rs >= 1; rs -= pair ? 2 : 1) {
        const int steps = (out_w + rs - 1) / rs;
        const int rounds = (steps + compute_units - 1) / compute_units;
        const long cost = static_cast<long>(rounds) * rs;
        if (!best_rs || cost * 100 < best_cost * 98) {   // a smaller step must save at least 2 %
            best_rs = rs;
            best_cost = cost;
        }
    }
    if (best_rs > out_w) best_rs = out_w;   // tiny matrices: shrink to the rows there are
    g->rows_per_step = best_rs;
    g->threads = (best_rs * upr + 63) / 64 * 64;
    g->steps = (out_w + best_rs - 1) / best_rs;
    g->groups = g->steps < compute_units ? g->steps : compute_units;
    return true;
}

// Dynamic LDS a row-tiled launch may use: every further input row of the tile costs 8 KB of static partial sums.
constexpr int max_dynamic_lds(int mr) { return kMaxDynamicLds - (mr - 1) * 2 * kMaxWG * static_cast<int>(sizeof(float)); }

// Input rows that share one pass over the weights.  Four (or two) when their staging areas fit LDS, and only for the
// formats whose single-row kernel waits on memory: measured on 21504x5376 Q8_0, 4 rows take 50 us instead of 75 us; the
// K-quants, bound by their arithmetic, got slower (17408x5120 Q4_K, 4 rows: 50 us against 45 us), so they keep one row
// per pass.
template <class Q, int PRE>
int row_tile_of(int rows, size_t lds_one_row)
{
    if constexpr (PRE == kPreNone && (std::is_same<Q, Q8_0Unit>::value || std::is_same<Q, BF16Unit>::value)) {
        if (rows >= 3 && 4 * lds_one_row <= static_cast<size_t>(max_dynamic_lds(4))) return 4;
        if (rows >= 2 && 2 * lds_one_row <= static_cast<size_t>(max_dynamic_lds(2))) return 2;
    }
    return 1;
}

// The whole launch shape of matvec_rowstep_kernel<Q, PRE, MR> for one call; false if a row does not fit a workgroup.
template <class Q, int PRE>
bool rowstep_shape(int rows, int in_w, int out_w, int compute_units, int* mr, Geometry* g, bool pair = false)
{
    const size_t lds = static_cast<size_t>(kChunkPieces) * (in_w / kUnitW) * sizeof(float4);
    *mr = pair ? 1 : row_tile_of<Q, PRE>(rows, lds);
    if (!plan(in_w, out_w, compute_units, Shape<Q>::kMaxT, kYBuf / (Shape<Q>::kDepth * *mr), g, pair)) return false;
    if (PRE == kPreRmsNorm && g->threads < 128) g->threads = 128;     // the norm's partial sums take 128 lanes
    return true;
}

template <class Q, int PRE, int MR, bool PAIR = false>
hipError_t launch_rowstep_tiled(Lane* lane, const MatvecArgs& args, const Geometry& g, int rows, size_t lds)
{
    // what the kernel's result buffer and partial-sum arrays assume (see plan)
    if (Shape<Q>::kDepth * g.rows_per_step * MR > kYBuf || g.threads > Shape<Q>::kMaxT ||
        g.rows_per_step * args.units_per_row > g.threads)
        return hipErrorInvalidConfiguration;
    static LdsLimit big_lds;
    if (lds > 32 * 1024) {
        const hipError_t e = big_lds.ensure(lane->device, reinterpret_cast<const void*>(&matvec_rowstep_kernel<Q, PRE, MR, PAIR>),
                                            max_dynamic_lds(MR));
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((matvec_rowstep_kernel<Q, PRE, MR, PAIR>), dim3(g.groups, (rows + MR - 1) / MR), dim3(g.threads), lds,
                       lane->stream, args, args.bias);
    return hipGetLastError();
}

template <class Q, int PRE = kPreNone>
hipError_t launch_rowstep(Lane* lane, MatvecArgs args, int rows)
{
    Geometry g;
    int mr = 1;
    const bool pair = args.pair_rows > 0;
    if (!rowstep_shape<Q, PRE>(rows, args.in_w, args.out_w, lane->compute_units, &mr, &g, pair)) return hipErrorInvalidValue;
    args.rows_per_step = g.rows_per_step;
    args.steps = g.steps;
    args.rows = rows;
    const size_t lds = static_cast<size_t>(kChunkPieces) * args.units_per_row * sizeof(float4);
    if constexpr (PRE == kPreNone || PRE == kPreRmsNorm) {
        if (pair) return launch_rowstep_tiled<Q, PRE, 1, true>(lane, args, g, rows, lds);
    } else {
        if (pair) return hipErrorInvalidValue;
    }
    if constexpr (PRE == kPreNone && (std::is_same<Q, Q8_0Unit>::value || std::is_same<Q, BF16Unit>::value)) {
        if (mr == 4) return launch_rowstep_tiled<Q, PRE, 4>(lane, args, g, rows, 4 * lds);
        if (mr == 2) return launch_rowstep_tiled<Q, PRE, 2>(lane, args, g, rows, 2 * lds);
    }
    return launch_rowstep_tiled<Q, PRE, 1>(lane, args, g, rows, lds);
}


// Launches the persistent kernel over the entries of one block format; `table` is their slice of the device table.
template <class Q>
hipError_t launch_batch_of(Lane* lane, const BatchEntry* table, int total_chunks, int max_in_w)
{
    const size_t lds = static_cast<size_t>(kChunkPieces) * (max_in_w / kUnitW) * sizeof(float4);
    static LdsLimit big_lds;
    if (lds > 48 * 1024) {
        const hipError_t e = big_lds.ensure(lane->device, reinterpret_cast<const void*>(&matvec_batch_kernel<Q>), kMaxDynamicLds);
        if (e != hipSuccess) return e;
    }
    const int groups = total_chunks < lane->compute_units ? total_chunks : lane->compute_units;
    hipLaunchKernelGGL(matvec_batch_kernel<Q>, dim3(groups), dim3(Shape<Q>::kMaxT), lds, lane->stream, table, total_chunks);
    return hipGetLastError();
}

// The descriptor table reaches the device as kernel arguments: a chunk of entries is passed by value to a one-workgroup
// kernel that stores it.  The write is ordered on the lane's stream like the launches that read the table, so a table
// can be rewritten without waiting for the host or the device, nothing is staged in host memory that would have to
// outlive the call, and a captured graph carries the table's contents with it.
constexpr int kEntryWords = static_cast<int>(sizeof(BatchEntry) / sizeof(uint32_t));
constexpr int kWriteEntries = 48;                  // 48 * 80 bytes + 12 stay below the 4 KB of kernel arguments
struct TableChunk {
    uint32_t words[kWriteEntries * kEntryWords];
};

__global__ __launch_bounds__(1024) void table_write_kernel(uint32_t* __restrict__ dst, TableChunk chunk, int words)
{
    const int i = threadIdx.x;
    if (i < words) dst[i] = chunk.words[i];
}
static_assert(kWriteEntries * kEntryWords <= 1024, "one workgroup writes a chunk");
static_assert(sizeof(BatchEntry) == 80 && sizeof(TableChunk) + 12 <= 4096, "a chunk must fit the kernel arguments");

hipError_t write_table(Lane* lane, void* device_table, const BatchEntry* entries, size_t count)
{
    TableChunk chunk;
    for (size_t done = 0; done < count; done += kWriteEntries) {
        const size_t n = count - done < static_cast<size_t>(kWriteEntries) ? count - done : kWriteEntries;
        memcpy(chunk.words, entries + done, n * sizeof(BatchEntry));
        hipLaunchKernelGGL(table_write_kernel, dim3(1), dim3(1024), 0, lane->stream,
                           reinterpret_cast<uint32_t*>(static_cast<char*>(device_table) + done * sizeof(BatchEntry)), chunk,
                           static_cast<int>(n * kEntryWords));
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        lane->counters.kernel_launches += 1;
    }
    return hipSuccess;
}

// Fixed device workspace of nnhip_quant_matvec_batch_static: the descriptor table of a batch, in a file-scope device
// array so that the entry point never allocates.  Every device holds its own copy at its own address; host code uses
// the address hipGetSymbolAddress returns for the current device (kept in the lane), never the array's name.
constexpr int kStaticTableEntries = NNHIP_STATIC_BATCH_MAX_ENTRIES;
constexpr int kStaticLaneSlices = NNHIP_STATIC_BATCH_LANES;
static __device__ __align__(256) unsigned char scratch[kStaticLaneSlices * kStaticTableEntries * sizeof(BatchEntry)];

void shape_of(uint32_t type, int* max_t, int* depth)
{
    switch (type) {
    case NNHIP_TYPE_Q8_0: *max_t = Shape<Q8_0Unit>::kMaxT; *depth = Shape<Q8_0Unit>::kBatchDepth; break;
    case NNHIP_TYPE_Q4_K: *max_t = Shape<Q4KUnit>::kMaxT; *depth = Shape<Q4KUnit>::kBatchDepth; break;
    case NNHIP_TYPE_Q5_K: *max_t = Shape<Q5KUnit>::kMaxT; *depth = Shape<Q5KUnit>::kBatchDepth; break;
    case NNHIP_TYPE_Q6_K: *max_t = Shape<Q6KUnit>::kMaxT; *depth = Shape<Q6KUnit>::kBatchDepth; break;
    case NNHIP_TYPE_IQ3_S: *max_t = Shape<IQ3SUnit>::kMaxT; *depth = Shape<IQ3SUnit>::kBatchDepth; break;
    case NNHIP_TYPE_BF16: *max_t = Shape<BF16Unit>::kMaxT; *depth = Shape<BF16Unit>::kBatchDepth; break;
    default: *max_t = Shape<IQ2SUnit>::kMaxT; *depth = Shape<IQ2SUnit>::kBatchDepth; break;
    }
}

}  // namespace

int matvec_max_in_w(uint32_t type)
{
    const int by_lds = kMaxDynamicLds / (kChunkPieces * static_cast<int>(sizeof(float4))) * kUnitW;
    // one row must fit the workgroup: 768 lanes for the narrowest block-format shape, 512 for bfloat16 rows
    const int by_lanes = (type == NNHIP_TYPE_BF16 ? Shape<BF16Unit>::kMaxT : 768) * kUnitW;
    return by_lds < by_lanes ? by_lds : by_lanes;
}

namespace {

template <class Q>
bool describe_rowstep(int rows, int in_w, int out_w, int compute_units, nnhip_matvec_plan_info* info)
{
    Geometry g;
    int mr = 1;
    if (!rowstep_shape<Q, kPreNone>(rows, in_w, out_w, compute_units, &mr, &g)) return false;
    info->kernel = NNHIP_MATVEC_KERNEL_ROWSTEP;
    info->threads = g.threads;
    info->rows_per_step = g.rows_per_step;
    info->steps = g.steps;
    info->groups = g.groups;
    info->row_tile = mr;
    info->ring_depth = Shape<Q>::kDepth;
    info->result_buffer_floats = kYBuf;
    info->dynamic_lds_bytes = static_cast<int32_t>(static_cast<size_t>(mr) * kChunkPieces * (in_w / kUnitW) * sizeof(float4));
    return true;
}

}  // namespace

bool describe_matvec(uint32_t type, int rows, int in_w, int out_w, int compute_units, nnhip_matvec_plan_info* info)
{
    // (the plan is made without the weight pointer: the matrix-core path also needs it 16-byte aligned)
    if (const int per_pass = matvec_rows_per_pass(type, rows, in_w, out_w, nullptr, compute_units))
        return describe_matvec_rows_shared(type, rows, in_w, out_w, per_pass, compute_units, info);
    if (type == NNHIP_TYPE_Q8_0 && ((in_w / 32) & 1)) {
        info->kernel = NNHIP_MATVEC_KERNEL_Q8_0_ODD_BLOCKS;
        info->threads = 256;
        info->rows_per_step = 4;
        info->steps = (out_w + 3) / 4;
        info->groups = info->steps;
        info->row_tile = 1;
        info->ring_depth = 0;
        info->result_buffer_floats = 0;
        info->dynamic_lds_bytes = 0;
        return true;
    }
    switch (type) {
    case NNHIP_TYPE_Q8_0: return describe_rowstep<Q8_0Unit>(rows, in_w, out_w, compute_units, info);
    case NNHIP_TYPE_Q4_K: return describe_rowstep<Q4KUnit>(rows, in_w, out_w, compute_units, info);
    case NNHIP_TYPE_Q5_K: return describe_rowstep<Q5KUnit>(rows, in_w, out_w, compute_units, info);
    case NNHIP_TYPE_Q6_K: return describe_rowstep<Q6KUnit>(rows, in_w, out_w, compute_units, info);
    case NNHIP_TYPE_IQ3_S: return describe_rowstep<IQ3SUnit>(rows, in_w, out_w, compute_units, info);
    case NNHIP_TYPE_BF16: return describe_rowstep<BF16Unit>(rows, in_w, out_w, compute_units, info);
    case NNHIP_TYPE_IQ2_S: return describe_rowstep<IQ2SUnit>(rows, in_w, out_w, compute_units, info);
    default: return false;
    }
}

hipError_t launch_matvec(Lane* lane, uint32_t type, const float* x, const void* w, const float* bias, float* y,
                         int rows, int in_w, int out_w)
{
    int elems = 0, bytes = 0;
    type_block(type, &elems, &bytes);
    MatvecArgs a{};
    a.x = x;
    a.w = static_cast<const uint8_t*>(w);
    a.bias = bias;
    a.y = y;
    a.in_w = in_w;
    a.out_w = out_w;
    a.row_bytes = static_cast<uint32_t>(in_w / elems) * static_cast<uint32_t>(bytes);

    if (type == NNHIP_TYPE_Q8_0 && ((in_w / 32) & 1)) {
        hipLaunchKernelGGL(matvec_q8_0_oddrow_kernel, dim3((out_w + 3) / 4, rows), dim3(256), 0, lane->stream, a);
        return hipGetLastError();
    }

    a.units_per_row = in_w / kUnitW;
    a.magic = static_cast<uint32_t>((0x100000000ull + a.units_per_row - 1) / a.units_per_row);
    switch (type) {
    case NNHIP_TYPE_Q8_0: return launch_rowstep<Q8_0Unit>(lane, a, rows);
    case NNHIP_TYPE_Q4_K: return launch_rowstep<Q4KUnit>(lane, a, rows);
    case NNHIP_TYPE_Q5_K: return launch_rowstep<Q5KUnit>(lane, a, rows);
    case NNHIP_TYPE_Q6_K: return launch_rowstep<Q6KUnit>(lane, a, rows);
    case NNHIP_TYPE_IQ3_S: return launch_rowstep<IQ3SUnit>(lane, a, rows);
    case NNHIP_TYPE_BF16: return launch_rowstep<BF16Unit>(lane, a, rows);
    case NNHIP_TYPE_IQ2_S: return launch_rowstep<IQ2SUnit>(lane, a, rows);
    default: return hipErrorInvalidValue;
    }
}


template <int PRE>
hipError_t launch_fused_of(Lane* lane, uint32_t type, const MatvecArgs& a)
{
    switch (type) {
    case NNHIP_TYPE_Q8_0: return launch_rowstep<Q8_0Unit, PRE>(lane, a, 1);
    case NNHIP_TYPE_Q4_K: return launch_rowstep<Q4KUnit, PRE>(lane, a, 1);
    case NNHIP_TYPE_Q5_K: return launch_rowstep<Q5KUnit, PRE>(lane, a, 1);
    case NNHIP_TYPE_Q6_K: return launch_rowstep<Q6KUnit, PRE>(lane, a, 1);
    case NNHIP_TYPE_IQ3_S: return launch_rowstep<IQ3SUnit, PRE>(lane, a, 1);
    case NNHIP_TYPE_BF16: return launch_rowstep<BF16Unit, PRE>(lane, a, 1);
    case NNHIP_TYPE_IQ2_S: return launch_rowstep<IQ2SUnit, PRE>(lane, a, 1);
    default: return hipErrorInvalidValue;
    }
}

bool matvec_fused_supported(uint32_t type, int in_w)
{
    return !(type == NNHIP_TYPE_Q8_0 && ((in_w / 32) & 1));     // rows of an odd number of Q8_0 blocks take another kernel
}

hipError_t launch_matvec_fused(Lane* lane, const nnhip_fused_matvec_desc& d)
{
    int elems = 0, bytes = 0;
    type_block(d.ggml_type, &elems, &bytes);
    MatvecArgs a{};
    a.x = d.x;
    a.w = static_cast<const uint8_t*>(d.w);
    a.bias = d.bias;
    a.y = d.y;
    a.in_w = d.in_w;
    a.out_w = d.out_w;
    a.row_bytes = static_cast<uint32_t>(d.in_w / elems) * static_cast<uint32_t>(bytes);
    a.units_per_row = d.in_w / kUnitW;
    a.magic = static_cast<uint32_t>((0x100000000ull + a.units_per_row - 1) / a.units_per_row);
    a.x2 = d.x2;
    a.gamma = d.norm_weight;
    a.x_out = d.x_out;
    a.sum_out = d.sum_out;
    a.addend = d.addend;
    a.epsilon = d.epsilon;
    a.lora_z = d.lora_z;
    a.lora_b = d.lora_b;
    a.lora_rank = d.lora_rank;
    a.lora_scale = d.lora_scale;
    a.head4 = d.x_head_width >> 2;
    a.head_group = d.x_head_group;
    a.pair_rows = d.post_op == NNHIP_POST_SILU_PAIR ? d.out_w / 2 : 0;
    if (d.x_head_width > 0) return launch_fused_of<kPreHeadGather>(lane, d.ggml_type, a);
    switch (d.pre_op) {
    case NNHIP_PRE_NONE: return launch_fused_of<kPreNone>(lane, d.ggml_type, a);
    case NNHIP_PRE_RMS_NORM: return launch_fused_of<kPreRmsNorm>(lane, d.ggml_type, a);
    case NNHIP_PRE_SILU_MULTIPLY: return launch_fused_of<kPreSiluMultiply>(lane, d.ggml_type, a);
    default: return hipErrorInvalidValue;
    }
}

namespace {

struct BatchGroup {
    uint32_t type;
    size_t begin, end;       // entries [begin, end) of the table
    int total_chunks, max_in_w;
    int mfma;                // 0, or the form of the matrix-core kernel (1 - 3): entries are MfmaTableEntry, total_chunks counts tiles
    int x_changes;           // matrix-core groups: how often the activations change from one entry to the next
};
constexpr int kBatchTypes = 7;
constexpr int kBatchGroupsMax = kBatchTypes + 8;      // row-step groups plus matrix-core groups (one per type and in_w)
// Fewest 16-row tiles for which a group goes to the matrix-core kernel: it streams faster (measured on 17408 x 5120 Q4_K:
// 8.4 us per matrix against 10.8 us in a launch of twenty, 12.4 against 13.8 in a launch of two) but takes longer to
// start, so a single matrix of that size stays with the row-step kernel.
constexpr int kMfmaBatchMinTiles = 2048;
// The same floor for a single call whose three or more input rows share a pass over a super-block format (measured:
// 4096 x 5120 with rows = 3 / 4, 13 / 14 us against 15 - 18 / 19 - 23 us for one row-step pass per row; 1024 x 5120 breaks
// even at eight rows, 2048 x 2048 between four and six).  Q8_0 keeps the higher floor: its row-step kernel already
// multiplies four input rows per pass.
constexpr int kSharedPassMinTiles = 768;
// ... and for a pass per input row on the matrix cores (rows too long for shared passes): the codebook formats, whose
// row-step kernels are bound by their arithmetic, from fewer tiles on than the K-quants (measured on 5120 x 17408, us per
// call with 2 / 3 / 4 input rows: IQ2_S 34 / 38 / 45 against 38 / 55 / 70 with row-step passes, IQ3_S 45 / 52 / 62 against
// 41 / 59 / 75, Q4_K 35 at four rows against 36 at three).
constexpr int kSeparatePassMinTiles = 1024, kSeparatePassMinTilesIQ3S = 768, kSeparatePassMinTilesIQ2S = 512;
const uint32_t kBatchTypeOrder[kBatchTypes] = {NNHIP_TYPE_Q8_0, NNHIP_TYPE_Q4_K, NNHIP_TYPE_Q5_K, NNHIP_TYPE_Q6_K,
                                               NNHIP_TYPE_IQ3_S, NNHIP_TYPE_IQ2_S, NNHIP_TYPE_BF16};

// Entries of the batch, grouped by block format (one persistent launch per format); one entry per input row of a
// descriptor.  Returns the number of entries, or -1 if they exceed `cap`.  Q8_0 rows with an odd number of blocks get no
// entry: they are launched one by one.
static_assert(sizeof(MfmaTableEntry) == sizeof(BatchEntry), "both kinds of entry fill one table slot");

// Fewest input rows of a descriptor for which a shared pass on the matrix cores beats the row-step kernels: Q8_0's
// row-step kernel already reads the matrix once for up to four rows and wins at two (31.8 against 35.7 us on
// 21504 x 5376), loses from three on (four rows: 52.8 against 39.6 us).
int shared_pass_min_rows(uint32_t type) { return type == NNHIP_TYPE_Q8_0 ? 3 : 2; }

long build_batch(const nnhip_matvec_desc* descs, int count, BatchEntry* out, size_t cap, BatchGroup* groups, int* ngroups,
                 uint8_t* forms, bool row_step_only = false)
{
    size_t n = 0;
    *ngroups = 0;
    // matrix-core groups first: per (type, in_w, form) with enough tiles.  Forms: 1 = operand A in registers (in_w splits
    // into one or two whole stages), 2 = the wide form with one input row per entry, 3 = the wide form with up to four
    // input rows of a descriptor sharing a pass (descriptors with rows >= 2).  `forms` is `count` bytes of scratch: the
    // form of every descriptor is worked out once (a model's batch has hundreds of descriptors).
    for (int i = 0; i < count; ++i) {
        const nnhip_matvec_desc& d = descs[i];
        int form = 0;
        if (row_step_only) form = 0;
        else if (d.rows >= shared_pass_min_rows(d.ggml_type) && matvec_mfma_wide_geometry(d.ggml_type, d.in_w, d.out_w, d.w, 4)) form = 3;
        else if (matvec_mfma_geometry(d.ggml_type, d.in_w, d.out_w, d.w, nullptr)) form = 1;
        else if (matvec_mfma_wide_geometry(d.ggml_type, d.in_w, d.out_w, d.w, 1)) form = 2;
        forms[i] = static_cast<uint8_t>(form);
    }
    struct Key { uint32_t type; int in_w, form; long tiles; };
    Key keys[kBatchGroupsMax - kBatchTypes];
    int nkeys = 0;
    auto key_of = [&](int i) {
        for (int k = 0; k < nkeys; ++k)
            if (keys[k].type == descs[i].ggml_type && keys[k].in_w == descs[i].in_w && keys[k].form == forms[i]) return k;
        return -1;
    };
    for (int i = 0; i < count; ++i) {
        if (!forms[i]) continue;
        int k = key_of(i);
        if (k < 0) {
            if (nkeys == kBatchGroupsMax - kBatchTypes) {      // (further kinds stay with the row-step kernel)
                forms[i] = 0;
                continue;
            }
            k = nkeys++;
            keys[k] = Key{descs[i].ggml_type, descs[i].in_w, forms[i], 0};
        }
        keys[k].tiles += static_cast<long>(descs[i].rows) * ((descs[i].out_w + 15) / 16);
    }
    for (int i = 0; i < count; ++i)
        if (forms[i] && keys[key_of(i)].tiles < kMfmaBatchMinTiles) forms[i] = 0;
    for (int k = 0; k < nkeys; ++k) {
        if (keys[k].tiles < kMfmaBatchMinTiles) continue;
        const int form = keys[k].form;
        BatchGroup g{keys[k].type, n, n, 0, keys[k].in_w, form, 0};
        const float* last_x = nullptr;
        for (int j = 0; j < count; ++j) {
            const nnhip_matvec_desc& d = descs[j];
            if (forms[j] != form || d.ggml_type != keys[k].type || d.in_w != keys[k].in_w) continue;
            const int share = form == 3 ? 4 : 1;
            for (int r = 0; r < d.rows; r += share) {
                if (n >= cap) return -1;
                MfmaTableEntry e = matvec_mfma_entry(d.ggml_type, d.x + static_cast<size_t>(r) * d.in_w, d.w, d.bias,
                                                     d.y + static_cast<size_t>(r) * d.out_w, d.in_w, d.out_w, g.total_chunks);
                e.rows = d.rows - r < share ? d.rows - r : share;
                if (last_x && e.x != last_x) g.x_changes += 1;
                last_x = e.x;
                memcpy(&out[n++], &e, sizeof(e));
                g.total_chunks += e.tiles;
            }
        }
        g.end = n;
        groups[(*ngroups)++] = g;
    }
    for (uint32_t type : kBatchTypeOrder) {
        BatchGroup g{type, n, n, 0, 0, 0, 0};
        int max_t = 0, depth = 0;
        shape_of(type, &max_t, &depth);
        int elems = 0, bytes = 0;
        type_block(type, &elems, &bytes);
        for (int i = 0; i < count; ++i) {
            const nnhip_matvec_desc& d = descs[i];
            if (d.ggml_type != type) continue;
            if (type == NNHIP_TYPE_Q8_0 && ((d.in_w / 32) & 1)) continue;
            if (forms[i]) continue;                       // in a matrix-core group
            const int upr = d.in_w / kUnitW;
            int rs = max_t / upr;
            if (rs > d.out_w) rs = d.out_w;
            for (int r = 0; r < d.rows; ++r) {
                if (n >= cap) return -1;
                BatchEntry e{};
                e.x = (decltype(e.x))(d.x + static_cast<size_t>(r) * d.in_w);
                e.w = (decltype(e.w))(d.w);
                e.bias = (decltype(e.bias))(d.bias);
                e.y = (decltype(e.y))(d.y + static_cast<size_t>(r) * d.out_w);
                e.in_w = d.in_w;
                e.out_w = d.out_w;
                e.upr = upr;
                e.rs = rs;
                e.steps = (d.out_w + rs - 1) / rs;
                e.row_bytes = static_cast<uint32_t>(d.in_w / elems) * static_cast<uint32_t>(bytes);
                e.magic = static_cast<uint32_t>((0x100000000ull + upr - 1) / upr);
                e.first_chunk = g.total_chunks;
                e.chunks = (e.steps + depth - 1) / depth;
                g.total_chunks += e.chunks;
                if (d.in_w > g.max_in_w) g.max_in_w = d.in_w;
                out[n++] = e;
            }
        }
        g.end = n;
        if (g.end > g.begin) groups[(*ngroups)++] = g;
    }
    return static_cast<long>(n);
}

hipError_t launch_batch_groups(Lane* lane, const void* device_table, const BatchGroup* groups, int ngroups,
                               const nnhip_matvec_desc* descs, int count)
{
    for (int i = 0; i < ngroups; ++i) {
        const BatchGroup& g = groups[i];
        const BatchEntry* t = reinterpret_cast<const BatchEntry*>(device_table) + g.begin;
        hipError_t e = hipSuccess;
        if (g.mfma) {
            const MfmaTableEntry* mt = reinterpret_cast<const MfmaTableEntry*>(t);
            const int entries = static_cast<int>(g.end - g.begin);
            // With two or more changes of activations along the table the workgroups take runs of consecutive tiles (a
            // workgroup converts the vectors of its run only: 7.9 against 9.3 us per Q4_K mat-vec when every matrix has
            // its own); with shared activations every G-th tile streams 2 % faster.
            const bool runs = g.x_changes >= 2;
            e = g.mfma == 1 ? launch_matvec_mfma_table(lane, g.type, g.max_in_w, mt, entries, g.total_chunks, runs)
                            : launch_matvec_mfma_wide_table(lane, g.type, g.max_in_w, g.mfma == 3 ? 4 : 1, mt, entries, g.total_chunks, runs);
            if (e != hipSuccess) return e;
            lane->counters.kernel_launches += 1;
            continue;
        }
        switch (g.type) {
        case NNHIP_TYPE_Q8_0: e = launch_batch_of<Q8_0Unit>(lane, t, g.total_chunks, g.max_in_w); break;
        case NNHIP_TYPE_Q4_K: e = launch_batch_of<Q4KUnit>(lane, t, g.total_chunks, g.max_in_w); break;
        case NNHIP_TYPE_Q5_K: e = launch_batch_of<Q5KUnit>(lane, t, g.total_chunks, g.max_in_w); break;
        case NNHIP_TYPE_Q6_K: e = launch_batch_of<Q6KUnit>(lane, t, g.total_chunks, g.max_in_w); break;
        case NNHIP_TYPE_IQ3_S: e = launch_batch_of<IQ3SUnit>(lane, t, g.total_chunks, g.max_in_w); break;
        case NNHIP_TYPE_BF16: e = launch_batch_of<BF16Unit>(lane, t, g.total_chunks, g.max_in_w); break;
        default: e = launch_batch_of<IQ2SUnit>(lane, t, g.total_chunks, g.max_in_w); break;
        }
        if (e != hipSuccess) return e;
        lane->counters.kernel_launches += 1;
    }
    for (int i = 0; i < count; ++i) {
        const nnhip_matvec_desc& d = descs[i];
        if (d.ggml_type == NNHIP_TYPE_Q8_0 && ((d.in_w / 32) & 1)) {
            hipError_t e = launch_matvec(lane, d.ggml_type, d.x, d.w, d.bias, d.y, d.rows, d.in_w, d.out_w);
            if (e != hipSuccess) return e;
            lane->counters.kernel_launches += 1;
        }
    }
    return hipSuccess;
}

}  // namespace

// The lane's table grows by allocating a larger one; the old one is kept until the lane is destroyed, because a
// captured graph may still name it.  Outside a capture the write is skipped when the device already holds these entries
// (the common case of a decode loop that repeats one batch).
hipError_t launch_matvec_batch(Lane* lane, const nnhip_matvec_desc* descs, int count)
{
    size_t cap = 0;
    for (int i = 0; i < count; ++i) cap += static_cast<size_t>(descs[i].rows);
    std::vector<BatchEntry> all(cap);
    std::vector<uint8_t> forms(static_cast<size_t>(count > 0 ? count : 1));
    BatchGroup groups[kBatchGroupsMax];
    int ngroups = 0;
    const long n = build_batch(descs, count, all.data(), cap, groups, &ngroups, forms.data(), lane->row_step_only);
    if (n < 0) return hipErrorInvalidValue;
    const size_t bytes = static_cast<size_t>(n) * sizeof(BatchEntry);
    if (bytes) {
        if (bytes > lane->batch_table_bytes) {
            if (lane->capturing) return hipErrorStreamCaptureUnsupported;     // the table cannot grow inside a capture
            const size_t want = bytes * 2 < 65536 ? 65536 : bytes * 2;
            void* fresh = nullptr;
            const hipError_t e = hipMalloc(&fresh, want);
            if (e == hipSuccess) ++lane->counters.driver_allocations;
            if (e != hipSuccess) return e;
            if (lane->batch_table) lane->retired_tables.push_back(lane->batch_table);
            lane->batch_table = fresh;
            lane->batch_table_bytes = want;
            lane->batch_shadow.clear();
        }
        const bool same = !lane->capturing && lane->batch_shadow.size() == bytes &&
                          memcmp(lane->batch_shadow.data(), all.data(), bytes) == 0;
        if (!same) {
            const hipError_t e = write_table(lane, lane->batch_table, all.data(), static_cast<size_t>(n));
            if (e != hipSuccess) return e;
            if (lane->capturing) {
                lane->batch_shadow.clear();     // recorded, not executed: the device contents are unknown until replay
            } else {
                lane->batch_shadow.assign(reinterpret_cast<const char*>(all.data()),
                                          reinterpret_cast<const char*>(all.data()) + bytes);
            }
        }
    }
    return launch_batch_groups(lane, lane->batch_table, groups, ngroups, descs, count);
}

int plan_matvec_batch(const nnhip_matvec_desc* descs, int count, int compute_units, nnhip_batch_launch_info* launches,
                      int capacity)
{
    size_t cap = 0;
    for (int i = 0; i < count; ++i) cap += static_cast<size_t>(descs[i].rows);
    std::vector<BatchEntry> all(cap ? cap : 1);
    std::vector<uint8_t> forms(static_cast<size_t>(count > 0 ? count : 1));
    BatchGroup groups[kBatchGroupsMax];
    int ngroups = 0;
    if (build_batch(descs, count, all.data(), cap, groups, &ngroups, forms.data()) < 0) return -1;
    int n = 0;
    auto next = [&]() -> nnhip_batch_launch_info* {
        nnhip_batch_launch_info* slot = n < capacity ? &launches[n] : nullptr;
        n += 1;
        if (slot) {
            const uint32_t size = slot->struct_size;
            *slot = nnhip_batch_launch_info{};
            slot->struct_size = size;
        }
        return slot;
    };
    for (int i = 0; i < ngroups; ++i) {
        const BatchGroup& g = groups[i];
        nnhip_batch_launch_info* info = next();
        if (!info) continue;
        info->ggml_type = g.type;
        info->in_w = g.max_in_w;
        info->entries = static_cast<int32_t>(g.end - g.begin);
        info->units = g.total_chunks;
        info->groups = g.total_chunks < compute_units ? g.total_chunks : compute_units;
        info->rows_per_pass = 1;
        if (g.mfma) {
            info->kernel = NNHIP_MATVEC_KERNEL_MATRIX_CORE;
            if (!describe_matvec_mfma_launch(g.type, g.max_in_w, g.mfma, g.x_changes >= 2, info)) return -1;
            if (g.mfma == 3) {
                const MfmaTableEntry* e = reinterpret_cast<const MfmaTableEntry*>(all.data()) + g.begin;
                for (size_t k = 0; k < g.end - g.begin; ++k)
                    if (e[k].rows > info->rows_per_pass) info->rows_per_pass = e[k].rows;
            }
        } else {
            int max_t = 0, depth = 0;
            shape_of(g.type, &max_t, &depth);
            info->kernel = NNHIP_MATVEC_KERNEL_ROWSTEP;
            info->threads = max_t;
            info->dynamic_lds_bytes = static_cast<int32_t>(static_cast<size_t>(kChunkPieces) * (g.max_in_w / kUnitW) * sizeof(float4));
        }
    }
    for (int i = 0; i < count; ++i) {           // (Q8_0 rows with an odd number of blocks: one launch each)
        const nnhip_matvec_desc& d = descs[i];
        if (d.ggml_type != NNHIP_TYPE_Q8_0 || !((d.in_w / 32) & 1)) continue;
        nnhip_batch_launch_info* info = next();
        if (!info) continue;
        nnhip_matvec_plan_info single{};
        single.struct_size = sizeof(single);
        if (!describe_matvec(d.ggml_type, d.rows, d.in_w, d.out_w, compute_units, &single)) return -1;
        info->ggml_type = d.ggml_type;
        info->kernel = single.kernel;
        info->in_w = d.in_w;
        info->entries = 1;
        info->units = single.steps;
        info->groups = single.groups;
        info->threads = single.threads;
        info->rows_per_pass = single.row_tile;
        info->dynamic_lds_bytes = single.dynamic_lds_bytes;
    }
    return n;
}

int matvec_rows_per_pass(uint32_t type, int rows, int in_w, int out_w, const void* w, int compute_units)
{
    if (rows < shared_pass_min_rows(type)) return 0;
    const long work = static_cast<long>(rows) * ((out_w + 15) / 16);
    const long floor = rows >= 3 && type != NNHIP_TYPE_Q8_0 ? kSharedPassMinTiles : kMfmaBatchMinTiles;
    bool split = false;
    const bool shared = matvec_mfma_wide_geometry(type, in_w, out_w, w, 4, &split);
    if (work >= floor && shared && !split) return 4;
    // Rows too long for four sets of activation planes in LDS (more than about 8700 values): shared passes in the split
    // form, the planes of one group of block columns at a time.
    // It pays from three and a half rounds of (16 matrix rows x 4 input rows) over the workgroups on (IQ2_S: two and a
    // half): fewer leave compute units idle in the last round, and every change of entry costs a workgroup a conversion
    // per part, while a pass per input row deals four times as many tiles.  IQ3_S, whose codebook lookups a shared
    // pass makes once for four rows, gains from three rows on.  Measured on 5120 x 17408, us per call, shared against a
    // pass per row: Q4_K 8 rows 85 / 68, 9 rows 69 / 89, 16 rows 77 / 136; IQ2_S 4 rows 49 / 46, 8 rows 77 / 89, 16 rows
    // 91 / 173; IQ3_S 4 rows 53 / 64, 16 rows 98 / 242; on 17408 x 14336 Q4_K 4 rows 67 / 82, 16 rows 233 / 332.
    const long shared_units = static_cast<long>((rows + 3) / 4) * ((out_w + 15) / 16);
    const long shared_floor = type == NNHIP_TYPE_IQ3_S ? 0 : type == NNHIP_TYPE_IQ2_S ? 5L * compute_units : 7L * compute_units;
    if (work >= floor && shared && split && 2 * shared_units >= shared_floor) return 4;
    // Rows too long for four sets of activation planes in LDS (more than about 8700 values): the super-block formats
    // still stream faster on the matrix cores, one pass per input row (Q8_0's row-step kernel multiplies four input rows
    // per pass and stays).
    const long separate_floor = type == NNHIP_TYPE_IQ2_S ? kSeparatePassMinTilesIQ2S
                              : type == NNHIP_TYPE_IQ3_S ? kSeparatePassMinTilesIQ3S : kSeparatePassMinTiles;
    if (type != NNHIP_TYPE_Q8_0 && work >= separate_floor && (!shared || split) && matvec_mfma_wide_geometry(type, in_w, out_w, w, 1))
        return 1;
    return 0;
}

// The slice of the fixed workspace for the `serial`-th lane created on the current device.
hipError_t static_table_address(void** address, unsigned serial)
{
    void* base = nullptr;
    const hipError_t e = hipGetSymbolAddress(&base, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !base) return e != hipSuccess ? e : hipErrorInvalidSymbol;
    *address = static_cast<unsigned char*>(base) + static_cast<size_t>(serial % kStaticLaneSlices) * kStaticTableEntries * sizeof(BatchEntry);
    return hipSuccess;
}

// As launch_matvec_batch with the table in the device's fixed workspace: no device or host allocation on this path.
// hipErrorInvalidValue: more entries than the workspace holds.
hipError_t launch_matvec_batch_static(Lane* lane, const nnhip_matvec_desc* descs, int count)
{
    if (!lane->static_table) return hipErrorNotInitialized;
    if (count > kStaticTableEntries) return hipErrorInvalidValue;       // (every descriptor takes at least one entry)
    BatchEntry entries[kStaticTableEntries];
    uint8_t forms[kStaticTableEntries];
    BatchGroup groups[kBatchGroupsMax];
    int ngroups = 0;
    const long n = build_batch(descs, count, entries, kStaticTableEntries, groups, &ngroups, forms, lane->row_step_only);
    if (n < 0) return hipErrorInvalidValue;
    if (n > 0) {
        const hipError_t e = write_table(lane, lane->static_table, entries, static_cast<size_t>(n));
        if (e != hipSuccess) return e;
    }
    return launch_batch_groups(lane, lane->static_table, groups, ngroups, descs, count);
}

}  // namespace nnhip
