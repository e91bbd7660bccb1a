// Dequantization-fused mat-vec kernels for raw GGUF blocks on gfx950 (wave64).
//
// y[r, o] = bias[o] + sum_k x[r, k] * w[o, k]     (NNtrain.Arc/Kernels/qwen.cl:374-406 defines the operator)
//
// Work decomposition (the same for every block format):
//   * a row of the matrix is cut into "units" of 64 consecutive weights (two Q8_0 blocks, a quarter of a
//     256-weight super-block); a unit is the work of one lane: it loads the unit's bytes with 128-bit loads,
//     unpacks scales / nibbles in registers and produces one FP32 partial dot product;
//   * a workgroup owns a contiguous range of output rows and walks the (row, unit) pairs of that range as ONE flat
//     index space, 1024 lanes at a time, so consecutive lanes read consecutive memory across row ends and no lane
//     idles when units-per-row is not a multiple of 64;
//   * the activation vector is staged once per workgroup in LDS as float4 pieces, transposed so that the 64 lanes of
//     a wave read 64 consecutive pieces with every ds_read_b128 (piece k/4 lives at [(k/4)%16][k/64]);
//   * unit partials go to LDS as part[row][unit]; after one barrier each row is summed in a fixed order
//     (lane-strided, then a DPP butterfly).  The order depends only on in_w, never on the launch geometry, so the
//     result for a row is bit-identical for any `rows`, out_w or batch composition.
#include "nnhip_internal.h"
#include "quant_device.h"

#include "iq_grids.inc"

namespace nnhip {

namespace {

__device__ const uint64_t g_iq2s_grid[1024] = { NNHIP_IQ2S_GRID_VALUES };

constexpr int kWG = 1024;          // lanes per workgroup (16 waves: 4 per SIMD)
constexpr int kUnitW = 64;         // weights per lane-unit
constexpr int kMaxLds = 160 * 1024;

struct MatvecArgs {
    const float* x;
    const uint8_t* w;
    const float* bias;
    float* y;
    int in_w;
    int out_w;
    int units_per_row;     // in_w / 64
    int cpad;              // odd stride (in float4 pieces) between the 16 piece-planes of the staged x
    int rows_per_wg;
    uint32_t row_bytes;
    uint32_t magic;        // ceil(2^32 / units_per_row): u / units_per_row == umulhi(u, magic) for u < 2^32 / upr
};

// LDS view shared by the unit functions.
struct Staged {
    const float4* xp;      // transposed activation pieces
    const float* xs;       // per-type block sums of x (32-wide for Q4_K/Q5_K, 16-wide for Q6_K), or nullptr
    const uint64_t* grid;  // IQ2_S codebook copy, or nullptr
    int cpad;
};

__device__ __forceinline__ float4 xpiece(const Staged& s, int chunk, int q) { return s.xp[q * s.cpad + chunk]; }

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

// ---------------------------------------------------------------------------------------------------- Q8_0
// Unit = two consecutive 34-byte blocks (68 bytes, 4-byte aligned because a row holds an even number of blocks).
struct Q8_0Unit {
    static constexpr int kXsWidth = 0;
    static constexpr bool kGrid = false;
    static constexpr int kUnitBytes = 68;

    static __device__ __forceinline__ float dot(const uint8_t* row, int unit, const Staged& s)
    {
        const uint8_t* p = row + static_cast<uint32_t>(unit) * 68u;
        const u32x4 a = ld128(p), b = ld128(p + 16), c = ld128(p + 32), d = ld128(p + 48);
        const uint32_t e = ld32(p + 64);
        const uint32_t w[17] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3], c[0], c[1], c[2], c[3],
                                d[0], d[1], d[2], d[3], e};
        const float d0 = half_bits_to_float(w[0]);
        const float d1 = half_bits_to_float(w[8] >> 16);
        float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t q = __builtin_amdgcn_alignbyte(w[i + 1], w[i], 2);  // quants of block 0 start at byte 2
            acc0 = dot4s(q, xpiece(s, unit, i), acc0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) acc1 = dot4s(w[9 + i], xpiece(s, unit, 8 + i), acc1);
        return fmaf(d1, acc1, d0 * acc0);
    }
};

// ---------------------------------------------------------------------------------------------------- Q4_K
// Unit j of a super-block = sub-blocks 2j (low nibbles) and 2j+1 (high nibbles) of qs[32j .. 32j+31].
// sum_k x (s*q - m) = s * sum(q x) - m * sum(x); the 32-wide sums of x are staged once per workgroup.
struct Q4KUnit {
    static constexpr int kXsWidth = 32;
    static constexpr bool kGrid = false;

    static __device__ __forceinline__ float dot(const uint8_t* row, int unit, const Staged& s)
    {
        const int sb = unit >> 2, j = unit & 3;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 144u;
        const u32x4 h = *reinterpret_cast<const u32x4*>(blk);
        const u32x4 qa = *reinterpret_cast<const u32x4*>(blk + 16 + 32 * j);
        const u32x4 qb = *reinterpret_cast<const u32x4*>(blk + 32 + 32 * j);
        const float d = half_bits_to_float(h[0]), dmin = half_bits_to_float(h[0] >> 16);
        uint32_t sc, mn;
        k4_scale_pair(h[1], h[2], h[3], j, sc, mn);
        const uint32_t q[8] = {qa[0], qa[1], qa[2], qa[3], qb[0], qb[1], qb[2], qb[3]};
        float lo = 0.0f, hi = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t l4 = opaque(q[i] & 0x0f0f0f0fu);
            const uint32_t h4 = opaque(q[i] & 0xf0f0f0f0u);   // 16 * high nibble; the 1/16 is folded into the scale
            lo = dot4u(l4, xpiece(s, unit, i), lo);
            hi = dot4u(h4, xpiece(s, unit, 8 + i), hi);
        }
        const float s_lo = d * ubyte0(sc), s_hi = d * ubyte1(sc) * 0.0625f;
        const float m_lo = dmin * ubyte0(mn), m_hi = dmin * ubyte1(mn);
        const float xs_lo = s.xs[2 * unit], xs_hi = s.xs[2 * unit + 1];
        float acc = s_lo * lo;
        acc = fmaf(s_hi, hi, acc);
        acc = fmaf(-m_lo, xs_lo, acc);
        acc = fmaf(-m_hi, xs_hi, acc);
        return acc;
    }
};

// ---------------------------------------------------------------------------------------------------- Q5_K
// As Q4_K plus one high bit per weight: bit g of qh[i] belongs to element i of sub-block g.
struct Q5KUnit {
    static constexpr int kXsWidth = 32;
    static constexpr bool kGrid = false;

    static __device__ __forceinline__ float dot(const uint8_t* row, int unit, const Staged& s)
    {
        const int sb = unit >> 2, j = unit & 3;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 176u;
        const u32x4 h = *reinterpret_cast<const u32x4*>(blk);
        const u32x4 ha = *reinterpret_cast<const u32x4*>(blk + 16);
        const u32x4 hb = *reinterpret_cast<const u32x4*>(blk + 32);
        const u32x4 qa = *reinterpret_cast<const u32x4*>(blk + 48 + 32 * j);
        const u32x4 qb = *reinterpret_cast<const u32x4*>(blk + 64 + 32 * j);
        const float d = half_bits_to_float(h[0]), dmin = half_bits_to_float(h[0] >> 16);
        uint32_t sc, mn;
        k4_scale_pair(h[1], h[2], h[3], j, sc, mn);
        const uint32_t q[8] = {qa[0], qa[1], qa[2], qa[3], qb[0], qb[1], qb[2], qb[3]};
        const uint32_t hq[8] = {ha[0], ha[1], ha[2], ha[3], hb[0], hb[1], hb[2], hb[3]};
        float lo = 0.0f, hi = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t hb2 = hq[i] >> (2 * j);                       // bit 0: sub-block 2j, bit 1: sub-block 2j+1
            const uint32_t l5 = opaque((q[i] & 0x0f0f0f0fu) | ((hb2 << 4) & 0x10101010u));
            const uint32_t h5 = opaque(((q[i] >> 4) & 0x0f0f0f0fu) | ((hb2 << 3) & 0x10101010u));
            lo = dot4u(l5, xpiece(s, unit, i), lo);
            hi = dot4u(h5, xpiece(s, unit, 8 + i), hi);
        }
        const float s_lo = d * ubyte0(sc), s_hi = d * ubyte1(sc);
        const float m_lo = dmin * ubyte0(mn), m_hi = dmin * ubyte1(mn);
        const float xs_lo = s.xs[2 * unit], xs_hi = s.xs[2 * unit + 1];
        float acc = s_lo * lo;
        acc = fmaf(s_hi, hi, acc);
        acc = fmaf(-m_lo, xs_lo, acc);
        acc = fmaf(-m_hi, xs_hi, acc);
        return acc;
    }
};

// ---------------------------------------------------------------------------------------------------- Q6_K
// Unit (sb, half h, part p): elements 128h + 32e + 16p + i, i < 16, e < 4 - the four 16-runs that share
// ql[64h+16p ..], ql[64h+32+16p ..] and qh[32h+16p ..].  w = d*scale*(q - 32): sum(q x) - 32 sum16(x).
struct Q6KUnit {
    static constexpr int kXsWidth = 16;
    static constexpr bool kGrid = false;

    static __device__ __forceinline__ float dot(const uint8_t* row, int unit, const Staged& s)
    {
        const int sb = unit >> 2, h = (unit >> 1) & 1, p = unit & 1;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 210u;
        const u32x4 la = ld128(blk + 64 * h + 16 * p);
        const u32x4 lb = ld128(blk + 64 * h + 32 + 16 * p);
        const u32x4 hh = ld128(blk + 128 + 32 * h + 16 * p);
        const u32x2 scw = ld64(blk + 192 + 8 * h);
        const float d = half_bits_to_float(ld16(blk + 208));
        float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
        const int c0 = 4 * sb + 2 * h;       // 64-chunk holding e = 0,1; e = 2,3 are in chunk c0 + 1
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t a = la[i], b = lb[i], q2 = hh[i];
            const uint32_t q1 = opaque((a & 0x0f0f0f0fu) | ((q2 << 4) & 0x30303030u));
            const uint32_t q2v = opaque((b & 0x0f0f0f0fu) | ((q2 << 2) & 0x30303030u));
            const uint32_t q3 = opaque(((a >> 4) & 0x0f0f0f0fu) | (q2 & 0x30303030u));
            const uint32_t q4 = opaque(((b >> 4) & 0x0f0f0f0fu) | ((q2 >> 2) & 0x30303030u));
            a0 = dot4u(q1, xpiece(s, c0, 4 * p + i), a0);
            a1 = dot4u(q2v, xpiece(s, c0, 8 + 4 * p + i), a1);
            a2 = dot4u(q3, xpiece(s, c0 + 1, 4 * p + i), a2);
            a3 = dot4u(q4, xpiece(s, c0 + 1, 8 + 4 * p + i), a3);
        }
        // int8 sub-scales 8h + 2e + p; 16-wide sums of x at run index 16 sb + 8 h + 2 e + p
        const uint32_t s01 = scw[0] >> (8 * p), s23 = scw[1] >> (8 * p);
        const float sc0 = sbyte0(s01), sc1 = sbyte2(s01), sc2 = sbyte0(s23), sc3 = sbyte2(s23);
        const float* xs = s.xs + 16 * sb + 8 * h + p;
        float acc = (d * sc0) * fmaf(-32.0f, xs[0], a0);
        acc = fmaf(d * sc1, fmaf(-32.0f, xs[2], a1), acc);
        acc = fmaf(d * sc2, fmaf(-32.0f, xs[4], a2), acc);
        acc = fmaf(d * sc3, fmaf(-32.0f, xs[6], a3), acc);
        return acc;
    }
};

// ---------------------------------------------------------------------------------------------------- IQ2_S
// Unit gp of a super-block = 32-groups 2gp and 2gp+1.  Each octet: 10-bit index into the 1024-entry codebook held
// in LDS (8 magnitude bytes), 8 sign bits, 4-bit sub-scale shared by two octets.
struct IQ2SUnit {
    static constexpr int kXsWidth = 0;
    static constexpr bool kGrid = true;

    static __device__ __forceinline__ float signed_mag(float mag, uint32_t signs, int t)
    {
        const uint32_t sign = (signs << (31 - t)) & 0x80000000u;
        return __uint_as_float(__float_as_uint(mag) | sign);
    }

    static __device__ __forceinline__ float dot(const uint8_t* row, int unit, const Staged& s)
    {
        const int sb = unit >> 2, gp = unit & 3;
        const uint8_t* blk = row + static_cast<uint32_t>(sb) * 82u;
        const u32x2 qs = ld64(blk + 2 + 8 * gp);
        const u32x2 sg = ld64(blk + 34 + 8 * gp);
        const uint32_t qh = ld16(blk + 66 + 2 * gp);
        const uint32_t scl = ld16(blk + 74 + 2 * gp);
        const float d = half_bits_to_float(ld16(blk));
        float acc = 0.0f;
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const uint32_t q4 = qs[g], s4 = sg[g];
            const uint32_t hbits = (qh >> (8 * g)) & 0xffu;
            const uint32_t sc = (scl >> (8 * g)) & 0xffu;
#pragma unroll
            for (int o = 0; o < 4; ++o) {
                const uint32_t idx = ((q4 >> (8 * o)) & 0xffu) | (((hbits >> (2 * o)) & 3u) << 8);
                const uint64_t gv = s.grid[idx];
                const uint32_t glo = static_cast<uint32_t>(gv), ghi = static_cast<uint32_t>(gv >> 32);
                const uint32_t signs = (s4 >> (8 * o)) & 0xffu;
                const float4 xa = xpiece(s, unit, 8 * g + 2 * o), xb = xpiece(s, unit, 8 * g + 2 * o + 1);
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

// ---------------------------------------------------------------------------------------------- the kernel
// grid.x = row groups, grid.y = input rows.  Dynamic LDS: [16 * cpad float4][xs floats][grid 8 KB][part floats].
template <class Q>
__global__ __launch_bounds__(kWG) void matvec_flat_kernel(MatvecArgs a)
{
    extern __shared__ float4 lds[];
    float4* xp = lds;
    float* xs = reinterpret_cast<float*>(xp + 16 * a.cpad);
    constexpr int kXsDiv = Q::kXsWidth ? Q::kXsWidth : 1;
    const int n_xs = Q::kXsWidth ? a.in_w / kXsDiv : 0;
    uint64_t* grid = reinterpret_cast<uint64_t*>(xs + ((n_xs + 3) & ~3));
    float* part = reinterpret_cast<float*>(grid + (Q::kGrid ? 1024 : 0));

    const int tid = threadIdx.x;
    const int m = blockIdx.y;
    const int row0 = blockIdx.x * a.rows_per_wg;
    const int nrows = min(a.rows_per_wg, a.out_w - row0);
    const float4* xg = reinterpret_cast<const float4*>(a.x + static_cast<size_t>(m) * a.in_w);

    // stage x (and its block sums, and the codebook)
    const int pieces = a.in_w >> 2;
    for (int L = tid; L < pieces; L += kWG) {
        const float4 v = xg[L];
        xp[(L & 15) * a.cpad + (L >> 4)] = v;
        if (Q::kXsWidth == 32) {
            const float t = oct_sum((v.x + v.y) + (v.z + v.w));
            if ((L & 7) == 0) xs[L >> 3] = t;
        } else if (Q::kXsWidth == 16) {
            float t = (v.x + v.y) + (v.z + v.w);
            t += dpp_mov<0xB1>(t);
            t += dpp_mov<0x4E>(t);
            if ((L & 3) == 0) xs[L >> 2] = t;
        }
    }
    if (Q::kGrid) grid[tid] = g_iq2s_grid[tid];
    __syncthreads();

    Staged s{xp, xs, grid, a.cpad};
    const int upr = a.units_per_row;
    const int units = nrows * upr;
    for (int u = tid; u < units; u += kWG) {
        const int r = upr == 1 ? u : static_cast<int>(__umulhi(static_cast<uint32_t>(u), a.magic));
        const int c = u - r * upr;
        const uint8_t* row = a.w + static_cast<size_t>(row0 + r) * a.row_bytes;
        part[u] = Q::dot(row, c, s);
    }
    __syncthreads();

    const int wave = tid >> 6, lane = tid & 63;
    for (int r = wave; r < nrows; r += kWG / 64) {
        float t = 0.0f;
        for (int c = lane; c < upr; c += 64) t += part[r * upr + c];
        t = wave_sum(t);
        if (lane == 0) {
            const int o = row0 + r;
            a.y[static_cast<size_t>(m) * a.out_w + o] = (a.bias ? a.bias[o] : 0.0f) + t;
        }
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
    int cpad;
    int rows_per_wg;
    int groups;
    size_t lds_bytes;
};

// Picks rows per workgroup so that one workgroup per compute unit covers the matrix, within the LDS budget.
bool plan(uint32_t type, int in_w, int out_w, int compute_units, Geometry* g)
{
    const int upr = in_w / kUnitW;
    const int cpad = upr | 1;
    int xs_width = (type == NNHIP_TYPE_Q4_K || type == NNHIP_TYPE_Q5_K) ? 32 : type == NNHIP_TYPE_Q6_K ? 16 : 0;
    size_t fixed = static_cast<size_t>(16) * cpad * sizeof(float4);
    if (xs_width) fixed += static_cast<size_t>(((in_w / xs_width) + 3) & ~3) * sizeof(float);
    if (type == NNHIP_TYPE_IQ2_S) fixed += 1024 * sizeof(uint64_t);
    if (fixed + static_cast<size_t>(upr) * sizeof(float) > static_cast<size_t>(kMaxLds)) return false;
    const int max_rows = static_cast<int>((kMaxLds - fixed) / (static_cast<size_t>(upr) * sizeof(float)));
    int rpw = (out_w + compute_units - 1) / compute_units;
    if (rpw > max_rows) rpw = max_rows;
    if (rpw < 1) rpw = 1;
    g->cpad = cpad;
    g->rows_per_wg = rpw;
    g->groups = (out_w + rpw - 1) / rpw;
    g->lds_bytes = fixed + static_cast<size_t>(rpw) * upr * sizeof(float);
    return true;
}

template <class Q>
hipError_t launch_flat(Lane* lane, const MatvecArgs& args, const Geometry& g, int rows)
{
    static size_t configured = 0;  // largest dynamic LDS size this kernel has been enabled for
    if (g.lds_bytes > 64 * 1024 && g.lds_bytes > configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&matvec_flat_kernel<Q>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds);
        if (e != hipSuccess) return e;
        configured = kMaxLds;
    }
    hipLaunchKernelGGL(matvec_flat_kernel<Q>, dim3(g.groups, rows), dim3(kWG), g.lds_bytes, lane->stream, args);
    return hipGetLastError();
}

}  // namespace

int matvec_max_in_w(uint32_t type)
{
    // 16 planes of (in_w/64 | 1) float4 pieces plus side tables must leave room for at least one row of partials.
    int best = 0;
    for (int k = 256; k <= 65536; k += 256) {
        Geometry g;
        if (plan(type, k, 1, 1, &g)) best = k;
    }
    return best;
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

    Geometry g;
    if (!plan(type, in_w, out_w, lane->compute_units, &g)) return hipErrorInvalidValue;
    a.units_per_row = in_w / kUnitW;
    a.cpad = g.cpad;
    a.rows_per_wg = g.rows_per_wg;
    a.magic = static_cast<uint32_t>((0x100000000ull + a.units_per_row - 1) / a.units_per_row);
    switch (type) {
    case NNHIP_TYPE_Q8_0: return launch_flat<Q8_0Unit>(lane, a, g, rows);
    case NNHIP_TYPE_Q4_K: return launch_flat<Q4KUnit>(lane, a, g, rows);
    case NNHIP_TYPE_Q5_K: return launch_flat<Q5KUnit>(lane, a, g, rows);
    case NNHIP_TYPE_Q6_K: return launch_flat<Q6KUnit>(lane, a, g, rows);
    case NNHIP_TYPE_IQ2_S: return launch_flat<IQ2SUnit>(lane, a, g, rows);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace nnhip
