// Prefill mat-mul for raw GGUF block-quantized weights (Q4_K, Q5_K, Q6_K, Q8_0, IQ2_S, IQ3_S) and bfloat16 matrices on gfx950:
// y[M, N] = bias + x[M, K] (bf16) . W[N, K]^T.
//
// Replaces the XMX prefill launches of the reference (NNtrain.Arc/Kernels/qwen35_prefill_xmx.cl:112-184, the
// q35l_prefill_xmx_<format>_f16x2 family): weight tiles are dequantized to bfloat16 in LDS and contracted on the matrix
// cores (v_mfma_f32_16x16x32_bf16) with FP32 accumulators.  A weight is the CPU decoder's value, e.g. (d*sc)*q - dmin*m
// for Q4_K (NNtrain.Core/Serialization/GgufQ4K.cs:34-41), evaluated in FP32 and rounded once to bf16, which is what the
// 2e-3 relative-L2 bar of this path allows for (the rounding alone is 1.6e-3 rms; against a product taken with
// bf16-rounded weights the kernel agrees to FP32 accumulation accuracy).
//
// Tiling.  A workgroup owns BM rows (128 or 256) and a strip of up to 16 * CT output columns (CT = 5 or 9 column tiles)
// for the whole K range; the strip width is chosen on the host so that strips x row tiles split evenly over the
// compute units (17408 columns: 256 strips of 68 for M <= 256, 128 strips of 136 for larger M).  A weight sub-block
// is dequantized once per workgroup.  K advances 64 per iteration (for Q4_K the two sub-blocks that share 32 bytes of
// nibbles); a slice is two x sub-tiles [BM][32] bf16 and two weight sub-tiles [16 CT][32] bf16 in LDS (rows are 64
// bytes, placed so that the 16 rows x 4 k-groups an MFMA operand needs are one conflict-free read), in three stages:
// the slice being multiplied, the finished next one, and the one being made.
//
// The 16 waves of a workgroup are specialised, each role with a code path (and so a register allocation) of its own:
//   - 8 consumer waves (8 x 1, or 4 x 2 with 64-row, 5- or 4-tile wave tiles) only read operands from LDS and issue
//     MFMAs.  Operand reads run one tile ahead of their use, also across the barrier into the finished next slice, so
//     the matrix pipe restarts right after a barrier;
//   - 5 decoder waves, two threads per strip column: each keeps the 16 nibble bytes of its next two slices and the
//     (d * scale, dmin * min) pairs of the current 256-block in registers (the header of the next block is requested a
//     block ahead), and turns a slice into 16 low-nibble and 16 high-nibble bf16 weights;
//   - 3 waves move the x tile: requested two iterations ahead into registers, then written to the sub-tiles.
//     Nothing a producer needs after a barrier has to be waited for.
// One barrier per iteration joins the groups: while the consumers multiply slice i, the producers build slice i + 2.
// Measured with groups switched off (M = 512, 80 iterations): consumers alone 0.83 us per iteration (72 MFMAs per SIMD;
// 0.62 us at the back-to-back MFMA rate; 0.76 us without the weight-operand reads), decoders alone 0.72 us, x movers
// alone 0.64 us, all producers 0.88 us, everything together 1.33 us.  LDS is about as busy as the matrix pipe: 144 KB
// of operand reads (4 cycles per 1 KB wave read) and 50 KB of tile writes (13 cycles per 1 KB wave write, 8 cycles per
// 512-byte write: 64-bit writes gain nothing) per iteration.
#include <type_traits>

#include "nnhip_internal.h"
#include "quant_device.h"

#include "iq_grids.inc"

namespace nnhip {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kRowBytes = 64;           // one sub-tile row: 32 bf16

struct GemmArgs {
    const uint16_t* x;     // bf16 [M, K]
    const uint8_t* w;      // Q4_K [N, K/256 * 144]
    const float* bias;
    float* y;
    int M, K, N;
    int cols;              // strip width actually used, <= 16 * CT
    int strips;            // ceil(N / cols)
    int accumulate;        // 1: the products are added to what y holds (bias is not)
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b)
{
    // round to nearest even, two at a time (v_cvt_pk_bf16_f32)
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
    return __builtin_bit_cast(uint32_t, v);
}

// Two weights as bf16: their values rounded (LO = false), or what that rounding left over, w - bf16(w), rounded in turn
// (LO = true).  A launch with the second form supplies the low-order part of the weights to the three-product form of
// the mat-mul (x_hi w_hi + x_lo w_hi + x_hi w_lo).
template <bool LO>
__device__ __forceinline__ uint32_t pack_w(float a, float b)
{
    if constexpr (LO) {
        const uint32_t hi = pack_bf16(a, b);
        a -= __uint_as_float(hi << 16);
        b -= __uint_as_float(hi & 0xffff0000u);
    }
    return pack_bf16(a, b);
}

// 6-bit scale and min of sub-block g from the three dwords holding the 12 packed bytes (GgufQ4K.cs:51-60).
__device__ __forceinline__ void q4k_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int g, uint32_t& sc, uint32_t& mn)
{
    const int sh = (g & 3) * 8;
    if (g < 4) {
        sc = (s0 >> sh) & 63u;
        mn = (s1 >> sh) & 63u;
    } else {
        sc = ((s2 >> sh) & 15u) | ((((s0 >> sh) >> 6) & 3u) << 4);
        mn = (((s2 >> sh) >> 4) & 15u) | ((((s1 >> sh) >> 6) & 3u) << 4);
    }
}

template <bool LO>
__device__ __forceinline__ u32x4 q4k_decode8(uint32_t q_lo, uint32_t q_hi, float scale, float mnv)
{
    // eight weights (d*sc)*q - dmin*m as one fused multiply-add each (the bf16 rounding that follows is 2^16 times
    // coarser than the difference to the separately rounded form), packed to bf16 two at a time
    q_lo = opaque(q_lo);
    q_hi = opaque(q_hi);
    const float w0 = fmaf(scale, ubyte0(q_lo), -mnv), w1 = fmaf(scale, ubyte1(q_lo), -mnv);
    const float w2 = fmaf(scale, ubyte2(q_lo), -mnv), w3 = fmaf(scale, ubyte3(q_lo), -mnv);
    const float w4 = fmaf(scale, ubyte0(q_hi), -mnv), w5 = fmaf(scale, ubyte1(q_hi), -mnv);
    const float w6 = fmaf(scale, ubyte2(q_hi), -mnv), w7 = fmaf(scale, ubyte3(q_hi), -mnv);
    return u32x4{pack_w<LO>(w0, w1), pack_w<LO>(w2, w3), pack_w<LO>(w4, w5), pack_w<LO>(w6, w7)};
}

// A 64-byte LDS row holds four 16-byte k-groups.  Group g of row r sits in slot g ^ ((r >> 1) & 3): with that
// placement the 64 lanes of an MFMA operand read (16 rows x 4 groups) spread evenly over the banks (measured:
// 4 cycles per 128-bit read against 6.6 for the plain row-major placement), and writes stay row-contiguous.
__device__ __forceinline__ int lds_slot(int row, int group) { return group ^ ((row >> 1) & 3); }

// ---------------------------------------------------------------------------------------------------- decoders
// A decoding thread (column dc of the strip, half dh) turns its share of every 64-weight K slice into bf16 in the two
// weight sub-tiles of a stage (`lo`: weights 0-31 of the slice, `hi`: weights 32-63; a column is one 64-byte row of
// each).  What it needs for a slice was requested two slices earlier, block headers a block earlier.  One struct per
// storage format: `start()` issues the first loads, `make<J>(t, lo, hi)` writes slice t (J = t % 4) and requests ahead.
struct DecodeCtx {
    const uint8_t* wbase;    // first row of the strip (wave-uniform)
    uint32_t wrow;           // byte offset of this thread's row
    int dc, dh;
    int iters;               // K / 64
    int nblocks;             // K / 256
    bool live;               // this thread has a column
};

// Decoder threads beyond the strip's columns run the same code (no branch around the loads) and store nothing.
__device__ __forceinline__ void st128(const DecodeCtx& c, uint8_t* dst, const u32x4 v)
{
    if (c.live) *reinterpret_cast<u32x4*>(dst) = v;
}

__device__ __forceinline__ u32x4 gld128(const DecodeCtx& c, uint32_t uniform_off, uint32_t lane_off)
{
    asm volatile("" : "+s"(uniform_off));      // keeps the address as scalar base + 32-bit lane offset
    return ld128(c.wbase + uniform_off + opaque(c.wrow + lane_off));
}

// (d * scale, dmin * min) of the eight sub-blocks of a Q4_K / Q5_K block header; 6-bit fields as in GgufQ4K.cs:51-60:
// sub-blocks 0-3 sit in the low six bits of bytes j and 4 + j, 4-7 are split between bytes 8 + j (low nibble scale, high
// nibble min) and the top two bits of bytes j and 4 + j.
__device__ __forceinline__ void k4_block_scales(const u32x4 hdr, float sm[16])
{
    const float d = half_bits_to_float(hdr[0]), dmin = half_bits_to_float(hdr[0] >> 16);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t b0 = (hdr[1] >> (8 * j)) & 255u, b1 = (hdr[2] >> (8 * j)) & 255u, b2 = (hdr[3] >> (8 * j)) & 255u;
        sm[2 * j] = d * static_cast<float>(b0 & 63u);
        sm[2 * j + 1] = dmin * static_cast<float>(b1 & 63u);
        sm[8 + 2 * j] = d * static_cast<float>((b2 & 15u) | ((b0 >> 6) << 4));
        sm[8 + 2 * j + 1] = dmin * static_cast<float>((b2 >> 4) | ((b1 >> 6) << 4));
    }
}

// Q4_K: the thread owns bytes [16 dh, 16 dh + 16) of the 32 nibble bytes of a slice: 16 low-nibble weights of sub-block 2J
// and 16 high-nibble weights of sub-block 2J + 1.
template <bool LO>
struct Q4KDecodeT {
    static constexpr int kBlockBytes = 144;
    static constexpr int kAhead = 2;       // (four slices ahead measured the same)
    u32x4 nq[kAhead];           // nibble bytes of K slices t .. t + kAhead - 1
    u32x4 hdr;                  // header (d, dmin, packed scales) of the next 256-block
    float sm[16];               // (d * scale, dmin * min) of the eight sub-blocks of the current block

    __device__ __forceinline__ u32x4 load_q(const DecodeCtx& c, int t)
    {
        const int tt = min(t, c.iters - 1);
        return gld128(c, static_cast<uint32_t>(tt >> 2) * 144u + 16u + static_cast<uint32_t>(tt & 3) * 32u,
                      static_cast<uint32_t>(c.dh) * 16u);
    }
    __device__ __forceinline__ void load_hdr(const DecodeCtx& c, int blk)
    {
        hdr = gld128(c, static_cast<uint32_t>(min(blk, c.nblocks - 1)) * 144u, 0u);
    }
    __device__ __forceinline__ void start(const DecodeCtx& c)
    {
        load_hdr(c, 0);
#pragma unroll
        for (int i = 0; i < kAhead; ++i) nq[i] = load_q(c, i);
        k4_block_scales(hdr, sm);
    }
    template <int J>
    __device__ __forceinline__ void make(const DecodeCtx& c, int t, uint8_t* lo, uint8_t* hi)
    {
        const u32x4 q = nq[J % kAhead];
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const uint32_t a0 = q[2 * g], a1 = q[2 * g + 1];
            const int slot = lds_slot(c.dc, 2 * c.dh + g) * 16;
            st128(c, lo + slot, q4k_decode8<LO>(a0 & 0x0f0f0f0fu, a1 & 0x0f0f0f0fu, sm[4 * J], sm[4 * J + 1]));
            st128(c, hi + slot, q4k_decode8<LO>((a0 >> 4) & 0x0f0f0f0fu, (a1 >> 4) & 0x0f0f0f0fu, sm[4 * J + 2], sm[4 * J + 3]));
        }
        nq[J % kAhead] = load_q(c, t + kAhead);
        if (J == 0) load_hdr(c, (t >> 2) + 1);
        if (J == 3) k4_block_scales(hdr, sm);
    }
};

// Q5_K: as Q4_K with one more bit per weight: bit g of qh[i] belongs to element i of sub-block g (qh: 32 bytes after
// the header, nibbles after that).  The thread keeps bytes [16 dh, 16 dh + 16) of qh for the whole block.
template <bool LO>
struct Q5KDecodeT {
    static constexpr int kBlockBytes = 176;
    u32x4 nq[2];
    u32x4 hdr, qh_next;         // of the next block
    u32x4 qh;                   // high bits of the current block
    float sm[16];

    __device__ __forceinline__ u32x4 load_q(const DecodeCtx& c, int t)
    {
        const int tt = min(t, c.iters - 1);
        return gld128(c, static_cast<uint32_t>(tt >> 2) * 176u + 48u + static_cast<uint32_t>(tt & 3) * 32u,
                      static_cast<uint32_t>(c.dh) * 16u);
    }
    __device__ __forceinline__ void load_hdr(const DecodeCtx& c, int blk)
    {
        const uint32_t off = static_cast<uint32_t>(min(blk, c.nblocks - 1)) * 176u;
        hdr = gld128(c, off, 0u);
        qh_next = gld128(c, off + 16u, static_cast<uint32_t>(c.dh) * 16u);
    }
    __device__ __forceinline__ void start(const DecodeCtx& c)
    {
        load_hdr(c, 0);
        nq[0] = load_q(c, 0);
        nq[1] = load_q(c, 1);
        k4_block_scales(hdr, sm);
        qh = qh_next;
    }
    template <int J>
    __device__ __forceinline__ void make(const DecodeCtx& c, int t, uint8_t* lo, uint8_t* hi)
    {
        const u32x4 q = nq[J & 1];
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            const uint32_t a0 = q[2 * g], a1 = q[2 * g + 1], h0 = qh[2 * g], h1 = qh[2 * g + 1];
            const int slot = lds_slot(c.dc, 2 * c.dh + g) * 16;
            st128(c, lo + slot, q4k_decode8<LO>((a0 & 0x0f0f0f0fu) | (((h0 >> (2 * J)) & 0x01010101u) << 4),
                            (a1 & 0x0f0f0f0fu) | (((h1 >> (2 * J)) & 0x01010101u) << 4), sm[4 * J], sm[4 * J + 1]));
            st128(c, hi + slot, q4k_decode8<LO>(((a0 >> 4) & 0x0f0f0f0fu) | (((h0 >> (2 * J + 1)) & 0x01010101u) << 4),
                            ((a1 >> 4) & 0x0f0f0f0fu) | (((h1 >> (2 * J + 1)) & 0x01010101u) << 4), sm[4 * J + 2], sm[4 * J + 3]));
        }
        nq[J & 1] = load_q(c, t + 2);
        if (J == 0) load_hdr(c, (t >> 2) + 1);
        if (J == 3) {
            k4_block_scales(hdr, sm);
            qh = qh_next;
        }
    }
};

// Q6_K (GgufQ6K.cs:9-54): a block is two halves of 128 weights; in a half, weights 0-31 / 32-63 take the low nibbles of
// ql[l] / ql[32 + l] with bits 0-1 / 2-3 of qh[l], weights 64-95 / 96-127 the high nibbles with bits 4-5 / 6-7; weight =
// d * scale[16-group] * (q - 32).  Slice J of a block is half J / 2, nibble J % 2.  The thread keeps bytes
// [16 dh, 16 dh + 16) of both ql runs and of qh for a half (two slices), and the 16 scales and d for a block.
template <bool LO>
struct Q6KDecodeT {
    static constexpr int kBlockBytes = 210;
    u32x4 qa[2], qb[2], qhv[2];     // [half parity]: ql[l], ql[32 + l], qh[l] runs of the current and the next half
    u32x4 sc_next;                  // the 16 scale bytes of the next block
    uint32_t d_next;
    float ds[8];                    // d * scale of the thread's 16-weight groups: [half][group of the half]

    __device__ __forceinline__ void load_half(const DecodeCtx& c, int half_index, int set)
    {
        const int hh = min(half_index, 2 * c.nblocks - 1);
        const uint32_t blk = static_cast<uint32_t>(hh >> 1) * 210u, h = static_cast<uint32_t>(hh & 1);
        const uint32_t lane_off = static_cast<uint32_t>(c.dh) * 16u;
        qa[set] = gld128(c, blk + 64u * h, lane_off);
        qb[set] = gld128(c, blk + 64u * h + 32u, lane_off);
        qhv[set] = gld128(c, blk + 128u + 32u * h, lane_off);
    }
    __device__ __forceinline__ void load_tail(const DecodeCtx& c, int blk)
    {
        uint32_t off = static_cast<uint32_t>(min(blk, c.nblocks - 1)) * 210u;
        sc_next = gld128(c, off + 192u, 0u);
        asm volatile("" : "+s"(off));
        d_next = ld16(c.wbase + off + 208u + opaque(c.wrow));
    }
    int dh_sel;
    __device__ __forceinline__ void block_scales()
    {
        const float d = half_bits_to_float(d_next);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            // group i = 4 * half + group-of-the-half uses scale byte 2 i + dh of the 16
            const uint32_t two = (sc_next[i >> 1] >> (16 * (i & 1))) & 0xffffu;
            ds[i] = d * static_cast<float>(static_cast<int8_t>(dh_sel ? (two >> 8) : (two & 0xffu)));
        }
    }
    __device__ __forceinline__ void start(const DecodeCtx& c)
    {
        dh_sel = c.dh;
        load_tail(c, 0);
        load_half(c, 0, 0);
        load_half(c, 1, 1);
        block_scales();
    }
    // 16 weights: bytes q (6-bit values) -> d * scale * (q - 32), as one fused multiply-add each (exact: 32 * ds is a
    // power-of-two multiple of ds, so the result is ds * (q - 32) rounded once, the reference's value)
    static __device__ __forceinline__ void put16(const DecodeCtx& c, uint8_t* row, int group0, const u32x4 bytes, float dsv)
    {
        const float off = 32.0f * dsv;
#pragma unroll
        for (int g = 0; g < 2; ++g)
            st128(c, row + lds_slot(c.dc, group0 + g) * 16, q4k_decode8<LO>(bytes[2 * g], bytes[2 * g + 1], dsv, off));
    }
    template <int J>
    __device__ __forceinline__ void make(const DecodeCtx& c, int t, uint8_t* lo, uint8_t* hi)
    {
        constexpr int H = J >> 1, P = J & 1;        // half of the block, nibble
        const u32x4 a = qa[H], b = qb[H], h = qhv[H];
        u32x4 lo_b, hi_b;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lo_b[i] = ((a[i] >> (4 * P)) & 0x0f0f0f0fu) | (((h[i] >> (4 * P)) & 0x03030303u) << 4);
            hi_b[i] = ((b[i] >> (4 * P)) & 0x0f0f0f0fu) | (((h[i] >> (4 * P + 2)) & 0x03030303u) << 4);
        }
        put16(c, lo, 2 * c.dh, lo_b, ds[4 * H + 2 * P]);
        put16(c, hi, 2 * c.dh, hi_b, ds[4 * H + 2 * P + 1]);
        if (P == 1) load_half(c, (t >> 1) + 2, H);          // this half's registers are free: request the half after next
        if (J == 0) load_tail(c, (t >> 2) + 1);
        if (J == 3) block_scales();
    }
};

// Q8_0: a slice is two 34-byte blocks (d, 32 signed bytes); thread dh decodes block dh of the slice, a whole 64-byte
// row of its sub-tile.
template <bool LO>
struct Q8_0DecodeT {
    static constexpr int kBlockBytes = 34 * 8;     // bytes per 256 weights
    u32x4 q0[2], q1[2];
    uint32_t dbits[2];

    __device__ __forceinline__ void load(const DecodeCtx& c, int t, int set)
    {
        uint32_t off = static_cast<uint32_t>(min(t, c.iters - 1)) * 68u;
        const uint32_t lane_off = static_cast<uint32_t>(c.dh) * 34u;
        q0[set] = gld128(c, off + 2u, lane_off);
        q1[set] = gld128(c, off + 18u, lane_off);
        asm volatile("" : "+s"(off));
        dbits[set] = ld16(c.wbase + off + opaque(c.wrow + lane_off));
    }
    __device__ __forceinline__ void start(const DecodeCtx& c)
    {
        load(c, 0, 0);
        load(c, 1, 1);
    }
    static __device__ __forceinline__ u32x4 decode8(uint32_t a, uint32_t b, float d)
    {
        return u32x4{pack_w<LO>(d * sbyte0(a), d * sbyte1(a)), pack_w<LO>(d * sbyte2(a), d * sbyte3(a)),
                     pack_w<LO>(d * sbyte0(b), d * sbyte1(b)), pack_w<LO>(d * sbyte2(b), d * sbyte3(b))};
    }
    template <int J>
    __device__ __forceinline__ void make(const DecodeCtx& c, int t, uint8_t* lo, uint8_t* hi)
    {
        const float d = half_bits_to_float(dbits[J & 1]);
        uint8_t* row = c.dh ? hi : lo;
        const u32x4 a = q0[J & 1], b = q1[J & 1];
        st128(c, row + lds_slot(c.dc, 0) * 16, decode8(a[0], a[1], d));
        st128(c, row + lds_slot(c.dc, 1) * 16, decode8(a[2], a[3], d));
        st128(c, row + lds_slot(c.dc, 2) * 16, decode8(b[0], b[1], d));
        st128(c, row + lds_slot(c.dc, 3) * 16, decode8(b[2], b[3], d));
        load(c, t + 2, J & 1);
    }
};

// The codebooks of the IQ formats (read through the vector caches: the LDS of this kernel is taken by the tile stages).
__device__ const uint64_t g_iq2s_grid_mm[1024] = { NNHIP_IQ2S_GRID_VALUES };
__device__ const uint32_t g_iq3s_grid_mm[512] = { NNHIP_IQ3S_GRID_VALUES };

// bf16 pair of two magnitudes times db with their sign bits (bit 0 of `signs`: first weight, bit 1: second)
template <bool LO>
__device__ __forceinline__ uint32_t iq_pair(float db, float m0, float m1, uint32_t signs)
{
    return pack_w<LO>(db * m0, db * m1) ^ (((signs & 1u) << 15) | ((signs & 2u) << 30));
}

// IQ2_S (82 bytes: d, 32 index bytes, 32 sign bytes, qh[8], scales[8]; NNtrain.Arc/Kernels/qwen35_iq.cl:411-419): thread
// dh decodes 32-weight group 2 (t % 4) + dh of block t / 4, a whole 64-byte row of its sub-tile = four codebook entries
// of eight magnitudes.  Index and sign bytes are requested three slices ahead, the codebook entries one slice ahead (from
// indices that arrived two slices earlier), qh / scales / d of a block a block ahead.
template <bool LO>
struct IQ2SDecodeT {
    static constexpr int kBlockBytes = 82;
    uint32_t qs[4], sg[4];      // index and sign bytes of slices t .. t + 3 (set = slice % 4)
    u32x2 grid[2][4];           // codebook entries of slices t, t + 1 (set = slice % 2)
    u32x4 tail, tail_next;      // qh[8] | scales[8] of the current and the next block
    uint32_t dbits, dbits_next;

    __device__ __forceinline__ void load_raw(const DecodeCtx& c, int t, int set)
    {
        const int tt = min(t, c.iters - 1);
        uint32_t off = static_cast<uint32_t>(tt >> 2) * 82u + static_cast<uint32_t>(tt & 3) * 8u;
        asm volatile("" : "+s"(off));
        const uint8_t* p = c.wbase + off + opaque(c.wrow + static_cast<uint32_t>(c.dh) * 4u);
        qs[set] = ld32(p + 2);
        sg[set] = ld32(p + 34);
    }
    __device__ __forceinline__ void load_hdr(const DecodeCtx& c, int blk)
    {
        uint32_t off = static_cast<uint32_t>(min(blk, c.nblocks - 1)) * 82u;
        tail_next = gld128(c, off + 66u, 0u);
        asm volatile("" : "+s"(off));
        dbits_next = ld16(c.wbase + off + opaque(c.wrow));
    }
    // requests the entries of group 2 J + dh whose index bytes are `q`, high bits taken from `tl`
    template <int J>
    __device__ __forceinline__ void load_grid(const DecodeCtx& c, uint32_t q, const u32x4& tl, u32x2* out)
    {
        const uint32_t qh = (tl[J >> 1] >> (16 * (J & 1) + 8 * c.dh)) & 0xffu;
#pragma unroll
        for (int o = 0; o < 4; ++o) {
            const uint32_t idx = ((q >> (8 * o)) & 0xffu) | (((qh >> (2 * o)) & 3u) << 8);
            const uint64_t v = g_iq2s_grid_mm[idx];
            out[o] = u32x2{static_cast<uint32_t>(v), static_cast<uint32_t>(v >> 32)};
        }
    }
    __device__ __forceinline__ void start(const DecodeCtx& c)
    {
        load_hdr(c, 0);
        tail = tail_next;
        dbits = dbits_next;
        load_hdr(c, 1);
        load_raw(c, 0, 0);
        load_raw(c, 1, 1);
        load_raw(c, 2, 2);
        load_grid<0>(c, qs[0], tail, grid[0]);
    }
    template <int J>
    __device__ __forceinline__ void make(const DecodeCtx& c, int t, uint8_t* lo, uint8_t* hi)
    {
        const float d = half_bits_to_float(dbits);
        const uint32_t scl = (tail[2 + (J >> 1)] >> (16 * (J & 1) + 8 * c.dh)) & 0xffu;
        const float db_lo = (d * (0.5f + static_cast<float>(scl & 15u))) * 0.25f;
        const float db_hi = (d * (0.5f + static_cast<float>(scl >> 4))) * 0.25f;
        uint8_t* row = c.dh ? hi : lo;
        const uint32_t signs = sg[J];
#pragma unroll
        for (int o = 0; o < 4; ++o) {
            const uint32_t m0 = grid[J & 1][o][0], m1 = grid[J & 1][o][1], sb = signs >> (8 * o);
            const float db = o < 2 ? db_lo : db_hi;
            st128(c, row + lds_slot(c.dc, o) * 16, u32x4{iq_pair<LO>(db, ubyte0(m0), ubyte1(m0), sb), iq_pair<LO>(db, ubyte2(m0), ubyte3(m0), sb >> 2),
                      iq_pair<LO>(db, ubyte0(m1), ubyte1(m1), sb >> 4), iq_pair<LO>(db, ubyte2(m1), ubyte3(m1), sb >> 6)});
        }
        // slice t + 1 belongs to the next block when J == 3
        load_grid<(J + 1) & 3>(c, qs[(J + 1) & 3], J == 3 ? tail_next : tail, grid[(J + 1) & 1]);
        load_raw(c, t + 3, (J + 3) & 3);
        if (J == 3) {
            tail = tail_next;
            dbits = dbits_next;
        }
        if (J == 0) load_hdr(c, (t >> 2) + 1);
    }
};

// IQ3_S (110 bytes: d, 64 index bytes, qh[8], 32 sign bytes, scales[4]; qwen35_iq.cl:421-429): as IQ2_S with eight
// codebook entries of four magnitudes per 32-weight group and w = (d * (1 + 2 s)) * magnitude * sign.
template <bool LO>
struct IQ3SDecodeT {
    static constexpr int kBlockBytes = 110;
    u32x2 qs[4];                // eight index bytes of slices t .. t + 3
    uint32_t sg[4];
    uint32_t grid[2][8];
    u32x2 qh, qh_next;          // ninth index bits, a byte per group
    uint32_t scales, scales_next;
    uint32_t dbits, dbits_next;

    __device__ __forceinline__ void load_raw(const DecodeCtx& c, int t, int set)
    {
        const int tt = min(t, c.iters - 1);
        uint32_t off = static_cast<uint32_t>(tt >> 2) * 110u;
        const uint32_t g = static_cast<uint32_t>(tt & 3) * 2u + static_cast<uint32_t>(c.dh);
        asm volatile("" : "+s"(off));
        const uint8_t* p = c.wbase + off;
        qs[set] = ld64(p + 2 + opaque(c.wrow + g * 8u));
        sg[set] = ld32(p + 74 + opaque(c.wrow + g * 4u));
    }
    __device__ __forceinline__ void load_hdr(const DecodeCtx& c, int blk)
    {
        uint32_t off = static_cast<uint32_t>(min(blk, c.nblocks - 1)) * 110u;
        asm volatile("" : "+s"(off));
        const uint8_t* p = c.wbase + off + opaque(c.wrow);
        qh_next = ld64(p + 66);
        scales_next = ld32(p + 106);
        dbits_next = ld16(p);
    }
    template <int J>
    __device__ __forceinline__ void load_grid(const DecodeCtx& c, const u32x2 q, const u32x2 high, uint32_t* out)
    {
        const uint32_t hb = (high[J >> 1] >> (16 * (J & 1) + 8 * c.dh)) & 0xffu;
#pragma unroll
        for (int o = 0; o < 8; ++o) {
            const uint32_t idx = ((q[o >> 2] >> (8 * (o & 3))) & 0xffu) | (((hb >> o) & 1u) << 8);
            out[o] = g_iq3s_grid_mm[idx];
        }
    }
    __device__ __forceinline__ void start(const DecodeCtx& c)
    {
        load_hdr(c, 0);
        qh = qh_next;
        scales = scales_next;
        dbits = dbits_next;
        load_hdr(c, 1);
        load_raw(c, 0, 0);
        load_raw(c, 1, 1);
        load_raw(c, 2, 2);
        load_grid<0>(c, qs[0], qh, grid[0]);
    }
    template <int J>
    __device__ __forceinline__ void make(const DecodeCtx& c, int t, uint8_t* lo, uint8_t* hi)
    {
        // group 2 J + dh: its scale nibble is nibble (2 J + dh) of the four scale bytes
        const uint32_t sub = (scales >> (8 * J + 4 * c.dh)) & 15u;
        const float db = half_bits_to_float(dbits) * static_cast<float>(1u + 2u * sub);
        uint8_t* row = c.dh ? hi : lo;
        const uint32_t signs = sg[J];
#pragma unroll
        for (int o = 0; o < 4; ++o) {
            const uint32_t m0 = grid[J & 1][2 * o], m1 = grid[J & 1][2 * o + 1], sb = signs >> (8 * o);
            st128(c, row + lds_slot(c.dc, o) * 16, u32x4{iq_pair<LO>(db, ubyte0(m0), ubyte1(m0), sb), iq_pair<LO>(db, ubyte2(m0), ubyte3(m0), sb >> 2),
                      iq_pair<LO>(db, ubyte0(m1), ubyte1(m1), sb >> 4), iq_pair<LO>(db, ubyte2(m1), ubyte3(m1), sb >> 6)});
        }
        load_grid<(J + 1) & 3>(c, qs[(J + 1) & 3], J == 3 ? qh_next : qh, grid[(J + 1) & 1]);
        load_raw(c, t + 3, (J + 3) & 3);
        if (J == 3) {
            qh = qh_next;
            scales = scales_next;
            dbits = dbits_next;
        }
        if (J == 0) load_hdr(c, (t >> 2) + 1);
    }
};

using Q4KDecode = Q4KDecodeT<false>;
using Q5KDecode = Q5KDecodeT<false>;
using Q6KDecode = Q6KDecodeT<false>;
using Q8_0Decode = Q8_0DecodeT<false>;
using IQ2SDecode = IQ2SDecodeT<false>;
using IQ3SDecode = IQ3SDecodeT<false>;

// Unquantized bfloat16 weights (matrix storage type 30, and the scratch copy the two-pass path decodes into): thread dh
// copies weights [32 dh, 32 dh + 32) of the slice, a whole 64-byte row of its sub-tile.
struct BF16Decode {
    static constexpr int kBlockBytes = 512;        // bytes per 256 weights
    u32x4 q[2][4];

    __device__ __forceinline__ void load(const DecodeCtx& c, int t, int set)
    {
        const uint32_t off = static_cast<uint32_t>(min(t, c.iters - 1)) * 128u;
        const uint32_t lane_off = static_cast<uint32_t>(c.dh) * 64u;
#pragma unroll
        for (int g = 0; g < 4; ++g) q[set][g] = gld128(c, off + 16u * g, lane_off);
    }
    __device__ __forceinline__ void start(const DecodeCtx& c)
    {
        load(c, 0, 0);
        load(c, 1, 1);
    }
    template <int J>
    __device__ __forceinline__ void make(const DecodeCtx& c, int t, uint8_t* lo, uint8_t* hi)
    {
        uint8_t* row = c.dh ? hi : lo;
#pragma unroll
        for (int g = 0; g < 4; ++g) st128(c, row + lds_slot(c.dc, g) * 16, q[J & 1][g]);
        load(c, t + 2, J & 1);
    }
};

constexpr int kConsumers = 512;         // 8 MFMA waves
constexpr int kProducers = 512;         // 8 waves that fill LDS: waves 8-12 decode weights, waves 13-15 move the x tile
constexpr int kDecoders = 320;          // producer threads reserved for decoding (two per strip column are used)
constexpr int kXThreads = kProducers - kDecoders;
constexpr int kGemmAll = kConsumers + kProducers;
constexpr int kStages = 3;              // LDS tile stages: multiplied, ready (being pre-read), being made

// Consumer waves are laid out WM x WN (8 in all); a wave owns RW rows and, when WN == 2, the first CTW or the
// remaining CT - CTW column tiles.
template <class F, int RW, int CT, int WN>
__global__ __launch_bounds__(kGemmAll) void matmul_bf16_kernel(GemmArgs a)
{
    constexpr int WM = 8 / WN;
    constexpr int BM = WM * RW;
    constexpr int MT = RW / 16;                     // 16-row MFMA tiles per wave
    constexpr int BN = 16 * CT;
    constexpr int CTW = (CT + WN - 1) / WN;         // column tiles of the widest wave
    constexpr int kXTile = BM * kRowBytes;          // bytes of one x sub-tile
    constexpr int kWTile = BN * kRowBytes;          // bytes of one weight sub-tile
    // dynamic LDS: xs[stage][k sub-tile][row][32 bf16] then ws[stage][k sub-tile][column][32 bf16], kStages stages
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* xs = smem;
    uint8_t* ws = smem + kStages * 2 * kXTile;

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int strip = blockIdx.x, m0 = blockIdx.y * BM;
    const int n0 = strip * a.cols;
    const int iters = a.K >> 6;

    if (wave >= kConsumers / 64) {
        // ------------------------------------------------------------------------------------------ producers
        // Both producer roles make slices 0 and 1 before the first barrier and then, between two barriers, slice
        // i + 2 while slice i is multiplied.  Everything a role consumes was requested two slices earlier.  The
        // roles are separate code paths so that each is allocated only its own registers.
        // With 128-row tiles the decoders are what an iteration waits for, with 256-row tiles the matrix pipes:
        // the group on the critical path gets the higher issue priority (measured: +3 % at M = 128, +2.5 % at M = 2048).
        if constexpr (BM <= 128) __builtin_amdgcn_s_setprio(3);
        const int p = tid - kConsumers;
        // K is a whole number of 256-blocks, so iters is a multiple of 4; `make(t, stage)` is given t % 4 statically
        auto run = [&](auto&& make) {
            using std::integral_constant;
            make(0, 0, integral_constant<int, 0>{});
            make(1, 1, integral_constant<int, 1>{});
            __syncthreads();
            int stage = 2;
            auto next_stage = [&]() { stage = stage == kStages - 1 ? 0 : stage + 1; };
            // No test on "is there a slice i + 2": the two slices past the end are made from repeated input into stages
            // that nobody reads any more.  With the calls unconditional the loop is one basic block per role, and the
            // compiler's wait before a slice's registers are used counts the younger requests as still outstanding
            // (with branches it waited for all of them, which left one iteration of cover instead of two: at 0.7 us
            // per iteration, M <= 256, that was the memory latency).
            for (int i = 0; i < iters; i += 4) {
                make(i + 2, stage, integral_constant<int, 2>{});
                next_stage();
                __syncthreads();
                make(i + 3, stage, integral_constant<int, 3>{});
                next_stage();
                __syncthreads();
                make(i + 4, stage, integral_constant<int, 0>{});
                next_stage();
                __syncthreads();
                make(i + 5, stage, integral_constant<int, 1>{});
                next_stage();
                __syncthreads();
            }
        };

        if (p >= kDecoders) {
            // ---- x movers (waves 13-15): a piece is one 16-byte group (8 of the 64 values) of one row of the tile; a
            // thread moves pieces xp, xp + 192, ...  Within a wave's 64 pieces (8 rows x 8 groups) a quarter-wave takes
            // 4 rows x 4 groups of one sub-tile: 256 contiguous bytes of LDS, every bank once.
            constexpr int kXPieces = 2 * kXTile / 16;
            constexpr int kXLoads = (kXPieces + kXThreads - 1) / kXThreads;
            const int xp = p - kDecoders;
            const uint8_t* xbase = reinterpret_cast<const uint8_t*>(a.x + static_cast<size_t>(m0) * a.K);   // wave-uniform
            uint32_t xsrc[kXLoads];     // byte offsets from xbase (a tile spans at most 256 rows)
            int xdst[kXLoads];
#pragma unroll
            for (int i = 0; i < kXLoads; ++i) {
                const int q = min(xp + i * kXThreads, kXPieces - 1);       // the last round is partly idle (not stored)
                const int l = q & 63, quarter = l >> 4, within = l & 15;
                const int r = (q >> 6) * 8 + (quarter >> 1) * 4 + (within >> 2), grp = (quarter & 1) * 4 + (within & 3);
                xsrc[i] = static_cast<uint32_t>((min(r, a.M - 1 - m0) * a.K + grp * 8) * 2);
                xdst[i] = (grp >> 2) * kXTile + r * kRowBytes + lds_slot(r, grp & 3) * 16;
            }
            u32x4 xset[2][kXLoads];     // x pieces of K slices t and t + 1
            auto load_x = [&](u32x4* set, int t) {
                uint32_t koff = static_cast<uint32_t>(min(t, iters - 1)) << 7;     // past the end: a harmless repeat
                asm volatile("" : "+s"(koff));      // keeps the address as scalar base + 32-bit lane offset
                const uint8_t* src = xbase + koff;
#pragma unroll
                for (int i = 0; i < kXLoads; ++i) set[i] = *reinterpret_cast<const u32x4*>(src + opaque(xsrc[i]));
            };
            load_x(xset[0], 0);
            load_x(xset[1], 1);
            run([&](int t, int stage, auto jt) {
                constexpr int J = decltype(jt)::value;
                u32x4* set = xset[J & 1];
                uint8_t* xb = xs + stage * 2 * kXTile;
#pragma unroll
                for (int i = 0; i < kXLoads; ++i)
                    if ((i + 1) * kXThreads <= kXPieces || xp + i * kXThreads < kXPieces)
                        *reinterpret_cast<u32x4*>(xb + xdst[i]) = set[i];
                load_x(set, t + 2);
            });
            return;
        }

        // ---- decoders (waves 8-12): two threads per strip column, see the format's decoder struct
        static_assert(2 * BN <= kDecoders, "two decoding threads per column");
        const int row_bytes = (a.K >> 8) * F::kBlockBytes;
        const bool d_role = p < 2 * BN;
        if ((p & ~63) >= 2 * BN) return;        // a whole wave without columns: ended waves do not count at barriers

        DecodeCtx c;
        c.live = d_role;
        c.dc = d_role ? p >> 1 : 0;
        c.dh = p & 1;
        c.wbase = a.w + static_cast<size_t>(n0) * row_bytes;                               // wave-uniform
        c.wrow = static_cast<uint32_t>(min(c.dc, a.N - 1 - n0) * row_bytes);              // byte offset
        c.iters = iters;
        c.nblocks = a.K >> 8;
        F dec;
        dec.start(c);
        run([&](int t, int stage, auto jt) {
            constexpr int J = decltype(jt)::value;
            uint8_t* wb = ws + stage * 2 * kWTile + c.dc * kRowBytes;
            dec.template make<J>(c, t, wb, wb + kWTile);
        });
        return;
    }

    // ---------------------------------------------------------------------------------------------- consumers
    // waves w and w + 4 usually share a SIMD: giving them different column halves balances the matrix pipes
    if constexpr (BM > 128) __builtin_amdgcn_s_setprio(3);
    const int uwave = __builtin_amdgcn_readfirstlane(wave);     // wave-uniform values stay in scalar registers
    const int wm = uwave % WM, wn = uwave / WM;
    const int ct0 = wn * CTW;                       // this wave's column tiles start here
    // operand address of this lane inside a 16-row tile: row lane % 16, k-group lane / 16
    const int frag = (lane & 15) * kRowBytes + lds_slot(lane & 15, lane >> 4) * 16;

    // The whole consumer body is instantiated per tile count NT, so the loop is straight-line code: a wave-uniform
    // "does this wave have a fifth tile" test inside the loop would put that tile's operand read and its wait in a
    // block of their own, twice per iteration.
    auto consume = [&](auto nt_tag) {
        constexpr int NT = decltype(nt_tag)::value;
        f32x4 acc[MT][NT];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        const uint8_t* xrow = xs + wm * RW * kRowBytes + frag;
        const uint8_t* wcol = ws + ct0 * 16 * kRowBytes + frag;
        __syncthreads();        // tiles 0 and 1 are ready
        // Operand fetches run ahead of the matrix instructions that use them, also across the barrier into the next
        // slice, which was completed one iteration earlier: the x fragments of a half-slice are read while the previous
        // half is multiplied.  The scheduling barriers keep the compiler from sinking the reads down to their first use.
        static_assert(kStages == 3, "the slice phase below is also the LDS stage");
        // Weight fragments in a ring of three, read two tiles ahead of their use.  The ring position of a slice's
        // first tile and the LDS stage both repeat every three slices, so the loop is unrolled by three and both
        // are compile-time constants; one or two more slices follow when K / 64 is not a multiple of three.
        constexpr int kTiles = 2 * NT;
        bf16x8 afrag[MT], afrag1[MT], bq[3];
        auto tile_at = [&](const uint8_t* w, int u) { return w + (u / NT) * kWTile + (u % NT) * 16 * kRowBytes; };
#pragma unroll
        for (int u = 0; u < 2; ++u) bq[u] = *reinterpret_cast<const bf16x8*>(tile_at(wcol, u));
#pragma unroll
        for (int i = 0; i < MT; ++i) afrag[i] = *reinterpret_cast<const bf16x8*>(xrow + i * 16 * kRowBytes);
        auto slice = [&](auto phase) {
            constexpr int P = decltype(phase)::value;         // iteration % 3 = LDS stage
            constexpr int PN = (P + 1) % kStages;
            const uint8_t* xb = xrow + P * 2 * kXTile;
            const uint8_t* wb = wcol + P * 2 * kWTile;
            const uint8_t* xn = xrow + PN * 2 * kXTile;
            const uint8_t* wn_ = wcol + PN * 2 * kWTile;
#pragma unroll
            for (int t = 0; t < kTiles; ++t) {
                constexpr int kShift = P * (kTiles % 3);
                const int slot = (kShift + t) % 3;
                bq[(slot + 2) % 3] = *reinterpret_cast<const bf16x8*>(t + 2 < kTiles ? tile_at(wb, t + 2) : tile_at(wn_, t + 2 - kTiles));
                if (t == 0) {
#pragma unroll
                    for (int i = 0; i < MT; ++i) afrag1[i] = *reinterpret_cast<const bf16x8*>(xb + kXTile + i * 16 * kRowBytes);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    acc[i][t % NT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t < NT ? afrag[i] : afrag1[i], bq[slot], acc[i][t % NT], 0, 0, 0);
                if (t == NT - 1) {
#pragma unroll
                    for (int i = 0; i < MT; ++i) afrag[i] = *reinterpret_cast<const bf16x8*>(xn + i * 16 * kRowBytes);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            __syncthreads();
        };
        int it = 0;
        for (; it + 3 <= iters; it += 3) {
            slice(std::integral_constant<int, 0>{});
            slice(std::integral_constant<int, 1>{});
            slice(std::integral_constant<int, 2>{});
        }
        if (it < iters) slice(std::integral_constant<int, 0>{});
        if (it + 1 < iters) slice(std::integral_constant<int, 1>{});
        // accumulator element v of a tile: row 4 * (lane / 16) + v, column lane % 16.  (The lane number is taken
        // afresh so that nothing derived from it occupies a register during the loop.)
        const int lane = static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)));
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const int cn = (ct0 + j) * 16 + (lane & 15);
            const int n = n0 + cn;
            if (cn < a.cols && n < a.N) {
                const float b = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
                for (int i = 0; i < MT; ++i) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int m = m0 + wm * RW + i * 16 + (lane >> 4) * 4 + v;
                        if (m < a.M) {
                            float* out = a.y + static_cast<size_t>(m) * a.N + n;
                            *out = a.accumulate ? *out + acc[i][j][v] : acc[i][j][v] + b;
                        }
                    }
                }
            }
        }
    };
    constexpr int kLastTiles = CT - (WN - 1) * CTW;     // tiles of the last wave column
    if (kLastTiles == CTW || wn < WN - 1) consume(std::integral_constant<int, CTW>{});
    else consume(std::integral_constant<int, kLastTiles>{});
}

template <class F, int RW, int CT, int WN>
hipError_t launch_gemm(Lane* lane, const GemmArgs& a, dim3 grid)
{
    constexpr int BM = (8 / WN) * RW, BN = 16 * CT;
    constexpr size_t lds = static_cast<size_t>(kStages) * 2 * (BM + BN) * kRowBytes;
    static LdsLimit big_lds;
    if (lds > 48 * 1024) {
        const hipError_t e = big_lds.ensure(lane->device, reinterpret_cast<const void*>(&matmul_bf16_kernel<F, RW, CT, WN>),
                                            static_cast<int>(lds));
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((matmul_bf16_kernel<F, RW, CT, WN>), grid, dim3(kGemmAll), lds, lane->stream, a);
    return hipGetLastError();
}

template <class F>
hipError_t launch_matmul_of(Lane* lane, const uint16_t* x, const void* w, const float* bias, float* y, int rows, int in_w,
                            int out_w, bool accumulate)
{
    GemmArgs a{};
    a.accumulate = accumulate ? 1 : 0;
    a.x = x;
    a.w = static_cast<const uint8_t*>(w);
    a.bias = bias;
    a.y = y;
    a.M = rows;
    a.K = in_w;
    a.N = out_w;
    // Three tilings: 128 rows x 80 columns, 256 x 80 and 256 x 144 per workgroup.  For each, the strips are as wide as the
    // column tiles allow, narrowed so that strips x row tiles is a whole number of rounds over the compute units when
    // that keeps them >= 70 % wide; the one with the shortest estimated launch is taken (rounds x time of a K step of
    // that tiling, measured on 17408 x 5120: 0.64 / 0.99 / 1.33 us, a quarter of it scaled with the strip width; ties go to the larger
    // tile).  The large tile wins where it fills the device (17408 columns at M >= 512); a matrix with few columns
    // (a down projection: 5120 x 17408 makes 76 workgroups of 256 x 144) runs on more, smaller tiles: measured at
    // M = 512, 0.261 -> 0.162 ms; 4096 x 4096 0.074 -> 0.042 ms.
    struct Tiling { int bm, max_cols; double step_us; };
    static const Tiling tilings[3] = {{128, 80, 0.64}, {256, 80, 0.99}, {256, 144, 1.33}};
    int best = -1, best_cols = 0, best_strips = 0, best_m_tiles = 0;
    double best_cost = 0.0;
    const int per_round = lane->compute_units;
    for (int t = 0; t < 3; ++t) {
        const Tiling& tl = tilings[t];
        if (t == 0 && rows > 128 && rows <= 256) continue;          // (two row tiles of 128 are never better than one of 256)
        const int m_tiles = (rows + tl.bm - 1) / tl.bm;
        int strips = (out_w + tl.max_cols - 1) / tl.max_cols;
        const int even = (strips * m_tiles + per_round - 1) / per_round * per_round / m_tiles;
        if (even > strips && (out_w + even - 1) / even * 10 >= tl.max_cols * 7) strips = even;
        const int cols = (out_w + strips - 1) / strips;
        strips = (out_w + cols - 1) / cols;
        const int rounds = (strips * m_tiles + per_round - 1) / per_round;
        // (rows of a last, ragged row tile cost as much as a full one)
        const double cost = rounds * tl.step_us * (0.75 + 0.25 * cols / tl.max_cols);
        if (best < 0 || cost <= best_cost * 1.02) {
            best = t;
            best_cost = cost;
            best_cols = cols;
            best_strips = strips;
            best_m_tiles = m_tiles;
        }
    }
    a.cols = best_cols;
    a.strips = best_strips;
    const dim3 grid(a.strips, best_m_tiles);
    if (best == 0) return launch_gemm<F, 16, 5, 1>(lane, a, grid);
    if (best == 1) return launch_gemm<F, 32, 5, 1>(lane, a, grid);
    return launch_gemm<F, 64, 9, 2>(lane, a, grid);
}

}  // namespace

namespace {

// FP32 -> bfloat16 (round to nearest even), eight values per thread; the last thread group handles the ragged end.
__global__ __launch_bounds__(256) void to_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ out, size_t count)
{
    const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
    if (i + 8 <= count) {
        const float4 a = *reinterpret_cast<const float4*>(x + i), b = *reinterpret_cast<const float4*>(x + i + 4);
        *reinterpret_cast<u32x4*>(out + i) = u32x4{pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w)};
    } else {
        for (size_t j = i; j < count; ++j) out[j] = static_cast<uint16_t>(pack_bf16(x[j], 0.0f) & 0xffffu);
    }
}

}  // namespace

namespace {

// FP32 -> the two bfloat16 parts of the three-product mat-mul: hi = bf16(x), lo = bf16(x - hi); x - hi - lo is below
// 2^-17 of x.  Eight values per thread.
__global__ __launch_bounds__(256) void to_bf16_parts_kernel(const float* __restrict__ x, uint16_t* __restrict__ hi,
                                                            uint16_t* __restrict__ lo, size_t count)
{
    const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
    if (i + 8 <= count) {
        const float4 a = *reinterpret_cast<const float4*>(x + i), b = *reinterpret_cast<const float4*>(x + i + 4);
        *reinterpret_cast<u32x4*>(hi + i) = u32x4{pack_w<false>(a.x, a.y), pack_w<false>(a.z, a.w), pack_w<false>(b.x, b.y), pack_w<false>(b.z, b.w)};
        *reinterpret_cast<u32x4*>(lo + i) = u32x4{pack_w<true>(a.x, a.y), pack_w<true>(a.z, a.w), pack_w<true>(b.x, b.y), pack_w<true>(b.z, b.w)};
    } else {
        for (size_t j = i; j < count; ++j) {
            hi[j] = static_cast<uint16_t>(pack_w<false>(x[j], 0.0f) & 0xffffu);
            lo[j] = static_cast<uint16_t>(pack_w<true>(x[j], 0.0f) & 0xffffu);
        }
    }
}

}  // namespace

hipError_t launch_to_bf16_parts(Lane* lane, const float* x, uint16_t* hi, uint16_t* lo, size_t count)
{
    const size_t groups = (count + 2047) / 2048;
    hipLaunchKernelGGL(to_bf16_parts_kernel, dim3(static_cast<unsigned>(groups)), dim3(256), 0, lane->stream, x, hi, lo, count);
    return hipGetLastError();
}

hipError_t launch_to_bf16(Lane* lane, const float* x, uint16_t* out, size_t count)
{
    const size_t groups = (count + 2047) / 2048;
    hipLaunchKernelGGL(to_bf16_kernel, dim3(static_cast<unsigned>(groups)), dim3(256), 0, lane->stream, x, out, count);
    return hipGetLastError();
}

bool matmul_bf16_supported(uint32_t type, int in_w)
{
    switch (type) {
    case NNHIP_TYPE_Q4_K: case NNHIP_TYPE_Q5_K: case NNHIP_TYPE_Q6_K: case NNHIP_TYPE_Q8_0: case NNHIP_TYPE_IQ2_S:
    case NNHIP_TYPE_IQ3_S: case NNHIP_TYPE_BF16: return in_w % 256 == 0;
    default: return false;
    }
}

hipError_t launch_matmul_bf16(Lane* lane, uint32_t type, const uint16_t* x, const void* w, const float* bias, float* y,
                              int rows, int in_w, int out_w, bool low_weight_part, bool accumulate)
{
    if (low_weight_part) {
        switch (type) {
        case NNHIP_TYPE_Q4_K: return launch_matmul_of<Q4KDecodeT<true>>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
        case NNHIP_TYPE_Q5_K: return launch_matmul_of<Q5KDecodeT<true>>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
        case NNHIP_TYPE_Q6_K: return launch_matmul_of<Q6KDecodeT<true>>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
        case NNHIP_TYPE_Q8_0: return launch_matmul_of<Q8_0DecodeT<true>>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
        case NNHIP_TYPE_IQ2_S: return launch_matmul_of<IQ2SDecodeT<true>>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
        case NNHIP_TYPE_IQ3_S: return launch_matmul_of<IQ3SDecodeT<true>>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
        default: return hipErrorNotSupported;        // (bfloat16 weights have no low-order part)
        }
    }
    switch (type) {
    case NNHIP_TYPE_Q4_K: return launch_matmul_of<Q4KDecode>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
    case NNHIP_TYPE_Q5_K: return launch_matmul_of<Q5KDecode>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
    case NNHIP_TYPE_Q6_K: return launch_matmul_of<Q6KDecode>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
    case NNHIP_TYPE_Q8_0: return launch_matmul_of<Q8_0Decode>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
    case NNHIP_TYPE_IQ2_S: return launch_matmul_of<IQ2SDecode>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
    case NNHIP_TYPE_IQ3_S: return launch_matmul_of<IQ3SDecode>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
    case NNHIP_TYPE_BF16: return launch_matmul_of<BF16Decode>(lane, x, w, bias, y, rows, in_w, out_w, accumulate);
    default: return hipErrorNotSupported;
    }
}

// y = bias + x w^T with both operands as the sum of two bfloat16 parts: three launches, x_hi w_hi (+ bias), then
// x_lo w_hi and x_hi w_lo added to it (the fourth product, x_lo w_lo, is below 2^-16 of the first and left out).
hipError_t launch_matmul_parts(Lane* lane, uint32_t type, const uint16_t* x_hi, const uint16_t* x_lo, const void* w, const float* bias,
                               float* y, int rows, int in_w, int out_w, int* launches)
{
    *launches = 0;
    hipError_t e = launch_matmul_bf16(lane, type, x_hi, w, bias, y, rows, in_w, out_w, false, false);
    if (e != hipSuccess) return e;
    ++*launches;
    e = launch_matmul_bf16(lane, type, x_lo, w, nullptr, y, rows, in_w, out_w, false, true);
    if (e != hipSuccess) return e;
    ++*launches;
    if (type == NNHIP_TYPE_BF16) return hipSuccess;
    e = launch_matmul_bf16(lane, type, x_hi, w, nullptr, y, rows, in_w, out_w, true, true);
    if (e == hipSuccess) ++*launches;
    return e;
}

}  // namespace nnhip
