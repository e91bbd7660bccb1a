// Prefill mat-mul for raw GGUF Q4_K weights on gfx950: y[M, N] = bias + x[M, K] (bf16) . W[N, K]^T.
//
// Replaces the XMX prefill launch of the reference (NNtrain.Arc/Kernels/qwen35_prefill_xmx.cl:112-184): weight tiles
// are dequantized to bfloat16 in LDS and contracted on the matrix cores (v_mfma_f32_16x16x32_bf16) with FP32
// accumulators.  The weight is the CPU decoder's (d*sc)*q - dmin*m (NNtrain.Core/Serialization/GgufQ4K.cs:34-41)
// evaluated in FP32 and rounded once to bf16, which is what the 2e-3 relative-L2 bar of this path allows for.
//
// Tiling.  A workgroup owns BM rows (128 or 256) and a strip of up to 16 * CT output columns (CT = 5 or 9 column tiles)
// for the whole K range; the strip width is chosen on the host so that strips x row tiles split evenly over the
// compute units (17408 columns: 256 strips of 68 for M <= 256, 128 strips of 136 for larger M).  A weight sub-block
// is dequantized once per workgroup.  K advances 64 per iteration = the two Q4_K sub-blocks that share 32 bytes of
// nibbles; per iteration two x sub-tiles [BM][32] bf16 and two weight sub-tiles [16 CT][32] bf16 live in LDS, double
// buffered (rows are 64 bytes, so the 16 rows x 4 k-groups an MFMA operand needs form one contiguous, conflict-free
// 1 KiB read).
//
// The 13 waves of a workgroup are specialised:
//   - 8 consumer waves (8 x 1, or 4 x 2 with 64-row, 5- or 4-tile wave tiles) only read operands from LDS and issue
//     MFMAs;
//   - 5 producer waves fill LDS.  Four of them move the x tile (requested two iterations ahead into registers, then
//     written to the swizzled sub-tiles).  The raw Q4_K blocks of the strip are staged in LDS one 256-block ahead
//     (144 contiguous bytes per column instead of 8-byte pieces per K slice, which keeps the cache-line count per
//     load instruction low), their eight (d * scale, dmin * min) pairs are computed once per block, and two threads
//     per column turn the 32 nibble bytes of a K slice into 32 low-nibble and 32 high-nibble bf16 weights.
// One barrier per iteration joins the two groups: while the consumers multiply slice i, the producers build slice
// i + 1 in the other LDS buffer.  Measured with either group switched off, the consumers alone take about 1.0 us per
// iteration (72 MFMAs per SIMD) and the producers alone about 1.2 us; together 1.6 us.
#include <type_traits>

#include "nnhip_internal.h"
#include "quant_device.h"

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
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b)
{
    // round to nearest even, two at a time (v_cvt_pk_bf16_f32)
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
    return __builtin_bit_cast(uint32_t, v);
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
    return u32x4{pack_bf16(w0, w1), pack_bf16(w2, w3), pack_bf16(w4, w5), pack_bf16(w6, w7)};
}

// A 64-byte LDS row holds four 16-byte k-groups.  Group g of row r sits in slot g ^ ((r >> 1) & 3): with that
// placement the 64 lanes of an MFMA operand read (16 rows x 4 groups) spread evenly over the banks (measured:
// 4 cycles per 128-bit read against 6.6 for the plain row-major placement), and writes stay row-contiguous.
__device__ __forceinline__ int lds_slot(int row, int group) { return group ^ ((row >> 1) & 3); }

constexpr int kConsumers = 512;         // 8 MFMA waves
constexpr int kProducers = 320;         // 5 waves that fetch, decode and fill LDS
constexpr int kXThreads = 256;          // the producer threads that also move the x tile
constexpr int kGemmAll = kConsumers + kProducers;

// Consumer waves are laid out WM x WN (8 in all); a wave owns RW rows and, when WN == 2, the first CTW or the
// remaining CT - CTW column tiles.
template <int RW, int CT, int WN>
__global__ __launch_bounds__(kGemmAll) void matmul_q4k_bf16_kernel(GemmArgs a)
{
    constexpr int WM = 8 / WN;
    constexpr int BM = WM * RW;
    constexpr int MT = RW / 16;                     // 16-row MFMA tiles per wave
    constexpr int BN = 16 * CT;
    constexpr int CTW = (CT + WN - 1) / WN;         // column tiles of the widest wave
    constexpr int kXTile = BM * kRowBytes;          // bytes of one x sub-tile
    constexpr int kWTile = BN * kRowBytes;          // bytes of one weight sub-tile
    constexpr int kRawBytes = BN * 144;             // one Q4_K block of every strip column
    constexpr int kSclBytes = BN * 64;              // its eight (scale, min) pairs
    // dynamic LDS: xs[buffer][k sub-tile][row][32 bf16] then ws[buffer][k sub-tile][column][32 bf16]
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* xs = smem;
    uint8_t* ws = smem + 4 * kXTile;
    uint8_t* raw = ws + 4 * kWTile;                 // raw[buffer][column][144]: the Q4_K blocks of two K blocks
    uint8_t* scl = raw + 2 * kRawBytes;             // scl[buffer][column][sub-block][d * scale, dmin * min] as FP32

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int strip = blockIdx.x, m0 = blockIdx.y * BM;
    const int n0 = strip * a.cols;
    const int iters = a.K >> 6;

    if (wave >= kConsumers / 64) {
        // ------------------------------------------------------------------------------------------ producers
        constexpr int kXLoads = 2 * kXTile / 16 / kXThreads;                   // 16-byte pieces of x per thread
        constexpr int kRawPieces = BN * 9;                                     // 16-byte pieces of one block column set
        constexpr int kRawLoads = (kRawPieces + kProducers - 1) / kProducers;
        static_assert(kXLoads >= 1, "tile too small for the producer count");
        static_assert(2 * BN <= kProducers, "two decoding threads per column");
        const int p = tid - kConsumers;
        const int row_bytes = (a.K >> 8) * 144;
        // x piece q of this thread: row q / 8 of the tile, 16-byte group q % 8 of the 64-value K slice
        const bool x_role = p < kXThreads;
        const uint8_t* xbase = reinterpret_cast<const uint8_t*>(a.x + static_cast<size_t>(m0) * a.K);   // wave-uniform
        uint32_t xsrc[kXLoads];     // byte offsets from xbase (a tile spans at most 256 rows)
        int xdst[kXLoads];
#pragma unroll
        for (int i = 0; i < kXLoads; ++i) {
            const int q = (x_role ? p : 0) + i * kXThreads;
            const int r = q >> 3, grp = q & 7;
            xsrc[i] = static_cast<uint32_t>((min(r, a.M - 1 - m0) * a.K + grp * 8) * 2);
            xdst[i] = (grp >> 2) * kXTile + r * kRowBytes + lds_slot(r, grp & 3) * 16;
        }
        // raw piece id of this thread: 16-byte part id % 9 of the 144-byte block of strip column id / 9; the staging
        // area is [column][144 bytes], so piece id lands at byte 16 * id
        const uint8_t* wbase = a.w + static_cast<size_t>(n0) * row_bytes;                               // wave-uniform
        uint32_t rsrc[kRawLoads];   // byte offsets from wbase
#pragma unroll
        for (int i = 0; i < kRawLoads; ++i) {
            const int id = min(p + i * kProducers, kRawPieces - 1);
            const int col = id / 9, part = id - col * 9;
            rsrc[i] = static_cast<uint32_t>(min(col, a.N - 1 - n0) * row_bytes + part * 16);
        }
        // decoding: thread (column dc, half dh) owns bytes [16 dh, 16 dh + 16) of the 32 nibble bytes of a K slice
        const bool d_role = p < 2 * BN;
        const int dc = d_role ? p >> 1 : 0, dh = p & 1;
        const int nblocks = a.K >> 8;
        u32x4 xset[2][kXLoads];
        u32x4 rawreg[kRawLoads];
        auto load_x = [&](u32x4* set, int t) {
            uint32_t koff = static_cast<uint32_t>(min(t, iters - 1)) << 7;     // past the end: a harmless repeat of the last slice
            asm volatile("" : "+s"(koff));      // keeps the address as scalar base + 32-bit lane offset
            const uint8_t* src = xbase + koff;
#pragma unroll
            for (int i = 0; i < kXLoads; ++i) set[i] = *reinterpret_cast<const u32x4*>(src + opaque(xsrc[i]));
        };
        auto load_raw = [&](int blk) {
            uint32_t boff = static_cast<uint32_t>(min(blk, nblocks - 1)) * 144u;
            asm volatile("" : "+s"(boff));
            const uint8_t* src = wbase + boff;
#pragma unroll
            for (int i = 0; i < kRawLoads; ++i) rawreg[i] = ld128(src + opaque(rsrc[i]));
        };
        auto store_raw = [&](int buf) {
            uint8_t* dst = raw + buf * kRawBytes;
#pragma unroll
            for (int i = 0; i < kRawLoads; ++i) {
                const int id = p + i * kProducers;
                if (id < kRawPieces) *reinterpret_cast<u32x4*>(dst + id * 16) = rawreg[i];
            }
        };
        // (d * scale, dmin * min) of sub-blocks 4 dh .. 4 dh + 3 of the staged block, as FP32, for the decoding steps
        auto make_scales = [&](int buf) {
            if (!d_role) return;
            const u32x4 hdr = *reinterpret_cast<const u32x4*>(raw + buf * kRawBytes + dc * 144);
            const float d = half_bits_to_float(hdr[0]), dmin = half_bits_to_float(hdr[0] >> 16);
            float v[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // 6-bit fields (GgufQ4K.cs:51-60): sub-blocks 0-3 sit in the low six bits of bytes j and 4 + j; 4-7 are
                // split between bytes 8 + j (low nibble scale, high nibble min) and the top two bits of bytes j, 4 + j
                const uint32_t b0 = (hdr[1] >> (8 * j)) & 255u, b1 = (hdr[2] >> (8 * j)) & 255u, b2 = (hdr[3] >> (8 * j)) & 255u;
                const uint32_t sc = dh ? ((b2 & 15u) | ((b0 >> 6) << 4)) : (b0 & 63u);
                const uint32_t mn = dh ? ((b2 >> 4) | ((b1 >> 6) << 4)) : (b1 & 63u);
                v[2 * j] = d * static_cast<float>(sc);
                v[2 * j + 1] = dmin * static_cast<float>(mn);
            }
            float* dst = reinterpret_cast<float*>(scl + buf * kSclBytes + dc * 64 + dh * 32);
            *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f32x4*>(dst + 4) = f32x4{v[4], v[5], v[6], v[7]};
        };
        // One production step makes the LDS tiles of K slice t: J = t % 4 is the 64-wide slice inside the Q4_K block
        // (sub-blocks 2J in the low nibbles and 2J + 1 in the high nibbles of its 32 bytes).
        // The decode inputs of a step are read from LDS one step early (before the barrier that ends the previous
        // step), so that after the barrier the step starts with arithmetic, not with an LDS round trip.
        u32x4 nq;
        f32x4 nsm;
        auto fetch_inputs = [&](int t, int j) {      // for K slice t, j = t % 4
            if (!d_role) return;
            const int buf = (t >> 2) & 1;
            nq = *reinterpret_cast<const u32x4*>(raw + buf * kRawBytes + dc * 144 + 16 + j * 32 + dh * 16);
            nsm = *reinterpret_cast<const f32x4*>(scl + buf * kSclBytes + dc * 64 + j * 16);
        };
        auto step = [&](int t, auto jt) {
            constexpr int J = decltype(jt)::value;
            const int blk = t >> 2;
            if (J == 0) load_raw(blk + 1);
            if (d_role) {
                const u32x4 q = nq;
                const f32x4 sm = nsm;
                uint8_t* wb = ws + (t & 1) * 2 * kWTile + dc * kRowBytes;
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    const uint32_t a0 = q[2 * g], a1 = q[2 * g + 1];
                    const int slot = lds_slot(dc, 2 * dh + g) * 16;
                    *reinterpret_cast<u32x4*>(wb + slot) = q4k_decode8(a0 & 0x0f0f0f0fu, a1 & 0x0f0f0f0fu, sm[0], sm[1]);
                    *reinterpret_cast<u32x4*>(wb + kWTile + slot) =
                        q4k_decode8((a0 >> 4) & 0x0f0f0f0fu, (a1 >> 4) & 0x0f0f0f0fu, sm[2], sm[3]);
                }
            }
            if (x_role) {
                u32x4* set = xset[t & 1];
                uint8_t* xb = xs + (t & 1) * 2 * kXTile;
#pragma unroll
                for (int i = 0; i < kXLoads; ++i) *reinterpret_cast<u32x4*>(xb + xdst[i]) = set[i];
                load_x(set, t + 2);
            }
            // the next block: requested at J = 0, staged at J = 1, its scales made at J = 2, all visible from J = 3 on
            if (J == 1) store_raw((blk + 1) & 1);
            if (J == 2) make_scales((blk + 1) & 1);
            fetch_inputs(t + 1, (J + 1) & 3);
        };
        using std::integral_constant;
        load_raw(0);
        if (x_role) {
            load_x(xset[0], 0);
            load_x(xset[1], 1);
        }
        store_raw(0);
        __syncthreads();
        make_scales(0);
        __syncthreads();
        fetch_inputs(0, 0);
        step(0, integral_constant<int, 0>{});
        __syncthreads();
        // K is a whole number of 256-blocks, so iters is a multiple of 4 and the last step of the last group is skipped
        for (int i = 0; i < iters; i += 4) {
            step(i + 1, integral_constant<int, 1>{});
            __syncthreads();
            step(i + 2, integral_constant<int, 2>{});
            __syncthreads();
            step(i + 3, integral_constant<int, 3>{});
            __syncthreads();
            if (i + 4 < iters) step(i + 4, integral_constant<int, 0>{});
            __syncthreads();
        }
        return;
    }

    // ---------------------------------------------------------------------------------------------- consumers
    // waves w and w + 4 usually share a SIMD: giving them different column halves balances the matrix pipes
    const int wm = wave % WM, wn = wave / WM;
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
        __syncthreads();        // the first raw blocks are staged
        __syncthreads();        // their scales are staged
        __syncthreads();        // the tiles of K slice 0 are ready
        for (int it = 0; it < iters; ++it) {
            const uint8_t* xb = xs + (it & 1) * 2 * kXTile + wm * RW * kRowBytes + frag;
            const uint8_t* wb = ws + (it & 1) * 2 * kWTile + ct0 * 16 * kRowBytes + frag;
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                bf16x8 afrag[MT];
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    afrag[i] = *reinterpret_cast<const bf16x8*>(xb + sub * kXTile + i * 16 * kRowBytes);
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    const bf16x8 bfrag = *reinterpret_cast<const bf16x8*>(wb + sub * kWTile + j * 16 * kRowBytes);
#pragma unroll
                    for (int i = 0; i < MT; ++i)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag[i], bfrag, acc[i][j], 0, 0, 0);
                }
            }
            __syncthreads();
        }
        // accumulator element v of a tile: row 4 * (lane / 16) + v, column lane % 16
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
                        if (m < a.M) a.y[static_cast<size_t>(m) * a.N + n] = acc[i][j][v] + b;
                    }
                }
            }
        }
    };
    constexpr int kLastTiles = CT - (WN - 1) * CTW;     // tiles of the last wave column
    if (kLastTiles == CTW || wn < WN - 1) consume(std::integral_constant<int, CTW>{});
    else consume(std::integral_constant<int, kLastTiles>{});
}

template <int RW, int CT, int WN>
hipError_t launch_gemm(Lane* lane, const GemmArgs& a, dim3 grid)
{
    constexpr int BM = (8 / WN) * RW, BN = 16 * CT;
    constexpr size_t lds = 4 * static_cast<size_t>(BM + BN) * kRowBytes + 2 * static_cast<size_t>(BN) * (144 + 64);
    static bool configured = false;
    if (lds > 48 * 1024 && !configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&matmul_q4k_bf16_kernel<RW, CT, WN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (e != hipSuccess) return e;
        configured = true;
    }
    hipLaunchKernelGGL((matmul_q4k_bf16_kernel<RW, CT, WN>), grid, dim3(kGemmAll), lds, lane->stream, a);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_matmul_bf16(Lane* lane, uint32_t type, const uint16_t* x, const void* w, const float* bias, float* y,
                              int rows, int in_w, int out_w)
{
    if (type != NNHIP_TYPE_Q4_K) return hipErrorNotSupported;
    GemmArgs a{};
    a.x = x;
    a.w = static_cast<const uint8_t*>(w);
    a.bias = bias;
    a.y = y;
    a.M = rows;
    a.K = in_w;
    a.N = out_w;
    // Row tile and strip width: BM = 128 rows for M <= 128, else 256; strips as wide as the column tiles allow, narrowed
    // so that strips x row tiles is a whole number of rounds over the compute units when that keeps them >= 70 % wide.
    const int bm = rows <= 128 ? 128 : 256;
    const int m_tiles = (rows + bm - 1) / bm;
    const int max_cols = (rows <= 256) ? 80 : 144;
    int strips = (out_w + max_cols - 1) / max_cols;
    const int per_round = lane->compute_units;
    const int even = (strips * m_tiles + per_round - 1) / per_round * per_round / m_tiles;
    if (even > strips && (out_w + even - 1) / even * 10 >= max_cols * 7) strips = even;
    a.cols = (out_w + strips - 1) / strips;
    a.strips = (out_w + a.cols - 1) / a.cols;
    const dim3 grid(a.strips, m_tiles);
    if (rows <= 128) return launch_gemm<16, 5, 1>(lane, a, grid);
    if (rows <= 256) return launch_gemm<32, 5, 1>(lane, a, grid);
    return launch_gemm<64, 9, 2>(lane, a, grid);
}

}  // namespace nnhip
