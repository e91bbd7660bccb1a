// Prefill mat-mul for raw GGUF Q4_K weights on gfx950: y[M, N] = bias + x[M, K] (bf16) . W[N, K]^T.
//
// Replaces the XMX prefill launch of the reference (NNtrain.Arc/Kernels/qwen35_prefill_xmx.cl:112-184): weight tiles
// are dequantized to bfloat16 in LDS and contracted on the matrix cores (v_mfma_f32_16x16x32_bf16) with FP32
// accumulators.  The FP32 dequantization formula and rounding order are those of the CPU decoder
// ((d*sc)*q - dmin*m, NNtrain.Core/Serialization/GgufQ4K.cs:34-41); the only rounding added is FP32 -> bf16 of the
// weight, which is what the 2e-3 relative-L2 bar of this path allows for.
//
// Tiling.  A workgroup of 8 waves owns BM = 8 * RW rows (RW = 16, 32 or 64 rows per wave) and a strip of up to 80
// output columns for the whole K range; the strip width is chosen on the host so that the strips split N evenly over
// the compute units (17408 columns -> 256 strips of 68).  Every wave spans the whole strip, so a weight sub-block
// is dequantized once per workgroup.  K advances in steps of 32 = one Q4_K sub-block per weight row:
//   - x tile  [BM][32] bf16 and weight tile [80][32] bf16 live in LDS, double buffered (rows are 64 bytes, so the 16
//     rows x 4 k-groups an MFMA operand needs form one contiguous, conflict-free 1 KiB read);
//   - while the MFMAs of step i run, the x tile of step i+1 travels global -> registers -> LDS and threads
//     0 .. 4*cols-1 each decode 8 weights of step i+1 (one 8-byte load of nibbles plus the block header);
//   - one barrier per step.
#include "nnhip_internal.h"
#include "quant_device.h"

namespace nnhip {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kGemmThreads = 512;
constexpr int kMaxCols = 80;            // five 16-column MFMA tiles
constexpr int kRowBytes = 64;           // one tile row: 32 bf16

struct GemmArgs {
    const uint16_t* x;     // bf16 [M, K]
    const uint8_t* w;      // Q4_K [N, K/256 * 144]
    const float* bias;
    float* y;
    int M, K, N;
    int cols;              // strip width actually used, <= 80
    int strips;            // ceil(N / cols)
};

__device__ __forceinline__ uint32_t pack_bf16(float a, float b)
{
    // round to nearest even, two at a time (v_cvt_pk_bf16_f32)
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 v = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
    return __builtin_bit_cast(uint32_t, v);
}

template <int RW>
__global__ __launch_bounds__(kGemmThreads) void matmul_q4k_bf16_kernel(GemmArgs a)
{
    constexpr int BM = 8 * RW;
    constexpr int MT = RW / 16;                     // 16-row MFMA tiles per wave
    constexpr int kXLoads = BM * kRowBytes / 16 / kGemmThreads;   // 16-byte pieces of the x tile per thread
    static_assert(kXLoads >= 1, "tile too small for the thread count");
    __shared__ __attribute__((aligned(16))) uint8_t xs[2][BM * kRowBytes];
    __shared__ __attribute__((aligned(16))) uint8_t ws[2][kMaxCols * kRowBytes];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int strip = blockIdx.x, m0 = blockIdx.y * BM;
    const int n0 = strip * a.cols;
    const int row_bytes = (a.K >> 8) * 144;

    // x tile piece p of this thread: row p / 4 of the tile, 16-byte group p % 4
    const uint16_t* xsrc[kXLoads];
    int xdst[kXLoads];
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) {
        const int p = tid + i * kGemmThreads;
        const int r = min(m0 + (p >> 2), a.M - 1);
        xsrc[i] = a.x + static_cast<size_t>(r) * a.K + (p & 3) * 8;
        xdst[i] = p * 16;
    }
    // weight item of this thread: column tid / 4 of the strip, quarter tid % 4 of the sub-block
    const bool decoder = tid < 4 * kMaxCols;
    const int wn = tid >> 2, wq = tid & 3;
    const uint8_t* wrow = a.w + static_cast<size_t>(min(n0 + wn, a.N - 1)) * row_bytes;

    u32x4 xreg[kXLoads];
    u32x4 hdr{};
    u32x2 qs{};
    auto load_step = [&](int k0) {
#pragma unroll
        for (int i = 0; i < kXLoads; ++i) xreg[i] = *reinterpret_cast<const u32x4*>(xsrc[i] + k0);
        if (decoder) {
            const uint8_t* blk = wrow + (k0 >> 8) * 144;
            const int g = (k0 >> 5) & 7;
            hdr = *reinterpret_cast<const u32x4*>(blk);
            qs = *reinterpret_cast<const u32x2*>(blk + 16 + (g >> 1) * 32 + wq * 8);
        }
    };
    auto store_step = [&](int k0, int buf) {
#pragma unroll
        for (int i = 0; i < kXLoads; ++i) *reinterpret_cast<u32x4*>(&xs[buf][xdst[i]]) = xreg[i];
        if (decoder) {
            const int g = (k0 >> 5) & 7;
            const float d = half_bits_to_float(hdr[0]), dmin = half_bits_to_float(hdr[0] >> 16);
            // 6-bit scale and min of sub-block g from the 12 packed bytes (GgufQ4K.cs:51-60)
            const uint32_t s0 = hdr[1], s1 = hdr[2], s2 = hdr[3];
            const int sh = (g & 3) * 8;
            uint32_t sc, mn;
            if (g < 4) {
                sc = (s0 >> sh) & 63u;
                mn = (s1 >> sh) & 63u;
            } else {
                sc = ((s2 >> sh) & 15u) | (((s0 >> sh) >> 6 & 3u) << 4);
                mn = ((s2 >> sh) >> 4 & 15u) | (((s1 >> sh) >> 6 & 3u) << 4);
            }
            const float scale = d * static_cast<float>(sc);
            const float mnv = dmin * static_cast<float>(mn);
            const int nib = (g & 1) * 4;
            uint32_t out[4];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t q4 = (qs[h] >> nib) & 0x0f0f0f0fu;
                const float w0 = __fsub_rn(__fmul_rn(scale, ubyte0(q4)), mnv), w1 = __fsub_rn(__fmul_rn(scale, ubyte1(q4)), mnv);
                const float w2 = __fsub_rn(__fmul_rn(scale, ubyte2(q4)), mnv), w3 = __fsub_rn(__fmul_rn(scale, ubyte3(q4)), mnv);
                out[2 * h] = pack_bf16(w0, w1);
                out[2 * h + 1] = pack_bf16(w2, w3);
            }
            const u32x4 v = {out[0], out[1], out[2], out[3]};
            *reinterpret_cast<u32x4*>(&ws[buf][wn * kRowBytes + wq * 16]) = v;
        }
    };

    f32x4 acc[MT][5];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 5; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    load_step(0);
    store_step(0, 0);
    __syncthreads();

    // operand address of this lane inside a 16-row tile: row lane % 16, k-group lane / 16
    const int frag = (lane & 15) * kRowBytes + (lane >> 4) * 16;
    int buf = 0;
    for (int k0 = 0; k0 < a.K; k0 += 32) {
        const bool more = k0 + 32 < a.K;
        if (more) load_step(k0 + 32);
        bf16x8 bfrag[5];
#pragma unroll
        for (int j = 0; j < 5; ++j) bfrag[j] = *reinterpret_cast<const bf16x8*>(&ws[buf][j * 16 * kRowBytes + frag]);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const bf16x8 afrag = *reinterpret_cast<const bf16x8*>(&xs[buf][(wave * RW + i * 16) * kRowBytes + frag]);
#pragma unroll
            for (int j = 0; j < 5; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afrag, bfrag[j], acc[i][j], 0, 0, 0);
        }
        if (more) store_step(k0 + 32, buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    // accumulator element v of a tile: row 4 * (lane / 16) + v, column lane % 16
#pragma unroll
    for (int j = 0; j < 5; ++j) {
        const int cn = j * 16 + (lane & 15);
        const int n = n0 + cn;
        if (cn < a.cols && n < a.N) {
            const float b = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int m = m0 + wave * RW + i * 16 + (lane >> 4) * 4 + v;
                    if (m < a.M) a.y[static_cast<size_t>(m) * a.N + n] = acc[i][j][v] + b;
                }
            }
        }
    }
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
    // strip width: as close to 80 columns as an even split of N over the compute units allows
    int strips = (out_w + kMaxCols - 1) / kMaxCols;
    const int even = (strips + lane->compute_units - 1) / lane->compute_units * lane->compute_units;
    if ((out_w + even - 1) / even >= 56) strips = even;
    a.cols = (out_w + strips - 1) / strips;
    a.strips = (out_w + a.cols - 1) / a.cols;
    if (rows <= 128) {
        hipLaunchKernelGGL(matmul_q4k_bf16_kernel<16>, dim3(a.strips, (rows + 127) / 128), dim3(kGemmThreads), 0, lane->stream, a);
    } else if (rows <= 256) {
        hipLaunchKernelGGL(matmul_q4k_bf16_kernel<32>, dim3(a.strips, (rows + 255) / 256), dim3(kGemmThreads), 0, lane->stream, a);
    } else {
        hipLaunchKernelGGL(matmul_q4k_bf16_kernel<64>, dim3(a.strips, (rows + 511) / 512), dim3(kGemmThreads), 0, lane->stream, a);
    }
    return hipGetLastError();
}

}  // namespace nnhip
