// One decode mat-vec per launch on the matrix cores, started fast: the kernel behind nnhip_quant_matvec (one input row)
// and nnhip_quant_matvec_fused for the shapes it takes.  Same tasks and the same data movement as the batched kernels
// of gemv_mfma_kernels.hip (coalesced non-temporal pieces into two register sets, two LDS stage buffers, digit planes of
// the activations in LDS, v_mfma_i32_16x16x32_i8), with three differences that make a lone launch cheap:
//
//   * the descriptor travels in the kernel arguments, the activations are requested first and the first two weight
//     stages right behind them, before anything else is computed;
//   * block fixed point: every 32 activations get an exponent of their own (v = rint(x * 2^e), |v| < 2^30, e from the
//     largest magnitude of the 32), so turning a vector into digit planes needs no maximum over the whole vector - no
//     workgroup reduction - and one huge activation costs the others no precision: the error per element is at most
//     2^-31 of the largest magnitude among its 32 neighbours;
//   * work is dealt in units of 16, 8 or 4 matrix rows (rows past the unit's end are not fetched), chosen on the host so
//     that the units split evenly over the workgroups.
//
// The activation preparation of the fused entry (RMSNorm with optional residual add, SiLU(x) * x2) is done by every
// workgroup on the vector it has just loaded, with the operation order of the row-operation kernels
// (rowop_kernels.hip; NNtrain.Arc/Kernels/qwen35_attention.cl:16-78), so fused and unfused launches agree bit for bit;
// the epilogue (bias, low-rank branch, addend) is that of the row-step kernel (gemv_kernels.hip).
//
// Summation order of a matrix row: block column b of the row belongs to wave b % 8; a wave adds its columns in
// increasing b (fused multiply-adds per 32-weight sub-block); the four 64-weight quarters of a column are lanes of one
// wave and meet as (q0 + q1) + (q2 + q3); the eight wave sums are added in wave order, then the bias.  It depends on
// the storage type and in_w only.
#include <cstdlib>

#include "gemv_mfma_tasks.h"

namespace nnhip {

namespace {

constexpr int kStreamWaves = 8;
constexpr int kStreamThreads = 64 * kStreamWaves;
constexpr int kXRegsWide = 11;            // float4 per lane that hold a vector on its way in: in_w <= 22528,
constexpr int kXRegsNarrow = 4;           // or in_w <= 8192 (fewer registers: wider stages fit)
constexpr int kNormRegs = 4;              // the same for vectors that are normalized: in_w <= 8192
constexpr int kStreamLds = 160 * 1024;
constexpr int kSyncSlots = 16;            // arrival counters per step of a chain (256 arrivals at one address take 4 us, at 16 addresses 2)
constexpr int kSyncStride = 32;           // words between them: a 128-byte line each

enum : int { kPreNone = 0, kPreRmsNorm = 1, kPreSiluMultiply = 2 };

// One mat-vec of a launch.
struct StreamEntry {
    const float* x;
    const float* x2;          // RMSNorm: residual added first (or null); SiLU: the second factor
    const float* gamma;       // RMSNorm weight
    float* x_out;             // where the prepared vector is stored (or null)
    float* sum_out;           // RMSNorm: where x + x2 is stored (or null)
    const uint8_t* w;
    const float* bias;
    const float* addend;
    float* y;
    const float* lora_z;
    const float* lora_b;
    int lora_rank;
    float lora_scale;
    float epsilon;
    int pre_op;
    int in_w;
    int out_w;
    uint32_t w_bytes;
    uint32_t row_bytes;
    int nblocks;              // 256-weight block columns of a row
    int kchunks;              // stages per unit = ceil(nblocks / cols)
    int tail_cols;            // block columns of a unit's last stage
    int unit_rows;            // matrix rows per unit of work: 16, 8 or 4
    int units;                // ceil(out_w / unit_rows)
    int first_unit;           // position of the matrix' first unit in the launch's unit sequence
    // chained launches only
    int x_head_width;         // > 0: x is gathered by heads, x[h * width + j] = source[(h / x_head_group) * width + j]
    int x_head_group;
    int wait;                 // 1: the entry's vectors are results of the entry before it in the table
    int signals;              // workgroups that own units of this entry: min(units, workgroups)
    int pair_rows;            // > 0: rows o and pair_rows + o of the matrix are multiplied together and y[o] = SiLU(z[o]) * z[pair_rows + o]:
                              // a unit is unit_rows of the first half (stage rows 0 ..) and the matching rows of the second (stage rows 8 ..)
};

struct StreamArgs {
    const StreamEntry* table;     // device table, or null: the entry below
    int entries;
    int total_units;
    int cols;                     // block columns per stage, 8 M
    int row_pieces;               // LDS row stride of a stage in 16-byte pieces (odd)
    uint32_t row_pieces_magic;    // ceil(2^32 / row_pieces)
    int stage_bytes;              // one stage buffer: 16 rows
    int plane_cap;                // bytes between the digit planes: the longest in_w of the launch + 16
    int sums_bytes;               // room for the FP32 sums of x (0 for formats without minima)
    uint32_t* sync;               // chained launches: kSyncSlots arrival counters per entry, then the exit counter and the status word (a line each)
    int spin_limit;               // polls of a counter before a workgroup gives up waiting (and records it in the status word)
    StreamEntry one;
};

// Accesses to vectors that another workgroup of the same launch wrote or will read: relaxed atomics at device scope,
// i.e. loads and stores that bypass the caches that are not shared by all compute units.  No cache-wide write-back or
// invalidate is needed around them (those cost microseconds per workgroup).
__device__ __forceinline__ float4 load4_device(const float4* p)
{
    unsigned long long* q = reinterpret_cast<unsigned long long*>(const_cast<float4*>(p));
    const unsigned long long lo = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long hi = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float4(__uint_as_float(static_cast<uint32_t>(lo)), __uint_as_float(static_cast<uint32_t>(lo >> 32)),
                       __uint_as_float(static_cast<uint32_t>(hi)), __uint_as_float(static_cast<uint32_t>(hi >> 32)));
}
__device__ __forceinline__ void store4_device(float4* p, const float4 v)
{
    unsigned long long* q = reinterpret_cast<unsigned long long*>(p);
    __hip_atomic_store(q, static_cast<unsigned long long>(__float_as_uint(v.x)) | (static_cast<unsigned long long>(__float_as_uint(v.y)) << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(q + 1, static_cast<unsigned long long>(__float_as_uint(v.z)) | (static_cast<unsigned long long>(__float_as_uint(v.w)) << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load1_device(const float* p)
{
    return __hip_atomic_load(const_cast<float*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store1_device(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

#if defined(NNHIP_STREAM_TRACE)
// Development builds only: time stamps (100 MHz) of every workgroup's progress through its last launch.
__device__ unsigned long long g_stream_trace[256 * 32];
#define NNHIP_TRACE(k) do { if (tid == 0 && bid < 256 && (k) < 32) g_stream_trace[bid * 32 + (k)] = wall_clock64(); } while (0)
#else
#define NNHIP_TRACE(k) do { } while (0)
#endif

// CHAIN: the entries of the table are steps of a dependency chain (see the end of the kernel).
template <class F, int M, int LPW, int XR, bool CHAIN = false>
__global__ __launch_bounds__(kStreamThreads) void matvec_mfma_stream_kernel(StreamArgs a)
{
    constexpr int W = kStreamWaves;
    constexpr int kXRegs = XR;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    __shared__ float part[2][W][kTileRows];
    __shared__ float tree[64];
    __shared__ float norm_sum;
    __shared__ __attribute__((aligned(16))) uint8_t zero_area[256];       // operand A outside the block diagonal
    __shared__ __attribute__((aligned(16))) uint8_t table_area[F::kLdsTableBytes > 0 ? F::kLdsTableBytes : 16];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row_l = lane & 15, quarter = lane >> 4;
    const int G = gridDim.x, bid = blockIdx.x;
    NNHIP_TRACE(0);

    const NNHIP_CONST_PTR StreamEntry* table =
        a.table ? (const NNHIP_CONST_PTR StreamEntry*)a.table
                : (const NNHIP_CONST_PTR StreamEntry*)((const NNHIP_CONST_PTR char*)__builtin_amdgcn_kernarg_segment_ptr() +
                                                       offsetof(StreamArgs, one));

    // ---- the activations of entry m on their way in (requested before anything else of that entry)
    constexpr bool kCanNormalize = CHAIN || XR <= kNormRegs;       // (vectors that are normalized are short: the wide variant leaves the code out)
    float4 xa[kXRegs], xb[kXRegs], ga[kCanNormalize ? kNormRegs : 1];
    auto request_x = [&](int m) __attribute__((always_inline)) {
        const NNHIP_CONST_PTR StreamEntry& e = table[m];
        const int n4 = e.in_w >> 2, pre = e.pre_op;
        const float4* x4 = reinterpret_cast<const float4*>(e.x);
        const float4* s4 = reinterpret_cast<const float4*>(e.x2);
        const float4* g4 = reinterpret_cast<const float4*>(e.gamma);
        const int head4 = CHAIN ? e.x_head_width >> 2 : 0, group = CHAIN ? e.x_head_group : 1;
#pragma unroll
        for (int j = 0; j < kXRegs; ++j) {
            int i = tid + j * kStreamThreads;
            if (CHAIN) {
                // (device-scope loads go to memory every time: whole waves past the end skip theirs; n4 % 64 == 0)
                if (i < n4) {
                    if (head4 > 0) {
                        const int h = i / head4;
                        i = (h / group) * head4 + (i - h * head4);
                    }
                    xa[j] = load4_device(x4 + i);
                }
            } else {
                xa[j] = x4[i < n4 ? i : 0];      // (unconditional: no branch between the requests; pieces past the end are not used)
            }
        }
        if (pre != kPreNone && s4) {
#pragma unroll
            for (int j = 0; j < kXRegs; ++j) {
                const int i = tid + j * kStreamThreads;
                if (CHAIN) {
                    if (i < n4) xb[j] = load4_device(s4 + i);
                } else {
                    xb[j] = s4[i < n4 ? i : 0];
                }
            }
        }
        if (kCanNormalize && pre == kPreRmsNorm) {
#pragma unroll
            for (int j = 0; j < (kCanNormalize ? kNormRegs : 0); ++j) {
                const int i = tid + j * kStreamThreads;
                ga[j] = g4[i < n4 ? i : 0];
            }
        }
    };
    // the entry that holds this workgroup's first unit (entries are few: a walk over the table)
    int c_m = 0;
    while (c_m + 1 < a.entries && bid >= table[c_m].first_unit + table[c_m].units) ++c_m;
    const bool early_x = !CHAIN || c_m == 0;          // (a later step's vector does not exist yet)
    if (early_x) request_x(c_m);

    // ---- this lane's pieces of a stage: piece I = wave + W * i is slots 64 I .. 64 I + 63; slot s is 16-byte piece
    // s % row_pieces of stage row s / row_pieces: piece q % kPieces of block column q / kPieces.
    int p_row[LPW];
    uint32_t p_col[LPW];                   // byte offset inside the row's stage span, or "no piece"
    uint32_t p_c[LPW];
    uint32_t in_stage = 0;
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const uint32_t slot = static_cast<uint32_t>(64 * (wave + W * i) + lane);
        const uint32_t r = __umulhi(slot, a.row_pieces_magic);
        const uint32_t q = slot - r * static_cast<uint32_t>(a.row_pieces);
        const uint32_t c = q / static_cast<uint32_t>(F::kPieces);
        const bool real = r < static_cast<uint32_t>(kTileRows) && c < static_cast<uint32_t>(a.cols);
        p_row[i] = static_cast<int>(r);
        p_c[i] = c;
        p_col[i] = real ? c * F::kBlockBytes + F::piece_src(q - c * F::kPieces, c & 1u) : kNoPiece;
        in_stage |= (r < static_cast<uint32_t>(kTileRows) ? 1u : 0u) << i;
    }
    const uint32_t chunk_bytes = static_cast<uint32_t>(a.cols) * F::kBlockBytes;

    // ---- prefetch side: units bid, bid + G, ... of the launch's unit sequence, kchunks stages each
    int f_u = bid, f_k = 0, f_m = -1;
    int fe_first = 0, fe_units = 0, fe_kchunks = 1, fe_unit_rows = kTileRows, fe_pair_rows = 0;
    uint32_t fe_row_bytes = 0;
    uint32_t rel[LPW];
    uint32_t in_tail = 0;
    __amdgpu_buffer_rsrc_t f_matrix;
    auto fetch_enter = [&]() __attribute__((always_inline)) {
        while (f_m < 0 || (f_u >= fe_first + fe_units && f_m + 1 < a.entries)) {
            const NNHIP_CONST_PTR StreamEntry& e = table[++f_m];
            fe_first = e.first_unit;
            fe_units = e.units;
        }
        const NNHIP_CONST_PTR StreamEntry& e = table[f_m];
        fe_kchunks = e.kchunks;
        fe_unit_rows = e.unit_rows;
        fe_row_bytes = e.row_bytes;
        fe_pair_rows = CHAIN ? e.pair_rows : 0;
        const int tail_cols = e.tail_cols;
        f_matrix = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(e.w), 0, static_cast<int>(e.w_bytes), 0x00020000);
        in_tail = 0;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            // the matrix row of stage row r, counted from the unit's first row: r, or with paired halves r (r < 8) and
            // pair_rows + r - 8
            const int half_row = p_row[i] & 7;
            const bool ok = (fe_pair_rows > 0 ? half_row < fe_unit_rows : p_row[i] < fe_unit_rows) && p_col[i] != kNoPiece;
            const uint32_t row = fe_pair_rows > 0 && p_row[i] >= 8 ? static_cast<uint32_t>(fe_pair_rows + half_row) : static_cast<uint32_t>(p_row[i]);
            rel[i] = ok ? row * fe_row_bytes + p_col[i] : kNoPiece;
            in_tail |= (ok && p_c[i] < static_cast<uint32_t>(tail_cols) ? 1u : 0u) << i;
        }
    };
    auto fetch = [&](u32x4 (&set)[LPW]) __attribute__((always_inline)) {
        const uint32_t base = f_u < a.total_units
            ? static_cast<uint32_t>(f_u - fe_first) * static_cast<uint32_t>(fe_unit_rows) * fe_row_bytes + static_cast<uint32_t>(f_k) * chunk_bytes
            : kNoPiece;
        const bool tail = f_k == fe_kchunks - 1;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            const bool none = rel[i] == kNoPiece || (tail && !((in_tail >> i) & 1u));
            set[i] = stream16(f_matrix, none ? kNoPiece : base + rel[i]);
        }
        if (++f_k == fe_kchunks) {
            f_k = 0;
            f_u += G;
            if (f_u < a.total_units && f_u >= fe_first + fe_units) fetch_enter();
        }
    };
    auto park = [&](uint8_t* buf, const u32x4 (&set)[LPW]) __attribute__((always_inline)) {
        uint8_t* dst = buf + wave * 1024 + lane * 16;
#pragma unroll
        for (int i = 0; i < LPW; ++i)
            if ((in_stage >> i) & 1u) *reinterpret_cast<u32x4*>(dst + W * i * 1024) = set[i];
    };

    // the first two stages are on their way before the activations are looked at
    u32x4 regs[2][LPW];
    fetch_enter();
    fetch(regs[0]);
    fetch(regs[1]);
    NNHIP_TRACE(1);

    uint8_t* const tables = table_area;
    uint8_t* const buf0 = smem;
    uint8_t* const buf1 = smem + a.stage_bytes;
    uint8_t* const planes = smem + 2 * a.stage_bytes;
    float* const sums = reinterpret_cast<float*>(planes + 4 * a.plane_cap);
    float* const exps = reinterpret_cast<float*>(planes + 4 * a.plane_cap + a.sums_bytes);
    F::init_tables(tables, tid, kStreamThreads);
    if (tid < 64) reinterpret_cast<uint32_t*>(zero_area)[tid] = 0u;
    const bool diag = (row_l >> 2) == quarter;
    const uint8_t* const a_zeros = diag ? nullptr : zero_area;

    // ---- float4 number i of the prepared vector -> digit planes, sums and the exponent of its 32-activation group
    // (eight consecutive lanes hold a group: i is a multiple of 8 in the first of them)
    auto to_planes = [&](int i, const float4& v) __attribute__((always_inline)) {
        uint32_t mx = umax_u(umax_u(__float_as_uint(v.x) & 0x7fffffffu, __float_as_uint(v.y) & 0x7fffffffu),
                             umax_u(__float_as_uint(v.z) & 0x7fffffffu, __float_as_uint(v.w) & 0x7fffffffu));
        mx = umax_u(mx, dpp_mov_u<0xB1>(mx));
        mx = umax_u(mx, dpp_mov_u<0x4E>(mx));
        mx = umax_u(mx, dpp_mov_u<0x141>(mx));
        // |x| < 2^(E - 126) for the biased exponent E of the largest magnitude; e = 156 - E puts it below 2^30
        const int E = static_cast<int>(mx >> 23);
        int e = 156 - E;
        e = e > 126 ? 126 : e;
        const float scale = __uint_as_float(static_cast<uint32_t>(e + 127) << 23);
        // a NaN or an infinity among the 32 makes every output NaN
        const float ie = E == 255 ? __uint_as_float(0x7fc00000u) : __uint_as_float(static_cast<uint32_t>(127 - e) << 23);
        uint32_t pl[4];
        digit_planes(__float2int_rn(v.x * scale), __float2int_rn(v.y * scale), __float2int_rn(v.z * scale),
                     __float2int_rn(v.w * scale), pl);
#pragma unroll
        for (int p = 0; p < 4; ++p) *reinterpret_cast<uint32_t*>(planes + p * a.plane_cap + 4 * i) = pl[p];
        if ((i & 7) == 0) exps[i >> 3] = ie;
        if (F::kNeedsSums) {
            float s = (v.x + v.y) + (v.z + v.w);
            if (F::kSumRun == 32) {
                s = oct_sum(s);
                if ((i & 7) == 0) sums[i >> 3] = s;
            } else {
                s += dpp_mov<0xB1>(s);
                s += dpp_mov<0x4E>(s);
                if ((i & 3) == 0) sums[i >> 2] = s;
            }
        }
    };

    // ---- the vector in xa (xb, ga) becomes digit planes in LDS; ends with a barrier
    auto convert_x = [&](int m) __attribute__((always_inline)) {
        const NNHIP_CONST_PTR StreamEntry& e = table[m];
        const int n4 = e.in_w >> 2, pre = e.pre_op;
        // the workgroup that stores the prepared vector: the owner of the entry's first unit
        const bool scribe = CHAIN ? bid == e.first_unit % G : bid == 0;
        auto store4 = [&](float4* p, const float4& v) __attribute__((always_inline)) {
            if (CHAIN) store4_device(p, v);
            else *p = v;
        };
        if (pre == kPreSiluMultiply) {
            float4* xo = scribe ? reinterpret_cast<float4*>(e.x_out) : nullptr;
#pragma unroll
            for (int j = 0; j < kXRegs; ++j) {
                const int i = tid + j * kStreamThreads;          // (whole groups of eight lanes are in or out: n4 % 64 == 0)
                if (i < n4) {
                    const float4 v = silu_mul4(xa[j], xb[j]);
                    if (xo) store4(xo + i, v);
                    to_planes(i, v);
                }
                __builtin_amdgcn_sched_barrier(0);       // (one piece at a time: hoisting all the exponentials together spills)
            }
        } else if (kCanNormalize && pre == kPreRmsNorm) {
            float4* so = scribe ? reinterpret_cast<float4*>(e.sum_out) : nullptr;
            float4* xo = scribe ? reinterpret_cast<float4*>(e.x_out) : nullptr;
            const bool second = e.x2 != nullptr;
            float* stage32 = reinterpret_cast<float*>(planes);          // the summed vector as FP32, until it is normalized
#pragma unroll
            for (int j = 0; j < (kCanNormalize ? kNormRegs : 0); ++j) {
                const int i = tid + j * kStreamThreads;
                if (i < n4) {
                    if (second) xa[j] = add4(xa[j], xb[j]);          // (without a residual the input keeps its bits: -0 stays -0)
                    reinterpret_cast<float4*>(stage32)[i] = xa[j];
                    if (so) store4(so + i, xa[j]);
                }
            }
            __syncthreads();
            // 128 lane-strided partial sums of squares, then the halving tree: 64 through LDS, 32 .. 1 inside wave 0
            float sq = 0.0f;
            if (tid < 128) {
                // (eight reads on their way at a time; the additions keep their order)
                int j = tid;
                for (; j + 7 * 128 < e.in_w; j += 8 * 128) {
                    float v[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) v[u] = stage32[j + u * 128];
#pragma unroll
                    for (int u = 0; u < 8; ++u) sq += v[u] * v[u];
                }
                for (; j < e.in_w; j += 128) {
                    const float v = stage32[j];
                    sq += v * v;
                }
            }
            if (tid >= 64 && tid < 128) tree[tid - 64] = sq;
            __syncthreads();
            if (tid < 64) {
                sq += tree[tid];
                const uint32_t u = __float_as_uint(sq);
                auto s32 = __builtin_amdgcn_permlane32_swap(u, u, false, false);
                sq = __uint_as_float(s32[0]) + __uint_as_float(s32[1]);
                const uint32_t v = __float_as_uint(sq);
                auto s16 = __builtin_amdgcn_permlane16_swap(v, v, false, false);
                sq = __uint_as_float(s16[0]) + __uint_as_float(s16[1]);
                sq += dpp_mov<0x108>(sq);
                sq += dpp_mov<0x104>(sq);
                sq += dpp_mov<0x102>(sq);
                sq += dpp_mov<0x101>(sq);
                if (tid == 0) norm_sum = sq;
            }
            __syncthreads();
            const float inverse = 1.0f / sqrtf(norm_sum / static_cast<float>(e.in_w) + e.epsilon);
#pragma unroll
            for (int j = 0; j < (kCanNormalize ? kNormRegs : 0); ++j) {
                const int i = tid + j * kStreamThreads;
                if (i < n4) {
                    const float4 h = xa[j], g = ga[j];
                    const float4 v = make_float4(h.x * inverse * g.x, h.y * inverse * g.y, h.z * inverse * g.z, h.w * inverse * g.w);
                    if (xo) store4(xo + i, v);
                    to_planes(i, v);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < kXRegs; ++j) {
                const int i = tid + j * kStreamThreads;
                if (i < n4) to_planes(i, xa[j]);
            }
        }
        __syncthreads();
    };

    // ---- consume side
    int c_u = bid, c_k = 0;
    int ce_first = 0, ce_units = 0, ce_kchunks = 1, ce_nblocks = 0;
    const uint32_t row_off = static_cast<uint32_t>(row_l) * (static_cast<uint32_t>(a.row_pieces) * 16u) +
                             static_cast<uint32_t>(wave) * (16u * F::kPieces);
    int pbuf = 0;
    bool done = false;
    int done_unit = 0;
    // Adds up and stores the unit whose wave partials sit in part[pbuf ^ 1] (a unit of entry c_m).
    auto finalize = [&]() __attribute__((always_inline)) {
        if (tid < kTileRows) {
            const NNHIP_CONST_PTR StreamEntry& e = table[c_m];
            const int ur = e.unit_rows, pair = CHAIN ? e.pair_rows : 0;
            const int out_w = pair > 0 ? pair : e.out_w;
            const int row0 = (done_unit - e.first_unit) * ur;
            int rows = out_w - row0;
            rows = rows < ur ? rows : ur;
            float t = 0.0f;
#pragma unroll
            for (int w2 = 0; w2 < W; ++w2) t += part[pbuf ^ 1][w2][tid];
            if (CHAIN && pair > 0) {
                // lanes 0-7 hold rows of the first half, lanes 8-15 the matching rows of the second
                const int row = (tid < 8 ? 0 : pair) + row0 + (tid & 7);
                if ((tid & 7) < rows && e.bias) t += e.bias[row];
                const float other = dpp_mov<0x128>(t);                  // row_ror:8: lane j receives lane j + 8 (mod 16)
                if (tid < 8 && tid < rows) store1_device(e.y + row0 + tid, silu_mul1(t, other));
            } else if (tid < rows) {
                const int row = row0 + tid;
                if (e.bias) t += e.bias[row];
                if (e.lora_rank > 0) {      // the branch of q35l_*_sg16_lora (NNtrain.Arc/Kernels/qwen35_linear_fast.cl:262-268)
                    const float* br = e.lora_b + static_cast<size_t>(row) * e.lora_rank;
                    float sum = 0.0f;
                    for (int r = 0; r < e.lora_rank; ++r) sum = fmaf(e.lora_z[r], br[r], sum);
                    t = t + e.lora_scale * sum;
                }
                if (CHAIN) store1_device(e.y + row, e.addend ? load1_device(e.addend + row) + t : t);
                else e.y[row] = e.addend ? e.addend[row] + t : t;
            }
        }
        done = false;
    };

    float accq = 0.0f, accm = 0.0f;
    auto compute = [&](const uint8_t* cur) __attribute__((always_inline)) {
        auto task = [&](const typename F::Raw& raw, int b) __attribute__((always_inline)) {
            typename F::X xs;
            F::load_x(xs, planes + (row_l & 3) * a.plane_cap, sums, b, quarter, a_zeros, exps);
            F::template run<true>(raw, xs, quarter, tables, accq, accm);
        };
        const int b0 = c_k * a.cols + wave;
        const uint8_t* stage = cur + row_off;
        if (b0 + (M - 1) * W < ce_nblocks) {
            typename F::Raw raw[M];
#pragma unroll
            for (int t = 0; t < M; ++t) raw[t] = F::load(stage + t * W * (16 * F::kPieces), quarter, (wave & 1) != 0);
#pragma unroll
            for (int t = 0; t < M; ++t) task(raw[t], b0 + t * W);
        } else {
#pragma unroll
            for (int t = 0; t < M - 1; ++t)
                if (b0 + t * W < ce_nblocks) task(F::load(stage + t * W * (16 * F::kPieces), quarter, (wave & 1) != 0), b0 + t * W);
        }
        if (++c_k == ce_kchunks) {
            c_k = 0;
            float p = accq - accm;
            p = quarter_sum(p);
            if (lane < kTileRows) part[pbuf][wave][lane] = p;
            accq = 0.0f;
            accm = 0.0f;
            done = true;
            done_unit = c_u;
            pbuf ^= 1;
            c_u += G;
        }
    };

    // This workgroup's units, entry by entry.  Within an entry its stages run in pairs (a turn of the two register sets
    // and stage buffers); an entry with an odd number of them leaves the next one a single step to begin with.
    auto stage_step = [&](uint8_t* cur, uint8_t* nxt, u32x4 (&refill)[LPW], const u32x4 (&landing)[LPW]) __attribute__((always_inline)) {
        fetch(refill);
        if (done) finalize();
        compute(cur);
        park(nxt, landing);
        __syncthreads();
    };
    bool first = true;
    int parity = 0;                    // 0: the next stage is in buf0 (and regs[0] is free), 1: in buf1
    while (c_u < a.total_units) {
        {
            const NNHIP_CONST_PTR StreamEntry& e = table[c_m];
            ce_first = e.first_unit;
            ce_units = e.units;
            ce_kchunks = e.kchunks;
            ce_nblocks = e.nblocks;
        }
        // (every wave has left the stage that last read the planes)
        if (CHAIN) NNHIP_TRACE(8 + 4 * c_m);
        if (CHAIN && c_m > 0 && table[c_m].wait) {
            // Every unit of the step before this one must have been stored: its owners count themselves in when they are
            // through with it.  The wait is bounded: a workgroup that gives up says so in the status word and goes on
            // (with whatever the vectors hold), so the launch always ends.
            if (tid < kSyncSlots) {
                // slot s counts the owners whose rank (workgroups from the owner of the step's first unit on) % 16 == s
                const int signals = table[c_m - 1].signals;
                const uint32_t target = static_cast<uint32_t>((signals - tid + kSyncSlots - 1) / kSyncSlots);
                const uint32_t* slot = a.sync + ((c_m - 1) * kSyncSlots + tid) * kSyncStride;
                int polls = 0;
                while (__hip_atomic_load(const_cast<uint32_t*>(slot), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                    if (++polls > a.spin_limit) {
                        __hip_atomic_store(a.sync + (a.entries * kSyncSlots + 1) * kSyncStride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        break;
                    }
                }
            }
            __syncthreads();
        }
        if (CHAIN) NNHIP_TRACE(8 + 4 * c_m + 1);
        if (!first || !early_x) request_x(c_m);
        convert_x(c_m);
        if (CHAIN) NNHIP_TRACE(8 + 4 * c_m + 2);
        if (first) {
            NNHIP_TRACE(2);
            park(buf0, regs[0]);
            __syncthreads();
            NNHIP_TRACE(3);
            first = false;
        }
        int left = ((ce_first + ce_units - 1 - c_u) / G + 1) * ce_kchunks;
        if (parity) {
            stage_step(buf1, buf0, regs[1], regs[0]);
            --left;
            parity = 0;
        }
        for (; left >= 2; left -= 2) {
            stage_step(buf0, buf1, regs[0], regs[1]);
            stage_step(buf1, buf0, regs[1], regs[0]);
        }
        if (left) {
            stage_step(buf0, buf1, regs[0], regs[1]);
            parity = 1;
        }
        NNHIP_TRACE(5);
        if (done) finalize();          // (while c_m is still the unit's entry)
        if (CHAIN) {
            // this workgroup's units of the step are stored (the stores are write-through; the wait below covers them):
            // count it in
            __builtin_amdgcn_s_waitcnt(0x0F70);             // vmcnt(0): every wave's stores (results, prepared vectors) have arrived
            __atomic_signal_fence(__ATOMIC_SEQ_CST);
            __syncthreads();
            if (tid == 0) {
                const int rank = (bid - ce_first % G + G) % G;
                __hip_atomic_fetch_add(a.sync + (c_m * kSyncSlots + rank % kSyncSlots) * kSyncStride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            NNHIP_TRACE(8 + 4 * c_m + 3);
        }
        NNHIP_TRACE(6);
        while (c_u < a.total_units && c_u >= table[c_m].first_unit + table[c_m].units) ++c_m;
    }
    if (CHAIN) {
        // The last workgroup to leave clears the counters for the next launch (nobody polls them any more).
        if (tid == 0) {
            uint32_t* exit_word = a.sync + a.entries * kSyncSlots * kSyncStride;
            const uint32_t before = __hip_atomic_fetch_add(exit_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (before == static_cast<uint32_t>(G) - 1u)
                for (int m = 0; m <= a.entries * kSyncSlots; ++m)
                    __hip_atomic_store(a.sync + m * kSyncStride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------- host side
struct StreamTraits { int block_bytes, pieces, sum_run, table_bytes; bool sums; int min_unit_rows; };

StreamTraits stream_traits(uint32_t type)
{
    switch (type) {
    case NNHIP_TYPE_Q8_0: return {Q8_0Task::kBlockBytes, Q8_0Task::kPieces, Q8_0Task::kSumRun, 0, Q8_0Task::kNeedsSums, 4};
    case NNHIP_TYPE_Q4_K: return {Q4KTask::kBlockBytes, Q4KTask::kPieces, Q4KTask::kSumRun, 0, Q4KTask::kNeedsSums, 8};
    case NNHIP_TYPE_Q5_K: return {Q5KTask::kBlockBytes, Q5KTask::kPieces, Q5KTask::kSumRun, 0, Q5KTask::kNeedsSums, 8};
    case NNHIP_TYPE_Q6_K: return {Q6KTask::kBlockBytes, Q6KTask::kPieces, Q6KTask::kSumRun, 0, Q6KTask::kNeedsSums, 8};
    case NNHIP_TYPE_IQ2_S: return {IQ2STask::kBlockBytes, IQ2STask::kPieces, IQ2STask::kSumRun, IQ2STask::kTableBytes, IQ2STask::kNeedsSums, 8};
    default: return {0, 0, 0, 0, false, 0};
    }
}

// The (M, LPW) pairs the kernel is instantiated for, per storage type, widest first; `wide_x`: also instantiated with
// the registers for vectors of more than 8192 activations.
struct StreamVariant { int m, lpw; bool wide_x; };
constexpr StreamVariant kQ8_0Variants[] = {{1, 5, true}};
constexpr StreamVariant kQ4KVariants[] = {{3, 7, false}, {2, 5, false}, {1, 3, true}};
constexpr StreamVariant kQ5KVariants[] = {{2, 6, false}, {1, 3, true}};
constexpr StreamVariant kQ6KVariants[] = {{1, 4, true}};
constexpr StreamVariant kIQ2SVariants[] = {{3, 5, false}, {2, 4, true}};

struct StreamPlan {
    int m, lpw, xr, cols, row_pieces, stage_bytes, plane_cap, sums_bytes;
    size_t lds_bytes;
};

constexpr int kStreamStaticLds = 2 * 1024;      // part, tree, zero area and alignment, rounded up

int env_int(const char* name, int fallback)
{
    const char* v = getenv(name);
    return v && *v ? atoi(v) : fallback;
}

// Picks M for (type, in_w): the widest stage whose two buffers fit LDS beside the planes and that a row fills at least
// once (a row of fewer columns than the stage is wide would leave most of every stage empty).
bool plan_stream(uint32_t type, int in_w, StreamPlan* out)
{
    const StreamTraits tr = stream_traits(type);
    if (!tr.pieces) return false;
    const int nblocks = in_w / 256;
    const StreamVariant* list = nullptr;
    int n = 0;
    switch (type) {
    case NNHIP_TYPE_Q8_0: list = kQ8_0Variants; n = 1; break;
    case NNHIP_TYPE_Q4_K: list = kQ4KVariants; n = 3; break;
    case NNHIP_TYPE_Q5_K: list = kQ5KVariants; n = 2; break;
    case NNHIP_TYPE_Q6_K: list = kQ6KVariants; n = 1; break;
    case NNHIP_TYPE_IQ2_S: list = kIQ2SVariants; n = 2; break;
    default: return false;
    }
    const int forced_m = env_int("NNHIP_STREAM_M", 0);
    for (int v = 0; v < n; ++v) {
        StreamPlan p{};
        p.m = list[v].m;
        p.lpw = list[v].lpw;
        if (forced_m && p.m != forced_m) continue;
        p.xr = in_w > kXRegsNarrow * 4 * kStreamThreads ? kXRegsWide : kXRegsNarrow;
        if (p.xr == kXRegsWide && !list[v].wide_x) continue;
        p.cols = kStreamWaves * p.m;
        if (!forced_m && p.cols > nblocks && v + 1 < n) continue;
        p.row_pieces = (p.cols * tr.pieces) | 1;
        const int loads = (kTileRows * p.row_pieces + 63) / 64;
        if ((loads + kStreamWaves - 1) / kStreamWaves > p.lpw) continue;
        p.stage_bytes = kTileRows * p.row_pieces * 16;
        p.plane_cap = in_w + 16;
        p.sums_bytes = tr.sums ? (in_w / tr.sum_run) * 4 : 0;
        p.lds_bytes = 2 * static_cast<size_t>(p.stage_bytes) + 4 * static_cast<size_t>(p.plane_cap) + p.sums_bytes + (in_w / 32) * 4;
        if (p.lds_bytes + kStreamStaticLds + tr.table_bytes > static_cast<size_t>(kStreamLds)) continue;
        *out = p;
        return true;
    }
    return false;
}

// Matrix rows per unit of work: the most rows (fewest units) that leave at most 6 % of a round of workgroups idle.
int pick_unit_rows(int out_w, int min_rows, int groups)
{
    const int forced = env_int("NNHIP_STREAM_UNIT_ROWS", 0);
    if (forced == 16 || forced == 8 || forced == 4) return forced;
    int ur = kTileRows;
    for (; ur > min_rows; ur >>= 1) {
        const long units = (out_w + ur - 1) / ur;
        const long rounds = (units + groups - 1) / groups;
        if (units >= groups && (rounds * groups - units) * 100 <= 6 * units) break;
    }
    return ur;
}

template <class F, int M, int LPW, int XR>
hipError_t launch_stream_variant(Lane* lane, const StreamArgs& a, size_t lds, int groups)
{
    static LdsLimit big_lds;
    const void* fn = reinterpret_cast<const void*>(&matvec_mfma_stream_kernel<F, M, LPW, XR>);
    const hipError_t e = big_lds.ensure(lane->device, fn, kStreamLds - kStreamStaticLds - F::kLdsTableBytes);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((matvec_mfma_stream_kernel<F, M, LPW, XR>), dim3(groups), dim3(kStreamThreads), lds, lane->stream, a);
    return hipGetLastError();
}

}  // namespace

#if defined(NNHIP_STREAM_TRACE)
extern "C" __attribute__((visibility("default"))) int nnhip_debug_stream_trace(unsigned long long* out)
{
    return static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_stream_trace), sizeof(g_stream_trace)));
}
#endif

bool matvec_stream_takes(uint32_t type, int pre_op, const void* x, const void* w, int in_w, int out_w)
{
    if (!env_int("NNHIP_STREAM", 0)) return false;      // (off unless asked for: the row-step kernels start faster on their own)
    const StreamTraits tr = stream_traits(type);
    if (!tr.pieces || in_w % 256 != 0 || in_w < 1024 || in_w > kXRegsWide * 4 * kStreamThreads) return false;
    if (pre_op == NNHIP_PRE_RMS_NORM && in_w > kNormRegs * 4 * kStreamThreads) return false;
    if ((reinterpret_cast<uintptr_t>(w) & 15u) || (reinterpret_cast<uintptr_t>(x) & 15u)) return false;
    if (tr.block_bytes % 16 != 0 && ((in_w / 256) & 1)) return false;          // (Q6_K, IQ2_S: a row must end with an odd block)
    const uint64_t bytes = static_cast<uint64_t>(out_w) * (in_w / 256) * tr.block_bytes;
    if (bytes >= 0x7fffffffull) return false;                                  // piece offsets are 32-bit and "no piece" is bit 31
    if ((out_w + kTileRows - 1) / kTileRows < env_int("NNHIP_STREAM_MIN_TILES", 128)) return false;
    StreamPlan p;
    return plan_stream(type, in_w, &p);
}

namespace {

void fill_entry(const nnhip_fused_matvec_desc& d, const StreamTraits& tr, int cols, int unit_rows, int first_unit, StreamEntry* out)
{
    StreamEntry e{};
    e.x = d.x;
    e.x2 = d.x2;
    e.gamma = d.norm_weight;
    e.x_out = d.x_out;
    e.sum_out = d.sum_out;
    e.w = static_cast<const uint8_t*>(d.w);
    e.bias = d.bias;
    e.addend = d.addend;
    e.y = d.y;
    e.lora_z = d.lora_z;
    e.lora_b = d.lora_b;
    e.lora_rank = d.lora_rank;
    e.lora_scale = d.lora_scale;
    e.epsilon = d.epsilon;
    e.pre_op = static_cast<int>(d.pre_op);
    e.in_w = d.in_w;
    e.out_w = d.out_w;
    e.nblocks = d.in_w / 256;
    e.row_bytes = static_cast<uint32_t>(e.nblocks) * static_cast<uint32_t>(tr.block_bytes);
    e.w_bytes = static_cast<uint32_t>(d.out_w) * e.row_bytes;
    e.kchunks = (e.nblocks + cols - 1) / cols;
    e.tail_cols = e.nblocks - (e.kchunks - 1) * cols;
    e.unit_rows = unit_rows;
    e.units = (d.out_w + unit_rows - 1) / unit_rows;
    e.first_unit = first_unit;
    e.x_head_width = d.x_head_width;
    e.x_head_group = d.x_head_group;
    e.pair_rows = d.post_op == NNHIP_POST_SILU_PAIR ? d.out_w / 2 : 0;
    if (e.pair_rows > 0) e.units = (e.pair_rows + unit_rows - 1) / unit_rows;
    *out = e;
}

void fill_args(const StreamPlan& p, StreamArgs* a)
{
    a->cols = p.cols;
    a->row_pieces = p.row_pieces;
    a->row_pieces_magic = static_cast<uint32_t>((0x100000000ull + p.row_pieces - 1) / p.row_pieces);
    a->stage_bytes = p.stage_bytes;
    a->plane_cap = p.plane_cap;
    a->sums_bytes = p.sums_bytes;
}

}  // namespace

hipError_t launch_matvec_stream(Lane* lane, const nnhip_fused_matvec_desc& d)
{
    const StreamTraits tr = stream_traits(d.ggml_type);
    StreamPlan p;
    if (!plan_stream(d.ggml_type, d.in_w, &p)) return hipErrorInvalidValue;
    StreamArgs a{};
    a.table = nullptr;
    a.entries = 1;
    fill_args(p, &a);
    fill_entry(d, tr, p.cols, pick_unit_rows(d.out_w, tr.min_unit_rows, lane->compute_units), 0, &a.one);
    a.total_units = a.one.units;
    const int groups = a.one.units < lane->compute_units ? a.one.units : lane->compute_units;
#define NNHIP_STREAM(F, MM, L, XR) \
    if (p.m == MM && p.lpw == L && p.xr == XR) return launch_stream_variant<F, MM, L, XR>(lane, a, p.lds_bytes, groups);
#define NNHIP_STREAM_BOTH(F, MM, L) NNHIP_STREAM(F, MM, L, kXRegsNarrow) NNHIP_STREAM(F, MM, L, kXRegsWide)
    switch (d.ggml_type) {
    case NNHIP_TYPE_Q8_0: NNHIP_STREAM_BOTH(Q8_0Task, 1, 5) break;
    case NNHIP_TYPE_Q4_K: NNHIP_STREAM(Q4KTask, 3, 7, kXRegsNarrow) NNHIP_STREAM(Q4KTask, 2, 5, kXRegsNarrow) NNHIP_STREAM_BOTH(Q4KTask, 1, 3) break;
    case NNHIP_TYPE_Q5_K: NNHIP_STREAM(Q5KTask, 2, 6, kXRegsNarrow) NNHIP_STREAM_BOTH(Q5KTask, 1, 3) break;
    case NNHIP_TYPE_Q6_K: NNHIP_STREAM_BOTH(Q6KTask, 1, 4) break;
    case NNHIP_TYPE_IQ2_S: NNHIP_STREAM(IQ2STask, 3, 5, kXRegsNarrow) NNHIP_STREAM_BOTH(IQ2STask, 2, 4) break;
    default: break;
    }
#undef NNHIP_STREAM_BOTH
#undef NNHIP_STREAM
    return hipErrorInvalidConfiguration;
}

// ------------------------------------------------------------------------------------------------------------- chains
// A chain is a list of fused mat-vecs in which a step may consume what the step before it produced.  Consecutive steps
// of one storage type that the kernel above takes become ONE launch of its CHAIN form: the units of all steps form one
// sequence dealt round-robin to the workgroups, a workgroup that has finished its units of a step goes on requesting
// the weights of the next one, and only the preparation of the next step's vector waits until every owner of the
// previous step has counted itself in.  Steps the kernel does not take are launched between those launches with
// nnhip_quant_matvec_fused's kernels.
namespace {

constexpr int kChainXRegs = kXRegsWide;

// (M, LPW) of the chain form per storage type: one block column per wave and stage, except IQ2_S (two: its blocks are small)
bool chain_variant(uint32_t type, int* m, int* lpw)
{
    switch (type) {
    case NNHIP_TYPE_Q8_0: *m = 1; *lpw = 5; return true;
    case NNHIP_TYPE_Q4_K: *m = 1; *lpw = 3; return true;
    case NNHIP_TYPE_Q5_K: *m = 1; *lpw = 3; return true;
    case NNHIP_TYPE_Q6_K: *m = 1; *lpw = 4; return true;
    case NNHIP_TYPE_IQ2_S: *m = 2; *lpw = 4; return true;
    default: return false;
    }
}

bool plan_chain(uint32_t type, int max_in_w, StreamPlan* out)
{
    const StreamTraits tr = stream_traits(type);
    StreamPlan p{};
    if (!tr.pieces || !chain_variant(type, &p.m, &p.lpw)) return false;
    p.xr = kChainXRegs;
    p.cols = kStreamWaves * p.m;
    p.row_pieces = (p.cols * tr.pieces) | 1;
    p.stage_bytes = kTileRows * p.row_pieces * 16;
    p.plane_cap = max_in_w + 16;
    p.sums_bytes = tr.sums ? (max_in_w / tr.sum_run) * 4 : 0;
    p.lds_bytes = 2 * static_cast<size_t>(p.stage_bytes) + 4 * static_cast<size_t>(p.plane_cap) + p.sums_bytes + (max_in_w / 32) * 4;
    if (p.lds_bytes + kStreamStaticLds + tr.table_bytes > static_cast<size_t>(kStreamLds)) return false;
    *out = p;
    return true;
}

// Rows per unit for a step of a chain: every workgroup should own the same number of rows of EVERY step (a step ends
// when its slowest owner does), so the rows per workgroup, ceil(out_w / groups), are cut into the fewest units of at
// most 16 rows that waste the least.
int chain_unit_rows(int out_w, int groups, int min_rows, int max_rows)
{
    const int forced = env_int("NNHIP_CHAIN_UNIT_ROWS", 0);
    if (forced >= 1 && forced <= max_rows) return forced;
    const int share = (out_w + groups - 1) / groups;
    if (share <= max_rows) return share < min_rows ? (min_rows < out_w ? min_rows : share) : share;
    // (large units keep more bytes on their way per workgroup: the fewest units that waste at most 6 % of a share)
    int best_rows = max_rows, best_waste = 1 << 30;
    const int n0 = (share + max_rows - 1) / max_rows;
    for (int n = n0; n <= n0 + 3; ++n) {
        const int rows = (share + n - 1) / n;
        if (rows < min_rows) break;
        const int waste = n * rows - share;
        if (waste * 100 <= 6 * share) return rows;
        if (waste < best_waste) {
            best_waste = waste;
            best_rows = rows;
        }
    }
    return best_rows;
}

template <class F, int M, int LPW>
hipError_t launch_chain_variant(Lane* lane, const StreamArgs& a, size_t lds, int groups)
{
    static LdsLimit big_lds;
    const void* fn = reinterpret_cast<const void*>(&matvec_mfma_stream_kernel<F, M, LPW, kChainXRegs, true>);
    const hipError_t e = big_lds.ensure(lane->device, fn, kStreamLds - kStreamStaticLds - F::kLdsTableBytes);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((matvec_mfma_stream_kernel<F, M, LPW, kChainXRegs, true>), dim3(groups), dim3(kStreamThreads), lds, lane->stream, a);
    return hipGetLastError();
}

bool chain_takes(const nnhip_fused_matvec_desc& d)
{
    const StreamTraits tr = stream_traits(d.ggml_type);
    if (!tr.pieces || d.in_w % 256 != 0 || d.in_w < 1024 || d.in_w > kChainXRegs * 4 * kStreamThreads) return false;
    if (d.pre_op == NNHIP_PRE_RMS_NORM && d.in_w > kNormRegs * 4 * kStreamThreads) return false;
    auto misaligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; };
    if (misaligned(d.w) || misaligned(d.x) || misaligned(d.x2) || misaligned(d.norm_weight) || misaligned(d.x_out) || misaligned(d.sum_out))
        return false;
    if (tr.block_bytes % 16 != 0 && ((d.in_w / 256) & 1)) return false;
    const uint64_t bytes = static_cast<uint64_t>(d.out_w) * (d.in_w / 256) * tr.block_bytes;
    if (bytes >= 0x7fffffffull) return false;
    StreamPlan p;
    return plan_chain(d.ggml_type, d.in_w, &p);
}

}  // namespace

struct ChainSegment {
    bool kernel;                            // true: one launch of the chain form over `entries` table entries
    nnhip_fused_matvec_desc step;           // false: this step through launch_matvec_fused
    uint32_t type;
    StreamArgs args;
    size_t lds_bytes;
    int m, lpw, groups;
};

struct ChainImpl {
    std::vector<ChainSegment> segments;
    void* device_block = nullptr;           // the tables of all segments, then their counters
    size_t device_bytes = 0;
};

void chain_free(ChainImpl* c)
{
    if (!c) return;
    if (c->device_block) (void)hipFree(c->device_block);
    delete c;
}

// Builds the launches of a chain; `steps` have been validated.  Blocking (one allocation, one upload).
hipError_t chain_build(Lane* lane, const nnhip_fused_matvec_desc* steps, int count, ChainImpl** out)
{
    ChainImpl* c = new ChainImpl();
    std::vector<StreamEntry> table;
    struct Run { size_t segment, first_entry, entries; };
    std::vector<Run> runs;
    const int G = lane->compute_units;
    for (int i = 0; i < count;) {
        const nnhip_fused_matvec_desc& d = steps[i];
        if (!chain_takes(d)) {
            if (d.x_head_width > 0 || d.post_op != NNHIP_POST_NONE) {
                chain_free(c);
                return hipErrorNotSupported;
            }
            ChainSegment seg{};
            seg.kernel = false;
            seg.step = d;
            c->segments.push_back(seg);
            ++i;
            continue;
        }
        // the longest run of steps of this type whose planes fit LDS together
        int j = i, max_in_w = 0;
        StreamPlan plan{};
        while (j < count && steps[j].ggml_type == d.ggml_type && chain_takes(steps[j])) {
            const int w = steps[j].in_w > max_in_w ? steps[j].in_w : max_in_w;
            StreamPlan p;
            if (!plan_chain(d.ggml_type, w, &p)) break;
            plan = p;
            max_in_w = w;
            ++j;
        }
        const StreamTraits tr = stream_traits(d.ggml_type);
        ChainSegment seg{};
        seg.kernel = true;
        seg.type = d.ggml_type;
        seg.lds_bytes = plan.lds_bytes;
        seg.m = plan.m;
        seg.lpw = plan.lpw;
        fill_args(plan, &seg.args);
        seg.args.entries = j - i;
        seg.args.spin_limit = env_int("NNHIP_CHAIN_SPIN_LIMIT", 1 << 18);
        int first_unit = 0;
        const size_t first_entry = table.size();
        for (int k = i; k < j; ++k) {
            StreamEntry e;
            const bool pair = steps[k].post_op == NNHIP_POST_SILU_PAIR;
            // (paired halves: a unit is up to 8 rows of each half)
            const int unit_rows = pair ? (env_int("NNHIP_CHAIN_PAIR_ROWS", 0) > 0 ? env_int("NNHIP_CHAIN_PAIR_ROWS", 0) : chain_unit_rows(steps[k].out_w / 2, G, 1, 8))
                                       : chain_unit_rows(steps[k].out_w, G, tr.min_unit_rows >= 8 ? 8 : 1, kTileRows);
            fill_entry(steps[k], tr, plan.cols, unit_rows, first_unit, &e);
            e.wait = k > i ? 1 : 0;
            e.signals = e.units < G ? e.units : G;
            first_unit += e.units;
            table.push_back(e);
        }
        seg.args.total_units = first_unit;
        seg.groups = first_unit < G ? first_unit : G;
        for (size_t k = first_entry; k < table.size(); ++k) table[k].signals = table[k].units < seg.groups ? table[k].units : seg.groups;
        runs.push_back({c->segments.size(), first_entry, table.size() - first_entry});
        c->segments.push_back(seg);
        i = j;
    }
    // device block: the entries, then per kernel segment its counters (entries + exit counter + status word)
    const size_t table_bytes = (table.size() * sizeof(StreamEntry) + 255) / 256 * 256;
    size_t sync_words = 0;
    for (const Run& r : runs) sync_words += (r.entries * kSyncSlots + 2) * kSyncStride;
    c->device_bytes = table_bytes + sync_words * sizeof(uint32_t) + 256;
    hipError_t e = hipMalloc(&c->device_block, c->device_bytes);
    if (e != hipSuccess) {
        c->device_block = nullptr;
        chain_free(c);
        return e;
    }
    e = hipMemset(c->device_block, 0, c->device_bytes);
    if (e == hipSuccess && !table.empty())
        e = hipMemcpy(c->device_block, table.data(), table.size() * sizeof(StreamEntry), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        chain_free(c);
        return e;
    }
    uint32_t* sync = reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(c->device_block) + table_bytes);
    for (const Run& r : runs) {
        ChainSegment& seg = c->segments[r.segment];
        seg.args.table = reinterpret_cast<const StreamEntry*>(c->device_block) + r.first_entry;
        seg.args.sync = sync;
        sync += (r.entries * kSyncSlots + 2) * kSyncStride;
    }
    *out = c;
    return hipSuccess;
}

int chain_launch_count(const ChainImpl* c) { return static_cast<int>(c->segments.size()); }

hipError_t chain_launch(Lane* lane, const ChainImpl* c)
{
    for (const ChainSegment& seg : c->segments) {
        hipError_t e = hipErrorInvalidConfiguration;
        if (!seg.kernel) {
            e = launch_matvec_fused(lane, seg.step);
        } else {
            switch (seg.type) {
            case NNHIP_TYPE_Q8_0: e = launch_chain_variant<Q8_0Task, 1, 5>(lane, seg.args, seg.lds_bytes, seg.groups); break;
            case NNHIP_TYPE_Q4_K: e = launch_chain_variant<Q4KTask, 1, 3>(lane, seg.args, seg.lds_bytes, seg.groups); break;
            case NNHIP_TYPE_Q5_K: e = launch_chain_variant<Q5KTask, 1, 3>(lane, seg.args, seg.lds_bytes, seg.groups); break;
            case NNHIP_TYPE_Q6_K: e = launch_chain_variant<Q6KTask, 1, 4>(lane, seg.args, seg.lds_bytes, seg.groups); break;
            case NNHIP_TYPE_IQ2_S: e = launch_chain_variant<IQ2STask, 2, 4>(lane, seg.args, seg.lds_bytes, seg.groups); break;
            default: break;
            }
        }
        if (e != hipSuccess) return e;
        ++lane->counters.kernel_launches;
    }
    return hipSuccess;
}

// 1 when a workgroup of some launch of the chain gave up waiting for a step since the status was last read (cleared by the read).
hipError_t chain_status(Lane* lane, const ChainImpl* c, int* gave_up)
{
    *gave_up = 0;
    hipError_t e = hipStreamSynchronize(lane->stream);
    for (const ChainSegment& seg : c->segments) {
        if (!seg.kernel || e != hipSuccess) continue;
        uint32_t* word = seg.args.sync + (seg.args.entries * kSyncSlots + 1) * kSyncStride;
        uint32_t v = 0;
        e = hipMemcpy(&v, word, sizeof(v), hipMemcpyDeviceToHost);
        if (e == hipSuccess && v) {
            *gave_up = 1;
            e = hipMemset(word, 0, sizeof(v));
        }
    }
    return e;
}

}  // namespace nnhip
