// Decode mat-vec on the matrix cores: for the super-block formats whose unpacking is too much vector-ALU work for the
// lane-per-unit kernels (gemv_kernels.hip), Q4_K, Q5_K, Q6_K and IQ2_S, and for Q8_0, whose signed bytes are operand B
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
#include "gemv_mfma_tasks.h"

namespace nnhip {

namespace {

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
    int chunked;                   // 1: a workgroup takes a run of consecutive tiles, 0: every G-th tile
    MfmaGeom g;
};

// grid.x = workgroups striding over the launch's 16-row tiles, blockDim.x = 64 * W.  KC = stages per tile (1 or 2),
// M = super-block columns a wave owns per stage, LPW = 1 KB pieces of a stage a wave moves.  A lane keeps operand A of its KC * M columns in registers for as long as the activations stay
// the same.
template <class F, int KC, int M, int LPW>
__global__ __launch_bounds__(64 * kMaxWaves) void matvec_mfma_kernel(MfmaArgs a)
{
    static_assert(KC == 1 || KC == 2, "a turn of the two register sets is one or two tiles");
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
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const uint32_t slot = static_cast<uint32_t>(64 * (wave + W * i) + lane);
        const uint32_t r = __umulhi(slot, a.row_pieces_magic);
        const uint32_t q = slot - r * static_cast<uint32_t>(g.row_pieces);
        const uint32_t c = q / static_cast<uint32_t>(F::kPieces);
        const bool real = r < static_cast<uint32_t>(kTileRows) && q < static_cast<uint32_t>(pieces_used);
        rel[i] = real ? r * a.row_bytes + c * F::kBlockBytes + F::piece_src(q - c * F::kPieces, c & 1u) : kNoPiece;
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
        for (int i = 0; i < LPW; ++i) *reinterpret_cast<u32x4*>(dst + W * i * 1024) = set[i];
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
    u32x4 regs[2][LPW];
    fetch_enter();
    fetch(regs[0]);
    fetch(regs[1]);

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
        fetch(refill);                  // (before the activations are dealt with: the stream must not pause for them)
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
        __syncthreads();                // publishes `nxt`, frees `cur`
    };

    park(buf0, regs[0]);
    __syncthreads();
    using std::integral_constant;
    for (int n = 0; n < total; n += 2) {
        stage_step(integral_constant<int, 0>{}, buf0, buf1, regs[0], regs[1]);
        if (n + 1 < total) stage_step(integral_constant<int, KC - 1>{}, buf1, buf0, regs[1], regs[0]);
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
    WideGeom g;
    MfmaEntry inline_entries[4];   // a call with up to 16 input rows needs no table in device memory
};

template <class F, int M, int LPW, int R, bool ONE = false>
__global__ __launch_bounds__(64 * kMaxWaves) void matvec_mfma_wide_kernel(WideArgs a)
{
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
    const int n4 = a.in_w >> 2;

    // ---- prefetch side
    int f_t = t_first, f_k = 0, f_m = 0;
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
        if (++f_k == KC) {
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
    auto prepare_x = [&]() {
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
        constexpr int kPrep = R > 1 && LPW <= 3 ? 8 : 0;
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
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r < rows) {
                const float4* x4 = reinterpret_cast<const float4*>(ce.x + static_cast<size_t>(r) * a.in_w);
                uint32_t mx = 0;
                for (int i = tid; i < n4; i += T) mx = umax4(mx, x4[i]);
                mx = wave_umax(mx);
                if (lane == 0) red[r][wave] = mx;
            }
        }
        __syncthreads();
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
                const float4* x4 = reinterpret_cast<const float4*>(ce.x + static_cast<size_t>(r) * a.in_w);
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
                if (done_bias) {
                    const NNHIP_CONST_PTR float* cb = (const NNHIP_CONST_PTR float*)done_bias + done_row0;
                    float bv = 0.0f;
#pragma unroll
                    for (int j = 0; j < kTileRows; ++j) {
                        const float v = cb[j < done_rows ? j : 0];
                        bv = j0 == j ? v : bv;
                    }
                    t += bv;
                }
                if (j0 < done_rows) done_y[static_cast<size_t>(r) * done_out_w + done_row0 + j0] = t;
            }
        }
        done = false;
    };

    float accq[R], accm[R];
#pragma unroll
    for (int r = 0; r < R; ++r) accq[r] = accm[r] = 0.0f;
    // The matrix of the stage about to be multiplied; true when its activations are not the ones in LDS.
    auto enter = [&]() {
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
            const uint8_t* stage = cur + row_off;
            constexpr int kSumsPerBlock = 256 / F::kSumRun;
#pragma unroll
            for (int t = 0; t < M; ++t) {
                const int b = b0 + t * W;
                if (b < a.nblocks)
                    F::run_stacked(F::load_stacked(stage + t * W * (16 * F::kPieces), quarter, (wave & 1) != 0), a_plane + 256 * b,
                                   d_sums + kSumsPerBlock * b, tables, acc_sq, acc_sm);
            }
            if (++c_k == KC) {
                c_k = 0;
                const float p = fmaf(acc_sq, inv_of_row[quarter], -acc_sm);     // (from LDS: a register array indexed by the lane would go to scratch memory)
                if (quarter < ce.rows) part[pbuf][quarter][wave][row_l] = p;
                acc_sq = 0.0f;
                acc_sm = 0.0f;
                done = true;
                done_row0 = (c_t - ce.first_tile) * kTileRows;
                pbuf ^= 1;
                c_t += t_step;
            }
        } else {
        // task t of this wave: block column c_k * cols + t * W + wave of the row (W is even: the block's parity is the
        // wave's).  Stages whose tasks all exist run them as one straight piece of code, so that the lookups and products
        // of one task overlap the other's; a tile's last stage may hold fewer.
        auto task = [&](const typename F::Raw& raw, int b) {
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
        if (++c_k == KC) {
            c_k = 0;
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
            c_t += t_step;
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
constexpr Variant kVariants[] = {{1, 2, 5}, {1, 2, 6}, {2, 1, 3}, {1, 1, 3}, {2, 2, 5}, {2, 2, 6}, {1, 1, 2}, {2, 1, 2},
                                 {1, 1, 4}, {2, 1, 4}};

// Picks W and C for (block bytes, in_w).  C = W * M columns per stage must divide the row's super-blocks into KC whole
// stages, two stage buffers must fit LDS (one of them doubles as scratch for the digit planes when the activations
// change), (KC, M, LPW) must be an instantiated variant, and among those the choice maximises the bytes a stage holds,
// then the waves.
bool plan_mfma(int block_pieces, int in_w, bool even_waves, MfmaGeom* out)
{
    const int nblocks = in_w / 256;
    const int bp = block_pieces;
    if (nblocks < 1 || bp < 1) return false;
    const int planes_bytes = 4 * (in_w + 16) + (in_w / 16) * 4;
    double best_score = -1.0;
    MfmaGeom best{};
    for (int W = 6; W <= kMaxWaves; ++W) {
        for (int m = 1; m <= 2; ++m) {
            MfmaGeom g{};
            if (even_waves && (W & 1)) continue;       // block parity must be wave parity (Q6_K)
            g.waves = W;
            g.cols = W * m;
            if (nblocks % g.cols != 0) continue;
            g.kchunks = nblocks / g.cols;
            g.tasks = m;
            g.row_pieces = (g.cols * bp) | 1;
            g.stage_loads = (kTileRows * g.row_pieces + 63) / 64;
            g.loads_per_wave = (g.stage_loads + W - 1) / W;
            g.stage_bytes = g.loads_per_wave * W * 1024;          // every wave parks loads_per_wave pieces
            if (g.stage_bytes < planes_bytes || 2 * g.stage_bytes > kLdsBudget) continue;
            bool ok = false;
            for (const Variant& v : kVariants) ok = ok || (v.kc == g.kchunks && v.m == m && v.lpw == g.loads_per_wave);
            if (!ok) continue;
            g.stages = 2;
            g.lds_bytes = 2 * static_cast<size_t>(g.stage_bytes);
            // one column per wave keeps the register sets small (no spills); then the larger stage, then the waves
            const double score = (m == 1 ? 1.0 : 0.0) + static_cast<double>(g.stage_bytes) / (256.0 * 1024) + 1e-3 * W;
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

template <class F, int KC, int M, int LPW>
hipError_t launch_mfma_variant(Lane* lane, const MfmaArgs& a, dim3 grid)
{
    static LdsLimit big_lds;
    const hipError_t e = big_lds.ensure(lane->device, reinterpret_cast<const void*>(&matvec_mfma_kernel<F, KC, M, LPW>), kLdsBudget);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((matvec_mfma_kernel<F, KC, M, LPW>), grid, dim3(64 * a.g.waves), a.g.lds_bytes, lane->stream, a);
    return hipGetLastError();
}

template <class F>
hipError_t launch_mfma(Lane* lane, const MfmaArgs& a)
{
    const int groups = a.total_tiles < lane->compute_units ? a.total_tiles : lane->compute_units;
    const dim3 grid(groups);
    const int kc = a.g.kchunks, m = a.g.tasks, lpw = a.g.loads_per_wave;
#define NNHIP_VARIANT(K, MM, L) if (kc == K && m == MM && lpw == L) return launch_mfma_variant<F, K, MM, L>(lane, a, grid);
    NNHIP_VARIANT(1, 2, 5) NNHIP_VARIANT(1, 2, 6) NNHIP_VARIANT(2, 1, 3) NNHIP_VARIANT(1, 1, 3) NNHIP_VARIANT(2, 2, 5)
    NNHIP_VARIANT(2, 2, 6) NNHIP_VARIANT(1, 1, 2) NNHIP_VARIANT(2, 1, 2) NNHIP_VARIANT(1, 1, 4) NNHIP_VARIANT(2, 1, 4)
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
        // (and of two equal products the fuller stages win: 16 blocks go as 2 x 8 rather than 12 + 4)
        const double score = fill * W / 12.0 * (W % 4 == 0 ? 1.0 : 0.95) * (0.9 + 0.1 * fill);
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
    if (type == NNHIP_TYPE_IQ2_S || type == NNHIP_TYPE_Q8_0) return false;       // (these have the wide form only)

    if (!entry_ok(type, in_w, out_w, w)) return false;
    MfmaGeom g;
    if (!plan_mfma(block_pieces_of(type), in_w, block_bytes_of(type) % 16 != 0, &g)) return false;
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
    if (!plan_mfma(block_pieces_of(type), in_w, block_bytes_of(type) % 16 != 0, &g)) return hipErrorInvalidValue;
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

bool matvec_mfma_wide_geometry(uint32_t type, int in_w, int out_w, const void* w, int inputs)
{
    WideGeom g;
    return inputs >= 1 && inputs <= 4 && entry_ok(type, in_w, out_w, w) && plan_wide(type, in_w, inputs == 1 ? 1 : 4, &g);
}

namespace {

hipError_t launch_wide_args(Lane* lane, uint32_t type, int in_w, int inputs, WideArgs& a)
{
    if (!plan_wide(type, in_w, inputs == 1 ? 1 : 4, &a.g)) return hipErrorInvalidValue;
    a.in_w = in_w;
    a.nblocks = in_w / 256;
    a.row_bytes = static_cast<uint32_t>(a.nblocks) * static_cast<uint32_t>(block_bytes_of(type));
    a.row_pieces_magic = static_cast<uint32_t>((0x100000000ull + a.g.row_pieces - 1) / a.g.row_pieces);
    switch (type) {
    case NNHIP_TYPE_Q4_K: return launch_wide<Q4KTask>(lane, a, inputs);
    case NNHIP_TYPE_Q5_K: return launch_wide<Q5KTask>(lane, a, inputs);
    case NNHIP_TYPE_Q6_K: return launch_wide<Q6KTask>(lane, a, inputs);
    case NNHIP_TYPE_IQ2_S: return launch_wide<IQ2STask>(lane, a, inputs);
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

bool describe_matvec_rows_shared(uint32_t type, int rows, int in_w, int out_w, int compute_units, nnhip_matvec_plan_info* info)
{
    WideGeom g;
    if (!plan_wide(type, in_w, 4, &g)) return false;
    const int tiles = (out_w + kTileRows - 1) / kTileRows * ((rows + 3) / 4);
    info->kernel = NNHIP_MATVEC_KERNEL_MATRIX_CORE;
    info->threads = 64 * g.waves;
    info->rows_per_step = kTileRows;
    info->steps = tiles;
    info->groups = tiles < compute_units ? tiles : compute_units;
    info->row_tile = rows < 4 ? rows : 4;
    info->ring_depth = 2;                                   // stage buffers
    info->result_buffer_floats = 2 * 4 * kMaxWaves * kTileRows;
    info->dynamic_lds_bytes = static_cast<int32_t>(g.lds_bytes);
    return true;
}

bool describe_matvec_mfma_launch(uint32_t type, int in_w, int form, bool runs, nnhip_batch_launch_info* info)
{
    if (form == 1) {
        MfmaGeom g;
        if (!plan_mfma(block_pieces_of(type), in_w, block_bytes_of(type) % 16 != 0, &g)) return false;
        info->threads = 64 * g.waves;
        info->stage_buffers = g.stages;
        info->dynamic_lds_bytes = static_cast<int32_t>(g.lds_bytes);
        info->activations_in_lds = 0;
        info->consecutive_runs = runs ? 1 : 0;
        return true;
    }
    WideGeom g;
    if (!plan_wide(type, in_w, form == 3 ? 4 : 1, &g)) return false;
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
                                     int rows, int in_w, int out_w)
{
    if (rows < 2 || rows > 16) return hipErrorInvalidValue;
    WideArgs a{};
    a.table = nullptr;
    for (int r = 0; r < rows; r += 4) {
        MfmaTableEntry e = matvec_mfma_entry(type, x + static_cast<size_t>(r) * in_w, w, bias, y + static_cast<size_t>(r) * out_w,
                                             in_w, out_w, a.total_tiles);
        e.rows = rows - r < 4 ? rows - r : 4;
        a.inline_entries[a.entries++] = e;
        a.total_tiles += e.tiles;
    }
    a.chunked = a.entries >= 3 ? 1 : 0;         // (9 - 16 input rows: three or four groups of rows, each with planes of its own)
    return launch_wide_args(lane, type, in_w, 4, a);
}

}  // namespace nnhip
