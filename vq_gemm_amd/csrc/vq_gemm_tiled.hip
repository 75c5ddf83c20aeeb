// Plain fp16 GEMM with the tile of the prefill kernel: the no-dequant control of the VQ path
// (reference strategy_1/src.cu:171-265, strategy_2/bsz128/src.cu:318-515) and the second pass of
// the two-pass strategy.
//   NN: y[M,N] = x[M,K] . w[K,N]      NT: y[M,N] = x[M,K] . w[N,K]^T
//
// Same frame as the VQ kernel: 256 threads (2x2 waves), a 256x256 tile of Y, 128x128 per wave as
// 8x8 pieces of 16x16 with v_mfma_f32_16x16x32_f16, the accumulators pinned in the AGPRs, every
// MFMA fenced and the other instructions dealt out between them by hand.  What differs is where
// the W operand comes from: W is staged through the LDS like X instead of being gathered from a
// codebook, which doubles the LDS bytes per k.
//
//   * A stage is 32 k (one MFMA step): 256 rows of X x 64 bytes and the matching 16 KB of W,
//     global -> LDS directly.  Five stages fill the 160 KB; the loads of stage s+5 are issued
//     while step s multiplies and have three whole steps to land.
//   * Every operand is double buffered in registers: while step s multiplies, the 16 operands of
//     step s+1 are read from the LDS.  One barrier per step publishes the next stage and frees
//     the buffer of the stage just consumed.
//   * X (and W in the NT layout) lies in the LDS as 64-byte rows, four to a 256-byte bank row,
//     XOR-swizzled so that the 16 rows x one 16-byte chunk a quarter wave reads fall into 16
//     different bank groups.
//   * W in the NN layout ([K,N], n contiguous) lies as 32 k-rows of 512 bytes and is read with
//     the transposing LDS read ds_read_b64_tr_b16: within 16 lanes, source lane 4d+q supplies
//     row d, columns 4q..4q+3, and lane l receives column l of rows 0..3 - four consecutive k
//     of one n, half an MFMA operand.  The 16-byte chunks of a k-row are XOR-swizzled with the
//     row number so that the rows one instruction touches fall into different bank windows.
//
//   * A tile half as wide (256x128, 128x64 per wave, six stages of 24 KB) puts twice as many
//     compute units to work when the 256x256 tiles are fewer than the units.
//
// K must be a multiple of 64 (and N a multiple of 8 in the NN layout); other shapes stay on the
// simple kernel of vq_gemm_plain.hip.
#include "vq_tile_helpers.h"

#include <type_traits>

namespace vq {

namespace {

constexpr int BM = 256;                              // rows of the tallest tile
constexpr int kThreads = 256;
constexpr int kStepK = 32;                           // k per stage

// The tile: MPW 16-row pieces of X and NP 16-row pieces of W per wave
// (8, 8: 256x256 tile; 8, 4: 256x128; 4, 4: 128x128).
template <int NP, int MPW>
struct TileCfg {
    static_assert((NP == 8 || NP == 4) && (MPW == 8 || MPW == 4) && MPW >= NP, "256x256, 256x128 or 128x128 tiles");
    static constexpr int WM = MPW * 16, BM = 2 * WM;
    static constexpr int WN = NP * 16, BN = 2 * WN;
    static constexpr int kXBytes = BM * kStepK * 2;                // the X part of a stage: 16 or 8 KB
    static constexpr int kXLoads = kXBytes / (kThreads * 16);      // 4 or 2
    static constexpr int kWBytes = BN * kStepK * 2;                // the W part of a stage
    static constexpr int kWLoads = kWBytes / (kThreads * 16);      // 4 or 2
    static constexpr int kStageBytes = kXBytes + kWBytes;          // 32, 24 or 16 KB
    static constexpr int NS = NP == 8 ? 5 : (MPW == 8 ? 6 : 8);    // stages in the LDS
    static constexpr int kLoads = kXLoads + kWLoads;               // loads per thread and stage
    static constexpr int kChunksPerK = BN / 8;                     // 16-byte chunks of a k-row (NN layout)
    static constexpr size_t kLdsBytes = (size_t)NS * kStageBytes;
};

typedef short short4_t __attribute__((__vector_size__(4 * sizeof(short))));

// Row-major part (X, or W in the NT layout): byte offset of 16-byte chunk cc (0..3) of row `row`.
__device__ __forceinline__ int row_offset(int row, int cc)
{
    const int bank_row = row >> 2;
    const int pos = (((row & 3) << 2) | cc) ^ (bank_row & 3);
    return (bank_row * 16 + pos) * 16;
}

// k-major part (W in the NN layout): the XOR applied to the chunk index of k-row `k` (below 16).
__device__ __forceinline__ int kmajor_swizzle(int k) { return 2 * ((k & 3) | (((k >> 3) & 1) << 2)); }

template <bool W_IS_KN, int NP, int MPW>
__global__ __launch_bounds__(kThreads, 1) void gemm_tiled_kernel(const half_t *__restrict__ x,
                                                                 const half_t *__restrict__ w,
                                                                 half_t *__restrict__ y, int M, int K, int N,
                                                                 int tiles_m, int tiles_n)
{
    typedef TileCfg<NP, MPW> C;
    constexpr int NS = C::NS, WN = C::WN, BN = C::BN, kStageBytes = C::kStageBytes;
    constexpr int MP = MPW, WM = C::WM, BM = C::BM, kXBytes = C::kXBytes, kXLoads = C::kXLoads;
    extern __shared__ __align__(16) uint8_t smem[];
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int r16 = lane & 15, kg = lane >> 4;

    // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2: re-number them so
    // that an XCD works on consecutive tiles of the row-band-major order.
    int wg = blockIdx.x;
    const int n_wg = tiles_m * tiles_n;
    if ((n_wg & 7) == 0) wg = (wg & 7) * (n_wg >> 3) + (wg >> 3);
    const int tm = wg / tiles_n, tn = wg % tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    const int n_stage = K / kStepK;

    // ---- staging: global -> LDS ---------------------------------------------------------------
    // Load i of wave v fills the 64 consecutive 16-byte slots [(4i+v)*64, +64) of a part; the lane
    // looks up which chunk lives in its slot under the swizzle and fetches that.
    uint32_t x_voff[kXLoads], w_voff[C::kWLoads];
#pragma unroll
    for (int i = 0; i < kXLoads; i++) {
        const int slot = (4 * i + wave) * 64 + lane;
        const int bank_row = slot >> 4;
        const int pos = (slot & 15) ^ (bank_row & 3);
        const int row = 4 * bank_row + (pos >> 2), cc = pos & 3;
        x_voff[i] = (uint32_t)(((int64_t)(min(m0 + row, M - 1) - m0) * K + cc * 8) * 2);
        if (!W_IS_KN && i < C::kWLoads) w_voff[i] = (uint32_t)(((int64_t)(min(n0 + row, N - 1) - n0) * K + cc * 8) * 2);
        if (W_IS_KN && i < C::kWLoads) {
            const int k = slot / C::kChunksPerK;
            const int c = (slot % C::kChunksPerK) ^ kmajor_swizzle(k);
            w_voff[i] = (uint32_t)(((int64_t)k * N + (min(n0 + c * 8, N - 8) - n0)) * 2);
        }
    }
    // Where the loads of the stage NS ahead of the current one read (the last stage again once K is
    // used up: harmless, and every stage so brings the same number of loads); moved on once per step.
    const int64_t w_step = W_IS_KN ? (int64_t)kStepK * N : kStepK;
    const int first_ahead = min(NS, n_stage - 1);
    const half_t *x_ahead = x + (int64_t)m0 * K + first_ahead * kStepK;
    const half_t *w_ahead = (W_IS_KN ? w + n0 : w + (int64_t)n0 * K) + first_ahead * w_step;
    // Load i of a stage into buffer `buf` from the stage bases xb / wb: first the X part, then the W part.
    auto issue = [&](int i, int buf, const half_t *xb, const half_t *wb) {
        if (i < kXLoads) load_to_lds_16(buf * kStageBytes + (4 * i + wave) * 1024, x_voff[i], xb);
        else load_to_lds_16(buf * kStageBytes + kXBytes + (4 * (i - kXLoads) + wave) * 1024, w_voff[i - kXLoads], wb);
    };

    float4_t acc[NP][MP];
#pragma unroll
    for (int j = 0; j < NP; j++)
#pragma unroll
        for (int i = 0; i < MP; i++) acc[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};

    // ---- operand reads ------------------------------------------------------------------------
    // X piece i is rows wm*128 + i*16 + r16, the lane's chunk is kg; a piece further is four bank
    // rows (1 KB) on and leaves the swizzle unchanged.
    const int x_rd = row_offset(wm * WM + r16, kg);
    int w_rd[NP];
    if (W_IS_KN) {
        // Source lane (kg, s = r16) of a transposing read supplies row kg*8 + h*4 + s/4, columns
        // piece*16 + 4*(s%4) .. +3: 8 bytes in chunk 2*piece + (s%4)/2 of its k-row.
        const int k = kg * 8 + (r16 >> 2);  // + 4h: four rows on, same swizzle
#pragma unroll
        for (int j = 0; j < NP; j++) {
            const int chunk = (wn * (WN / 8) + 2 * j + ((r16 & 3) >> 1)) ^ kmajor_swizzle(k);
            w_rd[j] = kXBytes + (k * C::kChunksPerK + chunk) * 16 + (r16 & 1) * 8;
        }
    } else {
        w_rd[0] = kXBytes + row_offset(wn * WN + r16, kg);
    }
    half8_t xs[2][MP];
    half4_t wlo[2][NP], whi[2][NP];
    auto load_x = [&](int set, int i, int buf) {
        xs[set][i] = *reinterpret_cast<const half8_t *>(smem + buf * kStageBytes + x_rd + i * 1024);
    };
    // half h of W piece j (NT: h = 0 reads the whole operand, h = 1 nothing)
    auto load_w = [&](int set, int j, int h, int buf) {
        if constexpr (W_IS_KN) {
            typedef __attribute__((address_space(3))) short4_t lds_short4_t;
            const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (lds_short4_t *)(smem + buf * kStageBytes + w_rd[j] + h * (4 * C::kChunksPerK * 16)));
            if (h == 0) wlo[set][j] = __builtin_bit_cast(half4_t, v);
            else whi[set][j] = __builtin_bit_cast(half4_t, v);
        } else {
            if (h == 0) {
                const half8_t v = *reinterpret_cast<const half8_t *>(smem + buf * kStageBytes + w_rd[0] + j * 1024);
                wlo[set][j] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
                whi[set][j] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
            }
        }
    };

    // ---- prologue -----------------------------------------------------------------------------
    // Loads complete in the order they were issued, so one count serves all of them.
#pragma unroll
    for (int d = 0; d < NS; d++) {
        const int st = min(d, n_stage - 1);
#pragma unroll
        for (int i = 0; i < C::kLoads; i++)
            issue(i, d, x + (int64_t)m0 * K + st * kStepK, (W_IS_KN ? w + n0 : w + (int64_t)n0 * K) + st * w_step);
    }
    wait_vmcnt<(NS - 1) * C::kLoads>();  // stage 0 has landed
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MP; i++) load_x(0, i, 0);
#pragma unroll
    for (int j = 0; j < NP; j++) {
        load_w(0, j, 0, 0);
        load_w(0, j, 1, 0);
    }

    // ---- main loop ----------------------------------------------------------------------------
    // Step `stage` multiplies register set `set` while the operands of the next step are read into
    // the other set and the loads of stage + NS are issued into the buffer this step's operands
    // came from.  A wave issues one instruction every four cycles and an MFMA holds the pipe for
    // sixteen: at most three other instructions fit between two MFMAs.
    constexpr int kReads = MP + (W_IS_KN ? 2 * NP : NP);
    constexpr int kReadGap = NP == 8 ? 2 : 1;   // MFMAs from one operand read to the next
    constexpr int kLoadGap = NP == 8 ? 8 : (MP == 8 ? 5 : 4);   // MFMAs from one global load to the next
    static_assert(kReads * kReadGap <= NP * MP - 4, "the reads of a step end ahead of its last MFMAs");
    static_assert(1 + (C::kLoads - 1) * kLoadGap < NP * MP, "the loads of a stage fit into a step");
#define VQ_FENCE __builtin_amdgcn_sched_barrier(0)
    int buf = 0;  // buffer of the current stage
    auto step = [&](auto set_const, int stage) {
        constexpr int set = decltype(set_const)::value;
        const int buf_next = buf + 1 == NS ? 0 : buf + 1;
        // Stage + 1 has landed when only the stages behind it are in flight; every wave has finished
        // reading this stage's buffer (its reads were issued a step ago and are waited for here,
        // where they have long completed).
        wait_vmcnt<(NS - 2) * C::kLoads>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __syncthreads();
        VQ_FENCE;
#pragma unroll
        for (int m = 0; m < NP * MP; m++) {
            // 4x4 quadrants of the pieces: (0,0) (1,0) (1,1) (0,1) for 8 pieces of W, (0,0) (0,1) for 4
            const int q = m >> 4, p = (m >> 2) & 3, f = m & 3;
            const int jh = NP == 8 ? ((q == 1 || q == 2) ? 1 : 0) : 0;
            const int ih = NP == 8 ? q >> 1 : q;   // (one quadrant only with 4 x 4 pieces)
            const int j = jh * 4 + p, i = ih * 4 + f;
            mfma_in_place(acc[j][i], __builtin_shufflevector(wlo[set][j], whi[set][j], 0, 1, 2, 3, 4, 5, 6, 7),
                          xs[set][i]);
            VQ_FENCE;
            if (m % kReadGap == 0 && m / kReadGap < kReads) {
                const int r = m / kReadGap;
                if (r < MP) load_x(set ^ 1, r, buf_next);
                else if (W_IS_KN) load_w(set ^ 1, (r - MP) >> 1, (r - MP) & 1, buf_next);
                else load_w(set ^ 1, r - MP, 0, buf_next);
                VQ_FENCE;
            }
            if (m % kLoadGap == 1 && m / kLoadGap < C::kLoads) {
                issue(m / kLoadGap, buf, x_ahead, w_ahead);
                VQ_FENCE;
            }
        }
        const bool more = stage + NS + 1 < n_stage;
        x_ahead += more ? kStepK : 0;
        w_ahead += more ? w_step : 0;
        buf = buf_next;
    };
    for (int stage = 0; stage < n_stage; stage += 2) {
        step(std::integral_constant<int, 0>{}, stage);
        step(std::integral_constant<int, 1>{}, stage + 1);
    }
#undef VQ_FENCE
    // Drain the clamped loads still in flight before the stage buffers are reused.
    wait_vmcnt<0>();
    __syncthreads();
    // the last MFMAs must have left the pipe before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: lane holds Y[m = i*16 + r16][n = j*16 + 4*kg + 0..3] of its wave tile ----------
    auto round4 = [](const float4_t &a) { return half4_t{(half_t)a[0], (half_t)a[1], (half_t)a[2], (half_t)a[3]}; };
    if ((N & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0) {
        // Through the LDS: each wave transposes its fp16 block, 64 rows at a time, in a
        // private region (padded rows) and stores whole row segments.
        constexpr int kPitch = WN * 2 + 16;
        constexpr int kRowChunks = WN / 8, kRowsPerPass = 64 / kRowChunks;
        uint8_t *stage_out = smem + wave * (64 * kPitch);
#pragma unroll
        for (int h = 0; h < MP / 4; h++) {
#pragma unroll
            for (int ii = 0; ii < 4; ii++) {
                const int i = 4 * h + ii;
#pragma unroll
                for (int j = 0; j < NP; j++)
                    *reinterpret_cast<half4_t *>(stage_out + (ii * 16 + r16) * kPitch + (j * 16 + 4 * kg) * 2) = round4(acc[j][i]);
            }
#pragma unroll
            for (int it = 0; it < 64 / kRowsPerPass; it++) {
                const int row = it * kRowsPerPass + lane / kRowChunks, c = lane % kRowChunks;
                const uint4_t v = *reinterpret_cast<const uint4_t *>(stage_out + row * kPitch + c * 16);
                const int m = m0 + wm * WM + h * 64 + row;
                const int n = n0 + wn * WN + c * 8;
                if (m < M && n < N) st_global_16_streaming(y + (int64_t)m * N + n, v);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < MP; i++) {
            const int m = m0 + wm * WM + i * 16 + r16;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < NP; j++) {
                const int n = n0 + wn * WN + j * 16 + 4 * kg;
                half_t *dst = y + (int64_t)m * N + n;
                const half4_t hv = round4(acc[j][i]);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < N) dst[e] = hv[e];
            }
        }
    }
}

// ---- geometry A, fused ---------------------------------------------------------------------------
// out[M, 2*Nc] = X[M,K] . W_dec with W_dec[k, 2n + r] = codebook[n/4][w[k,n]][r] (reference
// strategy_2/bsz512/src.cu:163-176, bench.py:46-56): the vector lies along N, so a dequantised
// row of W is n-contiguous - the [K,N] layout of the kernel above.  This kernel is that kernel with
// the W part of a stage produced on the compute unit instead of loaded: the tile's codebooks (one
// per 8 output columns, 1 KB each) and the code bytes of the coming stages sit in the LDS, and while
// step s multiplies, every thread dequantises two 16-byte chunks of stage s+2 - four code bytes, four
// 4-byte gathers, one 16-byte write into the k-major W buffer - which the transposing reads of step
// s+1 then pick up.  This is the reference's own scheme (gather into a shared-memory tile, then
// fragment loads), with the gather running two steps ahead of the matrix cores instead of between
// two barriers.
//
// 256x128 tile (64 code columns, 16 codebooks), 128x64 per wave; or 128x128, 64x64 per wave, when
// the taller tiles are fewer than the compute units.  LDS: six X stages (96 or 48 KB), two W buffers
// (16 KB), the codebooks (16 KB), four code tiles of two stages each (16 KB).
constexpr int kANP = 4;
constexpr int kABN = 2 * kANP * 16, kAWN = kANP * 16;       // 128, 64
constexpr int kANSX = 6;                                     // X stages in the LDS
constexpr int kAWBytes = kABN * kStepK * 2;                  // one dequantised W stage: 8 KB
constexpr int kAChunksPerK = kABN / 8;                       // 16
constexpr int kACbBytes = kAChunksPerK * 1024;               // 16 codebooks of 256 entries x 2 halves
constexpr int kACodeRow = kABN / 2;                          // code bytes of one k-row of the tile: 64
constexpr int kACodeTile = 2 * kStepK * kACodeRow;           // the codes of two stages: 4 KB
constexpr int kANSC = 4;                                     // code tiles in the LDS
constexpr int kAXBase = 0;

// Tile height and, with it, the LDS layout and where in a step of 4*MPA MFMAs the other work goes.
template <int MPA>
struct FusedACfg {
    static constexpr int WM = MPA * 16, BM = 2 * WM;
    static constexpr int kXBytes = BM * kStepK * 2;              // X part of a stage: 16 or 8 KB
    static constexpr int kXLoads = kXBytes / (kThreads * 16);    // 4 or 2
    static constexpr int kWBase = kAXBase + kANSX * kXBytes;
    static constexpr int kCbBase = kWBase + 2 * kAWBytes;
    static constexpr int kCodeBase = kCbBase + kACbBytes;
    static constexpr size_t kLdsBytes = kCodeBase + kANSC * kACodeTile;
    // MFMA slots (an MFMA index m of the step; the instruction goes behind that MFMA)
    static constexpr int kCodeRead1 = MPA == 8 ? 2 : 1;          // second code read (the first is at 0)
    static constexpr int kGather0 = MPA == 8 ? 9 : 3;            // eight gathers from here on
    static constexpr int kWrite0 = MPA == 8 ? 24 : 12;           // two writes
    static constexpr int kXIssue0 = MPA == 8 ? 1 : 13, kXIssueGap = MPA == 8 ? 5 : 1;   // global loads of X
    // the code tile load of even steps: behind the step's last X load, as the counted waits of the main loop assume
    // (with the code tile between two X loads, the wait of an odd step let the last X load of the next stage
    // still be in flight)
    static constexpr int kCodeIssue = MPA == 8 ? 21 : 15;
    static_assert(kCodeIssue > kXIssue0 + (kXLoads - 1) * kXIssueGap && kCodeIssue < 4 * MPA, "code tile behind the X loads, inside the step");
    static_assert(kLdsBytes <= 160 * 1024, "the fused geometry-A kernel fits the LDS");
};

template <int MPA>
__global__ __launch_bounds__(kThreads, 1) void gemm_a_fused_kernel(const half_t *__restrict__ x,
                                                                   const uint8_t *__restrict__ codes,
                                                                   const half_t *__restrict__ cb,
                                                                   half_t *__restrict__ y, int M, int K, int Nc,
                                                                   int tiles_m, int tiles_n)
{
    // MPA 16-row pieces of X per wave: 8 makes the 256x128 tile, 4 a 128x128 tile for problems whose
    // larger tiles are fewer than the compute units (every thread then dequantises as much per half
    // as many MFMAs, and twice as many units work).
    static_assert(MPA == 8 || MPA == 4, "8 or 4 pieces of X per wave");
    typedef FusedACfg<MPA> A;
    constexpr int NP = kANP, WN = kAWN, BN = kABN;
    constexpr int MP = MPA, WM = A::WM, BM = A::BM, kXBytes = A::kXBytes, kXLoads = A::kXLoads;
    constexpr int kAWBase = A::kWBase, kACbBase = A::kCbBase, kACodeBase = A::kCodeBase;
    extern __shared__ __align__(16) uint8_t smem[];
    const int N = 2 * Nc;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int r16 = lane & 15, kg = lane >> 4;

    int wg = blockIdx.x;
    const int n_wg = tiles_m * tiles_n;
    if ((n_wg & 7) == 0) wg = (wg & 7) * (n_wg >> 3) + (wg >> 3);
    const int tm = wg / tiles_n, tn = wg % tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    const int n_stage = K / kStepK, n_pair = n_stage / 2;

    // ---- staging: global -> LDS ---------------------------------------------------------------
    uint32_t x_voff[kXLoads];
#pragma unroll
    for (int i = 0; i < kXLoads; i++) {
        const int slot = (4 * i + wave) * 64 + lane;
        const int bank_row = slot >> 4;
        const int pos = (slot & 15) ^ (bank_row & 3);
        const int row = 4 * bank_row + (pos >> 2), cc = pos & 3;
        x_voff[i] = (uint32_t)(((int64_t)(min(m0 + row, M - 1) - m0) * K + cc * 8) * 2);
    }
    // A code tile is 64 k-rows x 64 code bytes, row-major; thread t fetches 16-byte piece t%4 of row
    // t/4 (columns past Nc: the last 16 columns again).
    const uint8_t *code_tile = codes + n0 / 2;
    const uint32_t code_voff = (uint32_t)((int64_t)(tid >> 2) * Nc + (min(n0 / 2 + (tid & 3) * 16, Nc - 16) - n0 / 2));
    const int64_t pair_step = (int64_t)2 * kStepK * Nc;
    const half_t *x_tile = x + (int64_t)m0 * K;
    auto issue_x = [&](int i, int buf, const half_t *xb) {
        load_to_lds_16(kAXBase + buf * kXBytes + (4 * i + wave) * 1024, x_voff[i], xb);
    };
    auto issue_codes = [&](int cbuf, const uint8_t *cbase) {
        load_to_lds_16(kACodeBase + cbuf * kACodeTile + wave * 1024, code_voff, cbase);
    };
    // what the loads issued during the current step read; moved on once per step / pair of steps
    const half_t *x_ahead = x_tile + min(kANSX, n_stage - 1) * kStepK;
    const uint8_t *c_ahead = code_tile + min(kANSC, n_pair - 1) * pair_step;

    float4_t acc[NP][MP];
#pragma unroll
    for (int j = 0; j < NP; j++)
#pragma unroll
        for (int i = 0; i < MP; i++) acc[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};

    // ---- operand reads (as in the plain kernel, W from its own two buffers) ----------------------
    const int x_rd = kAXBase + row_offset(wm * WM + r16, kg);
    int w_rd[NP];
    {
        const int k = kg * 8 + (r16 >> 2);
#pragma unroll
        for (int j = 0; j < NP; j++) {
            const int chunk = (wn * (WN / 8) + 2 * j + ((r16 & 3) >> 1)) ^ kmajor_swizzle(k);
            w_rd[j] = kAWBase + (k * kAChunksPerK + chunk) * 16 + (r16 & 1) * 8;
        }
    }
    half8_t xs[2][MP];
    half4_t wlo[2][NP], whi[2][NP];
    auto load_x = [&](int set, int i, int buf) {
        xs[set][i] = *reinterpret_cast<const half8_t *>(smem + buf * kXBytes + x_rd + i * 1024);
    };
    auto load_w = [&](int set, int j, int h, int wbuf) {
        typedef __attribute__((address_space(3))) short4_t lds_short4_t;
        const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4_t *)(smem + wbuf * kAWBytes + w_rd[j] + h * (4 * kAChunksPerK * 16)));
        if (h == 0) wlo[set][j] = __builtin_bit_cast(half4_t, v);
        else whi[set][j] = __builtin_bit_cast(half4_t, v);
    };

    // ---- dequantisation: thread t builds chunk c = t%16 of k-rows t/16 and t/16 + 16 of a stage --------
    // Chunk c (8 output columns = 4 code columns) uses codebook c of the tile.
    const int dq_c = tid & 15, dq_k = tid >> 4;
    const uint32_t dq_codes = kACodeBase + dq_k * kACodeRow + dq_c * 4;   // + code tile, + stage parity * 32 rows, + u * 16 rows
    const uint32_t dq_book = kACbBase + dq_c * 1024;
    const uint32_t dq_out = kAWBase + (dq_k * kAChunksPerK + (dq_c ^ kmajor_swizzle(dq_k))) * 16;  // + W buffer, + u * 16 rows
    uint32_t dq_code[2];
    uint4_t dq_val[2];
    auto dq_read_codes = [&](int u, int cbuf, int par) {
        dq_code[u] = *reinterpret_cast<const uint32_t *>(smem + dq_codes + cbuf * kACodeTile + (par * 32 + u * 16) * kACodeRow);
    };
    auto dq_gather = [&](int u, int b) {
        const uint32_t code = (dq_code[u] >> (8 * b)) & 0xffu;
        dq_val[u][b] = *reinterpret_cast<const uint32_t *>(smem + dq_book + code * 4);
    };
    auto dq_write = [&](int u, int wbuf) {
        *reinterpret_cast<uint4_t *>(smem + dq_out + wbuf * kAWBytes + u * 16 * kAChunksPerK * 16) = dq_val[u];
    };

    // ---- prologue -----------------------------------------------------------------------------
    // Loads complete in the order they were issued, so one count serves all of them.  The order is
    // the one the main loop would have issued them in (X stage s at step s-6, the code tile of
    // stages 2q, 2q+1 at step 2q-8, behind that step's X loads), with the codebooks in front.
    {
        const int g0 = n0 / 8;                       // first codebook of the tile
        const int avail = (Nc / 4 - g0) * 1024 - 16;  // last valid 16-byte piece behind it
        const uint8_t *src = reinterpret_cast<const uint8_t *>(cb) + (int64_t)g0 * 1024;
#pragma unroll
        for (int i = 0; i < kACbBytes / (kThreads * 16); i++) {
            const int byte = ((4 * i + wave) * 64 + lane) * 16;
            load_to_lds_16(kACbBase + (4 * i + wave) * 1024, (uint32_t)min(byte, avail), src);
        }
    }
    auto x_stage = [&](int st) { return x_tile + min(st, n_stage - 1) * kStepK; };
    auto c_pair = [&](int q) { return code_tile + min(q, n_pair - 1) * pair_step; };
    issue_codes(0, c_pair(0));
#pragma unroll
    for (int i = 0; i < kXLoads; i++) issue_x(i, 0, x_stage(0));
    issue_codes(1, c_pair(1));
#pragma unroll
    for (int i = 0; i < kXLoads; i++) issue_x(i, 1, x_stage(1));
#pragma unroll
    for (int i = 0; i < kXLoads; i++) issue_x(i, 2, x_stage(2));
    issue_codes(2, c_pair(2));
#pragma unroll
    for (int i = 0; i < kXLoads; i++) issue_x(i, 3, x_stage(3));
#pragma unroll
    for (int i = 0; i < kXLoads; i++) issue_x(i, 4, x_stage(4));
    issue_codes(3, c_pair(3));
#pragma unroll
    for (int i = 0; i < kXLoads; i++) issue_x(i, 5, x_stage(5));
    wait_vmcnt<4 * kXLoads + 2>();  // the codebooks, code tiles 0 and 1, X stages 0 and 1 have landed
    __syncthreads();
    // W of stages 0 and 1 from code tile 0
#pragma unroll
    for (int st = 0; st < 2; st++) {
#pragma unroll
        for (int u = 0; u < 2; u++) dq_read_codes(u, 0, st);
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int b = 0; b < 4; b++) dq_gather(u, b);
#pragma unroll
        for (int u = 0; u < 2; u++) dq_write(u, st);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MP; i++) load_x(0, i, 0);
#pragma unroll
    for (int j = 0; j < NP; j++) {
        load_w(0, j, 0, 0);
        load_w(0, j, 1, 0);
    }

    // ---- main loop ----------------------------------------------------------------------------
    // Step `stage` (parity `set`) multiplies register set `set`, reads the operands of stage+1 (X
    // buffer xbuf+1, W buffer set^1), dequantises stage+2 into W buffer `set` out of code tile cq
    // (the tile of stages stage+2 and its partner), and issues the X loads of stage+6 into the X
    // buffer it multiplies from; even steps also issue the code tile four tiles ahead of cq.
#define VQ_FENCE __builtin_amdgcn_sched_barrier(0)
    int xbuf = 0;  // X buffer of the current stage
    int cq = 1;    // code tile buffer of stage + 2
    auto step = [&](auto set_const, int stage) {
        constexpr int set = decltype(set_const)::value;
        const int xbuf_next = xbuf + 1 == kANSX ? 0 : xbuf + 1;
        // X of stage+1 and the code tile of stage+2 have landed when only what was issued behind
        // them is in flight: four X stages and the code tiles of the even steps among them.
        wait_vmcnt<4 * kXLoads + (set == 0 ? 2 : 3)>();
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __syncthreads();
        VQ_FENCE;
#pragma unroll
        for (int m = 0; m < NP * MP; m++) {
            const int q = m >> 4, p = (m >> 2) & 3, f = m & 3;
            const int j = p, i = q * 4 + f;
            mfma_in_place(acc[j][i], __builtin_shufflevector(wlo[set][j], whi[set][j], 0, 1, 2, 3, 4, 5, 6, 7),
                          xs[set][i]);
            VQ_FENCE;
            // Between the MFMAs: the operand reads of stage+1 (X, then W in halves), the dequantisation
            // of stage+2 (code bytes first, the gathers a good LDS latency behind them, the writes a
            // good LDS latency behind the gathers and ahead of the step's end), the global loads.
            if (m < MP) {
                load_x(set ^ 1, m, xbuf_next);
                VQ_FENCE;
            } else if (m < MP + 2 * NP) {
                load_w(set ^ 1, (m - MP) >> 1, (m - MP) & 1, set ^ 1);
                VQ_FENCE;
            }
            if (m == 0 || m == A::kCodeRead1) {
                dq_read_codes(m == 0 ? 0 : 1, cq, set);
                VQ_FENCE;
            }
            if (m >= A::kGather0 && m < A::kGather0 + 8) {
                dq_gather((m - A::kGather0) >> 2, (m - A::kGather0) & 3);
                VQ_FENCE;
            }
            if (m == A::kWrite0 || m == A::kWrite0 + 1) {
                dq_write(m - A::kWrite0, set);
                VQ_FENCE;
            }
            if (m >= A::kXIssue0 && (m - A::kXIssue0) % A::kXIssueGap == 0 && (m - A::kXIssue0) / A::kXIssueGap < kXLoads) {
                issue_x((m - A::kXIssue0) / A::kXIssueGap, xbuf, x_ahead);
                VQ_FENCE;
            }
            if (set == 0 && m == A::kCodeIssue) {
                issue_codes(cq == 0 ? kANSC - 1 : cq - 1, c_ahead);
                VQ_FENCE;
            }
        }
        x_ahead += stage + kANSX + 1 < n_stage ? kStepK : 0;
        if (set == 1) {
            c_ahead += (stage >> 1) + kANSC + 1 < n_pair ? pair_step : 0;
            cq = cq + 1 == kANSC ? 0 : cq + 1;
        }
        xbuf = xbuf_next;
    };
    for (int stage = 0; stage < n_stage; stage += 2) {
        step(std::integral_constant<int, 0>{}, stage);
        step(std::integral_constant<int, 1>{}, stage + 1);
    }
#undef VQ_FENCE
    wait_vmcnt<0>();
    __syncthreads();
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: lane holds Y[m = i*16 + r16][n = j*16 + 4*kg + 0..3] of its wave tile ----------
    auto round4 = [](const float4_t &a) { return half4_t{(half_t)a[0], (half_t)a[1], (half_t)a[2], (half_t)a[3]}; };
    if ((reinterpret_cast<uintptr_t>(y) & 15) == 0) {
        constexpr int kPitch = WN * 2 + 16;
        constexpr int kRowChunks = WN / 8, kRowsPerPass = 64 / kRowChunks;
        uint8_t *stage_out = smem + wave * (64 * kPitch);
#pragma unroll
        for (int h = 0; h < MP / 4; h++) {
#pragma unroll
            for (int ii = 0; ii < 4; ii++) {
                const int i = 4 * h + ii;
#pragma unroll
                for (int j = 0; j < NP; j++)
                    *reinterpret_cast<half4_t *>(stage_out + (ii * 16 + r16) * kPitch + (j * 16 + 4 * kg) * 2) = round4(acc[j][i]);
            }
#pragma unroll
            for (int it = 0; it < 64 / kRowsPerPass; it++) {
                const int row = it * kRowsPerPass + lane / kRowChunks, c = lane % kRowChunks;
                const uint4_t v = *reinterpret_cast<const uint4_t *>(stage_out + row * kPitch + c * 16);
                const int m = m0 + wm * WM + h * 64 + row;
                const int n = n0 + wn * WN + c * 8;
                if (m < M && n < N) st_global_16_streaming(y + (int64_t)m * N + n, v);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < MP; i++) {
            const int m = m0 + wm * WM + i * 16 + r16;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < NP; j++) {
                const int n = n0 + wn * WN + j * 16 + 4 * kg;
                half_t *dst = y + (int64_t)m * N + n;
                const half4_t hv = round4(acc[j][i]);
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < N) dst[e] = hv[e];
            }
        }
    }
}

template <bool W_IS_KN, int NP, int MPW>
hipError_t launch_tiled(const half_t *x, const half_t *w, half_t *y, int M, int K, int N, hipStream_t s)
{
    typedef TileCfg<NP, MPW> C;
    const int tiles_m = (M + C::BM - 1) / C::BM, tiles_n = (N + C::BN - 1) / C::BN;
    auto kern = gemm_tiled_kernel<W_IS_KN, NP, MPW>;
    const hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), C::kLdsBytes);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(kThreads), C::kLdsBytes, s, x, w, y, M, K, N,
                       tiles_m, tiles_n);
    return hipGetLastError();
}

}  // namespace

// K in whole pairs of stages, 16-byte aligned operands and rows, lane offsets within 32 bits.
bool gemm_tiled_supports(const half_t *x, const half_t *w, int M, int K, int N, bool w_is_kn)
{
    if (M < 1 || N < 1 || K < 2 * kStepK || K % (2 * kStepK) != 0) return false;
    if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(w) & 15) != 0) return false;
    if (w_is_kn && (N % 8 != 0 || (int64_t)kStepK * N * 2 >= (int64_t)1 << 31)) return false;
    return (int64_t)BM * K * 2 < (int64_t)1 << 31;
}

// tile: 0 = the tile expected to be fastest, 1 = 256x256, 2 = 256x128, 3 = 128x128
hipError_t launch_gemm_tiled(const half_t *x, const half_t *w, half_t *y, int M, int K, int N, bool w_is_kn, hipStream_t s,
                             int tile)
{
    if (!gemm_tiled_supports(x, w, M, K, N, w_is_kn)) return hipErrorInvalidValue;
    if (tile == 0) {
        // Rounds of tiles over the compute units.  A tile costs K/64 times a per-stage time that
        // grows with the share of the units at work (the clock drops under load): fitted to
        // measurements, 1.2 us for the 256x256 tile, 0.68 us for 256x128 and 0.40 us for 128x128 on
        // an idle device, 1.6 times that on a full one.
        const int cus = device_cu_count();
        auto cost = [&](int bm, int bn, double per_stage) {
            const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
            const int64_t rounds = (tiles + cus - 1) / cus;
            const double busy = (double)tiles / (double)(rounds * cus);
            return (double)rounds * (5.0 + K / 64.0 * per_stage * (1.0 + 0.6 * busy));
        };
        const double t1 = cost(256, 256, 1.2), t2 = cost(256, 128, 0.68), t3 = cost(128, 128, 0.40);
        tile = t3 < t2 && t3 < t1 ? 3 : (t2 < t1 ? 2 : 1);
    }
    if (tile == 3) return w_is_kn ? launch_tiled<true, 4, 4>(x, w, y, M, K, N, s) : launch_tiled<false, 4, 4>(x, w, y, M, K, N, s);
    if (tile == 2) return w_is_kn ? launch_tiled<true, 4, 8>(x, w, y, M, K, N, s) : launch_tiled<false, 4, 8>(x, w, y, M, K, N, s);
    return w_is_kn ? launch_tiled<true, 8, 8>(x, w, y, M, K, N, s) : launch_tiled<false, 8, 8>(x, w, y, M, K, N, s);
}

// Nc in whole 16-byte pieces of code bytes, K in whole pairs of stages, 16-byte aligned operands.
bool fused_a_supports(const ProblemA &p)
{
    if (p.M < 1 || p.Nc < 16 || p.Nc % 16 != 0 || p.K < 2 * kStepK || p.K % (2 * kStepK) != 0) return false;
    if ((reinterpret_cast<uintptr_t>(p.x) & 15) != 0 || (reinterpret_cast<uintptr_t>(p.w) & 15) != 0 ||
        (reinterpret_cast<uintptr_t>(p.cb) & 15) != 0)
        return false;
    return (int64_t)BM * p.K * 2 < (int64_t)1 << 31 && (int64_t)2 * kStepK * p.Nc < (int64_t)1 << 31;
}

hipError_t launch_fused_a(const ProblemA &p, hipStream_t s)
{
    if (!fused_a_supports(p)) return hipErrorInvalidValue;
    const int tiles_n = (2 * p.Nc + kABN - 1) / kABN;
    // 256x128 tiles, or 128x128 where those go over the compute units in fewer rounds at four fifths of the
    // time per round (measured at one round each: 48 against 60 us per 4096 k)
    const int cus = device_cu_count();
    const int64_t n_tall = (int64_t)((p.M + 255) / 256) * tiles_n, n_short = (int64_t)((p.M + 127) / 128) * tiles_n;
    const bool tall = (double)((n_tall + cus - 1) / cus) <= 0.8 * (double)((n_short + cus - 1) / cus);
    auto launch = [&](auto kern, int bm, size_t lds) {
        const int tiles_m = (p.M + bm - 1) / bm;
        const hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n)), dim3(kThreads), lds, s, p.x, p.w, p.cb, p.y, p.M, p.K,
                           p.Nc, tiles_m, tiles_n);
        return hipGetLastError();
    };
    return tall ? launch(gemm_a_fused_kernel<8>, 256, FusedACfg<8>::kLdsBytes) : launch(gemm_a_fused_kernel<4>, 128, FusedACfg<4>::kLdsBytes);
}

}  // namespace vq
