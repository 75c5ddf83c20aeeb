// Decode GEMV proper (one to four rows of X): y[m,n] = sum_k x[m,k] W[n,k], W given as codes and a
// codebook (described below for 8-bit codes of 8-vectors; GemvCfg holds what changes with the
// format).  A short launch of this path is a chain of latencies, not a stream, so the kernel is
// built to keep the chain short rather than to share work:
//
//   * A wave owns whole rows of W (four of them), so nothing is summed across waves: no partial
//     sums in the LDS, no barrier behind the multiply.  A row's sum is folded inside the wave with
//     DPP adds and four lane reads.
//   * No matrix core: with one row of X fifteen of an MFMA's sixteen columns would be padding, and
//     feeding it means laying X out in operand order through the LDS first.  Here a lane keeps
//     its share of x (the 8-vectors its codes meet) in registers, loaded straight from global
//     memory while the codes are on their way, and multiplies with v_dot2_f32_f16: four per code.
//   * Lane l takes the codes 4l..4l+3 of every run of 256 codes: one dword load per row and run
//     (a wave reads 256 contiguous bytes), x in 64-byte pieces per lane.
//   * The only barrier publishes the codebook (4 KB, one 16-byte entry per thread) in the LDS; the
//     gathers are 16-byte reads at code*16.  The codebook's load is the first one issued, so that
//     its copy and the barrier pass while the codes are still on their way from HBM.
//
// Four waves per workgroup, 16 rows of W: as many workgroups as the batched kernel has tiles.  It
// serves two to four rows of X and the other code formats; one row of X in the first format goes to
// the wide form below (decode_gemv_wide_kernel) at any N (Tuning::gemv_wide_min_rows_per_wave = 0:
// with its single-group instance the wide form is ahead from N = 256 on, cold, K = 4096: 2.55
// against 2.76 us; N = 2048: 2.71 against 2.98; K = 8192, N = 1024: 3.29 against 3.93), and so do
// two rows of X (K up to 16384) while a wave has few enough rows.
#include "vq_common.h"

#include <limits.h>
#include <type_traits>

namespace vq {

namespace {

constexpr int kGemvWaves = 4;
constexpr int kGemvRows = 4;                                // rows of W per wave
typedef _Float16 gemv_out_t __attribute__((ext_vector_type(kGemvRows)));
constexpr int kGemvTile = kGemvWaves * kGemvRows;           // rows of W per workgroup
constexpr int kRunCodes = 256;                              // codes of a row one wave load covers
constexpr int kRunK = kRunCodes * 8;                        // 2048 k
constexpr int kGemvMaxRuns = 4;                             // x stays in registers: 16 per run and row of X,
constexpr int kGemvMaxXRegs = 128;                          // at most this many in all

__device__ __forceinline__ float dpp_add_quad_perm_1032(float v)
{
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xb1, 0xf, 0xf, false));
}
__device__ __forceinline__ float dpp_add_quad_perm_2301(float v)
{
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4e, 0xf, 0xf, false));
}
__device__ __forceinline__ float dpp_add_row_half_mirror(float v)
{
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));
}
__device__ __forceinline__ float dpp_add_row_mirror(float v)
{
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));
}

// Sum of v over the 64 lanes, the same value in every lane: four DPP steps leave each row of 16
// lanes with its own sum, the four row sums are read out by lane and added in a fixed order.
__device__ __forceinline__ float wave_sum(float v)
{
    v = dpp_add_quad_perm_1032(v);
    v = dpp_add_quad_perm_2301(v);
    v = dpp_add_row_half_mirror(v);
    v = dpp_add_row_mirror(v);
    const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (r0 + r1) + (r2 + r3);
}

// Format of the codes: a lane takes the 32 / VEC codes that meet 32 consecutive halves of x in every
// run of 2048 k, as one load of 4, 8 or 16 bytes.
template <int VEC, typename CodeT>
struct GemvCfg {
    static constexpr int CPR = 32 / VEC;                      // codes per lane and run
    static constexpr int CW = CPR * (int)sizeof(CodeT) / 4;   // dwords per lane and run
    static constexpr int kMaxEntries = sizeof(CodeT) == 1 ? 256 : 4096;
    static constexpr int kTableBytes = kMaxEntries * VEC * 2;
    static_assert(CW == 1 || CW == 2 || CW == 4, "one load of 4, 8 or 16 bytes");
    static_assert(kTableBytes <= 64 * 1024, "the table is a static LDS array");
};

// RUNS: runs of 2048 k in a row of W; MX: rows of X (each gathered codeword meets MX shares of x).
// GATED: the epilogue of a gate/up pair (rows of W interleaved in groups of 16: rows 32g .. 32g+15 gate, the
// sixteen behind them the up rows of the same outputs).  A workgroup's sixteen code rows are then the gate and the
// up rows of eight outputs, a wave's four the pairs of two outputs - rows 0 and 1 the gate rows, 2 and 3 the up
// rows - and y is [M, N/2].
template <int VEC, typename CodeT, int RUNS, int MX, bool GATED>
__global__ __launch_bounds__(kGemvWaves * 64) void decode_gemv_kernel(const half_t *__restrict__ x,
                                                                       const CodeT *__restrict__ codes,
                                                                       const half_t *__restrict__ cb,
                                                                       half_t *__restrict__ y,
                                                                       const half_t *__restrict__ bias, int K,
                                                                       int N, int entries, int rows_per_cb)
{
    static_assert(!GATED || kGemvRows == 4, "a wave's rows are two gate/up pairs");
    typedef GemvCfg<VEC, CodeT> C;
    typedef uint32_t words_t __attribute__((ext_vector_type(C::CW)));
    __shared__ __align__(16) uint4_t table[C::kTableBytes / 16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // plain: the wave's rows are row0 .. row0+3.  GATED: out0 is the first of its two outputs, its code rows the
    // gate rows of out0 and out0+1 (neighbours inside one group of 16) and the up rows 16 further on.
    const int out0 = blockIdx.x * (kGemvTile / 2) + wave * (kGemvRows / 2);
    const int row0 = GATED ? 32 * (out0 >> 4) + (out0 & 15) : blockIdx.x * kGemvTile + wave * kGemvRows;
    auto code_row = [&](int r) { return GATED ? row0 + (r & 1) + 16 * (r >> 1) : row0 + r; };
    constexpr int J = RUNS * 64 * C::CPR;  // codes per row

    // The table's load goes out first and is the first to be back (it comes out of the L2): its copy
    // into the LDS and the barrier then pass while the codes (HBM) and x are still on their way.
    // (no division in front of the first load when there is one codebook)
    // (GATED: the workgroup's rows lie inside one group of 32, and a codebook holds whole groups)
    const int book = rows_per_cb >= N ? 0 : (GATED ? 32 * ((blockIdx.x * (kGemvTile / 2)) >> 4) : blockIdx.x * kGemvTile) / rows_per_cb;
    // (entries * VEC * 2 is a multiple of 16, so every codebook starts on a 16-byte boundary)
    const int chunks = entries * VEC * 2 / 16;
    const uint4_t *tsrc = reinterpret_cast<const uint4_t *>(cb + (int64_t)book * entries * VEC);
    uint4_t t0 = {0u, 0u, 0u, 0u};
    if ((int)threadIdx.x < chunks) t0 = tsrc[threadIdx.x];
    uint32_t cw[kGemvRows][RUNS][C::CW];
#pragma unroll
    for (int r = 0; r < kGemvRows; r++)
#pragma unroll
        for (int q = 0; q < RUNS; q++) {
            const words_t v = *reinterpret_cast<const words_t *>(codes + (int64_t)code_row(r) * J + (q * 64 + lane) * C::CPR);
#pragma unroll
            for (int i = 0; i < C::CW; i++) cw[r][q][i] = v[i];
        }
    uint32_t xr[MX][RUNS][16];  // the lane's 32 halves of x per run and row of X
#pragma unroll
    for (int m = 0; m < MX; m++)
#pragma unroll
        for (int q = 0; q < RUNS; q++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint4_t v = *reinterpret_cast<const uint4_t *>(x + (int64_t)m * K + ((q * 64 + lane) * 4 + c) * 8);
#pragma unroll
                for (int d = 0; d < 4; d++) xr[m][q][4 * c + d] = v[d];
            }
    // 8-bit codes: the whole table is written, zeros past a short codebook, so that a code at or past
    // `entries` gathers a defined value (16-bit codes can point past any table: the LDS returns zero
    // for reads outside the allocation, and short tables of that format are left as they are).
    constexpr int kSlots = C::kTableBytes / 16;
    static_assert(sizeof(CodeT) != 1 || kSlots <= kGemvWaves * 64, "one slot per thread covers a table of 8-bit codes");
    if ((int)threadIdx.x < (sizeof(CodeT) == 1 ? kSlots : chunks)) table[threadIdx.x] = t0;
    for (int i = threadIdx.x + kGemvWaves * 64; i < chunks; i += kGemvWaves * 64) table[i] = tsrc[i];
    __syncthreads();

    float acc[MX][kGemvRows];
#pragma unroll
    for (int m = 0; m < MX; m++)
#pragma unroll
        for (int r = 0; r < kGemvRows; r++) acc[m][r] = 0.f;
    const uint8_t *tbl = reinterpret_cast<const uint8_t *>(table);
#pragma unroll
    for (int q = 0; q < RUNS; q++)
#pragma unroll
        for (int c = 0; c < C::CPR; c++)
#pragma unroll
            for (int r = 0; r < kGemvRows; r++) {
                uint32_t code;
                if constexpr (sizeof(CodeT) == 1) code = (cw[r][q][c >> 2] >> (8 * (c & 3))) & 0xffu;
                else code = (cw[r][q][c >> 1] >> (16 * (c & 1))) & 0xffffu;
                // the codeword: VEC halves = VEC / 2 words
                uint32_t w[VEC / 2];
                if constexpr (VEC == 8) {
                    const uint4_t v = *reinterpret_cast<const uint4_t *>(tbl + code * 16);
#pragma unroll
                    for (int d = 0; d < 4; d++) w[d] = v[d];
                } else if constexpr (VEC == 4) {
                    const uint2_t v = *reinterpret_cast<const uint2_t *>(tbl + code * 8);
                    w[0] = v[0];
                    w[1] = v[1];
                } else {
                    w[0] = *reinterpret_cast<const uint32_t *>(tbl + code * 4);
                }
#pragma unroll
                for (int m = 0; m < MX; m++)
#pragma unroll
                    for (int d = 0; d < VEC / 2; d++) {
                        // (through scalars: a bit cast applied to a vector element reads element 0)
                        const uint32_t wd = w[d], xd = xr[m][q][c * (VEC / 2) + d];
                        acc[m][r] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, wd), __builtin_bit_cast(half2_t, xd),
                                                           acc[m][r], false);
                    }
            }
#pragma unroll
    for (int m = 0; m < MX; m++) {
        float sum[kGemvRows];
#pragma unroll
        for (int r = 0; r < kGemvRows; r++) {
            sum[r] = wave_sum(acc[m][r]);
            if (bias) sum[r] += (float)bias[code_row(r)];
        }
        if constexpr (GATED) {
            // outputs out0 and out0+1: silu(gate) * up, one rounding
            half2_t out;
#pragma unroll
            for (int j = 0; j < 2; j++) out[j] = (half_t)(silu_f32(sum[j]) * sum[2 + j]);
            if (lane == 0) *reinterpret_cast<half2_t *>(y + (int64_t)m * (N / 2) + out0) = out;
        } else {
            gemv_out_t out;
#pragma unroll
            for (int r = 0; r < kGemvRows; r++) out[r] = (half_t)sum[r];
            if (lane == 0) *reinterpret_cast<gemv_out_t *>(y + (int64_t)m * N + row0) = out;
        }
    }
}

// ---- the wide form: long runs of rows, long rows, and every launch of one or two rows of X in the first format -------
// One workgroup of sixteen waves per compute unit over a bank-replicated table (64 KB: 16 copies of
// each entry in one 256-byte bank row, lane l reading copy l % 16, so the gathers never collide):
// four waves per SIMD cover the latency of each other's gathers.  One or two rows of X, 8-vectors, 8-bit codes.
//   * The rows of W are dealt out to the waves of the whole grid in contiguous runs of equal length
//     (one more for the first N % waves), so no unit idles while another finishes a longer share.
//     A workgroup's rows may reach into a second codebook: it then holds two tables (128 KB) and a
//     row picks its table through the third byte of the gather address.
//   * x goes through the LDS once per workgroup (4 to 16 KB, laid out so that a wave reads its 16-byte
//     pieces side by side): sixteen waves each pulling all of x through the L1 would cost more than
//     the table.
//   * A wave works through its rows in groups of G, the codes of the next NBUF - 1 groups already
//     requested.  The loop holds no store: a wave keeps the result of its i-th row in lane i (at most
//     64 rows per wave) and writes them all at the end, so the only outstanding vector-memory operations inside the loop
//     are the code loads, they complete in order, and the compiler's own wait counts stay exact (a
//     pending store would make it drain every load).  The loads are unconditional (past the end the
//     last group is requested again) and only the multiply is skipped, for the same reason: a load
//     inside a branch would make the counts at the join imprecise.
//   * A row's sum is folded with six DPP additions (the last two broadcast row totals onward, so that
//     lane 63 holds the sum in a fixed order) and one lane read.
constexpr int kWideWaves = 16;
constexpr int kWideCopies = 16;
constexpr int kWideTableBytes = 256 * kWideCopies * 16;  // 64 KB

// (One instruction each: the rows the mask leaves out keep their value, which the compiler does not
// express through the builtin.  The s_nop covers the two wait states a DPP read needs behind a VALU write.)
__device__ __forceinline__ float dpp_add_row_bcast15(float v)
{
    // lane 15 of rows 0 and 2 is added to every lane of rows 1 and 3
    asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf" : "+v"(v));
    return v;
}
__device__ __forceinline__ float dpp_add_row_bcast31(float v)
{
    // lane 31 is added to every lane of rows 2 and 3
    asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf" : "+v"(v));
    return v;
}

// Sum of v over the 64 lanes, valid in lane 63 (returned from there as a wave-uniform value).
__device__ __forceinline__ float wave_sum_to_uniform(float v)
{
    v = dpp_add_quad_perm_1032(v);
    v = dpp_add_quad_perm_2301(v);
    v = dpp_add_row_half_mirror(v);
    v = dpp_add_row_mirror(v);
    v = dpp_add_row_bcast15(v);
    v = dpp_add_row_bcast31(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// floor(x / d) for 0 <= x < 2^23 or so through a float reciprocal and one correction step; rcp = 1.0f / d.
__device__ __forceinline__ int small_quotient(int x, int d, float rcp)
{
    int q = (int)((float)x * rcp);
    const int rem = x - q * d;
    q += rem >= d ? 1 : 0;
    q -= rem < 0 ? 1 : 0;
    return q;
}

// BOOKS: 0 = one codebook; 1 = several, no workgroup's rows reach into a second one; 2 = some workgroup's rows
// do, and every workgroup then fills two tables.  (A compile-time flag, like the unconditional loads below: a
// load inside a branch makes the compiler's wait counts at the join imprecise, and the table would then
// wait for the codes.)
//
// The order of the prologue matters more than its length suggests.  Loads complete in the order they were
// issued, so what is issued behind the code loads (which come from HBM) is only usable once they have
// landed: the table entry and the piece of x (both out of the L2) go out first, the code loads right
// behind them.  And a launch starts with a cold instruction cache, so every instruction ahead of these
// loads delays the one wait that cannot be shortened: nothing is computed ahead of them that they do not need.
//
// COPIES: 16 = the bank-replicated table (conflict-free gathers; 64 KB to fill), 1 = the plain 4 KB table (a wave
// with one or two rows gathers too little for the fill of the replicated table to pay).
//
// XM: rows of X (1 or 2).  With two, a lane keeps its shares of both rows in registers (RUNS <= 2), every gathered
// codeword is multiplied with both, and a wave folds and keeps two sums per row of W (cold, M = 2, K = 4096, the
// K-sliced matrix-core kernel -> this: N = 11008 7.2 -> 5.3 us, N = 28672 10.5 -> 8.7).  K beyond 4096 is the long
// form in pieces of two runs, both rows of x in the LDS (K = 14336, N = 4096: 10.9 -> 8.5 us).
//
// XRUNS: runs of 2048 k of x that the LDS holds.  XRUNS == RUNS is the form described so far (K = RUNS * 2048, all of a
// lane's x in registers).  XRUNS > RUNS is the form for a longer K, or one that is no multiple of 2048 (the
// down-projection of an MLP: K = 11008, 14336, 28672): a row is cut into pieces of RUNS runs, a wave goes through
// its rows once per piece with that piece's x in its registers (read from the LDS again at every change of piece),
// and a row's sum so far travels in its lane of `res`: the accumulator of lane 0 starts from it.  x is padded with
// zeros up to whole pieces, and a load that would reach past the end of a row reads the row's last dword instead: what
// it gathers meets zeros.  One codebook, or several without a workgroup whose rows reach into two; not gated.
template <int RUNS, int G, int NBUF, int BOOKS, int COPIES, int XRUNS = RUNS, int XM = 1>
__global__ __launch_bounds__(kWideWaves * 64) void decode_gemv_wide_kernel(const half_t *__restrict__ x,
                                                                           const uint8_t *__restrict__ codes,
                                                                           const half_t *__restrict__ cb, int entries,
                                                                           int rows_q, int rows_r, int n_total,
                                                                           int gated_row_bytes, int rows_per_cb,
                                                                           float rcp_rows_per_cb, int n_books,
                                                                           const half_t *__restrict__ bias,
                                                                           half_t *__restrict__ y, int rotate_priority)
{
    // (The order of the arguments is the order in which the kernel needs them: the build preloads the first fourteen
    // dwords of a kernel's arguments into scalar registers at wave launch, -amdgpu-kernarg-preload-count, and what the
    // first loads need - x, the codes, the codebook and the numbers the wave's rows follow from - lies inside them, so
    // that no wave waits for an argument fetch ahead of its first load.)
    // gated: the epilogue of a gate/up pair.  The rows of W are gate and up rows interleaved in groups of 16; what
    // is dealt out to the waves (rows_q, rows_r, n_total) are then the N/2 outputs, a wave's code rows are the gate
    // and the up row of each of its outputs in turn; a group of two rows is one output (G = 2), or the gate row and the
    // up row are two groups in turn (G = 1).
    // gated_row_bytes: bit 31 = gated, below it the bytes of a row of codes (K / 8; read by the long form only) - one
    // argument, so that everything the prologue needs stays inside the preloaded fourteen dwords.
    constexpr bool TWO = BOOKS == 2;
    constexpr bool LONG = XRUNS != RUNS;
    static_assert(!LONG || (BOOKS < 2 && COPIES == kWideCopies && NBUF == 2), "the long form: one table, replicated");
    static_assert(NBUF > 1 || G == 1, "a single group per wave: of one row");
    static_assert(XM == 1 || (XM == 2 && RUNS <= 2), "two rows of X: both in the lane's registers, 4096 k of each at a time");
    const int gated = LONG ? 0 : (gated_row_bytes < 0 ? 1 : 0);
    constexpr int kXChunks = XRUNS * kRunCodes;  // 16-byte pieces of x
    // table of the first codebook (at LDS address 0: a gather address is used as it comes out of the byte
    // permute) | table of the second one (TWO) | x
    static_assert(COPIES == kWideCopies || COPIES == 1, "replicated or plain table");
    constexpr int kTableSlots = (TWO ? 2 : 1) * 256 * COPIES;
    __shared__ __align__(16) uint4_t lds[kTableSlots + XM * kXChunks];
    uint4_t *table = lds, *xs = lds + kTableSlots;
    const int tid = threadIdx.x;
    // codes (bytes) per row, and the pieces a row is worked through in
    const int J = LONG ? (gated_row_bytes & 0xffffff) : RUNS * kRunCodes;
    constexpr int kPieceBytes = RUNS * kRunCodes;
    const int n_pieces = LONG ? (J + kPieceBytes - 1) / kPieceBytes : 1;

    // The prologue's duties are split between the waves so that each has little queued ahead of its code loads:
    // waves 0-7 fetch the table (two threads per entry), waves 8-15 fetch x (one or two pieces per thread).
    // These loads sit in wave-uniform branches; the code loads behind them are unconditional, so the wait
    // counts stay exact (the conditional loads are older than the code loads on every path).
    int book0 = 0, second_book_row = INT_MAX;  // the workgroup's first codebook; rows from second_book_row on read the second table
    // row of W behind a gated output: its gate row (the up row lies 16 further on)
    auto gate_row = [](int o) { return 32 * (o >> 4) + (o & 15); };
    bool second_table = false;
    if constexpr (BOOKS > 0) {
        // the workgroup's first and last share (rows, or outputs when gated) and the rows of W they reach
        const int wg_first = min((int)blockIdx.x * kWideWaves * rows_q + min((int)blockIdx.x * kWideWaves, rows_r), n_total - 1);
        const int wg_last = min(((int)blockIdx.x + 1) * kWideWaves * rows_q + min(((int)blockIdx.x + 1) * kWideWaves, rows_r), n_total) - 1;
        const int wg_row0 = gated ? gate_row(wg_first) : wg_first;
        const int wg_row_last = gated ? gate_row(max(wg_last, wg_first)) + 16 : wg_last;
        book0 = small_quotient(wg_row0, rows_per_cb, rcp_rows_per_cb);
        if (TWO) second_book_row = (book0 + 1) * rows_per_cb;
        // (only the workgroups whose rows cross into the next codebook fetch and fill the second table)
        second_table = TWO && second_book_row <= wg_row_last;
    }
    constexpr int kDutyThreads = kWideWaves * 64 / 2;
    constexpr int kXPerThread = (XM * kXChunks + kDutyThreads - 1) / kDutyThreads;   // (the rows of X lie one behind the other)
    const bool table_duty = tid < kDutyThreads;
    const int e = tid >> 1, half_of_copies = tid & 1;   // table duty: entry and which eight of its sixteen copies
    const int xt = tid - kDutyThreads;                  // x duty: pieces xt, xt + 512
    uint4_t entry0 = {0u, 0u, 0u, 0u}, entry1 = {0u, 0u, 0u, 0u};
    uint4_t xpiece[kXPerThread];
    if (table_duty) {
        // (entries past a short codebook are loaded clamped and zeroed afterwards)
        const int ec = min(e, entries - 1);
        entry0 = reinterpret_cast<const uint4_t *>(cb + (int64_t)book0 * entries * 8)[ec];
        if (second_table) entry1 = reinterpret_cast<const uint4_t *>(cb + (int64_t)min(book0 + 1, n_books - 1) * entries * 8)[ec];
    } else {
#pragma unroll
        for (int i = 0; i < kXPerThread; i++) {
            // (the long form: a row of x is J pieces in memory and kXChunks in the LDS)
            const int xi = xt + i * kDutyThreads, m = XM > 1 && xi >= kXChunks ? 1 : 0;
            xpiece[i] = reinterpret_cast<const uint4_t *>(x)[LONG ? m * J + min(xi - m * kXChunks, J - 1) : min(xi, XM * kXChunks - 1)];
        }
    }

    // the wave's share [row0, row0 + n_share) of the rows (gated: of the outputs) and its code rows: at most 64, one
    // result per lane
    const uint32_t lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int gw = blockIdx.x * kWideWaves + wave;
    const int row0 = min(gw * rows_q + min(gw, rows_r), n_total - 1);  // (a wave without a share reads the last row)
    const int n_share = rows_q + (gw < rows_r ? 1 : 0);
    const int n_rows = gated ? 2 * n_share : n_share;
    const int n_groups = (n_rows + G - 1) / G;
    // code row t of the wave (clamped: loads past the end read the last row again)
    auto code_row = [&](int t) {
        t = min(t, max(n_rows, 1) - 1);
        return gated ? gate_row(row0 + (t >> 1)) + 16 * (t & 1) : row0 + t;
    };
    // gated with a bias: lane i keeps the bias of its i-th output's gate and up row (loaded ahead of the codes, so
    // that the loop stays free of loads other than the codes)
    float bias_gate = 0.f, bias_up = 0.f;
    if (gated && bias) {
        const int o = row0 + min((int)lane, max(n_share, 1) - 1);
        bias_gate = (float)bias[gate_row(o)];
        bias_up = (float)bias[gate_row(o) + 16];
    }

    uint32_t cw[NBUF][G][RUNS];
    // group g of the wave's rows, piece `piece` of them (0 outside the long form)
    auto load_group = [&](int piece, int g, uint32_t (&dst)[G][RUNS]) {
#pragma unroll
        for (int r = 0; r < G; r++) {
            // (a wave-uniform row pointer and the lane as a 32-bit index: one scalar base per row, no vector address arithmetic)
            if constexpr (LONG) {
                const uint8_t *row = codes + (int64_t)code_row(g * G + r) * J + piece * kPieceBytes;
                const uint32_t last = (uint32_t)(J - 4 - piece * kPieceBytes);  // the row's last dword, from the piece on
#pragma unroll
                for (int q = 0; q < RUNS; q++)
                    dst[r][q] = __hip_atomic_load(reinterpret_cast<const uint32_t *>(row + min(q * kRunCodes + 4u * lane, last)),
                                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
            } else {
                const uint32_t *row = reinterpret_cast<const uint32_t *>(codes + (int64_t)code_row(g * G + r) * J);
#pragma unroll
                for (int q = 0; q < RUNS; q++)
                    // (a relaxed atomic load of wavefront scope is an ordinary load instruction that the compiler
                    // leaves where it is written: ahead of the table's stores and the barrier)
                    dst[r][q] = __hip_atomic_load(row + q * (kRunCodes / 4) + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
            }
        }
    };
    // the long form walks (piece, group) pairs, all groups of a piece before the next piece; the request runs
    // NBUF - 1 pairs ahead of the multiply and asks for the last pair again once it is past the end
    int req_piece = 0, req_group = 0;
    auto request_next = [&](uint32_t (&dst)[G][RUNS]) {
        const bool over = req_piece >= n_pieces || n_groups <= 0;
        load_group(over ? n_pieces - 1 : req_piece, over ? max(n_groups, 1) - 1 : req_group, dst);
        if (++req_group >= n_groups) req_group = 0, ++req_piece;
    };
#pragma unroll
    for (int u = 0; u < NBUF - 1; u++) {
        if constexpr (LONG) request_next(cw[u]);
        else load_group(0, min(u, max(n_groups, 1) - 1), cw[u]);
    }
    // (NBUF == 1: no wave has more than one group - its codes are all the loads there are, and there is no loop)
    if constexpr (NBUF == 1) load_group(0, 0, cw[0]);

    if (table_duty) {
        // Table: thread (e, h) writes copies 8h .. 8h+7 of entry e, in an order that sends the sixteen lanes
        // served together to sixteen different copies (bank groups).  Entries past a short codebook are zeros,
        // so any 8-bit code gathers a defined value.
        if (e >= entries) entry0 = entry1 = uint4_t{0u, 0u, 0u, 0u};
        if constexpr (COPIES == 1) {
            // (the plain table: the first table's entry from the thread's even twin, the second table's from the odd one)
            if (half_of_copies == 0) table[e] = entry0;
            else if (second_table) table[256 + e] = entry1;
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) table[e * kWideCopies + half_of_copies * 8 + ((e + i) & 7)] = entry0;
            if (second_table) {
#pragma unroll
                for (int i = 0; i < 8; i++) table[256 * kWideCopies + e * kWideCopies + half_of_copies * 8 + ((e + i) & 7)] = entry1;
            }
        }
    } else {
        // x: piece i = q*256 + 4*l + c (the 8 halves that code c of lane l's dword in run q meets) is kept at
        // q*256 + c*64 + l, so that the lanes of a wave read 64 neighbouring pieces.
#pragma unroll
        for (int i = 0; i < kXPerThread; i++) {
            const int xi = xt + i * kDutyThreads;
            // (the long form: zeros behind the end of x, up to whole pieces of rows)
            if (LONG && xi - (XM > 1 && xi >= kXChunks ? kXChunks : 0) >= J) xpiece[i] = uint4_t{0u, 0u, 0u, 0u};
            if (xi < XM * kXChunks) xs[(xi & ~255) + (xi & 3) * 64 + ((xi >> 2) & 63)] = xpiece[i];
        }
    }
    __syncthreads();
    if (n_rows <= 0) return;
    uint4_t xr[XM][RUNS][4];
    auto load_x_piece = [&](int piece) {
#pragma unroll
        for (int m = 0; m < XM; m++)
#pragma unroll
            for (int q = 0; q < RUNS; q++)
#pragma unroll
                for (int c = 0; c < 4; c++) xr[m][q][c] = xs[m * kXChunks + (piece * RUNS + q) * kRunCodes + c * 64 + lane];
    };
    load_x_piece(0);

    // Gather address = table * 65536 + code * 256 + copy * 16, put together by one byte permute out of the
    // lane's dword of codes (byte 1) and a per-row base (bytes 0 and 2).
    const uint32_t copy_base = (lane & (kWideCopies - 1)) * 16u;
    const uint8_t *tbl = reinterpret_cast<const uint8_t *>(table);
    float res[XM];       // lane i: the sum of the wave's row i (for each row of X)
    float gate_sum[XM];  // gated, G = 1: the gate row's sum (wave-uniform) until the up row's group has run
#pragma unroll
    for (int m = 0; m < XM; m++) res[m] = gate_sum[m] = 0.f;
    // rows [g*G, g*G + R) of the wave, R <= G (a compile-time count: the last group may be short)
    auto multiply_rows = [&](int g, const uint32_t (&cur)[G][RUNS], auto r_const) {
        constexpr int R = decltype(r_const)::value;
        float acc[XM][R];
        uint32_t base[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int m = 0; m < XM; m++) acc[m][r] = 0.f;
            // (the long form: the row's sum over the pieces before this one, zero at the first)
            if constexpr (LONG) {
#pragma unroll
                for (int m = 0; m < XM; m++)
                    acc[m][r] = lane == 0 ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, res[m]), g * G + r)) : 0.f;
            }
            if constexpr (COPIES == 1) base[r] = TWO && code_row(g * G + r) >= second_book_row ? 4096u : 0u;
            else base[r] = TWO ? copy_base | (code_row(g * G + r) >= second_book_row ? 0x10000u : 0u) : copy_base;
        }
#pragma unroll
        for (int q = 0; q < RUNS; q++) {
            // the four gathers of every row's dword go out together, the sixteen products follow
            uint4_t w[R][4];
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    // result bytes: 0 = byte 0 of the base, 1 = byte c of the codes, 2 = byte 2 of the base, 3 = zero
                    // (plain table: code * 16 behind the table's offset)
                    const uint32_t addr = COPIES == 1 ? (((cur[r][q] >> (8 * c)) & 0xffu) << 4) + base[r]
                                                      : __builtin_amdgcn_perm(cur[r][q], base[r], 0x0c020000u | ((4u + c) << 8));
                    w[r][c] = *reinterpret_cast<const uint4_t *>(tbl + addr);
                }
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int r = 0; r < R; r++)
#pragma unroll
                    for (int d = 0; d < 4; d++)
#pragma unroll
                        for (int m = 0; m < XM; m++) {
                            const uint32_t wd = w[r][c][d], xd = xr[m][q][c][d];
                            acc[m][r] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, wd), __builtin_bit_cast(half2_t, xd), acc[m][r], false);
                        }
        }
        if (G == 2 && R == 2 && gated) {
            // one output: gate and up sums, the bias of the output's lane, silu(gate) * up
#pragma unroll
            for (int m = 0; m < XM; m++) {
                const float sg = wave_sum_to_uniform(acc[m][0]) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, bias_gate), g));
                const float su = wave_sum_to_uniform(acc[m][R - 1]) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, bias_up), g));
                res[m] = (int)lane == g ? silu_f32(sg) * su : res[m];
            }
            return;
        }
        if (G == 1 && gated) {
            // even groups are gate rows, odd groups the up rows of the same output
            const int o = g >> 1;
#pragma unroll
            for (int m = 0; m < XM; m++) {
                const float s = wave_sum_to_uniform(acc[m][0]);
                if ((g & 1) == 0) {
                    gate_sum[m] = s + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, bias_gate), o));
                } else {
                    const float su = s + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, bias_up), o));
                    res[m] = (int)lane == o ? silu_f32(gate_sum[m]) * su : res[m];
                }
            }
            return;
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int m = 0; m < XM; m++) {
                // (the row's sum goes from the scalar register straight into lane g*G + r: one v_writelane instead of a
                // move, a compare and a select)
                const float s = wave_sum_to_uniform(acc[m][r]);
                // (on this target the instruction takes one scalar register: the lane number goes through m0)
                asm("s_mov_b32 m0, %2\n\tv_writelane_b32 %0, %1, m0" : "+v"(res[m]) : "s"(s), "s"(g * G + r) : "m0");
            }
    };
    auto multiply_group = [&](int g, const uint32_t (&cur)[G][RUNS]) {
        const int left = n_rows - g * G;  // wave-uniform
        if (left >= G) multiply_rows(g, cur, std::integral_constant<int, G>{});
        else if (G > 1 && left == 1) multiply_rows(g, cur, std::integral_constant<int, 1>{});
        else if (G > 2 && left == 2) multiply_rows(g, cur, std::integral_constant<int, (G > 2 ? 2 : 1)>{});
        else if (G > 3) multiply_rows(g, cur, std::integral_constant<int, (G > 3 ? 3 : 1)>{});
    };
    // rotate_priority: a SIMD issues for its oldest wave first.  With equal shares the four waves of a SIMD therefore
    // finish one after the other, and the youngest works through its last rows alone, with a single wave's loads in
    // flight and nobody to cover its waits (time stamps inside the kernel, K = 8192, N = 28672, seven rows per wave: the
    // four ages are done 5.7, 6.3, 7.4 and 8.9 us after they start; K = 4096: 3.6, 4.0, 4.7, 5.6).  The wave's issue
    // priority (s_setprio, 0 to 3) therefore steps down by one with every group and wraps around, starting from its age
    // class wave / 4: the four waves of a SIMD take turns at being served first (the same launches: 6.9, 8.0, 7.9, 7.6 us
    // and 4.5, 4.9, 4.7, 4.4 us; the last wave ends 0.9 resp. 1.1 us earlier).  A hint to the arbiter: no result
    // depends on it.
    const int age = wave >> 2;
    auto set_priority = [&](int v) {
        switch (v & 3) {
        case 0: __builtin_amdgcn_s_setprio(0); break;
        case 1: __builtin_amdgcn_s_setprio(1); break;
        case 2: __builtin_amdgcn_s_setprio(2); break;
        default: __builtin_amdgcn_s_setprio(3); break;
        }
    };
    if constexpr (NBUF == 1) {
        multiply_group(0, cw[0]);
    } else if constexpr (LONG) {
        int piece = 0, g = 0, turn = 0;
        while (piece < n_pieces) {
#pragma unroll
            for (int u = 0; u < NBUF; u++) {
                request_next(cw[(u + NBUF - 1) % NBUF]);
                if (rotate_priority) set_priority(age - turn++);
                if (piece < n_pieces) {
                    if (g == 0 && piece > 0) load_x_piece(piece);
                    multiply_group(g, cw[u]);
                    if (++g >= n_groups) g = 0, ++piece;
                }
            }
        }
    } else if constexpr (NBUF == 2) {
        // Two groups in flight: the loop runs while both of its requests are for groups that exist, and the last one or
        // two groups are multiplied behind it in straight-line code, so that no group is requested twice (a wave's
        // last request would otherwise be its last group again, and the wave ends only when that load has landed).
        // Inside either branch of the tail the order of loads and uses is fixed: the wait counts stay exact.
        int g = 0;
        for (; g + 2 < n_groups; g += 2) {
            load_group(0, g + 1, cw[1]);
            if (rotate_priority) set_priority(age - g);
            multiply_group(g, cw[0]);
            load_group(0, g + 2, cw[0]);
            if (rotate_priority) set_priority(age - (g + 1));
            multiply_group(g + 1, cw[1]);
        }
        if (n_groups - g == 2) {
            load_group(0, g + 1, cw[1]);
            if (rotate_priority) set_priority(age - g);
            multiply_group(g, cw[0]);
            if (rotate_priority) set_priority(age - (g + 1));
            multiply_group(g + 1, cw[1]);
        } else {
            if (rotate_priority) set_priority(age - g);
            multiply_group(g, cw[0]);
        }
    } else {
        for (int g = 0; g < n_groups; g += NBUF) {
#pragma unroll
            for (int u = 0; u < NBUF; u++) {
                // (unconditional: see the header; the group requested past the end is the last one again)
                load_group(0, min(g + u + NBUF - 1, n_groups - 1), cw[(u + NBUF - 1) % NBUF]);
                if (rotate_priority) set_priority(age - (g + u));
                if (g + u < n_groups) multiply_group(g + u, cw[u]);
            }
        }
    }
    if ((int)lane < n_share) {
        const float b = bias && !gated ? (float)bias[row0 + lane] : 0.f;
#pragma unroll
        for (int m = 0; m < XM; m++) y[(int64_t)m * n_total + row0 + lane] = (half_t)(res[m] + b);   // (a row of y: what was dealt out)
    }
}

}  // namespace

// Rows per group (1 or 2) and groups of codes in flight (2 or 3) of the wide form are runtime choices out of the
// tuning table, separately for K up to 4096 and beyond: `python -m vq_gemm_amd.tune --search` times the four
// combinations on the box at hand, on codes that come from HBM.
// A wave with one or two rows (Tuning::gemv_wide_single_rows_max) takes them one by one with two groups in flight
// whatever the table says: a group of two would request a row that is not there ahead of the one that is (cold, K = 4096,
// groups of two -> groups of one: one row per wave 3.36 -> 3.13 us, two rows 4.00 -> 3.75; from three rows on the two
// are level, from seven on groups of two are ahead).  Not for gated launches, where the group size says how a gate/up
// pair is dealt.
static bool wide_few_rows(const ProblemB &p)
{
    if (p.gated) return false;
    const int waves = device_cu_count() * kWideWaves;
    return (double)((p.N + waves - 1) / waves) <= tuning().gemv_wide_single_rows_max;
}
static int wide_rows_per_group(const ProblemB &p)
{
    const Tuning &tn = tuning();
    if (wide_few_rows(p)) return 1;
    return (p.K / kRunK > 2 ? tn.gemv_wide_rows_per_group_long_k : tn.gemv_wide_rows_per_group) >= 2.0 ? 2 : 1;
}
static int wide_groups_in_flight(const ProblemB &p)
{
    const Tuning &tn = tuning();
    if (wide_few_rows(p)) return 2;
    return (p.K / kRunK > 2 ? tn.gemv_wide_groups_in_flight_long_k : tn.gemv_wide_groups_in_flight) >= 3.0 ? 3 : 2;
}

// The long form's cut of a row (see the kernel): K beyond 8192 or no multiple of 2048, up to 32768, whole dwords of
// codes per row.  runs = runs of 2048 k per piece (3 or 4, whichever pads the row less), x_runs = what the LDS holds.
struct LongK {
    bool is_long;
    int runs, x_runs;
};
static LongK long_k_form(const ProblemB &p)
{
    LongK f{false, 0, 0};
    const int runs_needed = (int)((p.K + kRunK - 1) / kRunK);
    if (p.M == 2) {
        // two rows of X: a lane's registers hold two runs of each, so K beyond 4096 goes in pieces of two runs, and
        // the LDS has room for eight runs of each row beside the table
        if (p.K % kRunK == 0 && p.K / kRunK <= 2) return f;
        f.is_long = true;
        f.runs = 2;
        f.x_runs = (runs_needed + 1) / 2 * 2 <= 4 ? 4 : 8;
        return f;
    }
    if (p.K % kRunK == 0 && p.K / kRunK <= kGemvMaxRuns) return f;
    f.is_long = true;
    const int padded4 = (runs_needed + 3) / 4 * 4, padded3 = (runs_needed + 2) / 3 * 3;
    f.runs = padded3 < padded4 ? 3 : 4;
    f.x_runs = min(padded3, padded4) <= 8 ? 8 : 16;
    return f;
}

// The workgroups of a launch: one per compute unit - or, with several codebooks, a few less where that makes every
// workgroup's rows fall inside one codebook: a workgroup whose rows cross a boundary fills two tables, and the launch
// ends with the slowest workgroup (the q, k and v projections of a layer as three codebooks of 4096 rows: 192
// workgroups of 64 rows take 4.9 us cold where 256 workgroups of 48 rows take 5.25).  Not below
// Tuning::gemv_wide_min_units_share of the units.
static int wide_workgroups(const ProblemB &p)
{
    const int cus = device_cu_count();
    if (p.n_codebooks > 1 && !p.gated) {
        const int least = (int)(tuning().gemv_wide_min_units_share * cus);
        for (int w = cus; w >= least && w >= 1; w--) {
            const int per_wg = p.N / w;
            if (p.N % w == 0 && per_wg % kWideWaves == 0 && per_wg / kWideWaves <= 64 && p.rows_per_cb % per_wg == 0) return w;
        }
    }
    return cus;
}
// whether some workgroup's rows cross a codebook boundary (then every workgroup has room for two tables)
static bool wide_straddles(const ProblemB &p, int workgroups)
{
    const int waves = workgroups * kWideWaves;
    return p.n_codebooks > 1 && (p.gated || !(p.N % waves == 0 && p.rows_per_cb % (kWideWaves * (p.N / waves)) == 0));
}

// One row of X, 8-vectors, 8-bit codes, K a multiple of 2048 up to 8192 - or, not gated and with no workgroup reaching
// into two codebooks, any multiple of 32 from 2048 up to 32768 - and no workgroup's share of the rows reaching into
// more than two codebooks.
bool decode_gemv_wide_supports(const ProblemB &p)
{
    if (p.M < 1 || p.M > 2 || p.vec != 8 || p.code_bits != 8 || p.entries > 256 || p.packed) return false;
    if (p.K < kRunK || p.N < 1) return false;
    if (long_k_form(p).is_long) {
        // (two rows of X: K up to 16384)
        if (p.K % 32 != 0 || p.K > (p.M == 2 ? 8 : 16) * kRunK || p.gated) return false;
        const int workgroups = wide_workgroups(p);
        if (wide_straddles(p, workgroups)) return false;
        return (p.N + workgroups * kWideWaves - 1) / (workgroups * kWideWaves) <= 64;
    }
    const int waves = device_cu_count() * kWideWaves;
    if (p.gated) {
        // two code rows per output: one group of two rows, or two groups of one
        if (p.N % 32 != 0) return false;
        const int outs_per_wave = (p.N / 2 + waves - 1) / waves;
        if (outs_per_wave > 32) return false;
        // a workgroup's rows of W: its outputs' gate and up rows, in whole groups of 32
        return p.n_codebooks == 1 || (int64_t)2 * kWideWaves * outs_per_wave + 32 <= p.rows_per_cb;
    }
    const int rows_per_wave = (p.N + waves - 1) / waves;
    if (rows_per_wave > 64) return false;  // one result per lane
    return p.n_codebooks == 1 || (int64_t)kWideWaves * rows_per_wave <= p.rows_per_cb;
}

hipError_t launch_decode_gemv_wide(const ProblemB &p, hipStream_t s)
{
    if (!decode_gemv_wide_supports(p)) return hipErrorInvalidValue;
    const int cus = wide_workgroups(p);
    const int waves = cus * kWideWaves;
    const dim3 grid(cus), block(kWideWaves * 64);
    const uint8_t *codes = static_cast<const uint8_t *>(p.codes);
    const int books = p.n_codebooks == 1 ? 0 : (wide_straddles(p, cus) ? 2 : 1);
    const int n_dealt = p.gated ? p.N / 2 : p.N;  // what is dealt out to the waves: rows of W, or outputs
    // the waves of a SIMD take turns at the issue priority (see the kernel) once they have two rows or more each: a
    // single row per wave is over before a turn would come
    const int rotate_priority = tuning().gemv_wide_rotate_priority >= 1.0 && (n_dealt + waves - 1) / waves >= 2 ? 1 : 0;
    auto launch = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, block, 0, s, p.x, codes, p.cb, p.entries, n_dealt / waves, n_dealt % waves, n_dealt,
                           (int)((p.gated ? 0x80000000u : 0u) | (uint32_t)(p.K / 8)), p.rows_per_cb,
                           1.0f / (float)p.rows_per_cb, p.n_codebooks, p.bias, p.y, rotate_priority);
        return hipGetLastError();
    };
    using std::integral_constant;
    const int g = wide_rows_per_group(p);
    if (const LongK f = long_k_form(p); p.M == 2 && f.is_long) {
        auto pick_long2 = [&](auto g_c, auto x_c) {
            constexpr int GG = decltype(g_c)::value, XR = decltype(x_c)::value;
            return books == 0 ? launch(decode_gemv_wide_kernel<2, GG, 2, 0, kWideCopies, XR, 2>)
                              : launch(decode_gemv_wide_kernel<2, GG, 2, 1, kWideCopies, XR, 2>);
        };
        auto pick_x2 = [&](auto g_c) {
            return f.x_runs == 4 ? pick_long2(g_c, integral_constant<int, 4>{}) : pick_long2(g_c, integral_constant<int, 8>{});
        };
        return g == 2 ? pick_x2(integral_constant<int, 2>{}) : pick_x2(integral_constant<int, 1>{});
    }
    if (p.M == 2) {
        // two rows of X against every gathered codeword: the replicated table, one or two groups
        auto pick2 = [&](auto runs_c, auto g_c, auto nbuf_c) {
            constexpr int R = decltype(runs_c)::value, GG = decltype(g_c)::value, NB = decltype(nbuf_c)::value;
            return books == 0 ? launch(decode_gemv_wide_kernel<R, GG, NB, 0, kWideCopies, R, 2>)
                 : books == 1 ? launch(decode_gemv_wide_kernel<R, GG, NB, 1, kWideCopies, R, 2>)
                              : launch(decode_gemv_wide_kernel<R, GG, NB, 2, kWideCopies, R, 2>);
        };
        auto pick2_runs = [&](auto g_c, auto nbuf_c) {
            return p.K / kRunK == 1 ? pick2(integral_constant<int, 1>{}, g_c, nbuf_c) : pick2(integral_constant<int, 2>{}, g_c, nbuf_c);
        };
        if (!p.gated && (n_dealt + waves - 1) / waves <= 1) return pick2_runs(integral_constant<int, 1>{}, integral_constant<int, 1>{});
        return g == 2 ? pick2_runs(integral_constant<int, 2>{}, integral_constant<int, 2>{})
                      : pick2_runs(integral_constant<int, 1>{}, integral_constant<int, 2>{});
    }
    if (const LongK f = long_k_form(p); f.is_long) {
        // (the replicated table, one table per workgroup, two groups in flight: three were measured and are slower,
        // K = 11008 to 28672, N = 4096 to 16384: +3 to +6 %, one shape -3 %)
        auto pick_long = [&](auto runs_c, auto g_c, auto x_c) {
            constexpr int R = decltype(runs_c)::value, GG = decltype(g_c)::value, XR = decltype(x_c)::value;
            return books == 0 ? launch(decode_gemv_wide_kernel<R, GG, 2, 0, kWideCopies, XR>)
                              : launch(decode_gemv_wide_kernel<R, GG, 2, 1, kWideCopies, XR>);
        };
        auto pick_x = [&](auto runs_c, auto g_c) {
            return f.x_runs == 8 ? pick_long(runs_c, g_c, integral_constant<int, 8>{}) : pick_long(runs_c, g_c, integral_constant<int, 16>{});
        };
        auto pick_g = [&](auto runs_c) {
            return g == 2 ? pick_x(runs_c, integral_constant<int, 2>{}) : pick_x(runs_c, integral_constant<int, 1>{});
        };
        return f.runs == 3 ? pick_g(integral_constant<int, 3>{}) : pick_g(integral_constant<int, 4>{});
    }
    // The plain table while a wave gathers for at most Tuning::gemv_wide_plain_table_max_runs runs of 2048 k (8 gathers per
    // lane and run): measured cold, plain -> replicated, K = 4096: one row per wave 3.29 -> 3.43 us, two rows
    // 4.07 -> 3.89; K = 2048, one row 2.93 -> 3.12; K = 8192, one row 4.26 -> 4.02.
    const int code_rows_per_wave = (int)((p.N + waves - 1) / waves);
    const bool plain_table = (double)code_rows_per_wave * (double)(p.K / kRunK) <= tuning().gemv_wide_plain_table_max_runs;
    auto pick = [&](auto runs_c, auto g_c, auto nbuf_c) {
        constexpr int R = decltype(runs_c)::value, GG = decltype(g_c)::value, NB = decltype(nbuf_c)::value;
        if (plain_table)
            return books == 0 ? launch(decode_gemv_wide_kernel<R, GG, NB, 0, 1>)
                 : books == 1 ? launch(decode_gemv_wide_kernel<R, GG, NB, 1, 1>) : launch(decode_gemv_wide_kernel<R, GG, NB, 2, 1>);
        return books == 0 ? launch(decode_gemv_wide_kernel<R, GG, NB, 0, kWideCopies>)
             : books == 1 ? launch(decode_gemv_wide_kernel<R, GG, NB, 1, kWideCopies>) : launch(decode_gemv_wide_kernel<R, GG, NB, 2, kWideCopies>);
    };
    auto pick_runs = [&](auto g_c, auto nbuf_c) {
        switch (p.K / kRunK) {
        case 1: return pick(integral_constant<int, 1>{}, g_c, nbuf_c);
        case 2: return pick(integral_constant<int, 2>{}, g_c, nbuf_c);
        default: break;
        }
        // (two rows per group with three groups in flight do not fit the registers beyond K = 4096: not built)
        if constexpr (decltype(g_c)::value * decltype(nbuf_c)::value <= 4) {
            if (p.K / kRunK == 3) return pick(integral_constant<int, 3>{}, g_c, nbuf_c);
            return pick(integral_constant<int, 4>{}, g_c, nbuf_c);
        }
        return hipErrorInvalidValue;
    };
    // (a launch in which no wave has more than one row: no second group to request)
    const bool single = !p.gated && tuning().gemv_wide_single_rows_max >= 1.0 && (n_dealt + waves - 1) / waves <= 1;
    if (single) return pick_runs(integral_constant<int, 1>{}, integral_constant<int, 1>{});
    const int nbuf = (g == 2 && p.K / kRunK > 2) ? 2 : wide_groups_in_flight(p);
    if (g == 2) return nbuf == 3 ? pick_runs(integral_constant<int, 2>{}, integral_constant<int, 3>{})
                                 : pick_runs(integral_constant<int, 2>{}, integral_constant<int, 2>{});
    return nbuf == 3 ? pick_runs(integral_constant<int, 1>{}, integral_constant<int, 3>{})
                     : pick_runs(integral_constant<int, 1>{}, integral_constant<int, 2>{});
}

bool decode_gemv_wide_preferred(const ProblemB &p);

namespace {

// the four-wave kernel (decode_gemv_kernel)
bool decode_gemv_plain_supports(const ProblemB &p)
{
    const bool u8 = p.code_bits == 8;
    // 8- and 4-vectors with either code width, 2-vectors with 8-bit codes (one load of at most 16 bytes per run)
    if (!(p.vec == 8 || p.vec == 4 || (p.vec == 2 && u8))) return false;
    if (p.entries > (u8 ? 256 : 4096) || (p.entries * p.vec * 2) % 16 != 0) return false;
    // two rows of X at most outside the first format (three and four never pay)
    const int max_m = (p.vec == 8 && u8) ? 4 : 2;
    // gated: whole groups of 32 interleaved rows, per codebook too
    if (p.gated && (p.N % 32 != 0 || p.rows_per_cb % 32 != 0)) return false;
    return p.M >= 1 && p.M <= max_m && (int)(p.K / kRunK) * p.M * 16 <= kGemvMaxXRegs && !p.packed && p.K >= kRunK &&
           p.K % kRunK == 0 && p.K / kRunK <= kGemvMaxRuns && p.N % kGemvTile == 0 && p.rows_per_cb % kGemvTile == 0;
}

}  // namespace

bool decode_gemv_supports(const ProblemB &p) { return decode_gemv_wide_preferred(p) || decode_gemv_plain_supports(p); }

// From Tuning::gemv_wide_min_rows_per_wave rows per wave of the wide form on (sixteen waves per compute unit), one row
// of X goes to it: 0 by default, every launch it supports.

bool decode_gemv_wide_preferred(const ProblemB &p)
{
    // two rows of X: while a wave's rows are at most Tuning::gemv_wide_two_rows_max_runs runs of 2048 k (measured cold
    // against the K-sliced kernel, K = 4096: 8 rows per wave 9.8 against 11.2 us, 11 rows 12.6 against 13.1, 12 rows 13.8
    // against 13.7, 14 rows 16.5 against 14.9; K = 2048: 14 rows 10.3 against 11.1)
    if (p.M == 2) {
        const int waves = device_cu_count() * kWideWaves;
        const double runs = (double)(((p.gated ? p.N / 2 : p.N) + waves - 1) / waves) * (p.gated ? 2 : 1) * (double)(p.K / kRunK);
        // (K from 8192 on the K-sliced kernels walk K in chunks and fall behind later: K = 8192, 28 runs per wave 17.3
        // against 18.9 us, 32 runs 19.8 against 20.6, 40 runs 23.0 against 23.2; K = 14336, 35 runs 23.3 against 27.6)
        if (runs > (p.K >= 4 * kRunK ? tuning().gemv_wide_two_rows_max_runs_long_k : tuning().gemv_wide_two_rows_max_runs)) return false;
    }
    return decode_gemv_wide_supports(p) && (double)p.M <= tuning().gemv_wide_max_m &&
           (double)(p.gated ? p.N / 2 : p.N) >= tuning().gemv_wide_min_rows_per_wave * kWideWaves * device_cu_count();
}

namespace {

template <int VEC, typename CodeT, bool GATED>
hipError_t launch_gemv_format(const ProblemB &p, hipStream_t s)
{
    const dim3 grid(p.N / kGemvTile), block(kGemvWaves * 64);
    const CodeT *codes = static_cast<const CodeT *>(p.codes);
    auto launch = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, block, 0, s, p.x, codes, p.cb, p.y, p.bias, p.K, p.N, p.entries, p.rows_per_cb);
    };
    switch ((p.K / kRunK) * 10 + p.M) {
    case 11: launch(decode_gemv_kernel<VEC, CodeT, 1, 1, GATED>); break;
    case 12: launch(decode_gemv_kernel<VEC, CodeT, 1, 2, GATED>); break;
    case 21: launch(decode_gemv_kernel<VEC, CodeT, 2, 1, GATED>); break;
    case 22: launch(decode_gemv_kernel<VEC, CodeT, 2, 2, GATED>); break;
    case 31: launch(decode_gemv_kernel<VEC, CodeT, 3, 1, GATED>); break;
    case 32: launch(decode_gemv_kernel<VEC, CodeT, 3, 2, GATED>); break;
    case 41: launch(decode_gemv_kernel<VEC, CodeT, 4, 1, GATED>); break;
    case 42: launch(decode_gemv_kernel<VEC, CodeT, 4, 2, GATED>); break;
    default:
        if constexpr (VEC == 8 && sizeof(CodeT) == 1) {
            switch ((p.K / kRunK) * 10 + p.M) {
            case 13: launch(decode_gemv_kernel<8, uint8_t, 1, 3, GATED>); break;
            case 14: launch(decode_gemv_kernel<8, uint8_t, 1, 4, GATED>); break;
            case 23: launch(decode_gemv_kernel<8, uint8_t, 2, 3, GATED>); break;
            case 24: launch(decode_gemv_kernel<8, uint8_t, 2, 4, GATED>); break;
            default: return hipErrorInvalidValue;
            }
            break;
        }
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <bool GATED>
hipError_t launch_gemv_any_format(const ProblemB &p, hipStream_t s)
{
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? launch_gemv_format<8, uint8_t, GATED>(p, s) : launch_gemv_format<8, uint16_t, GATED>(p, s);
    case 4: return u8 ? launch_gemv_format<4, uint8_t, GATED>(p, s) : launch_gemv_format<4, uint16_t, GATED>(p, s);
    default: return launch_gemv_format<2, uint8_t, GATED>(p, s);
    }
}

}  // namespace

hipError_t launch_decode_gemv(const ProblemB &p, hipStream_t s)
{
    if (decode_gemv_wide_preferred(p)) return launch_decode_gemv_wide(p, s);
    if (!decode_gemv_plain_supports(p)) return hipErrorInvalidValue;
    return p.gated ? launch_gemv_any_format<true>(p, s) : launch_gemv_any_format<false>(p, s);
}

}  // namespace vq
