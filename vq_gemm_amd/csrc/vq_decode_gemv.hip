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
// wins while a compute unit has a few tiles; longer runs of rows go to the persistent form below
// (decode_gemv_stream_kernel) and, beyond that, to the batched kernel, whose waves share X and the
// table over many tiles.
#include "vq_common.h"

namespace vq {

namespace {

#ifndef VQ_GEMV_WAVES
#define VQ_GEMV_WAVES 4
#endif
#ifndef VQ_GEMV_ROWS
#define VQ_GEMV_ROWS 4
#endif
constexpr int kGemvWaves = VQ_GEMV_WAVES;
constexpr int kGemvRows = VQ_GEMV_ROWS;                     // rows of W per wave
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
template <int VEC, typename CodeT, int RUNS, int MX>
__global__ __launch_bounds__(kGemvWaves * 64) void decode_gemv_kernel(const half_t *__restrict__ x,
                                                                       const CodeT *__restrict__ codes,
                                                                       const half_t *__restrict__ cb,
                                                                       half_t *__restrict__ y,
                                                                       const half_t *__restrict__ bias, int K,
                                                                       int N, int entries, int rows_per_cb)
{
    typedef GemvCfg<VEC, CodeT> C;
    typedef uint32_t words_t __attribute__((ext_vector_type(C::CW)));
    __shared__ __align__(16) uint4_t table[C::kTableBytes / 16];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int row0 = blockIdx.x * kGemvTile + wave * kGemvRows;
    constexpr int J = RUNS * 64 * C::CPR;  // codes per row

    // The table's load goes out first and is the first to be back (it comes out of the L2): its copy
    // into the LDS and the barrier then pass while the codes (HBM) and x are still on their way.
    // (no division in front of the first load when there is one codebook)
    const int book = rows_per_cb >= N ? 0 : (blockIdx.x * kGemvTile) / rows_per_cb;
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
            const words_t v = *reinterpret_cast<const words_t *>(codes + (int64_t)(row0 + r) * J + (q * 64 + lane) * C::CPR);
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
        gemv_out_t out;
#pragma unroll
        for (int r = 0; r < kGemvRows; r++) {
            float s = wave_sum(acc[m][r]);
            if (bias) s += (float)bias[row0 + r];
            out[r] = (half_t)s;
        }
        if (lane == 0) *reinterpret_cast<gemv_out_t *>(y + (int64_t)m * N + row0) = out;
    }
}

// The same for long runs of rows: two workgroups per compute unit (four waves alone do not cover the
// latency of their own gathers; 64 KB of table each), each walking 16-row blocks of W with x and the
// table kept.  What a block no longer pays (x, the table, the launch of its
// waves) buys a bank-replicated table - one 256-byte bank row per entry holding 16 copies, lane l
// reading copy l % 16, so that the gathers are free of bank conflicts - and the codes of the next
// block are requested before the current one is multiplied.  One row of X, one codebook.
template <int RUNS>
__global__ __launch_bounds__(kGemvWaves * 64) void decode_gemv_stream_kernel(const half_t *__restrict__ x,
                                                                              const uint8_t *__restrict__ codes,
                                                                              const half_t *__restrict__ cb,
                                                                              half_t *__restrict__ y,
                                                                              const half_t *__restrict__ bias,
                                                                              int n_blocks, int entries)
{
#ifndef VQ_GEMV_STREAM_COPIES
#define VQ_GEMV_STREAM_COPIES 16
#endif
#ifndef VQ_GEMV_STREAM_WGS_PER_CU
#define VQ_GEMV_STREAM_WGS_PER_CU 2
#endif
    constexpr int kCopies = VQ_GEMV_STREAM_COPIES;
    __shared__ __align__(16) uint4_t table[256 * kCopies];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int J = RUNS * kRunCodes;  // codes per row
    const uint8_t *lane_codes = codes + (int64_t)(wave * kGemvRows) * J + 4 * lane;
    auto load_block = [&](int b, uint32_t (&cw)[kGemvRows][RUNS]) {
#pragma unroll
        for (int r = 0; r < kGemvRows; r++)
#pragma unroll
            for (int q = 0; q < RUNS; q++)
                cw[r][q] = *reinterpret_cast<const uint32_t *>(lane_codes + ((int64_t)b * kGemvTile + r) * J + q * kRunCodes);
    };
    int b = blockIdx.x;
    uint32_t cur[kGemvRows][RUNS], nxt[kGemvRows][RUNS];
    // (the table entry's load goes out first: it is back, copied and published while the codes are on their way)
    uint4_t entry = {0u, 0u, 0u, 0u};
    if ((int)threadIdx.x < entries) entry = reinterpret_cast<const uint4_t *>(cb)[threadIdx.x];
    load_block(b, cur);
    uint4_t xr[RUNS][4];
#pragma unroll
    for (int q = 0; q < RUNS; q++)
#pragma unroll
        for (int c = 0; c < 4; c++) xr[q][c] = *reinterpret_cast<const uint4_t *>(x + (q * kRunCodes + 4 * lane + c) * 8);
    {   // (every thread writes: entries past a short codebook are zeros, so any 8-bit code gathers a defined value)
        const uint4_t e = entry;
        // (copy (l + i) % 16 in turn i: the sixteen lanes of a group write sixteen different bank groups)
#pragma unroll
        for (int i = 0; i < kCopies; i++) table[threadIdx.x * kCopies + ((lane + i) & (kCopies - 1))] = e;
    }
    __syncthreads();
    const uint32_t copy = lane & (kCopies - 1);
    for (; b < n_blocks; b += gridDim.x) {
        const int bn = b + gridDim.x;
        if (bn < n_blocks) load_block(bn, nxt);
        float acc[kGemvRows];
#pragma unroll
        for (int r = 0; r < kGemvRows; r++) acc[r] = 0.f;
#pragma unroll
        for (int q = 0; q < RUNS; q++)
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int r = 0; r < kGemvRows; r++) {
                    const uint32_t code = (cur[r][q] >> (8 * c)) & 0xffu;
                    const uint4_t w = table[code * kCopies + copy];
#pragma unroll
                    for (int d = 0; d < 4; d++) {
                        const uint32_t wd = w[d], xd = xr[q][c][d];
                        acc[r] = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, wd), __builtin_bit_cast(half2_t, xd), acc[r], false);
                    }
                }
        const int row0 = b * kGemvTile + wave * kGemvRows;
        gemv_out_t out;
#pragma unroll
        for (int r = 0; r < kGemvRows; r++) {
            float s = wave_sum(acc[r]);
            if (bias) s += (float)bias[row0 + r];
            out[r] = (half_t)s;
        }
        if (lane == 0) *reinterpret_cast<gemv_out_t *>(y + row0) = out;
#pragma unroll
        for (int r = 0; r < kGemvRows; r++)
#pragma unroll
            for (int q = 0; q < RUNS; q++) cur[r][q] = nxt[r][q];
    }
}

}  // namespace

bool decode_gemv_stream_supports(const ProblemB &p)
{
    return decode_gemv_supports(p) && p.vec == 8 && p.code_bits == 8 && p.M == 1 && p.n_codebooks == 1;
}

hipError_t launch_decode_gemv_stream(const ProblemB &p, hipStream_t s)
{
    if (!decode_gemv_stream_supports(p)) return hipErrorInvalidValue;
    const int n_blocks = p.N / kGemvTile;
    const int cus = device_cu_count();
    // (four runs: x alone takes 64 registers, a unit holds one workgroup's waves, and a second one would only queue)
    const int wgs = cus * (p.K / kRunK <= 3 ? VQ_GEMV_STREAM_WGS_PER_CU : 1);
    const dim3 grid(n_blocks < wgs ? n_blocks : wgs), block(kGemvWaves * 64);
    const uint8_t *codes = static_cast<const uint8_t *>(p.codes);
    auto launch = [&](auto kern) { hipLaunchKernelGGL(kern, grid, block, 0, s, p.x, codes, p.cb, p.y, p.bias, n_blocks, p.entries); };
    switch (p.K / kRunK) {
    case 1: launch(decode_gemv_stream_kernel<1>); break;
    case 2: launch(decode_gemv_stream_kernel<2>); break;
    case 3: launch(decode_gemv_stream_kernel<3>); break;
    default: launch(decode_gemv_stream_kernel<4>); break;
    }
    return hipGetLastError();
}

bool decode_gemv_supports(const ProblemB &p)
{
    const bool u8 = p.code_bits == 8;
    // 8- and 4-vectors with either code width, 2-vectors with 8-bit codes (one load of at most 16 bytes per run)
    if (!(p.vec == 8 || p.vec == 4 || (p.vec == 2 && u8))) return false;
    if (p.entries > (u8 ? 256 : 4096) || (p.entries * p.vec * 2) % 16 != 0) return false;
    // two rows of X at most outside the first format (three and four never pay)
    const int max_m = (p.vec == 8 && u8) ? 4 : 2;
    return p.M >= 1 && p.M <= max_m && (int)(p.K / kRunK) * p.M * 16 <= kGemvMaxXRegs && !p.packed && p.K >= kRunK &&
           p.K % kRunK == 0 && p.K / kRunK <= kGemvMaxRuns && p.N % kGemvTile == 0 && p.rows_per_cb % kGemvTile == 0;
}

// From this many 16-row blocks per compute unit on, one row of X goes to the streaming kernel.
#ifndef VQ_GEMV_STREAM_MIN_BLOCKS_PER_CU
#define VQ_GEMV_STREAM_MIN_BLOCKS_PER_CU 4
#endif

namespace {

template <int VEC, typename CodeT>
hipError_t launch_gemv_format(const ProblemB &p, hipStream_t s)
{
    const dim3 grid(p.N / kGemvTile), block(kGemvWaves * 64);
    const CodeT *codes = static_cast<const CodeT *>(p.codes);
    auto launch = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, block, 0, s, p.x, codes, p.cb, p.y, p.bias, p.K, p.N, p.entries, p.rows_per_cb);
    };
    switch ((p.K / kRunK) * 10 + p.M) {
    case 11: launch(decode_gemv_kernel<VEC, CodeT, 1, 1>); break;
    case 12: launch(decode_gemv_kernel<VEC, CodeT, 1, 2>); break;
    case 21: launch(decode_gemv_kernel<VEC, CodeT, 2, 1>); break;
    case 22: launch(decode_gemv_kernel<VEC, CodeT, 2, 2>); break;
    case 31: launch(decode_gemv_kernel<VEC, CodeT, 3, 1>); break;
    case 32: launch(decode_gemv_kernel<VEC, CodeT, 3, 2>); break;
    case 41: launch(decode_gemv_kernel<VEC, CodeT, 4, 1>); break;
    case 42: launch(decode_gemv_kernel<VEC, CodeT, 4, 2>); break;
    default:
        if constexpr (VEC == 8 && sizeof(CodeT) == 1) {
            switch ((p.K / kRunK) * 10 + p.M) {
            case 13: launch(decode_gemv_kernel<8, uint8_t, 1, 3>); break;
            case 14: launch(decode_gemv_kernel<8, uint8_t, 1, 4>); break;
            case 23: launch(decode_gemv_kernel<8, uint8_t, 2, 3>); break;
            case 24: launch(decode_gemv_kernel<8, uint8_t, 2, 4>); break;
            default: return hipErrorInvalidValue;
            }
            break;
        }
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_decode_gemv(const ProblemB &p, hipStream_t s)
{
    if (!decode_gemv_supports(p)) return hipErrorInvalidValue;
    if (decode_gemv_stream_supports(p) && p.N / kGemvTile >= VQ_GEMV_STREAM_MIN_BLOCKS_PER_CU * device_cu_count())
        return launch_decode_gemv_stream(p, s);
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? launch_gemv_format<8, uint8_t>(p, s) : launch_gemv_format<8, uint16_t>(p, s);
    case 4: return u8 ? launch_gemv_format<4, uint8_t>(p, s) : launch_gemv_format<4, uint16_t>(p, s);
    default: return launch_gemv_format<2, uint8_t>(p, s);
    }
}

}  // namespace vq
