// Prefill kernel (large M): Y[M,N] = X[M,K] . W^T with W given as codes + codebook.
//
// MFMA-bound.  A 256-thread workgroup (4 waves, 2x2) computes a 256x256 tile of Y with
// v_mfma_f32_32x32x16_f16; each wave owns 128x128 of it (256 fp32 accumulator registers).
//
//   * W never exists as a tile anywhere: the codebooks of the workgroup's rows sit in the
//     LDS and every lane gathers the codeword of "its" W row straight into the 8-half MFMA
//     operand (vec = 8: one ds_read_b128 == one operand).  The order in which K is walked is
//     free, so it is chosen to make a lane's codes contiguous: one 16-byte global load per
//     lane feeds CPL/CPO MFMA steps.
//   * X tiles (256 rows x 64 k) are staged global -> registers -> LDS, double buffered, with
//     the 16-byte chunks of a row XOR-swizzled so that operand reads are conflict free; the
//     loads for stage i+2 are in flight while stage i is multiplied.
//   * fp32 accumulation; one rounding to fp16 in the epilogue.
//
// K order.  A lane of the 32x32x16 MFMA holds 8 consecutive k of one row; lanes 0-31 hold
// k-group 0 and lanes 32-63 k-group 1.  A "super stage" is the K range fed by one 16-byte
// code load per lane: lane group g covers the contiguous range
// [S*2*K_LANE + g*K_LANE, +K_LANE).  LDS stage t of the super stage holds, for both groups,
// the 32 k starting at offset t*32 of the group's range: two 64-byte pieces per X row.
#include "vq_common.h"

namespace vq {

namespace {

constexpr int BM = 256, BN = 256;     // workgroup tile
constexpr int WM = 128, WN = 128;     // wave tile
constexpr int MB = WM / 32, NB = WN / 32;
constexpr int kThreads = 256;
constexpr int kStageK = 64;           // k per LDS stage (4 MFMA steps)
constexpr int kStageBytes = BM * kStageK * 2;  // 32 KB
constexpr int kChunksPerThread = (BM * 8) / kThreads;  // 16-byte chunks of a stage per thread

template <int VEC, typename CodeT>
struct PrefillCfg {
    static constexpr int CPL = 16 / (int)sizeof(CodeT);
    static constexpr int CPO = 8 / VEC;
    static constexpr int K_LANE = CPL * VEC;          // k per lane per super stage
    static constexpr int K_SUPER = 2 * K_LANE;        // k per super stage
    static constexpr int STAGES = K_LANE / 32;        // LDS stages per super stage
    static_assert(CPO >= 1 && STAGES >= 1, "unsupported code layout");
};

template <typename CodeT>
__device__ __forceinline__ uint32_t code_of(const uint4_t &cw, int c)
{
    if constexpr (sizeof(CodeT) == 1)
        return (cw[c >> 2] >> (8 * (c & 3))) & 0xffu;
    else
        return (cw[c >> 1] >> (16 * (c & 1))) & 0xffffu;
}

// `book` must point into the LDS (the callers index the __shared__ array directly so that
// the compiler emits ds_read, not flat loads).
template <int VEC, typename CodeT>
__device__ __forceinline__ half8_t gather8(const uint8_t *book, const uint4_t &cw, int c0)
{
    if constexpr (VEC == 8) {
        return *reinterpret_cast<const half8_t *>(book + code_of<CodeT>(cw, c0) * 16u);
    } else if constexpr (VEC == 4) {
        const half4_t lo = *reinterpret_cast<const half4_t *>(book + code_of<CodeT>(cw, c0) * 8u);
        const half4_t hi = *reinterpret_cast<const half4_t *>(book + code_of<CodeT>(cw, c0 + 1) * 8u);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    } else {
        static_assert(VEC == 2, "vector length must be 2, 4 or 8");
        half2_t q[4];
#pragma unroll
        for (int i = 0; i < 4; i++) q[i] = *reinterpret_cast<const half2_t *>(book + code_of<CodeT>(cw, c0 + i) * 4u);
        const half4_t lo = __builtin_shufflevector(q[0], q[1], 0, 1, 2, 3);
        const half4_t hi = __builtin_shufflevector(q[2], q[3], 0, 1, 2, 3);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
}

// Physical 16-byte slot of logical chunk cc (0..7) of X-tile row `row`.
__device__ __forceinline__ int x_slot(int row, int cc) { return row * 8 + (cc ^ (row & 7)); }

template <int VEC, typename CodeT>
__global__ __launch_bounds__(kThreads, 1) void prefill_kernel(const half_t *__restrict__ x,
                                                              const CodeT *__restrict__ codes,
                                                              const half_t *__restrict__ cb,
                                                              half_t *__restrict__ y, int M, int K, int N,
                                                              int entries, int rows_per_cb, int tiles_m,
                                                              int tiles_n, int cb_lds_count)
{
    typedef PrefillCfg<VEC, CodeT> C;
    extern __shared__ __align__(16) uint8_t smem[];
    uint8_t *xbuf = smem;                       // 2 stages
    uint8_t *cb_lds = smem + 2 * kStageBytes;   // cb_lds_count codebooks

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, kg = lane >> 5;
    const int J = K / VEC;
    const int cb_bytes = entries * VEC * 2;

    // Tile mapping.  Consecutive workgroup ids go round-robin over the 8 XCDs; give each XCD
    // a contiguous band of tile columns so that its L2 sees one set of code rows and the X
    // rows are re-read by neighbours at about the same time.
    int wg = blockIdx.x;
    const int n_wg = tiles_m * tiles_n;
    {
        const int xcd = wg & 7, idx = wg >> 3;
        const int per_xcd = (n_wg + 7) >> 3;
        const int lin = xcd * per_xcd + idx;
        wg = (lin < n_wg && (n_wg & 7) == 0) ? lin : wg;
    }
    const int tm = wg % tiles_m, tn = wg / tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- codebooks of this tile's rows -> LDS ------------------------------------------
    const int g_first = n0 / rows_per_cb;
    {
        const uint4_t *src = reinterpret_cast<const uint4_t *>(cb + (int64_t)g_first * entries * VEC);
        const int n16 = cb_lds_count * cb_bytes / 16;
        const int g_total_16 = (int)(((int64_t)((N + rows_per_cb - 1) / rows_per_cb - g_first) * cb_bytes) / 16);
        for (int i = tid; i < n16; i += kThreads)
            if (i < g_total_16) reinterpret_cast<uint4_t *>(cb_lds)[i] = src[i];
    }

    // Per-lane W rows and codebook bases for the NB column blocks of this wave.
    uint32_t book[NB];  // byte offset of the lane's codebook inside smem
    const CodeT *code_row[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int n = min(n0 + wn * WN + nb * 32 + l32, N - 1);
        book[nb] = 2 * kStageBytes + (n / rows_per_cb - g_first) * cb_bytes;
        code_row[nb] = codes + (int64_t)n * J;
    }

    // ---- X staging: thread -> (row, chunk) of each stage ---------------------------------
    // chunk id q = i*256 + tid; row = q/8, cc = q%8 (k-group cc/4, step cc%4).
    const half_t *x_src[kChunksPerThread];
    int x_dst[kChunksPerThread];
    int x_koff[kChunksPerThread];
#pragma unroll
    for (int i = 0; i < kChunksPerThread; i++) {
        const int q = i * kThreads + tid;
        const int row = q >> 3, cc = q & 7;
        const int gm = min(m0 + row, M - 1);
        x_koff[i] = (cc >> 2) * C::K_LANE + (cc & 3) * 8;
        x_src[i] = x + (int64_t)gm * K + x_koff[i];
        x_dst[i] = x_slot(row, cc) * 16;
    }
    const int n_super = (K + C::K_SUPER - 1) / C::K_SUPER;
    const int n_stage = n_super * C::STAGES;

    uint4_t xreg[kChunksPerThread];
    auto issue_x = [&](int stage) {
        const int kbase = (stage / C::STAGES) * C::K_SUPER + (stage % C::STAGES) * 32;
#pragma unroll
        for (int i = 0; i < kChunksPerThread; i++) {
            uint4_t v = {0u, 0u, 0u, 0u};
            if (stage < n_stage && kbase + x_koff[i] < K) v = ld_global_16(x_src[i] + kbase);
            xreg[i] = v;
        }
    };
    auto commit_x = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kChunksPerThread; i++)
            *reinterpret_cast<uint4_t *>(xbuf + buf * kStageBytes + x_dst[i]) = xreg[i];
    };
    uint4_t cw[NB], cw_next[NB];
    auto issue_codes = [&](int super, uint4_t (&dst)[NB]) {
        const int k = super * C::K_SUPER + kg * C::K_LANE;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            uint4_t v = {0u, 0u, 0u, 0u};
            if (super < n_super && k < K) v = ld_global_16(code_row[nb] + k / VEC);
            dst[nb] = v;
        }
    };

    float16_t acc[NB][MB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[nb][mb][r] = 0.f;

    // ---- prologue ------------------------------------------------------------------------
    issue_codes(0, cw_next);
    issue_x(0);
    commit_x(0);
    issue_x(1);
    __syncthreads();

    // Operand read offsets inside a stage buffer: row = wm*128 + mb*32 + l32, chunk = kg*4 + s.
    int x_rd[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) x_rd[mb] = wm * WM + mb * 32 + l32;

    for (int super = 0; super < n_super; super++) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) cw[nb] = cw_next[nb];
        issue_codes(super + 1, cw_next);
#pragma unroll
        for (int t = 0; t < C::STAGES; t++) {
            const int stage = super * C::STAGES + t;
            const int buf = stage & 1;
            // Stage+1 data is in registers: park it in the other buffer (all waves finished
            // reading that buffer at the barrier that ended the previous iteration), then
            // start the loads of stage+2.
            commit_x(buf ^ 1);
            issue_x(stage + 2);
            const uint8_t *xs = xbuf + buf * kStageBytes;
#pragma unroll
            for (int s = 0; s < 4; s++) {
                half8_t wop[NB], xop[MB];
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    wop[nb] = gather8<VEC, CodeT>(smem + book[nb], cw[nb], (t * 4 + s) * C::CPO);
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
                    xop[mb] = *reinterpret_cast<const half8_t *>(xs + x_slot(x_rd[mb], kg * 4 + s) * 16);
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
#pragma unroll
                    for (int mb = 0; mb < MB; mb++)
                        acc[nb][mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wop[nb], xop[mb], acc[nb][mb], 0, 0, 0);
            }
            __syncthreads();
        }
    }

    // ---- epilogue: D[i][j], i = W row = 8*(r/4) + 4*kg + r%4, j = X row = l32 --------------
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        const int m = m0 + wm * WM + mb * 32 + l32;
        if (m >= M) continue;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int n = n0 + wn * WN + nb * 32 + 8 * q + 4 * kg;
                half_t *dst = y + (int64_t)m * N + n;
                if ((N & 3) == 0 && n + 3 < N) {
                    half4_t h = {(half_t)acc[nb][mb][4 * q], (half_t)acc[nb][mb][4 * q + 1],
                                 (half_t)acc[nb][mb][4 * q + 2], (half_t)acc[nb][mb][4 * q + 3]};
                    *reinterpret_cast<half4_t *>(dst) = h;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (n + r < N) dst[r] = (half_t)acc[nb][mb][4 * q + r];
                }
            }
        }
    }
}

constexpr size_t kLdsLimit = 160 * 1024;

int codebooks_per_tile(const ProblemB &p)
{
    // Worst case number of codebooks a 256-row band of W touches.
    int n;
    if (p.n_codebooks == 1) n = 1;
    else if (p.rows_per_cb >= BN && p.rows_per_cb % BN == 0) n = 1;
    else if (BN % p.rows_per_cb == 0) n = BN / p.rows_per_cb;
    else n = (BN + p.rows_per_cb - 1) / p.rows_per_cb + 1;
    return n < p.n_codebooks ? n : p.n_codebooks;
}

template <int VEC, typename CodeT>
hipError_t launch_prefill_typed(const ProblemB &p, hipStream_t s)
{
    const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    const int n_cb = codebooks_per_tile(p);
    const size_t smem = (size_t)2 * kStageBytes + (size_t)n_cb * p.entries * VEC * 2;
    auto kern = prefill_kernel<VEC, CodeT>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(kThreads), smem, s, p.x,
                       static_cast<const CodeT *>(p.codes), p.cb, p.y, p.M, p.K, p.N, p.entries, p.rows_per_cb,
                       tiles_m, tiles_n, n_cb);
    return hipGetLastError();
}

template <int VEC, typename CodeT>
bool prefill_cfg_supports(const ProblemB &p)
{
    return p.K % PrefillCfg<VEC, CodeT>::K_LANE == 0;
}

}  // namespace

bool prefill_supports(const ProblemB &p)
{
    if (p.M < 1 || p.N < 1 || p.K < 1) return false;
    if (p.vec != 2 && p.vec != 4 && p.vec != 8) return false;
    if (((size_t)p.entries * p.vec * 2) % 16 != 0) return false;
    if ((size_t)2 * kStageBytes + (size_t)codebooks_per_tile(p) * p.entries * p.vec * 2 > kLdsLimit) return false;
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? prefill_cfg_supports<8, uint8_t>(p) : prefill_cfg_supports<8, uint16_t>(p);
    case 4: return u8 ? prefill_cfg_supports<4, uint8_t>(p) : prefill_cfg_supports<4, uint16_t>(p);
    default: return u8 ? prefill_cfg_supports<2, uint8_t>(p) : false;  // 16-bit codes of 2-vectors: generic kernel
    }
}

hipError_t launch_prefill_b(const ProblemB &p, hipStream_t s)
{
    if (!prefill_supports(p)) return hipErrorInvalidValue;
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? launch_prefill_typed<8, uint8_t>(p, s) : launch_prefill_typed<8, uint16_t>(p, s);
    case 4: return u8 ? launch_prefill_typed<4, uint8_t>(p, s) : launch_prefill_typed<4, uint16_t>(p, s);
    default: return u8 ? launch_prefill_typed<2, uint8_t>(p, s) : hipErrorInvalidValue;
    }
}

}  // namespace vq
