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
//   * X tiles (256 rows x 64 k) go global -> LDS directly (global_load_lds_dwordx4, no register
//     staging) through four buffers (three when the codebooks are large), issued three stages
//     ahead of their use so that an HBM miss is covered by two stages of MFMA work.
//     The LDS has 64 banks of 4 bytes: two 128-byte tile rows form one 256-byte bank row and
//     the sixteen 16-byte chunks of a bank row are XOR-swizzled with the bank-row index, which
//     makes the operand reads (32 consecutive rows x one chunk per half wave) conflict free.
//     A direct load fills 64 consecutive slots per wave, so each lane fetches whatever chunk
//     the swizzle assigns to its slot.
//   * The MFMA operands of step s+1 are fetched from the LDS while step s is multiplied, also
//     across stage boundaries: the barrier that publishes stage i+2 sits a whole stage ahead
//     of its first read.
//   * fp32 accumulation; one rounding to fp16 in the epilogue, which transposes through the
//     LDS so that Y is written in 256-byte row segments.
//
// K order.  A lane of the 32x32x16 MFMA holds 8 consecutive k of one row; lanes 0-31 hold
// k-group 0 and lanes 32-63 k-group 1.  A "super stage" is the K range fed by one 16-byte
// code load per lane: lane group g covers the contiguous range
// [S*2*K_LANE + g*K_LANE, +K_LANE).  LDS stage t of the super stage holds, for both groups,
// the 32 k starting at offset t*32 of the group's range: two 64-byte pieces per X row.
// K must be a multiple of K_LANE; when it is not a multiple of 2*K_LANE the last super stage
// has no data for group 1 and the TAIL instantiation zeroes that group's W operand.
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

// Byte offset inside a stage buffer of logical 16-byte chunk cc (0..7) of X-tile row `row`.
__device__ __forceinline__ int x_offset(int row, int cc)
{
    const int bank_row = row >> 1;
    const int pos = (((row & 1) << 3) | cc) ^ (bank_row & 15);
    return (bank_row * 16 + pos) * 16;
}

// s_waitcnt for the vector-memory counter only (gfx9 encoding: vmcnt = simm16[15:14]:[3:0]).
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// 16-byte global load straight into the LDS: lane l writes smem[lds_base + 16*l ..].  The
// compiler knows nothing about this transfer, so every consumer sits behind an explicit
// wait_vmcnt + barrier.  `lds_base` must be wave-uniform.
__device__ __forceinline__ void load_to_lds_16(uint32_t lds_base, uint32_t voff, const void *sbase)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_base), "v"(voff), "s"(sbase)
                 : "memory");
}

// 16-byte global load into registers outside the compiler's vmcnt bookkeeping (so that its own
// waits never drain the LDS-bound loads in flight).  The result must not be touched before a
// wait_vmcnt that covers it; pin_loaded() ties that wait to the registers.
__device__ __forceinline__ uint4_t load_16_untracked(const void *p)
{
    uint4_t v;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template <int NB_>
__device__ __forceinline__ void pin_loaded(uint4_t (&r)[NB_])
{
#pragma unroll
    for (int i = 0; i < NB_; i++) asm volatile("" : "+v"(r[i]));
}

template <int VEC, typename CodeT, bool TAIL, int NS>
__global__ __launch_bounds__(kThreads, 1) void prefill_kernel(const half_t *__restrict__ x,
                                                              const CodeT *__restrict__ codes,
                                                              const half_t *__restrict__ cb,
                                                              half_t *__restrict__ y, int M, int K, int N,
                                                              int entries, int rows_per_cb, int tiles_m,
                                                              int tiles_n, int cb_lds_count)
{
    typedef PrefillCfg<VEC, CodeT> C;
    static_assert(NS == 3 || NS == 4, "three or four X stages");
    constexpr int D = NS - 1;                 // X loads run D stages ahead of the MFMAs
    constexpr int kInFlight = (D - 2) * kChunksPerThread;  // loads allowed to stay in flight at a stage end
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int kCbBase = NS * kStageBytes;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, kg = lane >> 5;
    const int J = K / VEC;
    const int cb_bytes = entries * VEC * 2;

    // Tile mapping.  Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
    // Re-number them so that an XCD works on consecutive tiles of the (row band major) tile
    // order: its workgroups then share a few 256-row bands of X, the large operand.
    int wg = blockIdx.x;
    const int n_wg = tiles_m * tiles_n;
    if ((n_wg & 7) == 0) wg = (wg & 7) * (n_wg >> 3) + (wg >> 3);
    const int tm = wg / tiles_n, tn = wg % tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    const int n_super = (K + C::K_SUPER - 1) / C::K_SUPER;
    const int n_stage = n_super * C::STAGES;

    // ---- per-lane W rows, codebook bases and code streams ---------------------------------
    const int g_first = n0 / rows_per_cb;
    uint32_t book[NB];  // byte offset of the lane's codebook inside smem
    const CodeT *code_row[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int n = min(n0 + wn * WN + nb * 32 + l32, N - 1);
        book[nb] = kCbBase + (n / rows_per_cb - g_first) * cb_bytes;
        code_row[nb] = codes + (int64_t)n * J;
    }
    auto issue_codes = [&](int super, uint4_t (&dst)[NB]) {
        super = min(super, n_super - 1);  // past the end: harmless re-reads instead of branches
        int k = super * C::K_SUPER + kg * C::K_LANE;
        if (TAIL && k >= K) k = 0;  // k-group 1 of a partial last super stage: any valid codes (operand is zeroed)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            // The codeword sizes below 16 bytes run out of registers; a register spilled while a
            // hand-issued load is still writing it would save stale data, so these variants
            // leave their code loads to the compiler's own (more conservative) waits.
            if constexpr (VEC == 8) dst[nb] = load_16_untracked(code_row[nb] + k / VEC);
            else dst[nb] = ld_global_16(code_row[nb] + k / VEC);
        }
    };

    // ---- X staging: global -> LDS directly ------------------------------------------------
    // Load i of wave w fills the 64 consecutive 16-byte slots [(4i+w)*64, +64) of a stage buffer;
    // the lane looks up which (row, chunk) lives in its slot under the swizzle and reads that.
    uint32_t x_voff[kChunksPerThread];
#pragma unroll
    for (int i = 0; i < kChunksPerThread; i++) {
        const int slot = (4 * i + wave) * 64 + lane;
        const int bank_row = slot >> 4;
        const int v = (slot & 15) ^ (bank_row & 15);
        const int row = 2 * bank_row + (v >> 3), cc = v & 7;
        const int gm = min(m0 + row, M - 1) - m0;
        const int koff = (cc >> 2) * C::K_LANE + (cc & 3) * 8;
        x_voff[i] = (uint32_t)(((int64_t)gm * K + koff) * 2);
    }
    const half_t *x_tile = x + (int64_t)m0 * K;
    // Load i (0..7) of a stage: one 16-byte chunk per lane, 1 KB per wave.
    auto issue_x_one = [&](int stage, int buf, int i) {
        stage = min(stage, n_stage - 1);  // past the end: harmless re-reads instead of branches
        const int super = stage / C::STAGES;
        const half_t *sbase = x_tile + super * C::K_SUPER + (stage % C::STAGES) * 32;
        uint32_t voff = x_voff[i];
        if (TAIL && super == n_super - 1) {
            // k-group 1 of the partial last super stage lies past K: read k-group 0's bytes again
            // (that group's W operand is zeroed).
            const int slot = (4 * i + wave) * 64 + lane;
            const int hi = (((slot & 15) ^ ((slot >> 4) & 15)) >> 2) & 1;
            voff -= hi ? C::K_LANE * 2 : 0;
        }
        load_to_lds_16(buf * kStageBytes + (4 * i + wave) * 1024, voff, sbase);
    };

    float16_t acc[NB][MB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[nb][mb][r] = 0.f;

    // Operand read offsets inside a stage buffer: row = wm*128 + mb*32 + l32, chunk = kg*4 + s.
    int x_rd[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int s = 0; s < 4; s++) x_rd[mb][s] = x_offset(wm * WM + mb * 32 + l32, kg * 4 + s);

    half8_t wop[2][NB], xop[2][MB];
    auto fetch_operands = [&](int set, int buf, const uint4_t (&c)[NB], int t, int s, bool last_super) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            half8_t w = gather8<VEC, CodeT>(smem + book[nb], c[nb], (t * 4 + s) * C::CPO);
            if (TAIL && last_super && kg == 1) w = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            wop[set][nb] = w;
        }
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
            xop[set][mb] = *reinterpret_cast<const half8_t *>(smem + buf * kStageBytes + x_rd[mb][s]);
    };

    // ---- prologue --------------------------------------------------------------------------
    uint4_t cw[NB], cw1[NB], cw2[NB];  // codes of super stage S, S+1, S+2
    issue_codes(0, cw);
    issue_codes(1, cw1);
    issue_codes(2, cw2);
#pragma unroll
    for (int d = 0; d < D; d++)
#pragma unroll
        for (int i = 0; i < kChunksPerThread; i++) issue_x_one(d, d, i);
    {
        const uint4_t *src = reinterpret_cast<const uint4_t *>(cb + (int64_t)g_first * entries * VEC);
        const int n16 = cb_lds_count * cb_bytes / 16;
        const int g_total_16 = (int)(((int64_t)((N + rows_per_cb - 1) / rows_per_cb - g_first) * cb_bytes) / 16);
        for (int i = tid; i < n16; i += kThreads)
            if (i < g_total_16) reinterpret_cast<uint4_t *>(smem + kCbBase)[i] = src[i];
    }
    wait_vmcnt<0>();
    pin_loaded(cw);
    pin_loaded(cw1);
    pin_loaded(cw2);
    __syncthreads();

    int buf = 0;  // buffer of the current stage; stage+j lives in (buf + j) % NS
    fetch_operands(0, buf, cw, 0, 0, n_super == 1);

    for (int super = 0; super < n_super; super++) {
        const bool last_super = super == n_super - 1;
        const bool next_last = super + 1 == n_super - 1;
#pragma unroll
        for (int t = 0; t < C::STAGES; t++) {
            const int stage = super * C::STAGES + t;
            const int buf_next = buf + 1 == NS ? 0 : buf + 1;
            // Stage+D goes into the buffer that was read during stage-1 (every wave has passed the
            // barrier that ended it); its eight loads are spread over the four steps.
            const int buf_load = buf == 0 ? NS - 1 : buf - 1;
#pragma unroll
            for (int s = 0; s < 4; s++) {
                const int cur = s & 1;
                // Fetch the operands of the next step and multiply this step's.  A wave issues in
                // order and an MFMA holds the matrix pipe for 32 cycles, so the LDS reads and their
                // address arithmetic are dealt out between the MFMAs instead of ahead of them.
                if (s < 3)
                    fetch_operands(cur ^ 1, buf, cw, t, s + 1, last_super);
                else if (t + 1 < C::STAGES)
                    fetch_operands(cur ^ 1, buf_next, cw, t + 1, 0, last_super);
                else
                    fetch_operands(cur ^ 1, buf_next, cw1, 0, 0, next_last);
                auto mfma = [&](int j) {
                    const int nb = j / MB, mb = j % MB;
                    acc[nb][mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wop[cur][nb], xop[cur][mb], acc[nb][mb], 0, 0, 0);
                };
#pragma unroll
                for (int j = 0; j < 8; j++) mfma(j);
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
                    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);  // a few VALU (gather addresses)
                }
                __builtin_amdgcn_sched_barrier(0);
                issue_x_one(stage + D, buf_load, 2 * s);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 8; j < 12; j++) mfma(j);
                __builtin_amdgcn_sched_barrier(0);
                issue_x_one(stage + D, buf_load, 2 * s + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 12; j < 16; j++) mfma(j);
                __builtin_amdgcn_sched_barrier(0);
            }
            // Publish stage+2: its loads (issued D-2 stages ago) must have landed in every wave.
            wait_vmcnt<kInFlight>();
            pin_loaded(cw2);
            __syncthreads();
            buf = buf_next;
        }
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            cw[nb] = cw1[nb];
            cw1[nb] = cw2[nb];
        }
        issue_codes(super + 3, cw2);
    }
    // Drain the clamped loads still in flight before the stage buffers are reused.
    wait_vmcnt<0>();
    pin_loaded(cw2);
    __syncthreads();

    // ---- epilogue: D[i][j], i = W row = 8*(r/4) + 4*kg + r%4, j = X row = l32 --------------
    if ((N & 7) == 0) {
        // Through the LDS: each wave transposes its 128x128 fp16 block, 64 rows at a time, in a
        // private region (row pitch 272 bytes) and stores 256-byte row segments.
        constexpr int kPitch = 272;
        uint8_t *stage_out = smem + wave * (64 * kPitch);
#pragma unroll
        for (int h = 0; h < 2; h++) {
#pragma unroll
            for (int mbh = 0; mbh < 2; mbh++) {
                const int mb = 2 * h + mbh;
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        half4_t hv = {(half_t)acc[nb][mb][4 * q], (half_t)acc[nb][mb][4 * q + 1],
                                      (half_t)acc[nb][mb][4 * q + 2], (half_t)acc[nb][mb][4 * q + 3]};
                        *reinterpret_cast<half4_t *>(stage_out + (mbh * 32 + l32) * kPitch + (nb * 32 + 8 * q + 4 * kg) * 2) = hv;
                    }
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int row = i * 4 + (lane >> 4), c = lane & 15;
                const uint4_t v = *reinterpret_cast<const uint4_t *>(stage_out + row * kPitch + c * 16);
                const int m = m0 + wm * WM + h * 64 + row;
                const int n = n0 + wn * WN + c * 8;
                if (m < M && n < N) st_global_16(y + (int64_t)m * N + n, v);
            }
        }
    } else {
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

size_t lds_bytes(const ProblemB &p, int n_stages)
{
    return (size_t)n_stages * kStageBytes + (size_t)codebooks_per_tile(p) * p.entries * p.vec * 2;
}

// Four X stages when the codebooks leave room for them, else three.
int pick_stages(const ProblemB &p) { return lds_bytes(p, 4) <= kLdsLimit ? 4 : 3; }

template <int VEC, typename CodeT>
hipError_t launch_prefill_typed(const ProblemB &p, hipStream_t s)
{
    typedef PrefillCfg<VEC, CodeT> C;
    const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    const int n_cb = codebooks_per_tile(p);
    const int ns = pick_stages(p);
    const size_t smem = lds_bytes(p, ns);
    const bool tail = (p.K % C::K_SUPER) != 0;
    auto kern = ns == 4 ? (tail ? prefill_kernel<VEC, CodeT, true, 4> : prefill_kernel<VEC, CodeT, false, 4>)
                        : (tail ? prefill_kernel<VEC, CodeT, true, 3> : prefill_kernel<VEC, CodeT, false, 3>);
    hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
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
    if (lds_bytes(p, 3) > kLdsLimit) return false;
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
