// Prefill kernel (large M): Y[M,N] = X[M,K] . W^T with W given as codes + codebook.
//
// MFMA-bound, and on this part MFMA-bound means power-bound: with random fp16 operands the
// matrix pipes draw enough power to pull the clock far below nominal, and what a tile costs is
// the energy it spends.  Two things follow.  v_mfma_f32_16x16x32_f16 needs clearly less energy
// per multiply-add than the 32x32x16 shape (a register-only loop reaches about 1.7 PFLOP/s with
// it against 1.3 PFLOP/s).  And every byte moved counts: X is walked in whole 128-byte lines.
//
// A 256-thread workgroup (4 waves, 2x2) computes a 256x256 tile of Y; each wave owns 128x128 of
// it as 8x8 pieces of 16x16 (256 fp32 accumulator registers, pinned in the AGPRs).
//
//   * W never exists as a tile anywhere: the codebooks of the workgroup's rows sit in the
//     LDS and every lane gathers the codeword of "its" W row straight into the 8-half MFMA
//     operand, in two 8-byte halves.
//   * X tiles (256 rows x 64 k, one cache line per row) and code tiles (256 rows x the codes
//     of 64 or 128 k) go global -> LDS directly (global_load_lds_dwordx4, no register staging)
//     through four buffers (fewer when the codebooks are large), issued so far ahead that a
//     stage's loads have two whole stages of MFMA work to land.
//     The LDS has 64 banks of 4 bytes: two 128-byte X rows form one 256-byte bank row and
//     the sixteen 16-byte chunks of a bank row are XOR-swizzled with the bank-row index, which
//     makes the operand reads (16 consecutive rows x one chunk per quarter wave) conflict free.
//     A direct load fills 64 consecutive slots per wave, so each lane fetches whatever chunk
//     the swizzle assigns to its slot.
//   * One MFMA step (k = 32) is 64 MFMAs on 8 W pieces and 8 X pieces, walked as four 4x4
//     quadrants.  The walk alternates between two orders so that every group of four pieces has
//     its last use at least one quadrant (16 MFMAs, 256 cycles) before the group's successor is
//     first needed: each quadrant re-loads exactly one group of four operands into the registers
//     that just went dead, also across stage boundaries.  No operand is double buffered.
//   * fp32 accumulation; one rounding to fp16 in the epilogue, which transposes through the
//     LDS so that Y is written in 256-byte row segments.
//
// K is walked in order: stage i is k in [64 i, 64 i + 64), MFMA step s of it the 32 k from
// 32 s on, and lane group g (lanes 16g..16g+15) holds the 8 k from 8 g on.  K must be a
// multiple of the k that 16 bytes of codes cover; a last stage of 32 k runs in the TAIL
// instantiation, which points the W operands of the missing step at zeros.
#include "vq_prefill_common.h"

#include <type_traits>

namespace vq {

namespace {

// The prologue of the 256x256 kernel puts up to three X loads of stage D into buffer D: 12 KB from its
// start on are taken, the rest is free until the main loop.
constexpr int kWideSplitSkip = 12 * 1024;

// SPLIT: the codebooks lie in the LDS in the split layout (vq_prefill_common.h).
template <int VEC, typename CodeT, bool TAIL, int NS, bool SPLIT>
__global__ __launch_bounds__(kThreads, 1) void prefill_kernel(const half_t *__restrict__ x,
                                                              const CodeT *__restrict__ codes,
                                                              const half_t *__restrict__ cb,
                                                              half_t *__restrict__ y,
                                                              const half_t *__restrict__ bias, int M, int K, int N,
                                                              int n_begin, int ldn, int entries, int rows_per_cb,
                                                              int tiles_m, int tiles_n, int cb_lds_count, int gated)
{
    // The launch covers the W rows (columns of Y) [n_begin, N) of a problem with ldn rows in all:
    // ldn is the row stride of Y and counts the codebooks, N bounds the rows that are touched.
    typedef PrefillCfg<VEC, CodeT> C;
    static_assert(NS >= 2 && NS <= 4, "two to four X stages");
    constexpr int D = NS - 1;                 // loads run D stages ahead of the MFMAs
    constexpr int NC = C::code_bufs(NS);
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int kCodeBase = NS * kStageBytes;
    constexpr int kCbBase = kCodeBase + NC * C::kTileBytes;
    constexpr int kSplitTemp = D * kStageBytes + kWideSplitSkip;  // where the plain copy of the codebooks waits
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const bool mirrored = wm == 1;  // which of the two walks through a stage the wave takes
    const int r16 = lane & 15, kg = lane >> 4;
    const int J = K / VEC;
    const int cb_bytes = entries * VEC * 2;
    // 16 zero bytes behind the codebooks, whose region is padded to whole 1 KB copy steps
    const uint32_t zero_off = kCbBase + ((cb_lds_count * cb_bytes + 1023) & ~1023);

    // Tile mapping.  Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
    // Re-number them so that an XCD works on consecutive tiles of the (row band major) tile
    // order: its workgroups then share a few 256-row bands of X, the large operand.
    int wg = blockIdx.x;
    const int n_wg = tiles_m * tiles_n;
    if ((n_wg & 7) == 0) wg = (wg & 7) * (n_wg >> 3) + (wg >> 3);
    const int tm = wg / tiles_n, tn = wg % tiles_n;
    const int m0 = tm * BM, n0 = n_begin + tn * BN;
    const int n_stage = (K + kStageK - 1) / kStageK;
    const int n_super = (n_stage + C::STAGES - 1) / C::STAGES;

    // ---- per-lane codebook bases ------------------------------------------------------------
    const int g_first = n0 / rows_per_cb;
    uint32_t book[NP];  // byte offset inside smem of the codebook of W row j*16 + r16 of the wave tile
    {
        const int n_base = min(n0 + wn * WN, N - 1);
        const int g_base = n_base / rows_per_cb, rem_base = n_base - g_base * rows_per_cb;
        const float rcp = 1.0f / (float)rows_per_cb;
#pragma unroll
        for (int j = 0; j < NP; j++) {
            const int n = min(n0 + wn * WN + j * 16 + r16, N - 1);
            const int g = g_base + small_div(n - n_base + rem_base, rows_per_cb, rcp);
            book[j] = kCbBase + (g - g_first) * cb_bytes;
        }
    }

    // ---- staging: global -> LDS directly ----------------------------------------------------
    // X load i of wave w fills the 64 consecutive 16-byte slots [(4i+w)*64, +64) of a stage
    // buffer; the lane looks up which (row, chunk) lives in its slot under the swizzle and reads
    // that.  Chunk cc of a row is the 8 k from 8 cc on.
    uint32_t x_voff[kChunksPerThread];
    uint32_t x_voff_tail[TAIL ? kChunksPerThread : 1];  // last stage of 32 k: chunks 4..7 re-read chunks 0..3
#pragma unroll
    for (int i = 0; i < kChunksPerThread; i++) {
        const int slot = (4 * i + wave) * 64 + lane;
        const int bank_row = slot >> 4;
        const int v = (slot & 15) ^ (bank_row & 15);
        const int row = 2 * bank_row + (v >> 3), cc = v & 7;
        const int gm = min(m0 + row, M - 1) - m0;
        x_voff[i] = (uint32_t)(((int64_t)gm * K + cc * 8) * 2);
        if (TAIL) x_voff_tail[i] = x_voff[i] - (cc >= 4 ? 64u : 0u);
    }
    const half_t *x_tile = x + (int64_t)m0 * K;
    // X load i (0..7) of stage `stage` into buffer `buf`: one 16-byte chunk per lane, 1 KB per
    // wave.  Past the end the last stage is read again (harmless) instead of branching.
    auto issue_x = [&](int i, int buf, int stage) {
        const bool is_last = stage >= n_stage - 1;
        const half_t *sbase = x_tile + min(stage, n_stage - 1) * kStageK;
        uint32_t voff = x_voff[i];
        if (TAIL) voff = is_last ? x_voff_tail[i] : voff;
        load_to_lds_16(buf * kStageBytes + (4 * i + wave) * 1024, voff, sbase);
    };
    // Code tile of a super stage: chunk c of tile row w*64 + lane goes to [c][row]; 1 KB per wave.
    const CodeT *code_tile = codes + (int64_t)n0 * J;
    const uint32_t code_voff = (uint32_t)(min(wave * 64 + lane, N - 1 - n0) * J * C::CSZ);
    auto issue_codes = [&](int c, int cbuf, int super) {
        const bool is_last = super >= n_super - 1;
        super = min(super, n_super - 1);
        // a last stage of 32 k has only chunk 0; read it twice
        const int chunk = (TAIL && is_last) ? 0 : c;
        const uint8_t *sbase = reinterpret_cast<const uint8_t *>(code_tile) + (int64_t)super * (C::K_SUPER / VEC * C::CSZ) + chunk * 16;
        load_to_lds_16(kCodeBase + cbuf * C::kTileBytes + c * (BN * 16) + wave * 1024, code_voff, sbase);
    };

    float4_t acc[NP][MP];
#pragma unroll
    for (int j = 0; j < NP; j++)
#pragma unroll
        for (int i = 0; i < MP; i++) acc[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};

    // Operand read offsets inside a stage buffer: X piece i is rows wm*128 + i*16 + r16; the
    // lane's chunk in MFMA step s is s*4 + kg.  Two pieces further is 16 bank rows (4 KB) on and
    // leaves the swizzle unchanged.
    int x_rd[2][2];
#pragma unroll
    for (int par = 0; par < 2; par++)
#pragma unroll
        for (int s = 0; s < 2; s++) x_rd[par][s] = x_offset(wm * WM + par * 16 + r16, s * 4 + kg);
    // Where the lane's codes of W piece 0 start inside a code tile.
    const uint32_t code_rd = kCodeBase + (wn * WN + r16) * 16 + kg * C::RB;

    half4_t wlo[NP], whi[NP];
    half8_t xp[MP];
    uint32_t cr[2][4];  // codes behind the two W groups whose gathers come next
    // X piece i of MFMA step s out of stage buffer `buf`
    auto load_x1 = [&](int i, int buf, int s) {
        xp[i] = *reinterpret_cast<const half8_t *>(smem + buf * kStageBytes + x_rd[i & 1][s] + (i >> 1) * 4096);
    };
    // the codes of W piece j for MFMA step s of stage t (of its super stage) out of code buffer `cbuf`
    auto load_c1 = [&](int set, int j, int cbuf, int t, int s) {
        const int pos = (t % C::STAGES) * 2 * C::HALF + s * C::HALF;   // + kg*RB stays inside the 16-byte chunk
        cr[set][j & 3] = read_codes<C::RB>(smem + code_rd + cbuf * C::kTileBytes + (pos / 16) * (BN * 16) + j * 256 + pos % 16);
    };
    // the two halves of W piece j from the codes read before
    // 8-vectors out of the plain table: one 16-byte gather per operand.  (This kernel is bound by the energy it spends,
    // not by issue slots or LDS cycles: half as many gather instructions took 1 % off C4 and C5, while the conflicts
    // the split layout saves cost it nothing.  The smaller tiles, which the LDS does bound, gather in halves.)
    constexpr bool kWholeGather = VEC == 8 && !SPLIT;
    auto load_w1 = [&](int set, int j, bool zero) {
        if constexpr (kWholeGather) {
            uint32_t a = book[j] + cr[set][j & 3] * 16u;
            if (TAIL) a = zero ? zero_off : a;
            const half8_t v = *reinterpret_cast<const half8_t *>(smem + a);
            wlo[j] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
            whi[j] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
        } else {
            wlo[j] = gather4<VEC, CodeT, TAIL, SPLIT>(smem, book[j], cr[set][j & 3], 0, zero, zero_off);
        }
    };
    auto load_w2 = [&](int set, int j, bool zero) {
        if constexpr (!kWholeGather) whi[j] = gather4<VEC, CodeT, TAIL, SPLIT>(smem, book[j], cr[set][j & 3], 1, zero, zero_off);
    };
    // MFMA f of group p of the 4x4 quadrant (jh, ih): a group is W piece p against the four X
    // pieces, or (x_outer) X piece p against the four W pieces
    auto mfma_one = [&](int jh, int ih, int p, int f, bool x_outer) {
        const int j = jh * 4 + (x_outer ? f : p), i = ih * 4 + (x_outer ? p : f);
        mfma_in_place(acc[j][i], __builtin_shufflevector(wlo[j], whi[j], 0, 1, 2, 3, 4, 5, 6, 7), xp[i]);
    };

    // ---- prologue --------------------------------------------------------------------------
    // Loads complete in the order they were issued, so one count serves all of them: the
    // codebooks first, then X stages 0..D-1 with the code tiles of the super stages that open
    // there, then what the two quadrants ahead of stage 0 would have issued for stage D.
    // loads a stage brings along: 8 of X, plus its code tile when it opens a super stage
    auto loads_of = [](int stage_mod) constexpr { return kChunksPerThread + (stage_mod % C::STAGES == 0 ? C::CH : 0); };
    {
        const uint8_t *src = reinterpret_cast<const uint8_t *>(cb + (int64_t)g_first * entries * VEC);
        const int n16 = cb_lds_count * cb_bytes / 16;
        const int g_total_16 = (int)(((int64_t)((ldn + rows_per_cb - 1) / rows_per_cb - g_first) * cb_bytes) / 16);
        // past the last codebook: read its last 16 bytes again.  SPLIT: a plain copy first, into the
        // part of X buffer D that the prologue's loads of stage D leave alone, re-laid below.
        const int dst = SPLIT ? kSplitTemp : kCbBase;
        for (int i0 = wave * 64; i0 < n16; i0 += kThreads)
            load_to_lds_16(dst + i0 * 16, (uint32_t)min(i0 + lane, g_total_16 - 1) * 16u, src);
    }
#pragma unroll
    for (int d = 0; d < D; d++) {
        if (d % C::STAGES == 0) {
#pragma unroll
            for (int c = 0; c < C::CH; c++) issue_codes(c, (d / C::STAGES) % NC, d / C::STAGES);
        }
#pragma unroll
        for (int i = 0; i < kChunksPerThread; i++) issue_x(i, d, d);
    }
    if (D % C::STAGES == 0) {
#pragma unroll
        for (int c = 0; c < C::CH; c++) issue_codes(c, (D / C::STAGES) % NC, D / C::STAGES);
    }
    issue_x(0, D, D);
    issue_x(1, D, D);
    if (mirrored) issue_x(2, D, D);  // the mirrored walk has three quadrants behind its barrier
    if (tid < 4) reinterpret_cast<uint32_t *>(smem + zero_off)[tid] = 0u;
    {
        // stage 0 (and everything older) must have landed; stages 1..D may be in flight
        constexpr int in_flight = [&]() constexpr {
            int n = 2 + (D % C::STAGES == 0 ? C::CH : 0);
            for (int d = 1; d < D; d++) n += loads_of(d);
            return n;
        }();
        if (mirrored) wait_vmcnt<in_flight + 1>();
        else wait_vmcnt<in_flight>();
    }
    __syncthreads();
    if constexpr (SPLIT) {
        split_codebooks(smem, kSplitTemp, kCbBase, cb_lds_count, tid, kThreads);
        __syncthreads();
    }
    int buf = 0;   // X buffer of the current stage; stage+j lives in (buf + j) % NS
    int cbuf = 0;  // code buffer of the current super stage; super+j lives in (cbuf + j) % NC
#pragma unroll
    for (int p = 0; p < 4; p++) {
        load_c1(0, p, cbuf, 0, 0);
        load_c1(1, 4 + p, cbuf, 0, 0);
    }
#pragma unroll
    for (int p = 0; p < 4; p++) {
        load_w1(0, p, false);
        load_w2(0, p, false);
        load_x1(p, buf, 0);
    }

    // One quadrant: four groups of four MFMAs.  A wave issues one instruction every four cycles
    // and a 16x16x32 MFMA holds the matrix pipe for sixteen, so at most three other instructions
    // fit between two MFMAs without starving the pipe: every MFMA is fenced and the other work
    // is dealt out by hand.  In the middle of group p, LOADP(p) re-fills one operand register
    // that went dead in the quadrant before and CODEP(p) reads the codes of a W piece that the
    // next quadrant gathers; the operand loaded during the previous quadrant is walked in the
    // outer position, so that every piece has 15 MFMAs between its load and its first use.  One
    // of the stage's eight X loads follows group 0, a code tile load group 2.
#define VQ_FENCE __builtin_amdgcn_sched_barrier(0)
#define VQ_NONE(p) do {} while (0)
#define VQ_QUADRANT(LOADP, CODEP, jh, ih, x_outer, xi, TGT)                         \
    _Pragma("unroll") for (int p_ = 0; p_ < 4; p_++) {                              \
        mfma_one(jh, ih, p_, 0, x_outer); VQ_FENCE;                                 \
        LOADP(p_); VQ_FENCE;                                                        \
        mfma_one(jh, ih, p_, 1, x_outer); VQ_FENCE;                                 \
        LOADP##2(p_); CODEP(p_); VQ_FENCE;                                          \
        mfma_one(jh, ih, p_, 2, x_outer); VQ_FENCE;                                 \
        if (p_ == 0) { issue_x(xi, TGT##_buf, TGT##_stage); VQ_FENCE; }             \
        if (p_ == 2 && TGT##_codes && xi < C::CH) { issue_codes(xi, TGT##_cbuf, TGT##_super); VQ_FENCE; } \
        mfma_one(jh, ih, p_, 3, x_outer); VQ_FENCE;                                 \
    }

    // Two walks.  Gathers are the expensive LDS reads (random codewords collide in the banks), and
    // a walk loads W in four of its eight quadrants and X in the other four.  If every wave loaded
    // W at the same time the LDS would be saturated in those quadrants and idle in the others, so
    // the waves of the lower half of the tile take the mirrored walk (roles of W and X swapped):
    // at any time two waves gather and two read X.
    //
    //   plain:     (Wl,Xl) (Wh,Xl) (Wh,Xh) (Wl,Xh) | (Wh,Xl) (Wl,Xl) | barrier | (Wl,Xh) (Wh,Xh)
    //     loads     Wh      Xh      Xl'     Wh'       Wl'     Xh'                  Xl"     Wl"
    //   mirrored:  (Wl,Xl) (Wl,Xh) (Wh,Xh) (Wh,Xl) | (Wl,Xh) | barrier | (Wl,Xl) (Wh,Xl) (Wh,Xh)
    //     loads     Xh      Wh      Wl'     Xh'       Xl'                 Wh'     Wl"     Xl"
    //
    // (' = step B of the stage, " = step A of the next stage).  The barrier of a stage sits behind
    // its last read of X and of its code tile.  From there on the stage's buffer is free and the
    // quadrants left issue the first X loads of stage+1+D into it (and that stage's code tile,
    // when it opens a super stage); the quadrants ahead of the barrier issue the rest of the eight
    // X loads of stage+D into the buffer of stage-1.  A stage's loads so have two whole stages to
    // land before the barrier that publishes them.
#define VQ_STAGE_SETUP                                                              \
    constexpr int t = decltype(t_const)::value;                                     \
    const int stage = super * C::STAGES + t;                                        \
    const int buf_next = buf + 1 == NS ? 0 : buf + 1;                               \
    const int tgt_a_buf = buf == 0 ? NS - 1 : buf - 1, tgt_a_stage = stage + D;     \
    constexpr bool tgt_a_codes = false;                                             \
    const int tgt_a_cbuf = 0, tgt_a_super = 0;                                      \
    const int tgt_b_buf = buf, tgt_b_stage = stage + 1 + D;                         \
    constexpr bool tgt_b_codes = (t + 1 + D) % C::STAGES == 0;                      \
    constexpr int d_super = (t + 1 + D) / C::STAGES;                                \
    const int tgt_b_super = super + d_super;                                        \
    const int tgt_b_cbuf = (cbuf + d_super) % NC;                                   \
    /* the stage after this one: same super stage or the next */                   \
    constexpr bool same_super = t + 1 < C::STAGES;                                  \
    const int cbuf_n = same_super ? cbuf : (cbuf + 1 == NC ? 0 : cbuf + 1);         \
    constexpr int t_n = same_super ? t + 1 : 0;                                     \
    /* a last stage of 32 k has no step 1 */                                       \
    const bool no_b = TAIL && stage == n_stage - 1;                                 \
    /* publish stage+1: in flight may be what stages +2..+D bring along */         \
    constexpr int in_flight = [&]() constexpr {                                     \
        int n = 0;                                                                  \
        for (int d = 2; d <= D; d++) n += loads_of(t + d);                          \
        return n;                                                                   \
    }();                                                                            \
    VQ_FENCE

#define L_XHI_A(p) load_x1(4 + (p), buf, 0)
#define L_XLO_B(p) load_x1((p), buf, 1)
#define L_XHI_B(p) load_x1(4 + (p), buf, 1)
#define L_XLO_N(p) load_x1((p), buf_next, 0)
#define L_XHI_A2(p) do {} while (0)
#define L_XLO_B2(p) do {} while (0)
#define L_XHI_B2(p) do {} while (0)
#define L_XLO_N2(p) do {} while (0)
    if (!mirrored) {
        for (int super = 0; super < n_super; super++) {
            // stage t (a compile-time 0 or 1) of the super stage
            auto stage_body = [&](auto t_const) {
                VQ_STAGE_SETUP;
                // W low/X low are in registers, the codes of W high in cr[1]
#define L_WHI_A(p) load_w1(1, 4 + (p), false)
#define L_WHI_A2(p) load_w2(1, 4 + (p), false)
#define L_WHI_B(p) load_w1(0, 4 + (p), no_b)
#define L_WHI_B2(p) load_w2(0, 4 + (p), no_b)
#define L_WLO_B(p) load_w1(1, (p), no_b)
#define L_WLO_B2(p) load_w2(1, (p), no_b)
#define L_WLO_N(p) load_w1(0, (p), false)
#define L_WLO_N2(p) load_w2(0, (p), false)
#define C_WHI_B(p) load_c1(0, 4 + (p), cbuf, t, 1)
#define C_WLO_B(p) load_c1(1, (p), cbuf, t, 1)
#define C_WLO_N(p) load_c1(0, (p), cbuf_n, t_n, 0)
#define C_WHI_N(p) load_c1(1, 4 + (p), cbuf_n, t_n, 0)
                VQ_QUADRANT(L_WHI_A, VQ_NONE, 0, 0, false, 2, tgt_a);   // W low (just loaded) x X low
                VQ_QUADRANT(L_XHI_A, VQ_NONE, 1, 0, false, 3, tgt_a);   // W high (just loaded) x X low
                VQ_QUADRANT(L_XLO_B, C_WHI_B, 1, 1, true, 4, tgt_a);    // W high x X high (just loaded)
                VQ_QUADRANT(L_WHI_B, C_WLO_B, 0, 1, false, 5, tgt_a);   // W low x X high
                VQ_QUADRANT(L_WLO_B, VQ_NONE, 1, 0, false, 6, tgt_a);   // W high' (just loaded) x X low'
                VQ_QUADRANT(L_XHI_B, VQ_NONE, 0, 0, false, 7, tgt_a);   // W low' (just loaded) x X low'
                wait_vmcnt<in_flight>();
                __syncthreads();
                VQ_QUADRANT(L_XLO_N, C_WLO_N, 0, 1, true, 0, tgt_b);    // W low' x X high' (just loaded)
                VQ_QUADRANT(L_WLO_N, C_WHI_N, 1, 1, false, 1, tgt_b);   // W high' x X high'
#undef L_WHI_A
#undef L_WHI_A2
#undef L_WHI_B
#undef L_WHI_B2
#undef L_WLO_B
#undef L_WLO_B2
#undef L_WLO_N
#undef L_WLO_N2
#undef C_WHI_B
#undef C_WLO_B
#undef C_WLO_N
#undef C_WHI_N
                buf = buf_next;
            };
            stage_body(std::integral_constant<int, 0>{});
            if constexpr (C::STAGES == 2) stage_body(std::integral_constant<int, 1>{});
            cbuf = cbuf + 1 == NC ? 0 : cbuf + 1;
        }
    } else {
        for (int super = 0; super < n_super; super++) {
            auto stage_body = [&](auto t_const) {
                VQ_STAGE_SETUP;
                // W low/X low are in registers
#define C_WHI_A(p) load_c1(0, 4 + (p), cbuf, t, 0)
#define L_WHI_A(p) load_w1(0, 4 + (p), false)
#define L_WHI_A2(p) load_w2(0, 4 + (p), false)
#define C_WLO_B(p) load_c1(1, (p), cbuf, t, 1)
#define L_WLO_B(p) load_w1(1, (p), no_b)
#define L_WLO_B2(p) load_w2(1, (p), no_b)
#define C_WHI_B(p) load_c1(0, 4 + (p), cbuf, t, 1)
#define L_WHI_B(p) load_w1(0, 4 + (p), no_b)
#define L_WHI_B2(p) load_w2(0, 4 + (p), no_b)
#define C_WLO_N(p) load_c1(1, (p), cbuf_n, t_n, 0)
#define L_WLO_N(p) load_w1(1, (p), false)
#define L_WLO_N2(p) load_w2(1, (p), false)
                VQ_QUADRANT(L_XHI_A, C_WHI_A, 0, 0, true, 3, tgt_a);    // W low x X low (just loaded)
                VQ_QUADRANT(L_WHI_A, C_WLO_B, 0, 1, true, 4, tgt_a);    // W low x X high (just loaded)
                VQ_QUADRANT(L_WLO_B, VQ_NONE, 1, 1, false, 5, tgt_a);   // W high (just loaded) x X high
                VQ_QUADRANT(L_XHI_B, VQ_NONE, 1, 0, false, 6, tgt_a);   // W high x X low
                VQ_QUADRANT(L_XLO_B, C_WHI_B, 0, 1, true, 7, tgt_a);    // W low' x X high' (just loaded)
                wait_vmcnt<in_flight>();
                __syncthreads();
                VQ_QUADRANT(L_WHI_B, C_WLO_N, 0, 0, true, 0, tgt_b);    // W low' x X low' (just loaded)
                VQ_QUADRANT(L_WLO_N, VQ_NONE, 1, 0, false, 1, tgt_b);   // W high' (just loaded) x X low'
                VQ_QUADRANT(L_XLO_N, VQ_NONE, 1, 1, false, 2, tgt_b);   // W high' x X high'
#undef C_WHI_A
#undef L_WHI_A
#undef L_WHI_A2
#undef C_WLO_B
#undef L_WLO_B
#undef L_WLO_B2
#undef C_WHI_B
#undef L_WHI_B
#undef L_WHI_B2
#undef C_WLO_N
#undef L_WLO_N
#undef L_WLO_N2
                buf = buf_next;
            };
            stage_body(std::integral_constant<int, 0>{});
            if constexpr (C::STAGES == 2) stage_body(std::integral_constant<int, 1>{});
            cbuf = cbuf + 1 == NC ? 0 : cbuf + 1;
        }
    }
#undef L_XHI_A
#undef L_XHI_A2
#undef L_XLO_B2
#undef L_XHI_B2
#undef L_XLO_N2
#undef L_XLO_B
#undef L_XHI_B
#undef L_XLO_N
#undef VQ_STAGE_SETUP
#undef VQ_QUADRANT
#undef VQ_FENCE
    // Drain the clamped loads still in flight before the stage buffers are reused.
    wait_vmcnt<0>();
    __syncthreads();
    // the last MFMAs must have left the pipe before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    // ---- epilogue: lane holds Y[m = i*16 + r16][n = j*16 + 4*kg + 0..3] of its wave tile ------
    auto epilogue = [&](auto has_bias_const) {
        constexpr bool HB = decltype(has_bias_const)::value;
        float bj[NP][4];
#pragma unroll
        for (int j = 0; j < NP; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int n = n0 + wn * WN + j * 16 + 4 * kg + e;
                bj[j][e] = HB && n < N ? (float)bias[n] : 0.f;
            }
        if ((ldn & 7) == 0) {
            // Through the LDS: each wave transposes its 128x128 fp16 block, 64 rows at a time, in a
            // private region (row pitch 272 bytes) and stores 256-byte row segments.
            constexpr int kPitch = 272;
            uint8_t *stage_out = smem + wave * (64 * kPitch);
#pragma unroll
            for (int h = 0; h < 2; h++) {
#pragma unroll
                for (int ii = 0; ii < 4; ii++) {
                    const int i = 4 * h + ii;
#pragma unroll
                    for (int j = 0; j < NP; j++)
                        *reinterpret_cast<half4_t *>(stage_out + (ii * 16 + r16) * kPitch + (j * 16 + 4 * kg) * 2) =
                            round4<HB>(acc[j][i], bj[j]);
                }
#pragma unroll
                for (int it = 0; it < 16; it++) {
                    const int row = it * 4 + (lane >> 4), c = lane & 15;
                    const uint4_t v = *reinterpret_cast<const uint4_t *>(stage_out + row * kPitch + c * 16);
                    const int m = m0 + wm * WM + h * 64 + row;
                    const int n = n0 + wn * WN + c * 8;
                    if (m < M && n < N) st_global_16_streaming(y + (int64_t)m * ldn + n, v);
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
                    half_t *dst = y + (int64_t)m * ldn + n;
                    const half4_t hv = round4<HB>(acc[j][i], bj[j]);
                    if ((ldn & 3) == 0 && n + 3 < N) {
                        *reinterpret_cast<half4_t *>(dst) = hv;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (n + e < N) dst[e] = hv[e];
                    }
                }
            }
        }
    };
    if (gated) {
        // gate and up rows of W interleaved in groups of 16: a lane holds both factors of its outputs
        if (bias) store_gated<NP, MP, true>(acc, y, bias, M, N, ldn, m0 + wm * WM, n0 + wn * WN, r16, kg);
        else store_gated<NP, MP, false>(acc, y, bias, M, N, ldn, m0 + wm * WM, n0 + wn * WN, r16, kg);
        return;
    }
    if (bias) epilogue(std::true_type{});
    else epilogue(std::false_type{});
}

// ---- the 256x128 tile ------------------------------------------------------------------------
// When the 256x256 tiles of a problem are fewer than the compute units (medium M, small N), a
// tile half as wide puts twice as many units to work: the same 256 threads (2x2 waves), 256
// rows of X, 128 rows of W, each wave 128x64 as 8 X pieces x 4 W pieces.  Half the accumulators
// leave room to double buffer every operand, so the schedule is plain: while MFMA step s
// multiplies, all operands of step s+1 are loaded (per quadrant of 16 MFMAs: four X reads, two W
// pieces gathered in halves, the codes of the two pieces after those), everything at least 16
// MFMAs ahead of its use.  A stage is 64 MFMAs per wave.  Its barrier sits behind the first
// quadrant: the loads of stage+3 (two per quadrant) start right behind it, into the buffer that
// stage-1 was read from, and the data of stage+1 is read from the second quadrant on.
constexpr int NPN = 4;                 // W pieces per wave in the narrow tile
constexpr int WNN = NPN * 16, BNN = 2 * WNN;

template <int VEC, typename CodeT, bool TAIL, bool SPLIT>
__global__ __launch_bounds__(kThreads, 1) void prefill_narrow_kernel(const half_t *__restrict__ x,
                                                                     const CodeT *__restrict__ codes,
                                                                     const half_t *__restrict__ cb,
                                                                     half_t *__restrict__ y,
                                                                     const half_t *__restrict__ bias, int M, int K,
                                                                     int N, int n_begin, int ldn, int entries,
                                                                     int rows_per_cb, int tiles_m, int tiles_n,
                                                                     int cb_lds_count, int gated)
{
    typedef PrefillCfg<VEC, CodeT> C;
    constexpr int NS = 4, D = NS - 1;
    constexpr int NC = C::code_bufs(NS);
    constexpr int kTile = C::CH * BNN * 16;   // code tile: [chunk][128 rows][16 bytes]
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int kCodeBase = NS * kStageBytes;
    constexpr int kCbBase = kCodeBase + NC * kTile;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int r16 = lane & 15, kg = lane >> 4;
    const int J = K / VEC;
    const int cb_bytes = entries * VEC * 2;
    const uint32_t zero_off = kCbBase + ((cb_lds_count * cb_bytes + 1023) & ~1023);

    int wg = blockIdx.x;
    const int n_wg = tiles_m * tiles_n;
    if ((n_wg & 7) == 0) wg = (wg & 7) * (n_wg >> 3) + (wg >> 3);
    const int tm = wg / tiles_n, tn = wg % tiles_n;
    const int m0 = tm * BM, n0 = n_begin + tn * BNN;
    const int n_stage = (K + kStageK - 1) / kStageK;
    const int n_super = (n_stage + C::STAGES - 1) / C::STAGES;

    const int g_first = n0 / rows_per_cb;
    uint32_t book[NPN];
    {
        const int n_base = min(n0 + wn * WNN, N - 1);
        const int g_base = n_base / rows_per_cb, rem_base = n_base - g_base * rows_per_cb;
        const float rcp = 1.0f / (float)rows_per_cb;
#pragma unroll
        for (int j = 0; j < NPN; j++) {
            const int n = min(n0 + wn * WNN + j * 16 + r16, N - 1);
            const int g = g_base + small_div(n - n_base + rem_base, rows_per_cb, rcp);
            book[j] = kCbBase + (g - g_first) * cb_bytes;
        }
    }

    uint32_t x_voff[kChunksPerThread];
    uint32_t x_voff_tail[TAIL ? kChunksPerThread : 1];
#pragma unroll
    for (int i = 0; i < kChunksPerThread; i++) {
        const int slot = (4 * i + wave) * 64 + lane;
        const int bank_row = slot >> 4;
        const int v = (slot & 15) ^ (bank_row & 15);
        const int row = 2 * bank_row + (v >> 3), cc = v & 7;
        const int gm = min(m0 + row, M - 1) - m0;
        x_voff[i] = (uint32_t)(((int64_t)gm * K + cc * 8) * 2);
        if (TAIL) x_voff_tail[i] = x_voff[i] - (cc >= 4 ? 64u : 0u);
    }
    const half_t *x_tile = x + (int64_t)m0 * K;
    auto issue_x = [&](int i, int buf, int stage) {
        const bool is_last = stage >= n_stage - 1;
        const half_t *sbase = x_tile + min(stage, n_stage - 1) * kStageK;
        uint32_t voff = x_voff[i];
        if (TAIL) voff = is_last ? x_voff_tail[i] : voff;
        load_to_lds_16(buf * kStageBytes + (4 * i + wave) * 1024, voff, sbase);
    };
    // The code tile has 128 rows, two waves' worth: the waves of the lower half of the tile load
    // the same chunks to the same place again, which keeps every wave's load count the same.
    const CodeT *code_tile = codes + (int64_t)n0 * J;
    const uint32_t code_voff = (uint32_t)(min(wn * 64 + lane, N - 1 - n0) * J * C::CSZ);
    auto issue_codes = [&](int c, int cbuf, int super) {
        const bool is_last = super >= n_super - 1;
        super = min(super, n_super - 1);
        const int chunk = (TAIL && is_last) ? 0 : c;
        const uint8_t *sbase = reinterpret_cast<const uint8_t *>(code_tile) + (int64_t)super * (C::K_SUPER / VEC * C::CSZ) + chunk * 16;
        load_to_lds_16(kCodeBase + cbuf * kTile + c * (BNN * 16) + wn * 1024, code_voff, sbase);
    };

    float4_t acc[NPN][MP];
#pragma unroll
    for (int j = 0; j < NPN; j++)
#pragma unroll
        for (int i = 0; i < MP; i++) acc[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};

    int x_rd[2][2];
#pragma unroll
    for (int par = 0; par < 2; par++)
#pragma unroll
        for (int s = 0; s < 2; s++) x_rd[par][s] = x_offset(wm * WM + par * 16 + r16, s * 4 + kg);
    const uint32_t code_rd = kCodeBase + (wn * WNN + r16) * 16 + kg * C::RB;

    // operand set 0 serves MFMA step 0 of a stage, set 1 step 1
    half4_t wlo[2][NPN], whi[2][NPN];
    half8_t xp[2][MP];
    uint32_t cr[2][2];  // codes behind the two W pairs whose gathers come next
    auto load_x1 = [&](int set, int i, int buf, int s) {
        xp[set][i] = *reinterpret_cast<const half8_t *>(smem + buf * kStageBytes + x_rd[i & 1][s] + (i >> 1) * 4096);
    };
    auto load_c1 = [&](int cset, int j, int cbuf, int t, int s) {
        const int pos = (t % C::STAGES) * 2 * C::HALF + s * C::HALF;
        cr[cset][j & 1] = read_codes<C::RB>(smem + code_rd + cbuf * kTile + (pos / 16) * (BNN * 16) + j * 256 + pos % 16);
    };
    auto load_w_half = [&](int set, int cset, int j, int h, bool zero) {
        const half4_t v = gather4<VEC, CodeT, TAIL, SPLIT>(smem, book[j], cr[cset][j & 1], h, zero, zero_off);
        if (h == 0) wlo[set][j] = v;
        else whi[set][j] = v;
    };
    auto mfma_one = [&](int set, int j, int i) {
        mfma_in_place(acc[j][i], __builtin_shufflevector(wlo[set][j], whi[set][j], 0, 1, 2, 3, 4, 5, 6, 7), xp[set][i]);
    };

    // ---- prologue: codebooks, stages 0 and 1, the first six X loads of stage 2 ------------------
    auto loads_of = [](int stage_mod) constexpr { return kChunksPerThread + (stage_mod % C::STAGES == 0 ? C::CH : 0); };
    {
        const uint8_t *src = reinterpret_cast<const uint8_t *>(cb + (int64_t)g_first * entries * VEC);
        const int n16 = cb_lds_count * cb_bytes / 16;
        const int g_total_16 = (int)(((int64_t)((ldn + rows_per_cb - 1) / rows_per_cb - g_first) * cb_bytes) / 16);
        // SPLIT: a plain copy first, into X buffer D (nothing is loaded into it before the main loop), re-laid below
        const int dst = SPLIT ? D * kStageBytes : kCbBase;
        for (int i0 = wave * 64; i0 < n16; i0 += kThreads)
            load_to_lds_16(dst + i0 * 16, (uint32_t)min(i0 + lane, g_total_16 - 1) * 16u, src);
    }
#pragma unroll
    for (int d = 0; d < D; d++) {
        if (d % C::STAGES == 0) {
#pragma unroll
            for (int c = 0; c < C::CH; c++) issue_codes(c, (d / C::STAGES) % NC, d / C::STAGES);
        }
#pragma unroll
        for (int i = 0; i < (d == D - 1 ? 6 : kChunksPerThread); i++) issue_x(i, d, d);
    }
    if (tid < 4) reinterpret_cast<uint32_t *>(smem + zero_off)[tid] = 0u;
    {
        // stage 0 (and everything older) must have landed
        constexpr int in_flight = loads_of(1) + loads_of(2) - 2;
        wait_vmcnt<in_flight>();
    }
    __syncthreads();
    if constexpr (SPLIT) {
        split_codebooks(smem, D * kStageBytes, kCbBase, cb_lds_count, tid, kThreads);
        __syncthreads();
    }

    int buf = 0, cbuf = 0;
    // step 0 of stage 0: all of its operands; and the codes of the first W pair of step 1
#pragma unroll
    for (int j = 0; j < NPN; j += 2) {
        load_c1(0, j, cbuf, 0, 0);
        load_c1(0, j + 1, cbuf, 0, 0);
        load_w_half(0, 0, j, 0, false);
        load_w_half(0, 0, j, 1, false);
        load_w_half(0, 0, j + 1, 0, false);
        load_w_half(0, 0, j + 1, 1, false);
    }
#pragma unroll
    for (int i = 0; i < MP; i++) load_x1(0, i, buf, 0);
    load_c1(0, 0, cbuf, 0, 1);
    load_c1(0, 1, cbuf, 0, 1);

#define VQ_FENCE __builtin_amdgcn_sched_barrier(0)
    // One quadrant: W pieces 0..3 of operand set `set` against X pieces ih*4.. of the same set.
    // Between the MFMAs: LX(p) one X read, LW(p) one half of a gather, LC(p) one code read
    // (p = 0, 2), one X load global->LDS (p = 1, 3), the code tile chunks (p = 0, 2).
#define VQ_NQUADRANT(set, ih, LX, LW, LC, xi, TGT)                                  \
    _Pragma("unroll") for (int p_ = 0; p_ < 4; p_++) {                              \
        mfma_one(set, p_, (ih) * 4 + 0); VQ_FENCE;                                  \
        LX(p_); VQ_FENCE;                                                           \
        mfma_one(set, p_, (ih) * 4 + 1); VQ_FENCE;                                  \
        LW(p_); VQ_FENCE;                                                           \
        mfma_one(set, p_, (ih) * 4 + 2); VQ_FENCE;                                  \
        if ((p_ & 1) == 0) { LC(p_ >> 1); VQ_FENCE; }                               \
        else { issue_x((xi) + (p_ >> 1), TGT##_buf, TGT##_stage); VQ_FENCE; }       \
        mfma_one(set, p_, (ih) * 4 + 3); VQ_FENCE;                                  \
        if ((p_ & 1) == 0 && TGT##_codes && (xi) == 0 && (p_ >> 1) < C::CH) {       \
            issue_codes(p_ >> 1, TGT##_cbuf, TGT##_super); VQ_FENCE;                \
        }                                                                           \
    }

    for (int super = 0; super < n_super; super++) {
        auto stage_body = [&](auto t_const) {
            constexpr int t = decltype(t_const)::value;
            const int stage = super * C::STAGES + t;
            const int buf_next = buf + 1 == NS ? 0 : buf + 1;
            // first quadrant: X loads 6, 7 of stage+2; the others: X loads 0..5 of stage+3 and its code tile
            const int tgt_a_buf = (buf + 2) % NS, tgt_a_stage = stage + 2;
            constexpr bool tgt_a_codes = false;
            const int tgt_a_cbuf = 0, tgt_a_super = 0;
            const int tgt_b_buf = buf == 0 ? NS - 1 : buf - 1, tgt_b_stage = stage + D;
            constexpr bool tgt_b_codes = (t + D) % C::STAGES == 0;
            constexpr int d_super = (t + D) / C::STAGES;
            const int tgt_b_super = super + d_super;
            const int tgt_b_cbuf = (cbuf + d_super) % NC;
            constexpr bool same_super = t + 1 < C::STAGES;
            const int cbuf_n = same_super ? cbuf : (cbuf + 1 == NC ? 0 : cbuf + 1);
            constexpr int t_n = same_super ? t + 1 : 0;
            const bool no_b = TAIL && stage == n_stage - 1;
            VQ_FENCE;
            // step 0 multiplies (set 0); step 1's operands are loaded into set 1
#define LX_B_LO(p) load_x1(1, (p), buf, 1)
#define LX_B_HI(p) load_x1(1, 4 + (p), buf, 1)
#define LW_B_01(p) load_w_half(1, 0, (p) >> 1, (p) & 1, no_b)
#define LW_B_23(p) load_w_half(1, 1, 2 + ((p) >> 1), (p) & 1, no_b)
#define LC_B_23(q) load_c1(1, 2 + (q), cbuf, t, 1)
#define LC_N_01(q) load_c1(0, (q), cbuf_n, t_n, 0)
            VQ_NQUADRANT(0, 0, LX_B_LO, LW_B_01, LC_B_23, 6, tgt_a);
            // Publish stage+1: only what stage+2 brings along may still be in flight.
            wait_vmcnt<loads_of(t + 2)>();
            __syncthreads();
            VQ_NQUADRANT(0, 1, LX_B_HI, LW_B_23, LC_N_01, 0, tgt_b);
            // step 1 multiplies (set 1); the next stage's step 0 operands are loaded into set 0
#define LX_N_LO(p) load_x1(0, (p), buf_next, 0)
#define LX_N_HI(p) load_x1(0, 4 + (p), buf_next, 0)
#define LW_N_01(p) load_w_half(0, 0, (p) >> 1, (p) & 1, false)
#define LW_N_23(p) load_w_half(0, 1, 2 + ((p) >> 1), (p) & 1, false)
#define LC_N_23(q) load_c1(1, 2 + (q), cbuf_n, t_n, 0)
#define LC_NB_01(q) load_c1(0, (q), cbuf_n, t_n, 1)
            VQ_NQUADRANT(1, 0, LX_N_LO, LW_N_01, LC_N_23, 2, tgt_b);
            VQ_NQUADRANT(1, 1, LX_N_HI, LW_N_23, LC_NB_01, 4, tgt_b);
#undef LX_B_LO
#undef LX_B_HI
#undef LW_B_01
#undef LW_B_23
#undef LC_B_23
#undef LC_N_01
#undef LX_N_LO
#undef LX_N_HI
#undef LW_N_01
#undef LW_N_23
#undef LC_N_23
#undef LC_NB_01
            buf = buf_next;
        };
        stage_body(std::integral_constant<int, 0>{});
        if constexpr (C::STAGES == 2) stage_body(std::integral_constant<int, 1>{});
        cbuf = cbuf + 1 == NC ? 0 : cbuf + 1;
    }
#undef VQ_NQUADRANT
#undef VQ_FENCE
    wait_vmcnt<0>();
    __syncthreads();
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: lane holds Y[m = i*16 + r16][n = j*16 + 4*kg + 0..3] of its 128x64 wave tile --
    auto epilogue = [&](auto has_bias_const) {
        constexpr bool HB = decltype(has_bias_const)::value;
        float bj[NPN][4];
#pragma unroll
        for (int j = 0; j < NPN; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int n = n0 + wn * WNN + j * 16 + 4 * kg + e;
                bj[j][e] = HB && n < N ? (float)bias[n] : 0.f;
            }
        if ((ldn & 7) == 0) {
            constexpr int kPitch = 144;  // 64 fp16 + 16 bytes: rows land in different banks
            uint8_t *stage_out = smem + wave * (128 * kPitch);
#pragma unroll
            for (int i = 0; i < MP; i++)
#pragma unroll
                for (int j = 0; j < NPN; j++)
                    *reinterpret_cast<half4_t *>(stage_out + (i * 16 + r16) * kPitch + (j * 16 + 4 * kg) * 2) =
                        round4<HB>(acc[j][i], bj[j]);
#pragma unroll
            for (int it = 0; it < 16; it++) {
                const int row = it * 8 + (lane >> 3), c = lane & 7;
                const uint4_t v = *reinterpret_cast<const uint4_t *>(stage_out + row * kPitch + c * 16);
                const int m = m0 + wm * WM + row;
                const int n = n0 + wn * WNN + c * 8;
                if (m < M && n < N) st_global_16_streaming(y + (int64_t)m * ldn + n, v);
            }
        } else {
#pragma unroll
            for (int i = 0; i < MP; i++) {
                const int m = m0 + wm * WM + i * 16 + r16;
                if (m >= M) continue;
#pragma unroll
                for (int j = 0; j < NPN; j++) {
                    const int n = n0 + wn * WNN + j * 16 + 4 * kg;
                    half_t *dst = y + (int64_t)m * ldn + n;
                    const half4_t hv = round4<HB>(acc[j][i], bj[j]);
                    if ((ldn & 3) == 0 && n + 3 < N) {
                        *reinterpret_cast<half4_t *>(dst) = hv;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (n + e < N) dst[e] = hv[e];
                    }
                }
            }
        }
    };
    if (gated) {
        if (bias) store_gated<NPN, MP, true>(acc, y, bias, M, N, ldn, m0 + wm * WM, n0 + wn * WNN, r16, kg);
        else store_gated<NPN, MP, false>(acc, y, bias, M, N, ldn, m0 + wm * WM, n0 + wn * WNN, r16, kg);
        return;
    }
    if (bias) epilogue(std::true_type{});
    else epilogue(std::false_type{});
}

template <int VEC, typename CodeT>
size_t lds_bytes(const ProblemB &p, int n_stages)
{
    typedef PrefillCfg<VEC, CodeT> C;
    return (size_t)n_stages * kStageBytes + (size_t)C::code_bufs(n_stages) * C::kTileBytes + books_bytes(p, BN);
}

template <int VEC, typename CodeT>
size_t lds_bytes_narrow(const ProblemB &p)
{
    typedef PrefillCfg<VEC, CodeT> C;
    return (size_t)4 * kStageBytes + (size_t)C::code_bufs(4) * C::CH * BNN * 16 + books_bytes(p, BNN);
}

// Microseconds a launch over `cols` tile columns of `bn` W rows is expected to take, fitted to
// measurements: a tile costs 5 us of prologue and epilogue plus K/64 stages of 1.0 us (256x256) or
// 0.56 us (256x128) when the device is mostly idle, up to 1.6 times that when every compute unit
// works (the clock the device holds under load); the tiles go over the compute units in rounds.
double tile_cost_us(const ProblemB &p, int bn, int cols)
{
    const int64_t tiles = (int64_t)((p.M + BM - 1) / BM) * cols;
    const int cus = device_cu_count();
    const Tuning &tn = tuning();
    const double stages = p.K / 64.0 * (bn == BN ? tn.prefill_stage_us_256x256 : tn.prefill_stage_us_256x128);
    const int64_t full = tiles / cus, rem = tiles % cus;
    double t = (double)full * (tn.prefill_tile_fixed_us + stages * tn.prefill_full_device_factor);
    if (rem) t += tn.prefill_tile_fixed_us + stages * (1.0 + (tn.prefill_full_device_factor - 1.0) * (double)rem / cus);
    return t;
}

// How a launch is cut into tiles: W rows [0, n_split) in 256x256 tiles, [n_split, N) in 256x128
// tiles (either part may be empty).  The narrow tile pays when it brings more compute units to
// work: for the whole problem when its 256x256 tiles are fewer than the units, or for the columns
// left over after whole rounds of 256x256 tiles (two launches then).
struct TilePlan {
    int n_split;
    double cost_us;
};

template <int VEC, typename CodeT>
TilePlan plan_tiles(const ProblemB &p)
{
    const int cols_wide = (p.N + BN - 1) / BN, cols_narrow = (p.N + BNN - 1) / BNN;
    TilePlan best = {p.N, tile_cost_us(p, BN, cols_wide)};
    if (lds_bytes_narrow<VEC, CodeT>(p) > kLdsLimit) return best;
    const double all_narrow = tile_cost_us(p, BNN, cols_narrow);
    if (all_narrow < 0.97 * best.cost_us) best = {0, all_narrow};
    // whole rounds of wide tiles, the rest narrow
    const int tiles_m = (p.M + BM - 1) / BM, cus = device_cu_count();
    const int64_t rounds = (int64_t)tiles_m * cols_wide / cus;
    const int cols_head = (int)(rounds * cus / tiles_m);
    if (rounds >= 1 && cols_head >= 1 && cols_head < cols_wide) {
        const int n_split = cols_head * BN;
        const double t = tile_cost_us(p, BN, cols_head) + tile_cost_us(p, BNN, (p.N - n_split + BNN - 1) / BNN) + 3.0;
        if (t < 0.97 * best.cost_us) best = {n_split, t};
    }
    return best;
}

// tile: 0 = as planned, 1 = 256x256 only, 2 = 256x128 only.  n_end > 0: only the W rows [0, n_end) (a multiple of 256;
// the rest of the columns is another launch's)
template <int VEC, typename CodeT>
hipError_t launch_prefill_typed(const ProblemB &p, hipStream_t s, int tile, int n_end = 0)
{
    const bool tail = (p.K % kStageK) != 0;
    const int tiles_m = (p.M + BM - 1) / BM;
    if (n_end <= 0 || n_end > p.N) n_end = p.N;
    int n_split = n_end;
    if (tile == 2) n_split = 0;
    else if (tile == 0) n_split = min(plan_tiles<VEC, CodeT>(p).n_split, n_end);
    if (n_split > 0) {
        const int tiles_n = (n_split + BN - 1) / BN;
        const int n_cb = codebooks_per_tile(p, BN);
        // Four X stages when the codebooks leave room for them, else three; two (every stage then
        // waits for its own loads) only so that very large codebooks still run.
        const int ns = lds_bytes<VEC, CodeT>(p, 4) <= kLdsLimit ? 4 : lds_bytes<VEC, CodeT>(p, 3) <= kLdsLimit ? 3 : 2;
        const size_t smem = lds_bytes<VEC, CodeT>(p, ns);
        // (the 256x256 tile takes its codebooks plain and gathers whole entries; the split layout is the narrow tile's)
        auto pick = [&](auto tail_c, auto ns_c) {
            constexpr bool T = decltype(tail_c)::value;
            constexpr int S = decltype(ns_c)::value;
            return prefill_kernel<VEC, CodeT, T, S, false>;
        };
        using std::integral_constant;
        auto kern = ns == 4   ? (tail ? pick(std::true_type{}, integral_constant<int, 4>{}) : pick(std::false_type{}, integral_constant<int, 4>{}))
                    : ns == 3 ? (tail ? pick(std::true_type{}, integral_constant<int, 3>{}) : pick(std::false_type{}, integral_constant<int, 3>{}))
                              : (tail ? pick(std::true_type{}, integral_constant<int, 2>{}) : pick(std::false_type{}, integral_constant<int, 2>{}));
        hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(kThreads), smem, s, p.x,
                           static_cast<const CodeT *>(p.codes), p.cb, p.y, p.bias, p.M, p.K, n_split, 0, p.N, p.entries,
                           p.rows_per_cb, tiles_m, tiles_n, n_cb, p.gated ? 1 : 0);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (n_split < n_end) {
        if (lds_bytes_narrow<VEC, CodeT>(p) > kLdsLimit) return hipErrorInvalidValue;
        const int tiles_n = (n_end - n_split + BNN - 1) / BNN;
        const size_t smem = lds_bytes_narrow<VEC, CodeT>(p);
        constexpr bool can_split = VEC == 8 && sizeof(CodeT) == 1;
        const bool split = can_split && split_layout_applies(p, codebooks_per_tile(p, BNN), kStageBytes);
        auto kern = split ? (tail ? prefill_narrow_kernel<VEC, CodeT, true, can_split> : prefill_narrow_kernel<VEC, CodeT, false, can_split>)
                          : (tail ? prefill_narrow_kernel<VEC, CodeT, true, false> : prefill_narrow_kernel<VEC, CodeT, false, false>);
        hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(kThreads), smem, s, p.x,
                           static_cast<const CodeT *>(p.codes), p.cb, p.y, p.bias, p.M, p.K, n_end, n_split, p.N, p.entries,
                           p.rows_per_cb, tiles_m, tiles_n, codebooks_per_tile(p, BNN), p.gated ? 1 : 0);
        return hipGetLastError();
    }
    return hipSuccess;
}

template <int VEC, typename CodeT>
bool prefill_cfg_supports(const ProblemB &p)
{
    // whole 16-byte code chunks per row, a tile's code offsets within 32 bits
    return p.K % PrefillCfg<VEC, CodeT>::KC == 0 && lds_bytes<VEC, CodeT>(p, 2) <= kLdsLimit &&
           (int64_t)BN * (p.K / VEC) * (int64_t)sizeof(CodeT) < ((int64_t)1 << 31) &&
           (int64_t)BM * p.K * 2 < ((int64_t)1 << 32);
}

// wide: the kernel serves the shape; narrow: so does its narrow tile; cost_us: expected time of
// the launch as it would be cut into tiles
struct PrefillQuery {
    bool wide, narrow;
    double cost_us;
};

template <int VEC, typename CodeT>
void prefill_cfg_query(const ProblemB &p, PrefillQuery &what)
{
    what.wide = prefill_cfg_supports<VEC, CodeT>(p);
    what.narrow = what.wide && lds_bytes_narrow<VEC, CodeT>(p) <= kLdsLimit;
    what.cost_us = what.wide ? plan_tiles<VEC, CodeT>(p).cost_us : 1e30;
}

void prefill_query(const ProblemB &p, PrefillQuery &what)
{
    what = {false, false, 1e30};
    if (p.M < 1 || p.N < 1 || p.K < 1) return;
    if (p.vec != 2 && p.vec != 4 && p.vec != 8) return;
    if (((size_t)p.entries * p.vec * 2) % 16 != 0) return;
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? prefill_cfg_query<8, uint8_t>(p, what) : prefill_cfg_query<8, uint16_t>(p, what);
    case 4: return u8 ? prefill_cfg_query<4, uint8_t>(p, what) : prefill_cfg_query<4, uint16_t>(p, what);
    default:
        if (u8) prefill_cfg_query<2, uint8_t>(p, what);  // 16-bit codes of 2-vectors: generic kernel
    }
}

}  // namespace

bool prefill_supports(const ProblemB &p)
{
    PrefillQuery what;
    prefill_query(p, what);
    return what.wide;
}

bool prefill_narrow_supports(const ProblemB &p)
{
    PrefillQuery what;
    prefill_query(p, what);
    return what.narrow;
}

// 128x128 tiles are taken when they are expected to be clearly faster than the best cut into large tiles
constexpr double kSmallTileMargin = 0.95;

double prefill_cost_us(const ProblemB &p)
{
    PrefillQuery what;
    prefill_query(p, what);
    if (!what.wide) return what.cost_us;
    const double small = prefill_small_cost_us(p);
    return small < kSmallTileMargin * what.cost_us ? small : what.cost_us;
}

// ---- whole rounds of large tiles, then the columns that are left in 128x128 tiles with K split ------------------
// A launch whose large tiles are a few more than a multiple of the compute units pays a whole further round for them.
// With a workspace the left-over columns go to the 128x128 kernel instead, K split over as many workgroups as fill
// the device: the second launch then takes a fraction of a round (M = 1536, K = 4096, N = 11008: 6 x 43 = 258 tiles of
// 256x256 on 256 units; 42 columns make one round, the 43rd is 48 small tiles with K in 8 slices).
TailSplitPlan prefill_tail_split_plan(const ProblemB &p)
{
    TailSplitPlan best = {false, 0, 0, 0, 1e30, 0};
    if (p.gated || !prefill_supports(p) || !prefill_small_supports(p)) return best;
    const int cus = device_cu_count(), tiles_m = (p.M + BM - 1) / BM;
    const bool narrow_ok = prefill_narrow_supports(p);
    for (int head_tile = 1; head_tile <= 2; head_tile++) {
        if (head_tile == 2 && !narrow_ok) break;
        const int bn = head_tile == 1 ? BN : BNN;
        const int cols = (p.N + bn - 1) / bn;
        const int64_t rounds = (int64_t)tiles_m * cols / cus;
        // as many columns as whole rounds hold (in whole 256-row steps, so that either tile can serve them)
        int cols_head = (int)(rounds * cus / tiles_m);
        if (head_tile == 2) cols_head &= ~1;
        if (rounds < 1 || cols_head < 1 || cols_head >= cols) continue;
        const int n_split = cols_head * bn;
        ProblemB tail = p;  // the left-over columns as the 128x128 kernel's cost model sees them
        tail.N = p.N - n_split;
        double t_tail = 1e30;
        int sp = prefill_splitk_choice(tail, &t_tail, 1);
        if (sp < 1 || t_tail >= 1e29) continue;
        // (Tuning::splitk_force_splits, for measurements and tests: that many slices where the shape allows)
        const int forced = (int)tuning().splitk_force_splits;
        if (forced >= 2 && prefill_splitk_supports(tail, forced)) sp = forced;
        const double t = tile_cost_us(p, bn, cols_head) + t_tail + 3.0;
        if (t < best.cost_us) best = {true, head_tile, n_split, sp, t, sp > 1 ? prefill_splitk_workspace_bytes(tail, sp) : 0};
    }
    return best;
}

hipError_t launch_prefill_tail_split(const ProblemB &p, const TailSplitPlan &plan, hipStream_t s, void *workspace)
{
    if (!plan.ok || plan.n_split <= 0 || plan.n_split >= p.N || plan.n_split % BN != 0) return hipErrorInvalidValue;
    const bool u8 = p.code_bits == 8;
    hipError_t e;
    switch (p.vec) {
    case 8: e = u8 ? launch_prefill_typed<8, uint8_t>(p, s, plan.head_tile, plan.n_split) : launch_prefill_typed<8, uint16_t>(p, s, plan.head_tile, plan.n_split); break;
    case 4: e = u8 ? launch_prefill_typed<4, uint8_t>(p, s, plan.head_tile, plan.n_split) : launch_prefill_typed<4, uint16_t>(p, s, plan.head_tile, plan.n_split); break;
    default: e = u8 ? launch_prefill_typed<2, uint8_t>(p, s, plan.head_tile, plan.n_split) : hipErrorInvalidValue;
    }
    if (e != hipSuccess) return e;
    return launch_prefill_small_b(p, s, plan.splits, workspace, plan.n_split);
}

hipError_t launch_prefill_b(const ProblemB &p, hipStream_t s, int tile)
{
    if (!prefill_supports(p)) return hipErrorInvalidValue;
    if (tile == 0) {
        PrefillQuery what;
        prefill_query(p, what);
        if (prefill_small_cost_us(p) < kSmallTileMargin * what.cost_us) return launch_prefill_small_b(p, s);
    }
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? launch_prefill_typed<8, uint8_t>(p, s, tile) : launch_prefill_typed<8, uint16_t>(p, s, tile);
    case 4: return u8 ? launch_prefill_typed<4, uint8_t>(p, s, tile) : launch_prefill_typed<4, uint16_t>(p, s, tile);
    default: return u8 ? launch_prefill_typed<2, uint8_t>(p, s, tile) : hipErrorInvalidValue;
    }
}

}  // namespace vq
