// Prefill kernel with 128x128 tiles, for medium M: Y[M,N] = X[M,K] . W^T with W given as codes +
// codebook, where the 256-row tiles of vq_prefill.hip are fewer than the compute units and a
// 16-row slab kernel re-reads the codes too often.
//
// The same means as the large tiles - codebooks in the LDS, codewords gathered straight into the
// operands of v_mfma_f32_16x16x32_f16 in two 8-byte halves, X (whole 128-byte lines) and code
// tiles global -> LDS directly, accumulators pinned in the AGPRs, every MFMA fenced - at a quarter
// of the size: 256 threads (2x2 waves), 64x64 per wave as 4x4 pieces.  64 accumulator registers
// and 76 KB of LDS leave room for two workgroups per compute unit.  A 64x64 wave tile reads one
// operand per two MFMAs, twice the rate of the 128x128 wave tile, and the LDS is what bounds it:
// per tile and k it is slower than the large tiles, and pays where those leave most units idle.
//
// A stage is 64 k = two MFMA steps of 16 MFMAs.  Every operand is double buffered in registers
// (set 0 serves step 0 of a stage, set 1 step 1): while a step multiplies, the eight gather halves
// and four X reads of the next step are issued, and the codes of the step after that are read.
// One barrier per stage publishes stage+1 (X and, when it opens a code tile, the tile) and frees
// the buffer of stage-1, into which the loads of stage+3 go.
//
// K must be a multiple of the k one code tile covers (64, or 128 for 8-vectors with 8-bit codes).
//
// Split K.  Where even these tiles are fewer than the compute units, `splits` workgroups share a tile, each
// multiplying k_len = K / splits of K.  Nothing waits for anything: a workgroup writes its fp32 sums to a partial
// buffer with device-scope stores, waits for them, and counts itself in on the tile's counter; the one that
// finds itself last adds the partial sums up in the order of the slices and runs the epilogue.  The sum is the same whoever comes last, so
// results do not depend on the order in which the workgroups finish.
#include "vq_prefill_common.h"

#include <type_traits>

namespace vq {

namespace {

constexpr int SBM = 128, SBN = 128;        // workgroup tile
constexpr int SWM = 64, SWN = 64;          // wave tile
constexpr int SMP = SWM / 16, SNP = SWN / 16;
constexpr int kSmallStage = SBM * kStageK * 2;               // 16 KB
constexpr int kSmallXLoads = kSmallStage / (kThreads * 16);  // 16-byte chunks of an X stage per thread: 4

// code tiles in the LDS for NS X stages: the one being read plus those loaded ahead
template <int VEC, typename CodeT>
constexpr int small_code_bufs(int ns)
{
    return PrefillCfg<VEC, CodeT>::STAGES == 1 ? ns : (ns - 1) / 2 + 2;
}

// SPLIT: the codebooks lie in the LDS in the split layout (vq_prefill_common.h).
template <int VEC, typename CodeT, int NS, bool SPLIT>
__global__ __launch_bounds__(kThreads, 2) void prefill_small_kernel(const half_t *__restrict__ x,
                                                                    const CodeT *__restrict__ codes,
                                                                    const half_t *__restrict__ cb,
                                                                    half_t *__restrict__ y,
                                                                    const half_t *__restrict__ bias, int M, int K,
                                                                    int N, int n_begin, int ldn, int entries,
                                                                    int rows_per_cb, int tiles_m,
                                                                    int tiles_n, int cb_lds_count, int gated, int k_len,
                                                                    int splits, float4_t *__restrict__ partials,
                                                                    unsigned int *__restrict__ counters, int fenced)
{
    typedef PrefillCfg<VEC, CodeT> C;
    constexpr int D = NS - 1;                 // loads run D stages ahead
    constexpr int NC = small_code_bufs<VEC, CodeT>(NS);
    constexpr int kTile = C::CH * SBN * 16;   // code tile: [chunk][128 rows][16 bytes]
    static_assert(C::CH <= 4, "at most four code chunks per tile row");
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int kCodeBase = NS * kSmallStage;
    constexpr int kCbBase = kCodeBase + NC * kTile;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int r16 = lane & 15, kg = lane >> 4;
    const int J = K / VEC;
    const int cb_bytes = entries * VEC * 2;

    // Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2: re-number them so
    // that an XCD works on consecutive tiles of the row-band-major order.
    // (with split K the slices of a tile lie n_wg workgroup ids apart: a multiple of 8 whenever the re-numbering applies)
    const int n_wg = tiles_m * tiles_n;
    const int split = (int)blockIdx.x / n_wg;
    int wg = (int)blockIdx.x - split * n_wg;
    if ((n_wg & 7) == 0) wg = (wg & 7) * (n_wg >> 3) + (wg >> 3);
    const int tm = wg / tiles_n, tn = wg % tiles_n;
    // The launch covers the W rows (columns of Y) [n_begin, N) of a problem with ldn rows in all.
    const int m0 = tm * SBM, n0 = n_begin + tn * SBN;
    const int n_stage = k_len / kStageK;
    const int n_super = n_stage / C::STAGES;

    // ---- per-lane codebook bases ------------------------------------------------------------
    const int g_first = n0 / rows_per_cb;
    uint32_t book[SNP];  // byte offset inside smem of the codebook of W row j*16 + r16 of the wave tile
    {
        const int n_base = min(n0 + wn * SWN, N - 1);
        const int g_base = n_base / rows_per_cb, rem_base = n_base - g_base * rows_per_cb;
        const float rcp = 1.0f / (float)rows_per_cb;
#pragma unroll
        for (int j = 0; j < SNP; j++) {
            const int n = min(n0 + wn * SWN + j * 16 + r16, N - 1);
            const int g = g_base + small_div(n - n_base + rem_base, rows_per_cb, rcp);
            book[j] = kCbBase + (g - g_first) * cb_bytes;
        }
    }

    // ---- staging: global -> LDS directly ----------------------------------------------------
    uint32_t x_voff[kSmallXLoads];
#pragma unroll
    for (int i = 0; i < kSmallXLoads; i++) {
        const int slot = (4 * i + wave) * 64 + lane;
        const int bank_row = slot >> 4;
        const int v = (slot & 15) ^ (bank_row & 15);
        const int row = 2 * bank_row + (v >> 3), cc = v & 7;
        x_voff[i] = (uint32_t)(((int64_t)(min(m0 + row, M - 1) - m0) * K + cc * 8) * 2);
    }
    const half_t *x_tile = x + (int64_t)m0 * K + (int64_t)split * k_len;
    // X load i (0..3) of a stage that starts at `xb` into buffer `buf`.
    auto issue_x = [&](int i, int buf, const half_t *xb) {
        load_to_lds_16(buf * kSmallStage + (4 * i + wave) * 1024, x_voff[i], xb);
    };
    // The code tile has 128 rows, two waves' worth: the waves of the lower half of the tile load
    // the same chunks to the same place again, which keeps every wave's load count the same.
    const uint8_t *code_tile = reinterpret_cast<const uint8_t *>(codes + (int64_t)n0 * J + (int64_t)split * (k_len / VEC));
    uint32_t code_voff[C::CH];
#pragma unroll
    for (int c = 0; c < C::CH; c++) code_voff[c] = (uint32_t)(min(wn * 64 + lane, N - 1 - n0) * J * C::CSZ) + c * 16;
    constexpr int kSuperBytes = C::K_SUPER / VEC * C::CSZ;  // bytes of one row's codes per code tile
    auto issue_codes = [&](int c, int cbuf, const uint8_t *cbase) {
        load_to_lds_16(kCodeBase + cbuf * kTile + c * (SBN * 16) + wn * 1024, code_voff[c], cbase);
    };
    // Where the loads issued during the current stage read: stage + D and the code tile it may open.
    // Past the end the last stage (tile) is read again (harmless) instead of branching, so that
    // every stage brings the same number of loads; the pointers move on once per stage.
    const half_t *x_ahead = x_tile + min(D, n_stage - 1) * kStageK;
    const uint8_t *c_ahead = code_tile + (int64_t)min(D / C::STAGES, n_super - 1) * kSuperBytes;

    float4_t acc[SNP][SMP];
#pragma unroll
    for (int j = 0; j < SNP; j++)
#pragma unroll
        for (int i = 0; i < SMP; i++) acc[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};

    // ---- operand reads ------------------------------------------------------------------------
    int x_rd[2][2];
#pragma unroll
    for (int par = 0; par < 2; par++)
#pragma unroll
        for (int s = 0; s < 2; s++) x_rd[par][s] = x_offset(wm * SWM + par * 16 + r16, s * 4 + kg);
    const uint32_t code_rd = kCodeBase + (wn * SWN + r16) * 16 + kg * C::RB;

    half4_t wlo[2][SNP], whi[2][SNP];
    half8_t xp[2][SMP];
    uint32_t cr[SNP];  // the codes behind the W pieces of the step whose gathers come next
    auto load_x1 = [&](int set, int i, int buf, int s) {
        xp[set][i] = *reinterpret_cast<const half8_t *>(smem + buf * kSmallStage + x_rd[i & 1][s] + (i >> 1) * 4096);
    };
    // the codes of W piece j for MFMA step s of stage t (of its code tile) out of code buffer `cbuf`
    auto load_c1 = [&](int j, int cbuf, int t, int s) {
        const int pos = (t % C::STAGES) * 2 * C::HALF + s * C::HALF;
        cr[j] = read_codes<C::RB>(smem + code_rd + cbuf * kTile + (pos / 16) * (SBN * 16) + j * 256 + pos % 16);
    };
    auto load_w_half = [&](int set, int j, int h) {
        const half4_t v = gather4<VEC, CodeT, false, SPLIT>(smem, book[j], cr[j], h, false, 0);
        if (h == 0) wlo[set][j] = v;
        else whi[set][j] = v;
    };
    auto mfma_one = [&](int set, int j, int i) {
        mfma_in_place(acc[j][i], __builtin_shufflevector(wlo[set][j], whi[set][j], 0, 1, 2, 3, 4, 5, 6, 7), xp[set][i]);
    };

    // ---- prologue: codebooks, stages 0..2 ---------------------------------------------------------
    // Loads complete in the order they were issued, so one count serves all of them.
    auto loads_of = [](int stage_mod) constexpr { return kSmallXLoads + (stage_mod % C::STAGES == 0 ? C::CH : 0); };
    {
        const uint8_t *src = reinterpret_cast<const uint8_t *>(cb + (int64_t)g_first * entries * VEC);
        const int n16 = cb_lds_count * cb_bytes / 16;
        const int g_total_16 = (int)(((int64_t)((N + rows_per_cb - 1) / rows_per_cb - g_first) * cb_bytes) / 16);
        // past the last codebook: read its last 16 bytes again
        // SPLIT: into the last X buffer first (free until stage 0 issues the loads of stage D), re-laid below
        const int dst = SPLIT ? D * kSmallStage : kCbBase;
        for (int i0 = wave * 64; i0 < n16; i0 += kThreads)
            load_to_lds_16(dst + i0 * 16, (uint32_t)min(i0 + lane, g_total_16 - 1) * 16u, src);
    }
#pragma unroll
    for (int d = 0; d < D; d++) {
        if (d % C::STAGES == 0) {
#pragma unroll
            for (int c = 0; c < C::CH; c++)
                issue_codes(c, (d / C::STAGES) % NC, code_tile + (int64_t)min(d / C::STAGES, n_super - 1) * kSuperBytes);
        }
#pragma unroll
        for (int i = 0; i < kSmallXLoads; i++) issue_x(i, d, x_tile + min(d, n_stage - 1) * kStageK);
    }
    {
        // the codebooks and stage 0 have landed when only the stages behind it are in flight
        constexpr int in_flight = [&]() constexpr {
            int n = 0;
            for (int d = 1; d < D; d++) n += loads_of(d);
            return n;
        }();
        wait_vmcnt<in_flight>();
    }
    __syncthreads();
    if constexpr (SPLIT) {
        split_codebooks(smem, D * kSmallStage, kCbBase, cb_lds_count, tid, kThreads);
        __syncthreads();
    }

    int buf = 0, cbuf = 0;
    // step 0 of stage 0: all of its operands; then the codes of step 1
#pragma unroll
    for (int j = 0; j < SNP; j++) load_c1(j, cbuf, 0, 0);
#pragma unroll
    for (int j = 0; j < SNP; j++) {
        load_w_half(0, j, 0);
        load_w_half(0, j, 1);
    }
#pragma unroll
    for (int i = 0; i < SMP; i++) load_x1(0, i, buf, 0);
#pragma unroll
    for (int j = 0; j < SNP; j++) load_c1(j, cbuf, 0, 1);

#define VQ_FENCE __builtin_amdgcn_sched_barrier(0)
    for (int super = 0; super < n_super; super++) {
        auto stage_body = [&](auto t_const) {
            constexpr int t = decltype(t_const)::value;
            const int stage = super * C::STAGES + t;
            const int buf_next = buf + 1 == NS ? 0 : buf + 1;
            // the loads of stage+D go into the buffer stage-1 was read from
            const int tgt_buf = buf == 0 ? NS - 1 : buf - 1;
            constexpr bool tgt_codes = (t + D) % C::STAGES == 0;
            constexpr int d_super = (t + D) / C::STAGES;
            const int tgt_cbuf = (cbuf + d_super) % NC;
            // the stage after this one: same code tile or the next
            constexpr bool same_super = t + 1 < C::STAGES;
            const int cbuf_n = same_super ? cbuf : (cbuf + 1 == NC ? 0 : cbuf + 1);
            constexpr int t_n = same_super ? t + 1 : 0;
            // Publish stage+1: only what the stages behind it bring along may still be in flight.
            constexpr int in_flight = [&]() constexpr {
                int n = 0;
                for (int d = 2; d < D; d++) n += loads_of(t + d);
                return n;
            }();
            wait_vmcnt<in_flight>();
            __syncthreads();
            VQ_FENCE;
            // A step: 16 MFMAs of set `set`; between them the gathers (in halves) and X reads of the
            // next step into the other set, the codes of the step after that, and this step's share
            // of the global loads.  A wave issues one instruction every four cycles and an MFMA holds
            // the pipe for sixteen: a few instructions fit between two MFMAs.
#pragma unroll
            for (int step = 0; step < 2; step++) {
#pragma unroll
                for (int m = 0; m < SNP * SMP; m++) {
                    mfma_one(step, m >> 2, m & 3);
                    VQ_FENCE;
                    if (m < 2 * SNP) {
                        load_w_half(step ^ 1, m >> 1, m & 1);
                        VQ_FENCE;
                        if (m & 1) {
                            if (step == 0) load_x1(1, m >> 1, buf, 1);
                            else load_x1(0, m >> 1, buf_next, 0);
                            VQ_FENCE;
                        }
                    } else if (m < 3 * SNP) {
                        // the gathers above have taken their addresses from cr[]: read the next codes
                        if (step == 0) load_c1(m - 2 * SNP, cbuf_n, t_n, 0);
                        else load_c1(m - 2 * SNP, cbuf_n, t_n, 1);
                        VQ_FENCE;
                    } else {
                        const int q = m - 3 * SNP;  // 0..3
                        if ((q & 1) == 0) {
                            issue_x(2 * step + (q >> 1), tgt_buf, x_ahead);
                            VQ_FENCE;
                        } else if (tgt_codes && 2 * step + (q >> 1) < C::CH) {
                            issue_codes(2 * step + (q >> 1), tgt_cbuf, c_ahead);
                            VQ_FENCE;
                        }
                    }
                }
            }
            // the next stage loads stage+D+1, and with it the code tile that stage may open
            x_ahead += stage + D + 1 < n_stage ? kStageK : 0;
            if ((t + D + 1) % C::STAGES == 0) c_ahead += (stage + D + 1) / C::STAGES < n_super ? kSuperBytes : 0;
            buf = buf_next;
        };
        stage_body(std::integral_constant<int, 0>{});
        if constexpr (C::STAGES == 2) stage_body(std::integral_constant<int, 1>{});
        cbuf = cbuf + 1 == NC ? 0 : cbuf + 1;
    }
#undef VQ_FENCE
    // Drain the clamped loads still in flight before the stage buffers are reused.
    wait_vmcnt<0>();
    __syncthreads();
    // the last MFMAs must have left the pipe before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- split K: partial sums out, and the workgroup that comes last adds them up -------------------
    // The partial sums are written and read with device-scope memory instructions (sc1: through the L2 of the
    // XCD, which is not coherent with the other seven), and the waits are written out: a release / acquire fence
    // of device scope would write back and invalidate the whole L2 under the workgroups that are still multiplying
    // (measured: 3 us per MB of partial sums).  A store is complete, and visible device-wide, when the counter
    // has counted it; the count itself is a relaxed device-scope atomic; the loads of the last workgroup are issued
    // behind the barrier that follows its count.
#if !defined(__HIP_DEVICE_COMPILE__) || defined(__gfx942__) || defined(__gfx950__)
    // (what "sc1" means for a store and a load, and that a counted store is visible device-wide, are properties of
    // these two targets; another target has to re-establish them or build with the fences below)
#else
#error "the split-K exchange relies on the gfx942/gfx950 behaviour of device-scope (sc1) loads and stores"
#endif
    if (splits > 1) {
        // partial sums of (tile, slice): half h (two floats) of accumulator (j, i) of thread tid at
        // [((j * SMP + i) * 2 + h) * 256 + tid], moved as 64-bit words (the widest scoped access there is)
        constexpr int kPartial = SNP * SMP * 2 * kThreads;  // 64-bit words per tile and slice
        typedef float float2_t __attribute__((ext_vector_type(2)));
        uint64_t *tile_partials = reinterpret_cast<uint64_t *>(partials) + (int64_t)wg * splits * kPartial;
        uint64_t *mine = tile_partials + (int64_t)split * kPartial + tid;
#pragma unroll
        for (int j = 0; j < SNP; j++)
#pragma unroll
            for (int i = 0; i < SMP; i++)
#pragma unroll
                for (int h = 0; h < 2; h++)
                    __hip_atomic_store(mine + ((j * SMP + i) * 2 + h) * kThreads,
                                       __builtin_bit_cast(uint64_t, float2_t{acc[j][i][2 * h], acc[j][i][2 * h + 1]}), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        // Every partial-sum store of this thread is complete (counted back) here, and the barrier extends that to the
        // workgroup: nothing may be moved across this wait - not the stores above it, not the count below it.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        // (validation path, Tuning::splitk_validate_fences: the textbook release / acquire pair of device scope around
        // the count, as the memory model asks for; same results bit for bit, at the cost of the L2 write-backs)
        if (fenced) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        __syncthreads();
        uint32_t *flag = reinterpret_cast<uint32_t *>(smem);
        if (tid == 0) *flag = __hip_atomic_fetch_add(counters + wg, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const bool last = *flag == (uint32_t)(splits - 1);
        __syncthreads();  // the flag's word belongs to the epilogue's staging area again
        if (!last) return;
        if (fenced) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        // The sum in the order of the slices, whoever is last - this workgroup's own sums are read back like the
        // others' (the same bits it wrote; its registers are free for the loads that way).
        for (int sl = 0; sl < splits; sl++) {
            const uint64_t *src = tile_partials + (int64_t)sl * kPartial + tid;
#pragma unroll
            for (int j = 0; j < SNP; j++)
#pragma unroll
                for (int i = 0; i < SMP; i++)
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const float2_t v = __builtin_bit_cast(
                            float2_t, __hip_atomic_load(src + ((j * SMP + i) * 2 + h) * kThreads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                        acc[j][i][2 * h] = sl == 0 ? v[0] : acc[j][i][2 * h] + v[0];
                        acc[j][i][2 * h + 1] = sl == 0 ? v[1] : acc[j][i][2 * h + 1] + v[1];
                    }
        }
    }

    // ---- epilogue: lane holds Y[m = i*16 + r16][n = j*16 + 4*kg + 0..3] of its 64x64 wave tile ----
    auto epilogue = [&](auto has_bias_const) {
        constexpr bool HB = decltype(has_bias_const)::value;
        float bj[SNP][4];
#pragma unroll
        for (int j = 0; j < SNP; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int n = n0 + wn * SWN + j * 16 + 4 * kg + e;
                bj[j][e] = HB && n < N ? (float)bias[n] : 0.f;
            }
        if ((ldn & 7) == 0) {
            constexpr int kPitch = 144;  // 64 fp16 + 16 bytes: rows land in different banks
            uint8_t *stage_out = smem + wave * (SWM * kPitch);
#pragma unroll
            for (int i = 0; i < SMP; i++)
#pragma unroll
                for (int j = 0; j < SNP; j++)
                    *reinterpret_cast<half4_t *>(stage_out + (i * 16 + r16) * kPitch + (j * 16 + 4 * kg) * 2) =
                        round4<HB>(acc[j][i], bj[j]);
#pragma unroll
            for (int it = 0; it < SWM / 8; it++) {
                const int row = it * 8 + (lane >> 3), c = lane & 7;
                const uint4_t v = *reinterpret_cast<const uint4_t *>(stage_out + row * kPitch + c * 16);
                const int m = m0 + wm * SWM + row;
                const int n = n0 + wn * SWN + c * 8;
                if (m < M && n < N) st_global_16_streaming(y + (int64_t)m * ldn + n, v);
            }
        } else {
#pragma unroll
            for (int i = 0; i < SMP; i++) {
                const int m = m0 + wm * SWM + i * 16 + r16;
                if (m >= M) continue;
#pragma unroll
                for (int j = 0; j < SNP; j++) {
                    const int n = n0 + wn * SWN + j * 16 + 4 * kg;
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
        if (bias) store_gated<SNP, SMP, true>(acc, y, bias, M, N, ldn, m0 + wm * SWM, n0 + wn * SWN, r16, kg);
        else store_gated<SNP, SMP, false>(acc, y, bias, M, N, ldn, m0 + wm * SWM, n0 + wn * SWN, r16, kg);
        return;
    }
    if (bias) epilogue(std::true_type{});
    else epilogue(std::false_type{});
}

template <int VEC, typename CodeT>
size_t lds_bytes_small(const ProblemB &p, int ns)
{
    typedef PrefillCfg<VEC, CodeT> C;
    return (size_t)ns * kSmallStage + (size_t)small_code_bufs<VEC, CodeT>(ns) * C::CH * SBN * 16 + books_bytes(p, SBN);
}

// whole code tiles along K, a tile's offsets within 32 bits, the LDS holds the tile's codebooks
template <int VEC, typename CodeT>
bool small_cfg_supports(const ProblemB &p)
{
    typedef PrefillCfg<VEC, CodeT> C;
    return p.K >= C::K_SUPER && p.K % C::K_SUPER == 0 && lds_bytes_small<VEC, CodeT>(p, 4) <= kLdsLimit &&
           (int64_t)SBN * (p.K / VEC) * (int64_t)sizeof(CodeT) < ((int64_t)1 << 31) &&
           (int64_t)SBM * p.K * 2 < ((int64_t)1 << 32);
}

// float4 slots of partial sums per tile and slice, and where the tiles' counters start inside the workspace
constexpr size_t kPartialBytes = (size_t)SNP * SMP * kThreads * 16;  // 64 KB

// n_begin: the launch covers the W rows [n_begin, N) only (a multiple of the tile's 128 rows)
template <int VEC, typename CodeT>
hipError_t launch_small_typed(const ProblemB &p, hipStream_t s, int splits, void *workspace, int n_begin)
{
    typedef PrefillCfg<VEC, CodeT> C;
    if (!small_cfg_supports<VEC, CodeT>(p)) return hipErrorInvalidValue;
    if (splits < 1 || p.K % splits != 0 || (p.K / splits) % C::K_SUPER != 0 || (splits > 1 && !workspace)) return hipErrorInvalidValue;
    if (n_begin < 0 || n_begin >= p.N || n_begin % SBN != 0) return hipErrorInvalidValue;
    const int tiles_m = (p.M + SBM - 1) / SBM, tiles_n = (p.N - n_begin + SBN - 1) / SBN;
    // workspace: the tiles' counters (cleared here, by a kernel: the launch may be captured), then the partial sums
    unsigned int *counters = static_cast<unsigned int *>(workspace);
    float4_t *partials = nullptr;
    if (splits > 1) {
        const size_t counter_bytes = prefill_splitk_counter_bytes(tiles_m * tiles_n);
        partials = reinterpret_cast<float4_t *>(static_cast<uint8_t *>(workspace) + counter_bytes);
        const hipError_t e = launch_clear_words(counters, tiles_m * tiles_n, s);
        if (e != hipSuccess) return e;
    }
    const size_t smem = lds_bytes_small<VEC, CodeT>(p, 4);
    // the split codebook layout is built out of a copy in the last X buffer
    constexpr bool can_split = VEC == 8 && sizeof(CodeT) == 1;
    const bool split = can_split && split_layout_applies(p, codebooks_per_tile(p, SBN), kSmallStage);
    auto kern = split ? prefill_small_kernel<VEC, CodeT, 4, can_split> : prefill_small_kernel<VEC, CodeT, 4, false>;
    const hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n * splits)), dim3(kThreads), smem, s, p.x,
                       static_cast<const CodeT *>(p.codes), p.cb, p.y, p.bias, p.M, p.K, p.N, n_begin, p.N, p.entries,
                       p.rows_per_cb, tiles_m, tiles_n, codebooks_per_tile(p, SBN), p.gated ? 1 : 0, p.K / splits, splits, partials, counters,
                       tuning().splitk_validate_fences >= 1.0 ? 1 : 0);
    return hipGetLastError();
}

}  // namespace

bool prefill_small_supports(const ProblemB &p)
{
    if (p.M < 1 || p.N < 1 || p.K < 1) return false;
    if (((size_t)p.entries * p.vec * 2) % 16 != 0) return false;
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? small_cfg_supports<8, uint8_t>(p) : small_cfg_supports<8, uint16_t>(p);
    case 4: return u8 ? small_cfg_supports<4, uint8_t>(p) : small_cfg_supports<4, uint16_t>(p);
    case 2: return u8 && small_cfg_supports<2, uint8_t>(p);
    default: return false;
    }
}

// Microseconds the kernel is expected to take, fitted to measurements: the tiles go over the
// compute units in rounds (a second workgroup on a unit shares its LDS bandwidth, which is what
// bounds this tile, and gains nothing in the main loop; it does overlap its prologue and epilogue
// with the other's work); a tile costs 4 us plus K/64 stages of 0.46 us on an idle device, 0.56 us
// when every unit works.
double prefill_small_cost_us(const ProblemB &p)
{
    if (!prefill_small_supports(p)) return 1e30;
    const int cus = device_cu_count();
    const int64_t tiles = (int64_t)((p.M + SBM - 1) / SBM) * ((p.N + SBN - 1) / SBN);
    const int64_t rounds = (tiles + cus - 1) / cus, resident_rounds = (tiles + 2 * cus - 1) / (2 * cus);
    const double busy = tiles >= cus ? 1.0 : (double)tiles / cus;
    const Tuning &tn = tuning();
    return (double)resident_rounds * tn.prefill_small_tile_fixed_us +
           (double)rounds * (p.K / 64.0 * (tn.prefill_small_stage_us_idle + (tn.prefill_small_stage_us_busy - tn.prefill_small_stage_us_idle) * busy));
}

hipError_t launch_prefill_small_b(const ProblemB &p, hipStream_t s, int splits, void *workspace, int n_begin)
{
    if (!prefill_small_supports(p)) return hipErrorInvalidValue;
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? launch_small_typed<8, uint8_t>(p, s, splits, workspace, n_begin) : launch_small_typed<8, uint16_t>(p, s, splits, workspace, n_begin);
    case 4: return u8 ? launch_small_typed<4, uint8_t>(p, s, splits, workspace, n_begin) : launch_small_typed<4, uint16_t>(p, s, splits, workspace, n_begin);
    default: return launch_small_typed<2, uint8_t>(p, s, splits, workspace, n_begin);
    }
}

// the k one code tile of the format covers: a slice of K is whole code tiles
static int small_k_super(const ProblemB &p)
{
    const int csz = p.code_bits / 8;
    const int kc = (16 / csz) * p.vec;
    return kc > kStageK ? kc : kStageK;
}

size_t prefill_splitk_counter_bytes(int64_t tiles) { return ((size_t)tiles * 4 + 255) & ~(size_t)255; }

size_t prefill_splitk_workspace_bytes(const ProblemB &p, int splits)
{
    if (splits <= 1) return 0;
    const int64_t tiles = (int64_t)((p.M + SBM - 1) / SBM) * ((p.N + SBN - 1) / SBN);
    return prefill_splitk_counter_bytes(tiles) + (size_t)tiles * splits * kPartialBytes;
}

bool prefill_splitk_supports(const ProblemB &p, int splits)
{
    return splits >= 2 && splits <= 8 && prefill_small_supports(p) && p.K % splits == 0 && (p.K / splits) % small_k_super(p) == 0 &&
           p.K / splits >= 2 * small_k_super(p);
}

// The number of slices of K (1: none) that the cost model expects to be fastest with 128x128 tiles, and its time.
// A slice is a workgroup of its own: `splits` times the tiles, each over K / splits; on top of that the clearing launch
// and, per tile, the partial sums written and read once (Tuning::splitk_fixed_us, splitk_us_per_partial_mb).
int prefill_splitk_choice(const ProblemB &p, double *cost_us, int min_splits)
{
    int best = min_splits <= 1 ? 1 : 0;
    double best_us = min_splits <= 1 ? prefill_small_cost_us(p) : 1e30;
    const Tuning &tn = tuning();
    const int64_t tiles = (int64_t)((p.M + SBM - 1) / SBM) * ((p.N + SBN - 1) / SBN);
    if (min_splits >= 2 && tn.splitk_force_splits >= 2.0 && prefill_splitk_supports(p, (int)tn.splitk_force_splits)) {
        if (cost_us) *cost_us = 0.0;
        return (int)tn.splitk_force_splits;
    }
    for (int sp = 2; sp <= 8; sp *= 2) {
        if (!prefill_splitk_supports(p, sp)) break;
        ProblemB q = p;  // the slices as the kernel sees them: sp times the tiles over K / sp
        q.K = p.K / sp;
        const int cus = device_cu_count();
        const int64_t wgs = tiles * sp;
        const int64_t rounds = (wgs + cus - 1) / cus, resident_rounds = (wgs + 2 * cus - 1) / (2 * cus);
        const double busy = wgs >= cus ? 1.0 : (double)wgs / cus;
        const double main_us = (double)resident_rounds * tn.prefill_small_tile_fixed_us +
                               (double)rounds * (q.K / 64.0 * (tn.prefill_small_stage_us_idle + (tn.prefill_small_stage_us_busy - tn.prefill_small_stage_us_idle) * busy));
        const double fix_us = tn.splitk_fixed_us + tn.splitk_us_per_partial_mb * (double)(wgs * kPartialBytes) / 1e6;
        if (main_us + fix_us < best_us) {
            best_us = main_us + fix_us;
            best = sp;
        }
    }
    if (cost_us) *cost_us = best_us;
    return best;
}

}  // namespace vq
