// General decode kernel (16 rows of X per launch): Y[M,N] = X[M,K] . W^T with W given as codes +
// codebook, for the shapes the batched kernel of vq_decode.hip does not take: K beyond 4096 or
// not a multiple of 256, several codebooks, N not a multiple of 16.
//
//   * A workgroup owns tiles of 16 output columns (16 rows of W).  Each of its up to eight waves
//     owns a 512-wide (K <= 4096) or 1024-wide slice of K and keeps the matching slice of X in
//     registers, already in MFMA operand order; K beyond eight slices goes in chunks, X being
//     reloaded per chunk.
//   * The codebook (entries*vec*2 bytes) is resident in the LDS.  A lane streams 16 bytes of
//     codes of one W row, gathers the codewords and uses them directly as the 8-half A operand
//     of v_mfma_f32_16x16x32_f16.  The order in which a lane walks K is irrelevant to a dot
//     product, so it is chosen so that each lane's codes are contiguous in memory; X is loaded
//     in the same order.
//   * Per tile the partial 16x16 fp32 results of the waves are summed through 1 KB LDS slots,
//     and one wave converts and stores the tile.
//   * The gated epilogue of a gate/up pair (rows of W interleaved in groups of 16, so an even tile
//     holds gate rows and the tile behind it the up rows of the same sixteen outputs): the
//     workgroups are dealt whole pairs of tiles, one wave sums both tiles of a pair - it keeps the
//     gate sums in registers until the up tile has been multiplied - and stores silu(gate) * up
//     into Y [M, N/2].
//
// M < 16 pads the X operand with zeros; fp32 accumulation throughout, one rounding to fp16.
#include "vq_common.h"

namespace vq {

namespace {

constexpr int kTileN = 16;
constexpr int kMaxWaves = 8;   // 512 threads: leaves 256 registers per lane

// STEPS = MFMA steps (32 k each) of the K slice one wave owns: 16 (512 k) up to K = 4096,
// 32 (1024 k, X slice of 128 registers) beyond, so that K = 8192 still needs one pass.
template <int VEC, typename CodeT, int STEPS = 16>
struct DecodeCfg {
    static constexpr int kSliceK = 32 * STEPS;
    static constexpr int kSteps = STEPS;
    static constexpr int CPL = 16 / (int)sizeof(CodeT);  // codes in one 16-byte lane load
    static constexpr int CPO = 8 / VEC;                  // codes per 8-half MFMA operand
    static constexpr int SPL = CPL / CPO;                // MFMA steps fed by one lane load
    static constexpr int K_LANE = CPL * VEC;             // k covered by one lane load
    static constexpr int K_WAVE = 4 * K_LANE;            // k covered by one wave load (4 k-groups)
    static constexpr int LPT = kSliceK / K_WAVE;         // lane loads per slice
    // (tile, chunk) code loads kept in flight, as many as the registers allow
    static constexpr int PF = STEPS <= 16 ? (LPT <= 4 ? 4 : 2) : (LPT <= 2 ? 2 : 1);
    static_assert(CPO >= 1 && SPL >= 1 && LPT >= 1 && LPT * SPL == kSteps, "unsupported code layout");
};

template <typename CodeT, int CPL>
__device__ __forceinline__ uint32_t extract_code(const uint4_t &cw, int c)
{
    if constexpr (sizeof(CodeT) == 1)
        return (cw[c >> 2] >> (8 * (c & 3))) & 0xffu;
    else
        return (cw[c >> 1] >> (16 * (c & 1))) & 0xffffu;
}

// Gather the 8-half operand made of CPO consecutive codewords starting at code c0.
// STRIDE is the byte distance between codebook entries in the LDS: the entry size for a plain
// codebook, 256 for the bank-replicated one (see decode_kernel).
template <int VEC, typename CodeT, int STRIDE>
__device__ __forceinline__ half8_t gather_operand(const uint8_t *cb_lds, const uint4_t &cw, int c0)
{
    typedef DecodeCfg<VEC, CodeT> C;
    if constexpr (VEC == 8) {
        const uint32_t code = extract_code<CodeT, C::CPL>(cw, c0);
        return *reinterpret_cast<const half8_t *>(cb_lds + code * (uint32_t)STRIDE);
    } else if constexpr (VEC == 4) {
        const uint32_t a = extract_code<CodeT, C::CPL>(cw, c0);
        const uint32_t b = extract_code<CodeT, C::CPL>(cw, c0 + 1);
        const half4_t lo = *reinterpret_cast<const half4_t *>(cb_lds + a * (uint32_t)STRIDE);
        const half4_t hi = *reinterpret_cast<const half4_t *>(cb_lds + b * (uint32_t)STRIDE);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    } else {
        static_assert(VEC == 2, "vector length must be 2, 4 or 8");
        half2_t q[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t c = extract_code<CodeT, C::CPL>(cw, c0 + i);
            q[i] = *reinterpret_cast<const half2_t *>(cb_lds + c * (uint32_t)STRIDE);
        }
        const half4_t lo = __builtin_shufflevector(q[0], q[1], 0, 1, 2, 3);
        const half4_t hi = __builtin_shufflevector(q[2], q[3], 0, 1, 2, 3);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
}


// s_waitcnt for the vector-memory counter only (gfx9 encoding: vmcnt = simm16[15:14]:[3:0]).
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
    asm volatile("" ::: "memory");  // keep the compiler from moving LDS reads above the wait
}

// stage_off >= 0: the X slices are staged through the LDS at that offset (n_chunks == 1 only);
// `aliased` says that the staging area overlaps the codebook, which is then loaded afterwards.
//
// REPL: bank-replicated codebook.  A gather at uniformly random entries loses more than half of
// the LDS bandwidth to bank conflicts, and at 16 LDS bytes read per code byte streamed the LDS is
// what bounds a long u8/v8 GEMV.  With at most 256 entries the codebook is laid out as one
// 256-byte bank row per entry holding 256/entry_bytes copies of it; lane l reads copy
// l % copies, so the lanes served together never share a bank whatever the codes are.
template <int VEC, typename CodeT, int STEPS, bool REPL>
__global__ __launch_bounds__(512) void decode_general_kernel(const half_t *__restrict__ x,
                                                      const CodeT *__restrict__ codes,
                                                      const half_t *__restrict__ cb,
                                                      half_t *__restrict__ y,
                                                      const half_t *__restrict__ bias, int M, int K, int N,
                                                      int entries, int rows_per_cb, int tiles_q,
                                                      int tiles_r, int n_chunks, int stage_off,
                                                      int aliased, int gated)
{
    typedef DecodeCfg<VEC, CodeT, STEPS> C;
    constexpr int kSliceK = C::kSliceK;
    constexpr int kSteps = C::kSteps;
    constexpr int kStagePitch = kSliceK * 2 + 16;  // bytes per staged X row slice; the pad spreads rows over the banks
    extern __shared__ __align__(16) uint8_t smem[];
    const int n_waves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15;  // W row within the tile (A operand) / X row m (B operand)
    const int kq = lane >> 4;   // k-group of the lane, 0..3
    const int J = K / VEC;
    const int cb_bytes = entries * VEC * 2;
    constexpr int kEntryBytes = VEC * 2;
    constexpr int kStride = REPL ? 256 : kEntryBytes;
    const int cb_lds_bytes = REPL ? entries * 256 : ((cb_bytes + 15) & ~15);
    uint8_t *cb_lds = smem;
    // Lane's copy of the entries in the replicated layout (0 in the plain one).
    const uint8_t *cb_gather = smem + (REPL ? (lane % (256 / kEntryBytes)) * kEntryBytes : 0);
    float4_t *red = reinterpret_cast<float4_t *>(smem + cb_lds_bytes);

    // Balanced contiguous split of the tiles over the workgroups: tiles_q each, one more for the
    // first tiles_r (quotient and remainder of tiles / workgroups, computed by the host).
    // (gated: tiles_q and tiles_r count pairs of a gate and an up tile)
    const int wg = blockIdx.x;
    const int deal = gated ? 2 : 1;
    const int tile_begin = deal * (wg * tiles_q + min(wg, tiles_r));
    const int tile_end = tile_begin + deal * (tiles_q + (wg < tiles_r ? 1 : 0));
    if (tile_begin >= tile_end) return;

    // k of MFMA step s for this lane inside a slice that starts at k0.
    auto step_k = [&](int k0, int s) { return k0 + (s / C::SPL) * C::K_WAVE + kq * C::K_LANE + (s % C::SPL) * 8; };

    half8_t xr[kSteps];
    auto load_x = [&](int k0) {
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            const int k = step_k(k0, s);
            uint4_t v = {0u, 0u, 0u, 0u};
            if (r16 < M && k < K) v = ld_global_16(x + (int64_t)r16 * K + k);
            xr[s] = as_half8(v);
        }
    };
    auto load_codes = [&](int tile, int k0, uint4_t (&cw)[C::LPT]) {
        const int row = min(tile * kTileN + r16, N - 1);
#pragma unroll
        for (int t = 0; t < C::LPT; t++) {
            const int k = k0 + t * C::K_WAVE + kq * C::K_LANE;
            uint4_t v = {0u, 0u, 0u, 0u};
            if (k < K) v = ld_global_16(codes + (int64_t)row * J + k / VEC);
            cw[t] = v;
        }
    };
    auto load_codebook = [&](int g) {
        if constexpr (REPL) {
            // 16-byte slot i of the table belongs to entry i / 16; it holds 16 / entry_bytes copies.
            // All loads are issued before the first write so that their latencies overlap.
            typedef uint32_t entry_t __attribute__((ext_vector_type(kEntryBytes / 4)));
            const entry_t *src = reinterpret_cast<const entry_t *>(cb + (int64_t)g * entries * VEC);
            constexpr int kMaxIter = 4;  // loads in flight per thread and round
            for (int base = 0; base < entries * 16; base += kMaxIter * (int)blockDim.x) {
                entry_t e[kMaxIter];
#pragma unroll
                for (int j = 0; j < kMaxIter; j++) {
                    const int i = base + j * (int)blockDim.x + (int)threadIdx.x;
                    e[j] = src[(i < entries * 16 ? i : 0) >> 4];
                }
#pragma unroll
                for (int j = 0; j < kMaxIter; j++) {
                    const int i = base + j * (int)blockDim.x + (int)threadIdx.x;
                    uint4_t v;
#pragma unroll
                    for (int d = 0; d < 4; d++) v[d] = e[j][d % (kEntryBytes / 4)];
                    if (i < entries * 16) reinterpret_cast<uint4_t *>(cb_lds)[i] = v;
                }
            }
        } else {
            const uint4_t *src = reinterpret_cast<const uint4_t *>(cb + (int64_t)g * entries * VEC);
            for (int i = threadIdx.x; i < cb_bytes / 16; i += blockDim.x) reinterpret_cast<uint4_t *>(cb_lds)[i] = src[i];
        }
    };

    const int chunk_k = n_waves * kSliceK;
    // The unit of work is a (tile, chunk) pair; the codes of the next PF units are always in
    // flight, so a workgroup with only a few tiles pays the memory latency once, not per tile.
    const int q_begin = tile_begin * n_chunks, q_end = tile_end * n_chunks;
    constexpr int PF = C::PF;
    uint4_t cwq[PF][C::LPT];
    auto load_unit = [&](int q, uint4_t (&cw)[C::LPT]) {
        const int tile = n_chunks == 1 ? q : q / n_chunks, chunk = q - tile * n_chunks;
        load_codes(tile, chunk * chunk_k + wave * kSliceK, cw);
    };
#pragma unroll
    for (int u = 0; u < PF; u++)
        if (q_begin + u < q_end) load_unit(q_begin + u, cwq[u]);

    // Small codebooks are fetched into registers up front so that their latency overlaps the
    // X staging even when the staging area and the codebook share LDS space.
    const int cb_chunks = cb_bytes / 16;
    const bool cb_in_regs = !REPL && cb_chunks <= 4 * (int)blockDim.x;
    uint4_t cb_regs[4];
    auto fetch_codebook = [&](int g) {
        const uint4_t *src = reinterpret_cast<const uint4_t *>(cb + (int64_t)g * entries * VEC);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = threadIdx.x + j * blockDim.x;
            cb_regs[j] = i < cb_chunks ? src[i] : uint4_t{0u, 0u, 0u, 0u};
        }
    };
    auto store_codebook = [&]() {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = threadIdx.x + j * blockDim.x;
            if (i < cb_chunks) reinterpret_cast<uint4_t *>(cb_lds)[i] = cb_regs[j];
        }
    };

    // Everything the first tile waits for is requested before anything is waited for: codes
    // (above), codebook, X.
    int cur_cb = -1;
    const int g0 = rows_per_cb >= N ? 0 : (tile_begin * kTileN) / rows_per_cb;
    if (stage_off < 0 && cb_in_regs) fetch_codebook(g0);
    if (stage_off >= 0) {
        // X -> registers through the LDS.  A lane needs 16-byte pieces scattered over its row
        // slice; fetched directly, every load instruction touches dozens of cache lines and
        // uses 16 bytes of each.  Instead the wave copies each row slice (1 KB, contiguous) into
        // a private LDS window and the lanes pick their pieces from there.
        const int k0 = wave * kSliceK;
        const uint32_t win = stage_off + wave * M * kStagePitch;
        for (int i = 0; i < M; i++)
#pragma unroll
            for (int h = 0; h < kSliceK / 512; h++) {
                const int kl = k0 + h * 512 + 8 * lane;
                load_to_lds_16(win + i * kStagePitch + h * 1024, (uint32_t)((i * K + (kl < K ? kl : 0)) * 2), x);
            }
        const int g = g0;
        if (cb_in_regs) fetch_codebook(g);
        else if (!aliased) load_codebook(g);
        wait_vmcnt<0>();
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            const int k = step_k(k0, s);
            uint4_t v = {0u, 0u, 0u, 0u};
            if (r16 < M && k < K) v = *reinterpret_cast<const uint4_t *>(smem + win + r16 * kStagePitch + (k - k0) * 2);
            xr[s] = as_half8(v);
        }
        if (aliased) __syncthreads();  // every wave has picked up its X before the codebook overwrites it
        if (cb_in_regs) store_codebook();
        else if (aliased) load_codebook(g);
        __syncthreads();
        cur_cb = g;
    } else {
        if (n_chunks == 1) load_x(wave * kSliceK);
        if (cb_in_regs) {
            store_codebook();
            __syncthreads();
            cur_cb = g0;
        }
    }

    int parity = 0;
    float4_t gate_sum = {0.f, 0.f, 0.f, 0.f};  // gated: the gate tile's sums, in the wave that takes the pair, until the up tile is done
    // Four accumulators: consecutive MFMAs do not wait on each other's result.
    float4_t acc[4];
#pragma unroll
    for (int a = 0; a < 4; a++) acc[a] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int qb = q_begin; qb < q_end; qb += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const int q = qb + u;
            if (q >= q_end) break;
            const int tile = n_chunks == 1 ? q : q / n_chunks, chunk = q - tile * n_chunks;
            const int g = rows_per_cb >= N ? 0 : (tile * kTileN) / rows_per_cb;
            if (g != cur_cb) {
                // (Re)load the codebook of this row block into the LDS.
                if (cur_cb >= 0) __syncthreads();
                load_codebook(g);
                __syncthreads();
                cur_cb = g;
            }
            uint4_t cw[C::LPT];
#pragma unroll
            for (int t = 0; t < C::LPT; t++) cw[t] = cwq[u][t];
            if (q + PF < q_end) load_unit(q + PF, cwq[u]);
            if (n_chunks > 1) load_x(chunk * chunk_k + wave * kSliceK);
#pragma unroll
            for (int s = 0; s < kSteps; s++) {
                const half8_t a = gather_operand<VEC, CodeT, kStride>(cb_gather, cw[s / C::SPL], (s % C::SPL) * C::CPO);
                acc[s & 3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, xr[s], acc[s & 3], 0, 0, 0);
                // Bound how far the scheduler hoists gathers ahead of their MFMAs (register pressure).
                if (STEPS > 16 && (s & 7) == 7) __builtin_amdgcn_sched_barrier(0);
            }
            if (chunk != n_chunks - 1) continue;

            const float4_t p = (acc[0] + acc[1]) + (acc[2] + acc[3]);
#pragma unroll
            for (int a = 0; a < 4; a++) acc[a] = float4_t{0.f, 0.f, 0.f, 0.f};
            // Sum the K slices of the waves through LDS slots (parity, wave, lane); the waves take
            // turns at adding up and storing a tile.
            red[(parity * n_waves + wave) * 64 + lane] = p;
            __syncthreads();
            // (gated: both tiles of a pair go to the same wave)
            if (wave == ((gated ? tile >> 1 : tile) % n_waves)) {
                float4_t sum = red[(parity * n_waves) * 64 + lane];
                for (int w = 1; w < n_waves; w++) {
                    const float4_t v = red[(parity * n_waves + w) * 64 + lane];
                    sum += v;
                }
                // D[i][j]: j = lane % 16 is the X row m, i = 4*(lane/16) + r is the W row.
                const int m = r16;
                const int n = tile * kTileN + 4 * kq;
                if (bias) {
#pragma unroll
                    for (int r = 0; r < 4; r++) sum[r] += n + r < N ? (float)bias[n + r] : 0.f;
                }
                if (gated) {
                    if ((tile & 1) == 0) {
                        gate_sum = sum;
                    } else if (m < M) {
                        // outputs (tile / 2) * 16 + 4*kq .. + 3 (N is a multiple of 32: no ragged edge)
                        half4_t h;
#pragma unroll
                        for (int r = 0; r < 4; r++) h[r] = (half_t)(silu_f32(gate_sum[r]) * sum[r]);
                        *reinterpret_cast<half4_t *>(y + (int64_t)m * (N / 2) + (tile >> 1) * kTileN + 4 * kq) = h;
                    }
                } else if (m < M) {
                    half_t *dst = y + (int64_t)m * N + n;
                    if ((N & 3) == 0 && n + 3 < N) {
                        half4_t h = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
                        *reinterpret_cast<half4_t *>(dst) = h;
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (n + r < N) dst[r] = (half_t)sum[r];
                    }
                }
            }
            parity ^= 1;
        }
    }
}

constexpr size_t kDecodeLdsLimit = 160 * 1024;
constexpr size_t kStageMinBytes = 32 * 1024;
constexpr size_t kDisjointBudget = 96 * 1024;  // keep at least two workgroups per CU when staging beside the codebook

template <int VEC, typename CodeT, int STEPS>
hipError_t launch_decode_steps(const ProblemB &p, hipStream_t s)
{
    typedef DecodeCfg<VEC, CodeT, STEPS> C;
    constexpr int kSliceK = C::kSliceK;
    const int slices = (p.K + kSliceK - 1) / kSliceK;
    const int n_waves = slices < kMaxWaves ? slices : kMaxWaves;
    const int n_chunks = (slices + n_waves - 1) / n_waves;
    const int n_tiles = (p.N + kTileN - 1) / kTileN;
    const int n_dealt = p.gated ? n_tiles / 2 : n_tiles;  // what the workgroups share: tiles, or pairs of a gate and an up tile
    const int cb_bytes = p.entries * VEC * 2;
    // Workgroups resident per CU: the kernel needs 129+ registers per lane, i.e. at most 3 waves
    // per SIMD.
    int per_cu = 12 / n_waves > 0 ? 12 / n_waves : 1;
    const int cus = device_cu_count();
    int grid = n_dealt < cus * per_cu ? n_dealt : cus * per_cu;
    const int tiles_per_wg = (p.gated ? 2 : 1) * ((n_dealt + grid - 1) / grid);
    // Replicated codebook (one 256-byte bank row per entry, <= 64 KB): worth its fill time only
    // when the workgroup gathers from it for several tiles.
    const bool repl = p.entries <= 256 && tiles_per_wg >= 4;
    const size_t base = (repl ? (size_t)p.entries * 256 : (size_t)((cb_bytes + 15) & ~15)) +
                        (size_t)2 * n_waves * 64 * sizeof(float4_t);
    const size_t stage = (size_t)n_waves * p.M * (kSliceK * 2 + 16);
    size_t smem = base;
    int stage_off = -1, aliased = 0;
    // Staging pays off when X is large enough for its scattered fetch to load the L1/L2 path;
    // a small X is read directly (one LDS round trip less on the critical path).
    if (n_chunks == 1 && (size_t)p.M * p.K * 2 > kStageMinBytes) {
        if (base + stage <= kDisjointBudget) {
            stage_off = (int)base;
            smem = base + stage;
        } else if (stage <= kDecodeLdsLimit) {
            stage_off = 0;
            aliased = 1;
            smem = stage > base ? stage : base;
        }
    }
    if ((size_t)per_cu * smem > kDecodeLdsLimit) {
        per_cu = (int)(kDecodeLdsLimit / smem) > 0 ? (int)(kDecodeLdsLimit / smem) : 1;
        grid = n_dealt < cus * per_cu ? n_dealt : cus * per_cu;
    }
    auto kern = repl ? decode_general_kernel<VEC, CodeT, STEPS, true> : decode_general_kernel<VEC, CodeT, STEPS, false>;
    hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(n_waves * 64), smem, s, p.x, static_cast<const CodeT *>(p.codes), p.cb,
                       p.y, p.bias, p.M, p.K, p.N, p.entries, p.rows_per_cb, n_dealt / grid, n_dealt % grid, n_chunks, stage_off, aliased,
                       p.gated ? 1 : 0);
    return hipGetLastError();
}

template <int VEC, typename CodeT>
hipError_t launch_decode_typed(const ProblemB &p, hipStream_t s)
{
    // 512-wide K slices up to K = 4096 (eight waves cover it), 1024-wide beyond - for the code
    // formats whose 1024-wide slice fits the registers (at most four lane loads per slice: 8-vectors,
    // 4-vectors with 8-bit codes).  The others would spill; they keep 512-wide slices and walk a
    // longer K in chunks.
    if constexpr (DecodeCfg<VEC, CodeT, 32>::LPT <= 4) {
        if (p.K > 8 * 512) return launch_decode_steps<VEC, CodeT, 32>(p, s);
    }
    return launch_decode_steps<VEC, CodeT, 16>(p, s);
}

template <int VEC, typename CodeT>
bool decode_cfg_supports(const ProblemB &p)
{
    typedef DecodeCfg<VEC, CodeT> C;
    return p.K % C::K_LANE == 0;  // whole 16-byte code loads, 16-byte aligned code rows
}

constexpr size_t kDecodeLdsBudget = 144 * 1024;  // codebook + reduction slots must fit the 160 KB LDS

}  // namespace

bool decode_general_supports(const ProblemB &p)
{
    if (p.M < 1 || p.N < 1 || p.K < 1) return false;
    // gated: whole pairs of a gate and an up tile (a pair may lie in two codebooks: the table is picked per tile)
    if (p.gated && p.N % (2 * kTileN) != 0) return false;
    if (p.vec != 2 && p.vec != 4 && p.vec != 8) return false;
    if (p.n_codebooks > 1 && p.rows_per_cb % kTileN != 0) return false;
    if ((size_t)p.entries * p.vec * 2 + 2 * kMaxWaves * 1024 > kDecodeLdsBudget) return false;
    if (p.K % 8 != 0) return false;
    if (((size_t)p.entries * p.vec * 2) % 16 != 0) return false;
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? decode_cfg_supports<8, uint8_t>(p) : decode_cfg_supports<8, uint16_t>(p);
    case 4: return u8 ? decode_cfg_supports<4, uint8_t>(p) : decode_cfg_supports<4, uint16_t>(p);
    default: return u8 ? decode_cfg_supports<2, uint8_t>(p) : decode_cfg_supports<2, uint16_t>(p);
    }
}

// One slab of at most 16 rows of X.
hipError_t launch_decode_general(const ProblemB &p, hipStream_t s)
{
    if (p.M > 16 || !decode_general_supports(p)) return hipErrorInvalidValue;
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? launch_decode_typed<8, uint8_t>(p, s) : launch_decode_typed<8, uint16_t>(p, s);
    case 4: return u8 ? launch_decode_typed<4, uint8_t>(p, s) : launch_decode_typed<4, uint16_t>(p, s);
    default: return u8 ? launch_decode_typed<2, uint8_t>(p, s) : launch_decode_typed<2, uint16_t>(p, s);
    }
}

}  // namespace vq
