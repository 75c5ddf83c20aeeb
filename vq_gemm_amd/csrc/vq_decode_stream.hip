// Small-batch decode on long rows of W (K beyond what the K-sliced batched kernel holds of X in its registers: it then
// walks K in chunks, and every chunk costs it a round of barriers, a fresh copy of X through the LDS and the latency
// of its first codes).  8-vectors, 8-bit codes, up to 16 rows of X per workgroup (taller X: one 16-row slab per
// index of the second grid dimension).
//
// One workgroup of sixteen waves per compute unit owns a group of one to seven tiles of 16 rows of W over the whole of
// K.  K is cut into pieces of 128 k and the pieces are dealt to the waves in turn (wave w takes pieces w, w + 16, ...):
// every wave streams its own pieces with no barrier and nothing shared inside the stream.
//   * The codes of all of a wave's pieces (one dword per piece and tile, from HBM) are requested at once, behind the
//     first pieces of X: their latency is paid once per group.
//   * X goes global memory -> registers -> the wave's own 4 KB block of the LDS -> MFMA operand registers, two or three
//     pieces ahead of the multiply.  (An operand holds 16 rows across adjacent lanes: loaded straight from global
//     memory a wave load is 64 separate 16-byte requests, and the launch then follows the number of rows of X at
//     0.6 us per row.  Fetched row-wise a wave load is four rows of 256 contiguous bytes.)
//   * A piece is four steps of v_mfma_f32_16x16x32_f16 per tile: lane (r, q) gathers the codeword of row r for the
//     q-th 8 k of each step out of the table in the LDS and meets row r of X with it.
//   * At the end the sixteen partial tiles of a tile are summed through the LDS in the order of the waves.
//   * The sixteen waves of a unit read sixteen neighbouring pieces at a time: two cache lines per row of the codes,
//     4 KB per row of X, so that the lines a wave touches are the ones its neighbours touch at the same time.
//   * Loads are unconditional (past the end of a wave's pieces the last one is requested again) and only the multiply
//     of a piece that does not exist is skipped, so that the compiler's wait counts stay exact.
// What a piece costs does not depend on M: X passes through the LDS as 16 rows whatever M is (4 KB written, 4 KB read
// per wave and piece, beside 4 KB of gathers per tile), and that traffic is what bounds the stream.
#include "vq_common.h"

#include <type_traits>

namespace vq {

namespace {

constexpr int kStreamWaves = 16;
constexpr int kPieceK = 128;                      // k per piece: four MFMA steps
constexpr int kPieceSteps = kPieceK / 32;
constexpr int kTile = 16;                         // rows of W per tile
constexpr int kReduceTiles = 4;                   // tiles summed per barrier
constexpr int kCopies = 16;                       // replicated table: copies per entry (one 256-byte bank row)
constexpr int kMaxTiles = 7;                      // tiles per group

// T: tiles per group; NP: pieces per wave at most (the loop over a wave's pieces is unrolled NP times: code registers
// and ring slots are then compile-time indices); REPL: the bank-replicated table (64 KB, conflict-free gathers) or the
// plain one (4 KB)
template <int T, int NP, bool REPL>
__global__ __launch_bounds__(kStreamWaves * 64) void decode_stream_kernel(const half_t *__restrict__ x,
                                                                         const uint8_t *__restrict__ codes,
                                                                         const half_t *__restrict__ cb,
                                                                         half_t *__restrict__ y,
                                                                         const half_t *__restrict__ bias, int m_total,
                                                                         int K, int N, int entries, int rows_per_cb,
                                                                         int groups_q, int groups_r, int n_tiles)
{
    constexpr int kTableSlots = REPL ? 256 * kCopies : 256;
    constexpr int kRT = T < kReduceTiles ? T : kReduceTiles;
    // table | per wave: one piece of X, 16 rows of 256 bytes, 16-byte chunks XOR-swizzled by the row | partial tiles
    // [tile of the round][wave][lane], a float4 each (they lie over the X blocks: the stream is over when they are written)
    constexpr int kXSlots = kStreamWaves * kTile * 16;
    constexpr int kPartialSlots = kRT * kStreamWaves * 64;
    __shared__ __align__(16) uint4_t lds[kTableSlots + (kXSlots > kPartialSlots ? kXSlots : kPartialSlots)];
    uint4_t *table = lds;
    float4_t *partial = reinterpret_cast<float4_t *>(lds + kTableSlots);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, kq = lane >> 4;
    const int slab_row = blockIdx.y * kTile;
    const int M = min(kTile, m_total - slab_row);
    const int J = K / 8;  // bytes per row of codes
    const int n_pieces = K / kPieceK;
    const int n_mine = (n_pieces - w + kStreamWaves - 1) / kStreamWaves;  // pieces w, w + 16, ... (may be none)

    // the workgroup's groups of T tiles: groups_q each, one more for the first groups_r workgroups
    const int g_begin = (int)blockIdx.x * groups_q + min((int)blockIdx.x, groups_r);
    const int g_end = g_begin + groups_q + ((int)blockIdx.x < groups_r ? 1 : 0);

    // X goes global memory -> registers -> the wave's own block of the LDS -> MFMA operand registers.  An operand holds
    // 16 rows across adjacent lanes, so loading it straight from global memory is 64 separate 16-byte requests per wave
    // load; fetched row-wise instead, a wave load is four rows of 256 contiguous bytes.  Load j of a piece: lane l takes
    // row 4j + l / 16 (rows past M read row M - 1: their columns of the product are never stored) and the chunk that
    // belongs into slot l % 16 of that row's LDS line, chunk = slot ^ row; the LDS write is then 1 KB contiguous.  Lane
    // (r16, kq) reads its operand of step s, chunk kq * 4 + s of row r16, from slot chunk ^ r16: sixteen rows, sixteen
    // different bank groups.  Nothing but the wave itself touches its block: no barrier, LDS operations of a wave
    // complete in order.
    const uint8_t *x_slab = reinterpret_cast<const uint8_t *>(x + (int64_t)slab_row * K);
    uint4_t *x_block = lds + kTableSlots + w * (kTile * 16);
    const int x_read_slot = r16 * 16;  // + (chunk ^ r16)
    const uint32_t code_lane_off = (uint32_t)(r16 * J + kq * 4);
    const uint32_t gather_base = REPL ? (uint32_t)(lane & (kCopies - 1)) * 16u : 0u;
    const uint8_t *tbl = reinterpret_cast<const uint8_t *>(table);

    for (int g = g_begin; g < g_end; g++) {
        const int tile0 = g * T;
        // The loads are unconditional (a piece past the wave's last is the last again, a tile past the end of a short
        // last group the last tile, every thread fetches a table entry) and only the multiply of a piece that does
        // not exist is skipped: no load sits in a branch, and the compiler's wait counts stay exact.  Order of issue =
        // order of completion: the table entry (L2) first, then all the codes (HBM), then the first pieces of X (L2).
        const half_t *cbg = cb + (int64_t)(tile0 * kTile / rows_per_cb) * entries * 8;
        const int e = (tid >> 1) & 255, h = tid & 1;
        uint4_t entry = reinterpret_cast<const uint4_t *>(cbg)[min(e, entries - 1)];
        // (the count of the wave's pieces goes through an empty asm once per group, so that the fourteen comparisons
        // with it are not all made ahead of the loop over the groups and kept in scalar registers)
        int n_mine_g = n_mine;
        asm volatile("" : "+s"(n_mine_g));
        const int last_piece = min(w + kStreamWaves * (max(n_mine_g, 1) - 1), n_pieces - 1);
        auto piece_of = [&](int i) { return min(w + kStreamWaves * i, last_piece); };
        // (the lane offsets go through an empty asm once per group: what does not change from group to group - X
        // altogether, the lane's part of every address - would otherwise be computed, or loaded, ahead of the loop over
        // the groups and held in registers through it)
        uint32_t c_off = code_lane_off, x_off[4];  // x_off[j]: row and chunk of the lane in load j, as a byte offset inside the slab
        int lane_g = lane;
        asm volatile("" : "+v"(c_off), "+v"(lane_g));
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int row = 4 * j + (lane_g >> 4);
            x_off[j] = (uint32_t)(min(row, M - 1) * K * 2 + (((lane_g & 15) ^ row) & 15) * 16);
        }
        // two pieces of X on their way in registers while a third is put into the wave's LDS block (what is in flight
        // has to cover the latency of the L2 at the rate the unit's L1 delivers: 16 waves x 2 pieces x 4 KB), one in
        // the block, one in operand registers
        // (with many code registers one piece less: its iterations are longer, and the registers are needed)
        constexpr int kXRing = (NP * T >= 16 || NP > 8 || T > 2) ? 2 : 3;
        uint4_t xs[kXRing][4];
        auto load_x = [&](int i, uint4_t (&xd)[4]) {
            const uint32_t piece_off = (uint32_t)(piece_of(i) * (kPieceK * 2));
#pragma unroll
            for (int j = 0; j < 4; j++) xd[j] = *reinterpret_cast<const uint4_t *>(x_slab + (uint32_t)(x_off[j] + piece_off));
        };
        // (only the rows of X that exist go through the LDS: the traffic of a piece is what the stream waits for)
        auto stage_x = [&](const uint4_t (&xd)[4]) {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (4 * j < M) x_block[j * 64 + lane] = xd[j];
        };
        auto pick_x = [&](uint4_t (&xo)[kPieceSteps]) {
            if (r16 < M) {
#pragma unroll
                for (int s2 = 0; s2 < kPieceSteps; s2++) xo[s2] = x_block[x_read_slot + (((kq * 4 + s2) ^ r16) & 15)];
            }
        };
        // (the first pieces of X go out ahead of the codes: they come out of the L2 and are in the block and in operand
        // registers by the time the codes arrive from HBM)
#pragma unroll
        for (int i = 0; i < kXRing && i < NP; i++) load_x(i, xs[i]);
        __builtin_amdgcn_sched_barrier(0);
        uint32_t cw[NP][T];
#pragma unroll
        for (int i = 0; i < NP; i++) {
            const int p = piece_of(i);
#pragma unroll
            for (int t = 0; t < T; t++) {
                const int tile = min(tile0 + t, n_tiles - 1);
                // (the tile's rows as the wave-uniform base, the piece inside the 32-bit offset)
                const uint8_t *base = codes + (int64_t)tile * kTile * J;
                cw[i][t] = __hip_atomic_load(reinterpret_cast<const uint32_t *>(base + (uint32_t)(c_off + p * (kPieceK / 8))),
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
            }
        }
        __builtin_amdgcn_sched_barrier(0);

        // ---- the table of the group's codebook (the waves are past the barrier behind the sums of the group before:
        // its gathers are long done) ----------------------------------------------------------------
        if (e >= entries) entry = uint4_t{0u, 0u, 0u, 0u};  // entries past a short codebook are zeros
        if constexpr (REPL) {
            // thread (e, h) of the first 512 writes eight of entry e's sixteen copies, rotated so that the sixteen lanes
            // served together go to sixteen different bank groups
            if (tid < 512) {
#pragma unroll
                for (int i = 0; i < 8; i++) table[e * kCopies + h * 8 + ((e + i) & 7)] = entry;
            }
        } else if (tid < 512 && h == 0) {
            table[e] = entry;
        }
        __syncthreads();

        // ---- the stream ---------------------------------------------------------------------------
        // (two accumulators per tile while there are one or two tiles: a chain of dependent MFMAs is half as long; with
        // more tiles the tiles' chains interleave)
        constexpr int kAcc = T > 2 ? 1 : 2;
        float4_t acc[T][kAcc];
#pragma unroll
        for (int t = 0; t < T; t++)
#pragma unroll
            for (int a = 0; a < kAcc; a++) acc[t][a] = float4_t{0.f, 0.f, 0.f, 0.f};
        auto multiply_piece = [&](const uint4_t (&xd)[kPieceSteps], const uint32_t (&cd)[T]) {
#pragma unroll
            for (int t = 0; t < T; t++) {
                // the four gathers of the tile's dword go out together, the four products follow
                uint4_t wv[kPieceSteps];
#pragma unroll
                for (int s = 0; s < kPieceSteps; s++) {
                    // gather address: code * 256 + copy * 16 through one byte permute (replicated), code * 16 (plain)
                    const uint32_t addr = REPL ? __builtin_amdgcn_perm(cd[t], gather_base, 0x0c0c0000u | ((4u + s) << 8))
                                               : ((cd[t] >> (8 * s)) & 0xffu) << 4;
                    wv[s] = *reinterpret_cast<const uint4_t *>(tbl + addr);
                }
#pragma unroll
                for (int s = 0; s < kPieceSteps; s++)
                    acc[t][s % kAcc] = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(wv[s]), as_half8(xd[s]), acc[t][s % kAcc], 0, 0, 0);
            }
        };
        // piece 0 into the block and out of it into operand registers; then per piece: the next piece into the block and
        // out of it into the other set of operand registers (the wave's own LDS operations complete in order), the piece
        // after the ring requested, the multiply
        // (with two tiles a single set of operand registers, picked up in front of the multiply)
        constexpr int kXO = T > 1 ? 1 : 2;
        uint4_t xo[kXO][kPieceSteps];
        stage_x(xs[0]);
        if (kXO == 2) pick_x(xo[0]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < NP; i++) {
            if (kXO == 1 && i < n_mine_g) pick_x(xo[0]);
            // (pieces past the wave's last are requested - clamped - but not put through the LDS)
            if (i + 1 < NP && i + 1 < n_mine_g) {
                stage_x(xs[(i + 1) % kXRing]);
                if (kXO == 2) pick_x(xo[(i + 1) % kXO]);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (i + kXRing < NP) load_x(i + kXRing, xs[i % kXRing]);  // (the slot of piece i, which went into the block one piece ago)
            __builtin_amdgcn_sched_barrier(0);
            if (i < n_mine_g) multiply_piece(xo[i % kXO], cw[i]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (T > 0) __syncthreads();  // every wave is done with its block of X: the partial tiles lie over the blocks

        // ---- the sums across the waves, kRT tiles per round ------------------------------------------
#pragma unroll
        for (int r0 = 0; r0 < T; r0 += kRT) {
            if (r0 > 0) __syncthreads();  // the round before has been read
#pragma unroll
            for (int t = r0; t < r0 + kRT && t < T; t++) partial[((t - r0) * kStreamWaves + w) * 64 + lane] = kAcc == 2 ? acc[t][0] + acc[t][kAcc - 1] : acc[t][0];
            __syncthreads();
            // thread (t, l) of the first kRT * 64 sums lane l's entries of tile r0 + t in the order of the waves:
            // D[4 * (l / 16) + e][l % 16], rows of W by rows of X
            if (tid < kRT * 64) {
                const int t = r0 + (tid >> 6), l = tid & 63;
                const int tile = tile0 + t;
                float4_t sum = partial[((t - r0) * kStreamWaves) * 64 + l];
#pragma unroll
                for (int ww = 1; ww < kStreamWaves; ww++) sum += partial[((t - r0) * kStreamWaves + ww) * 64 + l];
                const int m = l & 15, n = tile * kTile + 4 * (l >> 4);
                if (t < T && tile < n_tiles && m < M) {
                    if (bias) {
                        const half4_t b = *reinterpret_cast<const half4_t *>(bias + n);
                        sum += float4_t{(float)b[0], (float)b[1], (float)b[2], (float)b[3]};
                    }
                    const half4_t h = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
                    *reinterpret_cast<half4_t *>(y + (int64_t)(slab_row + m) * N + n) = h;
                }
            }
        }
        if (g + 1 < g_end) __syncthreads();  // the sums are read before the next group writes its own
    }
}

// tiles per group: as many as give every compute unit one group, at most kMaxTiles, and - with several codebooks - a
// divisor of the tiles of a codebook, so that a group reads one table; a wave keeps one code register per piece and
// tile, kMaxCodeRegs at most
constexpr int kMaxCodeRegs = 28;
int stream_pieces_per_wave(const ProblemB &p) { return (int)((p.K / kPieceK + kStreamWaves - 1) / kStreamWaves); }
int stream_tiles_per_group(const ProblemB &p)
{
    const int n_tiles = p.N / kTile, cus = device_cu_count();
    const int pieces = stream_pieces_per_wave(p);
    const int unrolled = pieces <= 4 ? 4 : (pieces <= 8 ? 8 : 14);  // (the kernels are built for these piece counts)
    const int most = min(kMaxTiles, max(1, kMaxCodeRegs / unrolled));
    const int rounds = (n_tiles + most * cus - 1) / (most * cus);
    int t = (n_tiles + cus * rounds - 1) / (cus * rounds);
    if (t < 1) t = 1;
    if (p.n_codebooks > 1) {
        const int per_cb = p.rows_per_cb / kTile;
        while (per_cb % t != 0) t--;
    }
    return t;
}

}  // namespace

// 8-vectors, 8-bit codes, at most 256 entries, K in whole pieces of 128 and at most 14 pieces per wave (K <= 28672), N
// and the rows of a codebook in whole tiles
bool decode_stream_supports(const ProblemB &p)
{
    if (p.vec != 8 || p.code_bits != 8 || p.entries > 256 || p.entries < 1 || p.packed || p.gated) return false;
    if (p.M < 1 || p.K < kPieceK || p.K % kPieceK != 0 || p.N < kTile || p.N % kTile != 0 || p.rows_per_cb % kTile != 0) return false;
    if (stream_pieces_per_wave(p) > 14) return false;
    return (p.M + kTile - 1) / kTile <= 65535;
}

// Where it was measured ahead of the batched kernel's chunks (cold, 256 units, batched -> this), always with at most
// one group of tiles per unit.  9 to 16 rows of X from K = 8192 on, one to seven tiles per group: M = 16, K = 14336 /
// N = 4096 17.3 -> 13.1 us, 28672 / 8192 37.2 -> 28.3, 16384 / 8192 22.8 -> 18.0, 8192 / 8192 13.3 -> 11.8, 8192 / 12288
// 15.9 -> 13.7, 8192 / 28672 25.8 -> 23.9; M = 12: 1.02 to 1.24x on the same shapes.  Eight rows and fewer from
// K = 14336 on with one or two tiles per group: M = 4, 14336 / 4096 13.0 -> 10.9, 14336 / 8192 15.7 -> 14.8, 28672 /
// 8192 25.6 -> 23.6 (three tiles per group: 0.97 - 0.99x; K = 8192 and 12288: 0.84 - 1.0x).  More groups per unit and
// taller X (one workgroup per 16-row slab, the codes read again by each) stay with the batched kernel: 0.5 - 0.9x.
bool decode_stream_preferred(const ProblemB &p)
{
    const Tuning &tn = tuning();
    if (!decode_stream_supports(p) || (double)p.K < (p.M <= 8 ? tn.decode_stream_min_k_few_rows : tn.decode_stream_min_k)) return false;
    if ((double)p.M < tn.decode_stream_min_m || (double)p.M > tn.decode_stream_max_m) return false;
    const int t = stream_tiles_per_group(p);
    if (p.M <= 8 && t > 2) return false;  // (few rows of X on three tiles and more per group: 1 to 15 % behind)
    const int n_groups = (p.N / kTile + t - 1) / t;
    return (double)n_groups <= tn.decode_stream_max_groups_per_unit * device_cu_count();
}

hipError_t launch_decode_stream(const ProblemB &p, hipStream_t s)
{
    if (!decode_stream_supports(p)) return hipErrorInvalidValue;
    const int n_tiles = p.N / kTile;
    const int t = stream_tiles_per_group(p);
    const int n_groups = (n_tiles + t - 1) / t;
    const int wgs = min(n_groups, device_cu_count());
    const dim3 grid(wgs, (p.M + kTile - 1) / kTile), block(kStreamWaves * 64);
    // the replicated table from a few gathers per lane on (its fill is 64 KB of LDS stores per workgroup and group)
    const int pieces = stream_pieces_per_wave(p);
    const bool repl = (double)(pieces * t * kPieceSteps) >= tuning().decode_stream_replicated_min_gathers;
    auto launch = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, block, 0, s, p.x, static_cast<const uint8_t *>(p.codes), p.cb, p.y, p.bias, p.M, p.K, p.N,
                           p.entries, p.rows_per_cb, n_groups / wgs, n_groups % wgs, n_tiles);
        return hipGetLastError();
    };
    using std::integral_constant;
    auto pick = [&](auto t_c, auto np_c) {
        constexpr int TT = decltype(t_c)::value, NPP = decltype(np_c)::value;
        return repl ? launch(decode_stream_kernel<TT, NPP, true>) : launch(decode_stream_kernel<TT, NPP, false>);
    };
    // (pieces per wave in steps of 4, 8 and 14; tiles per group within what the code registers hold)
    if (pieces <= 4) {
        switch (t) {
        case 1: return pick(integral_constant<int, 1>{}, integral_constant<int, 4>{});
        case 2: return pick(integral_constant<int, 2>{}, integral_constant<int, 4>{});
        case 3: return pick(integral_constant<int, 3>{}, integral_constant<int, 4>{});
        case 4: return pick(integral_constant<int, 4>{}, integral_constant<int, 4>{});
        case 5: return pick(integral_constant<int, 5>{}, integral_constant<int, 4>{});
        case 6: return pick(integral_constant<int, 6>{}, integral_constant<int, 4>{});
        default: return pick(integral_constant<int, 7>{}, integral_constant<int, 4>{});
        }
    }
    if (pieces <= 8) {
        switch (t) {
        case 1: return pick(integral_constant<int, 1>{}, integral_constant<int, 8>{});
        case 2: return pick(integral_constant<int, 2>{}, integral_constant<int, 8>{});
        default: return pick(integral_constant<int, 3>{}, integral_constant<int, 8>{});
        }
    }
    return t == 1 ? pick(integral_constant<int, 1>{}, integral_constant<int, 14>{})
                  : pick(integral_constant<int, 2>{}, integral_constant<int, 14>{});
}

}  // namespace vq
