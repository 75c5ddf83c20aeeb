// Decode path (at most 64 rows of X, 16 per launch): Y[M,N] = X[M,K] . W^T with W given as
// codes + codebook.  This file holds the batched kernel, which takes the common shapes (one
// codebook, K a multiple of 256 up to 4096, N a multiple of 16), and the dispatch; every other
// shape goes to the general kernel of vq_decode_general.hip.
//
// The path is bound by the HBM stream of the code matrix (N*K/vec code bytes), so the design
// goal is one pass over the codes with every other operand resident on the CU:
//
//   * A workgroup owns tiles of 16 output columns (16 rows of W).  Wave w owns K slice w (256 k)
//     and keeps the matching slice of X in registers, already in MFMA operand order, for the
//     whole kernel; K = 4096 makes 16 waves, four per SIMD at 128 registers each.
//   * The codebook (entries*vec*2 bytes) is resident in the LDS.  A lane streams the codes of
//     one W row, gathers the codewords and uses them *directly* as the 8-half A operand of
//     v_mfma_f32_16x16x32_f16: with vec = 8 one ds_read_b128 is one operand.  The order in which
//     a lane walks K is irrelevant to a dot product, so it is chosen so that each lane's codes
//     are contiguous in memory; X is loaded in the same order.
//   * Per tile a wave issues 8 MFMAs (its K slice); the partial 16x16 fp32 results of the waves
//     are summed through the LDS and one wave converts and stores them.
//
// M < 16 pads the X operand with zeros (the matrix core is idle anyway: the kernel is
// bandwidth bound by a wide margin); fp32 accumulation throughout, one rounding to fp16.
#include "vq_common.h"

#include <type_traits>

namespace vq {

namespace {

constexpr int kTileN = 16;
constexpr int kSliceK = 256;     // K owned by one wave
constexpr int kSteps = 8;        // MFMA steps (32 k each) per slice
constexpr int kMaxWaves = 16;    // 1024 threads, 128 registers per lane
constexpr int kGeneralMaxM = 64;    // the general kernel: one launch per 16-row slab of X up to this height
constexpr int kBatchedMaxM = 4096;  // the batched kernel: the slabs are a grid dimension
constexpr int kStageK = 512;     // X is staged in pieces of 512 k of one row (1 KB, one wave instruction)
constexpr int kStagePitch = kStageK * 2 + 16;  // LDS bytes per staged piece; the pad spreads rows over the banks

template <int VEC, typename CodeT>
struct DecodeCfg {
    // bytes of codes a lane loads at a time: 16, or 8 where 16 would span more than the slice
    static constexpr int LB = 16 / (int)sizeof(CodeT) * VEC * 4 > kSliceK ? 8 : 16;
    static constexpr int CPL = LB / (int)sizeof(CodeT);  // codes in one lane load
    static constexpr int CPO = 8 / VEC;                  // codes per 8-half MFMA operand
    static constexpr int SPL = CPL / CPO;                // MFMA steps fed by one lane load
    static constexpr int K_LANE = CPL * VEC;             // k covered by one lane load
    static constexpr int K_WAVE = 4 * K_LANE;            // k covered by one wave load (4 k-groups)
    static constexpr int LPT = kSliceK / K_WAVE;         // lane loads per slice
    static constexpr int WPL = LB / 4;                   // 32-bit words per lane load
    // tiles a wave works through between two cross-wave reductions
    static constexpr int TB = LPT * WPL <= 2 ? 4 : (LPT <= 2 ? 2 : 1);
    static_assert(CPO >= 1 && SPL >= 1 && LPT >= 1 && LPT * SPL == kSteps, "unsupported code layout");
};

// The codes one lane holds for one slice: LPT loads of WPL words.
//
// The loads are inline assembly that the compiler does not wait for (see the gathers below for
// the technique): its own bookkeeping drains every load in flight once a store is pending too,
// because the counter cannot tell loads from stores, and the tile loop would pay a full memory
// latency per tile.  Loads complete in order among themselves, so the oldest unit in flight has
// landed once at most `younger loads` operations are outstanding, whatever stores are pending.
template <int VEC, typename CodeT>
struct LaneCodes {
    typedef DecodeCfg<VEC, CodeT> C;
    typedef uint32_t words_t __attribute__((ext_vector_type(C::WPL)));
    words_t w[C::LPT];

    // Load t of the slice, from a wave-uniform base plus a 32-bit lane offset and an immediate: the address
    // of the next tile costs the scalar unit two additions and the vector unit nothing.
    template <int IMM>
    __device__ __forceinline__ void load_async_s(int t, uint32_t voff, const void *sbase)
    {
        if constexpr (C::WPL == 4)
            asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(w[t]) : "v"(voff), "s"(sbase), "n"(IMM) : "memory");
        else
            asm volatile("global_load_dwordx2 %0, %1, %2 offset:%3" : "=v"(w[t]) : "v"(voff), "s"(sbase), "n"(IMM) : "memory");
    }
    __device__ __forceinline__ void pin()
    {
#pragma unroll
        for (int t = 0; t < C::LPT; t++) asm volatile("" : "+v"(w[t]));
    }
};

// ---- hand-issued LDS gathers ------------------------------------------------------------
// Left to the compiler, only two gathers are in flight ahead of the MFMAs that use them and
// every step waits for the LDS latency.  The gathers are therefore issued as inline assembly,
// which the compiler neither reorders nor waits for; the code below waits for them itself
// (lgkmcnt counts LDS instructions, which complete in order) and ties each wait to the
// registers with an empty asm (`pin`) so that no use can be moved above it.  A gathered
// operand is consumed in the straight-line code that issued it: nothing in flight is ever
// live across a branch, where the compiler might copy or spill a register still being written.
__device__ __forceinline__ void lds_read_async(uint4_t &dst, uint32_t addr)
{
    asm volatile("ds_read_b128 %0, %1" : "=v"(dst) : "v"(addr) : "memory");
}
__device__ __forceinline__ void lds_read_async(uint2_t &dst, uint32_t addr)
{
    asm volatile("ds_read_b64 %0, %1" : "=v"(dst) : "v"(addr) : "memory");
}
__device__ __forceinline__ void lds_read_async(uint32_t &dst, uint32_t addr)
{
    asm volatile("ds_read_b32 %0, %1" : "=v"(dst) : "v"(addr) : "memory");
}

// s_waitcnt for the LDS counter only (gfx9 encoding: lgkmcnt = simm16[11:8], at most 15).
template <int N>
__device__ __forceinline__ void wait_lgkmcnt()
{
    static_assert(N >= 0 && N <= 15, "lgkmcnt has four bits");
    __builtin_amdgcn_s_waitcnt(0xc07f | (N << 8));
}

// The same for a count that is only constant after unrolling (values above 15 wait for 15).
__device__ __forceinline__ void wait_lgkmcnt_upto(int n)
{
    switch (n < 15 ? n : 15) {
    case 0: wait_lgkmcnt<0>(); break;
    case 1: wait_lgkmcnt<1>(); break;
    case 2: wait_lgkmcnt<2>(); break;
    case 3: wait_lgkmcnt<3>(); break;
    case 4: wait_lgkmcnt<4>(); break;
    case 5: wait_lgkmcnt<5>(); break;
    case 6: wait_lgkmcnt<6>(); break;
    case 7: wait_lgkmcnt<7>(); break;
    case 8: wait_lgkmcnt<8>(); break;
    case 9: wait_lgkmcnt<9>(); break;
    case 10: wait_lgkmcnt<10>(); break;
    case 11: wait_lgkmcnt<11>(); break;
    case 12: wait_lgkmcnt<12>(); break;
    case 13: wait_lgkmcnt<13>(); break;
    case 14: wait_lgkmcnt<14>(); break;
    default: wait_lgkmcnt<15>(); break;
    }
}

// s_waitcnt vmcnt(n) for a count that is only known at run time (wave-uniform, at most 8; more waits for 8)
__device__ __forceinline__ void wait_vmcnt_upto(int n);

// Returns v through an empty asm: the compiler cannot tell that it is loop invariant, so nothing
// derived from it is computed ahead of the tile loop and kept in registers through it.
__device__ __forceinline__ int opaque(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// One 8-half MFMA operand as the pieces it is gathered in: one codeword per piece.
template <int VEC> struct OperandPiece;
template <> struct OperandPiece<8> { typedef uint4_t type; };
template <> struct OperandPiece<4> { typedef uint2_t type; };
template <> struct OperandPiece<2> { typedef uint32_t type; };

template <int VEC>
struct Operand {
    static constexpr int kPieces = 8 / VEC;
    typename OperandPiece<VEC>::type p[kPieces];

    __device__ __forceinline__ void pin()
    {
#pragma unroll
        for (int i = 0; i < kPieces; i++) asm volatile("" : "+v"(p[i]));
    }
    __device__ __forceinline__ half8_t value() const
    {
        uint4_t v;
        if constexpr (VEC == 8) {
            v = p[0];
        } else if constexpr (VEC == 4) {
            v = uint4_t{p[0][0], p[0][1], p[1][0], p[1][1]};
        } else {
            v = uint4_t{p[0], p[1], p[2], p[3]};
        }
        return as_half8(v);
    }
};

// LDS byte address of codeword number c of a lane's 16 bytes of codes.
//   plain table:      code * entry_bytes (the table starts at LDS address 0)
//   replicated table: code * 256 + base, base < 256 being the lane's copy: one byte permute
//                     puts the code into byte 1 and the base into byte 0 of the address.
template <int VEC, typename CodeT, bool REPL>
__device__ __forceinline__ uint32_t codeword_addr(const LaneCodes<VEC, CodeT> &cw, int c, uint32_t base)
{
    typedef DecodeCfg<VEC, CodeT> C;
    constexpr bool u8 = sizeof(CodeT) == 1;
    const int t = c / C::CPL, ci = c % C::CPL;  // lane load, code within it
    const uint32_t word = u8 ? cw.w[t][ci >> 2] : cw.w[t][ci >> 1];
    const int byte = u8 ? (ci & 3) : 2 * (ci & 1);
    if constexpr (REPL) {
        // selector bytes: 0 = byte 0 of `base`, 4 + b = byte b of `word`, 0x0c = zero
        return __builtin_amdgcn_perm(word, base, 0x0c0c0000u | ((4u + byte) << 8));
    } else {
        const uint32_t code = u8 ? ((word >> (8 * byte)) & 0xffu) : ((word >> (8 * byte)) & 0xffffu);
        return code * (uint32_t)(VEC * 2);
    }
}

// Issue the gathers of the operand of MFMA step s: codewords s*CPO .. s*CPO + CPO-1 of the slice.
template <int VEC, typename CodeT, bool REPL>
__device__ __forceinline__ void gather_issue(Operand<VEC> &o, const LaneCodes<VEC, CodeT> &cw, int s, uint32_t base)
{
    typedef DecodeCfg<VEC, CodeT> C;
#pragma unroll
    for (int i = 0; i < Operand<VEC>::kPieces; i++)
        lds_read_async(o.p[i], codeword_addr<VEC, CodeT, REPL>(cw, s * C::CPO + i, base));
}

// s_waitcnt for the vector-memory counter only (gfx9 encoding: vmcnt = simm16[15:14]:[3:0]).
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
    asm volatile("" ::: "memory");  // keep the compiler from moving LDS reads above the wait
}

__device__ __forceinline__ void wait_vmcnt_upto(int n)
{
    switch (n < 8 ? n : 8) {
    case 0: wait_vmcnt<0>(); break;
    case 1: wait_vmcnt<1>(); break;
    case 2: wait_vmcnt<2>(); break;
    case 3: wait_vmcnt<3>(); break;
    case 4: wait_vmcnt<4>(); break;
    case 5: wait_vmcnt<5>(); break;
    case 6: wait_vmcnt<6>(); break;
    case 7: wait_vmcnt<7>(); break;
    default: wait_vmcnt<8>(); break;
    }
}

// ---- batched kernel -----------------------------------------------------------------------
// The common case (one codebook, K a multiple of 256 and at most 4096, N a multiple of 16) gets
// a loop that is lean in instructions: a CU issues one vector and one scalar instruction per
// cycle in total, whatever the number of waves, and a loop that spends a hundred instructions
// per wave and tile on control flow, addresses and the reduction is bound by exactly that.
//   * A wave works through TB consecutive tiles (its K slice of each) before the waves meet, so
//     barriers, waits and loop control are paid once per TB tiles (TB = 1 for workgroups with
//     fewer tiles than a full batch).
//   * Code loads take a scalar base per tile and one lane offset computed before the loop.
//   * The MFMA chain of a tile starts from a zero constant: no accumulator is cleared or summed.
//   * The partial results go to the LDS packed as [slot][wave], slot = (tile, k-group, X row)
//     over the rows of X that exist only; a reducing wave takes 64 slots per pass, every lane
//     summing the 16-byte entries of its slot, so a pass covers 16/M tiles.
// X taller than 16 rows is served by the second grid dimension: one 16-row slab per index.
// `recip_tail` = ceil(65536 / rows of the last slab), for the division of a slot number by M.
constexpr int kSlotPitch = 16 * kMaxWaves + 16;  // LDS bytes per slot; the pad spreads the slots over the banks
// what the X staging area lies over (it is only live while X is being loaded)
constexpr int kStageOverTable = 1, kStageOverSlots = 2;

__device__ __forceinline__ const half_t *bias_of() { return nullptr; }
__device__ __forceinline__ const half_t *bias_of(const half_t *b) { return b; }

//
// GATED: the epilogue of a gate/up pair.  The rows of W are gate and up rows interleaved in groups of 16, so an
// even tile holds gate rows and the tile behind it the up rows of the same 16 outputs: workgroups are dealt whole
// pairs of tiles (tiles_q and tiles_r then count pairs), TB is even, and a reducing lane sums the gate slot and the
// matching up slot and stores silu(gate) * up into Y [m_total, N/2].
template <int VEC, typename CodeT, bool REPL, int TB, bool PACKED, bool GATED, typename... Bias>
__global__ __launch_bounds__(1024) void decode_batched_kernel(const half_t *__restrict__ x,
                                                               const CodeT *__restrict__ codes,
                                                               const half_t *__restrict__ cb,
                                                               half_t *__restrict__ y, int m_total, int K, int N,
                                                               int entries, int n_books, int wgs_per_cb,
                                                               int books_per_wg, int tiles_per_cb, int tiles_q,
                                                               int tiles_r, int n_chunks, int red_off,
                                                               int stage_off, int stage_over, int acc_off,
                                                               int recip_tail, Bias... bias_arg)
{
    typedef DecodeCfg<VEC, CodeT> C;
    typedef LaneCodes<VEC, CodeT> Codes;
    // The bias pointer is a kernel argument only in the instantiation that adds one, so that a
    // launch without bias fetches and tests nothing for it.
    constexpr bool kHasBias = sizeof...(Bias) > 0;
    const half_t *bias = bias_of(bias_arg...);
    // All kernel arguments are fetched at once: left to first use, each pointer costs the
    // prologue a scalar-load round trip of its own.
    asm volatile("" ::"s"(x), "s"(codes), "s"(cb), "s"(y), "s"(m_total), "s"(K), "s"(N), "s"(entries),
                 "s"(n_books), "s"(wgs_per_cb), "s"(books_per_wg), "s"(tiles_per_cb), "s"(tiles_q), "s"(tiles_r),
                 "s"(n_chunks), "s"(red_off), "s"(stage_off), "s"(stage_over), "s"(acc_off), "s"(recip_tail));
    // blockIdx.y picks the 16-row slab of X (and of Y) this workgroup multiplies.
    const int slab_row = blockIdx.y * kTileN;
    const int M = min(kTileN, m_total - slab_row);
    const int recip_m = M == kTileN ? 65536 / kTileN : recip_tail;
    x += (int64_t)slab_row * K;
    static_assert(!GATED || TB % 2 == 0, "gate and up tiles come in pairs");
    constexpr int kDeal = GATED ? 2 : 1;  // tiles per unit that is dealt to the workgroups
    const int ldy = GATED ? N / 2 : N;
    y += (int64_t)slab_row * ldy;
    constexpr int kPieces = Operand<VEC>::kPieces;
    constexpr int kEntryBytes = VEC * 2;
    extern __shared__ __align__(16) uint8_t smem[];
    // K goes in n_chunks chunks of (at most) n_waves slices of 256 k: wave w owns slice w of the
    // current chunk; the last chunk may leave the upper waves without one.
    const int n_waves = blockDim.x >> 6;
    const int total_slices = K / kSliceK;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int r16 = lane & 15;  // W row within the tile (A operand) / X row m (B operand)
    const int kq = lane >> 4;   // k-group of the lane, 0..3
    const int J = K / VEC;
    const int cb_slots = REPL ? entries * 16 : entries * kEntryBytes / 16;  // 16-byte slots of the LDS table
    uint4_t *cb_lds = reinterpret_cast<uint4_t *>(smem);
    const uint32_t gather_base = REPL ? (lane % (256 / kEntryBytes)) * kEntryBytes : 0;
    const uint32_t red_base = red_off;

    // blockIdx.x picks the codebooks.  Either wgs_per_cb workgroups share the tiles_per_cb tiles
    // of one codebook (a contiguous range each: tiles_q, one more for the first tiles_r; quotient
    // and remainder computed by the host), or one workgroup takes books_per_wg whole codebooks in
    // turn, keeping its X and replacing the table in the LDS between them.
    const int book_begin = wgs_per_cb > 1 ? (int)blockIdx.x / wgs_per_cb : (int)blockIdx.x * books_per_wg;
    const int book_end = min(n_books, book_begin + books_per_wg);
    const int wg = wgs_per_cb > 1 ? (int)blockIdx.x - book_begin * wgs_per_cb : 0;
    int book = book_begin;
    int tile_begin = book * tiles_per_cb + kDeal * (wg * tiles_q + min(wg, tiles_r));
    int tile_end = tile_begin + kDeal * (tiles_q + (wg < tiles_r ? 1 : 0));
    if (book >= book_end || tile_begin >= tile_end) return;
    cb += (int64_t)book * entries * VEC;
    int n_units = (tile_end - tile_begin + TB - 1) / TB;
    int chunk = 0;
    int n_act = min(n_waves, total_slices);  // waves with a slice in the current chunk
    bool active = w < n_act;

    // Codes: lane offset inside a tile and chunk, scalar base per tile and chunk.  The last unit
    // may hold fewer than TB tiles.
    // Plain layout [N, K/VEC]: a lane load is LB bytes of row r16, the four k-groups of a wave load
    // lie 4*LB bytes apart in each of 16 rows.  Packed layout (pack_codes_kernel below): the 64 lane
    // loads of a wave load are contiguous, [tile][slice][load][lane], so that a wave instruction
    // reads 64*LB consecutive bytes instead of 16 pieces of 4*LB.
    constexpr int kLoadPitch = PACKED ? 64 * C::LB : 4 * C::LB;  // bytes between the loads of a slice
    const uint32_t voff = PACKED ? (uint32_t)((w * C::LPT * 64 + lane) * C::LB)
                                 : (uint32_t)((r16 * J + (w * kSliceK + kq * C::K_LANE) / VEC) * (int)sizeof(CodeT));
    const int64_t tile_bytes = (int64_t)kTileN * J * (int)sizeof(CodeT);
    const int chunk_bytes = n_waves * kSliceK / VEC * (int)sizeof(CodeT) * (PACKED ? kTileN : 1);
    auto load_unit = [&](int q, Codes (&cw)[TB]) {
#pragma unroll
        for (int j = 0; j < TB; j++) {
            const int tile = tile_begin + q * TB + j;
            if (tile >= tile_end) break;
            const uint8_t *sbase = reinterpret_cast<const uint8_t *>(codes) + tile * tile_bytes + chunk * chunk_bytes;
            if constexpr (C::LPT >= 1) cw[j].template load_async_s<0>(0, voff, sbase);
            if constexpr (C::LPT >= 2) cw[j].template load_async_s<kLoadPitch>(1, voff, sbase);
            if constexpr (C::LPT >= 3) cw[j].template load_async_s<2 * kLoadPitch>(2, voff, sbase);
            if constexpr (C::LPT >= 4) cw[j].template load_async_s<3 * kLoadPitch>(3, voff, sbase);
            static_assert(C::LPT <= 4, "at most four lane loads per slice");
        }
    };
    // Two units of codes are in flight: ring slot q % 2 holds unit q.
    Codes cwq[2][TB];
    // (returns the number of loads it issued)
    auto load_first_units = [&]() {
        if (!active) return 0;
        load_unit(0, cwq[0]);
        if (n_units > 1) load_unit(1, cwq[1]);
        return min(2 * TB, tile_end - tile_begin) * C::LPT;
    };
    // A workgroup with a single tile has nothing to do until its codes are there: they are requested first.  With
    // more tiles the first codes go out behind the table's and X's loads: loads complete in the order they were
    // issued, and the codes come from HBM - requested first they hold back X and the table (out of the L2), which
    // the waves could pick up and publish while the codes are still on their way (cold, first -> behind: one tile per
    // workgroup 6.55 -> 7.15 us at M = 16 on 4096 x 4096, three tiles 12.1 -> 11.95 us on 11008 rows, seven 12.5 -> 12.1).
    const bool codes_first = tile_end - tile_begin < 2;
    int first_code_loads = 0;
    if (codes_first) load_first_units();

    // Codebook: global -> registers -> LDS, fetched now, stored once the LDS is free.
    constexpr int kCbRegs = 4;
    const bool cb_in_regs = cb_slots <= kCbRegs * (int)blockDim.x;
    uint4_t cb_regs[kCbRegs];
    auto read_slot = [&](int i) {
        if constexpr (REPL) {
            typedef uint32_t entry_t __attribute__((ext_vector_type(kEntryBytes / 4)));
            const entry_t e = reinterpret_cast<const entry_t *>(cb)[i >> 4];
            uint4_t v;
#pragma unroll
            for (int d = 0; d < 4; d++) v[d] = e[d % (kEntryBytes / 4)];
            return v;
        } else {
            return reinterpret_cast<const uint4_t *>(cb)[i];
        }
    };
    auto store_codebook = [&]() {
        if (cb_in_regs) {
#pragma unroll
            for (int j = 0; j < kCbRegs; j++) {
                const int i = threadIdx.x + j * blockDim.x;
                if (i < cb_slots) cb_lds[i] = cb_regs[j];
            }
        } else {
            for (int i = threadIdx.x; i < cb_slots; i += blockDim.x) cb_lds[i] = read_slot(i);
        }
    };
    if (cb_in_regs) {
        // (whole waves past the end of the table issue no load: every vector memory instruction
        // of the prologue queues behind the others of the CU)
#pragma unroll
        for (int j = 0; j < kCbRegs; j++) {
            const int i = threadIdx.x + j * blockDim.x;
            if ((i & ~63) < cb_slots) cb_regs[j] = read_slot(i < cb_slots ? i : 0);
        }
    }

    // X slice of the wave -> registers, in MFMA operand order; rows past M are zero.  Through the
    // LDS in pieces of 512 k of one row (1 KB, contiguous): a few whole-wave copies per workgroup
    // instead of eight mostly idle loads per wave.  Every vector memory instruction of the
    // prologue queues behind the others of the CU, so their number is what the first tile waits
    // for.  Piece (row i, block b of the chunk) sits at (b*M + i) * kStagePitch.
    half8_t xr[kSteps];
    auto stage_x = [&]() {
        const int kc0 = chunk * n_waves * kSliceK;
        const int n_blocks = (n_act * kSliceK + kStageK - 1) / kStageK;
        const int ln = opaque(lane);
        for (int pc = w; pc < n_blocks * M; pc += n_waves) {
            const int b = pc / M, i = pc - b * M;
            const int kl = kc0 + b * kStageK + 8 * ln;
            load_to_lds_16(stage_off + pc * kStagePitch, (uint32_t)((i * K + (kl < K ? kl : 0)) * 2), x);
        }
    };
    auto pick_x = [&]() {
        const int k0 = w * kSliceK;  // inside the chunk
        const int ln = opaque(lane);
        const int row = ln & 15, kg = ln >> 4;
        const uint32_t win = stage_off + ((k0 / kStageK) * M + row) * kStagePitch + (k0 % kStageK) * 2;
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            const int k = (s / C::SPL) * C::K_WAVE + kg * C::K_LANE + (s % C::SPL) * 8;
            uint4_t v = {0u, 0u, 0u, 0u};
            if (active && row < M) v = *reinterpret_cast<const uint4_t *>(smem + win + k * 2);
            xr[s] = as_half8(v);
        }
    };
    stage_x();
    if (!codes_first) first_code_loads = load_first_units();
    if (!(stage_over & kStageOverTable)) store_codebook();
    wait_vmcnt_upto(first_code_loads);  // X staged (and everything older); the codes may still be in flight
    __syncthreads();  // pieces staged by the other waves
    pick_x();
    if (stage_over) {
        __syncthreads();  // every wave has picked up its X before the staging area is written again
        if (stage_over & kStageOverTable) {
            store_codebook();
            __syncthreads();
        }
    }

    // Partial results: slot (j, kq, m) = (j*4 + kq)*M + m for tile j of the unit; this lane writes
    // entry w of the slots (j, kq, r16).
    const uint32_t wr_addr = red_base + (uint32_t)(kq * M + r16) * kSlotPitch + w * 16;
    const uint32_t wr_stride = (uint32_t)(4 * M) * kSlotPitch;
    const int n_slots = TB * 4 * M;
    const int n_out_slots = n_slots / kDeal;  // what the reducing lanes are dealt: slots, or pairs of a gate and an up slot
    const int n_passes = (n_out_slots + 63) >> 6;
    int turn = 0;  // the wave that takes the next reduction pass

    auto process_unit = [&](int q, Codes (&cur)[TB]) {
        const int nt = min(TB, tile_end - (tile_begin + q * TB));  // tiles of this unit
        float4_t acc[TB];
        const float4_t c0 = {0.f, 0.f, 0.f, 0.f};
        if (active) {
            // This unit's codes have landed when only the loads of the next unit are out (a short
            // last unit has fewer of them: then everything is awaited).
            if (tile_begin + (q + 2) * TB <= tile_end) wait_vmcnt<TB * C::LPT>();
            else wait_vmcnt<0>();
#pragma unroll
            for (int j = 0; j < TB; j++) cur[j].pin();

            if (nt == TB) {
                // One branch-free stream of TB*8 MFMA steps; ops[] holds the gathered operands of a
                // tile, and each is replaced by the next tile's as soon as it has been multiplied.
                Operand<VEC> ops[kSteps];
#pragma unroll
                for (int s = 0; s < kSteps; s++) gather_issue<VEC, CodeT, REPL>(ops[s], cur[0], s, gather_base);
#pragma unroll
                for (int i = 0; i < TB * kSteps; i++) {
                    const int j = i / kSteps, s = i % kSteps;
                    Operand<VEC> &o = ops[s];
                    const int left = TB * kSteps - 1 - i;  // steps after this one
                    wait_lgkmcnt_upto((left < kSteps - 1 ? left : kSteps - 1) * kPieces);  // younger gathers in flight
                    o.pin();
                    acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(o.value(), xr[s], s == 0 ? c0 : acc[j], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    const int t = i + kSteps;
                    if (t < TB * kSteps) gather_issue<VEC, CodeT, REPL>(o, cur[t / kSteps], t % kSteps, gather_base);
                    // All gather addresses of the unit are computed: its ring slot takes the unit after next.
                    if (t == TB * kSteps - 1 || (TB == 1 && i == 0))
                        if (q + 2 < n_units) load_unit(q + 2, cur);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                // Short last unit: tile by tile, nothing in flight from one tile to the next.
#pragma unroll
                for (int j = 0; j < TB; j++) {
                    acc[j] = c0;
                    if (j < nt) {
                        Operand<VEC> ops[kSteps];
#pragma unroll
                        for (int s = 0; s < kSteps; s++) gather_issue<VEC, CodeT, REPL>(ops[s], cur[j], s, gather_base);
#pragma unroll
                        for (int s = 0; s < kSteps; s++) {
                            wait_lgkmcnt_upto((kSteps - 1 - s) * kPieces);
                            ops[s].pin();
                            acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ops[s].value(), xr[s], acc[j], 0, 0, 0);
                        }
                    }
                }
            }
        }

        if (q > 0) __syncthreads();  // the reducers of the previous unit are done with the slots
        if (active && r16 < M) {
#pragma unroll
            for (int j = 0; j < TB; j++)
                if (j < nt) *reinterpret_cast<float4_t *>(smem + wr_addr + j * wr_stride) = acc[j];
        }
        // A pass of the reduction: 64 slots, one per lane.  Where the slot goes is worked out
        // first (`locate`), the sum and the store follow (`finish`).
        struct Target { uint32_t src, carry; half_t *dst; int n; bool live; };  // LDS offsets, output address, first W row
        auto locate = [&](int pass) {
            const int out = pass * 64 + opaque(lane);
            const int jq = (out * recip_m) >> 16;  // out / M = j*4 + kq (GATED: j counts pairs of tiles)
            const int m = out - jq * M;
            const int j = kDeal * (jq >> 2);       // tile of the unit (GATED: the gate tile)
            const int tile = tile_begin + q * TB + j;
            const int slot = GATED ? (j * 4 + (jq & 3)) * M + m : out;
            Target t;
            t.src = red_base + slot * kSlotPitch;
            // with several chunks the sums are carried from chunk to chunk in the LDS, one entry per slot of the range
            t.carry = (uint32_t)acc_off + (uint32_t)(q * n_slots + slot) * 16u;
            // D[i][j] of the tile: the slot holds rows i = 4*kq .. 4*kq+3 of column j = m.
            t.n = tile * kTileN + 4 * (jq & 3);
            t.dst = GATED ? y + (int64_t)m * ldy + (tile >> 1) * kTileN + 4 * (jq & 3) : y + (int64_t)m * N + t.n;
            t.live = pass < n_passes && out < n_out_slots && tile < tile_end;
            return t;
        };
        // the sum over the waves of one slot, carried across the chunks of K; `last` = this was the last chunk
        auto sum_slot = [&](uint32_t src_off, uint32_t carry_off, int n_bias, bool &last) {
            const float4_t *src = reinterpret_cast<const float4_t *>(smem + src_off);
            float4_t sum;
            if (n_act == kMaxWaves) {
                // four interleaved chains, to keep the run of dependent additions short
                float4_t c[4];
#pragma unroll
                for (int i = 0; i < 4; i++) c[i] = src[i];
#pragma unroll
                for (int i = 4; i < kMaxWaves; i++) c[i & 3] += src[i];
                sum = (c[0] + c[1]) + (c[2] + c[3]);
            } else {
                sum = src[0];
                for (int i = 1; i < n_act; i++) sum += src[i];
            }
            float4_t *carry = reinterpret_cast<float4_t *>(smem + carry_off);
            if (chunk > 0) sum += *carry;
            last = chunk >= n_chunks - 1;
            if (!last) {
                *carry = sum;
            } else if constexpr (kHasBias) {
                const half4_t b = *reinterpret_cast<const half4_t *>(bias + n_bias);
                sum += float4_t{(float)b[0], (float)b[1], (float)b[2], (float)b[3]};
            }
            return sum;
        };
        auto finish = [&](const Target &t) {
            if (!t.live) return;
            bool last;
            float4_t sum = sum_slot(t.src, t.carry, t.n, last);
            if constexpr (GATED) {
                // the up slot of the same outputs: one tile (4*M slots) further on
                const float4_t up = sum_slot(t.src + (uint32_t)(4 * M) * kSlotPitch, t.carry + (uint32_t)(4 * M) * 16u, t.n + kTileN, last);
#pragma unroll
                for (int e = 0; e < 4; e++) sum[e] = silu_f32(sum[e]) * up[e];
            }
            if (last) {
                half4_t h = {(half_t)sum[0], (half_t)sum[1], (half_t)sum[2], (half_t)sum[3]};
                *reinterpret_cast<half4_t *>(t.dst) = h;
            }
        };
        // The waves take the passes in turn; a wave's first pass is located before the barrier,
        // so that only the sum and the store follow it.
        int pass = w - turn;
        if (pass < 0) pass += n_waves;
        const Target first = locate(pass);
        __syncthreads();
        finish(first);
        for (pass += n_waves; pass < n_passes; pass += n_waves) finish(locate(pass));
        turn += n_passes;
        while (turn >= n_waves) turn -= n_waves;
    };

    for (;;) {
        for (int q = 0; q < n_units; q += 2) {
            process_unit(q, cwq[0]);
            if (q + 1 < n_units) process_unit(q + 1, cwq[1]);
        }
        // Next chunk of K for the same tiles, or the next codebook (books_per_wg > 1 means whole
        // codebooks: all of its tiles).
        if (++chunk >= n_chunks) {
            chunk = 0;
            if (++book >= book_end) break;
            tile_begin = book * tiles_per_cb;
            tile_end = tile_begin + tiles_per_cb;
            n_units = (tiles_per_cb + TB - 1) / TB;
            cb += (int64_t)entries * VEC;
        }
        n_act = min(n_waves, total_slices - chunk * n_waves);
        active = w < n_act;
        // The first codes are requested before the table or X are replaced, to overlap the latencies.
        load_first_units();
        __syncthreads();  // every gather from the old table has been consumed, every slot read
        if (n_chunks > 1) stage_x();
        if (chunk == 0) {
            // (the thread index goes through an empty asm so that nothing derived from it is kept
            // in registers across the tile loop just to be reused here)
            int tid = threadIdx.x;
            asm volatile("" : "+v"(tid));
            for (int i0 = tid; i0 < cb_slots; i0 += 2 * (int)blockDim.x) {
                const int i1 = i0 + (int)blockDim.x;
                const uint4_t a = read_slot(i0);
                const uint4_t b = read_slot(i1 < cb_slots ? i1 : i0);
                cb_lds[i0] = a;
                if (i1 < cb_slots) cb_lds[i1] = b;
            }
        }
        if (n_chunks > 1) {
            wait_vmcnt<0>();
            __syncthreads();  // pieces staged by the other waves, and the new table
            pick_x();
        }
        __syncthreads();  // X picked up before the slots (which the staging area may lie over) are written
    }
}

constexpr size_t kDecodeLdsLimit = 160 * 1024;
constexpr size_t kDisjointBudget = 80 * 1024;  // keep two workgroups per CU when staging beside the codebook

// How the batched kernel is launched on a shape: the split of K, of X and of the tiles, and the
// layout of the LDS.  `ok` is false when the shape is not for this kernel.
struct BatchedPlan {
    bool ok;
    int n_waves, n_chunks;                        // waves per workgroup = slices per chunk of K
    int n_slabs, per_slab;                        // grid
    int wgs_per_cb, books_per_wg, tiles_per_cb;   // workgroups of a slab <-> codebooks
    int tiles_per_wg;                             // per codebook
    int per_cu;                                   // workgroups resident per CU, by waves
    bool repl, full;                              // replicated table; batches of TB tiles (else of one)
    int red_off, stage_off, stage_over, acc_off;  // LDS
    size_t smem;
};

// K a multiple of 256, N and the rows per codebook multiples of 16; the LDS must hold the table,
// the slots, the staged X and, when K goes in chunks, the carried sums of the workgroup's tiles.
template <int VEC, typename CodeT>
BatchedPlan plan_batched(const ProblemB &p)
{
    typedef DecodeCfg<VEC, CodeT> C;
    BatchedPlan g = {};
    if (p.K % kSliceK != 0 || p.N % kTileN != 0 || p.rows_per_cb % kTileN != 0) return g;
    // gated: whole pairs of a gate and an up tile per codebook, dealt to the workgroups as pairs, in batches of an even
    // number of tiles; the packed code layout is not read
    const int deal = p.gated ? 2 : 1;
    if (p.gated && (p.rows_per_cb % (2 * kTileN) != 0 || C::TB % 2 != 0 || p.packed)) return g;
    const int slices = p.K / kSliceK;
    g.n_chunks = (slices + kMaxWaves - 1) / kMaxWaves;
    g.n_waves = (slices + g.n_chunks - 1) / g.n_chunks;
    const int m_slab = p.M < kTileN ? p.M : kTileN;  // rows of X one workgroup multiplies
    g.tiles_per_cb = p.rows_per_cb / kTileN;
    g.per_cu = kMaxWaves / g.n_waves;
    g.n_slabs = (p.M + kTileN - 1) / kTileN;
    // As many workgroups as the device holds at once, shared among the slabs.  Within a slab a
    // workgroup reads one codebook at a time: several workgroups share the tiles of a codebook,
    // or one takes several whole codebooks in turn.
    const int resident = device_cu_count() * g.per_cu;
    int per_slab = resident / g.n_slabs;
    if (per_slab < 1) per_slab = 1;
    if (per_slab >= p.n_codebooks) {
        const int per_cb = per_slab / p.n_codebooks;
        g.wgs_per_cb = per_cb < g.tiles_per_cb / deal ? per_cb : g.tiles_per_cb / deal;
        g.books_per_wg = 1;
    } else {
        g.wgs_per_cb = 1;
        g.books_per_wg = (p.n_codebooks + per_slab - 1) / per_slab;
    }
    const size_t plain = (size_t)p.entries * VEC * 2;
    const size_t stage = (size_t)((g.n_waves * kSliceK + kStageK - 1) / kStageK) * m_slab * kStagePitch;
    const size_t slot_bytes = (size_t)4 * m_slab * kSlotPitch;  // per tile of a batch
    const size_t carry_bytes = (size_t)4 * m_slab * 16;         // per tile of the workgroup's range
    for (;;) {
        g.tiles_per_wg = deal * ((g.tiles_per_cb / deal + g.wgs_per_cb - 1) / g.wgs_per_cb);
        g.full = g.tiles_per_wg >= 2;
        const int tb = g.full ? C::TB : 1;
        const size_t slots = tb * slot_bytes;
        const int units = (g.tiles_per_wg + tb - 1) / tb;
        const size_t carry = g.n_chunks > 1 ? (size_t)units * tb * carry_bytes : 0;
        // Replicated codebook (one 256-byte bank row per entry, <= 64 KB): worth its fill time as
        // soon as the workgroup gathers from it for more than one tile, where it fits.
        for (int repl = (p.entries <= 256 && (double)g.tiles_per_wg >= tuning().decode_replicated_table_min_tiles) ? 1 : 0; repl >= 0; repl--) {
            const size_t table = repl ? (size_t)p.entries * 256 : plain;
            g.repl = repl != 0;
            g.acc_off = g.n_chunks > 1 ? (int)table : -1;
            g.red_off = (int)(table + carry);
            if (g.n_chunks == 1 && table + carry + slots + stage <= kDisjointBudget) {
                // everything side by side, and room for a second workgroup on the CU
                g.stage_off = g.red_off + (int)slots;
                g.stage_over = 0;
                g.smem = table + slots + stage;
                g.ok = true;
                return g;
            }
            if (g.n_chunks == 1) {
                // X staged over the table and the slots (both are written after X is picked up)
                g.stage_off = 0;
                g.stage_over = kStageOverTable | kStageOverSlots;
                g.smem = stage > table + slots ? stage : table + slots;
            } else {
                // X staged over the slots only: table and carried sums live across the chunks
                g.stage_off = g.red_off;
                g.stage_over = kStageOverSlots;
                g.smem = table + carry + (stage > slots ? stage : slots);
            }
            if (g.smem <= kDecodeLdsLimit) {
                g.ok = true;
                return g;
            }
        }
        // Too many carried sums: fewer tiles per workgroup (more workgroups than are resident).
        if (g.n_chunks == 1 || g.wgs_per_cb >= g.tiles_per_cb / deal) return g;
        if (g.books_per_wg > 1) g.books_per_wg = 1;  // one codebook per workgroup first
        else g.wgs_per_cb = g.wgs_per_cb * 2 < g.tiles_per_cb / deal ? g.wgs_per_cb * 2 : g.tiles_per_cb / deal;
    }
}

BatchedPlan plan_batched(const ProblemB &p)
{
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? plan_batched<8, uint8_t>(p) : plan_batched<8, uint16_t>(p);
    case 4: return u8 ? plan_batched<4, uint8_t>(p) : plan_batched<4, uint16_t>(p);
    default: return u8 ? plan_batched<2, uint8_t>(p) : plan_batched<2, uint16_t>(p);
    }
}

template <int VEC, typename CodeT, bool PACKED>
hipError_t launch_decode_batched(const ProblemB &p, hipStream_t s)
{
    typedef DecodeCfg<VEC, CodeT> C;
    BatchedPlan g = plan_batched<VEC, CodeT>(p);
    if (!g.ok) return hipErrorInvalidValue;
    g.per_slab = g.books_per_wg > 1 ? (p.n_codebooks + g.books_per_wg - 1) / g.books_per_wg : g.wgs_per_cb * p.n_codebooks;
    const int tail_rows = p.M - (g.n_slabs - 1) * kTileN;
    const int dealt = p.gated ? g.tiles_per_cb / 2 : g.tiles_per_cb;  // what the workgroups of a codebook share: tiles, or pairs
    // the same launch for the instantiation with a bias argument and the one without
    auto launch = [&](auto kern, auto... bias) {
        hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void *>(kern), g.smem);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kern, dim3(g.per_slab, g.n_slabs), dim3(g.n_waves * 64), g.smem, s, p.x,
                           static_cast<const CodeT *>(p.codes), p.cb, p.y, p.M, p.K, p.N, p.entries, p.n_codebooks,
                           g.wgs_per_cb, g.books_per_wg, g.tiles_per_cb, dealt / g.wgs_per_cb,
                           dealt % g.wgs_per_cb, g.n_chunks, g.red_off, g.stage_off, g.stage_over, g.acc_off,
                           (65536 + tail_rows - 1) / tail_rows, bias...);
        return hipGetLastError();
    };
    // a full batch of one tile is the only case with a replicated table and TB = 1
    const int tb = g.full ? C::TB : 1;
    if constexpr (!PACKED && C::TB % 2 == 0) {
        if (p.gated) {
            if (p.bias) return g.repl ? launch(decode_batched_kernel<VEC, CodeT, true, C::TB, false, true, const half_t *>, p.bias)
                                      : launch(decode_batched_kernel<VEC, CodeT, false, C::TB, false, true, const half_t *>, p.bias);
            return g.repl ? launch(decode_batched_kernel<VEC, CodeT, true, C::TB, false, true>)
                          : launch(decode_batched_kernel<VEC, CodeT, false, C::TB, false, true>);
        }
    }
    if (p.gated) return hipErrorInvalidValue;
    if (p.bias) {
        if (g.repl) return tb == 1 ? launch(decode_batched_kernel<VEC, CodeT, true, 1, PACKED, false, const half_t *>, p.bias)
                                   : launch(decode_batched_kernel<VEC, CodeT, true, C::TB, PACKED, false, const half_t *>, p.bias);
        return tb == 1 ? launch(decode_batched_kernel<VEC, CodeT, false, 1, PACKED, false, const half_t *>, p.bias)
                       : launch(decode_batched_kernel<VEC, CodeT, false, C::TB, PACKED, false, const half_t *>, p.bias);
    }
    if (g.repl) return tb == 1 ? launch(decode_batched_kernel<VEC, CodeT, true, 1, PACKED, false>)
                               : launch(decode_batched_kernel<VEC, CodeT, true, C::TB, PACKED, false>);
    return tb == 1 ? launch(decode_batched_kernel<VEC, CodeT, false, 1, PACKED, false>)
                   : launch(decode_batched_kernel<VEC, CodeT, false, C::TB, PACKED, false>);
}

// ---- packed code layout ---------------------------------------------------------------------
// The batched kernel's lane (k-group kq, row r) of the wave that owns slice s loads, for load t of
// the slice, LB bytes of row r starting at code (s*256 + t*K_WAVE + kq*K_LANE)/VEC.  The packed
// layout stores exactly these pieces in the order the lanes ask for them:
//     packed[tile][s][t][kq][r][LB bytes],   tile = n / 16, r = n % 16,
// so that a wave load is one contiguous run of 64*LB bytes.  Same size as the plain matrix; the
// permutation moves whole pieces, codes keep their values.  One thread moves one piece.
template <int LB>
__global__ __launch_bounds__(256) void pack_codes_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                        int64_t n_pieces, int row_bytes, bool inverse)
{
    typedef uint32_t piece_t __attribute__((ext_vector_type(LB / 4)));
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;  // index in the packed order
    if (i >= n_pieces) return;
    const int r = (int)(i & 15), kq = (int)((i >> 4) & 3);
    const int64_t rest = i >> 6;  // (tile * slices + s) * lpt + t
    const int per_tile = row_bytes / (4 * LB);  // slices * lpt
    const int64_t tile = rest / per_tile;
    const int st = (int)(rest - tile * per_tile);  // s * lpt + t: wave loads follow each other along the row
    const int64_t plain = ((tile * kTileN + r) * (int64_t)row_bytes + (int64_t)st * 4 * LB + kq * LB) / LB;
    const piece_t *s = reinterpret_cast<const piece_t *>(src);
    piece_t *d = reinterpret_cast<piece_t *>(dst);
    if (inverse) d[plain] = s[i];
    else d[i] = s[plain];
}

template <int VEC, typename CodeT>
hipError_t launch_pack(const void *src, void *dst, int64_t N, int64_t K, bool inverse, hipStream_t s)
{
    typedef DecodeCfg<VEC, CodeT> C;
    static_assert(C::LPT * C::K_WAVE == kSliceK, "a slice is a whole number of wave loads");
    const int row_bytes = (int)(K / VEC) * (int)sizeof(CodeT);
    const int64_t n_pieces = N * row_bytes / C::LB;
    if (n_pieces == 0) return hipSuccess;
    const unsigned blocks = (unsigned)((n_pieces + 255) / 256);
    hipLaunchKernelGGL(pack_codes_kernel<C::LB>, dim3(blocks), dim3(256), 0, s, static_cast<const uint8_t *>(src),
                       static_cast<uint8_t *>(dst), n_pieces, row_bytes, inverse);
    return hipGetLastError();
}

bool batched_supports(const ProblemB &p) { return plan_batched(p).ok; }

}  // namespace

bool decode_packed_supports(const ProblemB &p)
{
    return p.M >= 1 && p.M <= kBatchedMaxM && decode_general_supports(p) && batched_supports(p);
}

bool pack_codes_supports(int64_t N, int64_t K, int vec, int code_bits)
{
    return (vec == 2 || vec == 4 || vec == 8) && (code_bits == 8 || code_bits == 16) && K % kSliceK == 0 && N % kTileN == 0;
}

hipError_t launch_pack_codes(const void *src, void *dst, int64_t N, int64_t K, int vec, int code_bits, bool inverse,
                             hipStream_t s)
{
    if (!pack_codes_supports(N, K, vec, code_bits)) return hipErrorInvalidValue;
    const bool u8 = code_bits == 8;
    switch (vec) {
    case 8: return u8 ? launch_pack<8, uint8_t>(src, dst, N, K, inverse, s) : launch_pack<8, uint16_t>(src, dst, N, K, inverse, s);
    case 4: return u8 ? launch_pack<4, uint8_t>(src, dst, N, K, inverse, s) : launch_pack<4, uint16_t>(src, dst, N, K, inverse, s);
    default: return u8 ? launch_pack<2, uint8_t>(src, dst, N, K, inverse, s) : launch_pack<2, uint16_t>(src, dst, N, K, inverse, s);
    }
}

// the gated epilogue: both K-sliced kernels carry it (as the plain product: the general kernel in slabs up to 64 rows of X)
bool decode_gated_supports(const ProblemB &p) { return p.gated && decode_supports(p); }

bool decode_supports(const ProblemB &p)
{
    if (p.M < 1 || !decode_general_supports(p)) return false;
    return p.M <= kGeneralMaxM || (p.M <= kBatchedMaxM && batched_supports(p));
}

// Rough times (us) of the two tiled kernels on a shape both can take; the automatic choice takes
// the smaller.  Fitted to measurements on a 256-CU MI355X:
//   decode path   per workgroup a prologue (3), then per codebook and chunk of K its tiles at
//                 0.75 us per tile and 4096 k (1.25 when K goes in chunks: X is staged again per
//                 chunk), plus 5 per change of codebook or chunk; workgroups beyond those
//                 resident run in further rounds.  With K of 2048 or less two workgroups share a
//                 compute unit: prologue 8, and a tile then costs each of them 1.0 us per 2048 k;
//   prefill       the prefill kernels' own estimate for the tiles they would choose.
// microseconds the batched decode kernel is expected to take on a shape it supports (M above what the general
// kernel serves: below that the decode path is taken without a comparison)
static double batched_cost_us(const ProblemB &p)
{
    const BatchedPlan g = plan_batched(p);
    const int cus = device_cu_count();
    const int per_slab = g.books_per_wg > 1 ? (p.n_codebooks + g.books_per_wg - 1) / g.books_per_wg : g.wgs_per_cb * p.n_codebooks;
    const int rounds_d = (per_slab * g.n_slabs + cus * g.per_cu - 1) / (cus * g.per_cu);
    const bool shared = g.per_cu > 1;
    const Tuning &tn = tuning();
    const double t_tile = (g.n_chunks == 1 ? tn.decode_tile_us : tn.decode_tile_chunked_us) * g.n_waves / kMaxWaves * g.per_cu * (shared ? 1.35 : 1.0);
    const int passes = g.books_per_wg * g.n_chunks;
    return rounds_d * ((shared ? tn.decode_prologue_shared_cu_us : tn.decode_prologue_us) + passes * g.tiles_per_wg * t_tile +
                       (passes - 1) * tn.decode_pass_change_us);
}

bool decode_preferred(const ProblemB &p)
{
    if (!decode_supports(p)) return false;
    if (p.M <= kGeneralMaxM) return true;
    const double t_prefill = prefill_supports(p) ? 1.0 + prefill_cost_us(p) : 1e30;
    return batched_cost_us(p) <= t_prefill;
}

double decode_cost_us(const ProblemB &p)
{
    if (!decode_supports(p) || p.M <= kGeneralMaxM || !batched_supports(p)) return 1e30;
    return batched_cost_us(p);
}

// The GEMV kernels have no work shared between their waves.  One row of X in the first format
// (8-vectors, 8-bit codes, at most two codebooks per workgroup's share of the rows) goes to the wide
// form at any N (Tuning::gemv_wide_min_rows_per_wave rows per wave, 0 by default): measured against the batched kernel
// on a 256-CU MI355X, cold HBM, K = 4096: N = 4096 4.96 -> 3.4 us, N = 16384 7.5 -> 5.1, N = 28672
// 9.9 -> 7.1, N = 65536 15.6 -> 12.4; K = 8192: N = 8192 8.3 -> 5.6, N = 28672 18.3 -> 10.8.
// The four-wave kernel takes what is left where it was measured faster than the batched kernel
// (us, batched -> GEMV, cold HBM, K = 4096): 1 tile of 16 rows per compute unit 4.96 -> 3.85, 2 tiles
// 6.0 -> 4.8, 4 tiles 7.5 -> 6.6, 8 tiles 11.1 -> 11.1; K = 8192 (x takes 64 registers, two waves per
// SIMD) is a tie already at 2 tiles.  Two rows of X (every gathered codeword meets both): one tile per
// unit 5.0 -> 4.8, two tiles a tie; three and four rows lose everywhere (5.1 -> 5.6 and 6.6 on one tile).
bool decode_gemv_preferred(const ProblemB &p)
{
    if (decode_gemv_wide_preferred(p)) return true;
    // Other code formats (same kernel, other gather width): one row of X only, and not with a table
    // of more than 32 KB, which every workgroup has to fill (us cold at K = 4096, batched -> GEMV:
    // 4-vectors / 8-bit codes N = 4096 5.0 -> 4.2, N = 16384 9.2 -> 7.3; 2-vectors 6.0 -> 5.6; 4-vectors /
    // 16-bit codes / 4096 entries N = 11008 9.9 -> 9.5; 8-vectors / 16-bit codes / 4096 entries 5.6 -> 5.9).
    const bool first_format = p.vec == 8 && p.code_bits == 8;
    if (!first_format && (p.M != 1 || (int64_t)p.entries * p.vec * 2 > 32 * 1024)) return false;
    const Tuning &tn = tuning();
    const double max_tiles_per_cu = p.M == 1 ? tn.gemv_max_tiles_per_cu : (p.M == 2 ? 1.0 : 0.0);
    if (!decode_gemv_supports(p) || (double)(p.N / kTileN) > max_tiles_per_cu * device_cu_count()) return false;
    return (double)p.K <= tn.gemv_max_k;
}

hipError_t launch_decode_b(const ProblemB &p, hipStream_t s)
{
    if (!decode_supports(p)) return hipErrorInvalidValue;
    // long rows of W: the streaming kernel (the batched kernel would walk K in chunks)
    if (decode_stream_preferred(p)) return launch_decode_stream(p, s);
    const bool u8 = p.code_bits == 8;
    if (batched_supports(p)) {
        // one launch, the 16-row slabs of X on the second grid dimension
        if (p.packed) {
            switch (p.vec) {
            case 8: return u8 ? launch_decode_batched<8, uint8_t, true>(p, s) : launch_decode_batched<8, uint16_t, true>(p, s);
            case 4: return u8 ? launch_decode_batched<4, uint8_t, true>(p, s) : launch_decode_batched<4, uint16_t, true>(p, s);
            default: return u8 ? launch_decode_batched<2, uint8_t, true>(p, s) : launch_decode_batched<2, uint16_t, true>(p, s);
            }
        }
        switch (p.vec) {
        case 8: return u8 ? launch_decode_batched<8, uint8_t, false>(p, s) : launch_decode_batched<8, uint16_t, false>(p, s);
        case 4: return u8 ? launch_decode_batched<4, uint8_t, false>(p, s) : launch_decode_batched<4, uint16_t, false>(p, s);
        default: return u8 ? launch_decode_batched<2, uint8_t, false>(p, s) : launch_decode_batched<2, uint16_t, false>(p, s);
        }
    }
    if (p.packed) return hipErrorInvalidValue;  // only the batched kernel reads the packed layout
    // The general kernel multiplies 16 rows of X per launch; taller X goes in slabs, one launch
    // each: still far better than a 256-row MFMA tile that is mostly padding and fills only
    // N/256 compute units.
    for (int m0 = 0; m0 < p.M; m0 += 16) {
        ProblemB q = p;
        q.x = p.x + (int64_t)m0 * p.K;
        q.y = p.y + (int64_t)m0 * (p.gated ? p.N / 2 : p.N);
        q.M = p.M - m0 < 16 ? p.M - m0 : 16;
        const hipError_t e = launch_decode_general(q, s);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace vq
