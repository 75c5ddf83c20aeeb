// Device helpers and tile constants shared by the prefill kernels (vq_prefill.hip: 256x256 and
// 256x128 tiles; vq_prefill_small.hip: 128x128 tiles).
#pragma once

#include "vq_tile_helpers.h"

namespace vq {

namespace {

constexpr int BM = 256, BN = 256;     // workgroup tile
constexpr int WM = 128, WN = 128;     // wave tile
constexpr int MP = WM / 16, NP = WN / 16;  // 16-row pieces of X and of W per wave
constexpr int kThreads = 256;
constexpr int kStageK = 64;           // k per LDS stage (2 MFMA steps)
constexpr int kStageBytes = BM * kStageK * 2;  // 32 KB
constexpr int kChunksPerThread = (BM * 8) / kThreads;  // 16-byte chunks of an X stage per thread

template <int VEC, typename CodeT>
struct PrefillCfg {
    static constexpr int CSZ = (int)sizeof(CodeT);
    static constexpr int CPO = 8 / VEC;                 // codes per 8-half operand
    static constexpr int RB = CPO * CSZ;                // bytes of codes behind one operand (1, 2 or 4)
    static constexpr int KC = (16 / CSZ) * VEC;         // k covered by 16 bytes of one row's codes
    static constexpr int K_SUPER = KC > kStageK ? KC : kStageK;  // k per code tile (a "super stage")
    static constexpr int STAGES = K_SUPER / kStageK;    // LDS stages per super stage (1 or 2)
    static constexpr int CH = K_SUPER / KC;             // 16-byte chunks per row of a code tile (1 or 2)
    static constexpr int HALF = 32 / VEC * CSZ;         // bytes of one row's codes per MFMA step
    static constexpr int kTileBytes = CH * BN * 16;     // code tile in the LDS: [chunk][row][16 bytes]
    static_assert(RB == 1 || RB == 2 || RB == 4, "unsupported code layout");
    static_assert(STAGES == 1 || STAGES == 2, "unsupported code layout");
    // code tiles in flight: the one being read plus those loaded ahead
    static constexpr int code_bufs(int ns) { return STAGES == 1 ? ns : 3; }
};

// Byte offset inside a stage buffer of logical 16-byte chunk cc (0..7) of X-tile row `row`.
__device__ __forceinline__ int x_offset(int row, int cc)
{
    const int bank_row = row >> 1;
    const int pos = (((row & 1) << 3) | cc) ^ (bank_row & 15);
    return (bank_row * 16 + pos) * 16;
}

// The four fp32 sums of an accumulator rounded to fp16, with the bias of their columns added first.
template <bool HAS_BIAS>
__device__ __forceinline__ half4_t round4(const float4_t &a, const float (&b)[4])
{
    if constexpr (HAS_BIAS)
        return half4_t{(half_t)(a[0] + b[0]), (half_t)(a[1] + b[1]), (half_t)(a[2] + b[2]), (half_t)(a[3] + b[3])};
    else
        return half4_t{(half_t)a[0], (half_t)a[1], (half_t)a[2], (half_t)a[3]};
}

// The gated epilogue of a wave tile of MPC x NPC pieces: pieces 2q and 2q+1 along N are the gate and the up
// rows of output piece q (the rows of W are interleaved in groups of 16), so a lane holds both factors of its
// four outputs: out = silu(gate + bias) * (up + bias) in fp32, rounded once.  The lane holds rows
// i*16 + r16 and columns 4*kg .. 4*kg+3 of every piece; m_wave / n_wave are the tile's first row of Y and
// first (interleaved) row of W.  The rows of W are a multiple of 32 (pairs are whole), so the 8-byte stores are aligned.
template <int NPC, int MPC, bool HAS_BIAS>
__device__ __forceinline__ void store_gated(const float4_t (&acc)[NPC][MPC], half_t *__restrict__ y,
                                            const half_t *__restrict__ bias, int M, int n_limit, int n_rows_w,
                                            int m_wave, int n_wave, int r16, int kg)
{
    // n_rows_w: rows of the whole W (y has half as many columns); n_limit: the launch's last row of W + 1
    static_assert(NPC % 2 == 0, "whole pairs of pieces");
    const int ldy = n_rows_w / 2;
#pragma unroll
    for (int i = 0; i < MPC; i++) {
        const int m = m_wave + i * 16 + r16;
        if (m >= M) continue;
#pragma unroll
        for (int q = 0; q < NPC / 2; q++) {
            const int n = n_wave + 32 * q;  // the gate piece's first row of W
            if (n >= n_limit) continue;
            float4_t g = acc[2 * q][i], u = acc[2 * q + 1][i];
            if constexpr (HAS_BIAS) {
                const half4_t bg = *reinterpret_cast<const half4_t *>(bias + n + 4 * kg);
                const half4_t bu = *reinterpret_cast<const half4_t *>(bias + n + 16 + 4 * kg);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    g[e] += (float)bg[e];
                    u[e] += (float)bu[e];
                }
            }
            half4_t h;
#pragma unroll
            for (int e = 0; e < 4; e++) h[e] = (half_t)(silu_f32(g[e]) * u[e]);
            *reinterpret_cast<half4_t *>(y + (int64_t)m * ldy + n / 2 + 4 * kg) = h;
        }
    }
}

// floor(x / d) for 0 <= x and a quotient small enough that float rounding stays within one
// (here: x < d + 256); `rcp` = 1.0f / d.
__device__ __forceinline__ int small_div(int x, int d, float rcp)
{
    int qt = (int)((float)x * rcp);
    const int rem = x - qt * d;
    qt += rem >= d ? 1 : 0;
    qt -= rem < 0 ? 1 : 0;
    return qt;
}

// The RB bytes of codes behind one operand, zero-extended.
template <int RB>
__device__ __forceinline__ uint32_t read_codes(const uint8_t *p)
{
    if constexpr (RB == 1) return *p;
    else if constexpr (RB == 2) return *reinterpret_cast<const uint16_t *>(p);
    else return *reinterpret_cast<const uint32_t *>(p);
}

// Gathers half `h` (4 halves) of one MFMA operand: the codes packed in `cr` select codewords of
// the codebook at LDS byte offset `book`.  With `zero` set the reads go to the 16 zero bytes at
// `zero_off` instead (a step past the end of K).  An operand is fetched in two halves because a
// 16-byte gather with its bank conflicts holds the wave's issue longer than the gap between two
// MFMAs.
// SPLIT (8-vectors, 256 entries): a codebook lies in the LDS as two tables, the first 8 bytes of
// every entry and, kSplitHi bytes on, the second 8 bytes.  A half gather at a 16-byte stride reaches
// only every other pair of the 64 banks; at an 8-byte stride it spreads over all of them, and
// random codewords collide less often.
constexpr uint32_t kSplitEntries = 256, kSplitHi = kSplitEntries * 8;

template <int VEC, typename CodeT, bool TAIL, bool SPLIT = false>
__device__ __forceinline__ half4_t gather4(const uint8_t *lds, uint32_t book, uint32_t cr, int h, bool zero, uint32_t zero_off)
{
    constexpr int CPO = 8 / VEC, BITS = 8 * (int)sizeof(CodeT);
    static_assert(!SPLIT || VEC == 8, "the split layout is for 16-byte entries");
    if constexpr (SPLIT) {
        uint32_t a = book + cr * 8u + (h ? kSplitHi : 0u);
        if (TAIL) a = zero ? zero_off : a;
        return *reinterpret_cast<const half4_t *>(lds + a);
    }
    auto at = [&](int c, int byte_off) {
        const uint32_t code = CPO == 1 ? cr : (cr >> (BITS * c)) & ((1u << BITS) - 1u);
        uint32_t a = book + code * (uint32_t)(VEC * 2);
        if (TAIL) a = zero ? zero_off : a;
        return lds + a + byte_off;
    };
    if constexpr (VEC == 8) {
        return *reinterpret_cast<const half4_t *>(at(0, 8 * h));
    } else if constexpr (VEC == 4) {
        return *reinterpret_cast<const half4_t *>(at(h, 0));
    } else {
        static_assert(VEC == 2, "vector length must be 2, 4 or 8");
        const half2_t q0 = *reinterpret_cast<const half2_t *>(at(2 * h, 0));
        const half2_t q1 = *reinterpret_cast<const half2_t *>(at(2 * h + 1, 0));
        return __builtin_shufflevector(q0, q1, 0, 1, 2, 3);
    }
}

// Re-lays `count` codebooks of 256 16-byte entries from a plain copy at LDS offset `src` into the
// split layout at `dst` (all threads of the workgroup; the caller synchronises before and after).
__device__ __forceinline__ void split_codebooks(uint8_t *lds, uint32_t src, uint32_t dst, int count, int tid, int n_threads)
{
    for (int i = tid; i < count * (int)kSplitEntries; i += n_threads) {
        const int g = i / (int)kSplitEntries, e = i % (int)kSplitEntries;
        const uint4_t v = *reinterpret_cast<const uint4_t *>(lds + src + i * 16);
        *reinterpret_cast<uint2_t *>(lds + dst + g * (2 * kSplitHi) + e * 8) = uint2_t{v[0], v[1]};
        *reinterpret_cast<uint2_t *>(lds + dst + g * (2 * kSplitHi) + kSplitHi + e * 8) = uint2_t{v[2], v[3]};
    }
}

// whether a tile's codebooks can take the split layout, given the bytes free for the plain copy
inline bool split_layout_applies(const ProblemB &p, int codebooks, size_t temp_bytes)
{
    return p.vec == 8 && p.code_bits == 8 && p.entries == (int)kSplitEntries && (size_t)codebooks * 2 * kSplitHi <= temp_bytes;
}

constexpr size_t kLdsLimit = 160 * 1024;

// Worst case number of codebooks a band of `bn` rows of W touches.
inline int codebooks_per_tile(const ProblemB &p, int bn)
{
    int n;
    if (p.n_codebooks == 1) n = 1;
    else if (p.rows_per_cb >= bn && p.rows_per_cb % bn == 0) n = 1;
    else if (bn % p.rows_per_cb == 0) n = bn / p.rows_per_cb;
    else n = (bn + p.rows_per_cb - 1) / p.rows_per_cb + 1;
    return n < p.n_codebooks ? n : p.n_codebooks;
}

// codebooks of a tile, padded to the 1 KB steps they are copied in, plus 16 zero bytes
inline size_t books_bytes(const ProblemB &p, int bn)
{
    return (((size_t)codebooks_per_tile(p, bn) * p.entries * p.vec * 2 + 1023) & ~(size_t)1023) + 16;
}

}  // namespace

}  // namespace vq
