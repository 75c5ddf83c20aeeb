// Shared device helpers and launcher declarations for the gfx950 VQ-GEMM kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vq {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// Problem description shared by the geometry-B kernels.
struct ProblemB {
    const half_t *x;      // [M,K]
    const void *codes;    // [N, K/vec] u8 or u16
    const half_t *cb;     // [G, E, vec]
    half_t *y;            // [M,N]
    const half_t *bias;   // [N] added to the fp32 sums before the rounding to fp16, or nullptr
    int M, K, N;
    int vec, entries, n_codebooks, code_bits;
    int rows_per_cb;      // N / G
    bool packed;          // codes are in the packed layout of the batched decode kernel (launch_pack_codes)
    bool gated;           // gated epilogue: the rows of W are gate and up rows interleaved in groups of 16 (rows
                          // 32g .. 32g+15 gate, 32g+16 .. 32g+31 up) and y is [M, N/2]:
                          // y[m, 16g + r] = silu(P[m, 32g + r]) * P[m, 32g + 16 + r], P = X . W^T (+ bias) in fp32
};

// silu(g) = g / (1 + exp(-g)) in fp32, as every kernel with the gated epilogue and the element-wise kernel compute it
__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + __expf(-g)); }

struct ProblemA {
    const half_t *x;      // [M,K]
    const uint8_t *w;     // [K,Nc]
    const half_t *cb;     // [Nc/4, 256, 2]
    half_t *y;            // [M, 2*Nc]
    int M, K, Nc;
};

__device__ __forceinline__ uint32_t lane_id() { return threadIdx.x & (kWave - 1); }

// 16-byte global load / store helpers (addresses must be 16-byte aligned).
__device__ __forceinline__ uint4_t ld_global_16(const void *p) { return *reinterpret_cast<const uint4_t *>(p); }
__device__ __forceinline__ void st_global_16(void *p, uint4_t v) { *reinterpret_cast<uint4_t *>(p) = v; }

template <typename T>
__device__ __forceinline__ half8_t as_half8(T v)
{
    static_assert(sizeof(T) == 16, "16-byte value expected");
    union { T t; half8_t h; } u;
    u.t = v;
    return u.h;
}

// 16-byte global load straight into the LDS: lane l writes smem[lds_base + 16*l ..].  The
// compiler knows nothing about this transfer (completion is only visible through vmcnt), so
// every consumer sits behind an explicit vmcnt wait + barrier.  `lds_base` must be wave-uniform.
// The statement writes m0 and says so, so that compiler-generated uses of m0 stay correct.
__device__ __forceinline__ void load_to_lds_16(uint32_t lds_base, uint32_t voff, const void *sbase)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_base), "v"(voff), "s"(sbase)
                 : "memory", "m0");
}

// ---- launchers (defined one per .hip file) -------------------------------------------
hipError_t launch_dequant_b(const ProblemB &p, half_t *w_out, hipStream_t s);
hipError_t launch_dequant_a(const ProblemA &p, half_t *w_out, hipStream_t s);

// nearest-codeword codes of w[N,K] (p.x, p.y unused)
bool encode_supports(const ProblemB &p);
hipError_t launch_encode_b(const half_t *w, const ProblemB &p, void *codes_out, hipStream_t s);

hipError_t launch_generic_b(const ProblemB &p, hipStream_t s);
hipError_t launch_generic_a(const ProblemA &p, hipStream_t s);

bool decode_supports(const ProblemB &p);
// whether the decode path is expected to beat the prefill kernel on a shape it supports
bool decode_preferred(const ProblemB &p);
hipError_t launch_decode_b(const ProblemB &p, hipStream_t s);
// The packed code layout of the batched decode kernel: the pieces of the code matrix in the order
// the kernel's lanes load them (same size, codes unchanged).  `inverse` restores the plain matrix.
bool pack_codes_supports(int64_t N, int64_t K, int vec, int code_bits);
hipError_t launch_pack_codes(const void *src, void *dst, int64_t N, int64_t K, int vec, int code_bits, bool inverse,
                             hipStream_t s);
// whether launch_decode_b takes the shape with p.packed set (the batched kernel only)
bool decode_packed_supports(const ProblemB &p);
// the GEMV kernel behind launch_decode_b (vq_decode_gemv.hip): one row of X, 8-vectors, 8-bit codes,
// whole rows of W per wave; the automatic choice takes it while a compute unit has few rows to do
bool decode_gemv_supports(const ProblemB &p);
hipError_t launch_decode_gemv(const ProblemB &p, hipStream_t s);
// the wide form of the GEMV kernel (one 16-wave workgroup per compute unit, one row of X, 8-vectors, 8-bit
// codes) and whether launch_decode_gemv takes it for the shape (from one row per wave on)
bool decode_gemv_wide_supports(const ProblemB &p);
bool decode_gemv_wide_preferred(const ProblemB &p);
// whether the automatic choice takes the GEMV kernel rather than launch_decode_b for a shape both serve
bool decode_gemv_preferred(const ProblemB &p);
// the general kernel behind launch_decode_b: one slab of at most 16 rows of X
bool decode_general_supports(const ProblemB &p);
hipError_t launch_decode_general(const ProblemB &p, hipStream_t s);

// the streaming kernel behind launch_decode_b for long rows of W (vq_decode_stream.hip): 8-vectors, 8-bit codes
bool decode_stream_supports(const ProblemB &p);
bool decode_stream_preferred(const ProblemB &p);
hipError_t launch_decode_stream(const ProblemB &p, hipStream_t s);

// whether the batched K-sliced decode kernel takes the shape with its gated epilogue (p.gated set)
bool decode_gated_supports(const ProblemB &p);
// expected microseconds of the batched decode kernel for tall X (more rows than the general kernel serves); 1e30 otherwise
double decode_cost_us(const ProblemB &p);

bool prefill_supports(const ProblemB &p);
// whether the 256x128 tile of the prefill kernel can serve the shape (a subset of prefill_supports)
bool prefill_narrow_supports(const ProblemB &p);
// expected time of the prefill kernel with the tile width it would choose, microseconds
double prefill_cost_us(const ProblemB &p);
// tile: 0 = the tile expected to be fastest (256x256, 256x128, a mix of the two, or 128x128),
// 1 = 256x256, 2 = 256x128
hipError_t launch_prefill_b(const ProblemB &p, hipStream_t s, int tile = 0);

// Whole rounds of large tiles over the first columns of W, the columns that are left in 128x128 tiles with K split
// (needs a workspace when splits > 1): the plan with its expected time, and its two launches.
struct TailSplitPlan {
    bool ok;
    int head_tile;   // 1: 256x256 tiles, 2: 256x128 tiles over the W rows [0, n_split)
    int n_split;     // the 128x128 kernel takes the W rows [n_split, N)
    int splits;      // slices of K there (1: none)
    double cost_us;
    size_t workspace_bytes;
};
TailSplitPlan prefill_tail_split_plan(const ProblemB &p);
hipError_t launch_prefill_tail_split(const ProblemB &p, const TailSplitPlan &plan, hipStream_t s, void *workspace);

// the prefill kernel with 128x128 tiles (vq_prefill_small.hip), for medium M
bool prefill_small_supports(const ProblemB &p);
double prefill_small_cost_us(const ProblemB &p);  // expected time, microseconds (1e30: not supported)
// splits > 1: split K, `splits` workgroups per tile (workspace of prefill_splitk_workspace_bytes, device memory)
// n_begin > 0: the W rows [n_begin, N) only (a multiple of 128; the workspace is then sized for those columns)
hipError_t launch_prefill_small_b(const ProblemB &p, hipStream_t s, int splits = 1, void *workspace = nullptr, int n_begin = 0);
bool prefill_splitk_supports(const ProblemB &p, int splits);
size_t prefill_splitk_counter_bytes(int64_t tiles);
size_t prefill_splitk_workspace_bytes(const ProblemB &p, int splits);
// slices of K the cost model expects to be fastest with 128x128 tiles and the time it expects (min_splits 1: none is a
// candidate; 2: the best split); 0 when no split applies
int prefill_splitk_choice(const ProblemB &p, double *cost_us, int min_splits = 1);

// o[M,N] = x[M,K] . w[K,N]
hipError_t launch_gemm_nn(const half_t *x, const half_t *w, half_t *y, int M, int K, int N, hipStream_t s);
// y[M,N] = x[M,K] . w[N,K]^T
hipError_t launch_gemm_nt(const half_t *x, const half_t *w, half_t *y, int M, int K, int N, hipStream_t s);
// the tiled kernel behind the two above (w_is_kn: w is [K,N], else [N,K]) and the shapes it takes;
// tile: 0 = the width expected to be faster, 1 = 256x256, 2 = 256x128
bool gemm_tiled_supports(const half_t *x, const half_t *w, int M, int K, int N, bool w_is_kn);
hipError_t launch_gemm_tiled(const half_t *x, const half_t *w, half_t *y, int M, int K, int N, bool w_is_kn, hipStream_t s,
                             int tile = 0);

// geometry A, fused: the tiled [K,N] GEMM with its W stages dequantised on the compute unit
bool fused_a_supports(const ProblemA &p);
hipError_t launch_fused_a(const ProblemA &p, hipStream_t s);

// out[M,N] = silu(a[:, :N]) * a[:, N:] for a [M, 2N]
// (interleaved: gate and up columns alternate in groups of 16 instead of lying in the two halves of a row)
hipError_t launch_silu_mul(const half_t *a, half_t *out, int64_t M, int64_t N, hipStream_t s, bool interleaved = false);

// out[0] = the largest code of codes[0 .. count) (0 when count == 0); out is device memory
hipError_t launch_max_code(const void *codes, int64_t count, int code_bits, uint32_t *out, hipStream_t s);
// words[0 .. n) = 0, by a kernel (a launch that may be captured into a graph records no memset)
hipError_t launch_clear_words(uint32_t *words, int64_t n, hipStream_t s);

int device_cu_count();

// The constants of the cost models behind the automatic kernel choice.  The compiled-in values were fitted to
// measurements on one 256-CU MI355X; vqgemm_tuning_set / a file named by VQGEMM_TUNING_FILE (written by
// `python -m vq_gemm_amd.tune --fit`) replace them with what the box at hand measures.
struct Tuning {
    // prefill kernels: microseconds per tile of prologue + epilogue, and per 64-k stage on an idle device; a
    // full device holds a lower clock: the stage time grows by `prefill_full_device_factor` at one tile per unit
    double prefill_tile_fixed_us = 5.0;
    double prefill_stage_us_256x256 = 1.0;
    double prefill_stage_us_256x128 = 0.56;
    double prefill_full_device_factor = 1.6;
    double prefill_small_tile_fixed_us = 4.0;
    double prefill_small_stage_us_idle = 0.46;
    double prefill_small_stage_us_busy = 0.56;
    // batched decode kernel: per workgroup a prologue, then per tile of 16 rows and 4096 k
    double decode_prologue_us = 3.0;
    double decode_prologue_shared_cu_us = 8.0;
    double decode_tile_us = 0.75;
    double decode_tile_chunked_us = 1.25;
    double decode_pass_change_us = 5.0;
    // GEMV kernels: the four-wave kernel up to this many 16-row tiles per unit and this K; the wide form from this
    // many rows per wave on
    double gemv_max_tiles_per_cu = 4.0;
    double gemv_max_k = 8192.0;
    double gemv_wide_min_rows_per_wave = 0.0;
    double gemv_wide_max_m = 2.0;   // rows of X the automatic choice gives the wide form (it takes one or two)
    double gemv_wide_two_rows_max_runs = 22.0;   // ... two rows of X while a wave's rows are at most this many runs of 2048 k
    double gemv_wide_two_rows_max_runs_long_k = 36.0;   // ... the same from K = 8192 on
    // the wide form gathers from the plain 4 KB table while a wave's rows are at most this many runs of 2048 k, from the
    // bank-replicated one (64 KB to fill) beyond
    double gemv_wide_plain_table_max_runs = 2.0;
    // the wide form's loop: rows of W per group (1 or 2) and groups of codes in flight (2 or 3), for K up to 4096
    // and beyond
    double gemv_wide_single_rows_max = 2.0;  // up to this many rows per wave: groups of one row, two in flight
    double gemv_wide_rows_per_group = 2.0;
    double gemv_wide_groups_in_flight = 2.0;
    double gemv_wide_rows_per_group_long_k = 1.0;
    double gemv_wide_groups_in_flight_long_k = 2.0;
    // the wide form leaves up to this share of the compute units without a workgroup where that keeps every workgroup's
    // rows inside one codebook
    double gemv_wide_min_units_share = 0.7;
    // the wide form's waves step their issue priority round with every group (1) or leave it alone (0)
    double gemv_wide_rotate_priority = 1.0;
    // batched decode kernel: the bank-replicated table (64 KB to fill) from this many tiles per workgroup on
    double decode_replicated_table_min_tiles = 2.0;
    // streaming decode kernel (whole K per workgroup, K dealt to the waves in pieces): taken by the K-sliced path from
    // this K on (the batched kernel walks K beyond 4096 in chunks) for this range of rows of X and at most this many
    // groups of tiles per compute unit, and its bank-replicated table from this many gathers per lane on
    double decode_stream_min_k = 8192.0;
    double decode_stream_min_k_few_rows = 14336.0;  // with eight rows of X or fewer
    double decode_stream_min_m = 1.0;
    double decode_stream_max_m = 16.0;
    double decode_stream_max_groups_per_unit = 1.0;
    double decode_stream_replicated_min_gathers = 0.0;
    // whole rounds of large tiles plus the left-over columns in 128x128 tiles with K split: taken with a workspace when
    // expected below this share of the best single plan (0: never; 1000 and more: wherever the plan exists)
    double tail_split_margin = 0.93;
    // split K over 128x128 tiles: the clearing launch and the last workgroup's extra pass, and the partial sums
    // written and read once (microseconds per MB of partial sums)
    double splitk_fixed_us = 4.5;
    double splitk_us_per_partial_mb = 0.15;
    // 2, 4 or 8: VQGEMM_VARIANT_PREFILL_SPLITK takes this many slices where the shape allows (for measurements); 0: the cost model's
    double splitk_force_splits = 0.0;
    double splitk_validate_fences = 0.0;  // 1: release / acquire fences of device scope around the split-K count (validation)
};
const Tuning &tuning();

// Raises a kernel's dynamic-LDS limit when `bytes` needs it; remembers what was granted per
// (device, kernel) so that steady-state launches make no attribute call.
hipError_t ensure_dynamic_lds(const void *kernel, size_t bytes);

}  // namespace vq
