/*
 * vq_gemm.h — C ABI of the MI355X (gfx950) vector-quantized GEMM library, libvqgemm.so.
 *
 * Every pointer is a device pointer (HIP, current device) unless stated otherwise; all
 * matrices are dense row-major; `stream` is a hipStream_t passed as void* (NULL = the
 * default stream).  Calls only enqueue work; they do not synchronise.  Return value:
 * 0 on success, a negative VQGEMM_E_* code for rejected arguments (nothing was launched),
 * a positive hipError_t when the runtime refused the launch.
 *
 * Two data geometries are served.
 *   Geometry B (K-axis vectors):  Y[M,N] = X[M,K] . W^T,
 *       W[n, j*vec + t] = codebook[n / (N/n_codebooks)][codes[n, j]][t],
 *       codes [N, K/vec] uint8 or uint16, codebook [n_codebooks, entries, vec] fp16.
 *   Geometry A (the reference's native layout, bench.py:83-85 of the reference):
 *       out[M, 2*Nc] = X[M,K] . W_dec,  W_dec[k, 2n + r] = codebook[n/4][w[k,n]][r],
 *       w [K, Nc] uint8, codebook [Nc/4, 256, 2] fp16.
 * Products accumulate in fp32 and are rounded once to fp16.
 */
#ifndef VQ_GEMM_H
#define VQ_GEMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* argument errors */
#define VQGEMM_OK 0
#define VQGEMM_E_NULL (-1)      /* a required pointer is NULL */
#define VQGEMM_E_SHAPE (-2)     /* negative size, K % vec != 0, N % n_codebooks != 0, ... */
#define VQGEMM_E_CODEBITS (-3)  /* code_bits not 8/16, or entries > 2^code_bits */
#define VQGEMM_E_VARIANT (-4)   /* unknown variant, or the variant cannot serve this shape */
#define VQGEMM_E_ALIGN (-5)     /* a pointer is not aligned to its element size */
#define VQGEMM_E_SCRATCH (-6)   /* the problem needs more scratch than the library's fixed device array, or the
                                   workspace that was passed with its size, holds */

/* kernel selection for the fused GEMM */
#define VQGEMM_VARIANT_AUTO 0     /* pick by shape */
#define VQGEMM_VARIANT_GENERIC 1  /* simple scalar kernel, any shape */
#define VQGEMM_VARIANT_DECODE 2   /* small and medium M, 16 rows of X per workgroup: K-sliced waves, 16x16x32 MFMA,
                                     LDS-resident codebook; M <= 4096 when K % 256 == 0, N % 16 == 0 and
                                     (N / n_codebooks) % 16 == 0, M <= 64 otherwise.  Up to sixteen rows of X on long
                                     rows of W (K >= 8192, 8-vectors, 8-bit codes, few tiles per compute unit) go
                                     through the streaming kernel of this path: K dealt to the waves in pieces, no
                                     chunks of K */
#define VQGEMM_VARIANT_PREFILL 3  /* large M: 256x256 tiles of 16x16x32 MFMAs, codewords gathered into operands;
                                     256x128 tiles when those put more compute units to work */
#define VQGEMM_VARIANT_TWOPASS 4  /* dequantise to HBM scratch, then the plain fp16 GEMM */
#define VQGEMM_VARIANT_PREFILL_NARROW 5  /* the prefill kernel with 256x128 tiles, whatever the shape */
#define VQGEMM_VARIANT_PREFILL_SMALL 6   /* the prefill kernel with 128x128 tiles, two workgroups per compute unit
                                            (medium M); K a multiple of 64, of 128 for 8-vectors with 8-bit codes */
#define VQGEMM_VARIANT_DECODE_PACKED 7   /* VQGEMM_VARIANT_DECODE on a code matrix that vqgemm_pack_codes_b has put
                                            in the order the kernel's lanes load it (never chosen by AUTO: the
                                            layout is a property of the caller's data); the K-sliced MFMA kernel
                                            whatever the shape, same results bit for bit as that kernel on the plain
                                            matrix (where VQGEMM_VARIANT_DECODE takes its streaming kernel instead, the
                                            sums are added in another order) */
#define VQGEMM_VARIANT_DECODE_GEMV 8     /* the GEMV kernels: whole rows of W per wave, no matrix core.  One row of X,
                                            8-vectors with 8-bit codes, at most 256 entries, K a multiple of 2048 up
                                            to 8192, at most 64 rows of W per wave of a 16-wave workgroup per compute
                                            unit and at most two codebooks per workgroup: the wide form (AUTO takes it
                                            at any N).  Two rows of X in the same form with K = 2048 or 4096, and with
                                            any other multiple of 32 up to 16384 in pieces like the long rows below (AUTO
                                            takes two rows while a wave's rows of W make at most 22 runs of 2048 k, 36
                                            from K = 8192 on: the tuning table's gemv_wide_two_rows_max_runs and
                                            ..._long_k).  The wide form also takes any other K from
                                            2048 to 32768 that is a multiple of 32 (a row worked through in pieces of
                                            6144 or 8192 k: the down-projection of an MLP), then not gated and with
                                            every workgroup's rows inside one codebook.  Otherwise the four-wave form: M <= 4 for that
                                            format, M <= 2 for 4-vectors, 8-vectors with 16-bit codes and 2-vectors
                                            with 8-bit codes; at most 256 resp. 4096 entries, entries * vec a multiple
                                            of 8; K a multiple of 2048 with (K / 2048) * M <= 8, N and N / n_codebooks
                                            multiples of 16.  AUTO takes it where it was measured faster than
                                            VQGEMM_VARIANT_DECODE, the K-sliced MFMA kernels (the limits are constants
                                            of the tuning table below) */

#define VQGEMM_VARIANT_PREFILL_SPLITK 9  /* vqgemm_e2e_gemm_b_ws only: the 128x128 tiles with K split over 2, 4 or 8
                                            workgroups per tile (as many as the cost model expects to be fastest);
                                            medium M on few columns, where whole tiles are fewer than the compute
                                            units; fp32 partial sums through the workspace */

/*
 * Fused VQ GEMM, geometry B.
 * Replaces: torch::Tensor e2e_gemm(input, w, codebook) — reference bind.cpp:3,7 and the host
 * wrappers strategy_2/bsz128/src.cu:255-316 (and the four sibling copies) — for the K-axis
 * layout the measured configurations use.
 * `workspace` is only read by VQGEMM_VARIANT_TWOPASS (N*K fp16 scratch); NULL otherwise.
 */
int vqgemm_e2e_gemm_b(const void *x, const void *codes, const void *codebook, void *y,
                      int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries,
                      int32_t n_codebooks, int32_t code_bits, int32_t variant,
                      void *workspace, void *stream);

/*
 * The same with a bias: Y[m,n] = sum_k X[m,k] W[n,k] + bias[n], bias [N] fp16 (NULL = none), added
 * to the fp32 sum before the one rounding to fp16.  No counterpart in the reference (its e2e_gemm
 * has no epilogue); for call sites that hold a linear layer.  VQGEMM_VARIANT_TWOPASS does not take
 * a bias; the tiled kernels want `bias` 8-byte aligned (the automatic choice falls back to the scalar
 * kernel otherwise).
 */
int vqgemm_e2e_gemm_b_bias(const void *x, const void *codes, const void *codebook, const void *bias, void *y,
                           int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries,
                           int32_t n_codebooks, int32_t code_bits, int32_t variant,
                           void *workspace, void *stream);

/*
 * vqgemm_e2e_gemm_b_bias with a workspace whose size the library is told, so that the automatic choice may use
 * kernels that need scratch memory: split K over every 128x128 tile (VQGEMM_VARIANT_PREFILL_SPLITK), which
 * VQGEMM_VARIANT_AUTO takes where its cost model expects at least 10 % over what it would launch otherwise, and -
 * where the large tiles of a shape are a few more than whole rounds over the compute units - those whole rounds as
 * one launch and the columns of W that are left over as a second one, in 128x128 tiles with K split there; either
 * only when `workspace_bytes` suffices (a workspace that is too small, or NULL, is no error for AUTO: it does without).  vqgemm_workspace_bytes_b says
 * how many bytes the given variant (AUTO, PREFILL_SPLITK, TWOPASS) wants for a shape: 0 when it uses none, a
 * negative error for an invalid shape.  `workspace` must be 256-byte aligned device memory; its contents before the
 * call do not matter and are undefined after it; two calls that overlap in time need a workspace each.  An explicit
 * variant with too small a workspace returns VQGEMM_E_SCRATCH.  The partial sums of a tile are added in the order
 * of the slices of K whichever workgroup finishes last: results are the same from run to run.  No counterpart in
 * the reference (one workgroup per tile over all of K, strategy_2/bsz128/src.cu:179-253).
 */
int vqgemm_e2e_gemm_b_ws(const void *x, const void *codes, const void *codebook, const void *bias, void *y,
                         int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries,
                         int32_t n_codebooks, int32_t code_bits, int32_t variant,
                         void *workspace, int64_t workspace_bytes, void *stream);
int64_t vqgemm_workspace_bytes_b(int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries,
                                 int32_t n_codebooks, int32_t code_bits, int32_t variant);

/*
 * The fused VQ GEMM with a gated epilogue, for a gate/up projection pair (the MLP shapes among the measured
 * configurations): the rows of W (as codes) are the gate rows and the up rows of the pair interleaved in groups of
 * 16 - rows 32g .. 32g+15 are gate rows 16g .. 16g+15, rows 32g+16 .. 32g+31 the up rows of the same columns -
 * and
 *     y[m, 16g + r] = silu(P[m, 32g + r]) * P[m, 32g + 16 + r],   P = X . W^T (+ bias[n], indexed like the rows of W),
 * silu(t) = t / (1 + exp(-t)), everything in fp32 with one rounding to fp16: y is [M, N/2] and the [M, N] product
 * never exists in memory.  N % 32 == 0.  No counterpart in the reference (its storeC has no epilogue,
 * strategy_2/bsz128/src.cu:163-177).  Every fused kernel carries the epilogue: the prefill tiles (variants 3, 5, 6),
 * both K-sliced decode kernels (variant 2), both GEMV kernels (variant 8; the four-wave form and the batched K-sliced
 * kernel want (N / n_codebooks) % 32 == 0) and the scalar kernel (variant 1); VQGEMM_VARIANT_AUTO follows the plain
 * product's choice and needs no workspace.  VQGEMM_VARIANT_TWOPASS here means the plain product into `workspace`
 * ([M, N] fp16) followed by the element-wise pass (vqgemm_silu_mul's interleaved form), kept as the control; the
 * other variants ignore `workspace`.
 */
int vqgemm_e2e_gemm_b_gated(const void *x, const void *codes, const void *codebook, const void *bias, void *y,
                            int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries,
                            int32_t n_codebooks, int32_t code_bits, int32_t variant,
                            void *workspace, void *stream);

/*
 * Fused VQ GEMM, geometry A (reference-native tensors, same entry point of the reference:
 * bind.cpp:3,7; kernels strategy_2/bsz128/src.cu:213-253 and siblings, indexing per
 * strategy_2/bsz512/src.cu:163-176 and bench.py:46-56).  out is [M, 2*Nc].
 * VQGEMM_VARIANT_PREFILL is the fused tiled kernel (256x128 tiles; codebooks and code bytes in the
 * LDS, W dequantised there two MFMA steps ahead of its use): K % 64 == 0, Nc % 16 == 0, x, w and
 * codebook 16-byte aligned.  VQGEMM_VARIANT_TWOPASS needs `workspace` (K*2*Nc fp16).
 * VQGEMM_VARIANT_AUTO takes the fused kernel for M > 96 where it applies (with `workspace` given:
 * only while its tiles are at most one per compute unit, the two-pass route being faster beyond),
 * else the two-pass route when `workspace` is given and the scalar kernel when it is NULL.
 */
int vqgemm_e2e_gemm_a(const void *x, const void *w, const void *codebook, void *out,
                      int64_t M, int64_t K, int64_t Nc, int32_t variant,
                      void *workspace, void *stream);

/*
 * vqgemm_e2e_gemm_a without a workspace argument and without any allocation: the scratch of the
 * two-pass route (W_dec[K, 2*Nc] fp16) is a fixed device array inside the library,
 * VQGEMM_NOALLOC_SCRATCH_BYTES large, which every GPU the library runs on holds from load to the
 * end of the process.  No counterpart in the reference (its s1 wrapper allocates the intermediate
 * tensor per call, strategy_1/src.cu:351); it is for callers that cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  The call makes no hipMalloc,
 * hipFree or other allocating call.  Same arguments, same kernels, same results as
 * vqgemm_e2e_gemm_a with a workspace; shapes with K * 2*Nc * 2 bytes beyond the array are refused
 * with VQGEMM_E_SCRATCH, whichever route they would take.  All calls on one GPU share that GPU's
 * array: calls that overlap in time on one GPU (different streams) race on it.  Nothing in it has to
 * be cleared between calls - the dequant pass overwrites every element the GEMM pass reads.  The
 * array used is the one of the device that owns `stream` (the current device for the default stream).
 * The first call on a device looks the array's address up (which makes the runtime load the code object
 * that holds it): make that call outside stream capture - under capture it is refused with
 * hipErrorStreamCaptureUnsupported and nothing is recorded.
 */
#define VQGEMM_NOALLOC_SCRATCH_BYTES (16 << 20)
int vqgemm_e2e_gemm_a_noalloc(const void *x, const void *w, const void *codebook, void *out,
                              int64_t M, int64_t K, int64_t Nc, int32_t variant, void *stream);

/*
 * Which kernel VQGEMM_VARIANT_AUTO resolves to for a geometry-A shape with 16-byte aligned operands
 * (host only, no GPU call), so that a caller can tell whether the workspace will be used.
 */
int vqgemm_select_variant_a(int64_t M, int64_t K, int64_t Nc, int32_t has_workspace);

/*
 * Stand-alone dequantisation to fp16 in HBM.
 * Replaces: dequant_kernel + the intermediate B tensor of the two-pass strategy,
 * reference strategy_1/src.cu:268-321,351.
 * geometry B writes W[N,K]; geometry A writes W_dec[K, 2*Nc].
 */
int vqgemm_dequant_b(const void *codes, const void *codebook, void *w_out,
                     int64_t N, int64_t K, int32_t vec, int32_t entries,
                     int32_t n_codebooks, int32_t code_bits, void *stream);
int vqgemm_dequant_a(const void *w, const void *codebook, void *w_out,
                     int64_t K, int64_t Nc, void *stream);

/*
 * Nearest-codeword encoder, geometry B: the inverse of vqgemm_dequant_b for given codebooks,
 *   codes_out[n, j] = argmin_e sum_t (w[n, j*vec + t] - codebook[n / (N/n_codebooks)][e][t])^2,
 * w [N,K] fp16, codes_out [N, K/vec] uint8 or uint16.  Distances are accumulated in fp32 in vector
 * order with a fused multiply-add; ties go to the lowest index.  vec must be 2, 4 or 8.
 * No counterpart in the reference, whose harness multiplies random codes (bench.py:84): this is the
 * assignment step of the quantiser that produces the codes the GEMM path consumes.
 */
int vqgemm_encode_b(const void *w, const void *codebook, void *codes_out,
                    int64_t N, int64_t K, int32_t vec, int32_t entries,
                    int32_t n_codebooks, int32_t code_bits, void *stream);

/*
 * Element-wise pass behind a gate/up projection pair (the MLP shapes among the measured
 * configurations): out[m, n] = silu(gate_up[m, n]) * gate_up[m, N + n], gate_up [M, 2N] fp16 being
 * one fused VQ GEMM over the gate rows of W stacked on its up rows; silu(g) = g / (1 + exp(-g)),
 * fp32 arithmetic, one rounding to fp16.  No counterpart in the reference (its e2e_gemm has no
 * epilogue); for call sites that hold a gated MLP (vq_gemm_amd.nn.VQGatedMLP).
 */
int vqgemm_silu_mul(const void *gate_up, void *out, int64_t M, int64_t N, void *stream);

/*
 * Offline re-layout of a geometry-B code matrix for VQGEMM_VARIANT_DECODE_PACKED (the step before
 * the path; the reference keeps its w tensor as generated, bench.py:84, and has no counterpart).
 * The decode kernel's waves each own 256 k of 16 rows of W; in the plain [N, K/vec] matrix one wave
 * load is 16 pieces of 32 or 64 bytes in 16 different rows.  The packed matrix holds the same pieces
 * in the order the lanes ask for them,
 *     packed[n/16][s][t][q][n%16][c] = codes[n][(s*256 + t*kw)/vec + q*cpl + c],
 *     cpl = codes per lane load (16 bytes; 8 bytes for 8-vectors with 8-bit codes), c < cpl,
 *     kw = 4*cpl*vec (k per wave load), s < K/256, t < 256/kw, q < 4,
 * so that a wave load is one run of 512 or 1024 consecutive bytes.  Same size, codes unchanged.
 * inverse != 0 turns a packed matrix back into the plain one.  K % 256 == 0, N % 16 == 0, vec 2, 4
 * or 8, else VQGEMM_E_VARIANT; not in place.
 */
int vqgemm_pack_codes_b(const void *codes, void *codes_out, int64_t N, int64_t K, int32_t vec,
                        int32_t code_bits, int32_t inverse, void *stream);

/*
 * 1 when VQGEMM_VARIANT_DECODE_PACKED serves the shape (host only, no GPU call), 0 when it does
 * not, or a negative error for an invalid shape.
 */
int vqgemm_decode_packed_supports(int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries,
                                  int32_t n_codebooks, int32_t code_bits);

/*
 * The code-range contract, and the check for it.  Every code must be below `entries` (geometry A:
 * any byte is valid, its codebooks have 256 entries).  The fused kernels do not test codes: they
 * gather at code * entry size inside the workgroup's own LDS allocation (the GEMV kernel of 8-bit
 * codes reads zeros past a short table; the dequant and scalar kernels clamp to the last entry), so
 * a code at or past `entries` never touches foreign memory but gives a result that depends on the
 * kernel.  Callers that do not trust their codes run this first:
 *     *max_out = max(codes[0 .. count)), 0 for count == 0,
 * max_out being one uint32 in device memory (4-byte aligned), written on `stream`; the caller reads
 * it back and compares with `entries`.  One HBM pass over the codes.  The reference validates
 * nothing (strategy_3/naive/src.cu:42-54 prints runtime errors only); the torch modules of this
 * build run the check when VQGEMM_CHECK_CODES=1 is in the environment.
 */
int vqgemm_max_code(const void *codes, int64_t count, int32_t code_bits, void *max_out, void *stream);

/*
 * Plain fp16 GEMM o[M,N] = input[M,K] . w[K,N] (fp32 accumulate), the no-dequant control.
 * Replaces: torch::Tensor gemm(input, w) — reference bind.cpp:4,8, strategy_1/src.cu:171-265.
 */
int vqgemm_gemm_f16(const void *x, const void *w, void *y, int64_t M, int64_t K, int64_t N,
                    void *stream);

/*
 * Which kernel VQGEMM_VARIANT_AUTO resolves to for a geometry-B shape (host only, no GPU
 * call): returns a VQGEMM_VARIANT_* value, or a negative error for an invalid shape.
 */
int vqgemm_select_variant_b(int64_t M, int64_t K, int64_t N, int32_t vec, int32_t entries,
                            int32_t n_codebooks, int32_t code_bits);

/*
 * The constants of the cost models behind VQGEMM_VARIANT_AUTO (host only).  The compiled-in values were fitted
 * to measurements on one 256-CU MI355X; `python -m vq_gemm_amd.tune --fit` measures the box at hand and writes
 * a flat JSON object {"name": number, ...} that vqgemm_tuning_load reads (and that the library reads by itself,
 * once, from the file named by the environment variable VQGEMM_TUNING_FILE).  Names: vqgemm_tuning_name(i) for
 * 0 <= i < vqgemm_tuning_count(): per-tile and per-stage microseconds of the prefill tiles, per-tile
 * microseconds of the batched decode kernel, the limits between the GEMV kernels.  set/get return
 * VQGEMM_E_VARIANT for an unknown name; load returns the number of constants it set, or VQGEMM_E_NULL when the
 * file cannot be read.  No counterpart in the reference, whose tiling is compile-time macros
 * (strategy_1/src.cu:12-47).  Set them before launching from other threads.
 */
int vqgemm_tuning_count(void);
const char *vqgemm_tuning_name(int index);
int vqgemm_tuning_get(const char *name, double *value);
int vqgemm_tuning_set(const char *name, double value);
int vqgemm_tuning_load(const char *path);

/* Host string for a return code of this library (static storage). */
const char *vqgemm_error_string(int code);

/* Library version: major*10000 + minor*100 + patch. */
int vqgemm_version(void);

#ifdef __cplusplus
}
#endif
#endif /* VQ_GEMM_H */
