/*
 * vq_gemm_ref.h — C ABI of libvqgemm_ref.so, the library-GEMM baseline.
 *
 * A hipBLASLt fp16 GEMM with fp32 accumulation on uncompressed weights: what the fused VQ
 * kernels are compared against.  Kept in its own shared object so that libvqgemm.so has no
 * BLAS dependency.  Device pointers, row-major, `stream` is a hipStream_t as void*.
 * Returns 0, a negative VQREF_E_* code, or 1000 + hipblasStatus_t / a positive hipError_t.
 */
#ifndef VQ_GEMM_REF_H
#define VQ_GEMM_REF_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VQREF_E_ARG (-1)        /* NULL pointer or negative size */
#define VQREF_E_NOALGO (-2)     /* hipBLASLt returned no algorithm for the shape */

/*
 * y[M,N] = x[M,K] . W   with W = w[K,N] (w_is_nk == 0) or W = w[N,K]^T (w_is_nk != 0).
 * Replaces: torch::Tensor gemm(input, w) of the reference's cuBLAS module,
 * ref_gemm/cublas_gemm_fp16.cu:15-48 (which computes in fp16; this one accumulates in fp32).
 * The handle, the algorithm chosen for a shape and a 64 MiB workspace are cached per device.
 * The first call on a shape (outside stream capture) times up to 32 of the library's heuristic
 * answers on the caller's operands with cold caches (it synchronises the stream and allocates a
 * 512 MiB scratch buffer for the duration) and keeps the fastest; VQREF_TUNE=0 in the environment
 * keeps the first answer instead.
 */
int vqref_gemm_f16(const void *x, const void *w, void *y, int64_t M, int64_t K, int64_t N,
                   int32_t w_is_nk, void *stream);

/*
 * What the first call on a shape found (host only): how many heuristic answers were timed
 * (1 = none, the first answer was kept), which one was kept, its time and the time of the
 * library's first answer, microseconds, cold caches.  VQREF_E_NOALGO when the shape has not
 * been run on the current device.  Any output pointer may be NULL.  No counterpart in the
 * reference, which takes CUBLAS_GEMM_DEFAULT (ref_gemm/cublas_gemm_fp16.cu:46).
 */
int vqref_tuning_info(int64_t M, int64_t K, int64_t N, int32_t w_is_nk, int32_t *candidates,
                      int32_t *chosen, float *best_us, float *first_us);

const char *vqref_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* VQ_GEMM_REF_H */
