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
 */
int vqref_gemm_f16(const void *x, const void *w, void *y, int64_t M, int64_t K, int64_t N,
                   int32_t w_is_nk, void *stream);

const char *vqref_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* VQ_GEMM_REF_H */
