// Plain fp16 GEMM on the matrix cores, any shape: the kernel behind the tiled one of
// vq_gemm_tiled.hip, for short X and for shapes that one does not take.
//   NN: y[M,N] = x[M,K] . w[K,N]      NT: y[M,N] = x[M,K] . w[N,K]^T
// 128x128 workgroup tile, 4 waves of 64x64, v_mfma_f32_32x32x16_f16, 32-deep K steps staged
// through padded LDS rows with register prefetch of the next step.  Shape-agnostic (edges
// are zero filled / masked).  fp32 accumulation, one rounding to fp16.
#include "vq_common.h"

namespace vq {

namespace {

constexpr int TM = 128, TN = 128, TK = 32;
constexpr int kRowBytes = 80;  // 64 bytes of data + 16 of padding: conflict-free 16-byte column reads
constexpr int kTileBytes = 128 * kRowBytes;

// 8 consecutive halves of row `r` starting at column `c` of a [rows, cols] matrix, zero filled.
__device__ __forceinline__ uint4_t load8(const half_t *base, int r, int c, int rows, int cols, bool vec_ok)
{
    uint4_t v = {0u, 0u, 0u, 0u};
    if (r >= rows || c >= cols) return v;
    const half_t *p = base + (int64_t)r * cols + c;
    if (vec_ok && c + 8 <= cols) return ld_global_16(p);
    union { uint4_t u; half_t h[8]; } t;
    t.u = v;
    for (int i = 0; i < 8; i++)
        if (c + i < cols) t.h[i] = p[i];
    return t.u;
}

template <bool W_IS_KN>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const half_t *__restrict__ x,
                                                         const half_t *__restrict__ w,
                                                         half_t *__restrict__ y, int M, int K, int N,
                                                         bool x_vec, bool w_vec)
{
    __shared__ __align__(16) uint8_t xs[kTileBytes];
    __shared__ __align__(16) uint8_t ws[kTileBytes];
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, kg = lane >> 5;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;

    float16_t acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[a][b][r] = 0.f;

    uint4_t xr[2], wr[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int q = i * 256 + tid;
            xr[i] = load8(x, m0 + (q >> 2), k0 + (q & 3) * 8, M, K, x_vec);
            if constexpr (W_IS_KN)
                wr[i] = load8(w, k0 + (q >> 4), n0 + (q & 15) * 8, K, N, w_vec);
            else
                wr[i] = load8(w, n0 + (q >> 2), k0 + (q & 3) * 8, N, K, w_vec);
        }
    };
    auto park = [&]() {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int q = i * 256 + tid;
            *reinterpret_cast<uint4_t *>(xs + (q >> 2) * kRowBytes + (q & 3) * 16) = xr[i];
            if constexpr (W_IS_KN) {
                // transpose on the way in: 8 consecutive n of one k -> 8 rows of the n-major tile
                union { uint4_t u; half_t h[8]; } t;
                t.u = wr[i];
                const int krow = q >> 4, nc = (q & 15) * 8;
#pragma unroll
                for (int j = 0; j < 8; j++)
                    *reinterpret_cast<half_t *>(ws + (nc + j) * kRowBytes + krow * 2) = t.h[j];
            } else {
                *reinterpret_cast<uint4_t *>(ws + (q >> 2) * kRowBytes + (q & 3) * 16) = wr[i];
            }
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += TK) {
        __syncthreads();  // previous step's reads are done
        park();
        __syncthreads();
        if (k0 + TK < K) fetch(k0 + TK);
#pragma unroll
        for (int s = 0; s < 2; s++) {
            half8_t wop[2], xop[2];
#pragma unroll
            for (int b = 0; b < 2; b++) {
                wop[b] = *reinterpret_cast<const half8_t *>(ws + (wn * 64 + b * 32 + l32) * kRowBytes + (s * 2 + kg) * 16);
                xop[b] = *reinterpret_cast<const half8_t *>(xs + (wm * 64 + b * 32 + l32) * kRowBytes + (s * 2 + kg) * 16);
            }
#pragma unroll
            for (int nb = 0; nb < 2; nb++)
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
                    acc[nb][mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wop[nb], xop[mb], acc[nb][mb], 0, 0, 0);
        }
    }

    // D[i][j]: i = n offset = 8*(r/4) + 4*kg + r%4, j = m offset = l32.
#pragma unroll
    for (int mb = 0; mb < 2; mb++) {
        const int m = m0 + wm * 64 + mb * 32 + l32;
        if (m >= M) continue;
#pragma unroll
        for (int nb = 0; nb < 2; nb++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int n = n0 + wn * 64 + nb * 32 + 8 * q + 4 * kg;
                half_t *dst = y + (int64_t)m * N + n;
                if ((N & 3) == 0 && n + 3 < N && ((uintptr_t)y & 7) == 0) {
                    half4_t h = {(half_t)acc[nb][mb][4 * q], (half_t)acc[nb][mb][4 * q + 1],
                                 (half_t)acc[nb][mb][4 * q + 2], (half_t)acc[nb][mb][4 * q + 3]};
                    *reinterpret_cast<half4_t *>(dst) = h;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (n + r < N) dst[r] = (half_t)acc[nb][mb][4 * q + r];
                }
            }
    }
}

template <bool W_IS_KN>
hipError_t launch_plain(const half_t *x, const half_t *w, half_t *y, int M, int K, int N, hipStream_t s)
{
    if (M == 0 || N == 0) return hipSuccess;
    const bool x_vec = (K % 8 == 0) && (((uintptr_t)x & 15) == 0);
    const int w_cols = W_IS_KN ? N : K;
    const bool w_vec = (w_cols % 8 == 0) && (((uintptr_t)w & 15) == 0);
    dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
    hipLaunchKernelGGL((gemm_plain_kernel<W_IS_KN>), grid, dim3(256), 0, s, x, w, y, M, K, N, x_vec, w_vec);
    return hipGetLastError();
}

}  // namespace

// The tiled kernel serves every height it supports (its shortest tile has 128 rows, like the kernel
// in this file, and is several times faster); the threshold stays as a build-time switch for
// measurements.
#ifndef VQ_TILED_MIN_M
#define VQ_TILED_MIN_M 1
#endif

hipError_t launch_gemm_nn(const half_t *x, const half_t *w, half_t *y, int M, int K, int N, hipStream_t s)
{
    if (M >= VQ_TILED_MIN_M && gemm_tiled_supports(x, w, M, K, N, true)) return launch_gemm_tiled(x, w, y, M, K, N, true, s);
    return launch_plain<true>(x, w, y, M, K, N, s);
}

hipError_t launch_gemm_nt(const half_t *x, const half_t *w, half_t *y, int M, int K, int N, hipStream_t s)
{
    if (M >= VQ_TILED_MIN_M && gemm_tiled_supports(x, w, M, K, N, false)) return launch_gemm_tiled(x, w, y, M, K, N, false, s);
    return launch_plain<false>(x, w, y, M, K, N, s);
}

}  // namespace vq
