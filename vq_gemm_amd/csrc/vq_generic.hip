// Shape-agnostic fused VQ-GEMM kernels: one output element per thread, scalar loads,
// sequential fp32 accumulation.  They serve every shape the tiled kernels reject (odd K,
// unusual vector lengths, codebooks too large for the LDS) and act as an independent
// on-device statement of the math in the tests.  Not tuned.
#include "vq_common.h"

namespace vq {

template <typename CodeT>
__global__ __launch_bounds__(256) void generic_b_kernel(const half_t *__restrict__ x,
                                                        const CodeT *__restrict__ codes,
                                                        const half_t *__restrict__ cb,
                                                        half_t *__restrict__ y,
                                                        const half_t *__restrict__ bias, int M, int K, int N,
                                                        int vec, int entries, int rows_per_cb)
{
    // blockDim = (64, 4): x index -> n (coalesced y stores), y index -> m.
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= N) return;
    const int J = K / vec;
    const half_t *book = cb + (int64_t)(n / rows_per_cb) * entries * vec;
    const CodeT *crow = codes + (int64_t)n * J;
    const float b = bias ? (float)bias[n] : 0.0f;
    for (int m = blockIdx.y * blockDim.y + threadIdx.y; m < M; m += gridDim.y * blockDim.y) {
        const half_t *xrow = x + (int64_t)m * K;
        float acc = 0.0f;
        for (int j = 0; j < J; j++) {
            uint32_t c = crow[j];
            c = c < (uint32_t)entries ? c : (uint32_t)entries - 1;  // memory safety only
            const half_t *cw = book + (int64_t)c * vec;
            for (int t = 0; t < vec; t++) acc += (float)xrow[j * vec + t] * (float)cw[t];
        }
        y[(int64_t)m * N + n] = (half_t)(acc + b);
    }
}

// Gated epilogue: one thread per output column computes the gate and the up product (rows 32g + r and
// 32g + 16 + r of the interleaved W for output column 16g + r).
template <typename CodeT>
__global__ __launch_bounds__(256) void generic_b_gated_kernel(const half_t *__restrict__ x,
                                                              const CodeT *__restrict__ codes,
                                                              const half_t *__restrict__ cb,
                                                              half_t *__restrict__ y,
                                                              const half_t *__restrict__ bias, int M, int K, int N,
                                                              int vec, int entries, int rows_per_cb)
{
    const int o = blockIdx.x * blockDim.x + threadIdx.x;
    if (o >= N / 2) return;
    const int J = K / vec;
    const int ng = 32 * (o >> 4) + (o & 15), nu = ng + 16;
    const half_t *book_g = cb + (int64_t)(ng / rows_per_cb) * entries * vec;
    const half_t *book_u = cb + (int64_t)(nu / rows_per_cb) * entries * vec;
    const CodeT *crow_g = codes + (int64_t)ng * J, *crow_u = codes + (int64_t)nu * J;
    const float bg = bias ? (float)bias[ng] : 0.0f, bu = bias ? (float)bias[nu] : 0.0f;
    for (int m = blockIdx.y * blockDim.y + threadIdx.y; m < M; m += gridDim.y * blockDim.y) {
        const half_t *xrow = x + (int64_t)m * K;
        float ag = 0.0f, au = 0.0f;
        for (int j = 0; j < J; j++) {
            uint32_t cg = crow_g[j], cu = crow_u[j];
            cg = cg < (uint32_t)entries ? cg : (uint32_t)entries - 1;  // memory safety only
            cu = cu < (uint32_t)entries ? cu : (uint32_t)entries - 1;
            const half_t *wg = book_g + (int64_t)cg * vec, *wu = book_u + (int64_t)cu * vec;
            for (int t = 0; t < vec; t++) {
                const float xv = (float)xrow[j * vec + t];
                ag += xv * (float)wg[t];
                au += xv * (float)wu[t];
            }
        }
        y[(int64_t)m * (N / 2) + o] = (half_t)(silu_f32(ag + bg) * (au + bu));
    }
}

hipError_t launch_generic_b(const ProblemB &p, hipStream_t s)
{
    if (p.M == 0 || p.N == 0) return hipSuccess;
    if (p.gated) {
        dim3 block(64, 4);
        dim3 grid((p.N / 2 + 63) / 64, (unsigned)(((p.M + 3) / 4) < 32768 ? (p.M + 3) / 4 : 32768));
        if (p.code_bits == 8)
            hipLaunchKernelGGL((generic_b_gated_kernel<uint8_t>), grid, block, 0, s, p.x, static_cast<const uint8_t *>(p.codes),
                               p.cb, p.y, p.bias, p.M, p.K, p.N, p.vec, p.entries, p.rows_per_cb);
        else
            hipLaunchKernelGGL((generic_b_gated_kernel<uint16_t>), grid, block, 0, s, p.x, static_cast<const uint16_t *>(p.codes),
                               p.cb, p.y, p.bias, p.M, p.K, p.N, p.vec, p.entries, p.rows_per_cb);
        return hipGetLastError();
    }
    dim3 block(64, 4);
    dim3 grid((p.N + 63) / 64, (unsigned)(((p.M + 3) / 4) < 32768 ? (p.M + 3) / 4 : 32768));
    if (p.code_bits == 8)
        hipLaunchKernelGGL((generic_b_kernel<uint8_t>), grid, block, 0, s, p.x, static_cast<const uint8_t *>(p.codes),
                           p.cb, p.y, p.bias, p.M, p.K, p.N, p.vec, p.entries, p.rows_per_cb);
    else
        hipLaunchKernelGGL((generic_b_kernel<uint16_t>), grid, block, 0, s, p.x, static_cast<const uint16_t *>(p.codes),
                           p.cb, p.y, p.bias, p.M, p.K, p.N, p.vec, p.entries, p.rows_per_cb);
    return hipGetLastError();
}

// Geometry A: out[m, 2n + r] = sum_k x[m,k] * cb[n/4][w[k,n]][r].  One thread per code
// column computes both outputs of the codeword.
__global__ __launch_bounds__(256) void generic_a_kernel(const half_t *__restrict__ x,
                                                        const uint8_t *__restrict__ w,
                                                        const half_t *__restrict__ cb,
                                                        half_t *__restrict__ y, int M, int K, int Nc)
{
    const int n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= Nc) return;
    const half_t *book = cb + (int64_t)(n >> 2) * 256 * 2;
    for (int m = blockIdx.y * blockDim.y + threadIdx.y; m < M; m += gridDim.y * blockDim.y) {
        const half_t *xrow = x + (int64_t)m * K;
        float a0 = 0.0f, a1 = 0.0f;
        for (int k = 0; k < K; k++) {
            const uint32_t c = w[(int64_t)k * Nc + n];
            const float xv = (float)xrow[k];
            a0 += xv * (float)book[c * 2];
            a1 += xv * (float)book[c * 2 + 1];
        }
        y[(int64_t)m * (2 * Nc) + 2 * n] = (half_t)a0;
        y[(int64_t)m * (2 * Nc) + 2 * n + 1] = (half_t)a1;
    }
}

hipError_t launch_generic_a(const ProblemA &p, hipStream_t s)
{
    if (p.M == 0 || p.Nc == 0) return hipSuccess;
    dim3 block(64, 4);
    dim3 grid((p.Nc + 63) / 64, (unsigned)(((p.M + 3) / 4) < 32768 ? (p.M + 3) / 4 : 32768));
    hipLaunchKernelGGL(generic_a_kernel, grid, block, 0, s, p.x, p.w, p.cb, p.y, p.M, p.K, p.Nc);
    return hipGetLastError();
}

}  // namespace vq
