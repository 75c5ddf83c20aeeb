// Element-wise pass behind a gate/up projection pair: out[m, n] = silu(a[m, n]) * a[m, N + n] for
// a [M, 2N] (the product of X with the gate rows stacked on the up rows of W, one fused VQ GEMM).
// silu(g) = g / (1 + exp(-g)); both factors are widened to fp32, the product is rounded to fp16
// once.  HBM-bound: 6 bytes per output element.
#include "vq_common.h"

namespace vq {

namespace {

__device__ __forceinline__ float silu(float g) { return silu_f32(g); }

// VEC8: rows are whole 16-byte chunks (N % 8 == 0, 16-byte aligned pointers): one chunk of the gate
// half and the matching chunk of the up half per thread and step.
// INTERLEAVED: gate and up columns alternate in groups of 16 (columns 32g .. 32g+15 gate, 32g+16 .. 32g+31
// up, the layout of the fused kernels' gated epilogue; N % 16 == 0) instead of lying in the two halves of a row.
template <bool VEC8, bool INTERLEAVED>
__global__ __launch_bounds__(256) void silu_mul_kernel(const half_t *__restrict__ a, half_t *__restrict__ out,
                                                       int64_t M, int64_t N)
{
    auto gate_col = [&](int64_t n) { return INTERLEAVED ? 32 * (n >> 4) + (n & 15) : n; };
    constexpr int64_t kUpStep = 16;  // interleaved: the up column of a gate column
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if constexpr (VEC8) {
        const int64_t chunks = N / 8, total = M * chunks;
        for (int64_t i = first; i < total; i += stride) {
            const int64_t m = i / chunks, c = i - m * chunks;
            const int64_t gc = gate_col(c * 8);
            const half8_t g = *reinterpret_cast<const half8_t *>(a + m * 2 * N + gc);
            const half8_t u = *reinterpret_cast<const half8_t *>(a + m * 2 * N + gc + (INTERLEAVED ? kUpStep : N));
            half8_t r;
#pragma unroll
            for (int t = 0; t < 8; t++) r[t] = (half_t)(silu((float)g[t]) * (float)u[t]);
            *reinterpret_cast<half8_t *>(out + m * N + c * 8) = r;
        }
    } else {
        const int64_t total = M * N;
        for (int64_t i = first; i < total; i += stride) {
            const int64_t m = i / N, n = i - m * N;
            const int64_t gc = gate_col(n);
            out[i] = (half_t)(silu((float)a[m * 2 * N + gc]) * (float)a[m * 2 * N + gc + (INTERLEAVED ? kUpStep : N)]);
        }
    }
}

}  // namespace

hipError_t launch_silu_mul(const half_t *a, half_t *out, int64_t M, int64_t N, hipStream_t s, bool interleaved)
{
    if (M == 0 || N == 0) return hipSuccess;
    if (interleaved && N % 16 != 0) return hipErrorInvalidValue;
    const bool vec8 = N % 8 == 0 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const int64_t work = vec8 ? M * (N / 8) : M * N;
    int64_t blocks = (work + 255) / 256;
    const int64_t cap = (int64_t)device_cu_count() * 16;
    if (blocks > cap) blocks = cap;
    const dim3 grid((unsigned)blocks), block(256);
    if (interleaved) {
        if (vec8) hipLaunchKernelGGL((silu_mul_kernel<true, true>), grid, block, 0, s, a, out, M, N);
        else hipLaunchKernelGGL((silu_mul_kernel<false, true>), grid, block, 0, s, a, out, M, N);
    } else {
        if (vec8) hipLaunchKernelGGL((silu_mul_kernel<true, false>), grid, block, 0, s, a, out, M, N);
        else hipLaunchKernelGGL((silu_mul_kernel<false, false>), grid, block, 0, s, a, out, M, N);
    }
    return hipGetLastError();
}

}  // namespace vq
