// Stand-alone dequantisation kernels: codes + codebook -> fp16 weights in HBM.
// Pure indexing and bit copies, so results are bit-exact by construction.  The kernels are
// bound by the HBM write stream (16 B written per code byte read for vec = 8).
#include "vq_common.h"

namespace vq {

// ---- geometry B ------------------------------------------------------------------------
// One thread per code; consecutive threads take consecutive codes of a row, so each wave
// stores 64 * VEC * 2 contiguous bytes.  Codebooks stay in global memory: they are a few
// KB and every lookup after the first hits the L2.
template <int VEC, typename CodeT>
__global__ __launch_bounds__(256) void dequant_b_kernel(const CodeT *__restrict__ codes,
                                                        const half_t *__restrict__ cb,
                                                        half_t *__restrict__ w, int N, int J,
                                                        int entries, int rows_per_cb)
{
    typedef half_t vec_t __attribute__((ext_vector_type(VEC)));
    const int64_t total = (int64_t)N * J;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int n = (int)(i / J);
        uint32_t c = codes[i];
        c = c < (uint32_t)entries ? c : (uint32_t)entries - 1;  // memory safety only
        const half_t *src = cb + ((int64_t)(n / rows_per_cb) * entries + c) * VEC;
        *reinterpret_cast<vec_t *>(w + i * VEC) = *reinterpret_cast<const vec_t *>(src);
    }
}

// Any vector length (scalar copies).
template <typename CodeT>
__global__ __launch_bounds__(256) void dequant_b_anyvec_kernel(const CodeT *__restrict__ codes,
                                                               const half_t *__restrict__ cb,
                                                               half_t *__restrict__ w, int N, int J,
                                                               int vec, int entries, int rows_per_cb)
{
    const int64_t total = (int64_t)N * J;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int n = (int)(i / J);
        uint32_t c = codes[i];
        c = c < (uint32_t)entries ? c : (uint32_t)entries - 1;
        const half_t *src = cb + ((int64_t)(n / rows_per_cb) * entries + c) * vec;
        for (int t = 0; t < vec; t++) w[i * vec + t] = src[t];
    }
}

template <typename CodeT>
static hipError_t dequant_b_typed(const ProblemB &p, half_t *w_out, hipStream_t s)
{
    const int J = p.K / p.vec;
    const int64_t total = (int64_t)p.N * J;
    if (total == 0) return hipSuccess;
    int64_t blocks = (total + 255) / 256;
    const int64_t cap = (int64_t)device_cu_count() * 32;
    if (blocks > cap) blocks = cap;
    const CodeT *codes = static_cast<const CodeT *>(p.codes);
    dim3 grid((unsigned)blocks), block(256);
    // Vector copies need codeword-aligned source and destination; otherwise copy scalars.
    const bool aligned = (((uintptr_t)w_out | (uintptr_t)p.cb) % (uintptr_t)(p.vec * 2)) == 0;
    switch (aligned ? p.vec : 0) {
    case 2: hipLaunchKernelGGL((dequant_b_kernel<2, CodeT>), grid, block, 0, s, codes, p.cb, w_out, p.N, J, p.entries, p.rows_per_cb); break;
    case 4: hipLaunchKernelGGL((dequant_b_kernel<4, CodeT>), grid, block, 0, s, codes, p.cb, w_out, p.N, J, p.entries, p.rows_per_cb); break;
    case 8: hipLaunchKernelGGL((dequant_b_kernel<8, CodeT>), grid, block, 0, s, codes, p.cb, w_out, p.N, J, p.entries, p.rows_per_cb); break;
    default: hipLaunchKernelGGL((dequant_b_anyvec_kernel<CodeT>), grid, block, 0, s, codes, p.cb, w_out, p.N, J, p.vec, p.entries, p.rows_per_cb); break;
    }
    return hipGetLastError();
}

hipError_t launch_dequant_b(const ProblemB &p, half_t *w_out, hipStream_t s)
{
    return p.code_bits == 8 ? dequant_b_typed<uint8_t>(p, w_out, s) : dequant_b_typed<uint16_t>(p, w_out, s);
}

// ---- geometry A ------------------------------------------------------------------------
// W_dec[k, 2n + r] = cb[n/4][w[k,n]][r]: one thread per code writes one 4-byte codeword;
// a wave writes 256 contiguous bytes of a W_dec row.
__global__ __launch_bounds__(256) void dequant_a_kernel(const uint8_t *__restrict__ w,
                                                        const half_t *__restrict__ cb,
                                                        half_t *__restrict__ out, int K, int Nc)
{
    const int64_t total = (int64_t)K * Nc;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int n = (int)(i % Nc);
        const uint32_t c = w[i];
        const half_t *src = cb + ((int64_t)(n >> 2) * 256 + c) * 2;
        *reinterpret_cast<half2_t *>(out + i * 2) = *reinterpret_cast<const half2_t *>(src);
    }
}

hipError_t launch_dequant_a(const ProblemA &p, half_t *w_out, hipStream_t s)
{
    const int64_t total = (int64_t)p.K * p.Nc;
    if (total == 0) return hipSuccess;
    int64_t blocks = (total + 255) / 256;
    const int64_t cap = (int64_t)device_cu_count() * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(dequant_a_kernel, dim3((unsigned)blocks), dim3(256), 0, s, p.w, p.cb, w_out, p.K, p.Nc);
    return hipGetLastError();
}

}  // namespace vq
