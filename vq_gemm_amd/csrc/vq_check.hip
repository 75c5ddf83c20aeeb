// Largest code of a code matrix, for callers that want the code-range contract checked (codes
// below the number of codebook entries) before they trust a result.  The reference checks nothing
// (strategy_3/naive/src.cu:42-54 only prints runtime errors); the fused kernels gather at
// code * entry size inside the workgroup's own LDS allocation and never test the code, so a code
// at or past `entries` gives an undefined result without touching foreign memory.  HBM-bound:
// one pass over the codes.
#include "vq_common.h"

namespace vq {

namespace {

__global__ __launch_bounds__(64) void clear_word_kernel(uint32_t *out) { if (threadIdx.x == 0) *out = 0u; }

__global__ __launch_bounds__(256) void clear_words_kernel(uint32_t *out, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) out[i] = 0u;
}

// 16-byte loads over the aligned body, scalar loads for the ragged head and tail.
template <typename CodeT>
__global__ __launch_bounds__(256) void max_code_kernel(const CodeT *__restrict__ codes, int64_t count, uint32_t *out)
{
    constexpr int kPer = 16 / (int)sizeof(CodeT);
    const uintptr_t addr = reinterpret_cast<uintptr_t>(codes);
    int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(CodeT));
    if (head > count) head = count;
    const int64_t chunks = (count - head) / kPer;
    const int64_t first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t m = 0;
    const uint4_t *body = reinterpret_cast<const uint4_t *>(codes + head);
    for (int64_t i = first; i < chunks; i += stride) {
        const uint4_t v = body[i];
#pragma unroll
        for (int d = 0; d < 4; d++) {
            if constexpr (sizeof(CodeT) == 1) {
                m = max(m, max(max(v[d] & 0xffu, (v[d] >> 8) & 0xffu), max((v[d] >> 16) & 0xffu, v[d] >> 24)));
            } else {
                m = max(m, max(v[d] & 0xffffu, v[d] >> 16));
            }
        }
    }
    for (int64_t i = first; i < head; i += stride) m = max(m, (uint32_t)codes[i]);
    for (int64_t i = head + chunks * kPer + first; i < count; i += stride) m = max(m, (uint32_t)codes[i]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, 64));
    if ((threadIdx.x & 63) == 0 && m != 0) atomicMax(out, m);
}

}  // namespace

hipError_t launch_clear_words(uint32_t *words, int64_t n, hipStream_t s)
{
    if (n <= 0) return hipSuccess;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 64) blocks = 64;
    hipLaunchKernelGGL(clear_words_kernel, dim3((unsigned)blocks), dim3(256), 0, s, words, n);
    return hipGetLastError();
}

hipError_t launch_max_code(const void *codes, int64_t count, int code_bits, uint32_t *out, hipStream_t s)
{
    hipLaunchKernelGGL(clear_word_kernel, dim3(1), dim3(64), 0, s, out);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || count == 0) return e;
    int64_t blocks = (count / (code_bits == 8 ? 16 : 8) + 255) / 256;
    const int64_t cap = (int64_t)device_cu_count() * 8;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    if (code_bits == 8)
        hipLaunchKernelGGL(max_code_kernel<uint8_t>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const uint8_t *>(codes), count, out);
    else
        hipLaunchKernelGGL(max_code_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const uint16_t *>(codes), count, out);
    return hipGetLastError();
}

}  // namespace vq
