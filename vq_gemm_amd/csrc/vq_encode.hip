// Nearest-codeword encoder, geometry B: codes[n, j] = the entry of the row's codebook closest to
// W[n, j*vec .. j*vec+vec) in squared Euclidean distance.  This is the assignment step of a
// vector quantiser, the step before the GEMM path (the reference only ever multiplies random codes,
// bench.py:84).
//
// The arithmetic is fixed so that the result is reproducible bit for bit: operands are widened to
// fp32, the distance is accumulated element by element in vector order with a fused multiply-add
// (acc = fma(d, d, acc), d = w - c), entry 0 starts as the best and a later entry replaces it only
// when its distance is strictly smaller (ties keep the lowest index; a NaN distance never wins).
//
// The rows of one codebook are contiguous in W and in the codes, so a codebook's block is walked as
// a flat array of vectors.  A workgroup keeps a chunk of the codebook in the LDS as fp32; all lanes
// read the same entry at a time (a broadcast), each thread scores four vectors against it.
#include "vq_common.h"

namespace vq {

namespace {

constexpr int kEncThreads = 256;
constexpr int kEncPerThread = 4;                 // vectors per thread
constexpr int kEncChunkFloats = 16384;           // fp32 codebook chunk in the LDS: 64 KB

template <int VEC, typename CodeT>
__global__ __launch_bounds__(kEncThreads) void encode_b_kernel(const half_t *__restrict__ w,
                                                               const half_t *__restrict__ cb,
                                                               CodeT *__restrict__ codes, int64_t vectors_per_cb,
                                                               int entries, int wgs_per_cb)
{
    __shared__ __align__(16) float table[kEncChunkFloats];
    constexpr int kChunkEntries = kEncChunkFloats / VEC;
    const int g = blockIdx.x / wgs_per_cb, part = blockIdx.x % wgs_per_cb;
    const half_t *wg_w = w + (int64_t)g * vectors_per_cb * VEC;
    CodeT *wg_codes = codes + (int64_t)g * vectors_per_cb;
    const half_t *book = cb + (int64_t)g * entries * VEC;

    for (int64_t base = (int64_t)part * kEncThreads * kEncPerThread; base < vectors_per_cb;
         base += (int64_t)wgs_per_cb * kEncThreads * kEncPerThread) {
        float v[kEncPerThread][VEC];
        float best[kEncPerThread];
        uint32_t arg[kEncPerThread];
#pragma unroll
        for (int u = 0; u < kEncPerThread; u++) {
            const int64_t idx = base + u * kEncThreads + threadIdx.x;
            const int64_t src = idx < vectors_per_cb ? idx : vectors_per_cb - 1;
#pragma unroll
            for (int t = 0; t < VEC; t++) v[u][t] = (float)wg_w[src * VEC + t];
            best[u] = 0.f;
            arg[u] = 0;
        }
        for (int e0 = 0; e0 < entries; e0 += kChunkEntries) {
            const int n_e = entries - e0 < kChunkEntries ? entries - e0 : kChunkEntries;
            __syncthreads();  // the previous chunk has been read by every thread
            for (int i = threadIdx.x; i < n_e * VEC; i += kEncThreads) table[i] = (float)book[(int64_t)e0 * VEC + i];
            __syncthreads();
            for (int e = 0; e < n_e; e++) {
                float c[VEC];
#pragma unroll
                for (int t = 0; t < VEC; t++) c[t] = table[e * VEC + t];
#pragma unroll
                for (int u = 0; u < kEncPerThread; u++) {
                    float acc = 0.f;
#pragma unroll
                    for (int t = 0; t < VEC; t++) {
                        const float d = v[u][t] - c[t];
                        acc = __builtin_fmaf(d, d, acc);
                    }
                    // entry 0 is taken as it is; later entries must be strictly closer
                    const bool take = (e0 + e == 0) || acc < best[u];
                    best[u] = take ? acc : best[u];
                    arg[u] = take ? (uint32_t)(e0 + e) : arg[u];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kEncPerThread; u++) {
            const int64_t idx = base + u * kEncThreads + threadIdx.x;
            if (idx < vectors_per_cb) wg_codes[idx] = (CodeT)arg[u];
        }
    }
}

template <int VEC, typename CodeT>
hipError_t encode_b_typed(const half_t *w, const ProblemB &p, void *codes_out, hipStream_t s)
{
    const int64_t vectors_per_cb = (int64_t)p.rows_per_cb * (p.K / VEC);
    if (vectors_per_cb == 0) return hipSuccess;
    // enough workgroups per codebook to fill the device a few times over, none without work
    const int64_t want = ((int64_t)device_cu_count() * 8 + p.n_codebooks - 1) / p.n_codebooks;
    const int64_t have = (vectors_per_cb + kEncThreads * kEncPerThread - 1) / (kEncThreads * kEncPerThread);
    const int wgs_per_cb = (int)(want < have ? want : have);
    hipLaunchKernelGGL((encode_b_kernel<VEC, CodeT>), dim3((unsigned)(wgs_per_cb * p.n_codebooks)), dim3(kEncThreads), 0, s, w,
                       p.cb, static_cast<CodeT *>(codes_out), vectors_per_cb, p.entries, wgs_per_cb);
    return hipGetLastError();
}

}  // namespace

bool encode_supports(const ProblemB &p) { return p.vec == 2 || p.vec == 4 || p.vec == 8; }

hipError_t launch_encode_b(const half_t *w, const ProblemB &p, void *codes_out, hipStream_t s)
{
    if (!encode_supports(p)) return hipErrorInvalidValue;
    const bool u8 = p.code_bits == 8;
    switch (p.vec) {
    case 8: return u8 ? encode_b_typed<8, uint8_t>(w, p, codes_out, s) : encode_b_typed<8, uint16_t>(w, p, codes_out, s);
    case 4: return u8 ? encode_b_typed<4, uint8_t>(w, p, codes_out, s) : encode_b_typed<4, uint16_t>(w, p, codes_out, s);
    default: return u8 ? encode_b_typed<2, uint8_t>(w, p, codes_out, s) : encode_b_typed<2, uint16_t>(w, p, codes_out, s);
    }
}

}  // namespace vq
