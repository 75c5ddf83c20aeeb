// hipBLASLt fp16 GEMM (fp32 accumulate) on uncompressed weights: the vendor baseline the
// fused VQ kernels are measured against.  Takes the place of the reference's cuBLAS module
// (ref_gemm/cublas_gemm_fp16.cu:15-48), which created a handle per call and never freed it;
// here the handle, workspace and per-shape algorithm are cached per device.
//
// The algorithm of a shape is not the library's first heuristic answer: the first call on a
// shape asks for up to kMaxCandidates answers, times each on the caller's own operands (cold
// caches: a scratch buffer larger than the last-level cache is overwritten before every timed
// launch) and keeps the fastest.  A baseline is only worth comparing against when it is the
// best the vendor library can do on the shape.
#include "../../include/vq_gemm_ref.h"

#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdlib>
#include <map>
#include <mutex>
#include <tuple>

namespace {

constexpr size_t kWorkspaceBytes = 64ull << 20;
constexpr int kMaxCandidates = 32;
constexpr size_t kFlushBytes = 512ull << 20;  // larger than L2 + the 256 MB last-level cache
constexpr int kTimedRuns = 3;

struct Choice {
    hipblasLtMatmulAlgo_t algo;
    int candidates = 1;      // heuristic answers that were timed (1: not tuned)
    int chosen = 0;          // index of the one kept, in the library's own order
    float best_us = 0.f;     // its time, cold caches (0: not tuned)
    float first_us = 0.f;    // the time of the library's first answer
};

struct DeviceState {
    hipblasLtHandle_t handle = nullptr;
    void *workspace = nullptr;
    std::map<std::tuple<int64_t, int64_t, int64_t, int>, Choice> algos;
};

std::mutex g_mu;
std::map<int, DeviceState> g_state;

int blas_rc(hipblasStatus_t st) { return st == HIPBLAS_STATUS_SUCCESS ? 0 : 1000 + (int)st; }

bool tuning_enabled()
{
    const char *e = std::getenv("VQREF_TUNE");
    return !(e && e[0] == '0');
}

// Time every heuristic answer on the caller's operands and return the index of the fastest
// (-1 when timing is impossible: then the caller keeps the first answer).
int pick_fastest(DeviceState &st, hipblasLtMatmulDesc_t desc, hipblasLtMatrixLayout_t la, hipblasLtMatrixLayout_t lb,
                 hipblasLtMatrixLayout_t lc, const void *x, const void *w, void *y,
                 const hipblasLtMatmulHeuristicResult_t *res, int found, hipStream_t stream, float *best_us,
                 float *first_us)
{
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return -1;
    void *flush = nullptr;
    if (hipMalloc(&flush, kFlushBytes) != hipSuccess) {
        (void)hipGetLastError();
        flush = nullptr;  // timed warm then
    }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
        if (e0) (void)hipEventDestroy(e0);
        if (flush) (void)hipFree(flush);
        return -1;
    }
    const float alpha = 1.0f, beta = 0.0f;
    int best = -1;
    *best_us = 0.f;
    *first_us = 0.f;
    for (int i = 0; i < found; i++) {
        if (res[i].state != HIPBLAS_STATUS_SUCCESS || res[i].workspaceSize > kWorkspaceBytes) continue;
        float t_min = 0.f;
        bool ok = true;
        for (int r = 0; r < kTimedRuns + 1 && ok; r++) {  // the first run is not counted
            if (flush) ok = hipMemsetAsync(flush, r, kFlushBytes, stream) == hipSuccess;
            ok = ok && hipEventRecord(e0, stream) == hipSuccess;
            ok = ok && hipblasLtMatmul(st.handle, desc, &alpha, w, la, x, lb, &beta, y, lc, y, lc, &res[i].algo, st.workspace,
                                       kWorkspaceBytes, stream) == HIPBLAS_STATUS_SUCCESS;
            ok = ok && hipEventRecord(e1, stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess;
            float ms = 0.f;
            ok = ok && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
            if (ok && r > 0 && (t_min == 0.f || ms < t_min)) t_min = ms;
        }
        if (!ok) {
            (void)hipGetLastError();
            continue;
        }
        if (i == 0) *first_us = t_min * 1e3f;
        if (best < 0 || t_min * 1e3f < *best_us) {
            best = i;
            *best_us = t_min * 1e3f;
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (flush) (void)hipFree(flush);
    return best;
}

}  // namespace

extern "C" {

const char *vqref_error_string(int code)
{
    if (code == 0) return "success";
    if (code == VQREF_E_ARG) return "NULL pointer or negative size";
    if (code == VQREF_E_NOALGO) return "hipBLASLt has no algorithm for this shape";
    if (code >= 1000) return "hipBLASLt call failed (code - 1000 is the hipblasStatus_t)";
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown vqref error";
}

int vqref_gemm_f16(const void *x, const void *w, void *y, int64_t M, int64_t K, int64_t N, int32_t w_is_nk,
                   void *stream)
{
    if (M < 0 || K < 0 || N < 0) return VQREF_E_ARG;
    if (M == 0 || N == 0) return 0;
    if (!x || !w || !y || K == 0) return VQREF_E_ARG;
    int dev = 0;
    hipError_t he = hipGetDevice(&dev);
    if (he != hipSuccess) return (int)he;

    std::lock_guard<std::mutex> lock(g_mu);
    DeviceState &st = g_state[dev];
    if (!st.handle) {
        hipblasStatus_t bs = hipblasLtCreate(&st.handle);
        if (bs != HIPBLAS_STATUS_SUCCESS) { st.handle = nullptr; return blas_rc(bs); }
        he = hipMalloc(&st.workspace, kWorkspaceBytes);
        if (he != hipSuccess) { st.workspace = nullptr; return (int)he; }
    }

    // Row-major y[M,N] = x[M,K].W  is column-major  y^T[N,M] = W^T[N,K] . x^T[K,M].
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    hipblasLtMatmulPreference_t pref = nullptr;
    int rc = 0;
    auto fail = [&](hipblasStatus_t bs) { rc = blas_rc(bs); return bs != HIPBLAS_STATUS_SUCCESS; };
    do {
        if (fail(hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F))) break;
        const hipblasOperation_t opa = w_is_nk ? HIPBLAS_OP_T : HIPBLAS_OP_N, opb = HIPBLAS_OP_N;
        if (fail(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opa, sizeof(opa)))) break;
        if (fail(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opb, sizeof(opb)))) break;
        // w[K,N] row-major is a column-major N x K matrix (ld N); w[N,K] row-major is a
        // column-major K x N matrix (ld K) used transposed.
        if (w_is_nk) { if (fail(hipblasLtMatrixLayoutCreate(&la, HIP_R_16F, K, N, K))) break; }
        else         { if (fail(hipblasLtMatrixLayoutCreate(&la, HIP_R_16F, N, K, N))) break; }
        if (fail(hipblasLtMatrixLayoutCreate(&lb, HIP_R_16F, K, M, K))) break;
        if (fail(hipblasLtMatrixLayoutCreate(&lc, HIP_R_16F, N, M, N))) break;

        const auto key = std::make_tuple(M, K, N, (int)(w_is_nk != 0));
        auto it = st.algos.find(key);
        if (it == st.algos.end()) {
            if (fail(hipblasLtMatmulPreferenceCreate(&pref))) break;
            size_t ws = kWorkspaceBytes;
            if (fail(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws)))) break;
            hipblasLtMatmulHeuristicResult_t res[kMaxCandidates];
            int found = 0;
            const int want = tuning_enabled() ? kMaxCandidates : 1;
            if (fail(hipblasLtMatmulAlgoGetHeuristic(st.handle, desc, la, lb, lc, lc, pref, want, res, &found))) break;
            if (found < 1) { rc = VQREF_E_NOALGO; break; }
            Choice c;
            c.algo = res[0].algo;
            if (found > 1) {
                float best_us = 0.f, first_us = 0.f;
                const int best = pick_fastest(st, desc, la, lb, lc, x, w, y, res, found, static_cast<hipStream_t>(stream),
                                              &best_us, &first_us);
                if (best >= 0) {
                    c.algo = res[best].algo;
                    c.candidates = found;
                    c.chosen = best;
                    c.best_us = best_us;
                    c.first_us = first_us;
                }
            }
            it = st.algos.emplace(key, c).first;
        }
        const float alpha = 1.0f, beta = 0.0f;
        if (fail(hipblasLtMatmul(st.handle, desc, &alpha, w, la, x, lb, &beta, y, lc, y, lc, &it->second.algo,
                                 st.workspace, kWorkspaceBytes, static_cast<hipStream_t>(stream)))) break;
    } while (false);
    if (pref) hipblasLtMatmulPreferenceDestroy(pref);
    if (lc) hipblasLtMatrixLayoutDestroy(lc);
    if (lb) hipblasLtMatrixLayoutDestroy(lb);
    if (la) hipblasLtMatrixLayoutDestroy(la);
    if (desc) hipblasLtMatmulDescDestroy(desc);
    return rc;
}

int vqref_tuning_info(int64_t M, int64_t K, int64_t N, int32_t w_is_nk, int32_t *candidates, int32_t *chosen,
                      float *best_us, float *first_us)
{
    int dev = 0;
    hipError_t he = hipGetDevice(&dev);
    if (he != hipSuccess) return (int)he;
    std::lock_guard<std::mutex> lock(g_mu);
    const DeviceState &st = g_state[dev];
    const auto it = st.algos.find(std::make_tuple(M, K, N, (int)(w_is_nk != 0)));
    if (it == st.algos.end()) return VQREF_E_NOALGO;
    if (candidates) *candidates = it->second.candidates;
    if (chosen) *chosen = it->second.chosen;
    if (best_us) *best_us = it->second.best_us;
    if (first_us) *first_us = it->second.first_us;
    return 0;
}

}  // extern "C"
