// hipBLASLt fp16 GEMM (fp32 accumulate) on uncompressed weights: the vendor baseline the
// fused VQ kernels are measured against.  Takes the place of the reference's cuBLAS module
// (ref_gemm/cublas_gemm_fp16.cu:15-48), which created a handle per call and never freed it;
// here the handle, workspace and per-shape algorithm are cached per device.
#include "../../include/vq_gemm_ref.h"

#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

namespace {

constexpr size_t kWorkspaceBytes = 64ull << 20;

struct DeviceState {
    hipblasLtHandle_t handle = nullptr;
    void *workspace = nullptr;
    std::map<std::tuple<int64_t, int64_t, int64_t, int>, hipblasLtMatmulAlgo_t> algos;
};

std::mutex g_mu;
std::map<int, DeviceState> g_state;

int blas_rc(hipblasStatus_t st) { return st == HIPBLAS_STATUS_SUCCESS ? 0 : 1000 + (int)st; }

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
            hipblasLtMatmulHeuristicResult_t res[1];
            int found = 0;
            if (fail(hipblasLtMatmulAlgoGetHeuristic(st.handle, desc, la, lb, lc, lc, pref, 1, res, &found))) break;
            if (found < 1) { rc = VQREF_E_NOALGO; break; }
            it = st.algos.emplace(key, res[0].algo).first;
        }
        const float alpha = 1.0f, beta = 0.0f;
        if (fail(hipblasLtMatmul(st.handle, desc, &alpha, w, la, x, lb, &beta, y, lc, y, lc, &it->second,
                                 st.workspace, kWorkspaceBytes, static_cast<hipStream_t>(stream)))) break;
    } while (false);
    if (pref) hipblasLtMatmulPreferenceDestroy(pref);
    if (lc) hipblasLtMatrixLayoutDestroy(lc);
    if (lb) hipblasLtMatrixLayoutDestroy(lb);
    if (la) hipblasLtMatrixLayoutDestroy(la);
    if (desc) hipblasLtMatmulDescDestroy(desc);
    return rc;
}

}  // extern "C"
