// The entry point that allocates nothing: vqgemm_e2e_gemm_a with the scratch of its two-pass route
// (the dequantised weights W_dec[K, 2*Nc], fp16) in a file-scope device array instead of a
// caller-supplied workspace.  For callers that cannot call hipMalloc (code under HIP graph capture,
// tight serving loops, harnesses that forbid it).  Everything else - validation, kernel choice, the
// kernels themselves - is the existing entry point's, which gets the array's device address as
// its workspace.
#include "../../include/vq_gemm.h"
#include "vq_common.h"

#include <limits.h>
#include <mutex>

namespace {

// Every GPU the library runs on holds its own copy of this array at its own address from the load
// of the code object to the end of the process.  In host code the name is only a handle for
// hipGetSymbolAddress: kernels get the address that call returns.
static __device__ __align__(256) unsigned char scratch[VQGEMM_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_mu;
void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, looked up once

// Device address of the copy of `scratch` on the device that owns `stream` (the current device for the
// default stream).  The first look-up on a device makes the runtime load the code object that holds the
// array: it is refused while `stream` is capturing, where such work does not belong.
hipError_t scratch_address(hipStream_t stream, void **ptr)
{
    int current = 0;
    hipError_t e = hipGetDevice(&current);
    if (e != hipSuccess) return e;
    int dev = current;
    if (stream) {
        e = hipStreamGetDevice(stream, &dev);
        if (e != hipSuccess) return e;
    }
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_scratch_ptr[dev]) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (stream && hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
            return hipErrorStreamCaptureUnsupported;
        // (hipGetSymbolAddress answers for the current device)
        if (dev != current && (e = hipSetDevice(dev)) != hipSuccess) return e;
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (dev != current) (void)hipSetDevice(current);
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return hipSuccess;
}

}  // namespace

extern "C" {

int vqgemm_e2e_gemm_a_noalloc(const void *x, const void *w, const void *codebook, void *out, int64_t M, int64_t K,
                              int64_t Nc, int32_t variant, void *stream)
{
    if (M < 0 || K < 0 || Nc < 0 || M > INT_MAX / 2 || K > INT_MAX / 2 || Nc > INT_MAX / 4) return VQGEMM_E_SHAPE;
    // The dequantised weights must fit the array whatever route the call takes, so that the limit
    // does not depend on the kernel choice.
    if (K * 2 * Nc * 2 > (int64_t)VQGEMM_NOALLOC_SCRATCH_BYTES) return VQGEMM_E_SCRATCH;
    void *ptr = nullptr;
    const hipError_t e = scratch_address(static_cast<hipStream_t>(stream), &ptr);
    if (e != hipSuccess) return static_cast<int>(e);
    return vqgemm_e2e_gemm_a(x, w, codebook, out, M, K, Nc, variant, ptr, stream);
}

}  // extern "C"
