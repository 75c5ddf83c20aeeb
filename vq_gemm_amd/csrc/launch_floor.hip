// What one kernel launch costs on this device when the kernel does nothing: a chain of dependent
// launches replayed from a HIP graph, timed with events on the launch stream - the protocol of
// bench.py.  It is the part of a microsecond-scale launch (the decode GEMV moves 2 MB, 0.26 us at
// the HBM peak) that no kernel can remove.  Two kernels: one that returns at once, and one that
// does the least a GEMV has to (one global load per lane, an LDS write, a barrier, one store), each
// over a grid of one to four workgroups per compute unit.
//
// Stand-alone measurement tool (no library, no torch), run by `bench.py --launch-floor`; not part
// of libvqgemm.so.  Prints one line per case.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CHECK(e)                                                                        \
    do {                                                                                \
        hipError_t err_ = (e);                                                          \
        if (err_ != hipSuccess) {                                                       \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(err_)); \
            exit(1);                                                                    \
        }                                                                               \
    } while (0)

__global__ void empty_kernel(float *out, int n)
{
    if (n < 0) out[threadIdx.x] = 1.f;  // never taken: keeps the arguments alive
}

__global__ void touch_kernel(const float *in, float *out)
{
    extern __shared__ float sm[];
    sm[threadIdx.x] = in[blockIdx.x * blockDim.x + threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) out[blockIdx.x] = sm[blockDim.x - 1];
}

int main()
{
    constexpr int kLaunches = 200, kReplays = 5;
    int dev = 0, cus = 0;
    CHECK(hipGetDevice(&dev));
    CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    float *in, *out;
    CHECK(hipMalloc(&in, 16 << 20));
    CHECK(hipMalloc(&out, 1 << 20));
    CHECK(hipMemset(in, 0, 16 << 20));
    hipStream_t s;
    CHECK(hipStreamCreate(&s));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    printf("launch floor: %d dependent launches per HIP graph, best of %d replays, %d compute units\n", kLaunches, kReplays, cus);
    for (int kind = 0; kind < 2; kind++)
        for (int per_cu : {1, 2, 4})
            for (int block : {64, 256, 1024}) {
                const int grid = cus * per_cu;
                hipGraph_t graph;
                hipGraphExec_t exec;
                CHECK(hipStreamBeginCapture(s, hipStreamCaptureModeGlobal));
                for (int i = 0; i < kLaunches; i++) {
                    if (kind == 0) hipLaunchKernelGGL(empty_kernel, dim3(grid), dim3(block), 0, s, out, 1);
                    else hipLaunchKernelGGL(touch_kernel, dim3(grid), dim3(block), block * 4, s, in, out);
                }
                CHECK(hipStreamEndCapture(s, &graph));
                CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
                CHECK(hipGraphLaunch(exec, s));  // the first replay uploads the graph
                CHECK(hipStreamSynchronize(s));
                float best = 1e30f;
                for (int r = 0; r < kReplays; r++) {
                    CHECK(hipEventRecord(e0, s));
                    CHECK(hipGraphLaunch(exec, s));
                    CHECK(hipEventRecord(e1, s));
                    CHECK(hipEventSynchronize(e1));
                    float ms;
                    CHECK(hipEventElapsedTime(&ms, e0, e1));
                    if (ms < best) best = ms;
                }
                printf("%s kernel, %d workgroup(s) per unit of %4d threads: %.3f us per launch\n",
                       kind ? "touch" : "empty", per_cu, block, best * 1e3 / kLaunches);
                CHECK(hipGraphExecDestroy(exec));
                CHECK(hipGraphDestroy(graph));
            }
    return 0;
}
