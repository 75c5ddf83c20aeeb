// What the matrix cores sustain on this device with nothing else going on: a register-only MFMA
// loop, one wave per SIMD on every CU, 8192 (16x16x32) or 4096 (32x32x16) fp16 MFMAs per wave - the
// MFMA count of one 256x256 output tile over K = 4096.  The operands sit in registers for the
// whole kernel; they are either random (normal X, small normal W) or all zero.  With random
// operands the device runs into its power limit and lowers the clock, and how far depends on the
// MFMA shape; this is the ceiling the prefill kernel is measured against.
//
// Stand-alone measurement tool (no library, no torch), run by `bench.py --mfma-ceiling` and by the
// bench's reporting leg; not part of libvqgemm.so.  Prints one line per case with the time per launch,
// the rate, and the time, cycle count and clock seen from inside the kernel.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define CHECK(e)                                                                        \
    do {                                                                                \
        hipError_t err_ = (e);                                                          \
        if (err_ != hipSuccess) {                                                       \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(err_)); \
            exit(1);                                                                    \
        }                                                                               \
    } while (0)

__device__ uint64_t g_clock[4096 * 4];

// SHAPE 0: v_mfma_f32_32x32x16_f16 on a 4x4 grid of 32x32 accumulators.
// SHAPE 1: v_mfma_f32_16x16x32_f16 on an 8x8 grid of 16x16 accumulators, walked in 4x4 quadrants.
// Both are 2^19 multiply-adds per wave and iteration of 32 resp. 64 MFMAs.
template <int SHAPE>
__global__ __launch_bounds__(256, 1) void mfma_loop(const half8_t *a, const half8_t *b, float *out, int iters)
{
    const int tid = threadIdx.x + blockIdx.x * 256;
    half8_t A[8], B[8];
    for (int i = 0; i < 8; i++) {
        A[i] = a[(tid * 8 + i) % 65536];
        B[i] = b[(tid * 8 + i) % 65536];
    }
    const uint64_t t0 = wall_clock64(), c0 = clock64();
    float sum = 0.f;
    if (SHAPE == 0) {
        float16_t acc[4][4] = {};
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(A[s * 4 + i], B[s * 4 + j], acc[i][j], 0, 0, 0);
        }
        for (int i = 0; i < 4; i++)
            for (int j = 0; j < 4; j++)
                for (int r = 0; r < 16; r++) sum += acc[i][j][r];
    } else {
        float4_t acc[8][8] = {};
        auto quadrant = [&](int jh, int ih) {
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int f = 0; f < 4; f++) {
                    const int j = jh * 4 + e, i = ih * 4 + f;
                    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[j][i]) : "v"(A[j]), "v"(B[i]));
                }
        };
        for (int it = 0; it < iters; it++) {
            quadrant(0, 0);
            quadrant(1, 0);
            quadrant(1, 1);
            quadrant(0, 1);
        }
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
        for (int i = 0; i < 8; i++)
            for (int j = 0; j < 8; j++)
                for (int r = 0; r < 4; r++) sum += acc[i][j][r];
    }
    out[tid] = sum;
    const uint64_t t1 = wall_clock64(), c1 = clock64();
    if (threadIdx.x == 0) {
        g_clock[blockIdx.x * 4] = t0;
        g_clock[blockIdx.x * 4 + 1] = t1;
        g_clock[blockIdx.x * 4 + 2] = c1 - c0;
    }
}

static float gauss()
{
    const float u = (rand() + 1.0f) / ((float)RAND_MAX + 2.0f), v = rand() / (float)RAND_MAX;
    return sqrtf(-2 * logf(u)) * cosf(6.2831853f * v);
}

int main()
{
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int wgs = prop.multiProcessorCount;
    if (wgs > 4096) return 1;
    const int n = 65536 * 8, iters = 128;
    half8_t *a, *b;
    float *out;
    CHECK(hipMalloc(&a, n * 2));
    CHECK(hipMalloc(&b, n * 2));
    CHECK(hipMalloc(&out, (size_t)wgs * 256 * 4));
    for (int zero = 0; zero < 2; zero++) {
        std::vector<_Float16> ha(n), hb(n);
        srand(1);
        for (int i = 0; i < n; i++) {
            ha[i] = zero ? (_Float16)0 : (_Float16)gauss();
            hb[i] = zero ? (_Float16)0 : (_Float16)(0.02f * gauss());
        }
        CHECK(hipMemcpy(a, ha.data(), n * 2, hipMemcpyHostToDevice));
        CHECK(hipMemcpy(b, hb.data(), n * 2, hipMemcpyHostToDevice));
        for (int shape = 0; shape < 2; shape++) {
            auto launch = [&]() {
                if (shape == 0) mfma_loop<0><<<wgs, 256>>>(a, b, out, iters);
                else mfma_loop<1><<<wgs, 256>>>(a, b, out, iters);
            };
            hipEvent_t e0, e1;
            CHECK(hipEventCreate(&e0));
            CHECK(hipEventCreate(&e1));
            for (int w = 0; w < 30; w++) launch();
            CHECK(hipDeviceSynchronize());
            const int reps = 30;
            CHECK(hipEventRecord(e0));
            for (int w = 0; w < reps; w++) launch();
            CHECK(hipEventRecord(e1));
            CHECK(hipEventSynchronize(e1));
            float ms;
            CHECK(hipEventElapsedTime(&ms, e0, e1));
            std::vector<uint64_t> p(wgs * 4);
            CHECK(hipMemcpyFromSymbol(p.data(), HIP_SYMBOL(g_clock), (size_t)wgs * 4 * 8));
            double us = 0, cyc = 0;
            for (int i = 0; i < wgs; i++) {
                us += (p[i * 4 + 1] - p[i * 4]) / 100.0;  // the wall clock counts at 100 MHz
                cyc += p[i * 4 + 2];
            }
            us /= wgs;
            cyc /= wgs;
            const double flops = (double)wgs * 4 * iters * 2.0 * 524288;
            printf("%s operands, %s: %.1f us per launch, %.0f TFLOP/s; inside the kernel %.1f us, %.0f cycles, %.0f MHz\n",
                   zero ? "zero" : "random", shape ? "v_mfma_f32_16x16x32_f16" : "v_mfma_f32_32x32x16_f16", ms / reps * 1e3,
                   flops / (ms / reps * 1e-3) / 1e12, us, cyc, cyc / us);
        }
    }
    return 0;
}
