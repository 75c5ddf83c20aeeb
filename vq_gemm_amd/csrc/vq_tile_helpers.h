// Device helpers shared by the tiled MFMA kernels (prefill kernels, plain tiled GEMM).
#pragma once

#include "vq_common.h"

namespace vq {

namespace {

// s_waitcnt for the vector-memory counter only (gfx9 encoding: vmcnt = simm16[15:14]:[3:0]).
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// acc += a . b with the accumulator pinned to one AGPR tuple.  Left to itself the register
// allocator renames the 64 four-register accumulators from MFMA to MFMA and pays for it with
// copies at the loop edge and with spills.  The compiler cannot see into the statement, so the
// callers keep dependent MFMAs (same accumulator) far apart and pad before the accumulators are
// read back.
__device__ __forceinline__ void mfma_in_place(float4_t &acc, const half8_t &a, const half8_t &b)
{
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// 16-byte store of a result that this kernel does not read again: the non-temporal hint lets the
// write leave the L2 as it is issued instead of waiting for the write-back at the end of the kernel
// (all workgroups of a round finish at about the same time).
__device__ __forceinline__ void st_global_16_streaming(void *p, uint4_t v)
{
    __builtin_nontemporal_store(v, reinterpret_cast<uint4_t *>(p));
}

}  // namespace

}  // namespace vq
