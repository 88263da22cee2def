// LDS-direct loads (global memory -> LDS without passing through registers) and hand-placed load waits, shared by
// the prefill GEMM and the token-group decode GEMV.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace bitnet {

// LDS-direct load of 16 bytes per lane: m0 carries the LDS base of the wavefront's 1 KiB destination, lane l
// lands at base + 16*l.  The global address is a scalar base plus a 32-bit per-lane byte offset: where the offsets
// are loop invariant, advancing a stage costs two scalar additions and no vector instruction.
__device__ __forceinline__ void dma16(const void *sbase, uint32_t voff, uint32_t lds_off)
{
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1\n\t"
                 : : "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory", "m0");
}
// The same for 4 bytes per lane: lane l lands at base + 4*l.
__device__ __forceinline__ void dma4(const void *sbase, uint32_t voff, uint32_t lds_off)
{
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1\n\t"
                 : : "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane(lds_off)) : "memory", "m0");
}
// Loads return in issue order: waits until at most N of this wavefront's loads are still in flight.
template <int N>
__device__ __forceinline__ void wait_vm()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
// s_setprio takes an immediate.
__device__ __forceinline__ void set_wave_priority(int pr)
{
    if (pr == 0) __builtin_amdgcn_s_setprio(0);
    else if (pr == 1) __builtin_amdgcn_s_setprio(1);
    else if (pr == 2) __builtin_amdgcn_s_setprio(2);
    else __builtin_amdgcn_s_setprio(3);
}

}  // namespace bitnet
