// Dot product of one slot of a re-tiled weight tile with its int8 activations (decode kernels).
#pragma once
#include "common.hpp"

namespace bitnet {

__device__ __forceinline__ int dot4(uint32_t a, uint32_t c, int acc)
{
    return __builtin_amdgcn_sdot4((int)a, (int)c, acc, false);
}

// 64 weights (one slot of a tile: dword t = 16 columns at 64t + 16kq) against their activations; ag
// points at activation group kq of the tile, the groups of consecutive dwords are 4 apart.  The weights enter
// as their stored codes c = w + 1; the caller subtracts the sum of the activations once.
__device__ __forceinline__ int dot64(const uint4 &w4, const uint4 *ag, int acc)
{
    const uint32_t ws[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const uint32_t w = ws[t];
        const uint4 a4 = ag[4 * t];
        acc = dot4(a4.x, w & 0x03030303u, acc);
        acc = dot4(a4.y, (w >> 2) & 0x03030303u, acc);
        acc = dot4(a4.z, (w >> 4) & 0x03030303u, acc);
        acc = dot4(a4.w, (w >> 6) & 0x03030303u, acc);
    }
    return acc;
}

}  // namespace bitnet
