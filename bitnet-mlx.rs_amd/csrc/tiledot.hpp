// Dot product of one slot of a re-tiled weight tile with its int8 activations (decode kernels).
#pragma once
#include "common.hpp"

namespace bitnet {

// A slot of a weight tile (16 bytes per lane).  The weights of a GEMV are read once per call and never again, so the
// load is non-temporal (no cache line kept for them): measured 5.1 -> 5.7 TB/s on a 128 MiB weight matrix.
__device__ __forceinline__ uint4 load_weight_slot(const uint4 *ptr)
{
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const v4u v = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(ptr));
    return make_uint4(v[0], v[1], v[2], v[3]);
}

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
