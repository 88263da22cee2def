// Decode GEMV kernels: int8 activations x 2-bit ternary weights -> int32, for gfx950.
//
//   acc[t, n] = sum_k a[t, k] * w[n, k]         exact in int32 (|acc| <= 127*K)
//   out[t, n] = (float(acc) * w_scale) / a_scale[t] (+ bias[n]) (+ residual[t, n])
//
// Semantics: bitnet-quant/src/simd/matrix.rs:471-490 (GEMV) with the contract of
// bitnet-cuda/src/kernels/w2a8_gemv.cu:100-105 (u8 packed weights, i8 activations, i32 output).
//
// The kernels never decode to {-1,0,+1}.  They multiply by the stored code c = w + 1 in {0,1,2}
// (two VALU operations turn a packed dword into four code bytes: shift, and with 0x03030303) and
// subtract sum_k a[t, k] once per output:  sum a*(c-1) = sum a*c - sum a.
//
// gemv_tiled_kernel streams the re-tiled layout (weight_prep.hip).  A workgroup of four wavefronts owns
// one block of 16 output rows; its wavefronts take the k-tiles round-robin, so all of a workgroup's
// weight bytes are requested in the first few instructions.  Lane l of a wavefront loads the 16 bytes at
// offset 16*l of a 1 KiB tile: row r = l mod 16, four groups of 16 columns.  Activations sit in LDS
// (staged once per workgroup); the 16 lanes of a group read the same LDS address (a broadcast).
// Partial sums are combined with two wavefront shuffles (the four lanes of a row), then across the four
// wavefronts through LDS.  HBM traffic per call: n*k/4 weight bytes + k activation bytes per row block.
#include "kernels.hpp"

namespace bitnet {

namespace {

struct GemvParams {
    const uint8_t *w;
    const int8_t *a;
    int32_t *acc;
    const float *w_scale;
    const float *a_scale;
    const float *bias;
    const float *residual;
    float *out;
    int m;  // tokens in this launch (<= MB)
    int n;
    int k;
    int kt_count;
};

__device__ __forceinline__ int dot4(uint32_t a, uint32_t c, int acc)
{
    return __builtin_amdgcn_sdot4((int)a, (int)c, acc, false);
}

// 64 weights (one slot of a tile: dword t = 16 columns at 64t + 16kq) against their activations; ag
// points at activation group kq of the tile, the groups of consecutive dwords are 4 apart.
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

constexpr int GEMV_PREFETCH = 4;  // tiles in flight per wavefront

template <int MB>
__global__ __launch_bounds__(256) void gemv_tiled_kernel(GemvParams p)
{
    extern __shared__ uint4 lds_a[];  // [MB][groups]: activations, 16 per uint4, zero past K / past m
    __shared__ int red[4][TILE_ROWS][MB];
    __shared__ int asum[MB];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int groups = p.kt_count * 16;
    const uint4 *tiles = reinterpret_cast<const uint4 *>(p.w) + (size_t)blockIdx.x * p.kt_count * 64;

    // Request the first batch of weight tiles before anything else.
    uint4 wbuf[GEMV_PREFETCH];
#pragma unroll
    for (int u = 0; u < GEMV_PREFETCH; ++u) {
        int kt = wave + 4 * u;
        wbuf[u] = kt < p.kt_count ? tiles[(size_t)kt * 64 + lane] : make_uint4(0, 0, 0, 0);
    }

    // Stage activations; every thread also accumulates sum_k a[t, k] for the code offset.
    if (tid < MB) asum[tid] = 0;
    __syncthreads();
    const bool vec_ok = (p.k % 16 == 0) && ((reinterpret_cast<uintptr_t>(p.a) & 15) == 0);
#pragma unroll
    for (int t = 0; t < MB; ++t) {
        int local = 0;
        for (int g = tid; g < groups; g += 256) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (t < p.m) {
                const int8_t *src = p.a + (size_t)t * p.k + 16 * (size_t)g;
                if (vec_ok) {
                    if (16 * g < p.k) v = *reinterpret_cast<const uint4 *>(src);
                } else {
                    uint32_t d[4] = {0, 0, 0, 0};
                    for (int j = 0; j < 16; ++j)
                        if (16 * g + j < p.k) d[j >> 2] |= (uint32_t)(uint8_t)src[j] << (8 * (j & 3));
                    v = make_uint4(d[0], d[1], d[2], d[3]);
                }
            }
            lds_a[t * groups + g] = v;
            local = dot4(v.x, 0x01010101u, local);
            local = dot4(v.y, 0x01010101u, local);
            local = dot4(v.z, 0x01010101u, local);
            local = dot4(v.w, 0x01010101u, local);
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) local += __shfl_xor(local, off, 64);
        if (lane == 0) atomicAdd(&asum[t], local);
    }
    __syncthreads();

    int acc[MB];
#pragma unroll
    for (int t = 0; t < MB; ++t) acc[t] = 0;

    const int kq = lane >> 4;  // lane group: columns 64t + 16kq .. +15 of each tile, t = 0..3
    for (int kt0 = wave; kt0 < p.kt_count; kt0 += 4 * GEMV_PREFETCH) {
        uint4 wnext[GEMV_PREFETCH];
#pragma unroll
        for (int u = 0; u < GEMV_PREFETCH; ++u) {
            int kt = kt0 + 4 * (GEMV_PREFETCH + u);
            wnext[u] = kt < p.kt_count ? tiles[(size_t)kt * 64 + lane] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < GEMV_PREFETCH; ++u) {
            int kt = kt0 + 4 * u;
            if (kt < p.kt_count) {
                const uint4 *ag = lds_a + kt * 16 + kq;
#pragma unroll
                for (int t = 0; t < MB; ++t) acc[t] = dot64(wbuf[u], ag + t * groups, acc[t]);
            }
        }
#pragma unroll
        for (int u = 0; u < GEMV_PREFETCH; ++u) wbuf[u] = wnext[u];
    }

    // the four lanes l, l+16, l+32, l+48 hold the four column quarters of row l mod 16
#pragma unroll
    for (int t = 0; t < MB; ++t) {
        acc[t] += __shfl_xor(acc[t], 16, 64);
        acc[t] += __shfl_xor(acc[t], 32, 64);
    }
    if (lane < TILE_ROWS) {
#pragma unroll
        for (int t = 0; t < MB; ++t) red[wave][lane][t] = acc[t];
    }
    __syncthreads();

    if (tid < TILE_ROWS * MB) {
        const int r = tid / MB, t = tid % MB;
        const int n = blockIdx.x * TILE_ROWS + r;
        if (n < p.n && t < p.m) {
            int total = red[0][r][t] + red[1][r][t] + red[2][r][t] + red[3][r][t] - asum[t];
            size_t o = (size_t)t * p.n + n;
            if (p.acc) p.acc[o] = total;
            if (p.out) {
                float v = f32_mul((float)total, *p.w_scale);
                v = f32_div(v, p.a_scale[t]);
                if (p.bias) v = f32_add(v, p.bias[n]);
                if (p.residual) v = f32_add(v, p.residual[o]);
                p.out[o] = v;
            }
        }
    }
}

// The reference's flat row-major packing, any n and k (rows need not start on a byte boundary).
// One wavefront per output row; lane l takes columns 4l..4l+3, 4l+256.., gathers their codes one by one.
__global__ __launch_bounds__(256) void gemv_rowmajor_kernel(const uint8_t *packed, const int8_t *a,
                                                            int32_t *out, size_t n, size_t k)
{
    const int lane = threadIdx.x;
    const size_t row = (size_t)blockIdx.x * blockDim.y + threadIdx.y;
    if (row >= n) return;
    int acc = 0;
    if (k % 16 == 0 && (reinterpret_cast<uintptr_t>(packed) & 3) == 0 &&
        (reinterpret_cast<uintptr_t>(a) & 3) == 0) {
        // rows are dword aligned: 16 weights per load
        const uint32_t *wr = reinterpret_cast<const uint32_t *>(packed) + row * (k / 16);
        const uint32_t *ad = reinterpret_cast<const uint32_t *>(a);
        for (size_t g = lane; g < k / 16; g += 64) {
            uint32_t w = wr[g];
            w &= ~((w & (w >> 1) & 0x55555555u) << 1);  // code 3 -> code 1 (both are weight 0)
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                uint32_t byte = (w >> (8 * b)) & 0xffu;
                uint32_t c = (byte & 3u) | ((byte & 0xcu) << 6) | ((byte & 0x30u) << 12) | ((byte & 0xc0u) << 18);
                uint32_t av = ad[4 * g + b];
                acc = dot4(av, c, acc) - dot4(av, 0x01010101u, 0);  // codes are w + 1: take sum(a) off
            }
        }
    } else {
        for (size_t k0 = 4 * (size_t)lane; k0 < k; k0 += 256) {
            for (int j = 0; j < 4; ++j) {
                size_t kk = k0 + j;
                if (kk >= k) break;
                size_t e = row * k + kk;
                unsigned code = (packed[e >> 2] >> (2 * (e & 3))) & 3u;
                int w = code == 0 ? -1 : (code == 2 ? 1 : 0);
                acc += w * (int)a[kk];
            }
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) out[row] = acc;
}

template <int MB>
int launch_tiled_mb(const GemvParams &p, hipStream_t stream)
{
    size_t lds = (size_t)MB * p.kt_count * 16 * sizeof(uint4);
    if (lds > 60 * 1024)
        return fail(BITNET_HIP_UNSUPPORTED, "decode GEMV: %d tokens x k=%d need %zu bytes of LDS", MB, p.k, lds);
    dim3 grid((unsigned)row_blocks((size_t)p.n));
    hipLaunchKernelGGL((gemv_tiled_kernel<MB>), grid, dim3(256), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemv_tiled_kernel");
    return BITNET_HIP_OK;
}

}  // namespace

int launch_gemv_rowmajor(const uint8_t *packed, const int8_t *a, int32_t *out, size_t n, size_t k,
                         hipStream_t stream)
{
    if (n == 0) return BITNET_HIP_OK;
    hipLaunchKernelGGL(gemv_rowmajor_kernel, dim3((unsigned)((n + 3) / 4)), dim3(64, 4), 0, stream, packed, a,
                       out, n, k);
    BITNET_HIP_CHECK_LAUNCH("gemv_rowmajor_kernel");
    return BITNET_HIP_OK;
}

int launch_gemv_tiled(const uint8_t *tiled, const int8_t *a, size_t m, size_t n, size_t k, int32_t *acc,
                      const float *w_scale, const float *a_scale, const float *bias, const float *residual,
                      float *out, hipStream_t stream)
{
    if (m == 0 || n == 0) return BITNET_HIP_OK;
    GemvParams p;
    p.w = tiled; p.a = a; p.acc = acc; p.w_scale = w_scale; p.a_scale = a_scale; p.bias = bias;
    p.residual = residual; p.out = out; p.m = (int)m; p.n = (int)n; p.k = (int)k; p.kt_count = (int)k_tiles(k);
    // LDS holds MB activation rows; fall back to fewer rows per launch for very long rows.
    const size_t row_lds = (size_t)p.kt_count * 16 * sizeof(uint4);
    int mb = m >= 8 ? 8 : (m >= 4 ? 4 : (m >= 2 ? 2 : 1));
    while (mb > 1 && mb * row_lds > 60 * 1024) mb >>= 1;
    for (size_t t0 = 0; t0 < m; t0 += (size_t)mb) {
        GemvParams q = p;
        q.m = (int)((m - t0) < (size_t)mb ? (m - t0) : (size_t)mb);
        q.a = a + t0 * k;
        if (acc) q.acc = acc + t0 * n;
        if (out) q.out = out + t0 * n;
        if (a_scale) q.a_scale = a_scale + t0;
        if (residual) q.residual = residual + t0 * n;
        int rc;
        switch (mb) {
            case 8: rc = launch_tiled_mb<8>(q, stream); break;
            case 4: rc = launch_tiled_mb<4>(q, stream); break;
            case 2: rc = launch_tiled_mb<2>(q, stream); break;
            default: rc = launch_tiled_mb<1>(q, stream); break;
        }
        if (rc != BITNET_HIP_OK) return rc;
    }
    return BITNET_HIP_OK;
}

}  // namespace bitnet
