// Decode GEMV that streams base-3 bytes (five ternary values per byte, 1.6 bits per weight) instead of the 2-bit codes:
// the byte format of Base3PackedPacker (bitnet-quant/src/quantization/packing.rs:421-501: byte = sum_i (w_i + 1) * 3^i)
// consumed by the contraction itself, 20 % fewer weight bytes per output than the 2-bit layout.
//
//   acc[n] = sum_k a[k] * w[n, k]      int32, exact (bitnet-quant/src/simd/matrix.rs:471-490)
//
// Streaming layout (bitnet_hip_retile_base3): tiles of 16 rows x 320 columns = 1 KiB, stored [row_block][k_tile].
// Slot s = 16*kq + r (16 bytes) belongs to row r; its byte t holds columns 320*kt + 80*kq + 5*t .. +4 as base-3 digits
// (digit i = column + i).  Columns past k hold digit 1 (weight 0).  Lane l of a wavefront loads slot l: one contiguous
// 1 KiB burst per tile, as in the 2-bit layout.
//
// A base-3 byte cannot be split by shifts and masks: every byte goes through a 256-entry table in LDS (byte -> its five
// digits in one dword: four in the low bits of its bytes, the fifth beside the first), and the activations are staged in
// LDS in groups of five padded to eight bytes, so that a weight byte costs one table read (indexed by the byte: the lanes
// of a read hit LDS banks at random), (half) an activation read, two masks and two dot-product instructions where the
// 2-bit layout spends two instructions on four weights.  The kernel is bound by that, not by
// memory; it exists so that the cost of the denser format is a measured figure.
#include "kernels.hpp"
#include "rowquant.hpp"
#include "tiledot.hpp"

namespace bitnet {

namespace {

constexpr int B3_TILE_K = 320;  // columns per base-3 tile: 16 bytes per row and lane group, 4 lane groups

__device__ __forceinline__ unsigned b3_digit(unsigned byte, unsigned j)
{
    unsigned v = byte;
    for (unsigned i = 0; i < j; ++i) v /= 3;
    return v % 3;
}

// One thread per byte of the streaming layout.
__global__ __launch_bounds__(256) void retile_base3_kernel(const uint8_t *flat, size_t n, size_t k, size_t kt_count,
                                                           uint8_t *tiled, size_t total)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const size_t tile = i >> 10, in_tile = i & 1023;
    const size_t rb = tile / kt_count, kt = tile % kt_count;
    const size_t slot = in_tile >> 4, t = in_tile & 15;
    const size_t r = slot & 15, kq = slot >> 4;
    const size_t row = rb * 16 + r, col0 = kt * B3_TILE_K + kq * 80 + t * 5;
    unsigned byte = 0, mul = 1;
    for (unsigned d = 0; d < 5; ++d, mul *= 3) {
        unsigned digit = 1;  // weight 0 outside the matrix
        if (row < n && col0 + d < k) {
            const size_t e = row * k + col0 + d;  // element index of the flat [n, k] tensor the reference packs
            digit = b3_digit(flat[e / 5], (unsigned)(e % 5));
        }
        byte += digit * mul;
    }
    tiled[i] = (uint8_t)byte;
}

constexpr int B3_PREFETCH = 4;
constexpr int B3_ACT_SLOTS = 72;  // 8-byte LDS slots per k-tile: 4 lane groups of 16 activation groups + 2 slots of padding

__host__ __device__ constexpr int b3_act_slot(int g) { return g + (g >> 6) * 8 + ((g >> 4) & 3) * 2; }

// One token, int8 activations.  256 threads: wavefront w takes k-tiles w, w + 4, ...; one row block per workgroup.
__global__ __launch_bounds__(256) void gemv_base3_kernel(const uint8_t *tiled, const int8_t *a, int32_t *acc_out, float *out,
                                                         const float *w_scale, const float *a_scale, int n, int k, int kt_count)
{
    // groups of five activations, x = a[5g..5g+3], y = a[5g+4]; group g sits at b3_act_slot(g): the 16 groups of a lane
    // group are followed by 16 bytes of padding, so that the four lane groups of a wavefront, which read four addresses
    // 128 bytes apart otherwise, fall into different LDS banks
    extern __shared__ uint2 lds_act[];
    __shared__ uint32_t tab[256];        // byte -> digits 0..3 in bits 0..1 of its four bytes, digit 4 in bits 4..5
    __shared__ int red[4][TILE_ROWS];
    __shared__ int red_i[4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rb = blockIdx.x;
    const uint4 *tiles = reinterpret_cast<const uint4 *>(tiled) + (size_t)rb * kt_count * 64;

    uint4 wbuf[B3_PREFETCH];
#pragma unroll
    for (int u = 0; u < B3_PREFETCH; ++u)
        wbuf[u] = load_weight_slot(tiles + (size_t)min(wave + 4 * u, kt_count - 1) * 64 + lane);

    {
        const unsigned b = (unsigned)tid;
        const unsigned d0 = b % 3, d1 = (b / 3) % 3, d2 = (b / 9) % 3, d3 = (b / 27) % 3, d4 = (b / 81) % 3;
        tab[tid] = d0 | (d4 << 4) | (d1 << 8) | (d2 << 16) | (d3 << 24);
    }
    const int groups = kt_count * 64;
    int local = 0;
    if ((k & 3) == 0 && (reinterpret_cast<uintptr_t>(a) & 3) == 0) {
        // four groups (20 activations) per thread and step: five aligned dwords, regrouped by shifts
        const uint32_t *a32 = reinterpret_cast<const uint32_t *>(a);
        const int dwords = k >> 2;
        for (int g4 = tid; 4 * g4 < groups; g4 += 256) {
            uint32_t d[5];
#pragma unroll
            for (int j = 0; j < 5; ++j) d[j] = 5 * g4 + j < dwords ? a32[5 * g4 + j] : 0u;
            const uint2 grp[4] = {make_uint2(d[0], d[1] & 0xffu), make_uint2((d[1] >> 8) | (d[2] << 24), (d[2] >> 8) & 0xffu),
                                  make_uint2((d[2] >> 16) | (d[3] << 16), (d[3] >> 16) & 0xffu),
                                  make_uint2((d[3] >> 24) | (d[4] << 8), d[4] >> 24)};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                lds_act[b3_act_slot(4 * g4 + j)] = grp[j];
                local = dot4(grp[j].x, 0x01010101u, local);
                local = dot4(grp[j].y, 0x00000001u, local);
            }
        }
    } else {
        for (int g = tid; g < groups; g += 256) {
            uint32_t x = 0, y = 0;
#pragma unroll
            for (int j = 0; j < 5; ++j) {
                const int col = 5 * g + j;
                const uint32_t v = col < k ? (uint32_t)(uint8_t)a[col] : 0u;
                if (j < 4) x |= v << (8 * j); else y = v;
            }
            lds_act[b3_act_slot(g)] = make_uint2(x, y);
            local = dot4(x, 0x01010101u, local);
            local = dot4(y, 0x00000001u, local);
        }
    }
    local = wave_sum_i32(local);
    if (lane == 0) red_i[wave] = local;
    __syncthreads();

    int acc = 0;
    const int kq = lane >> 4;
    const uint8_t *tab_b = reinterpret_cast<const uint8_t *>(tab);
    auto dot_slot = [&](const uint4 &w4, int kt) {
        const uint4 *ag = reinterpret_cast<const uint4 *>(lds_act + b3_act_slot(kt * 64 + kq * 16));  // two groups per 16-byte read
        const uint32_t ws[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                const uint4 a2 = ag[2 * d + (j >> 1)];
                const uint32_t b0 = (ws[d] >> (8 * j)) & 0xffu, b1 = (ws[d] >> (8 * j + 8)) & 0xffu;
                const uint32_t e0 = *reinterpret_cast<const uint32_t *>(tab_b + b0 * 4);
                const uint32_t e1 = *reinterpret_cast<const uint32_t *>(tab_b + b1 * 4);
                acc = dot4(a2.x, e0 & 0x03030303u, acc);
                acc = dot4(a2.y, (e0 >> 4) & 3u, acc);
                acc = dot4(a2.z, e1 & 0x03030303u, acc);
                acc = dot4(a2.w, (e1 >> 4) & 3u, acc);
            }
        }
    };
    for (int kt0 = wave; kt0 < kt_count; kt0 += 4 * B3_PREFETCH) {
        if (kt0 + 4 * B3_PREFETCH < kt_count) {  // uniform over the wavefront
            uint4 wnext[B3_PREFETCH];
#pragma unroll
            for (int u = 0; u < B3_PREFETCH; ++u)
                wnext[u] = load_weight_slot(tiles + (size_t)min(kt0 + 4 * (B3_PREFETCH + u), kt_count - 1) * 64 + lane);
#pragma unroll
            for (int u = 0; u < B3_PREFETCH; ++u)
                if (kt0 + 4 * u < kt_count) dot_slot(wbuf[u], kt0 + 4 * u);
#pragma unroll
            for (int u = 0; u < B3_PREFETCH; ++u) wbuf[u] = wnext[u];
        } else {
#pragma unroll
            for (int u = 0; u < B3_PREFETCH; ++u)
                if (kt0 + 4 * u < kt_count) dot_slot(wbuf[u], kt0 + 4 * u);
        }
    }
    acc = sum_over_lane_groups(acc);  // lanes l, l+16, l+32, l+48: the four column groups of row l mod 16
    if (lane < TILE_ROWS) red[wave][lane] = acc;
    __syncthreads();
    if (tid < TILE_ROWS) {
        const int row = rb * TILE_ROWS + tid;
        if (row < n) {
            const int asum = red_i[0] + red_i[1] + red_i[2] + red_i[3];
            const int total = red[0][tid] + red[1][tid] + red[2][tid] + red[3][tid] - asum;  // digits are w + 1
            if (acc_out) acc_out[row] = total;
            if (out) out[row] = f32_div(f32_mul((float)total, *w_scale), a_scale ? *a_scale : 1.0f);
        }
    }
}

}  // namespace

size_t base3_tiled_bytes(size_t n, size_t k) { return row_blocks(n) * ((k + B3_TILE_K - 1) / B3_TILE_K) * (size_t)TILE_BYTES; }

int launch_retile_base3(const uint8_t *flat, size_t n, size_t k, uint8_t *tiled, hipStream_t stream)
{
    const size_t total = base3_tiled_bytes(n, k);
    if (total == 0) return BITNET_HIP_OK;
    const size_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffu) return fail(BITNET_HIP_INVALID_CONFIG, "retile_base3: %zu x %zu is too large", n, k);
    hipLaunchKernelGGL(retile_base3_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, flat, n, k, (k + B3_TILE_K - 1) / B3_TILE_K,
                       tiled, total);
    BITNET_HIP_CHECK_LAUNCH("retile_base3_kernel");
    return BITNET_HIP_OK;
}

int launch_gemv_base3(const uint8_t *tiled, const int8_t *a, int32_t *acc, float *out, const float *w_scale, const float *a_scale,
                      size_t n, size_t k, hipStream_t stream)
{
    if (n == 0) return BITNET_HIP_OK;
    const size_t kt_count = (k + B3_TILE_K - 1) / B3_TILE_K;
    const size_t lds = kt_count * B3_ACT_SLOTS * sizeof(uint2);
    if (kt_count == 0 || lds > 96 * 1024 || row_blocks(n) > 0x7fffffffu || k > 0x7fffffffu)
        return fail(BITNET_HIP_UNSUPPORTED, "gemv_base3: k = %zu needs %zu bytes of LDS for the activations (limit 98304)", k, lds);
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_base3_kernel),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
    BITNET_HIP_TRY(attr);
    hipLaunchKernelGGL(gemv_base3_kernel, dim3((unsigned)row_blocks(n)), dim3(256), lds, stream, tiled, a, acc, out, w_scale, a_scale,
                       (int)n, (int)k, (int)kt_count);
    BITNET_HIP_CHECK_LAUNCH("gemv_base3_kernel");
    return BITNET_HIP_OK;
}

}  // namespace bitnet
