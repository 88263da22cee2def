// Prefill GEMM: int8 activations [m, k] x 2-bit ternary weights [n, k] -> int32 [m, n] on the int8 MFMA
// units of gfx950 (v_mfma_i32_16x16x64_i8), with the fp32 scale epilogue fused into the store.
//
//   acc[t, n] = sum_k a[t, k] * w[n, k]      bitnet-quant/src/simd/matrix.rs:256-282 (ternary_gemm_scalar),
//                                            front door bitnet-quant/src/bitlinear/forward.rs:179-214
//   out[t, n] = (float(acc) * w_scale) / a_scale[t] (+ bias[n]) (+ residual[t, n])
//
// Operand mapping of one MFMA (64 lanes): the A operand of lane l is 16 consecutive int8 activations of
// token row l mod 16, k block l / 16; the B operand is 16 weights of output row l mod 16, same k block;
// result register r of lane l is C[4*(l/16) + r][l mod 16].
//
// Weights are never expanded in memory.  A wavefront loads slot l of a 1 KiB weight tile (16 bytes per
// lane, one coalesced burst per 16 rows x 256 columns); dword t of that slot becomes, after four
// shift-and-mask operations, the B operand of the t-th k-step of the tile.  The operand holds the stored
// codes c = w + 1 in {0,1,2}; the epilogue subtracts sum_k a[t, k] per token row (accumulated on the fly
// while the activation tile passes through registers on its way to LDS).
//
// Activations are staged through LDS in steps of 64 columns, double buffered, rows padded to 80 bytes so
// that the 16-byte fragment reads of 8 consecutive lanes fall in distinct banks.
#include "kernels.hpp"

namespace bitnet {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

struct GemmParams {
    const uint8_t *w;
    const int8_t *a;
    int32_t *acc;
    const float *w_scale;
    const float *a_scale;
    const float *bias;
    const float *residual;
    float *out;
    int m, n, k;
    int kt_count;   // 256-column weight tiles per row block
    int tiles_m, tiles_n;
};

constexpr int LDS_PITCH = 80;  // bytes per activation row per 64-column step

// BM x BN output tile per workgroup of 256 threads (2 x 2 wavefronts).
template <int BM, int BN>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(GemmParams p)
{
    constexpr int WTM = BM / 2, WTN = BN / 2;       // wavefront tile
    constexpr int FM = WTM / 16, FN = WTN / 16;     // MFMA tiles per wavefront
    constexpr int A_LOADS = BM * 64 / 16 / 256;     // 16-byte chunks each thread moves per k-step
    static_assert(WTM % 16 == 0 && WTN % 16 == 0 && A_LOADS >= 1, "tile shape");

    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][BM * LDS_PITCH];
    __shared__ int lds_rowsum[BM];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lr = lane & 15, lg = lane >> 4;

    // Workgroup -> output tile.  Consecutive workgroup ids land on different XCDs (8 of them, each with
    // its own L2), so ids are regrouped: all workgroups of one XCD walk one band of M tiles, N fastest,
    // and share its activation rows in that XCD's L2.
    int tile_id;
    {
        const int total = p.tiles_m * p.tiles_n;
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        const int per_xcd = (total + 7) >> 3;
        tile_id = xcd * per_xcd + idx;
        if (tile_id >= total) return;  // uniform per workgroup
    }
    const int tm = tile_id / p.tiles_n, tn = tile_id % p.tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- activation tile movement: thread -> (row, 16-byte chunk) ----
    // chunk c = tid + 256*i: row = c / 4, column chunk = c % 4 (64 columns = 4 chunks)
    const bool a_vec = (p.k % 16 == 0) && ((reinterpret_cast<uintptr_t>(p.a) & 15) == 0);
    int rowsum[A_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) rowsum[i] = 0;

    auto load_a = [&](int ks, uint4 (&regs)[A_LOADS]) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const int c = tid + 256 * i;
            const int row = m0 + (c >> 2), col = ks * 64 + (c & 3) * 16;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (row < p.m && col < p.k) {
                const int8_t *src = p.a + (size_t)row * p.k + col;
                if (a_vec) {
                    v = *reinterpret_cast<const uint4 *>(src);
                } else {
                    uint32_t d[4] = {0, 0, 0, 0};
                    for (int j = 0; j < 16; ++j)
                        if (col + j < p.k) d[j >> 2] |= (uint32_t)(uint8_t)src[j] << (8 * (j & 3));
                    v = make_uint4(d[0], d[1], d[2], d[3]);
                }
            }
            regs[i] = v;
        }
    };
    auto store_a = [&](int buf, const uint4 (&regs)[A_LOADS]) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const int c = tid + 256 * i;
            *reinterpret_cast<uint4 *>(&lds_a[buf][(c >> 2) * LDS_PITCH + (c & 3) * 16]) = regs[i];
            int s = rowsum[i];
            s = __builtin_amdgcn_sdot4((int)regs[i].x, 0x01010101, s, false);
            s = __builtin_amdgcn_sdot4((int)regs[i].y, 0x01010101, s, false);
            s = __builtin_amdgcn_sdot4((int)regs[i].z, 0x01010101, s, false);
            s = __builtin_amdgcn_sdot4((int)regs[i].w, 0x01010101, s, false);
            rowsum[i] = s;
        }
    };

    // ---- weight tiles: one uint4 per lane per 16-row block per 256 columns ----
    const int ksteps = p.kt_count * 4;
    const uint4 *wt[FN];
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int rb = (n0 + wn * WTN) / 16 + j;
        wt[j] = reinterpret_cast<const uint4 *>(p.w) + ((size_t)rb * p.kt_count) * 64 + lane;
    }
    const int rb_count = (p.n + 15) / 16;
    auto load_b = [&](int kt, uint4 (&regs)[FN]) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int rb = (n0 + wn * WTN) / 16 + j;
            regs[j] = rb < rb_count ? wt[j][(size_t)kt * 64] : make_uint4(0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u);
        }
    };

    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = (v4i){0, 0, 0, 0};

    uint4 a_regs[A_LOADS];
    uint4 b_cur[FN], b_next[FN];
    load_a(0, a_regs);
    load_b(0, b_cur);
    store_a(0, a_regs);
    __syncthreads();

    for (int kt = 0; kt < p.kt_count; ++kt) {
        if (kt + 1 < p.kt_count) load_b(kt + 1, b_next);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int ks = kt * 4 + t;
            const int buf = t & 1;
            if (ks + 1 < ksteps) load_a(ks + 1, a_regs);

            v4i afrag[FM];
#pragma unroll
            for (int i = 0; i < FM; ++i)
                afrag[i] = *reinterpret_cast<const v4i *>(&lds_a[buf][(wm * WTM + i * 16 + lr) * LDS_PITCH + lg * 16]);
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const uint32_t wd = t == 0 ? b_cur[j].x : (t == 1 ? b_cur[j].y : (t == 2 ? b_cur[j].z : b_cur[j].w));
                v4i bfrag;
                bfrag[0] = (int)(wd & 0x03030303u);
                bfrag[1] = (int)((wd >> 2) & 0x03030303u);
                bfrag[2] = (int)((wd >> 4) & 0x03030303u);
                bfrag[3] = (int)((wd >> 6) & 0x03030303u);
#pragma unroll
                for (int i = 0; i < FM; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afrag[i], bfrag, acc[i][j], 0, 0, 0);
            }

            if (ks + 1 < ksteps) store_a(buf ^ 1, a_regs);
            __syncthreads();
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) b_cur[j] = b_next[j];
    }

    // ---- row sums of the activations (for the +1 weight code): 4 adjacent threads share a row ----
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        int s = rowsum[i];
        s += __shfl_xor(s, 1, 64);
        s += __shfl_xor(s, 2, 64);
        if ((tid & 3) == 0) lds_rowsum[(tid + 256 * i) >> 2] = s;
    }
    __syncthreads();

    // ---- epilogue ----
    const float ws = p.out ? *p.w_scale : 0.0f;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int lrow = wm * WTM + i * 16 + lg * 4 + r;
            const int row = m0 + lrow;
            if (row >= p.m) continue;
            const int rs = lds_rowsum[lrow];
            const float as = p.out ? p.a_scale[row] : 1.0f;
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int col = n0 + wn * WTN + j * 16 + lr;
                if (col >= p.n) continue;
                const int total = acc[i][j][r] - rs;
                const size_t o = (size_t)row * p.n + col;
                if (p.acc) p.acc[o] = total;
                if (p.out) {
                    float v = f32_div(f32_mul((float)total, ws), as);
                    if (p.bias) v = f32_add(v, p.bias[col]);
                    if (p.residual) v = f32_add(v, p.residual[o]);
                    p.out[o] = v;
                }
            }
        }
    }
}

template <int BM, int BN>
int launch_tile(GemmParams p, hipStream_t stream)
{
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = (p.n + BN - 1) / BN;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL((gemm_tiled_kernel<BM, BN>), dim3(grid), dim3(256), 0, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemm_tiled_kernel");
    return BITNET_HIP_OK;
}

}  // namespace

int launch_gemm_tiled(const uint8_t *tiled, const int8_t *a, size_t m, size_t n, size_t k, int32_t *acc,
                      const float *w_scale, const float *a_scale, const float *bias, const float *residual,
                      float *out, hipStream_t stream)
{
    if (m == 0 || n == 0) return BITNET_HIP_OK;
    GemmParams p;
    p.w = tiled; p.a = a; p.acc = acc; p.w_scale = w_scale; p.a_scale = a_scale; p.bias = bias;
    p.residual = residual; p.out = out; p.m = (int)m; p.n = (int)n; p.k = (int)k; p.kt_count = (int)k_tiles(k);
    p.tiles_m = p.tiles_n = 0;
    // Tile choice: the largest tile that still gives every compute unit work.
    const size_t big = ((m + 255) / 256) * ((n + 255) / 256);
    if (m >= 256 && big >= 200) return launch_tile<256, 256>(p, stream);
    if (m >= 128) return launch_tile<128, 128>(p, stream);
    return launch_tile<64, 64>(p, stream);
}

}  // namespace bitnet
