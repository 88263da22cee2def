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
// Two kernels share this scheme.
//
// gemm_dma_kernel (k a multiple of 256, 16-byte aligned activations, row sums supplied by the activation
// quantiser): activations AND weight tiles travel global -> LDS with LDS-direct loads
// (global_load_lds_dwordx4), never through registers.  Three LDS stages of 128 columns are kept in flight;
// the wait counts are placed by hand (s_waitcnt vmcnt(N)) so that two stages of loads stay outstanding
// while one is computed.  An LDS-direct load writes lane l's 16 bytes at base + 16*l, so the XOR swizzle
// that keeps the fragment reads free of bank conflicts is applied to the global address each lane fetches.
//
// gemm_tiled_kernel (any shape, computes the row sums itself): activations pass through registers.
// Activations are staged through LDS one weight tile (256 columns) at a time, double buffered: the global
// loads of stage s+1 are issued before the 4 k-steps of stage s are computed and written to LDS after them,
// one barrier per stage.  Rows are padded to 272 bytes so that the 16-byte fragment reads of 8 consecutive
// lanes fall in distinct banks.
#include <cstdlib>

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
    const int32_t *a_sum;  // sum_k a[t, k] per token row (required by gemm_dma_kernel)
    float *out;
    int m, n, k;
    int kt_count;   // 256-column weight tiles per row block
    int tiles_m, tiles_n;
};

constexpr int STAGE_K = 256;              // columns per pipeline stage = one weight tile
constexpr int LDS_PITCH = STAGE_K + 16;   // bytes per activation row in LDS

// BM x BN output tile per workgroup of 256 threads (2 x 2 wavefronts).
template <int BM, int BN>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(GemmParams p)
{
    constexpr int WTM = BM / 2, WTN = BN / 2;       // wavefront tile
    constexpr int FM = WTM / 16, FN = WTN / 16;     // MFMA tiles per wavefront
    constexpr int A_LOADS = BM / 16;                // 16-byte chunks each thread moves per stage
    static_assert(WTM % 16 == 0 && WTN % 16 == 0 && A_LOADS >= 1, "tile shape");

    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    uint8_t *lds_a0 = lds_raw, *lds_a1 = lds_raw + BM * LDS_PITCH;
    int *lds_rowsum = reinterpret_cast<int *>(lds_raw + 2 * BM * LDS_PITCH);

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

    // ---- activation tile movement: chunk c = tid + 256*i -> row c / 16, 16-byte column chunk c % 16 ----
    const bool a_vec = (p.k % 16 == 0) && ((reinterpret_cast<uintptr_t>(p.a) & 15) == 0);
    const int a_row = tid >> 4, a_chunk = tid & 15;
    int rowsum[A_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) rowsum[i] = 0;

    auto load_a = [&](int kt, uint4 (&regs)[A_LOADS]) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const int row = m0 + a_row + 16 * i, col = kt * STAGE_K + a_chunk * 16;
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
    auto store_a = [&](uint8_t *buf, const uint4 (&regs)[A_LOADS]) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            *reinterpret_cast<uint4 *>(&buf[(a_row + 16 * i) * LDS_PITCH + a_chunk * 16]) = regs[i];
            int s = rowsum[i];
            s = __builtin_amdgcn_sdot4((int)regs[i].x, 0x01010101, s, false);
            s = __builtin_amdgcn_sdot4((int)regs[i].y, 0x01010101, s, false);
            s = __builtin_amdgcn_sdot4((int)regs[i].z, 0x01010101, s, false);
            s = __builtin_amdgcn_sdot4((int)regs[i].w, 0x01010101, s, false);
            rowsum[i] = s;
        }
    };

    // ---- weight tiles: one uint4 per lane per 16-row block per 256 columns ----
    const int rb0 = (n0 + wn * WTN) / 16;
    const int rb_count = (p.n + 15) / 16;
    const uint4 *wbase = reinterpret_cast<const uint4 *>(p.w) + lane;
    auto load_b = [&](int kt, uint4 (&regs)[FN]) {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int rb = rb0 + j;
            regs[j] = rb < rb_count ? wbase[((size_t)rb * p.kt_count + kt) * 64]
                                    : make_uint4(0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u);
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
    store_a(lds_a0, a_regs);
    __syncthreads();

    for (int kt = 0; kt < p.kt_count; ++kt) {
        uint8_t *cur = (kt & 1) ? lds_a1 : lds_a0;
        uint8_t *nxt = (kt & 1) ? lds_a0 : lds_a1;
        const bool more = kt + 1 < p.kt_count;
        if (more) {
            load_a(kt + 1, a_regs);
            load_b(kt + 1, b_next);
        }
        const uint8_t *arow = cur + (wm * WTM + lr) * LDS_PITCH + lg * 16;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            v4i afrag[FM];
#pragma unroll
            for (int i = 0; i < FM; ++i)
                afrag[i] = *reinterpret_cast<const v4i *>(arow + i * 16 * LDS_PITCH + t * 64);
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
        }
        if (more) {
            store_a(nxt, a_regs);
#pragma unroll
            for (int j = 0; j < FN; ++j) b_cur[j] = b_next[j];
        }
        __syncthreads();
    }

    // ---- row sums of the activations (for the +1 weight code): 16 adjacent threads share a row ----
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        int s = rowsum[i];
        s += __shfl_xor(s, 1, 64);
        s += __shfl_xor(s, 2, 64);
        s += __shfl_xor(s, 4, 64);
        s += __shfl_xor(s, 8, 64);
        if (a_chunk == 0) lds_rowsum[a_row + 16 * i] = s;
    }
    __syncthreads();

    // ---- epilogue ----
    const float ws = p.out ? *p.w_scale : 0.0f;
    const unsigned ws_expo = (__builtin_bit_cast(unsigned, ws) >> 23) & 0xffu;
    const bool ws_fast = ws > 0.0f && ws_expo > 64u && ws_expo < 160u;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int lrow = wm * WTM + i * 16 + lg * 4 + r;
            const int row = m0 + lrow;
            if (row >= p.m) continue;
            const int rs = lds_rowsum[lrow];
            const float as = p.out ? p.a_scale[row] : 1.0f;
            const float as_recip = f32_div(1.0f, as);
            // the short division needs a well-behaved divisor (per row) and dividends in range: float(total) * ws
            // is zero or has ws's exponent plus at most 24, so one check on ws covers them.  The choice is made
            // per wavefront so that the usual case runs no plain division at all.
            const bool row_fast = ws_fast && invariant_divisor_ok(as);
            const bool wave_fast = __builtin_amdgcn_ballot_w64(!row_fast) == 0;
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int col = n0 + wn * WTN + j * 16 + lr;
                if (col >= p.n) continue;
                const int total = acc[i][j][r] - rs;
                const size_t o = (size_t)row * p.n + col;
                if (p.acc) p.acc[o] = total;
                if (p.out) {
                    const float scaled = f32_mul((float)total, ws);
                    float v = wave_fast ? div_by_invariant_unchecked(scaled, as, as_recip) : f32_div(scaled, as);
                    if (p.bias) v = f32_add(v, p.bias[col]);
                    if (p.residual) v = f32_add(v, p.residual[o]);
                    p.out[o] = v;
                }
            }
        }
    }
}

// ---- LDS-direct pipeline -------------------------------------------------------------------------------

__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_off)
{
    // m0 carries the LDS base of the wavefront's 1 KiB destination; lane l lands at base + 16*l
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off\n\t" : : "v"(gptr), "s"(lds_off) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_vm()
{
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

constexpr int DMA_SK = 128;  // columns per activation stage
constexpr int DMA_NST = 3;   // activation stages in LDS

template <int BM, int BN>
constexpr size_t dma_lds_bytes() { return (size_t)DMA_NST * BM * DMA_SK + 2 * (BN / 16) * 1024; }

template <int BM, int BN>
__global__ __launch_bounds__(256, 2) void gemm_dma_kernel(GemmParams p)
{
    constexpr int WTM = BM / 2, WTN = BN / 2, FM = WTM / 16, FN = WTN / 16;
    constexpr int A_STAGE = BM * DMA_SK;
    constexpr int A_DMA = A_STAGE / 1024 / 4;  // LDS-direct loads per wavefront per activation stage
    constexpr int B_TILES = BN / 16;           // weight tiles per 256 columns
    constexpr int B_DMA = (B_TILES + 3) / 4;   // per wavefront (the last ones may repeat a tile)
    constexpr int B_STAGE = B_TILES * 1024;
    static_assert(A_STAGE % 4096 == 0 && WTM % 16 == 0 && WTN % 16 == 0, "tile shape");

    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];  // [NST][A_STAGE] then [2][B_STAGE]
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, lr = lane & 15, lg = lane >> 4;

    int tile_id;
    {
        const int total = p.tiles_m * p.tiles_n;
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        const int per_xcd = (total + 7) >> 3;
        tile_id = xcd * per_xcd + idx;
        if (tile_id >= total) return;
    }
    const int tm = tile_id / p.tiles_n, tn = tile_id % p.tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    const int nstage = p.kt_count * 2;

    // Activation loads: load q of this wavefront covers tile rows 8*(wave*A_DMA + q) .. +7; lane l lands in
    // row l/8 at physical 16-byte chunk l%8 and therefore fetches logical chunk (l%8) ^ (row & 7).
    // Rows past m re-read row m-1 (their results are never stored).
    const int8_t *a_src[A_DMA];
#pragma unroll
    for (int q = 0; q < A_DMA; ++q) {
        const int row = 8 * (wave * A_DMA + q) + (lane >> 3);
        const int lc = (lane & 7) ^ (row & 7);
        int grow = m0 + row;
        if (grow >= p.m) grow = p.m - 1;
        a_src[q] = p.a + (size_t)grow * p.k + lc * 16;
    }
    auto issue_a = [&](int s) {
        const uint32_t dst = lds_base + (s % DMA_NST) * A_STAGE + wave * A_DMA * 1024;
#pragma unroll
        for (int q = 0; q < A_DMA; ++q) dma16(a_src[q] + (size_t)s * DMA_SK, dst + q * 1024);
    };
    // Weight tiles: wavefront w fetches tiles w, w+4, ... of the workgroup's BN/16 row blocks; lane l = slot l.
    const int rb0 = n0 / 16;
    const int rb_last = (p.n + 15) / 16 - 1;
    auto issue_b = [&](int kt) {
        const uint32_t dst = lds_base + DMA_NST * A_STAGE + (kt & 1) * B_STAGE;
#pragma unroll
        for (int q = 0; q < B_DMA; ++q) {
            int tix = wave + 4 * q;
            if (tix >= B_TILES) tix = B_TILES - 1;
            int rb = rb0 + tix;
            if (rb > rb_last) rb = rb_last;
            dma16(p.w + (((size_t)rb * p.kt_count + kt) * 64 + lane) * 16, dst + tix * 1024);
        }
    };

    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = (v4i){0, 0, 0, 0};

    issue_b(0);
    issue_a(0);
    issue_a(1);

    uint32_t a_rd[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) a_rd[i] = (wm * WTM + i * 16 + lr) * DMA_SK;
    const int sw = lr & 7;

    auto compute = [&](int s, int kt, bool second_half) {
        const uint8_t *abuf = lds + (s % DMA_NST) * A_STAGE;
        const uint8_t *bbuf = lds + DMA_NST * A_STAGE + (kt & 1) * B_STAGE + (wn * FN) * 1024 + lane * 16;
        uint4 bp[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) bp[j] = *reinterpret_cast<const uint4 *>(bbuf + j * 1024);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            v4i afrag[FM];
#pragma unroll
            for (int i = 0; i < FM; ++i)
                afrag[i] = *reinterpret_cast<const v4i *>(abuf + a_rd[i] + (((t * 4 + lg) ^ sw) << 4));
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const uint32_t wd = second_half ? (t == 0 ? bp[j].z : bp[j].w) : (t == 0 ? bp[j].x : bp[j].y);
                v4i bfrag;
                bfrag[0] = (int)(wd & 0x03030303u);
                bfrag[1] = (int)((wd >> 2) & 0x03030303u);
                bfrag[2] = (int)((wd >> 4) & 0x03030303u);
                bfrag[3] = (int)((wd >> 6) & 0x03030303u);
#pragma unroll
                for (int i = 0; i < FM; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afrag[i], bfrag, acc[i][j], 0, 0, 0);
            }
        }
    };

    // Loads retire in issue order.  At the top of stage s everything issued before the previous stage's
    // issue group must have landed; that group (A_DMA loads, plus B_DMA after an even stage) may stay in flight.
    for (int s = 0; s < nstage; s += 2) {
        const int kt = s >> 1;
        wait_vm<A_DMA>();  // the previous (odd) stage issued one activation stage only
        __syncthreads();
        if (kt + 1 < p.kt_count) issue_b(kt + 1);
        if (s + 2 < nstage) issue_a(s + 2);
        compute(s, kt, false);

        if (s + 2 < nstage) {
            if (kt + 1 < p.kt_count) wait_vm<A_DMA + B_DMA>(); else wait_vm<A_DMA>();
        } else {
            wait_vm<0>();
        }
        __syncthreads();
        if (s + 3 < nstage) issue_a(s + 3);
        compute(s + 1, kt, true);
    }

    const float ws = p.out ? *p.w_scale : 0.0f;
    const unsigned ws_expo = (__builtin_bit_cast(unsigned, ws) >> 23) & 0xffu;
    const bool ws_fast = ws > 0.0f && ws_expo > 64u && ws_expo < 160u;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = m0 + wm * WTM + i * 16 + lg * 4 + r;
            if (row >= p.m) continue;
            const int rs = p.a_sum[row];
            const float as = p.out ? p.a_scale[row] : 1.0f;
            const float as_recip = f32_div(1.0f, as);
            // the short division needs a well-behaved divisor (per row) and dividends in range: float(total) * ws
            // is zero or has ws's exponent plus at most 24, so one check on ws covers them.  The choice is made
            // per wavefront so that the usual case runs no plain division at all.
            const bool row_fast = ws_fast && invariant_divisor_ok(as);
            const bool wave_fast = __builtin_amdgcn_ballot_w64(!row_fast) == 0;
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int col = n0 + wn * WTN + j * 16 + lr;
                if (col >= p.n) continue;
                const int total = acc[i][j][r] - rs;
                const size_t o = (size_t)row * p.n + col;
                if (p.acc) p.acc[o] = total;
                if (p.out) {
                    const float scaled = f32_mul((float)total, ws);
                    float v = wave_fast ? div_by_invariant_unchecked(scaled, as, as_recip) : f32_div(scaled, as);
                    if (p.bias) v = f32_add(v, p.bias[col]);
                    if (p.residual) v = f32_add(v, p.residual[o]);
                    p.out[o] = v;
                }
            }
        }
    }
}

template <int BM, int BN>
int launch_dma(GemmParams p, hipStream_t stream)
{
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = (p.n + BN - 1) / BN;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    constexpr size_t lds = dma_lds_bytes<BM, BN>();
    static bool attr_set = false;
    if (lds > 64 * 1024 && !attr_set) {
        BITNET_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_dma_kernel<BM, BN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    hipLaunchKernelGGL((gemm_dma_kernel<BM, BN>), dim3(grid), dim3(256), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemm_dma_kernel");
    return BITNET_HIP_OK;
}

template <int BM, int BN>
int launch_tile(GemmParams p, hipStream_t stream)
{
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = (p.n + BN - 1) / BN;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    constexpr size_t lds = 2 * BM * LDS_PITCH + BM * sizeof(int);
    static bool attr_set = false;  // raising the dynamic LDS limit is per kernel, once per process
    if (lds > 64 * 1024 && !attr_set) {
        BITNET_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_tiled_kernel<BM, BN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    hipLaunchKernelGGL((gemm_tiled_kernel<BM, BN>), dim3(grid), dim3(256), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemm_tiled_kernel");
    return BITNET_HIP_OK;
}

}  // namespace

int launch_gemm_tiled(const uint8_t *tiled, const int8_t *a, const int32_t *a_sum, size_t m, size_t n, size_t k,
                      int32_t *acc, const float *w_scale, const float *a_scale, const float *bias,
                      const float *residual, float *out, hipStream_t stream)
{
    if (m == 0 || n == 0) return BITNET_HIP_OK;
    GemmParams p;
    p.w = tiled; p.a = a; p.acc = acc; p.w_scale = w_scale; p.a_scale = a_scale; p.bias = bias;
    p.residual = residual; p.a_sum = a_sum; p.out = out; p.m = (int)m; p.n = (int)n; p.k = (int)k; p.kt_count = (int)k_tiles(k);
    p.tiles_m = p.tiles_n = 0;
    // Tile choice: wide in n (weights live in registers, so a wider tile costs no LDS traffic); among the
    // candidates take the one whose tile count wastes the fewest slots of the last round over 256 CUs.
    const bool dma_ok = a_sum != nullptr && m >= 96 && k % 256 == 0 && k >= 512 &&
                        (reinterpret_cast<uintptr_t>(a) & 15) == 0 && !getenv("BITNET_HIP_GEMM_NO_DMA");
    if (dma_ok) {
        // Tile width: the time of a launch is set by the compute unit that gets the most tiles, each tile
        // costing about its width (a 256-wide tile is ~10 % cheaper per column: fewer LDS reads per MFMA).
        auto cost = [&](size_t bn, double per_col) {
            const size_t tiles = ((m + 127) / 128) * ((n + bn - 1) / bn);
            return (double)((tiles + 255) / 256) * (double)bn * per_col;
        };
        int bn = 160;
        double best = cost(160, 1.0);
        if (cost(256, 0.9) < best) { best = cost(256, 0.9); bn = 256; }
        if (cost(128, 1.03) < best) { best = cost(128, 1.03); bn = 128; }
        if (const char *force = getenv("BITNET_HIP_GEMM_TILE")) bn = atoi(force);  // tuning aid
        if (bn == 256) return launch_dma<128, 256>(p, stream);
        if (bn == 128) return launch_dma<128, 128>(p, stream);
        return launch_dma<128, 160>(p, stream);
    }
    if (m < 96) return launch_tile<64, 128>(p, stream);
    if (const char *force = getenv("BITNET_HIP_GEMM_TILE")) {  // tuning aid
        const int bn = atoi(force);
        if (bn == 256) return launch_tile<128, 256>(p, stream);
        if (bn == 160) return launch_tile<128, 160>(p, stream);
        if (bn == 128) return launch_tile<128, 128>(p, stream);
    }
    auto waste = [&](size_t bn) {
        const size_t tiles = ((m + 127) / 128) * ((n + bn - 1) / bn), slots = 256;
        const size_t rounds = (tiles + slots - 1) / slots;
        return (double)(rounds * slots) / (double)tiles;
    };
    const double w256 = waste(256), w160 = waste(160), w128 = waste(128);
    if (w256 <= w160 && w256 <= w128) return launch_tile<128, 256>(p, stream);
    if (w160 <= w128) return launch_tile<128, 160>(p, stream);
    return launch_tile<128, 128>(p, stream);
}

}  // namespace bitnet
