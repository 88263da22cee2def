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
// Three kernels share this scheme.
//
// gemm_dma_kernel (k a multiple of 256, 16-byte aligned activations, row sums supplied by the activation
// quantiser): activations AND weight tiles travel global -> LDS with LDS-direct loads
// (global_load_lds_dwordx4), never through registers.  D LDS stages of 128 columns are kept in flight;
// the wait counts are placed by hand (s_waitcnt vmcnt(N)) so that D - 1 stages of loads stay outstanding
// while one is computed (D = 2 in the shipped instances: a plain double buffer, which leaves LDS and registers for
// three or four workgroups per compute unit).  An LDS-direct load writes lane l's 16 bytes at base + 16*l, so the XOR swizzle
// that keeps the fragment reads free of bank conflicts is applied to the global address each lane fetches.
// The MFMA takes the weight fragment as its first operand, so a lane ends up with four consecutive output
// columns of one token row and the epilogue stores 16 bytes per lane.  The epilogue's per-row operands (a_sum,
// a_scale) arrive by LDS-direct loads in the stage buffer that is free during the last stage; the usual case
// (f32 output only, n % 4 == 0, scales within the short division's range) is straight-line code
// (store_fragments_fast), everything else goes through store_fragments_general: same bits.
//
// gemm_ld8_kernel: the same data path with eight multiplying and two loading wavefronts per workgroup, for launches
// with at most one tile per compute unit (see its own comment).
//
// gemm_tiled_kernel (any shape, computes the row sums itself): activations pass through registers.
// Activations are staged through LDS one weight tile (256 columns) at a time, double buffered: the global
// loads of stage s+1 are issued before the 4 k-steps of stage s are computed and written to LDS after them,
// one barrier per stage.  Rows are padded to 272 bytes so that the 16-byte fragment reads of 8 consecutive
// lanes fall in distinct banks.
#include "kernels.hpp"
#include "ldsdma.hpp"

namespace bitnet {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

struct GemmProjDev {  // one projection of a launch of the LDS-direct kernels
    const uint8_t *w;
    const float *w_scale;
    const float *bias;
    const float *residual;
    float *out;
    int32_t *acc;
    int n;
    int tn_end;  // column tiles of projections 0..this one, cumulative
};

struct GemmParams {
    GemmProjDev proj[GEMM_MAX_PROJ];  // LDS-direct kernels: projections sharing the activation matrix
    int nproj;
    // single-projection view (the register-staged kernel)
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
    int rotate;     // gemm_dma_kernel: every workgroup of the launch is resident at once (see there)
    // gemm_dma_kernel<..., SPLIT = true>: k split across nsplit workgroups per output tile, st_per (even) stages each
    int nsplit, st_per;
    int *partials;        // [tile][part][fragment][thread] int4
    unsigned *counters;   // one per output tile, zero at launch; the last workgroup of a tile leaves it zero again
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

// Per-row epilogue operands of a BM-row tile, fetched into LDS by LDS-direct loads (no registers are held across
// the k loop): a_sum[BM] as int32, then a_scale[BM].  Wavefront w < BM/64 fetches rows 64*w .. of a_sum, the
// next BM/64 wavefronts the same rows of a_scale (skipped when there is no f32 output and hence no a_scale).
// Rows past m re-read row m-1.  The reader waits for vmcnt(0) and a workgroup barrier first.
template <int BM>
constexpr int rowp_bytes() { return BM * 8; }
template <int BM>
__device__ __forceinline__ void fetch_row_operands(const GemmParams &p, int m0, int wave, int lane, uint32_t lds_rowp)
{
    constexpr int CH = BM / 64;
    static_assert(BM % 64 == 0, "row operand chunks");
    if (wave < 2 * CH) {
        const int chunk = wave < CH ? wave : wave - CH;
        int grow = m0 + chunk * 64 + lane;
        if (grow >= p.m) grow = p.m - 1;
        if (wave < CH) dma4(p.a_sum, (uint32_t)grow * 4u, lds_rowp + chunk * 256);
        else if (p.a_scale) dma4(p.a_scale, (uint32_t)grow * 4u, lds_rowp + BM * 4 + chunk * 256);
    }
}

// The epilogue of one wavefront's fragments on the usual path: f32 output only, n % 4 == 0, w_scale and every
// a_scale of the tile suited to the short division (the caller checks).  Straight-line code: per output element
// a subtraction, a conversion, two multiplications, two FMAs and a sign copy; one 16-byte store per fragment row.
// Fragment i of lane l holds token row rows[i], columns col0 + 16*j + 0..3.  FULL: the tile lies inside the
// matrix, no bounds checks.  EXTRA: bias and / or residual may be present.
template <int NI, int FN, bool FULL, bool EXTRA>
__device__ __forceinline__ void store_fragments_fast(const v4i (&acc)[NI][FN], const int (&rs)[NI], const float (&as)[NI],
                                                     const float (&rcp)[NI], float ws, const GemmProjDev &PJ, int m,
                                                     const int (&rows)[NI], int col0)
{
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        if (!FULL && rows[i] >= m) continue;
        const size_t o = (size_t)rows[i] * PJ.n + col0;
        float *orow = PJ.out + o;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            if (!FULL && col0 + j * 16 >= PJ.n) continue;  // n % 4 == 0: a fragment row is inside or outside as a whole
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                v[r] = div_by_invariant_unchecked(f32_mul((float)(acc[i][j][r] - rs[i]), ws), as[i], rcp[i]);
            if (EXTRA) {
                if (PJ.bias) {
                    const float4 b = *reinterpret_cast<const float4 *>(PJ.bias + col0 + j * 16);
                    v[0] = f32_add(v[0], b.x); v[1] = f32_add(v[1], b.y); v[2] = f32_add(v[2], b.z); v[3] = f32_add(v[3], b.w);
                }
                if (PJ.residual) {
                    const float4 q = *reinterpret_cast<const float4 *>(PJ.residual + o + j * 16);
                    v[0] = f32_add(v[0], q.x); v[1] = f32_add(v[1], q.y); v[2] = f32_add(v[2], q.z); v[3] = f32_add(v[3], q.w);
                }
            }
            *reinterpret_cast<float4 *>(orow + j * 16) = make_float4(v[0], v[1], v[2], v[3]);
        }
    }
}

// The epilogue for every other case (int32 accumulator output, n % 4 != 0, scales outside the short division's
// range): the same arithmetic, choices made per fragment row, a_sum and a_scale read from global memory.
template <int NI, int FN>
__device__ __forceinline__ void store_fragments_general(const v4i (&acc)[NI][FN], const int (&rows)[NI], int col0, float ws,
                                                        bool ws_fast, const GemmProjDev &PJ, const GemmParams &p)
{
    const bool vec_ok = (PJ.n & 3) == 0;  // 16-byte alignment of out[row][4c]
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int row = rows[i];
        const bool row_ok = row < p.m;
        const int rs = row_ok ? p.a_sum[row] : 0;
        const float as = (PJ.out && row_ok) ? p.a_scale[row] : 1.0f;
        const float as_recip = f32_div(1.0f, as);
        // the short division needs a well-behaved divisor (per row) and dividends in range: float(total) * ws
        // is zero or has ws's exponent plus at most 24, so one check on ws covers them.  The choice is made
        // per wavefront so that the usual case runs no plain division at all.
        const bool row_fast = ws_fast && invariant_divisor_ok(as);
        const bool wave_fast = __builtin_amdgcn_ballot_w64(!row_fast) == 0;
        if (!row_ok) continue;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int col = col0 + j * 16;
            if (col >= PJ.n) continue;
            const size_t o = (size_t)row * PJ.n + col;
            int tot[4];
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                tot[r] = acc[i][j][r] - rs;
                const float scaled = f32_mul((float)tot[r], ws);
                v[r] = wave_fast ? div_by_invariant_unchecked(scaled, as, as_recip) : f32_div(scaled, as);
            }
            if (vec_ok) {  // col + 3 < n follows from n % 4 == 0
                if (PJ.acc) *reinterpret_cast<int4 *>(PJ.acc + o) = make_int4(tot[0], tot[1], tot[2], tot[3]);
                if (PJ.out) {
                    if (PJ.bias) {
                        const float4 b = *reinterpret_cast<const float4 *>(PJ.bias + col);
                        v[0] = f32_add(v[0], b.x); v[1] = f32_add(v[1], b.y); v[2] = f32_add(v[2], b.z); v[3] = f32_add(v[3], b.w);
                    }
                    if (PJ.residual) {
                        const float4 q = *reinterpret_cast<const float4 *>(PJ.residual + o);
                        v[0] = f32_add(v[0], q.x); v[1] = f32_add(v[1], q.y); v[2] = f32_add(v[2], q.z); v[3] = f32_add(v[3], q.w);
                    }
                    *reinterpret_cast<float4 *>(PJ.out + o) = make_float4(v[0], v[1], v[2], v[3]);
                }
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (col + r >= PJ.n) continue;
                    if (PJ.acc) PJ.acc[o + r] = tot[r];
                    if (PJ.out) {
                        float y = v[r];
                        if (PJ.bias) y = f32_add(y, PJ.bias[col + r]);
                        if (PJ.residual) y = f32_add(y, PJ.residual[o + r]);
                        PJ.out[o + r] = y;
                    }
                }
            }
        }
    }
}

// The whole epilogue of one wavefront.  Fragment i of lane l holds token row m0 + lrows[i] (lrows: row inside the
// BM-row tile), columns col0 + 16*j + 0..3.  rowp is the LDS copy of the tile's a_sum and a_scale
// (fetch_row_operands), complete and visible: the caller has waited for vmcnt(0) and passed a workgroup barrier.
// full: the workgroup's tile lies inside the matrix.
template <int BM, int NI, int FN>
__device__ __forceinline__ void finish_fragments(const v4i (&acc)[NI][FN], const int (&lrows)[NI], int m0, int col0, bool full,
                                                 const uint8_t *rowp, const GemmProjDev &PJ, const GemmParams &p)
{
    const float ws = PJ.out ? *PJ.w_scale : 0.0f;
    const unsigned ws_expo = (__builtin_bit_cast(unsigned, ws) >> 23) & 0xffu;
    const bool ws_fast = ws > 0.0f && ws_expo > 64u && ws_expo < 160u;
    int rows[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) rows[i] = m0 + lrows[i];
    if (PJ.out && !PJ.acc && (PJ.n & 3) == 0 && ws_fast) {
        const int *sum_l = reinterpret_cast<const int *>(rowp);
        const float *scale_l = reinterpret_cast<const float *>(rowp + BM * 4);
        int rs[NI];
        float as[NI], rcp[NI];
        bool ok = true;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            rs[i] = sum_l[lrows[i]];
            as[i] = scale_l[lrows[i]];
            rcp[i] = f32_div(1.0f, as[i]);
            ok = ok && invariant_divisor_ok(as[i]);
        }
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
            const bool extra = PJ.bias != nullptr || PJ.residual != nullptr;
            if (full && !extra) store_fragments_fast<NI, FN, true, false>(acc, rs, as, rcp, ws, PJ, p.m, rows, col0);
            else if (full) store_fragments_fast<NI, FN, true, true>(acc, rs, as, rcp, ws, PJ, p.m, rows, col0);
            else if (!extra) store_fragments_fast<NI, FN, false, false>(acc, rs, as, rcp, ws, PJ, p.m, rows, col0);
            else store_fragments_fast<NI, FN, false, true>(acc, rs, as, rcp, ws, PJ, p.m, rows, col0);
            return;
        }
    }
    store_fragments_general<NI, FN>(acc, rows, col0, ws, ws_fast, PJ, p);
}

constexpr int DMA_SK = 128;  // columns per activation stage; a 256-column weight tile serves two stages

// D activation stages and NB weight buffers live in LDS; loads run P = D - 1 stages ahead of the MFMAs.
template <int D>
constexpr int dma_nb() { return (D - 1 + 2 + 1) / 2; }
template <int BM, int BN, int D>
constexpr size_t dma_lds_bytes() { return (size_t)D * BM * DMA_SK + (size_t)dma_nb<D>() * (BN / 16) * 1024; }

// Loads of the groups issued after stage s's own group and before the wait at the top of stage s: the groups
// of stages s+1 .. s+P-1; a group holds A_DMA activation loads, plus B_DMA weight loads when its stage is even.
template <int PHASE, int P, int A_DMA, int B_DMA>
constexpr int dma_in_flight()
{
    int n = 0;
    for (int j = 1; j < P; ++j) n += A_DMA + (((PHASE + j) & 1) == 0 ? B_DMA : 0);
    return n;
}

// Four ints exchanged between workgroups inside one launch: device-scope (relaxed atomic) stores and loads, which the
// hardware writes through to, and reads from, the level every XCD shares, 8 bytes at a time.
__device__ __forceinline__ void store_shared4(int *ptr, v4i v)
{
    typedef volatile __attribute__((address_space(1))) v4i gv4i;
    *(gv4i *)(uintptr_t)ptr = v;
}
__device__ __forceinline__ v4i load_shared4(const int *ptr)
{
    typedef const volatile __attribute__((address_space(1))) v4i gv4i;
    return *(gv4i *)(uintptr_t)ptr;
}

template <int BM, int BN, int D, int OCC, bool SPLIT = false>
__global__ __launch_bounds__(256, OCC) void gemm_dma_kernel(GemmParams p)
{
    constexpr int WTM = BM / 2, WTN = BN / 2, FM = WTM / 16, FN = WTN / 16;
    constexpr int P = D - 1, NB = dma_nb<D>();
    constexpr int A_STAGE = BM * DMA_SK;
    constexpr int A_DMA = A_STAGE / 1024 / 4;  // LDS-direct loads per wavefront per activation stage
    constexpr int B_TILES = BN / 16;           // weight tiles per 256 columns
    constexpr int B_DMA = (B_TILES + 3) / 4;   // per wavefront (the last ones may repeat a tile)
    constexpr int B_STAGE = B_TILES * 1024;
    static_assert(A_STAGE % 4096 == 0 && WTM % 16 == 0 && WTN % 16 == 0 && D >= 2, "tile shape");
    static_assert(dma_in_flight<0, P, A_DMA, B_DMA>() < 64 && dma_in_flight<1, P, A_DMA, B_DMA>() < 64, "vmcnt range");

    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];  // [D][A_STAGE] then [NB][B_STAGE]
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, lr = lane & 15, lg = lane >> 4;

    int tile_id, ks = 0;
    {
        const int nsplit = SPLIT ? p.nsplit : 1;
        const int total = p.tiles_m * p.tiles_n * nsplit;
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        const int per_xcd = (total + 7) >> 3;
        tile_id = xcd * per_xcd + idx;
        if (tile_id >= total) return;
        if (SPLIT) { ks = tile_id % nsplit; tile_id /= nsplit; }  // the parts of a tile are neighbours: one XCD
    }
    // tiles_n counts the column tiles of all projections of the launch, one after the other
    const int tm = tile_id / p.tiles_n, tn_all = tile_id % p.tiles_n;
    int pj = 0;
    if (p.nproj > 1 && tn_all >= p.proj[0].tn_end) pj = 1;
    if (p.nproj > 2 && tn_all >= p.proj[1].tn_end) pj = 2;
    const GemmProjDev PJ = p.proj[pj];  // uniform over the workgroup
    const int tn = tn_all - (pj ? p.proj[pj - 1].tn_end : 0);
    const int m0 = tm * BM, n0 = tn * BN;
    const int s_first = SPLIT ? __builtin_amdgcn_readfirstlane(ks * p.st_per) : 0;  // even
    const int nstage = SPLIT ? min(p.st_per, p.kt_count * 2 - s_first) : p.kt_count * 2;  // stages of this workgroup (even)

    // Activation loads: load q of this wavefront covers tile rows 8*(wave*A_DMA + q) .. +7; lane l lands in
    // row l/8 at physical 16-byte chunk l%8 and therefore fetches logical chunk (l%8) ^ (row & 7).
    // Rows past m re-read row m-1 (their results are never stored).
    uint32_t a_off[A_DMA];  // byte offsets into the activation matrix (below 4 GiB: checked by the launcher)
#pragma unroll
    for (int q = 0; q < A_DMA; ++q) {
        const int row = 8 * (wave * A_DMA + q) + (lane >> 3);
        const int lc = (lane & 7) ^ (row & 7);
        int grow = m0 + row;
        if (grow >= p.m) grow = p.m - 1;
        a_off[q] = (uint32_t)grow * (uint32_t)p.k + lc * 16;
    }
    // Weight tiles: wavefront w fetches tiles w, w+4, ... of the workgroup's BN/16 row blocks; lane l = slot l.
    const int rb0 = n0 / 16;
    const int rb_last = (PJ.n + 15) / 16 - 1;
    uint32_t b_off[B_DMA], b_dst[B_DMA];  // byte offsets into the re-tiled weights, tile positions in a weight stage
#pragma unroll
    for (int q = 0; q < B_DMA; ++q) {
        int tix = wave + 4 * q;
        if (tix >= B_TILES) tix = B_TILES - 1;
        int rb = rb0 + tix;
        if (rb > rb_last) rb = rb_last;
        b_off[q] = ((uint32_t)rb * (uint32_t)p.kt_count * 64 + lane) * 16;
        b_dst[q] = tix * 1024;
    }
    // The load group of stage s: the weight tile of k-tile s/2 when s is even, then the activation stage.
    auto issue = [&](int s) {
        if ((s & 1) == 0) {
            const int kt = s >> 1;
            const uint32_t dst = lds_base + D * A_STAGE + (kt % NB) * B_STAGE;
#pragma unroll
            for (int q = 0; q < B_DMA; ++q) dma16(PJ.w + (size_t)(kt + (s_first >> 1)) * 1024, b_off[q], dst + b_dst[q]);
        }
        const uint32_t dst = lds_base + (s % D) * A_STAGE + wave * A_DMA * 1024;
#pragma unroll
        for (int q = 0; q < A_DMA; ++q) dma16(p.a + (size_t)(s + s_first) * DMA_SK, a_off[q], dst + q * 1024);
    };

    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = (v4i){0, 0, 0, 0};

#pragma unroll
    for (int s = 0; s < P; ++s)
        if (s < nstage) issue(s);

    uint32_t a_rd[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) a_rd[i] = (wm * WTM + i * 16 + lr) * DMA_SK;
    const int sw = lr & 7;

    // The MFMA computes C^T: the weight fragment is the first operand, so that result register r of lane l is
    // out[token row l % 16][output column 4*(l/16) + r]: four consecutive columns, one 16-byte store.
    uint4 bp[FN];  // the wavefront's slots of the current weight tiles: read at an even stage, used by two
    auto compute = [&](int s, bool second_half) {
        const int kt = s >> 1;
        const uint8_t *abuf = lds + (s % D) * A_STAGE;
        if (!second_half) {
            const uint8_t *bbuf = lds + D * A_STAGE + (kt % NB) * B_STAGE + (wn * FN) * 1024 + lane * 16;
#pragma unroll
            for (int j = 0; j < FN; ++j) bp[j] = *reinterpret_cast<const uint4 *>(bbuf + j * 1024);
        }
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
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bfrag, afrag[i], acc[i][j], 0, 0, 0);
            }
        }
    };

    // Loads retire in issue order.  At the top of stage s its own group must have landed; the groups of the
    // P - 1 later stages stay in flight.  The last P - 1 stages, with fewer groups behind them, drain everything.
    // When the whole launch is resident at once (OCC workgroups on every compute unit, all started together), the
    // hardware's oldest-first choice among wavefronts lets the OCC workgroups of a compute unit finish one after the
    // other, the last one running alone at a fraction of the MFMA rate.  Workgroup ids b, b + 256, ... share a
    // compute unit; rotating their wavefront priorities every k-tile keeps them level (measured: 5 % at
    // 2048 x 6912 x 2560).  With several rounds of workgroups the staggered finish is wanted and nothing is done.
    const int rank = blockIdx.x >> 8;
    for (int s = 0; s < nstage; s += 2) {
        if (p.rotate) set_wave_priority((rank + (s >> 1)) % OCC);
        if (s + P <= nstage) wait_vm<dma_in_flight<0, P, A_DMA, B_DMA>()>(); else wait_vm<0>();
        __syncthreads();
        if (s + P < nstage) issue(s + P);
        compute(s, false);

        if (s + 1 + P <= nstage) wait_vm<dma_in_flight<1, P, A_DMA, B_DMA>()>(); else wait_vm<0>();
        __syncthreads();
        if (s + 1 + P < nstage) issue(s + 1 + P);
        // In the last stage the buffer of the stage before it is free: the per-row epilogue operands land there
        // while the last MFMAs run.
        else if (s + 2 == nstage) fetch_row_operands<BM>(p, m0, wave, lane, lds_base + (s % D) * A_STAGE);
        compute(s + 1, true);
    }
    const uint32_t ROWP = ((nstage - 2) % D) * A_STAGE;
    static_assert(rowp_bytes<BM>() <= A_STAGE, "row operands fit an activation stage");
    wait_vm<0>();
    __syncthreads();
    if constexpr (SPLIT) {
        // Every part stores its int32 fragments (device-scope stores: written through to where every XCD reads them),
        // waits until they have been acknowledged, and draws a ticket from the tile's counter; the part that draws the
        // last one adds up all parts (integers: any order, same sum), leaves the counter at zero and runs the epilogue.
        // Nobody waits for anybody.
        __shared__ int last_ticket;
        constexpr int SLAB = FM * FN * 256 * 4;
        int *mine = p.partials + ((size_t)tile_id * p.nsplit + ks) * SLAB;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) store_shared4(mine + ((i * FN + j) * 256 + tid) * 4, acc[i][j]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (tid == 0)
            last_ticket = __hip_atomic_fetch_add(&p.counters[tile_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)(p.nsplit - 1);
        __syncthreads();
        if (!last_ticket) return;  // uniform over the workgroup
        if (tid == 0) __hip_atomic_store(&p.counters[tile_id], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int *slab = p.partials + (size_t)tile_id * p.nsplit * SLAB;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = (v4i){0, 0, 0, 0};
        for (int part = 0; part < p.nsplit; ++part, slab += SLAB)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) acc[i][j] += load_shared4(slab + ((i * FN + j) * 256 + tid) * 4);
    }
    int lrows[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) lrows[i] = wm * WTM + i * 16 + lr;
    finish_fragments<BM, FM, FN>(acc, lrows, m0, n0 + wn * WTN + lg * 4, m0 + BM <= p.m && n0 + BN <= PJ.n, lds + ROWP, PJ, p);
}

// Raising a kernel's dynamic LDS limit is needed once per process; a function-local static makes that once
// thread-safe (forward may be called from many threads).
template <typename Kernel>
hipError_t raise_lds_limit(Kernel kernel, size_t bytes)
{
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

template <int BM, int BN, int D, int OCC>
int launch_dma(GemmParams p, hipStream_t stream)
{
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = 0;
    for (int j = 0; j < p.nproj; ++j) p.proj[j].tn_end = p.tiles_n += (p.proj[j].n + BN - 1) / BN;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    p.rotate = total <= 256 * OCC && total > 256;
    constexpr size_t lds = dma_lds_bytes<BM, BN, D>();
    static_assert(lds <= 160 * 1024 && lds * OCC <= 160 * 1024 && OCC <= 4, "LDS budget, priorities 0..3");
    static const hipError_t attr = lds > 64 * 1024 ? raise_lds_limit(&gemm_dma_kernel<BM, BN, D, OCC>, lds) : hipSuccess;
    BITNET_HIP_TRY(attr);
    hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, D, OCC>), dim3(grid), dim3(256), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemm_dma_kernel");
    return BITNET_HIP_OK;
}

// ---- eight MFMA wavefronts per workgroup fed by two loader wavefronts -------------------------------------------
//
// For launches with at most one 128 x 160 tile per compute unit.  One wavefront per SIMD cannot keep the MFMA pipe
// busy (its own LDS waits and unpack instructions sit between its MFMAs); two can.  With too few tiles for two
// workgroups per compute unit the second wavefront per SIMD comes from inside the workgroup: wavefronts 0..3 take
// columns 0..127 of every 256-column stage and wavefronts 4..7 columns 128..255, each group accumulating the whole
// BM x BN tile; the two partial tiles are exchanged through LDS at the end (int32 sums: exact), each group
// finishing half of the fragments.  A stage is one 256-column weight tile plus BM x 256 activation bytes, three
// stages in LDS, loads two stages ahead.
// The LDS-direct loads are issued by two further wavefronts (8 and 9) that never multiply.  A wavefront that issues
// a load while the queue of the load path is full waits at that instruction, and while it waits it issues no MFMA;
// with the loads spread over the multiplying wavefronts every one of them paid that wait every stage (measured at
// 2048 x 2560 x 6912: 40.8 us with the loads on the eight wavefronts, 33.6 us with no loads in the loop at all,
// 35.8 us with the two loaders).  The multiplying wavefronts meet the loaders at the stage barrier and otherwise
// only read LDS and run MFMAs.
constexpr int LD8_NST = 3;
// The same kernel with k split across nsplit workgroups per output tile (st_per stages each; see the kernel's SPLIT branch).
template <int BM, int BN, int D, int OCC>
int launch_dma_split(GemmParams p, int nsplit, int st_per, const GemmSplitScratch &scratch, hipStream_t stream)
{
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = 0;
    for (int j = 0; j < p.nproj; ++j) p.proj[j].tn_end = p.tiles_n += (p.proj[j].n + BN - 1) / BN;
    const size_t tiles = (size_t)p.tiles_m * p.tiles_n;
    if (tiles * nsplit * BM * BN * sizeof(int32_t) > scratch.partial_bytes || tiles > scratch.counter_count)
        return fail(BITNET_HIP_MEMORY_ERROR, "split-k GEMM: scratch of %zu bytes / %zu counters for %zu tiles in %d parts",
                    scratch.partial_bytes, scratch.counter_count, tiles, nsplit);
    p.nsplit = nsplit; p.st_per = st_per; p.rotate = 0;
    p.partials = scratch.partials; p.counters = scratch.counters;
    const int total = (int)tiles * nsplit;
    const int grid = ((total + 7) / 8) * 8;
    constexpr size_t lds = dma_lds_bytes<BM, BN, D>();
    static const hipError_t attr = lds > 64 * 1024 ? raise_lds_limit(&gemm_dma_kernel<BM, BN, D, OCC, true>, lds) : hipSuccess;
    BITNET_HIP_TRY(attr);
    hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, D, OCC, true>), dim3(grid), dim3(256), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemm_dma_kernel (k split)");
    return BITNET_HIP_OK;
}

template <int BM, int BN>
constexpr size_t ld8_lds_bytes() { return (size_t)LD8_NST * (BM * 256 + (BN / 16) * 1024) + rowp_bytes<BM>(); }

template <int BM, int BN>
__global__ __launch_bounds__(640, 1) void gemm_ld8_kernel(GemmParams p)
{
    constexpr int WTM = BM / 2, WTN = BN / 2, FM = WTM / 16, FN = WTN / 16;
    constexpr int A_STAGE = BM * 256;
    constexpr int A_CHUNKS = A_STAGE / 1024;    // 1 KiB LDS-direct loads per stage
    constexpr int B_TILES = BN / 16;
    constexpr int B_STAGE = B_TILES * 1024;
    constexpr int STAGE = A_STAGE + B_STAGE;
    constexpr int A_PER = A_CHUNKS / 2, B_PER = (B_TILES + 1) / 2;  // per loader wavefront
    constexpr int GROUP = A_PER + B_PER;
    static_assert(A_CHUNKS % 2 == 0 && WTM % 32 == 0 && WTN % 16 == 0 && 2 * GROUP < 64, "tile shape, vmcnt range");
    static_assert((FM / 2) * FN * 4 * 256 * 8 <= LD8_NST * STAGE, "exchange area");

    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];  // [NST][A half 0 | A half 1 | B], then the row operands
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    int tile_id;
    {
        const int total = p.tiles_m * p.tiles_n;
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        const int per_xcd = (total + 7) >> 3;
        tile_id = xcd * per_xcd + idx;
        if (tile_id >= total) return;
    }
    const int tm = tile_id / p.tiles_n, tn_all = tile_id % p.tiles_n;
    int pj = 0;
    if (p.nproj > 1 && tn_all >= p.proj[0].tn_end) pj = 1;
    if (p.nproj > 2 && tn_all >= p.proj[1].tn_end) pj = 2;
    const GemmProjDev PJ = p.proj[pj];  // uniform over the workgroup
    const int tn = tn_all - (pj ? p.proj[pj - 1].tn_end : 0);
    const int m0 = tm * BM, n0 = tn * BN;
    constexpr uint32_t ROWP = LD8_NST * STAGE;

    if (wave >= 8) {
        // ---- loader wavefront L: activation chunks A_PER*L .. and weight tiles B_PER*L .. of every stage ----
        const int L = wave - 8;
        uint32_t a_off[A_PER], b_off[B_PER], b_dst[B_PER];
#pragma unroll
        for (int q = 0; q < A_PER; ++q) {
            const int c = L * A_PER + q;
            const int half = c / (BM / 8), row = 8 * (c % (BM / 8)) + (lane >> 3);
            const int lc = (lane & 7) ^ (row & 7);
            int grow = m0 + row;
            if (grow >= p.m) grow = p.m - 1;
            a_off[q] = (uint32_t)grow * (uint32_t)p.k + half * 128 + lc * 16;
        }
        const int rb0 = n0 / 16, rb_last = (PJ.n + 15) / 16 - 1;
#pragma unroll
        for (int q = 0; q < B_PER; ++q) {
            int tix = L * B_PER + q;
            if (tix >= B_TILES) tix = B_TILES - 1;
            int rb = rb0 + tix;
            if (rb > rb_last) rb = rb_last;
            b_off[q] = ((uint32_t)rb * (uint32_t)p.kt_count * 64 + lane) * 16;
            b_dst[q] = A_STAGE + tix * 1024;
        }
        auto issue = [&](int kt) {
            const uint32_t stage = lds_base + (kt % LD8_NST) * STAGE;
#pragma unroll
            for (int q = 0; q < B_PER; ++q) dma16(PJ.w + (size_t)kt * 1024, b_off[q], stage + b_dst[q]);
#pragma unroll
            for (int q = 0; q < A_PER; ++q) dma16(p.a + (size_t)kt * 256, a_off[q], stage + (L * A_PER + q) * 1024);
        };
        // the per-row epilogue operands: a_sum by loader 0, a_scale by loader 1 (BM / 64 loads of 64 rows each)
#pragma unroll
        for (int ch = 0; ch < BM / 64; ++ch) {
            int grow = m0 + ch * 64 + lane;
            if (grow >= p.m) grow = p.m - 1;
            if (L == 0) dma4(p.a_sum, (uint32_t)grow * 4u, lds_base + ROWP + ch * 256);
            else if (p.a_scale) dma4(p.a_scale, (uint32_t)grow * 4u, lds_base + ROWP + BM * 4 + ch * 256);
        }
        issue(0);
        if (p.kt_count > 1) issue(1);
        for (int kt = 0; kt < p.kt_count; ++kt) {
            if (kt + 1 < p.kt_count) wait_vm<GROUP>(); else wait_vm<0>();
            __syncthreads();
            if (kt + 2 < p.kt_count) issue(kt + 2);
        }
        __syncthreads();  // the two barriers of the exchange
        __syncthreads();
        return;
    }

    const int kg = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1, lr = lane & 15, lg = lane >> 4;
    v4i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = (v4i){0, 0, 0, 0};
    uint32_t a_rd[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) a_rd[i] = kg * (BM * 128) + (wm * WTM + i * 16 + lr) * 128;
    const int sw = lr & 7;

    auto compute = [&](int kt) {
        const uint8_t *abuf = lds + (kt % LD8_NST) * STAGE;
        const uint8_t *bbuf = abuf + A_STAGE + (wn * FN) * 1024 + lane * 16 + kg * 8;
        uint2 bp[FN];  // dwords 2*kg, 2*kg+1 of the slot: this group's two k-steps
#pragma unroll
        for (int j = 0; j < FN; ++j) bp[j] = *reinterpret_cast<const uint2 *>(bbuf + j * 1024);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            v4i afrag[FM];
#pragma unroll
            for (int i = 0; i < FM; ++i)
                afrag[i] = *reinterpret_cast<const v4i *>(abuf + a_rd[i] + (((t * 4 + lg) ^ sw) << 4));
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const uint32_t wd = t == 0 ? bp[j].x : bp[j].y;
                v4i bfrag;
                bfrag[0] = (int)(wd & 0x03030303u);
                bfrag[1] = (int)((wd >> 2) & 0x03030303u);
                bfrag[2] = (int)((wd >> 4) & 0x03030303u);
                bfrag[3] = (int)((wd >> 6) & 0x03030303u);
#pragma unroll
                for (int i = 0; i < FM; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bfrag, afrag[i], acc[i][j], 0, 0, 0);
            }
        }
    };
    for (int kt = 0; kt < p.kt_count; ++kt) {
        __syncthreads();  // the loaders arrive here once stage kt has landed
        compute(kt);
    }

    // ---- exchange: group 0 finishes fragments i < FM/2, group 1 the others ----
    __syncthreads();  // every wavefront is done with the stage buffers
    constexpr int HALF = FM / 2;
    {
        v4i *xch = reinterpret_cast<v4i *>(lds);
        const int mine = wave, partner = wave ^ 4;
#pragma unroll
        for (int i = 0; i < HALF; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
                xch[((mine * HALF + i) * FN + j) * 64 + lane] = acc[kg == 0 ? i + HALF : i][j];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < HALF; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const v4i o = xch[((partner * HALF + i) * FN + j) * 64 + lane];
                if (kg == 0) acc[i][j] += o; else acc[i + HALF][j] += o;
            }
    }
    v4i fin[HALF][FN];
    int lrows[HALF];
#pragma unroll
    for (int ii = 0; ii < HALF; ++ii) {
        lrows[ii] = wm * WTM + (ii + kg * HALF) * 16 + lr;
#pragma unroll
        for (int j = 0; j < FN; ++j) fin[ii][j] = kg == 0 ? acc[ii][j] : acc[ii + HALF][j];
    }
    finish_fragments<BM, HALF, FN>(fin, lrows, m0, n0 + wn * WTN + lg * 4, m0 + BM <= p.m && n0 + BN <= PJ.n, lds + ROWP, PJ, p);
}

template <int BM, int BN>
int launch_ld8(GemmParams p, hipStream_t stream)
{
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = 0;
    for (int j = 0; j < p.nproj; ++j) p.proj[j].tn_end = p.tiles_n += (p.proj[j].n + BN - 1) / BN;
    const int total = p.tiles_m * p.tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    constexpr size_t lds = ld8_lds_bytes<BM, BN>();
    static_assert(lds <= 160 * 1024, "LDS budget");
    static const hipError_t attr = raise_lds_limit(&gemm_ld8_kernel<BM, BN>, lds);
    BITNET_HIP_TRY(attr);
    hipLaunchKernelGGL((gemm_ld8_kernel<BM, BN>), dim3(grid), dim3(640), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemm_ld8_kernel");
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
    static const hipError_t attr = lds > 64 * 1024 ? raise_lds_limit(&gemm_tiled_kernel<BM, BN>, lds) : hipSuccess;
    BITNET_HIP_TRY(attr);
    hipLaunchKernelGGL((gemm_tiled_kernel<BM, BN>), dim3(grid), dim3(256), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemm_tiled_kernel");
    return BITNET_HIP_OK;
}

}  // namespace

// Up to GEMM_MAX_PROJ projections of the same activation matrix in one launch of the LDS-direct kernels (q, k, v
// or gate, up at prefill: small projections alone would leave most compute units idle).  Returns
// BITNET_HIP_UNSUPPORTED (without a message) when the shapes do not fit those kernels.
namespace {
// k split across workgroups: where, and into how many parts of how many 128-column stages (even).  tiles32: 64 x 32
// tiles of the launch.  One round of workgroups at four per compute unit holds 1024: three parts of at most 352 tiles.
bool plan_split(size_t m, size_t k, size_t tiles32, int *nsplit, int *st_per)
{
    if (m <= 96 || k < 4096 || k % 256 != 0 || tiles32 == 0 || tiles32 > 352) return false;
    const int nstage = (int)(k / 128);
    const int per = ((nstage + 2) / 3 + 1) & ~1;
    const int parts = (nstage + per - 1) / per;
    if (parts < 2) return false;
    *nsplit = parts; *st_per = per;
    return true;
}
}  // namespace

void gemm_split_plan(size_t m, size_t k, const size_t *n, int nproj, size_t *partial_bytes, size_t *counters)
{
    *partial_bytes = 0; *counters = 0;
    if (nproj <= 0 || nproj > GEMM_MAX_PROJ) return;
    size_t tiles32 = 0;
    for (int j = 0; j < nproj; ++j) tiles32 += ((m + 63) / 64) * ((n[j] + 31) / 32);
    int nsplit = 0, st_per = 0;
    if (!plan_split(m, k, tiles32, &nsplit, &st_per)) return;
    *partial_bytes = (tiles32 * nsplit * 64 * 32 * sizeof(int32_t) + 255) / 256 * 256;
    *counters = tiles32;
}

int launch_gemm_multi(const GemvProj *projs, int nproj, const int8_t *a, const int32_t *a_sum, const float *a_scale,
                      size_t m, size_t k, hipStream_t stream, const GemmSplitScratch *split)
{
    if (m == 0 || nproj <= 0) return BITNET_HIP_OK;
    if (nproj > GEMM_MAX_PROJ) return BITNET_HIP_UNSUPPORTED;
    bool dma_ok = a_sum != nullptr && m >= 96 && k % 256 == 0 && k >= 512 && (reinterpret_cast<uintptr_t>(a) & 15) == 0 &&
                  m * k < (1ull << 32);  // 32-bit lane offsets
    size_t tiles = 0, tiles128 = 0, tiles64 = 0, tiles32 = 0;  // 128 x 160 tiles; 128 x 128 tiles, or 0 if a projection is not a multiple of 128 wide
    bool all128 = true;
    GemmParams p = {};
    for (int j = 0; j < nproj && dma_ok; ++j) {
        const GemvProj &s = projs[j];
        dma_ok = s.n > 0 && s.n <= 0x7fffffffu && tiled_bytes(s.n, k) < (1ull << 32);
        tiles += ((m + 127) / 128) * ((s.n + 159) / 160);
        tiles128 += ((m + 127) / 128) * ((s.n + 127) / 128);
        tiles64 += ((m + 63) / 64) * ((s.n + 63) / 64);
        tiles32 += ((m + 63) / 64) * ((s.n + 31) / 32);
        all128 = all128 && s.n % 128 == 0;
        GemmProjDev &d = p.proj[j];
        d.w = s.tiled; d.w_scale = s.w_scale; d.bias = s.bias; d.residual = s.residual; d.out = s.out; d.acc = s.acc;
        d.n = (int)s.n; d.tn_end = 0;
    }
    if (!dma_ok) return BITNET_HIP_UNSUPPORTED;
    if (!all128) tiles128 = 0;
    for (int j = nproj; j < GEMM_MAX_PROJ; ++j) p.proj[j] = p.proj[nproj - 1];
    p.nproj = nproj; p.a = a; p.a_sum = a_sum; p.a_scale = a_scale; p.m = (int)m; p.k = (int)k; p.kt_count = (int)k_tiles(k);
    // Three shapes of the LDS-direct kernel, chosen by how many 128 x 160 tiles the outputs hold (256 compute
    // units; the MFMA pipe of a SIMD needs two or more resident wavefronts to stay busy).  Measured:
    //   2.5 or more tiles per compute unit   -> 128 x 160, three workgroups of 4 wavefronts per compute unit, two
    //                                           activation stages each (more resident wavefronts beat deeper
    //                                           pipelines: 2.45 POP/s at 8192 x 2560 x 6912, against 2.23 with two
    //                                           workgroups of three stages);
    //   0.4 to one tile per compute unit     -> 128 x 160, one workgroup of 8 multiplying wavefronts (k split inside it)
    //                                           and two loader wavefronts;
    //   otherwise                            -> 64 x 160, four workgroups of 4 wavefronts per compute unit.
    // A long k with few tiles: the 64 x 32 tiles of the launch in three parts of k each (plan_split).  Measured at
    // 6912 -> 2560: 128 / 192 / 256 tokens 15.7 / 15.7 / 17.9 us -> 12.1 / 13.2 / 14.6 us; from 320 tokens on, and at
    // k = 2560 at any token count, the partial tiles cost more to exchange than the shorter loops save.
    if (split && split->partials) {
        int nsplit = 0, st_per = 0;
        if (plan_split(m, k, tiles32, &nsplit, &st_per)) return launch_dma_split<64, 32, 4, 4>(p, nsplit, st_per, *split, stream);
    }
    if (tiles >= 640) return launch_dma<128, 160, 2, 3>(p, stream);
    // Few tiles: a workgroup walks the whole of k by itself and its time is a chain of load latencies, so small
    // launches take narrow tiles (more workgroups, all resident at once) with four stages of loads in flight.
    // tiles64 / tiles32: 64 x 64 and 64 x 32 tiles of the launch.  Measured at 6912 -> 2560: 384 tokens 35.4 -> 23.3 us,
    // 512 tokens 36.6 -> 25.8 us (64 x 32), 768 tokens 38.0 -> 29.6 us, 1024 tokens 36.8 -> 34.3 us (64 x 64);
    // 2560 -> 6912 at 192 tokens 17.5 -> 13.6 us, at 384 tokens 20.0 -> 17.7 us.
    if (tiles < 100 && tiles32 <= 704) return launch_dma<64, 32, 4, 4>(p, stream);
    if (tiles <= 140 && tiles64 <= 768) return launch_dma<64, 64, 4, 3>(p, stream);
    if (tiles >= 100 && tiles <= 256) return launch_ld8<128, 160>(p, stream);
    // between one and 2.5 tiles of 128 x 160 per compute unit: 128 x 128 tiles when they divide every projection and
    // fill the 768 workgroup slots almost three times (q + k + v at 3072 tokens: 33.0 us against 37.9 us with 64 x 160)
    if (tiles > 256 && tiles128 >= 640) return launch_dma<128, 128, 2, 3>(p, stream);
    return launch_dma<64, 160, 2, 4>(p, stream);
}

int launch_gemm_tiled(const uint8_t *tiled, const int8_t *a, const int32_t *a_sum, size_t m, size_t n, size_t k,
                      int32_t *acc, const float *w_scale, const float *a_scale, const float *bias,
                      const float *residual, float *out, hipStream_t stream)
{
    if (m == 0 || n == 0) return BITNET_HIP_OK;
    {
        const GemvProj one = {tiled, w_scale, bias, residual, out, acc, n};
        const int rc = launch_gemm_multi(&one, 1, a, a_sum, a_scale, m, k, stream);
        if (rc != BITNET_HIP_UNSUPPORTED) return rc;
    }
    GemmParams p = {};
    p.w = tiled; p.a = a; p.acc = acc; p.w_scale = w_scale; p.a_scale = a_scale; p.bias = bias;
    p.residual = residual; p.a_sum = a_sum; p.out = out; p.m = (int)m; p.n = (int)n; p.k = (int)k; p.kt_count = (int)k_tiles(k);
    p.tiles_m = p.tiles_n = 0;
    if (m < 96) return launch_tile<64, 128>(p, stream);
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

// ---- matrix-unit rate (diagnostic) -----------------------------------------------------------------------------
// A loop of nothing but v_mfma_i32_16x16x64_i8 with its operands in registers: eight independent accumulators per
// wavefront, two wavefronts per SIMD on every compute unit.  What it sustains is the ceiling of the GEMM above on the
// device at hand (clock under a matrix load included); RANDOM gives every lane different int8 activations and 2-bit
// codes 0..2 as weights, as the GEMM's operands are, otherwise every byte of both operands is 1.
namespace {
template <bool RANDOM>
__global__ __launch_bounds__(512, 1) void mfma_rate_kernel(int iters, int *sink, unsigned seed)
{
    v4i acc[8], a[4], b[4];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = (v4i){0, 0, 0, 0};
    unsigned w = seed * (threadIdx.x + 1) * 2654435761u + blockIdx.x * 97u + 12345u;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            w = w * 1664525u + 1013904223u;
            a[i][c] = RANDOM ? (int)w : 0x01010101;
            w = w * 1664525u + 1013904223u;
            const unsigned two = (w >> 8) & 0x03030303u;  // bytes 0..3; 3 becomes 2 (no carry between bytes)
            b[i][c] = RANDOM ? (int)(two - ((two >> 1) & two & 0x01010101u)) : 0x01010101;
        }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b[i & 3], a[(i + (i >> 2)) & 3], acc[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
}
}  // namespace

int launch_mfma_rate(bool random_operands, int iters, int compute_units, int *sink, hipStream_t stream)
{
    const dim3 grid((unsigned)compute_units), block(MFMA_RATE_THREADS);
    if (random_operands) hipLaunchKernelGGL((mfma_rate_kernel<true>), grid, block, 0, stream, iters, sink, 7u);
    else hipLaunchKernelGGL((mfma_rate_kernel<false>), grid, block, 0, stream, iters, sink, 7u);
    BITNET_HIP_CHECK_LAUNCH("mfma_rate_kernel");
    return BITNET_HIP_OK;
}

}  // namespace bitnet
