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
// offset 16*l of a 1 KiB tile: row r = l mod 16, four groups of 16 columns.  Activations sit in LDS; the 16
// lanes of a group read the same LDS address (a broadcast).  Partial sums are combined with two wavefront
// shuffles (the four lanes of a row), then across the four wavefronts through LDS.
//
// Two more things are folded into the same launch, because at one token the cost of a decode step is the
// number of dependent launches, not bytes:
//   * the activation quantiser: with MODE >= 0 the workgroup reads the f32 row itself, runs RMSNorm +
//     absmax + int8 rounding (rowquant.hpp, the same code and summation order as the stand-alone
//     quantiser) and writes the int8 row straight into LDS.  The weight tiles are requested first, so
//     their HBM latency overlaps this prologue.
//   * up to three projections that share the input row (q, k, v or gate, up): the grid is the
//     concatenation of their row blocks.
// HBM traffic per call: n*k/4 weight bytes; the input row (K or 4K bytes per workgroup) comes from L2.
// gemv_fused16_kernel is this launch with 16 wavefronts per workgroup (the default for one token; see its comment).
//
// gemv_mfma_kernel is the same weight-streaming scheme for 2..16 token rows: the 16 x 16 x 64 int8 MFMA takes
// the place of the dot-product chain (its A operand is 16 token rows x 64 columns, loaded straight from the
// int8 activation matrix, which stays in L2; its B operand is a decoded weight dword, exactly as in the
// prefill GEMM), so up to 16 tokens cost what one costs in weight traffic and instructions.  A workgroup
// owns RB adjacent 16-row blocks so that the activation matrix is re-read by fewer workgroups.
#include "kernels.hpp"
#include "rowquant.hpp"
#include "tiledot.hpp"
#include "ldsdma.hpp"

namespace bitnet {

namespace {

constexpr int MODE_PREQUANT = -1;
constexpr int GEMV_FUSED_MAX_ROWS = 8;   // tokens per fused quantiser + GEMV launch (a set of workgroups per token)
constexpr int GEMV_FUSED_MAX_WGS = 512;  // and its workgroups over all tokens: one round on 256 compute units
constexpr int FUSED_NCH = 7;  // 16-byte f32 chunks per thread kept in registers: K <= 7168

struct GemvProjDev {
    const uint8_t *w;
    const float *w_scale;
    const float *bias;
    const float *residual;
    float *out;
    int32_t *acc;
    int n;
    int rb_end;  // row blocks of projections 0..this one, cumulative
};

struct GemvParams {
    GemvProjDev proj[GEMV_MAX_PROJ];
    int nproj;
    // MODE_PREQUANT: activations already int8
    const int8_t *a;
    const float *a_scale;
    // MODE >= 0: f32 input, quantised in the prologue
    RowSource src;
    int8_t *q_out;        // optional copies of what the prologue produced (written by workgroup 0)
    float *a_scale_out;
    int32_t *a_sum_out;
    int m;  // tokens in this launch (<= MB)
    int k;
    int kt_count;
};

constexpr int GEMV_PREFETCH = 4;  // tiles in flight per wavefront

template <int MB, int MODE>
__global__ __launch_bounds__(256) void gemv_tiled_kernel(GemvParams p)
{
    extern __shared__ uint4 lds_a[];  // [MB][groups]: int8 activations, 16 per uint4, zero past K / past m
    __shared__ int red[4][TILE_ROWS][MB];
    __shared__ float red_f[MB][2][4];
    __shared__ int red_i[MB][4];
    __shared__ float scale_s[MB];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int groups = p.kt_count * 16;

    // which projection, which of its row blocks
    int pj = 0;
#pragma unroll
    for (int j = 0; j < GEMV_MAX_PROJ - 1; ++j)
        if (j + 1 < p.nproj && (int)blockIdx.x >= p.proj[j].rb_end) pj = j + 1;
    const GemvProjDev &P = p.proj[pj];
    const int rb = (int)blockIdx.x - (pj ? p.proj[pj - 1].rb_end : 0);
    const uint4 *tiles = reinterpret_cast<const uint4 *>(P.w) + (size_t)rb * p.kt_count * 64;

    // Loads retire in issue order, so what the prologue waits for first is requested first: the f32 input row
    // of token 0 and the RMSNorm weights (L2 hits), then the first batch of weight tiles (HBM), whose latency
    // the quantiser prologue then hides.
    float4 v0[MODE == MODE_PREQUANT ? 1 : FUSED_NCH], gm[MODE == MODE_PREQUANT ? 1 : FUSED_NCH];
    if constexpr (MODE != MODE_PREQUANT) {
        const int chunks = p.k >> 2;
        const bool norm = p.src.gamma != nullptr;
#pragma unroll
        for (int i = 0; i < FUSED_NCH; ++i) {
            int c = tid + 256 * i;
            v0[i] = c < chunks ? load_chunk<MODE, true>(p.src, 0, c) : make_float4(0.f, 0.f, 0.f, 0.f);
            gm[i] = (norm && c < chunks) ? load_gamma_chunk(p.src, c, true) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    uint4 wbuf[GEMV_PREFETCH];
#pragma unroll
    for (int u = 0; u < GEMV_PREFETCH; ++u) {
        int kt = wave + 4 * u;
        wbuf[u] = load_weight_slot(tiles + (size_t)min(kt, p.kt_count - 1) * 64 + lane);  // unconditional: the waits can be counted
    }

    if constexpr (MODE == MODE_PREQUANT) {
        // Stage the int8 activations; every thread also accumulates sum_k a[t, k] for the code offset.
        const bool vec_ok = (p.k % 16 == 0) && ((reinterpret_cast<uintptr_t>(p.a) & 15) == 0);
#pragma unroll
        for (int t = 0; t < MB; ++t) {
            int local = 0;
            for (int g = tid; g < groups; g += 256) {
                uint4 v = make_uint4(0, 0, 0, 0);
                if (t < p.m) {
                    const int8_t *srcp = p.a + (size_t)t * p.k + 16 * (size_t)g;
                    if (vec_ok) {
                        if (16 * g < p.k) v = *reinterpret_cast<const uint4 *>(srcp);
                    } else {
                        uint32_t d[4] = {0, 0, 0, 0};
                        for (int j = 0; j < 16; ++j)
                            if (16 * g + j < p.k) d[j >> 2] |= (uint32_t)(uint8_t)srcp[j] << (8 * (j & 3));
                        v = make_uint4(d[0], d[1], d[2], d[3]);
                    }
                }
                lds_a[t * groups + g] = v;
                local = dot4(v.x, 0x01010101u, local);
                local = dot4(v.y, 0x01010101u, local);
                local = dot4(v.z, 0x01010101u, local);
                local = dot4(v.w, 0x01010101u, local);
            }
            local = wave_sum_i32(local);
            if (lane == 0) red_i[t][wave] = local;
            if (tid == 0) scale_s[t] = (t < p.m && p.a_scale) ? p.a_scale[t] : 1.0f;
        }
    } else {
        // Quantise the f32 input row(s) here: thread tid is virtual lane tid of the declared summation order.
        const RowSource &src = p.src;
        const int chunks = p.k >> 2;  // the host takes this path only when K % 4 == 0
        const int lds_words = groups * 4;
        uint32_t *lds_w = reinterpret_cast<uint32_t *>(lds_a);
        const bool norm = src.gamma != nullptr;
#pragma unroll
        for (int t = 0; t < MB; ++t) {
            if (t >= p.m) {  // uniform
                for (int c = tid; c < lds_words; c += 256) lds_w[t * lds_words + c] = 0;
                if (lane == 0) red_i[t][wave] = 0;
                if (tid == 0) scale_s[t] = 1.0f;
                continue;
            }
            float4 v[FUSED_NCH];
#pragma unroll
            for (int i = 0; i < FUSED_NCH; ++i) {
                int c = tid + 256 * i;
                if (t == 0) v[i] = v0[i];
                else v[i] = c < chunks ? load_chunk<MODE, true>(src, (size_t)t, c) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            RowDivisor rdiv = {1.0f, 1.0f, false};
            if (norm) {
                float ss;
                if (src.sum_order == BITNET_HIP_SUM_SEQUENTIAL) {
                    ss = sum_squares_sequential<MODE>(src, (size_t)t);
                } else {
                    float part = 0.0f;
#pragma unroll
                    for (int i = 0; i < FUSED_NCH; ++i) part = sum_squares4(part, v[i]);
                    part = wave_sum_f32(part);
                    if (lane == 0) red_f[t][0][wave] = part;
                    __syncthreads();
                    ss = f32_add(f32_add(f32_add(red_f[t][0][0], red_f[t][0][1]), red_f[t][0][2]), red_f[t][0][3]);
                }
                rdiv = make_row_divisor(rms_from_ss(ss, p.k, src.eps));
            }
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < FUSED_NCH; ++i) {
                int c = tid + 256 * i;
                if (norm && c < chunks) v[i] = normalize4(v[i], rdiv, gm[i]);
                amax = absmax4(amax, v[i]);
            }
            amax = wave_max_f32(amax);
            if (lane == 0) red_f[t][1][wave] = amax;
            __syncthreads();
            amax = fmaxf(fmaxf(red_f[t][1][0], red_f[t][1][1]), fmaxf(red_f[t][1][2], red_f[t][1][3]));
            const float scale = scale_from_absmax(amax);
            int isum = 0;
#pragma unroll
            for (int i = 0; i < FUSED_NCH; ++i) {
                int c = tid + 256 * i;
                if (c < chunks) {
                    uint32_t packed = quant4_packed(v[i], scale, &isum);
                    lds_w[t * lds_words + c] = packed;
                    if (p.q_out && blockIdx.x == 0) reinterpret_cast<uint32_t *>(p.q_out)[(size_t)t * chunks + c] = packed;
                } else if (c < lds_words) {
                    lds_w[t * lds_words + c] = 0;
                }
            }
            isum = wave_sum_i32(isum);
            if (lane == 0) red_i[t][wave] = isum;
            if (tid == 0) scale_s[t] = scale;
        }
    }
    __syncthreads();

    if constexpr (MODE != MODE_PREQUANT) {
        if (blockIdx.x == 0 && tid < MB && tid < p.m) {
            if (p.a_scale_out) p.a_scale_out[tid] = scale_s[tid];
            if (p.a_sum_out) p.a_sum_out[tid] = red_i[tid][0] + red_i[tid][1] + red_i[tid][2] + red_i[tid][3];
        }
    }

    int acc[MB];
#pragma unroll
    for (int t = 0; t < MB; ++t) acc[t] = 0;

    const int kq = lane >> 4;  // lane group: columns 64t + 16kq .. +15 of each tile, t = 0..3
    auto dot_batch = [&](int kt0) {
#pragma unroll
        for (int u = 0; u < GEMV_PREFETCH; ++u) {
            int kt = kt0 + 4 * u;
            if (kt < p.kt_count) {
                const uint4 *ag = lds_a + kt * 16 + kq;
#pragma unroll
                for (int t = 0; t < MB; ++t) acc[t] = dot64(wbuf[u], ag + t * groups, acc[t]);
            }
        }
    };
    for (int kt0 = wave; kt0 < p.kt_count; kt0 += 4 * GEMV_PREFETCH) {
        // two straight-line bodies: the last batch requests nothing more and waits for nothing but itself
        if (kt0 + 4 * GEMV_PREFETCH < p.kt_count) {  // uniform over the wavefront
            uint4 wnext[GEMV_PREFETCH];
#pragma unroll
            for (int u = 0; u < GEMV_PREFETCH; ++u)
                wnext[u] = load_weight_slot(tiles + (size_t)min(kt0 + 4 * (GEMV_PREFETCH + u), p.kt_count - 1) * 64 + lane);
            dot_batch(kt0);
#pragma unroll
            for (int u = 0; u < GEMV_PREFETCH; ++u) wbuf[u] = wnext[u];
        } else {
            dot_batch(kt0);
        }
    }

    // the four lanes l, l+16, l+32, l+48 hold the four column groups of row l mod 16
#pragma unroll
    for (int t = 0; t < MB; ++t) {
        acc[t] = sum_over_lane_groups(acc[t]);
    }
    if (lane < TILE_ROWS) {
#pragma unroll
        for (int t = 0; t < MB; ++t) red[wave][lane][t] = acc[t];
    }
    __syncthreads();

    if (tid < TILE_ROWS * MB) {
        const int r = tid / MB, t = tid % MB;
        const int n = rb * TILE_ROWS + r;
        if (n < P.n && t < p.m) {
            const int asum = red_i[t][0] + red_i[t][1] + red_i[t][2] + red_i[t][3];
            int total = red[0][r][t] + red[1][r][t] + red[2][r][t] + red[3][r][t] - asum;
            size_t o = (size_t)t * P.n + n;
            if (P.acc) P.acc[o] = total;
            if (P.out) {
                float v = f32_mul((float)total, *P.w_scale);
                v = f32_div(v, scale_s[t]);
                if (P.bias) v = f32_add(v, P.bias[n]);
                if (P.residual) v = f32_add(v, P.residual[o]);
                P.out[o] = v;
            }
        }
    }
}

// One token, f32 input: the quantiser runs in the prologue (see the head of this file).  Every load of the
// workgroup - input row, RMSNorm weights, all of its weight tiles - is issued up front and unconditionally
// (indices past the end are clamped and the values discarded), in the order in which the data is needed.  Loads
// return in issue order, so the compiler can wait for "all but the last n" and the weight tiles stay in
// flight while the row is normalised and quantised; the workgroup barriers order LDS traffic only, for the same
// reason.  NCH: 16-byte chunks of the row per thread, and weight tiles per wavefront (k <= 1024 * NCH).
template <int MODE, bool NORM, int NCH, int RBW>
__global__ __launch_bounds__(256) void gemv_fused_kernel(GemvParams p)
{
    extern __shared__ uint4 lds_a[];  // int8 activations, 16 per uint4, zero past K
    __shared__ int red[4][RBW][TILE_ROWS];
    __shared__ float red_f[2][4];
    __shared__ int red_i[4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunks = p.k >> 2, lds_words = p.kt_count * 64;

    int pj = 0;
#pragma unroll
    for (int j = 0; j < GEMV_MAX_PROJ - 1; ++j)
        if (j + 1 < p.nproj && (int)blockIdx.x >= p.proj[j].rb_end) pj = j + 1;
    const GemvProjDev &P = p.proj[pj];
    const int rb0 = ((int)blockIdx.x - (pj ? p.proj[pj - 1].rb_end : 0)) * RBW;  // rb_end counts groups of RBW row blocks
    const int rb_count = (P.n + TILE_ROWS - 1) / TILE_ROWS;
    const uint4 *tiles = reinterpret_cast<const uint4 *>(P.w) + lane;

    float4 v[NCH], gm[NCH];
    uint4 wt[RBW][NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = min(tid + 256 * i, chunks - 1);
        v[i] = load_chunk<MODE, true>(p.src, 0, c);
    }
    // what the epilogue threads need from memory (weight scale, bias, residual of their output row) is requested
    // now as well, so that its latency is not paid at the end
    const int e_n = min((rb0 + (tid >> 4)) * TILE_ROWS + (tid & 15), P.n - 1);  // meaningful for tid < 16 * RBW
    const float e_ws = P.out ? *P.w_scale : 0.0f;
    const float e_bias = P.bias ? P.bias[e_n] : 0.0f;
    const float e_res = P.residual ? P.residual[e_n] : 0.0f;
    if constexpr (NORM) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) gm[i] = load_gamma_chunk(p.src, min(tid + 256 * i, chunks - 1), true);
    }
#pragma unroll
    for (int r = 0; r < RBW; ++r)
#pragma unroll
        for (int u = 0; u < NCH; ++u)  // row blocks past the end repeat the last one; their results are not stored
            wt[r][u] = load_weight_slot(tiles + ((size_t)min(rb0 + r, rb_count - 1) * p.kt_count + min(wave + 4 * u, p.kt_count - 1)) * 64);
#pragma unroll
    for (int i = 0; i < NCH; ++i)
        if (tid + 256 * i >= chunks) v[i] = make_float4(0.f, 0.f, 0.f, 0.f);

    // thread tid is virtual lane tid of the declared summation order
    RowDivisor rdiv = {1.0f, 1.0f, false};
    if constexpr (NORM) {
        float ss;
        if (p.src.sum_order == BITNET_HIP_SUM_SEQUENTIAL) {
            // the reference's literal order: the squares go through LDS (the launch sizes it for them; the int8 row
            // takes the same place later, behind the barrier of the absmax reduction) and every wavefront runs the chain
            float *sq_lds = reinterpret_cast<float *>(lds_a);
#pragma unroll
            for (int i = 0; i < NCH; ++i)
                if (tid + 256 * i < chunks) store_squares4(sq_lds, tid + 256 * i, v[i]);
            lds_barrier();
            ss = sum_sequential_lds(sq_lds, p.k);
        } else {
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < NCH; ++i) part = sum_squares4(part, v[i]);
            part = wave_sum_f32(part);
            if (lane == 0) red_f[0][wave] = part;
            lds_barrier();
            ss = f32_add(f32_add(f32_add(red_f[0][0], red_f[0][1]), red_f[0][2]), red_f[0][3]);
        }
        rdiv = make_row_divisor(rms_from_ss(ss, p.k, p.src.eps));
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        if (NORM && tid + 256 * i < chunks) v[i] = normalize4(v[i], rdiv, gm[i]);
        amax = absmax4(amax, v[i]);
    }
    amax = wave_max_f32(amax);
    if (lane == 0) red_f[1][wave] = amax;
    lds_barrier();
    amax = fmaxf(fmaxf(red_f[1][0], red_f[1][1]), fmaxf(red_f[1][2], red_f[1][3]));
    const float scale = scale_from_absmax(amax);
    uint32_t *lds_w = reinterpret_cast<uint32_t *>(lds_a);
    int isum = 0;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = tid + 256 * i;
        if (c < chunks) {
            const uint32_t packed = quant4_packed(v[i], scale, &isum);
            lds_w[c] = packed;
            if (p.q_out && blockIdx.x == 0) reinterpret_cast<uint32_t *>(p.q_out)[c] = packed;
        } else if (c < lds_words) {
            lds_w[c] = 0;
        }
    }
    isum = wave_sum_i32(isum);
    if (lane == 0) red_i[wave] = isum;
    lds_barrier();

    const int kq = lane >> 4;  // lane group: columns 64t + 16kq .. +15 of each tile, t = 0..3
#pragma unroll
    for (int r = 0; r < RBW; ++r) {
        int acc = 0;
#pragma unroll
        for (int u = 0; u < NCH; ++u) {
            const int kt = wave + 4 * u;
            if (kt < p.kt_count) acc = dot64(wt[r][u], lds_a + kt * 16 + kq, acc);
        }
        // the four lanes l, l+16, l+32, l+48 hold the four column groups of row l mod 16
        acc = sum_over_lane_groups(acc);
        if (lane < TILE_ROWS) red[wave][r][lane] = acc;
    }
    lds_barrier();

    if (tid < TILE_ROWS * RBW) {
        const int r = tid >> 4, row = tid & 15;
        const int n = (rb0 + r) * TILE_ROWS + row;
        const int asum = red_i[0] + red_i[1] + red_i[2] + red_i[3];
        if (blockIdx.x == 0 && tid == 0) {
            if (p.a_scale_out) p.a_scale_out[0] = scale;
            if (p.a_sum_out) p.a_sum_out[0] = asum;
        }
        if (n < P.n) {
            const int total = red[0][r][row] + red[1][r][row] + red[2][r][row] + red[3][r][row] - asum;
            if (P.acc) P.acc[n] = total;
            if (P.out) {
                float y = f32_mul((float)total, e_ws);
                y = f32_div(y, scale);
                if (P.bias) y = f32_add(y, e_bias);
                if (P.residual) y = f32_add(y, e_res);
                P.out[n] = y;
            }
        }
    }
}

// The same launch with up to 16 wavefronts per workgroup.  The prologue of gemv_fused_kernel is redundant arithmetic on
// one wavefront per SIMD (normalise, absmax, quantise: about half of the dependent work of a launch); a thread per
// chunk does the element-wise part four times faster.  A workgroup has nw wavefronts (bs = 64 nw threads), thread t
// owns chunks t, t + bs (NCHB of them) and wavefront w the k-tiles w, w + nw; the sum of squares
// keeps the declared order: chunk c belongs to virtual lane c % 256, whose chain runs over its chunks in ascending
// order, so threads 0..255 (one per virtual lane) also fetch their lane's chunks (from L2, with the first loads of the
// kernel) and add the squares up in that order, then the four 64-lane butterflies as before.
// A 256-column k-tile is the 64 chunks one wavefront quantises, so every wavefront multiplies the tiles of its own
// chunks (for each of the workgroup's RBW row blocks) straight after writing them to LDS, without a workgroup barrier
// between quantiser and dot products; the partial sums of a row meet in LDS atomics.

template <int MODE, bool NORM, int NCHB, int RBW>
__global__ __launch_bounds__(1024) void gemv_fused16_kernel(const float *hot_x, const float *hot_x2, const float *hot_gamma, int hot_k, int hot_head_dim,
                                                           int hot_gqa_group, int hot_ldx, GemvParams p)
{
    // A launch has one to eight tokens (input rows), each with its own workgroups.  Workgroup (x, y) of the grid works on
    // token x / 8 and on group 8y + x % 8 of row blocks: the workgroups of one group are neighbours in dispatch order and,
    // workgroups going to the XCDs in turn, run on the same XCD, so its L2 fetches their weight tiles once.
    // The leading scalar arguments repeat what the first loads need (input rows, RMSNorm weights, k): the file is
    // compiled with kernel-argument preloading, so they arrive in registers with the wavefront instead of through a
    // load from the argument buffer that the first address computation would have to wait for.
    RowSource hot;
    hot.x = hot_x; hot.x2 = hot_x2; hot.gamma = hot_gamma; hot.ldx = (size_t)hot_ldx; hot.k = hot_k; hot.head_dim = hot_head_dim;
    hot.gqa_group = hot_gqa_group & 0xffff; hot.sum_order = BITNET_HIP_SUM_BLOCK256; hot.eps = 0.0f;
    const size_t tok = blockIdx.x >> 3;
    const int group = (int)blockIdx.y * 8 + (int)(blockIdx.x & 7);  // may lie past the last group: such workgroups leave below
    extern __shared__ uint4 lds_a[];  // int8 activations, zero past K
    __shared__ float red_f[2][16];
    __shared__ int red_i[16];
    __shared__ int tot[RBW][TILE_ROWS];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int chunks = hot_k >> 2;
    // A row of at most 1024 chunks is launched with one wavefront per k-tile (at least the four of the summation order)
    // instead of 16: wavefronts without a chunk would only add their share of the redundant arithmetic between the
    // barriers to the SIMDs' queues.  Their slots of the cross-wavefront reductions hold the neutral element.
    const int nw = hot_gqa_group >> 16, bs = nw << 6;  // wavefronts and threads of the workgroup (preloaded with the GQA group)
    if (tid < 16 && tid >= nw) {
        red_f[1][tid] = 0.0f;
        red_i[tid] = 0;
    }

    // Every load is unconditional (clamped indices, values discarded), in the order in which the data is needed.
    // First what the preloaded arguments alone address: the input row and the RMSNorm weights.  The argument buffer is
    // read once these loads are on their way (it takes as long to arrive as the row: both come from memory), then
    // the sum of squares, so that the two latencies run side by side.
    float4 v[NCHB], gm[NORM ? NCHB : 1];
    constexpr int NSS = NORM ? 4 * NCHB : 1;  // chunks per virtual lane of the summation order
#pragma unroll
    for (int i = 0; i < NCHB; ++i) v[i] = load_chunk<MODE, true>(hot, tok, min(tid + bs * i, chunks - 1));
    float4 vs[NSS];
    if constexpr (NORM) {
        if (wave < 4) {  // thread tid < 256 is virtual lane tid: it fetches the lane's chunks itself (from L2)
#pragma unroll
            for (int i = 0; i < NSS; ++i) vs[i] = load_chunk<MODE, true>(hot, tok, min(tid + 256 * i, chunks - 1));
        }
#pragma unroll
        for (int i = 0; i < NCHB; ++i) gm[i] = load_gamma_chunk(hot, min(tid + bs * i, chunks - 1), true);
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing below moves above: the first wait for the argument buffer comes here

    const int lds_words = p.kt_count * 64;
    int pj = 0;
#pragma unroll
    for (int j = 0; j < GEMV_MAX_PROJ - 1; ++j)
        if (j + 1 < p.nproj && group >= p.proj[j].rb_end) pj = j + 1;
    const GemvProjDev &P = p.proj[pj];
    const int rb0 = (group - (pj ? p.proj[pj - 1].rb_end : 0)) * RBW;  // rb_end counts groups of RBW row blocks
    const int rb_count = (P.n + TILE_ROWS - 1) / TILE_ROWS;
    const uint4 *tiles = reinterpret_cast<const uint4 *>(P.w) + lane;
    // k-tile kt holds chunks 64*kt .. 64*kt + 63: exactly what wavefront kt % 16 quantises, so a wavefront multiplies
    // the tiles of its own chunks (tiles and row blocks past the end repeat the last one; their results are not added).
    // When the tiles are requested (measured on the 30-block token step, replayed from a graph): with RMSNorm, once
    // the argument buffer has arrived, ahead of the sum of squares (483.4 us a step against 489.7 behind the first
    // barrier); without it, behind the absmax barrier (requested as early there the step takes 494 us: the weight
    // stream then competes with the input row, which the kernel's chain of reductions hangs on).
    uint4 wt[RBW][NCHB];
    auto request_weight_tiles = [&]() {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < RBW; ++r)
#pragma unroll
            for (int i = 0; i < NCHB; ++i)
                wt[r][i] = load_weight_slot(tiles + ((size_t)min(rb0 + r, rb_count - 1) * p.kt_count + min(wave + nw * i, p.kt_count - 1)) * 64);
        __builtin_amdgcn_sched_barrier(0);
    };
    // epilogue operands: absent ones read the input row instead (always there) and are not used; the weight scale goes
    // through a per-lane address so that it is a vector load, which nothing waits for before the epilogue
    const int e_n = min((rb0 + (tid >> 4)) * TILE_ROWS + (tid & 15), P.n - 1);  // meaningful for tid < 16 * RBW
    int lane_zero = 0;
    asm volatile("" : "+v"(lane_zero));
    const float e_ws = (P.out ? P.w_scale : hot_x)[lane_zero];
    const float e_bias = *(P.bias ? P.bias + e_n : hot_x);
    const float e_res = *(P.residual ? P.residual + (tok * (size_t)P.n + e_n) : hot_x);
    if (tid < RBW * TILE_ROWS) tot[tid >> 4][tid & 15] = 0;
#pragma unroll
    for (int i = 0; i < NCHB; ++i)
        if (tid + bs * i >= chunks) v[i] = make_float4(0.f, 0.f, 0.f, 0.f);

    if constexpr (NORM) {
        request_weight_tiles();
        if (wave < 4) {
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < NSS; ++i)
                if (tid + 256 * i < chunks) part = sum_squares4(part, vs[i]);  // chunks past the end would add +0
            part = wave_sum_f32(part);
            if (lane == 0) red_f[0][wave] = part;
        }
        lds_barrier();
        const float ss = f32_add(f32_add(f32_add(red_f[0][0], red_f[0][1]), red_f[0][2]), red_f[0][3]);
        const RowDivisor rdiv = make_row_divisor(rms_from_ss(ss, p.k, p.src.eps));
#pragma unroll
        for (int i = 0; i < NCHB; ++i)
            if (tid + bs * i < chunks) v[i] = normalize4(v[i], rdiv, gm[i]);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCHB; ++i) amax = absmax4(amax, v[i]);
    amax = wave_max_f32(amax);
    if (lane == 0) red_f[1][wave] = amax;
    lds_barrier();
    if constexpr (!NORM) request_weight_tiles();
    amax = red_f[1][0];
#pragma unroll
    for (int w = 1; w < 16; ++w) amax = fmaxf(amax, red_f[1][w]);
    const float scale = scale_from_absmax(amax);
    uint32_t *lds_w = reinterpret_cast<uint32_t *>(lds_a);
    int isum = 0;
#pragma unroll
    for (int i = 0; i < NCHB; ++i) {
        const int c = tid + bs * i;
        if (c < chunks) {
            const uint32_t packed = quant4_packed(v[i], scale, &isum);
            lds_w[c] = packed;
            if (p.q_out && group == 0) reinterpret_cast<uint32_t *>(p.q_out + tok * (size_t)hot_k)[c] = packed;
        } else if (c < lds_words) {
            lds_w[c] = 0;
        }
    }
    isum = wave_sum_i32(isum);
    if (lane == 0) red_i[wave] = isum;
    // the int8 values this wavefront reads back below are its own: no workgroup barrier, only the LDS queue of the wavefront
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");

    // Dot products on the matrix unit: the tile's 16 rows are the B operand of v_mfma_i32_16x16x64_i8 (lane l: row l mod 16,
    // columns 64t + 16kq .. +15 for dword t, kq = l / 16), the activations are row 0 of the A operand (lanes 0, 16, 32, 48
    // hold the four column groups; the other 15 rows are zero), so result register 0 of lanes 0..15 is the sum over the
    // 64 columns of step t for rows 0..15.  Against dot4 this leaves only the unpacking of the 2-bit codes on the VALU.
    typedef int v4i_t __attribute__((ext_vector_type(4)));
    const int kq = lane >> 4;
    const bool row0 = (lane & 15) == 0;
#pragma unroll
    for (int i = 0; i < NCHB; ++i) {
        const int kt = wave + nw * i;
        if (kt < p.kt_count) {  // uniform over the wavefront
            // row blocks in batches of at most four: the accumulators of a batch are 16 registers
            constexpr int RBB = RBW < 4 ? RBW : 4;
#pragma unroll
            for (int r0 = 0; r0 < RBW; r0 += RBB) {
                v4i_t acc[RBB];
#pragma unroll
                for (int r = 0; r < RBB; ++r) acc[r] = (v4i_t){0, 0, 0, 0};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    v4i_t af = (v4i_t){0, 0, 0, 0};
                    if (row0) af = *reinterpret_cast<const v4i_t *>(lds_a + kt * 16 + 4 * t + kq);
#pragma unroll
                    for (int r = 0; r < RBB; ++r) {
                        const uint4 w4 = wt[r0 + r][i];
                        const uint32_t wd = t == 0 ? w4.x : (t == 1 ? w4.y : (t == 2 ? w4.z : w4.w));
                        v4i_t bf;
                        bf[0] = (int)(wd & 0x03030303u);
                        bf[1] = (int)((wd >> 2) & 0x03030303u);
                        bf[2] = (int)((wd >> 4) & 0x03030303u);
                        bf[3] = (int)((wd >> 6) & 0x03030303u);
                        acc[r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, bf, acc[r], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int r = 0; r < RBB; ++r)
                    if (lane < TILE_ROWS) atomicAdd(&tot[r0 + r][lane], acc[r][0]);  // int32: any order gives the same sum
            }
        }
    }
    lds_barrier();

    if (tid < TILE_ROWS * RBW) {
        const int r = tid >> 4, row = tid & 15;
        const int n = (rb0 + r) * TILE_ROWS + row;
        int asum = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) asum += red_i[w];
        if (group == 0 && tid == 0) {
            if (p.a_scale_out) p.a_scale_out[tok] = scale;
            if (p.a_sum_out) p.a_sum_out[tok] = asum;
        }
        if (n < P.n) {
            const int total = tot[r][row] - asum;
            if (P.acc) P.acc[tok * (size_t)P.n + n] = total;
            if (P.out) {
                float y = f32_mul((float)total, e_ws);
                y = f32_div(y, scale);
                if (P.bias) y = f32_add(y, e_bias);
                if (P.residual) y = f32_add(y, e_res);
                P.out[tok * (size_t)P.n + n] = y;
            }
        }
    }
}

typedef int v4i __attribute__((ext_vector_type(4)));

struct GemvMfmaParams {
    GemvProjDev proj[GEMV_MAX_PROJ];  // rb_end counts groups of RB row blocks
    int nproj;
    const int8_t *a;       // [m, k] int8
    const float *a_scale;  // [m]
    int m;                 // 1..16
    int k;
    int kt_count;
};

// MT: groups of 16 token rows (m <= 16 * MT); a decoded weight dword then feeds MT MFMAs.
// FAST: k is a multiple of 256 and the activations are 16-byte aligned.  Every load is then unconditional
// (indices past the end are clamped, the values discarded), so the compiler can count the loads in flight
// and the next batch of tiles really stays outstanding while the current one is multiplied.
// ONE: the wavefront's k-tiles (at most 8: k <= 8192) form a single batch, requested as a whole at the start: one
// memory latency instead of one per batch (RB = MT = 1 only, where the registers allow it).
template <int RB, int MT, bool FAST, bool ONE = false>
__global__ __launch_bounds__(256) void gemv_mfma_kernel(const int8_t *hot_a, int hot_k, int hot_m, int hot_kt_count, GemvMfmaParams p)
{
    // the leading scalar arguments repeat the fields a, k, m and kt_count of p, which the first address computations need;
    // they are preloaded into registers (see the Makefile) and used in place of the fields throughout
    __shared__ int red[4][RB][MT][64][4];  // partial accumulators of the four wavefronts
    __shared__ int red_sum[4][MT][16];     // per wavefront: sum_k a[t, k] over its k-tiles

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 15, lg = lane >> 4;

    // A operand of this lane in token group g: token row 16g + lr, the 16 columns 64t + 16lg of each k-tile
    // (rows past m read as zero)
    const bool a_vec = (hot_k % 16 == 0) && ((reinterpret_cast<uintptr_t>(hot_a) & 15) == 0);
    bool row_ok[MT];
    const int8_t *arow[MT];
#pragma unroll
    for (int g = 0; g < MT; ++g) {
        row_ok[g] = 16 * g + lr < hot_m;
        arow[g] = hot_a + (size_t)(row_ok[g] ? 16 * g + lr : 0) * hot_k + lg * 16;
    }
    auto load_a = [&](int g, int kt, int t) -> v4i {
        if constexpr (FAST) {
            const v4i v = *reinterpret_cast<const v4i *>(arow[g] + min(kt, hot_kt_count - 1) * TILE_K + t * 64);
            return row_ok[g] ? v : (v4i){0, 0, 0, 0};
        }
        v4i v = (v4i){0, 0, 0, 0};
        const int col = kt * TILE_K + t * 64 + lg * 16;
        if (row_ok[g] && col < hot_k) {
            const int8_t *src = arow[g] + kt * TILE_K + t * 64;
            if (a_vec) {
                v = *reinterpret_cast<const v4i *>(src);
            } else {
                int d[4] = {0, 0, 0, 0};
                for (int j = 0; j < 16; ++j)
                    if (col + j < hot_k) d[j >> 2] |= (int)((uint32_t)(uint8_t)src[j] << (8 * (j & 3)));
                v = (v4i){d[0], d[1], d[2], d[3]};
            }
        }
        return v;
    };
    static_assert(!ONE || MT == 1, "single batch: one token group");
    constexpr int PF = ONE ? (RB == 1 ? 8 : (RB == 2 ? 4 : 3))
                           : (RB * MT == 1 ? 4 : (RB * MT == 2 ? 3 : (MT <= 2 ? 2 : 1)));  // bounded by the register file
    // All loads of a batch of PF k-tiles are issued before the first MFMA of the batch, and the next
    // batch is requested while the current one is computed: the weight stream is what the kernel waits for.
    uint4 wcur[PF][RB], wnxt[ONE ? 1 : PF][RB];
    v4i acur[PF][MT][4], anxt[ONE ? 1 : PF][MT][4];
    // The first batch: the activations are addressed by the preloaded arguments alone, so with FAST they are requested
    // before anything reads the argument buffer (the weights' address comes from there).
    if constexpr (FAST) {
#pragma unroll
        for (int u = 0; u < PF; ++u)
#pragma unroll
            for (int g = 0; g < MT; ++g)
#pragma unroll
                for (int t = 0; t < 4; ++t) acur[u][g][t] = load_a(g, wave + 4 * u, t);
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing below moves above: the first wait for the argument buffer comes here

    int pj = 0;
#pragma unroll
    for (int j = 0; j < GEMV_MAX_PROJ - 1; ++j)
        if (j + 1 < p.nproj && (int)blockIdx.x >= p.proj[j].rb_end) pj = j + 1;
    const GemvProjDev &P = p.proj[pj];
    const int grp = (int)blockIdx.x - (pj ? p.proj[pj - 1].rb_end : 0);
    const int rb0 = grp * RB;
    const int rb_count = (P.n + TILE_ROWS - 1) / TILE_ROWS;
    const uint4 *wbase = reinterpret_cast<const uint4 *>(P.w) + lane;


    auto load_w = [&](int kt, uint4 (&w)[RB]) {
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const int rb = rb0 + r;
            if constexpr (FAST)  // results of row blocks past the end are never stored
                w[r] = load_weight_slot(wbase + ((size_t)min(rb, rb_count - 1) * hot_kt_count + min(kt, hot_kt_count - 1)) * 64);
            else
                w[r] = rb < rb_count ? load_weight_slot(wbase + ((size_t)rb * hot_kt_count + kt) * 64)
                                     : make_uint4(0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u);
        }
    };

    constexpr int NFRAG = RB * MT, FPW = (NFRAG + 3) / 4;  // fragments, fragments per wavefront
    v4i acc[RB][MT];
    int rowsum[MT];
#pragma unroll
    for (int g = 0; g < MT; ++g) {
        rowsum[g] = 0;
#pragma unroll
        for (int r = 0; r < RB; ++r) acc[r][g] = (v4i){0, 0, 0, 0};
    }

    auto load_batch = [&](int kt0, uint4 (&w)[PF][RB], v4i (&a)[PF][MT][4]) {
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            const int kt = kt0 + 4 * u;
            if (FAST || kt < hot_kt_count) {
                load_w(kt, w[u]);
#pragma unroll
                for (int g = 0; g < MT; ++g)
#pragma unroll
                    for (int t = 0; t < 4; ++t) a[u][g][t] = load_a(g, kt, t);
            }
        }
    };
    if constexpr (FAST) {  // the activations of the first batch are on their way already
#pragma unroll
        for (int u = 0; u < PF; ++u) load_w(wave + 4 * u, wcur[u]);
    } else {
        load_batch(wave, wcur, acur);
    }
    __builtin_amdgcn_sched_barrier(0);

    auto compute_batch = [&](int kt0) {
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            if (kt0 + 4 * u >= hot_kt_count) continue;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int g = 0; g < MT; ++g) {
                    const v4i af = acur[u][g][t];
                    rowsum[g] = __builtin_amdgcn_sdot4(af[0], 0x01010101, rowsum[g], false);
                    rowsum[g] = __builtin_amdgcn_sdot4(af[1], 0x01010101, rowsum[g], false);
                    rowsum[g] = __builtin_amdgcn_sdot4(af[2], 0x01010101, rowsum[g], false);
                    rowsum[g] = __builtin_amdgcn_sdot4(af[3], 0x01010101, rowsum[g], false);
                }
#pragma unroll
                for (int r = 0; r < RB; ++r) {
                    const uint4 w4 = wcur[u][r];
                    const uint32_t wd = t == 0 ? w4.x : (t == 1 ? w4.y : (t == 2 ? w4.z : w4.w));
                    v4i bf;
                    bf[0] = (int)(wd & 0x03030303u);
                    bf[1] = (int)((wd >> 2) & 0x03030303u);
                    bf[2] = (int)((wd >> 4) & 0x03030303u);
                    bf[3] = (int)((wd >> 6) & 0x03030303u);
#pragma unroll
                    for (int g = 0; g < MT; ++g)
                        acc[r][g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(acur[u][g][t], bf, acc[r][g], 0, 0, 0);
                }
            }
        }
    };
    // The RB * MT fragments (row block, token group) are finished by the wavefronts in turn: fragment
    // q = wave + 4 * f is (row block q / MT, token group q % MT); result register i of a lane belongs to token
    // 16g + 4*(lane/16) + i.  Scales, bias and residuals are requested now, behind the first batch of the main loads, so
    // that their latency is not paid at the end.  Absent operands read the weight tiles instead (always there; the
    // values are not used), which keeps this part free of branches, and the weight scale goes through a per-lane address:
    // a vector load, which nothing waits for before the epilogue.
    const float *absent = reinterpret_cast<const float *>(P.w);
    int lane_zero = 0;
    asm volatile("" : "+v"(lane_zero));
    const float ws = (P.out ? P.w_scale : absent)[lane_zero];
    float e_bias[FPW], e_scale[FPW][4], e_res[FPW][4];
#pragma unroll
    for (int f = 0; f < FPW; ++f) {
        const int q = min(wave + 4 * f, NFRAG - 1), fr = q / MT, fg = q % MT;
        const int e_n = min((rb0 + fr) * TILE_ROWS + lr, P.n - 1);
        e_bias[f] = *(P.bias ? P.bias + e_n : absent);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = min(16 * fg + lg * 4 + i, hot_m - 1);
            e_scale[f][i] = *(P.out ? p.a_scale + t : absent);
            e_res[f][i] = *(P.residual ? P.residual + ((size_t)t * P.n + e_n) : absent);
        }
    }

    if constexpr (ONE) {
        compute_batch(wave);
    } else
    for (int kt0 = wave; kt0 < hot_kt_count; kt0 += 4 * PF) {
        // two straight-line bodies, so that the wait before the MFMAs is for this batch only in both of them
        if constexpr (!ONE) {
            if (kt0 + 4 * PF < hot_kt_count) {  // uniform over the wavefront
                load_batch(kt0 + 4 * PF, wnxt, anxt);
                compute_batch(kt0);
#pragma unroll
                for (int u = 0; u < PF; ++u) {
#pragma unroll
                    for (int r = 0; r < RB; ++r) wcur[u][r] = wnxt[u][r];
#pragma unroll
                    for (int g = 0; g < MT; ++g)
#pragma unroll
                        for (int t = 0; t < 4; ++t) acur[u][g][t] = anxt[u][g][t];
                }
            } else {
                compute_batch(kt0);
            }
        }
    }

    // sum_k a[row, k] over this wavefront's tiles: lanes lr, lr+16, lr+32, lr+48 hold the four column groups
#pragma unroll
    for (int g = 0; g < MT; ++g) {
        rowsum[g] = sum_over_lane_groups(rowsum[g]);
        if (lane < 16) red_sum[wave][g][lane] = rowsum[g];
    }
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int g = 0; g < MT; ++g)
            *reinterpret_cast<v4i *>(&red[wave][r][g][lane][0]) = acc[r][g];
    lds_barrier();
#pragma unroll
    for (int f = 0; f < FPW; ++f) {
        if (wave + 4 * f >= NFRAG) break;  // uniform over the wavefront
        const int q = wave + 4 * f, fr = q / MT, fg = q % MT;
        const int n = (rb0 + fr) * TILE_ROWS + lr;  // result register i of lane l is C[4*(l/16) + i][l mod 16]
        const v4i s0 = *reinterpret_cast<const v4i *>(&red[0][fr][fg][lane][0]), s1 = *reinterpret_cast<const v4i *>(&red[1][fr][fg][lane][0]);
        const v4i s2 = *reinterpret_cast<const v4i *>(&red[2][fr][fg][lane][0]), s3 = *reinterpret_cast<const v4i *>(&red[3][fr][fg][lane][0]);
        const v4i sum = s0 + s1 + s2 + s3;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tl = lg * 4 + i, t = 16 * fg + tl;
            if (n < P.n && t < hot_m) {
                const int asum = red_sum[0][fg][tl] + red_sum[1][fg][tl] + red_sum[2][fg][tl] + red_sum[3][fg][tl];
                const int total = sum[i] - asum;
                const size_t o = (size_t)t * P.n + n;
                if (P.acc) P.acc[o] = total;
                if (P.out) {
                    float v = f32_div(f32_mul((float)total, ws), e_scale[f][i]);
                    if (P.bias) v = f32_add(v, e_bias[f]);
                    if (P.residual) v = f32_add(v, e_res[f][i]);
                    P.out[o] = v;
                }
            }
        }
    }
}

// gemv_mfma_kernel for up to 16 tokens with the activations staged through LDS.  There every wavefront gathers its A
// fragments straight from memory: 16 bytes per lane from 16 different rows, four loads per k-tile, and the address
// unit of the compute unit spends more time on those gathers than the weight stream needs.  Here the workgroup copies
// the m rows into LDS once with dense loads (thread t takes the 16-byte chunks t, t + 256, .. of every row) and the
// fragments are LDS reads.  Rows are k + 16 bytes apart in LDS.  KCLASS 0: k <= 3072 (one chunk column per thread,
// three k-tiles per wavefront), KCLASS 1: k <= 8192 and m <= 8 (two chunk columns, eight k-tiles).  k % 256 == 0, the
// activations 16-byte aligned, m * (k + 16) bytes of dynamic LDS.
template <int RB, int KCLASS>
__global__ __launch_bounds__(256) void gemv_mfma_lds_kernel(const int8_t *hot_a, int hot_k, int hot_m, int hot_kt_count, GemvMfmaParams p)
{
    constexpr int JN = KCLASS == 0 ? 1 : 2, NT = KCLASS == 0 ? 3 : 8;
    extern __shared__ uint4 lds_act[];        // [m][k / 16 + 1] chunks of 16 int8
    __shared__ int red[4][RB][64][4];         // partial accumulators of the four wavefronts
    __shared__ int red_sum[4][16];            // per wavefront: sum_k a[t, k] over its k-tiles

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    const int cpr = hot_k >> 4, stride = cpr + 1;  // chunks per row in memory and in LDS

    // the copy's loads first: they are addressed by the preloaded arguments alone (unconditional: rows past m repeat
    // the last row, chunks past the row its last chunk; those are not stored)
    v4i stage[16];
    const v4i *a_chunks = reinterpret_cast<const v4i *>(hot_a);
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        const int r = min(s / JN, hot_m - 1), cc = min(tid + 256 * (s % JN), cpr - 1);
        stage[s] = a_chunks[(size_t)r * cpr + cc];
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing below moves above: the first wait for the argument buffer comes here

    int pj = 0;
#pragma unroll
    for (int j = 0; j < GEMV_MAX_PROJ - 1; ++j)
        if (j + 1 < p.nproj && (int)blockIdx.x >= p.proj[j].rb_end) pj = j + 1;
    const GemvProjDev &P = p.proj[pj];
    const int rb0 = ((int)blockIdx.x - (pj ? p.proj[pj - 1].rb_end : 0)) * RB;
    const int rb_count = (P.n + TILE_ROWS - 1) / TILE_ROWS;
    const uint4 *wbase = reinterpret_cast<const uint4 *>(P.w) + lane;
    __builtin_amdgcn_sched_barrier(0);
    // The copy's stores, then everyone may read the rows.  The weight stream is requested only now: megabytes from all
    // workgroups at once, behind which the activations (and the argument buffers of workgroups that start a little
    // later) would queue in the memory system; this way they arrive about as early as they can, and the weights about
    // when they would have anyway.
#pragma unroll
    for (int s = 0; s < 16; ++s) {
        const int r = s / JN, cc = tid + 256 * (s % JN);
        if (r < hot_m && cc < cpr) reinterpret_cast<v4i *>(lds_act)[r * stride + cc] = stage[s];
    }
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // all k-tiles of this wavefront (kt = wave + 4u) in one batch; tiles and row blocks past the end repeat the last one
    uint4 w[NT][RB];
#pragma unroll
    for (int u = 0; u < NT; ++u)
#pragma unroll
        for (int r = 0; r < RB; ++r)
            w[u][r] = load_weight_slot(wbase + ((size_t)min(rb0 + r, rb_count - 1) * hot_kt_count + min(wave + 4 * u, hot_kt_count - 1)) * 64);

    // Row block q = wave + 4f of the workgroup is finished by this wavefront; scales, bias and residuals are requested now
    // (absent operands read the weight tiles instead, the values are not used; the weight scale goes through a per-lane
    // address: a vector load, which nothing waits for before the epilogue).
    constexpr int FPW = (RB + 3) / 4;
    const float *absent = reinterpret_cast<const float *>(P.w);
    int lane_zero = 0;
    asm volatile("" : "+v"(lane_zero));
    const float ws = (P.out ? P.w_scale : absent)[lane_zero];
    float e_bias[FPW], e_scale[FPW][4], e_res[FPW][4];
#pragma unroll
    for (int f = 0; f < FPW; ++f) {
        const int fr = min(wave + 4 * f, RB - 1);
        const int e_n = min((rb0 + fr) * TILE_ROWS + lr, P.n - 1);
        e_bias[f] = *(P.bias ? P.bias + e_n : absent);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = min(lg * 4 + i, hot_m - 1);
            e_scale[f][i] = *(P.out ? p.a_scale + t : absent);
            e_res[f][i] = *(P.residual ? P.residual + ((size_t)t * P.n + e_n) : absent);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    v4i acc[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[r] = (v4i){0, 0, 0, 0};
    int rowsum = 0;
    const bool row_ok = lr < hot_m;
    const uint4 *arow = lds_act + (row_ok ? lr : 0) * stride + lg;  // A operand: token row lr, columns 64t + 16lg .. +15 of a k-tile
#pragma unroll
    for (int u = 0; u < NT; ++u) {
        const int kt = wave + 4 * u;
        if (kt < hot_kt_count) {  // uniform over the wavefront
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                v4i af = (v4i){0, 0, 0, 0};
                if (row_ok) af = *reinterpret_cast<const v4i *>(arow + kt * 16 + t * 4);
                rowsum = __builtin_amdgcn_sdot4(af[0], 0x01010101, rowsum, false);
                rowsum = __builtin_amdgcn_sdot4(af[1], 0x01010101, rowsum, false);
                rowsum = __builtin_amdgcn_sdot4(af[2], 0x01010101, rowsum, false);
                rowsum = __builtin_amdgcn_sdot4(af[3], 0x01010101, rowsum, false);
#pragma unroll
                for (int r = 0; r < RB; ++r) {
                    const uint4 w4 = w[u][r];
                    const uint32_t wd = t == 0 ? w4.x : (t == 1 ? w4.y : (t == 2 ? w4.z : w4.w));
                    v4i bf;
                    bf[0] = (int)(wd & 0x03030303u);
                    bf[1] = (int)((wd >> 2) & 0x03030303u);
                    bf[2] = (int)((wd >> 4) & 0x03030303u);
                    bf[3] = (int)((wd >> 6) & 0x03030303u);
                    acc[r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, bf, acc[r], 0, 0, 0);
                }
            }
        }
    }

    // sum_k a[row, k] over this wavefront's tiles: lanes lr, lr+16, lr+32, lr+48 hold the four column groups
    rowsum = sum_over_lane_groups(rowsum);
    if (lane < 16) red_sum[wave][lane] = rowsum;
#pragma unroll
    for (int r = 0; r < RB; ++r) *reinterpret_cast<v4i *>(&red[wave][r][lane][0]) = acc[r];
    lds_barrier();
#pragma unroll
    for (int f = 0; f < FPW; ++f) {
        if (wave + 4 * f >= RB) break;  // uniform over the wavefront
        const int fr = wave + 4 * f;
        const int n = (rb0 + fr) * TILE_ROWS + lr;  // result register i of lane l is C[4*(l/16) + i][l mod 16]
        const v4i s0 = *reinterpret_cast<const v4i *>(&red[0][fr][lane][0]), s1 = *reinterpret_cast<const v4i *>(&red[1][fr][lane][0]);
        const v4i s2 = *reinterpret_cast<const v4i *>(&red[2][fr][lane][0]), s3 = *reinterpret_cast<const v4i *>(&red[3][fr][lane][0]);
        const v4i sum = s0 + s1 + s2 + s3;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = lg * 4 + i;
            if (n < P.n && t < hot_m) {
                const int asum = red_sum[0][t] + red_sum[1][t] + red_sum[2][t] + red_sum[3][t];
                const int total = sum[i] - asum;
                const size_t o = (size_t)t * P.n + n;
                if (P.acc) P.acc[o] = total;
                if (P.out) {
                    float v = f32_div(f32_mul((float)total, ws), e_scale[f][i]);
                    if (P.bias) v = f32_add(v, e_bias[f]);
                    if (P.residual) v = f32_add(v, e_res[f][i]);
                    P.out[o] = v;
                }
            }
        }
    }
}

// 17 and more tokens: gemv_mfma_lds_kernel's scheme with the tokens cut into groups of 16, one workgroup per
// (group of RB row blocks, token group).  gemv_mfma_kernel gives every workgroup ALL token rows (16 * MT of them) for
// its 16 * RB output rows, gathered per wavefront straight from memory: at 64 tokens that is 164 KB (k = 2560) to
// 442 KB (k = 6912) through the one L1 of a compute unit for 32 output rows, 70 MB of L2 traffic per launch for a
// 4.4 MB weight matrix, and the kernel takes 11 to 15 us.  Here a workgroup copies only its 16 token rows into LDS
// (dense 16-byte loads, rows k + 16 bytes apart) and the weight tiles are read once per token group: with the token
// groups of a row-block group placed on the same XCD, from HBM once and from that XCD's L2 afterwards.
// The copy is made by LDS-direct loads, all in flight at once, and the wavefront's k-tiles (kt = wave + 4u, at most NT of
// them) are requested as one batch right behind it, so the two latencies overlap.  k % 256 == 0, activations 16-byte
// aligned, m * k < 4 GiB, 16 * (k + 16) bytes of dynamic LDS rounded up to a whole KiB (the copy stores whole loads).
template <int RB, int NT>
__global__ __launch_bounds__(256) void gemv_mfma_tg_kernel(const int8_t *hot_a, int hot_k, int hot_m, int hot_kt_count, int hot_groups,
                                                           int hot_tgroups, GemvMfmaParams p)
{
    extern __shared__ uint4 lds_act[];        // [16][k / 16 + 1] chunks of 16 int8
    __shared__ int red[4][RB][64][4];         // partial accumulators of the four wavefronts
    __shared__ int red_sum[4][16];            // per wavefront: sum_k a[t, k] over its k-tiles

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 15, lg = lane >> 4;
    const int cpr = hot_k >> 4, stride = cpr + 1;  // chunks per row in memory and in LDS

    // Workgroups go to the eight XCDs in turn: the ids that share an XCD walk the (row-block group, token group) pairs
    // with the token group fastest, so the token groups of one row-block group meet in one L2.
    const int total = hot_groups * hot_tgroups;
    const int per_xcd = (total + 7) >> 3;
    const int idx = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (idx >= total) return;  // uniform over the workgroup
    const int grp_all = idx / hot_tgroups, tg = idx - grp_all * hot_tgroups;
    const int t0 = tg * 16, rows_here = min(16, hot_m - t0);

    // The copy, by LDS-direct loads (no registers, every load of the wavefront in flight at once): load q of the
    // workgroup fills the LDS chunks 64q .. 64q + 63, lane l the chunk L = 64q + l = (row L / stride, column chunk
    // L % stride); it fetches that chunk of its token row (rows past the end repeat the last one, the pad chunk of a
    // row repeats the chunk before it: neither is ever read).
    {
        const uint32_t lds_base = (uint32_t)(uintptr_t)lds_act;
        const int nl = 16 * stride;
        const uint32_t row_bytes = (uint32_t)hot_k;
        const uint32_t base_off = (uint32_t)t0 * row_bytes;  // the launcher keeps m * k below 4 GiB
        for (int q = wave; q * 64 < nl; q += 4) {
            const int L = min(q * 64 + lane, nl - 1);
            const int r = L / stride, cc = L - r * stride;
            dma16(hot_a, base_off + (uint32_t)min(r, rows_here - 1) * row_bytes + (uint32_t)min(cc, cpr - 1) * 16u,
                  lds_base + (uint32_t)q * 1024u);
        }
    }

    int pj = 0;
#pragma unroll
    for (int j = 0; j < GEMV_MAX_PROJ - 1; ++j)
        if (j + 1 < p.nproj && grp_all >= p.proj[j].rb_end) pj = j + 1;
    const GemvProjDev &P = p.proj[pj];
    const int rb0 = (grp_all - (pj ? p.proj[pj - 1].rb_end : 0)) * RB;
    const int rb_count = (P.n + TILE_ROWS - 1) / TILE_ROWS;
    const uint4 *wbase = reinterpret_cast<const uint4 *>(P.w) + lane;
    // all k-tiles of this wavefront in one batch, requested right behind the copy; tiles and row blocks past the end
    // repeat the last one.  The weights are read by the other token groups too, so these loads keep their cache lines
    // (no non-temporal hint).
    uint4 w[NT][RB];
#pragma unroll
    for (int u = 0; u < NT; ++u)
#pragma unroll
        for (int r = 0; r < RB; ++r)
            w[u][r] = wbase[((size_t)min(rb0 + r, rb_count - 1) * hot_kt_count + min(wave + 4 * u, hot_kt_count - 1)) * 64];
    __builtin_amdgcn_sched_barrier(0);
    wait_vm<NT * RB>();  // loads return in order: the copy has landed, the weight tiles may still be in flight
    lds_barrier();
    __builtin_amdgcn_sched_barrier(0);

    constexpr int FPW = (RB + 3) / 4;
    const float *absent = reinterpret_cast<const float *>(P.w);
    int lane_zero = 0;
    asm volatile("" : "+v"(lane_zero));
    const float ws = (P.out ? P.w_scale : absent)[lane_zero];
    float e_bias[FPW], e_scale[FPW][4], e_res[FPW][4];
#pragma unroll
    for (int f = 0; f < FPW; ++f) {
        const int fr = min(wave + 4 * f, RB - 1);
        const int e_n = min((rb0 + fr) * TILE_ROWS + lr, P.n - 1);
        e_bias[f] = *(P.bias ? P.bias + e_n : absent);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = t0 + min(lg * 4 + i, rows_here - 1);
            e_scale[f][i] = *(P.out ? p.a_scale + t : absent);
            e_res[f][i] = *(P.residual ? P.residual + ((size_t)t * P.n + e_n) : absent);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    v4i acc[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) acc[r] = (v4i){0, 0, 0, 0};
    int rowsum = 0;
    const bool row_ok = lr < rows_here;
    const uint4 *arow = lds_act + (row_ok ? lr : 0) * stride + lg;  // A operand: token row lr, columns 64t + 16lg .. +15 of a k-tile
#pragma unroll
    for (int u = 0; u < NT; ++u) {
        const int kt = wave + 4 * u;
        if (kt < hot_kt_count) {  // uniform over the wavefront
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                v4i af = (v4i){0, 0, 0, 0};
                if (row_ok) af = *reinterpret_cast<const v4i *>(arow + kt * 16 + t * 4);
                rowsum = __builtin_amdgcn_sdot4(af[0], 0x01010101, rowsum, false);
                rowsum = __builtin_amdgcn_sdot4(af[1], 0x01010101, rowsum, false);
                rowsum = __builtin_amdgcn_sdot4(af[2], 0x01010101, rowsum, false);
                rowsum = __builtin_amdgcn_sdot4(af[3], 0x01010101, rowsum, false);
#pragma unroll
                for (int r = 0; r < RB; ++r) {
                    const uint4 w4 = w[u][r];
                    const uint32_t wd = t == 0 ? w4.x : (t == 1 ? w4.y : (t == 2 ? w4.z : w4.w));
                    v4i bf;
                    bf[0] = (int)(wd & 0x03030303u);
                    bf[1] = (int)((wd >> 2) & 0x03030303u);
                    bf[2] = (int)((wd >> 4) & 0x03030303u);
                    bf[3] = (int)((wd >> 6) & 0x03030303u);
                    acc[r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, bf, acc[r], 0, 0, 0);
                }
            }
        }
    }

    rowsum = sum_over_lane_groups(rowsum);
    if (lane < 16) red_sum[wave][lane] = rowsum;
#pragma unroll
    for (int r = 0; r < RB; ++r) *reinterpret_cast<v4i *>(&red[wave][r][lane][0]) = acc[r];
    lds_barrier();
#pragma unroll
    for (int f = 0; f < FPW; ++f) {
        if (wave + 4 * f >= RB) break;  // uniform over the wavefront
        const int fr = wave + 4 * f;
        const int n = (rb0 + fr) * TILE_ROWS + lr;  // result register i of lane l is C[4*(l/16) + i][l mod 16]
        const v4i s0 = *reinterpret_cast<const v4i *>(&red[0][fr][lane][0]), s1 = *reinterpret_cast<const v4i *>(&red[1][fr][lane][0]);
        const v4i s2 = *reinterpret_cast<const v4i *>(&red[2][fr][lane][0]), s3 = *reinterpret_cast<const v4i *>(&red[3][fr][lane][0]);
        const v4i sum = s0 + s1 + s2 + s3;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int tl = lg * 4 + i;
            if (n < P.n && tl < rows_here) {
                const int asum = red_sum[0][tl] + red_sum[1][tl] + red_sum[2][tl] + red_sum[3][tl];
                const int total_acc = sum[i] - asum;
                const size_t o = (size_t)(t0 + tl) * P.n + n;
                if (P.acc) P.acc[o] = total_acc;
                if (P.out) {
                    float v = f32_div(f32_mul((float)total_acc, ws), e_scale[f][i]);
                    if (P.bias) v = f32_add(v, e_bias[f]);
                    if (P.residual) v = f32_add(v, e_res[f][i]);
                    P.out[o] = v;
                }
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
    acc = wave_sum_i32(acc);
    if (lane == 0) out[row] = acc;
}

template <int MB, int MODE>
int launch_mb_mode(const GemvParams &p, hipStream_t stream)
{
    size_t lds = (size_t)MB * p.kt_count * 16 * sizeof(uint4);
    dim3 grid((unsigned)p.proj[p.nproj - 1].rb_end);
    hipLaunchKernelGGL((gemv_tiled_kernel<MB, MODE>), grid, dim3(256), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemv_tiled_kernel");
    return BITNET_HIP_OK;
}

template <int MODE>
int launch_mode(const GemvParams &p, hipStream_t stream)
{
    return launch_mb_mode<1, MODE>(p, stream);  // one token row per launch; 2..16 rows take gemv_mfma_kernel
}

template <int MODE, int RBW>
int launch_fused_mode(const GemvParams &p, hipStream_t stream)
{
    const bool norm = p.src.gamma != nullptr, small = p.k <= 3 * 1024;
    // the int8 row, or (first) the f32 squares of the row for the literal summation order
    const size_t lds_q = (size_t)p.kt_count * 16 * sizeof(uint4), lds_sq = squares_lds_bytes(p.k);
    const size_t lds = (norm && p.src.sum_order == BITNET_HIP_SUM_SEQUENTIAL && lds_sq > lds_q) ? lds_sq : lds_q;
    const dim3 grid((unsigned)p.proj[p.nproj - 1].rb_end);
    if (norm && small) hipLaunchKernelGGL((gemv_fused_kernel<MODE, true, 3, RBW>), grid, dim3(256), lds, stream, p);
    else if (norm) hipLaunchKernelGGL((gemv_fused_kernel<MODE, true, FUSED_NCH, RBW>), grid, dim3(256), lds, stream, p);
    else if (small) hipLaunchKernelGGL((gemv_fused_kernel<MODE, false, 3, RBW>), grid, dim3(256), lds, stream, p);
    else hipLaunchKernelGGL((gemv_fused_kernel<MODE, false, FUSED_NCH, RBW>), grid, dim3(256), lds, stream, p);
    BITNET_HIP_CHECK_LAUNCH("gemv_fused_kernel");
    return BITNET_HIP_OK;
}

template <int MODE, int RBW>
int launch_fused16_mode(const GemvParams &p, hipStream_t stream)
{
    const bool norm = p.src.gamma != nullptr;
    const size_t lds = (size_t)p.kt_count * 16 * sizeof(uint4);
    const dim3 grid(8u * (unsigned)p.m, ((unsigned)p.proj[p.nproj - 1].rb_end + 7u) / 8u);
    // One wavefront per k-tile (at least the four of the summation order) for rows of up to 16 k-tiles, one chunk per
    // thread; 16 wavefronts and two chunks per thread above.  Fewer wavefronts with more chunks each are slower (the
    // element-wise steps lose their parallelism: 2560 columns on 5 wavefronts 581 us per 30-layer step against 507 on 10).
    const int nchb = p.kt_count <= 16 ? 1 : 2;
    const int nw = p.kt_count <= 16 ? row_workgroup_waves(p.src.k) : 16;
    if (p.src.gqa_group < 0 || p.src.gqa_group > 0xffff) return fail(BITNET_HIP_INVALID_CONFIG, "GQA group %d out of range", p.src.gqa_group);
    const dim3 block(64u * (unsigned)nw);
#define BITNET_HOT_ARGS p.src.x, p.src.x2, p.src.gamma, p.src.k, p.src.head_dim, p.src.gqa_group | (nw << 16), (int)p.src.ldx
#define BITNET_F16_LAUNCH(NCHB) \
    do { \
        if (norm) hipLaunchKernelGGL((gemv_fused16_kernel<MODE, true, NCHB, RBW>), grid, block, lds, stream, BITNET_HOT_ARGS, p); \
        else hipLaunchKernelGGL((gemv_fused16_kernel<MODE, false, NCHB, RBW>), grid, block, lds, stream, BITNET_HOT_ARGS, p); \
    } while (0)
    if (nchb == 1) {
        BITNET_F16_LAUNCH(1);
    } else if constexpr (RBW <= 8) {  // two k-tiles per wavefront: the tiles of 16 row blocks would not fit the registers
        BITNET_F16_LAUNCH(2);
    } else {
        return fail(BITNET_HIP_UNSUPPORTED, "gemv_fused16: %d row blocks per workgroup with %d k-tiles", RBW, p.kt_count);
    }
#undef BITNET_F16_LAUNCH
#undef BITNET_HOT_ARGS
    BITNET_HIP_CHECK_LAUNCH("gemv_fused16_kernel");
    return BITNET_HIP_OK;
}

// rbw: row blocks per workgroup (rb_end then counts groups of rbw row blocks, per projection)
int fill_projs(GemvParams &p, const GemvProj *projs, int nproj, size_t t0, size_t k, int rbw = 1)
{
    int rb_end = 0;
    for (int j = 0; j < nproj; ++j) {
        const GemvProj &s = projs[j];
        GemvProjDev &d = p.proj[j];
        d.w = s.tiled; d.w_scale = s.w_scale; d.bias = s.bias; d.n = (int)s.n;
        d.residual = s.residual ? s.residual + t0 * s.n : nullptr;
        d.out = s.out ? s.out + t0 * s.n : nullptr;
        d.acc = s.acc ? s.acc + t0 * s.n : nullptr;
        rb_end += (int)((row_blocks(s.n) + rbw - 1) / rbw);
        d.rb_end = rb_end;
    }
    for (int j = nproj; j < GEMV_MAX_PROJ; ++j) p.proj[j] = p.proj[nproj - 1];
    p.nproj = nproj;
    p.k = (int)k;
    p.kt_count = (int)k_tiles(k);
    return rb_end;
}

template <int RB, int MT>
int launch_mfma_rb(const GemvProj *projs, int nproj, const int8_t *a, const float *a_scale, size_t m, size_t k,
                   hipStream_t stream)
{
    GemvMfmaParams p = {};
    int end = 0;
    for (int j = 0; j < nproj; ++j) {
        const GemvProj &s = projs[j];
        GemvProjDev &d = p.proj[j];
        d.w = s.tiled; d.w_scale = s.w_scale; d.bias = s.bias; d.residual = s.residual; d.out = s.out; d.acc = s.acc;
        d.n = (int)s.n;
        end += (int)((row_blocks(s.n) + RB - 1) / RB);
        d.rb_end = end;
    }
    for (int j = nproj; j < GEMV_MAX_PROJ; ++j) p.proj[j] = p.proj[nproj - 1];
    p.nproj = nproj; p.a = a; p.a_scale = a_scale; p.m = (int)m; p.k = (int)k; p.kt_count = (int)k_tiles(k);
    if (end == 0) return BITNET_HIP_OK;
    const bool fast = k % TILE_K == 0 && (reinterpret_cast<uintptr_t>(a) & 15) == 0;
    if constexpr (MT == 1) {
        // 5 to 16 tokens whose rows fit LDS: the variant that stages the activations there (with fewer rows the gathers
        // of the other variant are cheap enough, and it is measurably ahead)
        const size_t lds = m * (k + 16);
        if (fast && m >= 5 && lds + 4096 * RB + 512 <= 64 * 1024 && (k <= 3072 || (k <= 8192 && m <= 8))) {  // + the kernel's static LDS
            if (k <= 3072)
                hipLaunchKernelGGL((gemv_mfma_lds_kernel<RB, 0>), dim3((unsigned)end), dim3(256), lds, stream, p.a, p.k, p.m, p.kt_count, p);
            else
                hipLaunchKernelGGL((gemv_mfma_lds_kernel<RB, 1>), dim3((unsigned)end), dim3(256), lds, stream, p.a, p.k, p.m, p.kt_count, p);
            BITNET_HIP_CHECK_LAUNCH("gemv_mfma_lds_kernel");
            return BITNET_HIP_OK;
        }
        // more than one double-buffered batch per wavefront, but few enough k-tiles for one batch without the second buffer
        constexpr int PF2 = RB == 1 ? 4 : (RB == 2 ? 3 : 2), PF1 = RB == 1 ? 8 : (RB == 2 ? 4 : 3);
        if (fast && p.kt_count > 4 * PF2 && p.kt_count <= 4 * PF1) {
            hipLaunchKernelGGL((gemv_mfma_kernel<RB, 1, true, true>), dim3((unsigned)end), dim3(256), 0, stream, p.a, p.k, p.m, p.kt_count, p);
            BITNET_HIP_CHECK_LAUNCH("gemv_mfma_kernel");
            return BITNET_HIP_OK;
        }
    }
    if (fast)
        hipLaunchKernelGGL((gemv_mfma_kernel<RB, MT, true>), dim3((unsigned)end), dim3(256), 0, stream, p.a, p.k, p.m, p.kt_count, p);
    else
        hipLaunchKernelGGL((gemv_mfma_kernel<RB, MT, false>), dim3((unsigned)end), dim3(256), 0, stream, p.a, p.k, p.m, p.kt_count, p);
    BITNET_HIP_CHECK_LAUNCH("gemv_mfma_kernel");
    return BITNET_HIP_OK;
}

// Dynamic LDS of gemv_mfma_tg_kernel: 16 token rows of k + 16 bytes, rounded up to the 1 KiB loads that fill it.
constexpr size_t tg_lds_bytes(size_t k) { return (16 * (k + 16) + 1023) / 1024 * 1024; }

// 17 and more token rows, k a multiple of 256 up to 8192, aligned activations: token groups of 16 (gemv_mfma_tg_kernel)
template <int RB>
int launch_mfma_tg(const GemvProj *projs, int nproj, const int8_t *a, const float *a_scale, size_t m, size_t k, hipStream_t stream)
{
    GemvMfmaParams p = {};
    int end = 0;
    for (int j = 0; j < nproj; ++j) {
        const GemvProj &s = projs[j];
        GemvProjDev &d = p.proj[j];
        d.w = s.tiled; d.w_scale = s.w_scale; d.bias = s.bias; d.residual = s.residual; d.out = s.out; d.acc = s.acc;
        d.n = (int)s.n;
        end += (int)((row_blocks(s.n) + RB - 1) / RB);
        d.rb_end = end;
    }
    for (int j = nproj; j < GEMV_MAX_PROJ; ++j) p.proj[j] = p.proj[nproj - 1];
    p.nproj = nproj; p.a = a; p.a_scale = a_scale; p.m = (int)m; p.k = (int)k; p.kt_count = (int)k_tiles(k);
    if (end == 0) return BITNET_HIP_OK;
    const int tgroups = (int)((m + 15) / 16), total = end * tgroups;
    const unsigned grid = (unsigned)((total + 7) / 8 * 8);
    // The copy fills LDS in whole loads of 1 KiB (64 lanes x 16 bytes); the last one runs past the 16 * (k + 16) bytes
    // of token rows, so the allocation is rounded up to whole loads.
    const size_t lds = tg_lds_bytes(k);
    if ((16 * (k / 16 + 1) + 63) / 64 * 1024 > lds)
        return fail(BITNET_HIP_KERNEL_ERROR, "gemv_mfma_tg: the activation copy would overrun its LDS allocation");
    if (p.kt_count <= 12) {
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_mfma_tg_kernel<RB, 3>),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)tg_lds_bytes(3072));
        BITNET_HIP_TRY(attr);
        hipLaunchKernelGGL((gemv_mfma_tg_kernel<RB, 3>), dim3(grid), dim3(256), lds, stream, p.a, p.k, p.m, p.kt_count, end, tgroups, p);
    } else {
        static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_mfma_tg_kernel<RB, 8>),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)tg_lds_bytes(8192));
        BITNET_HIP_TRY(attr);
        hipLaunchKernelGGL((gemv_mfma_tg_kernel<RB, 8>), dim3(grid), dim3(256), lds, stream, p.a, p.k, p.m, p.kt_count, end, tgroups, p);
    }
    BITNET_HIP_CHECK_LAUNCH("gemv_mfma_tg_kernel");
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

int launch_gemv_tiled(const GemvProj *projs, int nproj, const int8_t *a, const float *a_scale, size_t m, size_t k,
                      hipStream_t stream)
{
    if (m == 0 || nproj <= 0) return BITNET_HIP_OK;
    if (m >= 2) {
        // Several tokens: the MFMA variant, up to 64 token rows per launch (more: in groups of 64).  Workgroups
        // take more row blocks when there are plenty of them, so that fewer workgroups re-read the activations.
        size_t blocks = 0;
        for (int j = 0; j < nproj; ++j) blocks += row_blocks(projs[j].n);
        if (m > 16 && k % TILE_K == 0 && k <= 8192 && (reinterpret_cast<uintptr_t>(a) & 15) == 0 && m * k < ((size_t)1 << 32)) {
            // token groups of 16 with their rows in LDS.  Row blocks per workgroup: the activation copy is what a workgroup
            // spends its time on, so a workgroup takes several row blocks once there are enough workgroups for every
            // compute unit (LDS holds three workgroups up to k = 3072, one above).
            const size_t tgroups = (m + 15) / 16, slots = k <= 3072 ? 768 : 256;
            if (blocks * tgroups > 2 * slots) return launch_mfma_tg<4>(projs, nproj, a, a_scale, m, k, stream);
            if (blocks * tgroups > slots) return launch_mfma_tg<2>(projs, nproj, a, a_scale, m, k, stream);
            return launch_mfma_tg<1>(projs, nproj, a, a_scale, m, k, stream);
        }
        for (size_t t0 = 0; t0 < m; t0 += (size_t)GEMV_MFMA_MAX_M) {
            GemvProj sub[GEMV_MAX_PROJ];
            const size_t rows = m - t0 < (size_t)GEMV_MFMA_MAX_M ? m - t0 : (size_t)GEMV_MFMA_MAX_M;
            for (int j = 0; j < nproj; ++j) {
                sub[j] = projs[j];
                if (sub[j].residual) sub[j].residual += t0 * sub[j].n;
                if (sub[j].out) sub[j].out += t0 * sub[j].n;
                if (sub[j].acc) sub[j].acc += t0 * sub[j].n;
            }
            const int8_t *a0 = a + t0 * k;
            const float *s0 = a_scale ? a_scale + t0 : nullptr;
            int rc;
            if (rows > 32) rc = blocks >= 400 ? launch_mfma_rb<2, 4>(sub, nproj, a0, s0, rows, k, stream)
                                              : launch_mfma_rb<1, 4>(sub, nproj, a0, s0, rows, k, stream);
            else if (rows > 16) rc = blocks >= 400 ? launch_mfma_rb<2, 2>(sub, nproj, a0, s0, rows, k, stream)
                                                   : launch_mfma_rb<1, 2>(sub, nproj, a0, s0, rows, k, stream);
            else if (blocks >= 800) rc = launch_mfma_rb<4, 1>(sub, nproj, a0, s0, rows, k, stream);
            else if (blocks >= 400) rc = launch_mfma_rb<2, 1>(sub, nproj, a0, s0, rows, k, stream);
            else rc = launch_mfma_rb<1, 1>(sub, nproj, a0, s0, rows, k, stream);
            if (rc != BITNET_HIP_OK) return rc;
        }
        return BITNET_HIP_OK;
    }
    if (k_tiles(k) * 16 * sizeof(uint4) > 60 * 1024)
        return fail(BITNET_HIP_UNSUPPORTED, "decode GEMV: k=%zu does not fit the LDS activation buffer", k);
    GemvParams p = {};
    if (fill_projs(p, projs, nproj, 0, k) == 0) return BITNET_HIP_OK;
    p.m = 1;
    p.a = a;
    p.a_scale = a_scale;
    return launch_mode<MODE_PREQUANT>(p, stream);
}

// Row blocks per workgroup of gemv_fused16_kernel.  Every workgroup quantises its token's input row for itself: that
// arithmetic is repeated by every workgroup of the launch, and two workgroups on one compute unit take turns on its
// SIMDs, so the launch is sized to about one workgroup per compute unit where the registers allow (a wavefront holds
// the tiles of all its row blocks: 16 of them for rows of up to 16 k-tiles, 8 above).
int fused16_row_blocks_per_workgroup(size_t m, size_t k, size_t blocks)
{
    if (m == 1) {
        // one token, gate alone, 432 row blocks: 4.50 us with one row block per workgroup, 3.82 us with two
        if (blocks > 512 && k <= 4096) return 4;
        return (blocks > 256 && k <= 4096) ? 2 : 1;
    }
    // Several tokens, each with its own workgroups: the fewest row blocks per workgroup that keep the launch within one
    // workgroup per compute unit, at most 8 (16 lose: the dot products of 16 row blocks are a wavefront's serial work).
    // 30-block step at 2 / 3 / 4 / 6 / 8 tokens: 578 / 662 / 713 / 778 / 901 us; with a limit of 512 workgroups and at
    // most 4 row blocks each 646 / 733 / 779 / 1023 / 1150 us.
    int rbw = 1;
    while (rbw < 8 && (blocks + rbw - 1) / rbw * m > 256) rbw *= 2;
    return rbw;
}

bool gemv_fused_supported(const float *x, const float *x2, size_t ldx, size_t m, size_t k, int input_mode,
                          size_t head_dim, const float *gamma, int sum_order, size_t blocks)
{
    auto al16 = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
    // Two to GEMV_FUSED_MAX_ROWS tokens: the 16-wavefront kernel with a set of workgroups per token (half the launches;
    // the weight tiles are fetched once per token, from the caches after the first), where that kernel applies and the
    // workgroups of all tokens stay within GEMV_FUSED_MAX_WGS.  Otherwise: stand-alone quantiser (rows in parallel) + MFMA GEMV.
    if (m == 0 || m > (size_t)GEMV_FUSED_MAX_ROWS) return false;
    if (m > 1) {
        if (!((gamma == nullptr || sum_order == BITNET_HIP_SUM_BLOCK256) && k <= 8192 && ldx < ((size_t)1 << 31))) return false;
        const size_t rbw = (size_t)fused16_row_blocks_per_workgroup(m, k, blocks);
        if ((blocks + rbw - 1) / rbw * m > (size_t)GEMV_FUSED_MAX_WGS) return false;
    }
    if (k % 4 != 0 || ldx % 4 != 0 || k > (size_t)FUSED_NCH * 1024) return false;
    if (!al16(x) || (x2 && !al16(x2)) || (gamma && !al16(gamma))) return false;
    if (input_mode == BITNET_HIP_INPUT_GQA_BROADCAST && head_dim % 4 != 0) return false;
    return k_tiles(k) * 16 * sizeof(uint4) <= 60 * 1024;
}

int launch_gemv_fused(const GemvProj *projs, int nproj, const float *x, const float *x2, size_t ldx, size_t m,
                      size_t k, int input_mode, size_t gqa_group, size_t head_dim, const float *gamma, float eps,
                      int sum_order, int8_t *q_out, float *a_scale_out, int32_t *a_sum_out, hipStream_t stream)
{
    if (m == 0 || nproj <= 0) return BITNET_HIP_OK;
    // Every workgroup quantises the whole input row for itself, so launches with many row blocks give each
    // workgroup two (short rows only: the tiles of both must fit its registers).
    size_t blocks = 0;
    for (int j = 0; j < nproj; ++j) blocks += row_blocks(projs[j].n);
    // 16 wavefronts per workgroup (the declared summation order only; k <= 8192: two chunks per thread, 32 k-tiles)
    if ((gamma == nullptr || sum_order == BITNET_HIP_SUM_BLOCK256) && k <= 8192) {
        // row blocks per workgroup: one round of workgroups on the 256 compute units where the row is short enough for
        // a wavefront to hold the tiles of several row blocks (one token, gate alone, 432 row blocks: 4.50 us with one
        // row block per workgroup, 3.82 us with two)
        const int rbw16 = fused16_row_blocks_per_workgroup(m, k, blocks);
        GemvParams p = {};
        if (fill_projs(p, projs, nproj, 0, k, rbw16) == 0) return BITNET_HIP_OK;
        p.m = (int)m;
        p.src.x = x; p.src.x2 = x2; p.src.gamma = gamma; p.src.ldx = ldx; p.src.k = (int)k;
        p.src.head_dim = (int)(head_dim ? head_dim : 1); p.src.gqa_group = (int)(gqa_group ? gqa_group : 1);
        p.src.sum_order = sum_order; p.src.eps = eps;
        p.q_out = q_out; p.a_scale_out = a_scale_out; p.a_sum_out = a_sum_out;
#define BITNET_F16_MODES(RBW) \
    switch (input_mode) { \
        case BITNET_HIP_INPUT_PLAIN: return launch_fused16_mode<BITNET_HIP_INPUT_PLAIN, RBW>(p, stream); \
        case BITNET_HIP_INPUT_RELU2_MUL: return launch_fused16_mode<BITNET_HIP_INPUT_RELU2_MUL, RBW>(p, stream); \
        default: return launch_fused16_mode<BITNET_HIP_INPUT_GQA_BROADCAST, RBW>(p, stream); \
    }
        switch (rbw16) {
            case 16: BITNET_F16_MODES(16)
            case 8: BITNET_F16_MODES(8)
            case 4: BITNET_F16_MODES(4)
            case 2: BITNET_F16_MODES(2)
            default: BITNET_F16_MODES(1)
        }
#undef BITNET_F16_MODES
    }
    const int rbw = (blocks > 512 && k <= 3 * 1024) ? 2 : 1;
    GemvParams p = {};
    if (fill_projs(p, projs, nproj, 0, k, rbw) == 0) return BITNET_HIP_OK;
    p.m = (int)m;
    p.src.x = x; p.src.x2 = x2; p.src.gamma = gamma; p.src.ldx = ldx; p.src.k = (int)k;
    p.src.head_dim = (int)(head_dim ? head_dim : 1); p.src.gqa_group = (int)(gqa_group ? gqa_group : 1);
    p.src.sum_order = sum_order; p.src.eps = eps;
    p.q_out = q_out; p.a_scale_out = a_scale_out; p.a_sum_out = a_sum_out;
    if (rbw == 2) {
        switch (input_mode) {
            case BITNET_HIP_INPUT_PLAIN: return launch_fused_mode<BITNET_HIP_INPUT_PLAIN, 2>(p, stream);
            case BITNET_HIP_INPUT_RELU2_MUL: return launch_fused_mode<BITNET_HIP_INPUT_RELU2_MUL, 2>(p, stream);
            default: return launch_fused_mode<BITNET_HIP_INPUT_GQA_BROADCAST, 2>(p, stream);
        }
    }
    switch (input_mode) {
        case BITNET_HIP_INPUT_PLAIN: return launch_fused_mode<BITNET_HIP_INPUT_PLAIN, 1>(p, stream);
        case BITNET_HIP_INPUT_RELU2_MUL: return launch_fused_mode<BITNET_HIP_INPUT_RELU2_MUL, 1>(p, stream);
        default: return launch_fused_mode<BITNET_HIP_INPUT_GQA_BROADCAST, 1>(p, stream);
    }
}

}  // namespace bitnet
