// Stand-alone fused RMSNorm + per-token absmax int8 activation quantiser for gfx950 (the arithmetic and the
// declared summation order are in rowquant.hpp; the decode GEMV runs the same code inside its prologue).
//
// Three launch shapes, same bits:
//   act_quant_block_kernel    one 256-thread workgroup per token row, the row held in registers between the three
//                             passes (sum of squares, absmax, quantise): 4*K bytes read once, K + 8 bytes written.
//                             The usual shape (k <= 7168 with aligned rows), for one row or thousands.
//   act_quant_block16_kernel  one 1024-thread workgroup per token row: up to 16 rows (a decode batch), where the
//                             launch is as long as one row takes.
//   act_quant_wave_kernel     one wavefront per token row: many rows of any length or alignment.
#include "kernels.hpp"
#include "rowquant.hpp"

namespace bitnet {

namespace {

struct ActQuantParams {
    RowSource src;
    int8_t *q;
    float *a_scale;
    int32_t *a_sum;
    float *y;
    size_t m;
    int seq_in_lds;  // the launch carries LDS for the row's squares (literal summation order: sum_sequential_lds)
    unsigned *zero;  // optional: zero[0 .. zero_n) is cleared by the first workgroup (counters of the launch that follows)
    int zero_n;
};

// The clearing job: the threads of workgroup 0 (any block shape) write the zeros with vector stores.
__device__ __forceinline__ void clear_counters(const ActQuantParams &p)
{
    if (blockIdx.x == 0 && p.zero) {
        const int flat = threadIdx.y * blockDim.x + threadIdx.x, count = blockDim.x * blockDim.y;
        for (int i = flat; i < p.zero_n; i += count) p.zero[i] = 0u;
    }
}

// NCH > 0: a lane keeps its NCH chunks in registers (K <= 256*NCH).  NCH == 0: any K, the row is
// re-read (from cache) in each pass.
template <int MODE, int NCH, bool VEC>
__global__ __launch_bounds__(256) void act_quant_wave_kernel(ActQuantParams p)
{
    const RowSource &src = p.src;
    const int lane = threadIdx.x;
    clear_counters(p);
    const size_t row = (size_t)blockIdx.x * blockDim.y + threadIdx.y;
    if (row >= p.m) return;  // uniform per wavefront: a wavefront is one row
    const int k = src.k;
    const int chunks = (k + 3) >> 2;
    const int nloop = NCH > 0 ? NCH : (chunks + 63) >> 6;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);

    float4 v[NCH > 0 ? NCH : 1];
    if constexpr (NCH > 0) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            int c = lane + 64 * i;
            v[i] = c < chunks ? load_chunk<MODE, VEC>(src, row, c) : zero4;
        }
    }
    auto chunk_at = [&](int i, int c) -> float4 {
        if constexpr (NCH > 0) return v[i];
        else return c < chunks ? load_chunk<MODE, VEC>(src, row, c) : zero4;
    };

    RowDivisor rdiv = {1.0f, 1.0f, false};
    const bool norm = src.gamma != nullptr;
    if (norm) {
        float ss;
        if (src.sum_order == BITNET_HIP_SUM_SEQUENTIAL) {
            ss = sum_squares_sequential<MODE>(src, row);
        } else {
            // chunk c = lane + 64*i is virtual lane c mod 256 = lane + 64*(i mod 4): four partials per lane
            float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (NCH > 0) {
#pragma unroll
                for (int i = 0; i < NCH; ++i) part[i & 3] = sum_squares4(part[i & 3], v[i]);
            } else {
                for (int i = 0; i < nloop; i += 4)
#pragma unroll
                    for (int g = 0; g < 4; ++g) part[g] = sum_squares4(part[g], chunk_at(i + g, lane + 64 * (i + g)));
            }
            ss = f32_add(f32_add(f32_add(wave_sum_f32(part[0]), wave_sum_f32(part[1])), wave_sum_f32(part[2])),
                         wave_sum_f32(part[3]));
        }
        rdiv = make_row_divisor(rms_from_ss(ss, k, src.eps));
    }

    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < nloop; ++i) {
        int c = lane + 64 * i;
        float4 e = chunk_at(i, c);
        if (norm && c < chunks) e = normalize4(e, rdiv, load_gamma_chunk(src, c, VEC));
        if constexpr (NCH > 0) v[i] = e;
        amax = absmax4(amax, e);
    }
    amax = wave_max_f32(amax);
    const float scale = scale_from_absmax(amax);

    int isum = 0;
#pragma unroll
    for (int i = 0; i < nloop; ++i) {
        int c = lane + 64 * i;
        if (c >= chunks) continue;
        float4 e;
        if constexpr (NCH > 0) {
            e = v[i];
        } else {
            e = load_chunk<MODE, VEC>(src, row, c);
            if (norm) e = normalize4(e, rdiv, load_gamma_chunk(src, c, VEC));
        }
        size_t base = row * (size_t)k + 4 * (size_t)c;
        if constexpr (VEC) {
            *reinterpret_cast<uint32_t *>(p.q + base) = quant4_packed(e, scale, &isum);
            if (p.y) *reinterpret_cast<float4 *>(p.y + base) = e;
        } else {
            float es[4] = {e.x, e.y, e.z, e.w};
            for (int j = 0; j < 4; ++j) {
                if (4 * c + j < k) {
                    int qv = quant1(es[j], scale);
                    p.q[base + j] = (int8_t)qv;
                    if (p.y) p.y[base + j] = es[j];
                    isum += qv;
                }
            }
        }
    }
    isum = wave_sum_i32(isum);
    if (lane == 0) {
        p.a_scale[row] = scale;
        if (p.a_sum) p.a_sum[row] = isum;
    }
}

// One workgroup per row.  NCH chunks per thread in registers (K <= 1024*NCH), NCH == 0: re-read.
template <int MODE, int NCH, bool VEC>
__global__ __launch_bounds__(256) void act_quant_block_kernel(ActQuantParams p)
{
    __shared__ float red_f[2][4];
    __shared__ int red_i[4];
    const RowSource &src = p.src;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    clear_counters(p);
    const size_t row = blockIdx.x;
    const int k = src.k;
    const int chunks = (k + 3) >> 2;
    const int nloop = NCH > 0 ? NCH : (chunks + 255) >> 8;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);

    float4 v[NCH > 0 ? NCH : 1];
    if constexpr (NCH > 0) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            int c = tid + 256 * i;
            v[i] = c < chunks ? load_chunk<MODE, VEC>(src, row, c) : zero4;
        }
    }
    auto chunk_at = [&](int i, int c) -> float4 {
        if constexpr (NCH > 0) return v[i];
        else return c < chunks ? load_chunk<MODE, VEC>(src, row, c) : zero4;
    };

    RowDivisor rdiv = {1.0f, 1.0f, false};
    const bool norm = src.gamma != nullptr;
    if (norm) {
        float ss;
        if (src.sum_order == BITNET_HIP_SUM_SEQUENTIAL) {
            if (p.seq_in_lds) {
                extern __shared__ float sq_lds[];  // squares_lds_bytes(k)
#pragma unroll
                for (int i = 0; i < nloop; ++i) {
                    const int c = tid + 256 * i;
                    if (c < chunks) store_squares4(sq_lds, c, chunk_at(i, c));
                }
                __syncthreads();
                ss = sum_sequential_lds(sq_lds, k);
            } else {
                ss = sum_squares_sequential<MODE>(src, row);
            }
        } else {
            float part = 0.0f;  // thread tid is virtual lane tid
#pragma unroll
            for (int i = 0; i < nloop; ++i) part = sum_squares4(part, chunk_at(i, tid + 256 * i));
            part = wave_sum_f32(part);
            if (lane == 0) red_f[0][wave] = part;
            __syncthreads();
            ss = f32_add(f32_add(f32_add(red_f[0][0], red_f[0][1]), red_f[0][2]), red_f[0][3]);
        }
        rdiv = make_row_divisor(rms_from_ss(ss, k, src.eps));
    }

    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < nloop; ++i) {
        int c = tid + 256 * i;
        float4 e = chunk_at(i, c);
        if (norm && c < chunks) e = normalize4(e, rdiv, load_gamma_chunk(src, c, VEC));
        if constexpr (NCH > 0) v[i] = e;
        amax = absmax4(amax, e);
    }
    amax = wave_max_f32(amax);
    if (lane == 0) red_f[1][wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red_f[1][0], red_f[1][1]), fmaxf(red_f[1][2], red_f[1][3]));
    const float scale = scale_from_absmax(amax);

    int isum = 0;
#pragma unroll
    for (int i = 0; i < nloop; ++i) {
        int c = tid + 256 * i;
        if (c >= chunks) continue;
        float4 e;
        if constexpr (NCH > 0) {
            e = v[i];
        } else {
            e = load_chunk<MODE, VEC>(src, row, c);
            if (norm) e = normalize4(e, rdiv, load_gamma_chunk(src, c, VEC));
        }
        size_t base = row * (size_t)k + 4 * (size_t)c;
        if constexpr (VEC) {
            *reinterpret_cast<uint32_t *>(p.q + base) = quant4_packed(e, scale, &isum);
            if (p.y) *reinterpret_cast<float4 *>(p.y + base) = e;
        } else {
            float es[4] = {e.x, e.y, e.z, e.w};
            for (int j = 0; j < 4; ++j) {
                if (4 * c + j < k) {
                    int qv = quant1(es[j], scale);
                    p.q[base + j] = (int8_t)qv;
                    if (p.y) p.y[base + j] = es[j];
                    isum += qv;
                }
            }
        }
    }
    isum = wave_sum_i32(isum);
    if (lane == 0) red_i[wave] = isum;
    __syncthreads();
    if (tid == 0) {
        p.a_scale[row] = scale;
        if (p.a_sum) p.a_sum[row] = red_i[0] + red_i[1] + red_i[2] + red_i[3];
    }
}

// One workgroup of 16 wavefronts per row, for the few rows of a decode batch: a row is then one workgroup's whole
// work, so its time is the row's arithmetic divided by the threads that share it.  Thread t owns chunks t, t + 1024
// (NCHB of them; k <= 4096 * NCHB, 16-byte aligned rows).  The sum of squares keeps the declared order: chunk c belongs
// to virtual lane c % 256, so threads 0..255 also fetch the chunks of their lane and run its chain, then the four 64-lane
// butterflies.  Same bits as the other two kernels.
template <int MODE, int NCHB>
__global__ __launch_bounds__(1024) void act_quant_block16_kernel(const float *hot_x, int hot_ldx, int hot_k, const float *hot_x2,
                                                                const float *hot_gamma, int hot_head_dim, int hot_gqa_group,
                                                                ActQuantParams p)
{
    __shared__ float red_f[2][16];
    __shared__ int red_i[16];
    // the leading scalar arguments repeat what the first loads need; they are preloaded into registers (see the Makefile)
    RowSource src = p.src;
    src.x = hot_x; src.ldx = (size_t)hot_ldx; src.k = hot_k; src.x2 = hot_x2; src.gamma = hot_gamma;
    src.head_dim = hot_head_dim; src.gqa_group = hot_gqa_group;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const size_t row = blockIdx.x;
    const int k = src.k, chunks = k >> 2;
    const bool norm = src.gamma != nullptr;
    constexpr int NSS = 4 * NCHB;

    // all loads up front, unconditional (clamped indices, values discarded), addressed by the preloaded arguments alone:
    // the argument buffer is read only once they are on their way (wavefronts 0..3 fetch their lanes' chunks whatever
    // the summation order turns out to be)
    float4 v[NCHB], gm[NCHB], vs[NSS];
#pragma unroll
    for (int i = 0; i < NCHB; ++i) v[i] = load_chunk<MODE, true>(src, row, min(tid + 1024 * i, chunks - 1));
    if (norm && wave < 4) {
#pragma unroll
        for (int i = 0; i < NSS; ++i) vs[i] = load_chunk<MODE, true>(src, row, min(tid + 256 * i, chunks - 1));
    }
    if (norm) {
#pragma unroll
        for (int i = 0; i < NCHB; ++i) gm[i] = load_gamma_chunk(src, min(tid + 1024 * i, chunks - 1), true);
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing below moves above: the first wait for the argument buffer comes here
    clear_counters(p);
    const bool chain = norm && src.sum_order != BITNET_HIP_SUM_SEQUENTIAL && wave < 4;
#pragma unroll
    for (int i = 0; i < NCHB; ++i)
        if (tid + 1024 * i >= chunks) v[i] = make_float4(0.f, 0.f, 0.f, 0.f);

    if (norm) {
        float ss;
        if (src.sum_order == BITNET_HIP_SUM_SEQUENTIAL) {
            if (p.seq_in_lds) {
                extern __shared__ float sq_lds[];  // squares_lds_bytes(k)
#pragma unroll
                for (int i = 0; i < NCHB; ++i)
                    if (tid + 1024 * i < chunks) store_squares4(sq_lds, tid + 1024 * i, v[i]);
                lds_barrier();
                ss = sum_sequential_lds(sq_lds, k);
            } else {
                ss = sum_squares_sequential<MODE>(src, row);
            }
        } else {
            if (chain) {  // thread tid < 256 is virtual lane tid
                float part = 0.0f;
#pragma unroll
                for (int i = 0; i < NSS; ++i)
                    if (tid + 256 * i < chunks) part = sum_squares4(part, vs[i]);  // chunks past the end would add +0
                part = wave_sum_f32(part);
                if (lane == 0) red_f[0][wave] = part;
            }
            lds_barrier();
            ss = f32_add(f32_add(f32_add(red_f[0][0], red_f[0][1]), red_f[0][2]), red_f[0][3]);
        }
        const RowDivisor rdiv = make_row_divisor(rms_from_ss(ss, k, src.eps));
#pragma unroll
        for (int i = 0; i < NCHB; ++i)
            if (tid + 1024 * i < chunks) v[i] = normalize4(v[i], rdiv, gm[i]);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCHB; ++i) amax = absmax4(amax, v[i]);
    amax = wave_max_f32(amax);
    if (lane == 0) red_f[1][wave] = amax;
    lds_barrier();
    amax = red_f[1][0];
#pragma unroll
    for (int w = 1; w < 16; ++w) amax = fmaxf(amax, red_f[1][w]);
    const float scale = scale_from_absmax(amax);

    int isum = 0;
#pragma unroll
    for (int i = 0; i < NCHB; ++i) {
        const int c = tid + 1024 * i;
        if (c < chunks) {
            const size_t base = row * (size_t)k + 4 * (size_t)c;
            *reinterpret_cast<uint32_t *>(p.q + base) = quant4_packed(v[i], scale, &isum);
            if (p.y) *reinterpret_cast<float4 *>(p.y + base) = v[i];
        }
    }
    isum = wave_sum_i32(isum);
    if (lane == 0) red_i[wave] = isum;
    lds_barrier();
    if (tid == 0) {
        p.a_scale[row] = scale;
        if (p.a_sum) {
            int total = 0;
#pragma unroll
            for (int w = 0; w < 16; ++w) total += red_i[w];
            p.a_sum[row] = total;
        }
    }
}

template <int MODE, int NCH, bool VEC>
void launch_wave(const ActQuantParams &p, hipStream_t s)
{
    const int rows_per_block = 4;
    dim3 block(64, rows_per_block);
    dim3 grid((unsigned)((p.m + rows_per_block - 1) / rows_per_block));
    hipLaunchKernelGGL((act_quant_wave_kernel<MODE, NCH, VEC>), grid, block, 0, s, p);
}

// LDS for the row's squares where the literal summation order is asked for and a row fits the default limit
inline size_t launch_squares_lds(const ActQuantParams &p)
{
    if (!p.src.gamma || p.src.sum_order != BITNET_HIP_SUM_SEQUENTIAL) return 0;
    const size_t bytes = squares_lds_bytes(p.src.k);
    return bytes <= 60 * 1024 ? bytes : 0;
}

template <int MODE, int NCH, bool VEC>
void launch_block(ActQuantParams p, hipStream_t s)
{
    const size_t lds = launch_squares_lds(p);
    p.seq_in_lds = lds != 0;
    hipLaunchKernelGGL((act_quant_block_kernel<MODE, NCH, VEC>), dim3((unsigned)p.m), dim3(256), lds, s, p);
}

template <int MODE>
void launch_mode(const ActQuantParams &p, bool vec, hipStream_t s)
{
    const int chunks = (p.src.k + 3) >> 2;
    // Few rows (a decode batch): 16 wavefronts per row.
    if (p.m <= 16 && vec && chunks <= 2048 && p.src.ldx < (1u << 31)) {
#define BITNET_HOT_ARGS p.src.x, (int)p.src.ldx, p.src.k, p.src.x2, p.src.gamma, p.src.head_dim, p.src.gqa_group
        ActQuantParams q = p;
        const size_t lds = launch_squares_lds(p);
        q.seq_in_lds = lds != 0;
        if (chunks <= 1024) hipLaunchKernelGGL((act_quant_block16_kernel<MODE, 1>), dim3((unsigned)p.m), dim3(1024), lds, s, BITNET_HOT_ARGS, q);
        else hipLaunchKernelGGL((act_quant_block16_kernel<MODE, 2>), dim3((unsigned)p.m), dim3(1024), lds, s, BITNET_HOT_ARGS, q);
#undef BITNET_HOT_ARGS
        return;
    }
    // A workgroup per row for few rows, and for any number of rows whose chunks fit the threads' registers: with
    // more, shorter-lived workgroups in flight the load latency of one overlaps the arithmetic of others (measured
    // at 2048 rows: 8.0 us against 9.0 us at k = 2560, 16.9 us against 23.1 us at k = 6912).
    if (p.m <= 32 || (vec && ((chunks + 255) >> 8) <= 7)) {
        if (!vec) return launch_block<MODE, 0, false>(p, s);
        const int per_thread = (chunks + 255) >> 8;
        if (per_thread <= 3) return launch_block<MODE, 3, true>(p, s);
        if (per_thread <= 7) return launch_block<MODE, 7, true>(p, s);
        if (per_thread <= 16) return launch_block<MODE, 16, true>(p, s);
        return launch_block<MODE, 0, true>(p, s);
    }
    if (!vec) return launch_wave<MODE, 0, false>(p, s);
    const int per_lane = (chunks + 63) >> 6;
    if (per_lane <= 4) return launch_wave<MODE, 4, true>(p, s);
    if (per_lane <= 10) return launch_wave<MODE, 10, true>(p, s);
    if (per_lane <= 16) return launch_wave<MODE, 16, true>(p, s);
    if (per_lane <= 27) return launch_wave<MODE, 27, true>(p, s);
    if (per_lane <= 32) return launch_wave<MODE, 32, true>(p, s);
    return launch_wave<MODE, 0, true>(p, s);
}

inline bool aligned(const void *ptr, size_t a) { return (reinterpret_cast<uintptr_t>(ptr) % a) == 0; }

// ---- absmax_quantize_activations: one scale for the whole tensor (bitnet-quant/src/quantization/activations.rs:530-641) ----
//
// Pass 1: abs-max / min / max of the tensor (order-free).  Pass 2: q = ternary code or 8-bit value of x / scale and the
// squared error of every element, summed in f64 over "rows" of 4096 consecutive elements (lane l of a wavefront adds
// elements l, l + 64, ... of its row in ascending order, butterfly 32..1; the row sums are combined the same way by
// one wavefront).  Elements past the end count as +0.
struct AbsmaxState {
    float abs_max, lo, hi, scale;
};

__global__ __launch_bounds__(256) void absmax_partial_kernel(const float *x, size_t n, float *part /* [3][gridDim.x] */)
{
    float am = 0.0f, lo = __builtin_inff(), hi = -__builtin_inff();
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const float v = x[i];
        am = fmaxf(am, fabsf(v));
        lo = fminf(lo, v);
        hi = fmaxf(hi, v);
    }
    __shared__ float sh[3][4];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        am = fmaxf(am, __shfl_xor(am, off, 64));
        lo = fminf(lo, __shfl_xor(lo, off, 64));
        hi = fmaxf(hi, __shfl_xor(hi, off, 64));
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { sh[0][wave] = am; sh[1][wave] = lo; sh[2][wave] = hi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        part[blockIdx.x] = fmaxf(fmaxf(sh[0][0], sh[0][1]), fmaxf(sh[0][2], sh[0][3]));
        part[gridDim.x + blockIdx.x] = fminf(fminf(sh[1][0], sh[1][1]), fminf(sh[1][2], sh[1][3]));
        part[2 * gridDim.x + blockIdx.x] = fmaxf(fmaxf(sh[2][0], sh[2][1]), fmaxf(sh[2][2], sh[2][3]));
    }
}

__global__ __launch_bounds__(64) void absmax_scale_kernel(const float *part, int blocks, int precision, AbsmaxState *state)
{
    float am = 0.0f, lo = __builtin_inff(), hi = -__builtin_inff();
    for (int b = threadIdx.x; b < blocks; b += 64) {
        am = fmaxf(am, part[b]);
        lo = fminf(lo, part[blocks + b]);
        hi = fmaxf(hi, part[2 * blocks + b]);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        am = fmaxf(am, __shfl_xor(am, off, 64));
        lo = fminf(lo, __shfl_xor(lo, off, 64));
        hi = fmaxf(hi, __shfl_xor(hi, off, 64));
    }
    if (threadIdx.x == 0) {
        float scale = 1.0f;  // abs_max below f32::EPSILON: no division by (almost) zero, activations.rs:557-561
        if (!(am < 1.1920929e-07f)) scale = precision == BITNET_HIP_PRECISION_EIGHT_BIT ? f32_div(am, 127.0f) : am;
        state->abs_max = am; state->lo = lo; state->hi = hi; state->scale = scale;
    }
}

// one wavefront per row of 4096 elements
__global__ __launch_bounds__(256) void absmax_quantize_kernel(const float *x, size_t n, size_t rows, int precision,
                                                              const AbsmaxState *state, int8_t *q, double *row_sums)
{
    const int lane = threadIdx.x;
    const size_t row = (size_t)blockIdx.x * blockDim.y + threadIdx.y;
    if (row >= rows) return;
    const float scale = state->scale;
    double s = 0.0;
    for (size_t i = row * 4096 + lane; i < (row + 1) * 4096 && i < n; i += 64) {
        const float v = x[i];
        const float scaled = f32_div(v, scale);
        float qv;
        if (precision == BITNET_HIP_PRECISION_EIGHT_BIT) {
            float c = scaled > 127.0f ? 127.0f : scaled;
            c = c < -127.0f ? -127.0f : c;
            qv = roundf(c);  // halves away from zero, as f32::round
        } else {
            qv = scaled > 0.5f ? 1.0f : (scaled < -0.5f ? -1.0f : 0.0f);
        }
        const int8_t qi = (qv != qv) ? (int8_t)0 : (int8_t)qv;
        q[i] = qi;
        const float d = v - f32_mul((float)qi, scale);
        s = s + (double)f32_mul(d, d);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s = s + __shfl_xor(s, off, 64);
    if (lane == 0) row_sums[row] = s;
}

__global__ __launch_bounds__(64) void absmax_finish_kernel(const double *row_sums, size_t rows, size_t n, const AbsmaxState *state,
                                                           float *stats)
{
    double s = 0.0;
    for (size_t r = threadIdx.x; r < rows; r += 64) s = s + row_sums[r];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s = s + __shfl_xor(s, off, 64);
    if (threadIdx.x == 0) {
        stats[0] = state->scale;
        stats[1] = n ? (float)(s / (double)n) : 0.0f;
        stats[2] = state->lo;
        stats[3] = state->hi;
    }
}

// DynamicActivationQuantizer::quantize with a scale given from outside (activations.rs:269-294, 315-360): y = x * r with
// r = (float)(1.0 / (double)scale), as candle's affine(1.0 / scale as f64, 0.0) computes it on an f32 tensor.
//   ternary: +1 where y > 0.5, -1 where y < -0.5, else 0
//   8-bit:   round(clamp(y, -127, 127)) as int8, or, with reference_u8, the reference's literal clamp(0, 255).round()
//            as the byte of a u8 (every negative activation becomes 0 there)
__global__ __launch_bounds__(256) void scaled_quantize_kernel(const float *x, size_t n, int precision, float recip, int reference_u8,
                                                              int8_t *q)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const float y = f32_mul(x[i], recip);
        int v;
        if (precision == BITNET_HIP_PRECISION_EIGHT_BIT) {
            const float lo = reference_u8 ? 0.0f : -127.0f, hi = reference_u8 ? 255.0f : 127.0f;
            float c = y > hi ? hi : y;
            c = c < lo ? lo : c;
            const float r = roundf(c);  // halves away from zero, as f32::round
            v = (r != r) ? 0 : (int)r;
        } else {
            v = y > 0.5f ? 1 : (y < -0.5f ? -1 : 0);
        }
        q[i] = (int8_t)(uint8_t)(unsigned)v;  // 0..255 keep their byte in the u8 form
    }
}

}  // namespace

int launch_abs_max(const float *x, size_t n, void *scratch, hipStream_t stream)
{
    AbsmaxState *state = static_cast<AbsmaxState *>(scratch);
    float *part = reinterpret_cast<float *>(static_cast<uint8_t *>(scratch) + 256);
    int blocks = (int)((n + 255) / 256);
    blocks = blocks < 1 ? 1 : (blocks > 1024 ? 1024 : blocks);
    hipLaunchKernelGGL(absmax_partial_kernel, dim3(blocks), dim3(256), 0, stream, x, n, part);
    BITNET_HIP_CHECK_LAUNCH("absmax_partial_kernel");
    hipLaunchKernelGGL(absmax_scale_kernel, dim3(1), dim3(64), 0, stream, part, blocks, BITNET_HIP_PRECISION_ONE_FIVE_FIVE_BIT, state);
    BITNET_HIP_CHECK_LAUNCH("absmax_scale_kernel");
    return BITNET_HIP_OK;  // state->abs_max is the first float of the scratch
}

int launch_scaled_quantize(const float *x, size_t n, int precision, float scale, int reference_u8, int8_t *q, hipStream_t stream)
{
    if (n == 0) return BITNET_HIP_OK;
    const float recip = (float)(1.0 / (double)scale);
    size_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(scaled_quantize_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, n, precision, recip, reference_u8, q);
    BITNET_HIP_CHECK_LAUNCH("scaled_quantize_kernel");
    return BITNET_HIP_OK;
}

size_t absmax_quantize_scratch_bytes(size_t n)
{
    const size_t rows = (n + 4095) / 4096;
    return 256 + sizeof(float) * 3 * 1024 + sizeof(double) * (rows ? rows : 1);
}

int launch_absmax_quantize(const float *x, size_t n, int precision, void *scratch, int8_t *q, float *stats, hipStream_t stream)
{
    AbsmaxState *state = static_cast<AbsmaxState *>(scratch);
    float *part = reinterpret_cast<float *>(static_cast<uint8_t *>(scratch) + 256);
    double *row_sums = reinterpret_cast<double *>(static_cast<uint8_t *>(scratch) + 256 + sizeof(float) * 3 * 1024);
    const size_t rows = (n + 4095) / 4096;
    int blocks = (int)((n + 255) / 256);
    blocks = blocks < 1 ? 1 : (blocks > 1024 ? 1024 : blocks);
    hipLaunchKernelGGL(absmax_partial_kernel, dim3(blocks), dim3(256), 0, stream, x, n, part);
    BITNET_HIP_CHECK_LAUNCH("absmax_partial_kernel");
    hipLaunchKernelGGL(absmax_scale_kernel, dim3(1), dim3(64), 0, stream, part, blocks, precision, state);
    BITNET_HIP_CHECK_LAUNCH("absmax_scale_kernel");
    if (rows) {
        hipLaunchKernelGGL(absmax_quantize_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(64, 4), 0, stream, x, n, rows, precision,
                           state, q, row_sums);
        BITNET_HIP_CHECK_LAUNCH("absmax_quantize_kernel");
    }
    hipLaunchKernelGGL(absmax_finish_kernel, dim3(1), dim3(64), 0, stream, row_sums, rows, n, state, stats);
    BITNET_HIP_CHECK_LAUNCH("absmax_finish_kernel");
    return BITNET_HIP_OK;
}

int launch_act_quant(const float *x, const float *x2, size_t ldx, size_t m, size_t k, int input_mode,
                     size_t gqa_group, size_t head_dim, const float *gamma, float eps, int sum_order,
                     int8_t *q, float *a_scale, int32_t *a_sum, float *y, hipStream_t stream, unsigned *zero, size_t zero_n)
{
    ActQuantParams p;
    p.zero = zero; p.zero_n = (int)zero_n;
    p.src.x = x; p.src.x2 = x2; p.src.gamma = gamma; p.src.ldx = ldx; p.src.k = (int)k;
    p.src.head_dim = (int)(head_dim ? head_dim : 1); p.src.gqa_group = (int)(gqa_group ? gqa_group : 1);
    p.src.sum_order = sum_order; p.src.eps = eps;
    p.q = q; p.a_scale = a_scale; p.a_sum = a_sum; p.y = y; p.m = m; p.seq_in_lds = 0;

    bool vec = (k % 4 == 0) && (ldx % 4 == 0) && aligned(x, 16) && aligned(q, 4) && (!x2 || aligned(x2, 16)) &&
               (!y || aligned(y, 16)) && (!gamma || aligned(gamma, 16));
    if (input_mode == BITNET_HIP_INPUT_GQA_BROADCAST) vec = vec && (head_dim % 4 == 0);

    switch (input_mode) {
        case BITNET_HIP_INPUT_PLAIN: launch_mode<BITNET_HIP_INPUT_PLAIN>(p, vec, stream); break;
        case BITNET_HIP_INPUT_RELU2_MUL: launch_mode<BITNET_HIP_INPUT_RELU2_MUL>(p, vec, stream); break;
        default: launch_mode<BITNET_HIP_INPUT_GQA_BROADCAST>(p, vec, stream); break;
    }
    BITNET_HIP_CHECK_LAUNCH("act_quant kernel");
    return BITNET_HIP_OK;
}

}  // namespace bitnet
