// Fused RMSNorm + per-token absmax int8 activation quantiser for gfx950.
//
// Arithmetic (every f32 step is one IEEE operation; no contraction, no approximate divide/sqrt):
//   ss      = sum_k x[k]*x[k]                      bitnet-inference/src/engine/inference_integration.rs:476
//   rms     = sqrt(ss / K + eps)                   :477
//   y[k]    = (x[k] / rms) * gamma[k]              :481
//   absmax  = max_k |y[k]|                         bitnet-inference/src/engine/ternary_operations.rs:143-145
//   a_scale = absmax > 0 ? 127 / absmax : 1        :147-151
//   q[k]    = clamp(round(y[k] * a_scale),-128,127) :158-161  (round = half away from zero)
//
// One wavefront owns one token row and keeps it in registers between the three passes (sum of squares,
// absmax, quantise), so the row is read from HBM once: 4*K bytes in, K + 4 bytes out.
//
// Order of the f32 sum of squares (the only order-dependent step):
//   BITNET_HIP_SUM_WAVE64     the row is cut into chunks of 4 consecutive elements; chunk c belongs to
//                             lane c mod 64; a lane adds its squares in ascending chunk order and, inside
//                             a chunk, ascending element order, from +0; the 64 partials are combined by
//                             p += shfl_xor(p, off) for off = 32,16,8,4,2,1.
//   BITNET_HIP_SUM_SEQUENTIAL one running sum over k ascending (the reference's literal loop); every lane
//                             runs the same chain, so it costs about K dependent additions.
#include "kernels.hpp"

namespace bitnet {

namespace {

struct ActQuantParams {
    const float *x;
    const float *x2;
    const float *gamma;
    int8_t *q;
    float *a_scale;
    int32_t *a_sum;
    float *y;
    size_t ldx;
    size_t m;
    int k;
    int head_dim;
    int gqa_group;
    int sum_order;
    float eps;
};

__device__ __forceinline__ float wave_sum_f32(float p)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) p = f32_add(p, __shfl_xor(p, off, 64));
    return p;
}

__device__ __forceinline__ float wave_max_f32(float p)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) p = fmaxf(p, __shfl_xor(p, off, 64));
    return p;
}

__device__ __forceinline__ int wave_sum_i32(int p)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) p += __shfl_xor(p, off, 64);
    return p;
}

__device__ __forceinline__ float relu2_mul(float gate, float up)
{
    float r = gate > 0.0f ? gate : 0.0f;
    return f32_mul(up, f32_mul(r, r));
}

// Element i of the (virtual) input row `row` after the fused input transform.
template <int MODE>
__device__ __forceinline__ float load_elem(const ActQuantParams &p, size_t row, int i)
{
    if constexpr (MODE == BITNET_HIP_INPUT_PLAIN) {
        return p.x[row * p.ldx + i];
    } else if constexpr (MODE == BITNET_HIP_INPUT_RELU2_MUL) {
        return relu2_mul(p.x[row * p.ldx + i], p.x2[row * p.ldx + i]);
    } else {
        int h = i / p.head_dim, d = i - h * p.head_dim;
        return p.x[row * p.ldx + (size_t)(h / p.gqa_group) * p.head_dim + d];
    }
}

// Chunk c (elements 4c .. 4c+3).  VEC: 16-byte loads, all four elements inside the row.
template <int MODE, bool VEC>
__device__ __forceinline__ float4 load_chunk(const ActQuantParams &p, size_t row, int c)
{
    if constexpr (VEC) {
        if constexpr (MODE == BITNET_HIP_INPUT_PLAIN) {
            return *reinterpret_cast<const float4 *>(p.x + row * p.ldx + 4 * (size_t)c);
        } else if constexpr (MODE == BITNET_HIP_INPUT_RELU2_MUL) {
            float4 g = *reinterpret_cast<const float4 *>(p.x + row * p.ldx + 4 * (size_t)c);
            float4 u = *reinterpret_cast<const float4 *>(p.x2 + row * p.ldx + 4 * (size_t)c);
            return make_float4(relu2_mul(g.x, u.x), relu2_mul(g.y, u.y), relu2_mul(g.z, u.z),
                               relu2_mul(g.w, u.w));
        } else {
            int i = 4 * c;
            int h = i / p.head_dim, d = i - h * p.head_dim;
            return *reinterpret_cast<const float4 *>(p.x + row * p.ldx +
                                                     (size_t)(h / p.gqa_group) * p.head_dim + d);
        }
    } else {
        float4 v;
        int i = 4 * c;
        v.x = i + 0 < p.k ? load_elem<MODE>(p, row, i + 0) : 0.0f;
        v.y = i + 1 < p.k ? load_elem<MODE>(p, row, i + 1) : 0.0f;
        v.z = i + 2 < p.k ? load_elem<MODE>(p, row, i + 2) : 0.0f;
        v.w = i + 3 < p.k ? load_elem<MODE>(p, row, i + 3) : 0.0f;
        return v;
    }
}

__device__ __forceinline__ int quant1(float y, float scale)
{
    float t = roundf(f32_mul(y, scale));
    if (t != t) return 0;
    t = fminf(fmaxf(t, -128.0f), 127.0f);
    return (int)t;
}

// NCH > 0: a lane keeps its NCH chunks in registers (K <= 256*NCH).  NCH == 0: any K, the row is
// re-read (from cache) in each pass.
template <int MODE, int NCH, bool VEC>
__global__ __launch_bounds__(256) void act_quant_kernel(ActQuantParams p)
{
    const int lane = threadIdx.x;
    const size_t row = (size_t)blockIdx.x * blockDim.y + threadIdx.y;
    if (row >= p.m) return;  // uniform per wavefront: a wavefront is one row
    const int chunks = (p.k + 3) >> 2;
    const int nloop = NCH > 0 ? NCH : (chunks + 63) >> 6;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);

    float4 v[NCH > 0 ? NCH : 1];
    if constexpr (NCH > 0) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            int c = lane + 64 * i;
            v[i] = c < chunks ? load_chunk<MODE, VEC>(p, row, c) : zero4;
        }
    }
    auto chunk_at = [&](int i, int c) -> float4 {
        if constexpr (NCH > 0) return v[i];
        else return c < chunks ? load_chunk<MODE, VEC>(p, row, c) : zero4;
    };

    float rms = 1.0f;
    const bool norm = p.gamma != nullptr;
    if (norm) {
        float ss;
        if (p.sum_order == BITNET_HIP_SUM_SEQUENTIAL) {
            ss = 0.0f;
            for (int i = 0; i < p.k; ++i) {
                float e = load_elem<MODE>(p, row, i);
                ss = f32_add(ss, f32_mul(e, e));
            }
        } else {
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < nloop; ++i) {
                float4 e = chunk_at(i, lane + 64 * i);
                part = f32_add(part, f32_mul(e.x, e.x));
                part = f32_add(part, f32_mul(e.y, e.y));
                part = f32_add(part, f32_mul(e.z, e.z));
                part = f32_add(part, f32_mul(e.w, e.w));
            }
            ss = wave_sum_f32(part);
        }
        rms = f32_sqrt(f32_add(f32_div(ss, (float)p.k), p.eps));
    }

    // normalised value of element `idx` whose raw value is e
    auto normed = [&](float e, int idx) -> float {
        if (!norm) return e;
        float g = idx < p.k ? p.gamma[idx] : 0.0f;
        return f32_mul(f32_div(e, rms), g);
    };

    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < nloop; ++i) {
        int c = lane + 64 * i;
        float4 e = chunk_at(i, c);
        e.x = normed(e.x, 4 * c + 0);
        e.y = normed(e.y, 4 * c + 1);
        e.z = normed(e.z, 4 * c + 2);
        e.w = normed(e.w, 4 * c + 3);
        if constexpr (NCH > 0) v[i] = e;
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(e.x), fabsf(e.y)), fmaxf(fabsf(e.z), fabsf(e.w))));
    }
    amax = wave_max_f32(amax);
    const float scale = amax > 0.0f ? f32_div(127.0f, amax) : 1.0f;

    int isum = 0;
#pragma unroll
    for (int i = 0; i < nloop; ++i) {
        int c = lane + 64 * i;
        if (c >= chunks) continue;
        float4 e;
        if constexpr (NCH > 0) {
            e = v[i];
        } else {
            e = load_chunk<MODE, VEC>(p, row, c);
            e.x = normed(e.x, 4 * c + 0);
            e.y = normed(e.y, 4 * c + 1);
            e.z = normed(e.z, 4 * c + 2);
            e.w = normed(e.w, 4 * c + 3);
        }
        int q0 = quant1(e.x, scale), q1 = quant1(e.y, scale), q2 = quant1(e.z, scale),
            q3 = quant1(e.w, scale);
        size_t base = row * (size_t)p.k + 4 * (size_t)c;
        if constexpr (VEC) {
            uint32_t packed = (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) |
                              ((uint32_t)(q2 & 0xff) << 16) | ((uint32_t)(q3 & 0xff) << 24);
            *reinterpret_cast<uint32_t *>(p.q + base) = packed;
            if (p.y) *reinterpret_cast<float4 *>(p.y + base) = e;
            isum += q0 + q1 + q2 + q3;
        } else {
            int qs[4] = {q0, q1, q2, q3};
            float es[4] = {e.x, e.y, e.z, e.w};
            for (int j = 0; j < 4; ++j) {
                if (4 * c + j < p.k) {
                    p.q[base + j] = (int8_t)qs[j];
                    if (p.y) p.y[base + j] = es[j];
                    isum += qs[j];
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

template <int MODE, int NCH, bool VEC>
void launch_one(const ActQuantParams &p, hipStream_t s)
{
    const int rows_per_block = 4;
    dim3 block(64, rows_per_block);
    dim3 grid((unsigned)((p.m + rows_per_block - 1) / rows_per_block));
    hipLaunchKernelGGL((act_quant_kernel<MODE, NCH, VEC>), grid, block, 0, s, p);
}

template <int MODE>
void launch_mode(const ActQuantParams &p, bool vec, hipStream_t s)
{
    if (!vec) return launch_one<MODE, 0, false>(p, s);
    const int per_lane = (((p.k + 3) >> 2) + 63) >> 6;
    if (per_lane <= 4) return launch_one<MODE, 4, true>(p, s);
    if (per_lane <= 10) return launch_one<MODE, 10, true>(p, s);
    if (per_lane <= 16) return launch_one<MODE, 16, true>(p, s);
    if (per_lane <= 27) return launch_one<MODE, 27, true>(p, s);
    if (per_lane <= 32) return launch_one<MODE, 32, true>(p, s);
    return launch_one<MODE, 0, true>(p, s);
}

inline bool aligned(const void *ptr, size_t a) { return (reinterpret_cast<uintptr_t>(ptr) % a) == 0; }

}  // namespace

int launch_act_quant(const float *x, const float *x2, size_t ldx, size_t m, size_t k, int input_mode,
                     size_t gqa_group, size_t head_dim, const float *gamma, float eps, int sum_order,
                     int8_t *q, float *a_scale, int32_t *a_sum, float *y, hipStream_t stream)
{
    ActQuantParams p;
    p.x = x; p.x2 = x2; p.gamma = gamma; p.q = q; p.a_scale = a_scale; p.a_sum = a_sum; p.y = y;
    p.ldx = ldx; p.m = m; p.k = (int)k; p.head_dim = (int)(head_dim ? head_dim : 1);
    p.gqa_group = (int)(gqa_group ? gqa_group : 1); p.sum_order = sum_order; p.eps = eps;

    bool vec = (k % 4 == 0) && (ldx % 4 == 0) && aligned(x, 16) && aligned(q, 4) &&
               (!x2 || aligned(x2, 16)) && (!y || aligned(y, 16));
    if (input_mode == BITNET_HIP_INPUT_GQA_BROADCAST) vec = vec && (head_dim % 4 == 0);

    switch (input_mode) {
        case BITNET_HIP_INPUT_PLAIN: launch_mode<BITNET_HIP_INPUT_PLAIN>(p, vec, stream); break;
        case BITNET_HIP_INPUT_RELU2_MUL: launch_mode<BITNET_HIP_INPUT_RELU2_MUL>(p, vec, stream); break;
        default: launch_mode<BITNET_HIP_INPUT_GQA_BROADCAST>(p, vec, stream); break;
    }
    BITNET_HIP_CHECK_LAUNCH("act_quant_kernel");
    return BITNET_HIP_OK;
}

}  // namespace bitnet
