// Device-side pieces of the fused RMSNorm + per-token absmax int8 quantiser, shared by the stand-alone
// quantiser kernels (act_quant.hip) and by the decode GEMV, which quantises its input row itself
// (gemv_w2a8.hip).  Every caller produces the same bits for the same row.
//
// Arithmetic (each f32 step one IEEE operation):
//   ss      = sum_k x[k]*x[k]                      bitnet-inference/src/engine/inference_integration.rs:476
//   rms     = sqrt(ss / K + eps)                   :477
//   y[k]    = (x[k] / rms) * gamma[k]              :481
//   absmax  = max_k |y[k]|                         bitnet-inference/src/engine/ternary_operations.rs:143-145
//   a_scale = absmax > 0 ? 127 / absmax : 1        :147-151
//   q[k]    = clamp(round(y[k] * a_scale),-128,127) :158-161  (round = half away from zero)
//
// Order of the f32 sum of squares, the only order-dependent step (BITNET_HIP_SUM_BLOCK256):
//   the row is cut into chunks of 4 consecutive elements; chunk c belongs to virtual lane c mod 256; a lane
//   adds the squares of its chunks in ascending chunk order and, inside a chunk, ascending element order,
//   starting from +0; the 256 partials form 4 groups of 64 consecutive lanes, each combined by the butterfly
//   p[l] += p[l ^ off], off = 1,2,4,8,16,32; the four group sums are added as ((s0 + s1) + s2) + s3.
//   (After the step with offset `off` all lanes of an aligned group of 2*off lanes hold the same value, so a
//   step may fetch its operand from ANY lane of the partner group: the kernels use DPP quad permutes and row
//   mirrors for offsets 1..8 and the row / half swap instructions for 16 and 32.)
//   A 256-thread workgroup maps thread = virtual lane; a single wavefront keeps 4 partials per lane
//   (virtual lanes l, l+64, l+128, l+192).  Elements past K count as 0.
// BITNET_HIP_SUM_SEQUENTIAL is the reference's literal running sum over k ascending.
#pragma once
#include "common.hpp"
#include "ieee.hpp"

namespace bitnet {

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global load in flight,
// which would stall a kernel that requests its weight tiles ahead of the code that needs them.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Wavefronts per workgroup of gemv_fused16_kernel for a row of k columns: one per 256 columns, at least the four of
// the declared summation order, at most 16.  (The stand-alone quantiser with a workgroup per row gains nothing from
// the same rule: measured on the 8- to 16-token decoder stack.)
__host__ __device__ inline int row_workgroup_waves(int k)
{
    const int kt = (k + 255) >> 8;
    return kt > 16 ? 16 : (kt < 4 ? 4 : kt);
}

struct RowSource {
    const float *x;      // [m, ldx]
    const float *x2;     // second operand of RELU2_MUL
    const float *gamma;  // RMSNorm weight or nullptr
    size_t ldx;
    int k;
    int head_dim;
    int gqa_group;
    int sum_order;
    float eps;
};

// Lane exchanges of the butterfly.  CTRL is a DPP control word: 0xB1 = quad_perm[1,0,3,2] (l ^ 1),
// 0x4E = quad_perm[2,3,0,1] (l ^ 2), 0x141 = row_half_mirror (a lane of the other quad of the same 8),
// 0x140 = row_mirror (a lane of the other half of the same 16).
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
// Offsets 16 and 32 without a trip through LDS: gfx950's row and half swaps.  With both operands holding p,
// v_permlane16_swap leaves (rows 0,0,2,2 of p) in the first and (rows 1,1,3,3) in the second, v_permlane32_swap
// (lower half twice) and (upper half twice): every lane then holds its own value in one of them and its partner's
// in the other, and the combining operations here are commutative.  (Inline asm: the compiler's builtin for these
// instructions folds the two results into one.  The s_nop covers the wait states between a VALU write of the
// operands and the swap.)
template <typename T>
__device__ __forceinline__ void swap_rows16(T &a, T &b)
{
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
template <typename T>
__device__ __forceinline__ void swap_halves32(T &a, T &b)
{
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}

// 4-element sum over lanes l, l ^ 16, l ^ 32, l ^ 48 (the four column groups of a weight-tile row) in every lane.
__device__ __forceinline__ int sum_over_lane_groups(int v)
{
    int a = v, b = v;
    swap_rows16(a, b);
    a += b;
    b = a;
    swap_halves32(a, b);
    return a + b;
}

#define BITNET_WAVE_REDUCE(TYPE, NAME, COMBINE)                                                    \
    __device__ __forceinline__ TYPE NAME(TYPE p)                                                   \
    {                                                                                              \
        auto step = [](TYPE a, int other_bits) { TYPE b = __builtin_bit_cast(TYPE, other_bits); return COMBINE; }; \
        p = step(p, dpp_i32<0xB1>(__builtin_bit_cast(int, p)));                                    \
        p = step(p, dpp_i32<0x4E>(__builtin_bit_cast(int, p)));                                    \
        p = step(p, dpp_i32<0x141>(__builtin_bit_cast(int, p)));                                   \
        p = step(p, dpp_i32<0x140>(__builtin_bit_cast(int, p)));                                   \
        {                                                                                          \
            TYPE a = p, b = p;                                                                     \
            swap_rows16(a, b);                                                                     \
            p = COMBINE;                                                                           \
        }                                                                                          \
        {                                                                                          \
            TYPE a = p, b = p;                                                                     \
            swap_halves32(a, b);                                                                   \
            p = COMBINE;                                                                           \
        }                                                                                          \
        return p;                                                                                  \
    }
BITNET_WAVE_REDUCE(float, wave_sum_f32, f32_add(a, b))
BITNET_WAVE_REDUCE(float, wave_max_f32, fmaxf(a, b))
BITNET_WAVE_REDUCE(int, wave_sum_i32, a + b)
#undef BITNET_WAVE_REDUCE

__device__ __forceinline__ float relu2_mul(float gate, float up)
{
    float r = gate > 0.0f ? gate : 0.0f;
    return f32_mul(up, f32_mul(r, r));
}

// Element i of the (virtual) input row after the fused input transform.
template <int MODE>
__device__ __forceinline__ float load_elem(const RowSource &p, size_t row, int i)
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
__device__ __forceinline__ float4 load_chunk(const RowSource &p, size_t row, int c)
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

__device__ __forceinline__ float4 load_gamma_chunk(const RowSource &p, int c, bool vec)
{
    if (vec) return *reinterpret_cast<const float4 *>(p.gamma + 4 * (size_t)c);
    float4 g;
    int i = 4 * c;
    g.x = i + 0 < p.k ? p.gamma[i + 0] : 0.0f;
    g.y = i + 1 < p.k ? p.gamma[i + 1] : 0.0f;
    g.z = i + 2 < p.k ? p.gamma[i + 2] : 0.0f;
    g.w = i + 3 < p.k ? p.gamma[i + 3] : 0.0f;
    return g;
}

__device__ __forceinline__ float sum_squares4(float part, const float4 &e)
{
    part = f32_add(part, f32_mul(e.x, e.x));
    part = f32_add(part, f32_mul(e.y, e.y));
    part = f32_add(part, f32_mul(e.z, e.z));
    part = f32_add(part, f32_mul(e.w, e.w));
    return part;
}

// The reference's literal order: every lane runs the same chain over the whole row.
template <int MODE>
__device__ __forceinline__ float sum_squares_sequential(const RowSource &p, size_t row)
{
    float ss = 0.0f;
    for (int i = 0; i < p.k; ++i) {
        float e = load_elem<MODE>(p, row, i);
        ss = f32_add(ss, f32_mul(e, e));
    }
    return ss;
}

// The same literal order with the squares of the row staged in LDS: sq[i] = x[i] * x[i] in element order, written by
// the workgroup (store_squares4) and made visible by a barrier before the call.  Every lane runs the same chain of k
// additions; its reads are broadcasts (one address for all lanes), 16 bytes at a time.  What is left is the latency of
// a dependent v_add_f32, about 8.5 cycles an element (measured; reading further ahead of the additions gains nothing).
__host__ __device__ inline size_t squares_lds_bytes(int k) { return (size_t)((k + 3) >> 2) * 16; }
__device__ __forceinline__ void store_squares4(float *sq, int c, const float4 &e)  // chunk c: elements 4c .. 4c + 3
{
    *reinterpret_cast<float4 *>(sq + 4 * (size_t)c) =
        make_float4(f32_mul(e.x, e.x), f32_mul(e.y, e.y), f32_mul(e.z, e.z), f32_mul(e.w, e.w));
}
__device__ __forceinline__ float sum_sequential_lds(const float *sq, int k)
{
    float ss = 0.0f;
    const int full = k >> 2;
    const float4 *sq4 = reinterpret_cast<const float4 *>(sq);
#pragma unroll 8
    for (int c = 0; c < full; ++c) {
        const float4 s = sq4[c];
        ss = f32_add(f32_add(f32_add(f32_add(ss, s.x), s.y), s.z), s.w);
    }
    for (int i = full * 4; i < k; ++i) ss = f32_add(ss, sq[i]);
    return ss;
}

__device__ __forceinline__ float rms_from_ss(float ss, int k, float eps)
{
    return f32_sqrt(f32_add(f32_div(ss, (float)k), eps));
}

// (x / rms) * g for the four elements of a chunk.  The divisor is the same for the whole row, so the division
// uses div_by_invariant (ieee.hpp), which returns the same bits as x / rms.
struct RowDivisor {
    float d, recip;
    bool fast;
};
__device__ __forceinline__ RowDivisor make_row_divisor(float rms)
{
    RowDivisor r;
    r.d = rms;
    r.recip = f32_div(1.0f, rms);
    r.fast = invariant_divisor_ok(rms);
    return r;
}
__device__ __forceinline__ float4 normalize4(const float4 &e, const RowDivisor &r, const float4 &g)
{
    // the short division when the divisor and, in every lane of the wavefront, all four dividends allow it
    const bool lane_ok = dividend_ok(e.x) && dividend_ok(e.y) && dividend_ok(e.z) && dividend_ok(e.w);
    float4 q;
    if (r.fast && __builtin_amdgcn_ballot_w64(!lane_ok) == 0) {
        q = make_float4(div_by_invariant_unchecked(e.x, r.d, r.recip), div_by_invariant_unchecked(e.y, r.d, r.recip),
                        div_by_invariant_unchecked(e.z, r.d, r.recip), div_by_invariant_unchecked(e.w, r.d, r.recip));
    } else {
        q = make_float4(f32_div(e.x, r.d), f32_div(e.y, r.d), f32_div(e.z, r.d), f32_div(e.w, r.d));
    }
    return make_float4(f32_mul(q.x, g.x), f32_mul(q.y, g.y), f32_mul(q.z, g.z), f32_mul(q.w, g.w));
}

__device__ __forceinline__ float absmax4(float amax, const float4 &e)
{
    return fmaxf(amax, fmaxf(fmaxf(fabsf(e.x), fabsf(e.y)), fmaxf(fabsf(e.z), fabsf(e.w))));
}

__device__ __forceinline__ float scale_from_absmax(float amax)
{
    return amax > 0.0f ? f32_div(127.0f, amax) : 1.0f;
}

__device__ __forceinline__ int quant1(float y, float scale)
{
    // Round half away from zero, then a saturating conversion (NaN converts to 0, as Rust's `as i8` does), then the clamp
    // to [-128, 127] on the integer.  The rounding is one addition of +-(1/2 - 2^-25), the largest float below 1/2, and the
    // truncating conversion: with 1/2 itself the sum for |t| = 1/2 - 2^-25 would round up to 1; with its predecessor
    // that sum is exact, |t| = 1/2 still rounds up to 1, and every other sum is exact or rounds within the gap between
    // two integers (past 2^23, where it may not, the clamp decides).  Checked against roundf, cast and clamp over all
    // 2^32 bit patterns of t.  v_cvt_i32_f32 truncates, saturates and turns NaN into 0.
    const float t = f32_mul(y, scale);
    const float s = f32_add(t, __builtin_copysignf(0x1.fffffep-2f, t));
    int q;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(q) : "v"(s));
    return min(max(q, -128), 127);
}

// Four quantised values of a chunk packed little-endian (byte j = element j); *sum += their sum.
__device__ __forceinline__ uint32_t quant4_packed(const float4 &e, float scale, int *sum)
{
    int q0 = quant1(e.x, scale), q1 = quant1(e.y, scale), q2 = quant1(e.z, scale), q3 = quant1(e.w, scale);
    *sum += q0 + q1 + q2 + q3;
    return (uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8) | ((uint32_t)(q2 & 0xff) << 16) |
           ((uint32_t)(q3 & 0xff) << 24);
}

}  // namespace bitnet
