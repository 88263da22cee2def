/*
 * CPU baselines timed beside the GPU path.  TEST / MEASUREMENT INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * The reference is Rust and cannot be built where this runs, so these are C restatements of what its
 * CPU BitLinear does per call; they are timed, never used to produce a shipped result.
 *
 *   cpu_ref_f32_forward   what bitnet_quant::BitLinear::forward really executes
 *                         (bitnet-quant/src/bitlinear/forward.rs:153-258): materialise the f32 matrix
 *                         q * scale [N,K] on EVERY call (:238-258), then an f32 x @ W^T contraction
 *                         (:179-200) and the optional bias (:117-130).
 *   cpu_ref_simd_gemv     the reference's ternary "SIMD" GEMV semantics
 *                         (bitnet-quant/src/simd/matrix.rs:287-368 AVX2 body, :471-490 scalar):
 *                         i8 ternary weights widened to f32, multiply-add with f32 activations,
 *                         horizontal sum, times scale.
 *   (the third baseline, the int8 oracle itself, is orc_bitlinear_forward in bitlinear_oracle.c)
 *
 * Rows are shared among OpenMP threads; the caller sets the thread count and reports it.
 */
#include <immintrin.h>
#include <omp.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

int cpu_baseline_max_threads(void) { return omp_get_max_threads(); }
void cpu_baseline_set_threads(int n) { omp_set_num_threads(n > 0 ? n : 1); }

__attribute__((target("avx2,fma"))) static float dot_f32_avx2(const float *a, const float *b, size_t k)
{
    __m256 acc0 = _mm256_setzero_ps(), acc1 = _mm256_setzero_ps();
    size_t i = 0;
    for (; i + 16 <= k; i += 16) {
        acc0 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i), _mm256_loadu_ps(b + i), acc0);
        acc1 = _mm256_fmadd_ps(_mm256_loadu_ps(a + i + 8), _mm256_loadu_ps(b + i + 8), acc1);
    }
    acc0 = _mm256_add_ps(acc0, acc1);
    __m128 lo = _mm_add_ps(_mm256_castps256_ps128(acc0), _mm256_extractf128_ps(acc0, 1));
    lo = _mm_hadd_ps(lo, lo);
    lo = _mm_hadd_ps(lo, lo);
    float s = _mm_cvtss_f32(lo);
    for (; i < k; ++i) s += a[i] * b[i];
    return s;
}

__attribute__((target("avx512f"))) static float dot_f32_avx512(const float *a, const float *b, size_t k)
{
    __m512 acc0 = _mm512_setzero_ps(), acc1 = _mm512_setzero_ps();
    size_t i = 0;
    for (; i + 32 <= k; i += 32) {
        acc0 = _mm512_fmadd_ps(_mm512_loadu_ps(a + i), _mm512_loadu_ps(b + i), acc0);
        acc1 = _mm512_fmadd_ps(_mm512_loadu_ps(a + i + 16), _mm512_loadu_ps(b + i + 16), acc1);
    }
    float s = _mm512_reduce_add_ps(_mm512_add_ps(acc0, acc1));
    for (; i < k; ++i) s += a[i] * b[i];
    return s;
}

static float dot_f32(const float *a, const float *b, size_t k, int isa)
{
    if (isa == 2) return dot_f32_avx512(a, b, k);
    if (isa == 1) return dot_f32_avx2(a, b, k);
    float s = 0.0f;
    for (size_t i = 0; i < k; ++i) s += a[i] * b[i];
    return s;
}

/* 0 = scalar, 1 = AVX2+FMA, 2 = AVX-512F: the widest the running host supports. */
int cpu_baseline_isa(void)
{
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx512f")) return 2;
    if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) return 1;
    return 0;
}

/* x [m,k] f32, q [n,k] ternary i8, out [m,n] f32.  wf is caller-provided scratch of n*k floats so
 * that allocation cost is not timed, but it is refilled on every call as the reference does. */
void cpu_ref_f32_forward(const float *x, const int8_t *q, float scale, const float *bias, float *wf,
                         float *out, size_t m, size_t n, size_t k)
{
    int isa = cpu_baseline_isa();
#pragma omp parallel for schedule(static)
    for (long long r = 0; r < (long long)n; ++r) {
        const int8_t *qr = q + (size_t)r * k;
        float *wr = wf + (size_t)r * k;
        for (size_t i = 0; i < k; ++i) wr[i] = (float)qr[i] * scale;
    }
#pragma omp parallel for schedule(static)
    for (long long r = 0; r < (long long)n; ++r) {
        const float *wr = wf + (size_t)r * k;
        for (size_t t = 0; t < m; ++t) {
            float s = dot_f32(x + t * k, wr, k, isa);
            out[t * n + (size_t)r] = bias ? s + bias[r] : s;
        }
    }
}

__attribute__((target("avx2,fma"))) static float dot_i8w_f32_avx2(const int8_t *w, const float *x, size_t k)
{
    __m256 acc = _mm256_setzero_ps();
    size_t i = 0;
    for (; i + 8 <= k; i += 8) {
        __m128i b = _mm_loadl_epi64((const __m128i *)(w + i));
        __m256 wf = _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(b));
        acc = _mm256_fmadd_ps(wf, _mm256_loadu_ps(x + i), acc);
    }
    __m128 lo = _mm_add_ps(_mm256_castps256_ps128(acc), _mm256_extractf128_ps(acc, 1));
    lo = _mm_hadd_ps(lo, lo);
    lo = _mm_hadd_ps(lo, lo);
    float s = _mm_cvtss_f32(lo);
    for (; i < k; ++i) s += (float)w[i] * x[i];
    return s;
}

__attribute__((target("avx512f"))) static float dot_i8w_f32_avx512(const int8_t *w, const float *x, size_t k)
{
    __m512 acc = _mm512_setzero_ps();
    size_t i = 0;
    for (; i + 16 <= k; i += 16) {
        __m128i b = _mm_loadu_si128((const __m128i *)(w + i));
        __m512 wf = _mm512_cvtepi32_ps(_mm512_cvtepi8_epi32(b));
        acc = _mm512_fmadd_ps(wf, _mm512_loadu_ps(x + i), acc);
    }
    float s = _mm512_reduce_add_ps(acc);
    for (; i < k; ++i) s += (float)w[i] * x[i];
    return s;
}

/* q [n,k] ternary i8, x [m,k] f32, y [m,n] f32 */
void cpu_ref_simd_gemv(const int8_t *q, const float *x, float *y, float scale, size_t m, size_t n, size_t k)
{
    int isa = cpu_baseline_isa();
#pragma omp parallel for schedule(static)
    for (long long r = 0; r < (long long)n; ++r) {
        const int8_t *qr = q + (size_t)r * k;
        for (size_t t = 0; t < m; ++t) {
            const float *xt = x + t * k;
            float s;
            if (isa == 2) s = dot_i8w_f32_avx512(qr, xt, k);
            else if (isa == 1) s = dot_i8w_f32_avx2(qr, xt, k);
            else { s = 0.0f; for (size_t i = 0; i < k; ++i) s += (float)qr[i] * xt[i]; }
            y[t * n + (size_t)r] = s * scale;
        }
    }
}
