/* Exhaustive check of the rounding identity the HIP quantiser (csrc/rowquant.hpp, quant1) relies on:
 *
 *     clamp(sat_i32(roundf(t)), -128, 127)  ==  clamp(sat_i32(trunc(t + copysign(0.5 - 2^-25, t))), -128, 127)
 *
 * for every one of the 2^32 float bit patterns t, with one IEEE round-to-nearest-even addition on the right.  The left
 * side is the reference's activation quantiser (round half away from zero, clamp, cast:
 * bitnet-inference/src/engine/ternary_operations.rs:158-161, restated as orc_q8 in oracle/bitlinear_oracle.c); the right side is what the
 * kernel computes with v_add_f32 and v_cvt_i32_f32.  Prints the number of mismatches; exit status 0 if there are none.
 * Build: gcc -O2 -fopenmp -fno-fast-math rounding_identity_check.c -lm */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static inline int sat_i32(float f)
{
    if (f != f) return 0;
    if (f >= 2147483648.0f) return 2147483647;
    if (f <= -2147483648.0f) return -2147483647 - 1;
    return (int)f;
}
static inline int clamp8(int q) { return q < -128 ? -128 : (q > 127 ? 127 : q); }

int main(void)
{
    long long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (long long b = 0; b < (1LL << 32); ++b) {
        uint32_t u = (uint32_t)b;
        float t;
        memcpy(&t, &u, 4);
        const int ref = clamp8(sat_i32(roundf(t)));
        volatile float s = t + copysignf(0x1.fffffep-2f, t); /* volatile: exactly one f32 addition, no contraction or widening */
        const int got = clamp8(sat_i32(truncf(s)));
        if (got != ref) {
            if (bad < 5) printf("mismatch at %08x: t = %a, reference %d, identity %d\n", u, t, ref, got);
            ++bad;
        }
    }
    printf("mismatches: %lld\n", bad);
    return bad != 0;
}
