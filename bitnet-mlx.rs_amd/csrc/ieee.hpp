// Single-operation IEEE-754 binary32 arithmetic for device code.
//
// The quantiser must reproduce CPU arithmetic bit for bit, so every f32 step has to be exactly one
// correctly rounded operation.  Plain C operators give that under two conditions this build enforces:
// contraction is off (-ffp-contract=off on the command line and the pragma below, so a*b+c is never
// fused) and division / square root are the correctly rounded forms
// (-fhip-fp32-correctly-rounded-divide-sqrt, the compiler's default, named explicitly in the Makefile).
// HIP's __fsqrt_rn is NOT used: without OCML_BASIC_ROUNDED_OPERATIONS it maps to the approximate
// hardware square root.
#pragma once
#include <hip/hip_runtime.h>

#pragma clang fp contract(off)

namespace bitnet {
__device__ __forceinline__ float f32_add(float a, float b) { return a + b; }
__device__ __forceinline__ float f32_mul(float a, float b) { return a * b; }
__device__ __forceinline__ float f32_div(float a, float b) { return a / b; }
__device__ __forceinline__ float f32_sqrt(float a) { return __builtin_sqrtf(a); }

// x / d for a positive divisor d shared by many dividends.  recip must be the correctly rounded 1/d (one IEEE
// division).  q0 = RN(x*recip) is within one ulp of x/d; the remainder x - d*q0 is then exact in one FMA and
// the corrected quotient RN(q0 + rem*recip) is the correctly rounded x/d (Markstein's division step).  The
// theorem excludes divisors whose significand is all ones and needs the intermediate values to stay normal:
// invariant_divisor_ok(d) is tested once per divisor, dividend_ok(x) per dividend (zero is fine, tiny, huge
// and non-finite values are not); where either fails the caller uses the plain division.  Three operations
// per element instead of the full IEEE sequence, same bits.
__device__ __forceinline__ bool invariant_divisor_ok(float d)
{
    const unsigned bits = __builtin_bit_cast(unsigned, d);
    const unsigned expo = (bits >> 23) & 0xffu;
    return (bits >> 31) == 0u && (bits & 0x7fffffu) != 0x7fffffu && expo > 64u && expo < 190u;
}
__device__ __forceinline__ bool dividend_ok(float x)
{
    const unsigned mag = __builtin_bit_cast(unsigned, x) & 0x7fffffffu;
    return mag == 0u || (mag >= (64u << 23) && mag < (190u << 23));  // 0, or 2^-63 <= |x| < 2^63
}
__device__ __forceinline__ float div_by_invariant_unchecked(float x, float d, float recip)
{
    const float q0 = x * recip;
    const float rem = __builtin_fmaf(-q0, d, x);
    return __builtin_copysignf(__builtin_fmaf(rem, recip, q0), x);  // d > 0: the quotient has x's sign (also for -0)
}
}  // namespace bitnet
