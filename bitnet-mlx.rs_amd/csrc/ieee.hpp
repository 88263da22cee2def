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
}  // namespace bitnet
