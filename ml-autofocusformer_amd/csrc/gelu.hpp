// The exact (erf) GELU as the kernels of this library evaluate it.
#pragma once

#include "common.hpp"

namespace clusten {

// GELU(v) = v * Phi(v) with Phi(v) = erfc(-v / sqrt 2) / 2, and erfc(z) for z >= 0 as t * exp(-z^2 + P(t)), t = 1 / (1 + z/2),
// P a degree-9 polynomial: the classic Chebyshev fit whose fractional error stays below 1.2e-7 for every z.  No
// branches (eight of these interleave in the epilogue), and since it is erfc that is approximated to a relative
// bound the negative tail keeps its accuracy, which 0.5 * v * (1 + erf(v / sqrt 2)) loses to cancellation there:
// rounded to fp16 the result equals the exactly rounded GELU for all but a handful of the 63488 finite fp16 inputs
// (1 ulp), and differs from the erf formula only where that one is off (v < -2.5, by up to 6 ulp of values below
// 2e-4 in magnitude).
__device__ __forceinline__ float gelu_erf(float v) {
    const float z = fabsf(v) * 0.70710678118654752440f;
    const float t = __builtin_amdgcn_rcpf(1.f + 0.5f * z);
    float p = 0.17087277f;
    p = p * t - 0.82215223f;
    p = p * t + 1.48851587f;
    p = p * t - 1.13520398f;
    p = p * t + 0.27886807f;
    p = p * t - 0.18628806f;
    p = p * t + 0.09678418f;
    p = p * t + 0.37409196f;
    p = p * t + 1.00002368f;
    p = p * t - 1.26551223f;
    const float half_erfc = 0.5f * t * __expf(p - z * z);
    return v * (v < 0.f ? half_erfc : 1.f - half_erfc);
}

}  // namespace clusten
