// GELU (ERF mode) in single precision, shared by the stand-alone kernel and the GEMM epilogue so that
// both produce the same float for the same input.  Must be compiled with floating-point contraction off.
#pragma once
#include <hip/hip_runtime.h>

namespace hipie {

// 0.5 x (1 + erf(x / sqrt 2)) = x Phi(x) with Phi from erfc(|x| / sqrt 2): no cancellation for negative x, so
// single precision stays within 1e-6 relative (+ 1e-8 absolute) of the reference's double evaluation over
// the whole range (measured against it on 18.9 M points in [-9, 9]: worst case 0.61 of that bound, at
// x = -2.17).  erfc(z), z >= 0, is the Chebyshev fit t exp(-z^2 + P9(t)), t = 1 / (1 + z / 2), of
// Numerical Recipes (erfcc; fractional error below 1.2e-7 everywhere): a reciprocal, nine FMAs and one
// hardware exp2 instead of the library erfc's three dozen instructions, which made the kernel
// compute-bound (double-precision erf: 63 us for [6144, 3072]; library erfcf: 29 us; this: 25 us, the
// HBM time of its 151 MB).
__device__ __forceinline__ float gelu_one(float x) {
    const float z = fabsf(x) * 0.70710678118654752f;
    const float t = 1.0f / (1.0f + 0.5f * z);
    float p = 0.17087277f;
    p = fmaf(p, t, -0.82215223f);
    p = fmaf(p, t, 1.48851587f);
    p = fmaf(p, t, -1.13520398f);
    p = fmaf(p, t, 0.27886807f);
    p = fmaf(p, t, -0.18628806f);
    p = fmaf(p, t, 0.09678418f);
    p = fmaf(p, t, 0.37409196f);
    p = fmaf(p, t, 1.00002368f);
    p = fmaf(p, t, -1.26551223f);
    const float e = t * __expf(fmaf(-z, z, p));           // erfc(|x| / sqrt 2)
    return x * (x < 0.f ? 0.5f * e : 1.0f - 0.5f * e);
}

}  // namespace hipie
