// FakeQuantize arithmetic shared by the device kernels and the host-side planner checks.
// Reference expression: ngraph/core/reference/.../fake_quantize.hpp:175-194.
//
// The level index k = nearbyint((x - il) / (ih - il) * (L - 1)) is the only rounding-sensitive
// part.  Two evaluations are provided:
//   fq_level_div : IEEE division, the literal reference order;
//   fq_level_rcp : n * r with two FMA residual corrections (r = correctly rounded 1/d).  The
//                  second correction starts from a quotient within one ulp, so the result is the
//                  correctly rounded quotient (Markstein's division-by-FMA argument), i.e. the
//                  same float as IEEE division, at 5 instead of ~12 VALU instructions.
// This file must be compiled with floating-point contraction off.
#pragma once
#include <math.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define HIPIE_HD __host__ __device__ __forceinline__
#else
#define HIPIE_HD inline
#endif

namespace hipie {

struct FqChannel {   // 32 bytes, one per channel
    float il, ih;    // input_low / input_high as given
    float ol, oh;    // output_low / output_high as given
    float lo, hi;    // min(il, ih), max(il, ih)
    float d;         // fl(ih - il)
    float r;         // correctly rounded 1 / d (reciprocal path only)
};

HIPIE_HD float fq_level_div(const FqChannel& p, float lm1, float x) {
    return rintf((x - p.il) / p.d * lm1);
}

HIPIE_HD float fq_level_rcp(const FqChannel& p, float lm1, float x) {
    const float n = x - p.il;
    const float q0 = n * p.r;
    const float e0 = fmaf(-p.d, q0, n);
    const float q1 = fmaf(e0, p.r, q0);
    const float e1 = fmaf(-p.d, q1, n);
    const float q = fmaf(e1, p.r, q1);
    return rintf(q * lm1);
}

// level index with the saturating branches folded in; valid when il < ih
template <bool RCP>
HIPIE_HD float fq_level_clamped(const FqChannel& p, float lm1, float x) {
    // x <= il -> n = 0 -> k = 0;  x > ih -> n = d -> q = 1 -> k = L - 1
    const float xc = fminf(fmaxf(x, p.il), p.ih);
    return RCP ? fq_level_rcp(p, lm1, xc) : fq_level_div(p, lm1, xc);
}

// the op's f32 result, any bounds
template <bool RCP>
HIPIE_HD float fq_value(const FqChannel& p, float lm1, float x) {
    if (x <= p.lo) return p.ol;
    if (x > p.hi) return p.oh;
    const float k = RCP ? fq_level_rcp(p, lm1, x) : fq_level_div(p, lm1, x);
    return k / lm1 * (p.oh - p.ol) + p.ol;
}

}  // namespace hipie
