// Per-tensor FakeQuantize to i8 levels evaluated inside the kernel that produces its input (the
// transformer glue kernels and the attention kernel).
#pragma once
#include "common.h"
#include "fq.h"

namespace hipie {

// The level index of the reference's expression (fake_quantize.hpp:175-194) by IEEE division, or by
// the reciprocal sequence when that was proven to give the same index on both sides of every level
// boundary; stored as out_low + k.  levels == 0: no quantized output.
struct Requant {
    FqChannel p;
    float lm1;
    int levels;
    int rcp;   // the reciprocal evaluation was proven equal to the division on every level boundary
};

__device__ __forceinline__ int requant_level(const Requant& f, float x) {
    // x <= il -> level 0, x > ih -> level L - 1 through the clamp
    const float k = f.rcp ? fq_level_clamped<true>(f.p, f.lm1, x) : fq_level_clamped<false>(f.p, f.lm1, x);
    return static_cast<int>(k + f.p.ol);
}

__device__ __forceinline__ uint32_t requant4(const Requant& f, const float4& v) {
    return (static_cast<uint32_t>(requant_level(f, v.x)) & 0xffu) | ((static_cast<uint32_t>(requant_level(f, v.y)) & 0xffu) << 8) |
           ((static_cast<uint32_t>(requant_level(f, v.z)) & 0xffu) << 16) | (static_cast<uint32_t>(requant_level(f, v.w)) << 24);
}

// Host side: checks that the reference's output expression yields the integers out_low + k and picks
// the evaluation of the level index.
inline Requant make_requant(const hipie_requant* r, const char* what) {
    Requant f{};
    if (!r) return f;
    HIPIE_REQUIRE(r->levels >= 2 && r->levels <= 256 && r->in_low < r->in_high, HIPIE_PARAMETER_MISMATCH,
                  "%s: requantisation needs 2..256 levels and in_low < in_high", what);
    f.p.il = f.p.lo = r->in_low;
    f.p.ih = f.p.hi = r->in_high;
    f.p.d = r->in_high - r->in_low;
    f.p.r = fq_rounded_reciprocal(f.p.d);
    f.lm1 = static_cast<float>(r->levels - 1);
    f.p.ol = r->out_low;
    f.p.oh = r->out_low + f.lm1;
    f.levels = static_cast<int>(r->levels);
    f.rcp = fq_reciprocal_exact_on_boundaries(f.p, f.lm1) ? 1 : 0;
    const float oh = f.p.oh;
    HIPIE_REQUIRE(f.p.ol == std::nearbyintf(f.p.ol) && f.p.ol >= -128.f && oh <= 127.f, HIPIE_NOT_IMPLEMENTED,
                  "%s: output levels must be the i8 integers out_low .. out_low + levels - 1", what);
    for (int k = 0; k < f.levels; ++k)   // the reference's own output expression yields these integers
        HIPIE_REQUIRE(static_cast<float>(k) / f.lm1 * (oh - f.p.ol) + f.p.ol == f.p.ol + static_cast<float>(k),
                      HIPIE_NOT_IMPLEMENTED, "%s: output level %d is not an integer", what, k);
    return f;
}

}  // namespace hipie
