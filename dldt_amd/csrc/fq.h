// FakeQuantize load-time checks shared with the convolution epilogue planner.
#pragma once
#include <memory>

#include "common.h"
#include "fq_math.h"

namespace hipie {

// True when the reciprocal evaluation of the level index equals the dividing one on both sides
// of every level boundary of this channel (both are monotone step functions of x, so agreement
// around every step of the reference means agreement everywhere between il and ih).
bool fq_reciprocal_exact_on_boundaries(const FqChannel& p, float lm1);

// r = correctly rounded 1/d
float fq_rounded_reciprocal(float d);

}  // namespace hipie
