// Correctly rounded division by a per-channel constant in two operations.
//
// For a fixed divisor d and constants zh = RN(1/d), zl ~ RN(1/d - zh), the value
// fma(n, zh, RN(n * zl)) equals RN(n / d) for every float n except, for some d, a handful of n whose
// quotient lies within 2^-47 of a rounding boundary (Brisebarre, Muller, Raina, "Accelerating
// correctly rounded floating-point division when the divisor is known in advance", IEEE TC 2004).
// Instead of classifying divisors we test each (d, zh, zl) against the hardware's IEEE division
// on all 2^23 significands of n at load time: both sides scale exactly with powers of two, so one
// binade covers every n whose products stay normal, and n small enough to underflow them
// (n / d < 2^-100) quantizes to the lowest level on either path.  Divisors that fail are retried
// with zl moved by a few units in the last place; the caller keeps the slower sequence if one
// channel cannot be matched.
#pragma once
#include <vector>

namespace hipie {

// zh, zl sized like d.  Returns true when every channel has a verified pair.  device < 0: no
// verification is possible, returns false.
bool fq_div2_constants(int device, const std::vector<float>& d, std::vector<float>& zh, std::vector<float>& zl);

}  // namespace hipie
