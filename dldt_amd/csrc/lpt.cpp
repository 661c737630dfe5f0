// Load-time arithmetic of the low-precision transformations, restated so that a harness without
// OpenVINO can derive the same constants stock LPT leaves in the Function (u8/i8 levels, scales,
// zero points, folded i8 weights).  Pure float math on host arrays; no graph rewriting.
// Reference: inference-engine/src/low_precision_transformations/src/
//   layer_transformation.cpp:194-273 (getPrecisionDetails),
//   include/low_precision/layer_transformation.hpp:63-107 (DataPrecision::getMin/MaxValue),
//   network_helper.cpp:943-1087 (decomposeFakeQuantize), :700-827 (foldFakeQuantize), :216-292 (swapMultiplyAndAdd),
//   fake_quantize.cpp:127-183 (fuseElementwise), add.cpp:154-218 (AddTransformation), clamp.cpp:71-89.
#include <algorithm>
#include <cmath>
#include <limits>

#include "common.h"

using namespace hipie;

namespace {

// What one output interval [lo, hi] of a FakeQuantize asks of the integer type that will hold its levels
// (the per-interval decisions of getPrecisionDetails, layer_transformation.cpp:207-243).
enum IntervalKind { kUnsigned, kUnsignedWithZeroPoint, kSigned, kSignedWithZeroPoint };

IntervalKind classify_interval(float lo, float hi, int64_t levels) {
    const bool crosses_zero = std::signbit(lo) != std::signbit(hi);
    const bool lo_is_off_zero = std::fabs(lo) >= 1.e-6f;
    if (!(crosses_zero && lo_is_off_zero)) return lo_is_off_zero ? kUnsignedWithZeroPoint : kUnsigned;
    if (hi == 0.f) return kSignedWithZeroPoint;
    // a signed interval needs no zero point when lo / hi is the ratio of the type's own ends (-128 / 127, or -1 for
    // 255 levels) within 0.2 %
    const float want = levels == 256 ? -128.f / 127.f : -1.f;
    const float have = lo / hi;
    const float off = std::fabs((have - want) / std::min(have, want));
    return off > 0.002f ? kSignedWithZeroPoint : kSigned;
}

}  // namespace

extern "C" {

/* getPrecisionDetails: *precision = HIPIE_U8 / HIPIE_I8 / 0 (undefined) */
int hipie_lpt_precision_details(int64_t levels, const float* out_low, const float* out_high, int64_t n,
                                int* precision, int* has_negative, int* has_zero_point) {
    return guarded([&] {
        HIPIE_REQUIRE(out_low && out_high && precision && has_negative && has_zero_point && n > 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_lpt_precision_details: bad argument");
        int seen[4] = {0, 0, 0, 0};
        for (int64_t i = 0; i < n; ++i) ++seen[classify_interval(out_low[i], out_high[i], levels)];
        const bool any_signed = seen[kSigned] + seen[kSignedWithZeroPoint] > 0;
        const bool any_unsigned = seen[kUnsigned] + seen[kUnsignedWithZeroPoint] > 0;
        const bool zero_point = seen[kUnsignedWithZeroPoint] + seen[kSignedWithZeroPoint] > 0;
        // one integer type for all intervals, and only if none of them needs a zero point
        *precision = zero_point || any_signed == any_unsigned ? 0 : (any_signed ? HIPIE_I8 : HIPIE_U8);
        *has_negative = any_signed;
        *has_zero_point = zero_point;
    });
}

/* DataPrecision::getMinValue / getMaxValue for u8 / i8 at 255 or 256 levels */
int hipie_lpt_data_precision_range(int precision, int64_t levels, float* min, float* max) {
    return guarded([&] {
        HIPIE_REQUIRE(min && max, HIPIE_PARAMETER_MISMATCH, "hipie_lpt_data_precision_range: null argument");
        HIPIE_REQUIRE(levels == 255 || levels == 256, HIPIE_PARAMETER_MISMATCH, "unexpected levels %lld",
                      (long long)levels);
        if (precision == HIPIE_I8) {
            *min = levels == 255 ? -127.f : -128.f;
            *max = 127.f;
        } else if (precision == HIPIE_U8) {
            *min = 0.f;
            *max = 255.f - static_cast<float>(256 - levels);
        } else {
            fail(HIPIE_PARAMETER_MISMATCH, "unexpected precision %d", precision);
        }
    });
}

/* decomposeFakeQuantize: per output-range element i, the dequantization scale and shift that
 * follow a FakeQuantize re-targeted to [min, max]; new_low/new_high are that FQ's output range. */
int hipie_lpt_decompose_fake_quantize(const float* out_low, const float* out_high, int64_t n, float min,
                                      float max, float* scales, float* shifts, float* new_low,
                                      float* new_high) {
    return guarded([&] {
        HIPIE_REQUIRE(out_low && out_high && scales && shifts && new_low && new_high && n > 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_lpt_decompose_fake_quantize: bad argument");
        for (int64_t i = 0; i < n; ++i) {
            new_low[i] = min;
            new_high[i] = max;
            shifts[i] = 0.f;
            if (out_high[i] != out_low[i]) {
                shifts[i] = (min * out_high[i] - max * out_low[i]) / (out_high[i] - out_low[i]);
                scales[i] = (out_high[i] - out_low[i]) / (max - min);
                if (shifts[i] == -0.f) shifts[i] = 0.f;
            } else {
                scales[i] = out_high[i];
                new_low[i] = 1.f;
                new_high[i] = 1.f;
            }
            // scale clamp of network_helper.cpp:1000-1021
            const float lo = 1e-32f, hi = 1e32f;
            if (std::fabs(scales[i]) < lo) scales[i] = lo;
            else if (std::fabs(scales[i]) > hi) scales[i] = scales[i] > 0.f ? hi : -hi;
        }
    });
}

/* foldFakeQuantize on a constant [OC, inner] (outChannelsShapeIndex == 0): bounds have 1 or OC
 * values; round_values applies std::roundf to the result as for integral output types. */
int hipie_lpt_fold_fake_quantize(const float* values, int64_t oc, int64_t inner, const float* in_low,
                                 int64_t n_il, const float* in_high, int64_t n_ih, const float* out_low,
                                 int64_t n_ol, const float* out_high, int64_t n_oh, int64_t levels,
                                 int round_values, float* out) {
    return guarded([&] {
        HIPIE_REQUIRE(values && in_low && in_high && out_low && out_high && out, HIPIE_PARAMETER_MISMATCH,
                      "hipie_lpt_fold_fake_quantize: null argument");
        for (int64_t n : {n_il, n_ih, n_ol, n_oh})
            HIPIE_REQUIRE(n == 1 || n == oc, HIPIE_PARAMETER_MISMATCH, "unexpected bound count %lld for %lld channels",
                          (long long)n, (long long)oc);
        // shortcut of network_helper.cpp:705-731
        if (n_il == 1 && n_ih == 1 && n_ol == 1 && n_oh == 1 && in_low[0] == 0.f && in_high[0] == 254.f &&
            out_low[0] == -127.f && out_high[0] == 127.f) {
            for (int64_t i = 0; i < oc * inner; ++i) out[i] = values[i] + out_low[0];
            return;
        }
        const float levels_1 = static_cast<float>(levels) - 1.f;
        for (int64_t c = 0; c < oc; ++c) {
            const float il = in_low[n_il == 1 ? 0 : c], ih = in_high[n_ih == 1 ? 0 : c];
            const float ol = out_low[n_ol == 1 ? 0 : c], oh = out_high[n_oh == 1 ? 0 : c];
            for (int64_t i = 0; i < inner; ++i) {
                const float v = values[c * inner + i];
                float q;
                if (v <= il) q = round_values ? std::roundf(ol) : ol;
                else if (v > ih) q = round_values ? std::roundf(oh) : oh;
                else {
                    const float value = std::roundf((v - il) / (ih - il) * levels_1) / levels_1 * (oh - ol) + ol;
                    q = round_values ? std::roundf(value) : value;
                }
                out[c * inner + i] = q;
            }
        }
    });
}

/* NetworkHelper::swapMultiplyAndAdd (network_helper.cpp:216-292): x * a + b  ==>  (x + b / a) * a.  out[i] = b[i] / a[i]
 * with 1 or n values on either side, and 0 where both are 0 (the reference's guard against NaN). */
int hipie_lpt_swap_multiply_and_add(const float* b, int64_t n_b, const float* a, int64_t n_a, float* out, int64_t n) {
    return guarded([&] {
        HIPIE_REQUIRE(b && a && out && n > 0 && (n_b == 1 || n_b == n) && (n_a == 1 || n_a == n), HIPIE_PARAMETER_MISMATCH,
                      "hipie_lpt_swap_multiply_and_add: %lld and %lld values for %lld", (long long)n_b, (long long)n_a, (long long)n);
        for (int64_t i = 0; i < n; ++i) {
            const float bi = b[n_b == 1 ? 0 : i], ai = a[n_a == 1 ? 0 : i];
            out[i] = (bi != 0.f || ai != 0.f) ? bi / ai : 0.f;
        }
    });
}

/* FakeQuantizeTransformation::fuseElementwise (fake_quantize.cpp:127-183): the elementwise operation with a constant
 * in front of a FakeQuantize moves into its input range.  kind: HIPIE_LPT_MULTIPLY (range / value; not fused -
 * *fused = 0, range unchanged - when a value is <= 0 or a quotient is infinite), HIPIE_LPT_SUBTRACT (range + value),
 * HIPIE_LPT_ADD (range - value).  1 or n values on either side. */
int hipie_lpt_fuse_elementwise(int kind, const float* in_low, const float* in_high, int64_t n_range, const float* value,
                               int64_t n_value, float* new_low, float* new_high, int64_t n, int* fused) {
    return guarded([&] {
        HIPIE_REQUIRE(in_low && in_high && value && new_low && new_high && fused && n > 0 && (n_range == 1 || n_range == n) &&
                          (n_value == 1 || n_value == n),
                      HIPIE_PARAMETER_MISMATCH, "hipie_lpt_fuse_elementwise: bad argument");
        HIPIE_REQUIRE(kind >= HIPIE_LPT_MULTIPLY && kind <= HIPIE_LPT_ADD, HIPIE_PARAMETER_MISMATCH,
                      "hipie_lpt_fuse_elementwise: kind %d", kind);
        *fused = 1;
        for (int64_t i = 0; i < n; ++i) {
            const float lo = in_low[n_range == 1 ? 0 : i], hi = in_high[n_range == 1 ? 0 : i], v = value[n_value == 1 ? 0 : i];
            if (kind == HIPIE_LPT_MULTIPLY) {
                new_low[i] = lo / v;
                new_high[i] = hi / v;
                if (v <= 0.f || std::isinf(new_low[i]) || std::isinf(new_high[i])) *fused = 0;
            } else if (kind == HIPIE_LPT_SUBTRACT) {
                new_low[i] = lo + v;
                new_high[i] = hi + v;
            } else {
                new_low[i] = lo - v;
                new_high[i] = hi - v;
            }
        }
        if (!*fused)
            for (int64_t i = 0; i < n; ++i) {
                new_low[i] = in_low[n_range == 1 ? 0 : i];
                new_high[i] = in_high[n_range == 1 ? 0 : i];
            }
    });
}

/* AddTransformation with dequantizations on both branches (add.cpp:154-218):
 *   SC_full (X1 - SH_full) + SC_empty (X2 - SH_empty)  ==>  SC_empty ( SC' (X1 - SH') + X2 ),
 *   SC' = SC_full / SC_empty,  SH' = SH_full + SC_empty SH_empty / SC_full  (the comment at :178-182);
 * scale_after = SC_empty.  A missing Subtract is shift 0, a missing Multiply scale 1. */
int hipie_lpt_add_both_branches(const float* shift_full, const float* scale_full, const float* shift_empty,
                                const float* scale_empty, int64_t n, float* new_shift_full, float* new_scale_full,
                                float* scale_after) {
    return guarded([&] {
        HIPIE_REQUIRE(shift_full && scale_full && shift_empty && scale_empty && new_shift_full && new_scale_full && scale_after && n > 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_lpt_add_both_branches: bad argument");
        for (int64_t i = 0; i < n; ++i) {
            new_shift_full[i] = shift_full[i] + (shift_empty[i] * scale_empty[i]) / scale_full[i];
            new_scale_full[i] = scale_full[i] / scale_empty[i];
            scale_after[i] = scale_empty[i];
        }
    });
}

/* ClampTransformation (clamp.cpp:71-89): the bounds of a Clamp that moves in front of a per-tensor dequantization
 * (x - shift) * scale: divided by the scale (swapped first when it is negative), then the shift added; evaluated
 * in double as the reference does. */
int hipie_lpt_clamp_bounds(double min, double max, double scale, double shift, double* new_min, double* new_max) {
    return guarded([&] {
        HIPIE_REQUIRE(new_min && new_max && scale != 0.0, HIPIE_PARAMETER_MISMATCH, "hipie_lpt_clamp_bounds: bad argument");
        if (scale < 0.0) std::swap(min, max);
        *new_min = min / scale + shift;
        *new_max = max / scale + shift;
    });
}

}  // extern "C"
