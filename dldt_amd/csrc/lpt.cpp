// Load-time arithmetic of the low-precision transformations, restated so that a harness without
// OpenVINO can derive the same constants stock LPT leaves in the Function (u8/i8 levels, scales,
// zero points, folded i8 weights).  Pure float math on host arrays; no graph rewriting.
// Reference: inference-engine/src/low_precision_transformations/src/
//   layer_transformation.cpp:194-273 (getPrecisionDetails),
//   include/low_precision/layer_transformation.hpp:63-107 (DataPrecision::getMin/MaxValue),
//   network_helper.cpp:943-1087 (decomposeFakeQuantize), :700-827 (foldFakeQuantize).
#include <cmath>
#include <limits>

#include "common.h"

using namespace hipie;

extern "C" {

/* getPrecisionDetails: *precision = HIPIE_U8 / HIPIE_I8 / 0 (undefined) */
int hipie_lpt_precision_details(int64_t levels, const float* out_low, const float* out_high, int64_t n,
                                int* precision, int* has_negative, int* has_zero_point) {
    return guarded([&] {
        HIPIE_REQUIRE(out_low && out_high && precision && has_negative && has_zero_point && n > 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_lpt_precision_details: bad argument");
        const float zeroThreshold = 1.e-6f;
        const float asymmetryThreshold = 0.002f;
        const float ratio256 = -128.f / 127.f;
        bool hasNegative = false, signedPrecision = true, unsignedPrecision = true, hasZeroPoint = false;
        for (int64_t i = 0; i < n; ++i) {
            const bool signedInterval = std::signbit(out_low[i]) != std::signbit(out_high[i]);
            const bool lowIsNotZero = std::fabs(out_low[i]) >= zeroThreshold;
            if (signedInterval && lowIsNotZero) {
                unsignedPrecision = false;
                hasNegative = true;
                if (out_high[i] != 0.f) {
                    const float expectedRatio = levels == 256 ? ratio256 : -1.f;
                    const float actualRatio = out_low[i] / out_high[i];
                    const float actual = std::fabs((actualRatio - expectedRatio) / std::min(actualRatio, expectedRatio));
                    if (actual > asymmetryThreshold) hasZeroPoint = true;
                } else {
                    hasZeroPoint = true;
                }
            } else {
                signedPrecision = false;
                if (lowIsNotZero) hasZeroPoint = lowIsNotZero;
            }
        }
        *precision = 0;
        if (!hasZeroPoint) {
            if (signedPrecision && !unsignedPrecision) *precision = HIPIE_I8;
            if (!signedPrecision && unsignedPrecision) *precision = HIPIE_U8;
        }
        *has_negative = hasNegative;
        *has_zero_point = hasZeroPoint;
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

}  // extern "C"
