// FakeQuantize load-time checks shared with the convolution epilogue planner.
#pragma once
#include <array>
#include <map>
#include <memory>
#include <vector>

#include "common.h"
#include "fq_math.h"

namespace hipie {

// True when the reciprocal evaluation of the level index equals the dividing one on both sides
// of every level boundary of this channel (both are monotone step functions of x, so agreement
// around every step of the reference means agreement everywhere between il and ih).
bool fq_reciprocal_exact_on_boundaries(const FqChannel& p, float lm1);

// The same for n channels at once: one check per distinct (il, ih, d, r), spread over the host's threads.
// Returns true when every channel passes.
bool fq_reciprocal_exact_on_all(const FqChannel* p, int64_t n, float lm1);

// r = correctly rounded 1/d
float fq_rounded_reciprocal(float d);

// What the load-time checks found, keyed by the bits of their inputs: whether the reciprocal path gives the
// reference's level on every boundary, and the two-operation division constants of a divisor (or that it has none).
// Both are pure functions of their keys, so a table filled while one plan was built answers the same questions when
// an exported plan is loaded again, without running the checks.  A thread that wants its checks recorded, or answered
// from a table, installs one for a scope; the checks consult the calling thread's table only.
struct FqVerdicts {
    struct Div2 { float zh, zl; uint32_t ok; };
    std::map<std::array<uint32_t, 5>, uint32_t> rcp;   // il, ih, d, r, levels - 1  ->  1 exact / 0 not
    std::map<uint32_t, Div2> div2;                     // d  ->  verified pair, or ok = 0
    struct Scope {
        explicit Scope(FqVerdicts* v);
        ~Scope();
        Scope(const Scope&) = delete;
        Scope& operator=(const Scope&) = delete;
        FqVerdicts* previous;
    };
    static FqVerdicts* current();
};

// Elementwise nodes that no convolution / pooling / MatMul chain absorbs, on NHWC operands:
//     out = FakeQuantize?( act?( op(a, b) ) ),  op in {none (unary), Add, Subtract, Multiply, PRelu}, a and b in graph order.
// An operand is a per-channel constant, an f32 tensor, or a byte tensor behind its dequantization
// (float(level) - sub[c]) * mul[c].  Reference: reference::add / subtract / multiply (autobroadcast_binop.hpp), prelu.hpp, relu.hpp,
// clamp.hpp, fake_quantize.hpp:175-194, each step one f32 operation as in the graph.
struct EltOperand {
    const void* p = nullptr;          // tensor element (0, 0, 0, 0); null when the operand is `konst`
    int32_t dtype = 0;                // HIPIE_F32, HIPIE_U8B or HIPIE_I8
    int64_t sn = 0, sh = 0, sw = 0;   // element strides
    const float* sub = nullptr;       // per channel, padded to a multiple of 4, or null
    const float* mul = nullptr;
    const float* konst = nullptr;     // per-channel constant operand, padded to a multiple of 4
};
struct EltArgs {
    EltOperand a, b;
    int32_t op = 0;                   // 0 none, 1 add, 2 subtract, 3 multiply, 4 prelu (a < 0 ? a * b : a)
    int32_t act = 0;                  // 0 none, 1 relu, 2 clamp(lo, hi), 3 sigmoid, 4 hswish, 5 hsigmoid, 6 swish(beta = lo)
    float lo = 0, hi = 0;
    void* out = nullptr;
    int32_t out_dtype = HIPIE_F32;    // HIPIE_F32, or HIPIE_U8B / HIPIE_I8 behind a FakeQuantize
    int64_t out_sn = 0, out_sh = 0, out_sw = 0;
    int32_t N = 0, H = 0, W = 0, C = 0;
    int32_t device = 0;               // where the tensors live (an f32 result has no FakeQuantize object to tell)
};
}  // namespace hipie
struct hipie_fq;
namespace hipie {
// `fq` (null for an f32 result) must give integer levels (hipie_fq_create's q8 form); fq_gives_levels says whether it does
bool fq_gives_levels(const hipie_fq* fq);
void run_eltwise(const hipie_fq* fq, const EltArgs& a, hipStream_t s);

}  // namespace hipie
