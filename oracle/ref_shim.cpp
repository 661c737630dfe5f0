// TEST INFRASTRUCTURE ONLY.  Thin extern "C" shim over the reference's own header-template
// kernels (ngraph/core/reference), compiled in place from the reference checkout into
// oracle/_ref/libngraph_ref.so by oracle/Makefile.  No reference source is copied: the headers
// are found through -I paths.  Exports mirror the orc_* functions of ngraph_ops.c one to one so
// tests can fuzz the restatement against the real thing.
#include <cstdint>
#include <vector>

#include "ngraph/runtime/reference/add.hpp"
#include "ngraph/runtime/reference/avg_pool.hpp"
#include "ngraph/runtime/reference/clamp.hpp"
#include "ngraph/runtime/reference/convolution.hpp"
#include "ngraph/runtime/reference/divide.hpp"
#include "ngraph/runtime/reference/fake_quantize.hpp"
#include "ngraph/runtime/reference/gelu.hpp"
#include "ngraph/runtime/reference/group_convolution.hpp"
#include "ngraph/runtime/reference/matmul.hpp"
#include "ngraph/runtime/reference/max_pool.hpp"
#include "ngraph/runtime/reference/multiply.hpp"
#include "ngraph/runtime/reference/mvn.hpp"
#include "ngraph/runtime/reference/hsigmoid.hpp"
#include "ngraph/runtime/reference/hswish.hpp"
#include "ngraph/runtime/reference/prelu.hpp"
#include "ngraph/runtime/reference/sigmoid.hpp"
#include "ngraph/runtime/reference/swish.hpp"
#include "ngraph/runtime/reference/relu.hpp"
#include "ngraph/runtime/reference/softmax.hpp"
#include "ngraph/runtime/reference/subtract.hpp"

using namespace ngraph;
namespace ref = ngraph::runtime::reference;

static Shape mk_shape(const int64_t* s, int r) { return Shape(s, s + r); }

template <typename T>
static void conv_impl(const T* in, const T* f, T* out, const int64_t* in_shape,
                      const int64_t* f_shape, int rank, const int64_t* strides,
                      const int64_t* dil, const int64_t* pb, const int64_t* pe, bool grouped) {
    const int sp = rank - 2;
    Shape ishape = mk_shape(in_shape, rank);
    Shape fshape = mk_shape(f_shape, grouped ? rank + 1 : rank);
    Strides st(strides, strides + sp), di(dil, dil + sp);
    CoordinateDiff b(pb, pb + sp), e(pe, pe + sp);
    Shape oshape{ishape[0], grouped ? fshape[0] * fshape[1] : fshape[0]};
    for (int i = 0; i < sp; ++i) {
        size_t k = fshape[(grouped ? 3 : 2) + i];
        size_t padded = ishape[2 + i] + b[i] + e[i];
        oshape.push_back((padded - (di[i] * (k - 1) + 1)) / st[i] + 1);
    }
    if (grouped)
        ref::group_convolution<T, T, T, T>(in, f, out, ishape, fshape, oshape, st, di, b, e);
    else
        ref::convolution<T>(in, f, out, ishape, fshape, oshape, st, di, b, e);
}

extern "C" {

void ref_fake_quantize_f32(const float* x, const int64_t* xshape, int xrank, const float* il,
                           const int64_t* il_shape, int il_rank, const float* ih,
                           const int64_t* ih_shape, int ih_rank, const float* ol,
                           const int64_t* ol_shape, int ol_rank, const float* oh,
                           const int64_t* oh_shape, int oh_rank, int64_t levels, int bcast_axis,
                           float* out) {
    op::AutoBroadcastSpec spec = bcast_axis == -2
                                     ? op::AutoBroadcastSpec(op::AutoBroadcastType::NUMPY)
                                     : op::AutoBroadcastSpec(op::AutoBroadcastType::PDPD, bcast_axis);
    ref::v0::fake_quantize<float>(x, il, ih, ol, oh, out, mk_shape(xshape, xrank),
                                  mk_shape(il_shape, il_rank), mk_shape(ih_shape, ih_rank),
                                  mk_shape(ol_shape, ol_rank), mk_shape(oh_shape, oh_rank),
                                  static_cast<size_t>(levels), spec);
}

#define CONV_EXPORT(NAME, T, GROUPED)                                                          \
    void NAME(const T* in, const T* f, T* out, const int64_t* in_shape, const int64_t* f_shape, \
              int rank, const int64_t* strides, const int64_t* dil, const int64_t* pb,          \
              const int64_t* pe) {                                                              \
        conv_impl<T>(in, f, out, in_shape, f_shape, rank, strides, dil, pb, pe, GROUPED);       \
    }
CONV_EXPORT(ref_convolution_f32, float, false)
CONV_EXPORT(ref_convolution_i32, int32_t, false)
CONV_EXPORT(ref_convolution_i64, int64_t, false)
CONV_EXPORT(ref_convolution_f32_group, float, true)
CONV_EXPORT(ref_convolution_i32_group, int32_t, true)
CONV_EXPORT(ref_convolution_i64_group, int64_t, true)

#define MATMUL_EXPORT(NAME, T)                                                                  \
    void NAME(const T* a, const T* b, T* out, const int64_t* a_shape, int ar,                   \
              const int64_t* b_shape, int br, const int64_t* o_shape, int orank, int ta,        \
              int tb) {                                                                         \
        ref::matmul<T>(a, b, out, mk_shape(a_shape, ar), mk_shape(b_shape, br),                 \
                       mk_shape(o_shape, orank), ta != 0, tb != 0);                             \
    }
MATMUL_EXPORT(ref_matmul_f32, float)
MATMUL_EXPORT(ref_matmul_i32, int32_t)
MATMUL_EXPORT(ref_matmul_i64, int64_t)

#define BINOP_EXPORT(NAME, FN)                                                                  \
    void NAME(const float* a, const int64_t* a_shape, int ar, const float* b,                   \
              const int64_t* b_shape, int br, const int64_t*, int, float* out) {                \
        ref::FN<float>(a, b, out, mk_shape(a_shape, ar), mk_shape(b_shape, br),                 \
                       op::AutoBroadcastSpec(op::AutoBroadcastType::NUMPY));                    \
    }
void ref_prelu_f32(const float* a, const int64_t* a_shape, int ar, const float* slope, const int64_t* s_shape, int sr,
                   float* out) {
    ref::prelu<float>(a, slope, out, mk_shape(a_shape, ar), mk_shape(s_shape, sr));
}
void ref_sigmoid_f32(const float* x, float* out, int64_t n) { ref::sigmoid<float>(x, out, static_cast<size_t>(n)); }
void ref_hswish_f32(const float* x, float* out, int64_t n) { ref::hswish<float>(x, out, static_cast<size_t>(n)); }
void ref_hsigmoid_f32(const float* x, float* out, int64_t n) { ref::hsigmoid<float>(x, out, static_cast<size_t>(n)); }
void ref_swish_f32(const float* x, float beta, float* out, int64_t n) { ref::swish<float>(x, &beta, out, static_cast<size_t>(n)); }
BINOP_EXPORT(ref_add_f32, add)
BINOP_EXPORT(ref_subtract_f32, subtract)
BINOP_EXPORT(ref_multiply_f32, multiply)
void ref_divide_f32(const float* a, const int64_t* a_shape, int ar, const float* b,
                    const int64_t* b_shape, int br, const int64_t*, int, float* out) {
    ref::divide<float>(a, b, out, mk_shape(a_shape, ar), mk_shape(b_shape, br),
                       op::AutoBroadcastSpec(op::AutoBroadcastType::NUMPY), false);
}

void ref_relu_f32(const float* x, float* out, int64_t n) { ref::relu<float>(x, out, n); }
void ref_clamp_f32(const float* x, float* out, float mn, float mx, int64_t n) {
    ref::clamp<float>(x, out, mn, mx, n);
}

#define MAXPOOL_EXPORT(NAME, T)                                                                 \
    void NAME(const T* x, T* out, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh,       \
              int64_t kw, int64_t sh, int64_t sw, int64_t pbh, int64_t pbw, int64_t peh,        \
              int64_t pew, int64_t OH, int64_t OW) {                                            \
        ref::max_pool<T>(x, out, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W},             \
                         Shape{(size_t)N, (size_t)C, (size_t)OH, (size_t)OW},                   \
                         Shape{(size_t)kh, (size_t)kw}, Strides{(size_t)sh, (size_t)sw},        \
                         Shape{(size_t)pbh, (size_t)pbw}, Shape{(size_t)peh, (size_t)pew});     \
    }
MAXPOOL_EXPORT(ref_max_pool_f32, float)
MAXPOOL_EXPORT(ref_max_pool_u8, uint8_t)
MAXPOOL_EXPORT(ref_max_pool_i8, int8_t)
MAXPOOL_EXPORT(ref_max_pool_i32, int32_t)

#define AVGPOOL_EXPORT(NAME, T)                                                                 \
    void NAME(const T* x, T* out, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh,       \
              int64_t kw, int64_t sh, int64_t sw, int64_t pbh, int64_t pbw, int64_t peh,        \
              int64_t pew, int64_t OH, int64_t OW, int include_pad) {                           \
        ref::avg_pool<T>(x, out, Shape{(size_t)N, (size_t)C, (size_t)H, (size_t)W},             \
                         Shape{(size_t)N, (size_t)C, (size_t)OH, (size_t)OW},                   \
                         Shape{(size_t)kh, (size_t)kw}, Strides{(size_t)sh, (size_t)sw},        \
                         Shape{(size_t)pbh, (size_t)pbw}, Shape{(size_t)peh, (size_t)pew},      \
                         include_pad != 0);                                                     \
    }
AVGPOOL_EXPORT(ref_avg_pool_f32, float)
AVGPOOL_EXPORT(ref_avg_pool_u8, uint8_t)
AVGPOOL_EXPORT(ref_avg_pool_i8, int8_t)

void ref_softmax_f32(const float* x, float* out, int64_t outer, int64_t axis, int64_t inner) {
    ref::softmax<float>(x, out, Shape{(size_t)outer, (size_t)axis, (size_t)inner}, AxisSet{1});
}
void ref_mvn_last_axis_f32(const float* x, float* out, int64_t outer, int64_t axis,
                           int normalize_variance, double eps, int eps_inside) {
    ref::mvn_6<float>(x, out, Shape{(size_t)outer, (size_t)axis}, AxisSet{1},
                      normalize_variance != 0, eps,
                      eps_inside ? op::MVNEpsMode::INSIDE_SQRT : op::MVNEpsMode::OUTSIDE_SQRT);
}
void ref_gelu_erf_f32(const float* x, float* out, int64_t n) {
    ref::gelu<float>(x, out, op::GeluApproximationMode::ERF, n);
}

}  // extern "C"
