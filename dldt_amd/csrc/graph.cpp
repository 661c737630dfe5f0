// Graph description entry points: one call per nGraph node of the post-LPT Function, with the
// shape/type inference the planner relies on (ngraph/core/src/op/{convolution,group_conv,matmul,
// max_pool,avg_pool,fake_quantize}.cpp validate_and_infer_types).
#include "graph.h"

namespace hipie {

// the kinds hipie_graph_eltwise takes are the planner's own operation numbers
static_assert(HIPIE_OP_ADD == OP_ADD && HIPIE_OP_MULTIPLY == OP_MULTIPLY && HIPIE_OP_SUBTRACT == OP_SUBTRACT && HIPIE_OP_PRELU == OP_PRELU &&
                  HIPIE_OP_SIGMOID == OP_SIGMOID && HIPIE_OP_HSWISH == OP_HSWISH && HIPIE_OP_HSIGMOID == OP_HSIGMOID &&
                  HIPIE_OP_SWISH == OP_SWISH,
              "include/hipie.h and graph.h number the elementwise operations differently");

const char* op_name(int op) {
    static const char* names[] = {"Parameter", "Constant", "FakeQuantize", "Convolution",
                                  "GroupConvolution", "MatMul", "Add", "Multiply", "Subtract", "Relu",
                                  "Clamp", "Convert", "MaxPool", "AvgPool", "Reshape", "Result", "Softmax", "MVN",
                                  "Gelu", "Transpose", "Gather", "Concat", "Slice", "PRelu",
                                  "Sigmoid", "HSwish", "HSigmoid", "Swish"};
    return op >= 0 && op <= OP_SWISH ? names[op] : "?";
}

namespace {

constexpr int64_t kMaxAttr = int64_t(1) << 20;   // strides, dilations, pads, windows: products with a dimension stay in int64

size_t dtype_size(int dt) {
    switch (dt) {
    case HIPIE_F32: case HIPIE_I32: return 4;
    case HIPIE_U8: case HIPIE_I8: case HIPIE_U8B: return 1;
    default: fail(HIPIE_PARAMETER_MISMATCH, "unknown element type %d", dt);
    }
}

GNode& node(hipie_graph* g, int id, const char* what) {
    HIPIE_REQUIRE(g, HIPIE_PARAMETER_MISMATCH, "%s: null graph", what);
    HIPIE_REQUIRE(id >= 0 && id < static_cast<int>(g->nodes.size()), HIPIE_NOT_FOUND,
                  "%s: no value with id %d", what, id);
    HIPIE_REQUIRE(g->nodes[id].op != OP_RESULT, HIPIE_PARAMETER_MISMATCH, "%s: id %d is a Result", what, id);
    return g->nodes[id];
}

int add_node(hipie_graph* g, GNode&& n) {
    const int id = static_cast<int>(g->nodes.size());
    int64_t count = 1;
    for (int64_t d : n.shape) {   // element counts stay far inside int64 for everything computed from them
        HIPIE_REQUIRE(d >= 0 && (d == 0 || count <= (int64_t(1) << 40) / d), HIPIE_PARAMETER_MISMATCH,
                      "%s: a value of more than 2^40 elements", op_name(n.op));
        count *= d;
    }
    if (n.name.empty()) n.name = std::string(op_name(n.op)) + "_" + std::to_string(id);
    for (int i : n.in) g->nodes[i].users.push_back(id);
    g->nodes.push_back(std::move(n));
    return id;
}

std::vector<int64_t> broadcast_shape(const std::vector<int64_t>& a, const std::vector<int64_t>& b,
                                     const char* what) {
    const size_t r = std::max(a.size(), b.size());
    std::vector<int64_t> o(r);
    for (size_t i = 0; i < r; ++i) {
        const int64_t da = i + a.size() >= r ? a[i + a.size() - r] : 1;
        const int64_t db = i + b.size() >= r ? b[i + b.size() - r] : 1;
        HIPIE_REQUIRE(da == db || da == 1 || db == 1, HIPIE_PARAMETER_MISMATCH,
                      "%s: shapes do not broadcast", what);
        o[i] = std::max(da, db);
    }
    return o;
}

int64_t pooled(int64_t in, int64_t pb, int64_t pe, int64_t window, int64_t stride, bool ceil_mode) {
    const int64_t span = in + pb + pe - window;
    HIPIE_REQUIRE(span >= 0, HIPIE_PARAMETER_MISMATCH, "window larger than the padded input");
    return (ceil_mode ? ceil_div(span, stride) : span / stride) + 1;
}

}  // namespace
}  // namespace hipie

using namespace hipie;

extern "C" {

int hipie_graph_create(hipie_graph** g) {
    return guarded([&] {
        HIPIE_REQUIRE(g, HIPIE_PARAMETER_MISMATCH, "hipie_graph_create: null argument");
        *g = new hipie_graph();
    });
}

void hipie_graph_destroy(hipie_graph* g) { delete g; }

int hipie_graph_parameter(hipie_graph* g, const char* name, int dtype, const int64_t* dims, int rank, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(g && dims && id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_parameter: null argument");
        HIPIE_REQUIRE(rank >= 2 && rank <= 5, HIPIE_NOT_IMPLEMENTED, "hipie_graph_parameter: rank %d", rank);
        HIPIE_REQUIRE(dtype == HIPIE_F32 || dtype == HIPIE_U8 || dtype == HIPIE_I32, HIPIE_NOT_IMPLEMENTED,
                      "hipie_graph_parameter: element type %d", dtype);
        for (int i = 0; i < rank; ++i)
            HIPIE_REQUIRE(dims[i] > 0 && dims[i] < (int64_t(1) << 31), HIPIE_PARAMETER_MISMATCH,
                          "hipie_graph_parameter: dimension %d is %lld", i, (long long)dims[i]);
        GNode n;
        n.op = OP_PARAMETER;
        n.name = name ? name : "";
        n.dtype = dtype;
        n.shape.assign(dims, dims + rank);
        *id = add_node(g, std::move(n));
        g->params.push_back(*id);
    });
}

int hipie_graph_constant(hipie_graph* g, int dtype, const int64_t* dims, int rank, const void* data, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(g && id && data && (dims || rank == 0), HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_constant: null argument");
        HIPIE_REQUIRE(rank >= 0 && rank <= 8, HIPIE_PARAMETER_MISMATCH, "hipie_graph_constant: rank %d", rank);
        for (int i = 0; i < rank; ++i)
            HIPIE_REQUIRE(dims[i] >= 0 && dims[i] < (int64_t(1) << 31), HIPIE_PARAMETER_MISMATCH,
                          "hipie_graph_constant: dimension %d is %lld", i, (long long)dims[i]);
        GNode n;
        n.op = OP_CONSTANT;
        n.dtype = dtype;
        n.shape.assign(dims, dims + rank);
        const size_t bytes = static_cast<size_t>(n.numel()) * dtype_size(dtype);
        n.data.assign(static_cast<const uint8_t*>(data), static_cast<const uint8_t*>(data) + bytes);
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_fake_quantize(hipie_graph* g, int x, int il, int ih, int ol, int oh, int64_t levels,
                              int out_dtype, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_fake_quantize: null argument");
        GNode& X = node(g, x, "hipie_graph_fake_quantize");
        HIPIE_REQUIRE(X.dtype == HIPIE_F32, HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_fake_quantize: data must be f32");
        for (int b : {il, ih, ol, oh}) {
            GNode& B = node(g, b, "hipie_graph_fake_quantize");
            HIPIE_REQUIRE(B.op == OP_CONSTANT && B.dtype == HIPIE_F32, HIPIE_NOT_IMPLEMENTED,
                          "hipie_graph_fake_quantize: bounds must be f32 constants");
            broadcast_shape(X.shape, B.shape, "hipie_graph_fake_quantize");
        }
        HIPIE_REQUIRE(levels >= 2, HIPIE_PARAMETER_MISMATCH, "hipie_graph_fake_quantize: levels");
        HIPIE_REQUIRE(out_dtype == HIPIE_F32 || out_dtype == HIPIE_U8 || out_dtype == HIPIE_I8,
                      HIPIE_PARAMETER_MISMATCH, "hipie_graph_fake_quantize: output type %d", out_dtype);
        GNode n;
        n.op = OP_FAKE_QUANTIZE;
        n.in = {x, il, ih, ol, oh};
        n.levels = levels;
        n.dtype = out_dtype;
        n.shape = X.shape;
        *id = add_node(g, std::move(n));
    });
}

static int add_conv(hipie_graph* g, int x, int w, const int64_t* strides, const int64_t* dilations,
                    const int64_t* pads_begin, const int64_t* pads_end, bool grouped, int* id) {
    return guarded([&] {
        const char* what = grouped ? "hipie_graph_group_convolution" : "hipie_graph_convolution";
        HIPIE_REQUIRE(id && strides && dilations && pads_begin && pads_end, HIPIE_PARAMETER_MISMATCH,
                      "%s: null argument", what);
        GNode& X = node(g, x, what);
        GNode& W = node(g, w, what);
        // [N, C, W], [N, C, H, W] or [N, C, D, H, W]: one attribute per spatial dimension
        HIPIE_REQUIRE(X.shape.size() >= 3 && X.shape.size() <= 5, HIPIE_NOT_IMPLEMENTED, "%s: one to three spatial dimensions", what);
        const int sp = static_cast<int>(X.shape.size()) - 2;
        HIPIE_REQUIRE(W.shape.size() == X.shape.size() + (grouped ? 1u : 0u), HIPIE_PARAMETER_MISMATCH, "%s: filter rank", what);
        const int o = grouped ? 1 : 0;
        const int64_t G = grouped ? W.shape[0] : 1;
        HIPIE_REQUIRE(X.shape[1] == W.shape[o + 1] * G, HIPIE_PARAMETER_MISMATCH,
                      "%s: input channels %lld vs filter %lld x %lld groups", what, (long long)X.shape[1],
                      (long long)W.shape[o + 1], (long long)G);
        GNode n;
        n.op = grouped ? OP_GROUP_CONVOLUTION : OP_CONVOLUTION;
        n.in = {x, w};
        n.strides.assign(strides, strides + sp);
        n.dilations.assign(dilations, dilations + sp);
        n.pads_begin.assign(pads_begin, pads_begin + sp);
        n.pads_end.assign(pads_end, pads_end + sp);
        n.dtype = HIPIE_F32;  // TypeRelaxed<Convolution>: f32 holding the integer sum
        n.shape = {X.shape[0], W.shape[o] * G};
        for (int i = 0; i < sp; ++i) {
            HIPIE_REQUIRE(n.strides[i] > 0 && n.dilations[i] > 0 && n.pads_begin[i] >= 0 && n.pads_end[i] >= 0 &&
                              std::max(std::max(n.strides[i], n.dilations[i]), std::max(n.pads_begin[i], n.pads_end[i])) < kMaxAttr,
                          HIPIE_PARAMETER_MISMATCH, "%s: attributes", what);
            const int64_t dk = n.dilations[i] * (W.shape[o + 2 + i] - 1) + 1;
            const int64_t span = X.shape[2 + i] + n.pads_begin[i] + n.pads_end[i] - dk;
            HIPIE_REQUIRE(span >= 0, HIPIE_PARAMETER_MISMATCH, "%s: filter larger than padded input", what);
            n.shape.push_back(span / n.strides[i] + 1);
        }
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_convolution(hipie_graph* g, int x, int w, const int64_t* strides, const int64_t* dilations,
                            const int64_t* pads_begin, const int64_t* pads_end, int* id) {
    return add_conv(g, x, w, strides, dilations, pads_begin, pads_end, false, id);
}

int hipie_graph_group_convolution(hipie_graph* g, int x, int w, const int64_t* strides,
                                  const int64_t* dilations, const int64_t* pads_begin,
                                  const int64_t* pads_end, int* id) {
    return add_conv(g, x, w, strides, dilations, pads_begin, pads_end, true, id);
}

int hipie_graph_matmul(hipie_graph* g, int a, int b, int transpose_a, int transpose_b, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_matmul: null argument");
        GNode& A = node(g, a, "hipie_graph_matmul");
        GNode& B = node(g, b, "hipie_graph_matmul");
        HIPIE_REQUIRE(A.shape.size() >= 2 && B.shape.size() >= 2, HIPIE_NOT_IMPLEMENTED,
                      "hipie_graph_matmul: 1-D operands");
        std::vector<int64_t> sa = A.shape, sb = B.shape;
        if (transpose_a) std::swap(sa[sa.size() - 1], sa[sa.size() - 2]);
        if (transpose_b) std::swap(sb[sb.size() - 1], sb[sb.size() - 2]);
        HIPIE_REQUIRE(sa.back() == sb[sb.size() - 2], HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_matmul: inner dimensions %lld vs %lld", (long long)sa.back(),
                      (long long)sb[sb.size() - 2]);
        std::vector<int64_t> ba(sa.begin(), sa.end() - 2), bb(sb.begin(), sb.end() - 2);
        GNode n;
        n.op = OP_MATMUL;
        n.in = {a, b};
        n.ta = transpose_a != 0;
        n.tb = transpose_b != 0;
        n.dtype = HIPIE_F32;
        n.shape = broadcast_shape(ba, bb, "hipie_graph_matmul");
        n.shape.push_back(sa[sa.size() - 2]);
        n.shape.push_back(sb.back());
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_eltwise(hipie_graph* g, int kind, int a, int b, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_eltwise: null argument");
        HIPIE_REQUIRE(kind == OP_ADD || kind == OP_MULTIPLY || kind == OP_SUBTRACT || kind == OP_PRELU, HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_eltwise: kind %d", kind);
        GNode& A = node(g, a, "hipie_graph_eltwise");
        GNode& B = node(g, b, "hipie_graph_eltwise");
        HIPIE_REQUIRE(A.dtype == HIPIE_F32 && B.dtype == HIPIE_F32, HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_eltwise: operands must be f32 (insert Convert)");
        GNode n;
        n.op = kind;
        n.in = {a, b};
        n.dtype = HIPIE_F32;
        if (kind == OP_PRELU) {
            // op::v0::PRelu: the result has the argument's shape; a one-dimensional slope with one element per channel
            // is taken per channel (prelu.hpp:28-35), any other slope must broadcast onto the argument
            const size_t channel_axis = A.shape.size() > 1 ? 1 : 0;
            if (!(B.shape.size() == 1 && !A.shape.empty() && B.shape[0] == A.shape[channel_axis]))
                HIPIE_REQUIRE(broadcast_shape(A.shape, B.shape, "hipie_graph_eltwise") == A.shape, HIPIE_PARAMETER_MISMATCH,
                              "hipie_graph_eltwise: a PRelu slope larger than its argument");
            n.shape = A.shape;
        } else {
            n.shape = broadcast_shape(A.shape, B.shape, "hipie_graph_eltwise");
        }
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_relu(hipie_graph* g, int x, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_relu: null argument");
        GNode& X = node(g, x, "hipie_graph_relu");
        GNode n;
        n.op = OP_RELU;
        n.in = {x};
        n.dtype = X.dtype;
        n.shape = X.shape;
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_activation(hipie_graph* g, int kind, int x, float beta, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_activation: null argument");
        HIPIE_REQUIRE(kind == OP_SIGMOID || kind == OP_HSWISH || kind == OP_HSIGMOID || kind == OP_SWISH, HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_activation: kind %d", kind);
        GNode& X = node(g, x, "hipie_graph_activation");
        HIPIE_REQUIRE(X.dtype == HIPIE_F32, HIPIE_PARAMETER_MISMATCH, "hipie_graph_activation: data must be f32");
        GNode n;
        n.op = kind;
        n.in = {x};
        n.lo = kind == OP_SWISH ? beta : 0.f;
        n.dtype = HIPIE_F32;
        n.shape = X.shape;
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_clamp(hipie_graph* g, int x, float lo, float hi, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_clamp: null argument");
        HIPIE_REQUIRE(lo <= hi, HIPIE_PARAMETER_MISMATCH, "hipie_graph_clamp: min > max");
        GNode& X = node(g, x, "hipie_graph_clamp");
        GNode n;
        n.op = OP_CLAMP;
        n.in = {x};
        n.lo = lo;
        n.hi = hi;
        n.dtype = X.dtype;
        n.shape = X.shape;
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_convert(hipie_graph* g, int x, int dtype, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_convert: null argument");
        GNode& X = node(g, x, "hipie_graph_convert");
        dtype_size(dtype);
        GNode n;
        n.op = OP_CONVERT;
        n.in = {x};
        n.dtype = dtype;
        n.shape = X.shape;
        *id = add_node(g, std::move(n));
    });
}

static int add_pool(hipie_graph* g, int op, int x, const int64_t* kernel, const int64_t* strides,
                    const int64_t* pads_begin, const int64_t* pads_end, int exclude_pad, int ceil_mode,
                    int out_dtype, int* id) {
    return guarded([&] {
        const char* what = op == OP_MAX_POOL ? "hipie_graph_max_pool" : "hipie_graph_avg_pool";
        HIPIE_REQUIRE(id && kernel && strides && pads_begin && pads_end, HIPIE_PARAMETER_MISMATCH,
                      "%s: null argument", what);
        GNode& X = node(g, x, what);
        HIPIE_REQUIRE(X.shape.size() == 4 || X.shape.size() == 3, HIPIE_NOT_IMPLEMENTED, "%s: one or two spatial dimensions", what);
        const int sp = static_cast<int>(X.shape.size()) - 2;
        GNode n;
        n.op = op;
        n.in = {x};
        n.kernel.assign(kernel, kernel + sp);
        n.strides.assign(strides, strides + sp);
        n.pads_begin.assign(pads_begin, pads_begin + sp);
        n.pads_end.assign(pads_end, pads_end + sp);
        n.exclude_pad = exclude_pad != 0;
        n.ceil_mode = ceil_mode != 0;
        n.dtype = out_dtype;
        n.shape = {X.shape[0], X.shape[1]};
        for (int i = 0; i < sp; ++i) {
            HIPIE_REQUIRE(kernel[i] > 0 && strides[i] > 0 && pads_begin[i] >= 0 && pads_end[i] >= 0 &&
                              std::max(std::max(kernel[i], strides[i]), std::max(pads_begin[i], pads_end[i])) < kMaxAttr,
                          HIPIE_PARAMETER_MISMATCH, "%s: attributes", what);
            n.shape.push_back(pooled(X.shape[2 + i], pads_begin[i], pads_end[i], kernel[i], strides[i], n.ceil_mode));
            // every window must hold a cell of the tensor: one that lies in the padding alone has no maximum
            // and no divisor in the reference (max_pool.hpp starts from lowest(), avg_pool.hpp divides by 0 cells)
            const int64_t last_start = (n.shape.back() - 1) * strides[i] - pads_begin[i];
            HIPIE_REQUIRE(pads_begin[i] < kernel[i] && last_start < X.shape[2 + i], HIPIE_PARAMETER_MISMATCH,
                          "%s: a window along axis %d lies in the padding alone", what, 2 + i);
        }
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_max_pool(hipie_graph* g, int x, const int64_t* kernel, const int64_t* strides,
                         const int64_t* pads_begin, const int64_t* pads_end, int ceil_mode, int* id) {
    if (!g || x < 0 || x >= static_cast<int>(g->nodes.size()))
        return guarded([&] { fail(HIPIE_NOT_FOUND, "hipie_graph_max_pool: no value with id %d", x); });
    return add_pool(g, OP_MAX_POOL, x, kernel, strides, pads_begin, pads_end, 0, ceil_mode,
                    g->nodes[x].dtype, id);
}

int hipie_graph_avg_pool(hipie_graph* g, int x, const int64_t* kernel, const int64_t* strides,
                         const int64_t* pads_begin, const int64_t* pads_end, int exclude_pad, int ceil_mode,
                         int out_dtype, int* id) {
    return add_pool(g, OP_AVG_POOL, x, kernel, strides, pads_begin, pads_end, exclude_pad, ceil_mode,
                    out_dtype, id);
}

int hipie_graph_reshape(hipie_graph* g, int x, const int64_t* dims, int rank, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id && dims, HIPIE_PARAMETER_MISMATCH, "hipie_graph_reshape: null argument");
        GNode& X = node(g, x, "hipie_graph_reshape");
        GNode n;
        n.op = OP_RESHAPE;
        n.in = {x};
        n.dtype = X.dtype;
        HIPIE_REQUIRE(rank >= 1 && rank <= 8, HIPIE_PARAMETER_MISMATCH, "hipie_graph_reshape: rank %d", rank);
        for (int i = 0; i < rank; ++i)
            HIPIE_REQUIRE(dims[i] > 0 && dims[i] < (int64_t(1) << 31), HIPIE_PARAMETER_MISMATCH,
                          "hipie_graph_reshape: dimension %d is %lld", i, (long long)dims[i]);
        n.shape.assign(dims, dims + rank);
        HIPIE_REQUIRE(n.numel() == X.numel(), HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_reshape: element count changes");
        *id = add_node(g, std::move(n));
    });
}

/* op::v1::Softmax (ngraph/core/src/op/softmax.cpp): same shape and type; the axis may be negative */
int hipie_graph_softmax(hipie_graph* g, int x, int64_t axis, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_softmax: null argument");
        GNode& X = node(g, x, "hipie_graph_softmax");
        const int64_t r = static_cast<int64_t>(X.shape.size());
        HIPIE_REQUIRE(X.dtype == HIPIE_F32, HIPIE_PARAMETER_MISMATCH, "hipie_graph_softmax: data must be f32");
        HIPIE_REQUIRE(axis >= -r && axis < r, HIPIE_PARAMETER_MISMATCH, "hipie_graph_softmax: axis %lld of rank %lld",
                      (long long)axis, (long long)r);
        GNode n;
        n.op = OP_SOFTMAX;
        n.in = {x};
        n.axes = {axis < 0 ? axis + r : axis};
        n.dtype = HIPIE_F32;
        n.shape = X.shape;
        *id = add_node(g, std::move(n));
    });
}

/* op::v6::MVN (ngraph/core/src/op/mvn.cpp:93-140): the axes input is passed as an array */
int hipie_graph_mvn(hipie_graph* g, int x, const int64_t* axes, int n_axes, int normalize_variance, float eps,
                    int eps_inside_sqrt, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id && axes && n_axes > 0, HIPIE_PARAMETER_MISMATCH, "hipie_graph_mvn: null argument");
        GNode& X = node(g, x, "hipie_graph_mvn");
        const int64_t r = static_cast<int64_t>(X.shape.size());
        HIPIE_REQUIRE(X.dtype == HIPIE_F32, HIPIE_PARAMETER_MISMATCH, "hipie_graph_mvn: data must be f32");
        GNode n;
        n.op = OP_MVN;
        n.in = {x};
        for (int i = 0; i < n_axes; ++i) {
            HIPIE_REQUIRE(axes[i] >= -r && axes[i] < r, HIPIE_PARAMETER_MISMATCH, "hipie_graph_mvn: axis %lld of rank %lld",
                          (long long)axes[i], (long long)r);
            n.axes.push_back(axes[i] < 0 ? axes[i] + r : axes[i]);
        }
        n.normalize_variance = normalize_variance != 0;
        n.eps = eps;
        n.eps_inside_sqrt = eps_inside_sqrt != 0;
        n.dtype = HIPIE_F32;
        n.shape = X.shape;
        *id = add_node(g, std::move(n));
    });
}

/* op::v0::Gelu / op::v7::Gelu in ERF mode (ngraph/core/src/op/gelu.cpp) */
int hipie_graph_gelu(hipie_graph* g, int x, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_gelu: null argument");
        GNode& X = node(g, x, "hipie_graph_gelu");
        HIPIE_REQUIRE(X.dtype == HIPIE_F32, HIPIE_PARAMETER_MISMATCH, "hipie_graph_gelu: data must be f32");
        GNode n;
        n.op = OP_GELU;
        n.in = {x};
        n.dtype = HIPIE_F32;
        n.shape = X.shape;
        *id = add_node(g, std::move(n));
    });
}

/* op::v1::Transpose (ngraph/core/src/op/transpose.cpp:40-80): out.shape[i] = in.shape[order[i]] */
int hipie_graph_transpose(hipie_graph* g, int x, const int64_t* order, int rank, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id && order, HIPIE_PARAMETER_MISMATCH, "hipie_graph_transpose: null argument");
        GNode& X = node(g, x, "hipie_graph_transpose");
        HIPIE_REQUIRE(rank == static_cast<int>(X.shape.size()), HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_transpose: order has %d entries for a rank-%zu value", rank, X.shape.size());
        GNode n;
        n.op = OP_TRANSPOSE;
        n.in = {x};
        std::vector<char> seen(rank, 0);
        for (int i = 0; i < rank; ++i) {
            HIPIE_REQUIRE(order[i] >= 0 && order[i] < rank && !seen[order[i]], HIPIE_PARAMETER_MISMATCH,
                          "hipie_graph_transpose: order is not a permutation");
            seen[order[i]] = 1;
            n.axes.push_back(order[i]);
            n.shape.push_back(X.shape[order[i]]);
        }
        n.dtype = X.dtype;
        *id = add_node(g, std::move(n));
    });
}

/* op::v1::Gather (ngraph/core/src/op/gather.cpp): out.shape = data.shape[:axis] + indices.shape + data.shape[axis+1:] */
int hipie_graph_gather(hipie_graph* g, int data, int indices, int64_t axis, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_gather: null argument");
        GNode& D = node(g, data, "hipie_graph_gather");
        GNode& I = node(g, indices, "hipie_graph_gather");
        const int64_t r = static_cast<int64_t>(D.shape.size());
        HIPIE_REQUIRE(I.dtype == HIPIE_I32, HIPIE_PARAMETER_MISMATCH, "hipie_graph_gather: indices must be i32");
        HIPIE_REQUIRE(axis >= -r && axis < r, HIPIE_PARAMETER_MISMATCH, "hipie_graph_gather: axis %lld of rank %lld",
                      (long long)axis, (long long)r);
        GNode n;
        n.op = OP_GATHER;
        n.in = {data, indices};
        const int64_t ax = axis < 0 ? axis + r : axis;
        n.axes = {ax};
        n.dtype = D.dtype;
        n.shape.assign(D.shape.begin(), D.shape.begin() + ax);
        n.shape.insert(n.shape.end(), I.shape.begin(), I.shape.end());
        n.shape.insert(n.shape.end(), D.shape.begin() + ax + 1, D.shape.end());
        *id = add_node(g, std::move(n));
    });
}

/* op::v0::Concat (ngraph/core/src/op/concat.cpp validate_and_infer_types): same element type and rank, all
 * dimensions but `axis` equal; the axis may be negative */
int hipie_graph_concat(hipie_graph* g, const int* inputs, int n_inputs, int64_t axis, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id && inputs && n_inputs >= 1 && n_inputs <= 64, HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_concat: %d inputs (1 to 64)", n_inputs);
        const GNode& X0 = node(g, inputs[0], "hipie_graph_concat");
        const int64_t r = static_cast<int64_t>(X0.shape.size());
        HIPIE_REQUIRE(axis >= -r && axis < r, HIPIE_PARAMETER_MISMATCH, "hipie_graph_concat: axis %lld of rank %lld",
                      (long long)axis, (long long)r);
        const int64_t ax = axis < 0 ? axis + r : axis;
        GNode n;
        n.op = OP_CONCAT;
        n.axes = {ax};
        n.dtype = X0.dtype;
        n.shape = X0.shape;
        n.shape[ax] = 0;
        for (int i = 0; i < n_inputs; ++i) {
            const GNode& X = node(g, inputs[i], "hipie_graph_concat");
            HIPIE_REQUIRE(X.dtype == X0.dtype && X.shape.size() == X0.shape.size(), HIPIE_PARAMETER_MISMATCH,
                          "hipie_graph_concat: input %d differs in type or rank", i);
            for (int64_t k = 0; k < r; ++k)
                HIPIE_REQUIRE(k == ax || X.shape[k] == X0.shape[k], HIPIE_PARAMETER_MISMATCH,
                              "hipie_graph_concat: input %d differs in dimension %lld", i, (long long)k);
            n.shape[ax] += X.shape[ax];
            n.in.push_back(inputs[i]);
        }
        HIPIE_REQUIRE(n.shape[ax] < (int64_t(1) << 31), HIPIE_OUT_OF_BOUNDS, "hipie_graph_concat: concatenated dimension too large");
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_slice(hipie_graph* g, int x, int64_t axis, int64_t begin, int64_t end, int* id) {
    return guarded([&] {
        HIPIE_REQUIRE(id, HIPIE_PARAMETER_MISMATCH, "hipie_graph_slice: null argument");
        const GNode& X = node(g, x, "hipie_graph_slice");
        const int64_t r = static_cast<int64_t>(X.shape.size());
        HIPIE_REQUIRE(axis >= -r && axis < r, HIPIE_PARAMETER_MISMATCH, "hipie_graph_slice: axis %lld of rank %lld", (long long)axis, (long long)r);
        const int64_t ax = axis < 0 ? axis + r : axis;
        HIPIE_REQUIRE(begin >= 0 && begin < end && end <= X.shape[static_cast<size_t>(ax)], HIPIE_PARAMETER_MISMATCH,
                      "hipie_graph_slice: [%lld, %lld) of %lld elements", (long long)begin, (long long)end, (long long)X.shape[static_cast<size_t>(ax)]);
        GNode n;
        n.op = OP_SLICE;
        n.in = {x};
        n.axes = {ax, begin, end};
        n.dtype = X.dtype;
        n.shape = X.shape;
        n.shape[static_cast<size_t>(ax)] = end - begin;
        *id = add_node(g, std::move(n));
    });
}

int hipie_graph_result(hipie_graph* g, int x, const char* name) {
    return guarded([&] {
        GNode& X = node(g, x, "hipie_graph_result");
        GNode n;
        n.op = OP_RESULT;
        n.in = {x};
        n.name = name ? name : X.name;
        n.dtype = X.dtype;
        n.shape = X.shape;
        g->results.push_back(add_node(g, std::move(n)));
    });
}

int hipie_graph_set_name(hipie_graph* g, int id, const char* name) {
    return guarded([&] {
        HIPIE_REQUIRE(name, HIPIE_PARAMETER_MISMATCH, "hipie_graph_set_name: null name");
        node(g, id, "hipie_graph_set_name").name = name;
    });
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------
// Graph description as a byte stream (the model part of an exported plan).  Reading it REPLAYS the
// description through the entry points above, one call per node, so a stream gets exactly the
// validation and shape inference a freshly described graph gets; every length is checked against
// the bytes that remain before it is used.
namespace hipie {
namespace {

// writes into `dst` when there is one, counts the bytes either way
struct Writer {
    uint8_t* dst;
    size_t n = 0;
    void raw(const void* p, size_t len) {
        if (dst && len) std::memcpy(dst + n, p, len);
        n += len;
    }
    template <typename T> void pod(T v) { raw(&v, sizeof v); }
    void str(const std::string& s) { pod<uint32_t>(static_cast<uint32_t>(s.size())); raw(s.data(), s.size()); }
    void i64s(const std::vector<int64_t>& v) { pod<uint32_t>(static_cast<uint32_t>(v.size())); raw(v.data(), v.size() * 8); }
    void ints(const std::vector<int>& v) { pod<uint32_t>(static_cast<uint32_t>(v.size())); raw(v.data(), v.size() * 4); }
};

struct Reader {
    const uint8_t* p;
    size_t left;
    const uint8_t* take(size_t n) {
        HIPIE_REQUIRE(n <= left, HIPIE_NETWORK_NOT_READ, "plan stream is truncated");
        const uint8_t* q = p;
        p += n;
        left -= n;
        return q;
    }
    template <typename T> T pod() { T v; std::memcpy(&v, take(sizeof v), sizeof v); return v; }
    std::string str() {
        const uint32_t n = pod<uint32_t>();
        const uint8_t* q = take(n);
        return std::string(reinterpret_cast<const char*>(q), n);
    }
    std::vector<int64_t> i64s(size_t max_len) {
        const uint32_t n = pod<uint32_t>();
        HIPIE_REQUIRE(n <= max_len, HIPIE_NETWORK_NOT_READ, "plan stream: attribute with %u entries", n);
        std::vector<int64_t> v(n);
        if (n) std::memcpy(v.data(), take(size_t(n) * 8), size_t(n) * 8);
        return v;
    }
    std::vector<int> ints(size_t max_len) {
        const uint32_t n = pod<uint32_t>();
        HIPIE_REQUIRE(n <= max_len, HIPIE_NETWORK_NOT_READ, "plan stream: node with %u inputs", n);
        std::vector<int> v(n);
        if (n) std::memcpy(v.data(), take(size_t(n) * 4), size_t(n) * 4);
        return v;
    }
};

enum : uint8_t { F_TA = 1, F_TB = 2, F_EXCLUDE_PAD = 4, F_CEIL = 8, F_NORM_VAR = 16, F_EPS_INSIDE = 32 };

}  // namespace

size_t serialize_graph(const hipie_graph& g, uint8_t* dst) {
    Writer w{dst};
    w.pod<uint32_t>(static_cast<uint32_t>(g.nodes.size()));
    for (const GNode& n : g.nodes) {
        w.pod<int32_t>(n.op);
        w.str(n.name);
        w.ints(n.in);
        w.pod<int32_t>(n.dtype);
        w.i64s(n.shape);
        w.i64s(n.strides);
        w.i64s(n.dilations);
        w.i64s(n.pads_begin);
        w.i64s(n.pads_end);
        w.i64s(n.kernel);
        w.i64s(n.axes);
        w.pod<int64_t>(n.levels);
        w.pod<uint8_t>((n.ta ? F_TA : 0) | (n.tb ? F_TB : 0) | (n.exclude_pad ? F_EXCLUDE_PAD : 0) | (n.ceil_mode ? F_CEIL : 0) |
                       (n.normalize_variance ? F_NORM_VAR : 0) | (n.eps_inside_sqrt ? F_EPS_INSIDE : 0));
        w.pod<float>(n.lo);
        w.pod<float>(n.hi);
        w.pod<float>(n.eps);
        w.pod<uint64_t>(n.data.size());
        w.raw(n.data.data(), n.data.size());
    }
    return w.n;
}

hipie_graph* deserialize_graph(const uint8_t* bytes, size_t size) {
    Reader r{bytes, size};
    auto g = std::make_unique<hipie_graph>();
    hipie_graph* G = g.get();
    const uint32_t count = r.pod<uint32_t>();
    HIPIE_REQUIRE(count <= size, HIPIE_NETWORK_NOT_READ, "plan stream: %u nodes in %zu bytes", count, size);
    for (uint32_t i = 0; i < count; ++i) {
        const int op = r.pod<int32_t>();
        const std::string name = r.str();
        const std::vector<int> in = r.ints(64);
        const int dtype = r.pod<int32_t>();
        const std::vector<int64_t> shape = r.i64s(8), strides = r.i64s(3), dilations = r.i64s(3), pads_begin = r.i64s(3),
                                   pads_end = r.i64s(3), kernel = r.i64s(3), axes = r.i64s(8);
        const int64_t levels = r.pod<int64_t>();
        const uint8_t flags = r.pod<uint8_t>();
        const float lo = r.pod<float>(), hi = r.pod<float>(), eps = r.pod<float>();
        const uint64_t nbytes = r.pod<uint64_t>();
        HIPIE_REQUIRE(nbytes <= r.left, HIPIE_NETWORK_NOT_READ, "plan stream is truncated");
        const uint8_t* data = r.take(static_cast<size_t>(nbytes));
        auto arity = [&](size_t n) {
            HIPIE_REQUIRE(in.size() == n, HIPIE_NETWORK_NOT_READ, "plan stream: node %u (%s) has %zu inputs", i, op_name(op), in.size());
        };
        auto pair = [&](const std::vector<int64_t>& v) {     // one entry per spatial dimension of the node's input
            HIPIE_REQUIRE(!in.empty() && in[0] >= 0 && in[0] < static_cast<int>(G->nodes.size()), HIPIE_NETWORK_NOT_READ,
                          "plan stream: node %u (%s) reads a value that is not there", i, op_name(op));
            const size_t rank = G->nodes[static_cast<size_t>(in[0])].shape.size();
            HIPIE_REQUIRE(rank >= 3 && v.size() == rank - 2, HIPIE_NETWORK_NOT_READ, "plan stream: node %u (%s) lacks an attribute", i, op_name(op));
            return v.data();
        };
        int id = static_cast<int>(i), st = HIPIE_OK;
        switch (op) {
        case OP_PARAMETER:
            arity(0);
            st = hipie_graph_parameter(G, name.c_str(), dtype, shape.data(), static_cast<int>(shape.size()), &id);
            break;
        case OP_CONSTANT: {
            arity(0);
            uint64_t want = dtype == HIPIE_F32 || dtype == HIPIE_I32 ? 4 : 1;
            for (int64_t d : shape) {
                HIPIE_REQUIRE(d >= 0 && (d == 0 || want <= nbytes / static_cast<uint64_t>(d)), HIPIE_NETWORK_NOT_READ,
                              "plan stream: constant %u is larger than its payload", i);
                want *= static_cast<uint64_t>(d);
            }
            HIPIE_REQUIRE(want == nbytes, HIPIE_NETWORK_NOT_READ, "plan stream: constant %u has %llu bytes for its shape, %llu stored", i,
                          (unsigned long long)want, (unsigned long long)nbytes);
            st = hipie_graph_constant(G, dtype, shape.data(), static_cast<int>(shape.size()), data, &id);
            break;
        }
        case OP_FAKE_QUANTIZE:
            arity(5);
            st = hipie_graph_fake_quantize(G, in[0], in[1], in[2], in[3], in[4], levels, dtype, &id);
            break;
        case OP_CONVOLUTION:
        case OP_GROUP_CONVOLUTION:
            arity(2);
            st = (op == OP_CONVOLUTION ? hipie_graph_convolution : hipie_graph_group_convolution)(
                G, in[0], in[1], pair(strides), pair(dilations), pair(pads_begin), pair(pads_end), &id);
            break;
        case OP_MATMUL:
            arity(2);
            st = hipie_graph_matmul(G, in[0], in[1], flags & F_TA, flags & F_TB, &id);
            break;
        case OP_ADD: case OP_MULTIPLY: case OP_SUBTRACT: case OP_PRELU:
            arity(2);
            st = hipie_graph_eltwise(G, op, in[0], in[1], &id);
            break;
        case OP_RELU: arity(1); st = hipie_graph_relu(G, in[0], &id); break;
        case OP_CLAMP: arity(1); st = hipie_graph_clamp(G, in[0], lo, hi, &id); break;
        case OP_SIGMOID: case OP_HSWISH: case OP_HSIGMOID: case OP_SWISH: arity(1); st = hipie_graph_activation(G, op, in[0], lo, &id); break;
        case OP_CONVERT: arity(1); st = hipie_graph_convert(G, in[0], dtype, &id); break;
        case OP_MAX_POOL:
            arity(1);
            st = hipie_graph_max_pool(G, in[0], pair(kernel), pair(strides), pair(pads_begin), pair(pads_end), flags & F_CEIL, &id);
            break;
        case OP_AVG_POOL:
            arity(1);
            st = hipie_graph_avg_pool(G, in[0], pair(kernel), pair(strides), pair(pads_begin), pair(pads_end), flags & F_EXCLUDE_PAD,
                                      flags & F_CEIL, dtype, &id);
            break;
        case OP_RESHAPE: arity(1); st = hipie_graph_reshape(G, in[0], shape.data(), static_cast<int>(shape.size()), &id); break;
        case OP_SOFTMAX:
            arity(1);
            HIPIE_REQUIRE(axes.size() == 1, HIPIE_NETWORK_NOT_READ, "plan stream: Softmax %u without an axis", i);
            st = hipie_graph_softmax(G, in[0], axes[0], &id);
            break;
        case OP_MVN:
            arity(1);
            st = hipie_graph_mvn(G, in[0], axes.data(), static_cast<int>(axes.size()), flags & F_NORM_VAR, eps, flags & F_EPS_INSIDE, &id);
            break;
        case OP_GELU: arity(1); st = hipie_graph_gelu(G, in[0], &id); break;
        case OP_TRANSPOSE: arity(1); st = hipie_graph_transpose(G, in[0], axes.data(), static_cast<int>(axes.size()), &id); break;
        case OP_GATHER:
            arity(2);
            HIPIE_REQUIRE(axes.size() == 1, HIPIE_NETWORK_NOT_READ, "plan stream: Gather %u without an axis", i);
            st = hipie_graph_gather(G, in[0], in[1], axes[0], &id);
            break;
        case OP_CONCAT:
            HIPIE_REQUIRE(axes.size() == 1 && !in.empty(), HIPIE_NETWORK_NOT_READ, "plan stream: Concat %u without an axis or inputs", i);
            st = hipie_graph_concat(G, in.data(), static_cast<int>(in.size()), axes[0], &id);
            break;
        case OP_SLICE:
            arity(1);
            HIPIE_REQUIRE(axes.size() == 3, HIPIE_NETWORK_NOT_READ, "plan stream: Slice %u without its bounds", i);
            st = hipie_graph_slice(G, in[0], axes[0], axes[1], axes[2], &id);
            break;
        case OP_RESULT: arity(1); st = hipie_graph_result(G, in[0], name.c_str()); break;
        default: fail(HIPIE_NETWORK_NOT_READ, "plan stream: node %u has unknown operation %d", i, op);
        }
        if (st != HIPIE_OK) {
            const std::string why = hipie_last_error();
            fail(HIPIE_NETWORK_NOT_READ, "plan stream: node %u (%s) is rejected: %s", i, op_name(op), why.c_str());
        }
        HIPIE_REQUIRE(G->nodes.size() == size_t(i) + 1 && id == static_cast<int>(i), HIPIE_UNEXPECTED, "plan stream: node numbering");
        GNode& n = G->nodes[i];
        HIPIE_REQUIRE(n.shape == shape && n.dtype == dtype, HIPIE_NETWORK_NOT_READ,
                      "plan stream: node %u (%s): the stored shape or type is not the inferred one", i, op_name(op));
        n.name = name;
    }
    HIPIE_REQUIRE(r.left == 0, HIPIE_NETWORK_NOT_READ, "plan stream: %zu bytes behind the last node", r.left);
    return g.release();
}

}  // namespace hipie

