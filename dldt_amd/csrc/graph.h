// Post-LPT graph description (what LoadExeNetworkImpl receives as an ngraph::Function) and the
// compiled plan: fused steps over one static HBM arena.
#pragma once
#include <map>
#include <memory>
#include <string>

#include "common.h"
#include "conv.h"
#include "pool.h"

namespace hipie {

enum OpKind {
    OP_PARAMETER = 0, OP_CONSTANT, OP_FAKE_QUANTIZE, OP_CONVOLUTION, OP_GROUP_CONVOLUTION, OP_MATMUL,
    OP_ADD, OP_MULTIPLY, OP_SUBTRACT, OP_RELU, OP_CLAMP, OP_CONVERT, OP_MAX_POOL, OP_AVG_POOL,
    OP_RESHAPE, OP_RESULT, OP_SOFTMAX, OP_MVN, OP_GELU, OP_TRANSPOSE, OP_GATHER, OP_CONCAT, OP_SLICE, OP_PRELU,
    OP_SIGMOID, OP_HSWISH, OP_HSIGMOID, OP_SWISH          // (Swish: beta in GNode::lo)
};
const char* op_name(int op);

struct GNode {
    int op = 0;
    std::string name;
    std::vector<int> in;
    int dtype = HIPIE_F32;            // element type of the output (HIPIE_U8 = plain u8 levels)
    std::vector<int64_t> shape;       // NCHW / [N, C] as in the reference
    std::vector<int64_t> strides, dilations, pads_begin, pads_end, kernel;
    int64_t levels = 0;
    int64_t depth = 0;                // planner only: depth D of the input of a convolution over three spatial dimensions
                                      // whose values are held as [N, C, D * H, W] (never part of a description)
    bool ta = false, tb = false, exclude_pad = false, ceil_mode = false;
    float lo = 0, hi = 0;
    std::vector<int64_t> axes;        // Softmax / Gather / Concat axis, MVN axes, Transpose order, Slice {axis, begin, end}
    bool normalize_variance = true, eps_inside_sqrt = true;
    float eps = 0;
    std::vector<uint8_t> data;        // constant payload
    std::vector<int> users;
    int64_t numel() const {
        int64_t n = 1;
        for (auto d : shape) n *= d;
        return n;
    }
    const float* f32() const { return reinterpret_cast<const float*>(data.data()); }
};

}  // namespace hipie

struct hipie_graph {
    std::vector<hipie::GNode> nodes;
    std::vector<int> params, results;
};

namespace hipie {
// the description as a byte stream (written to `dst` unless it is null; returns the byte count), and
// back (through the validating entry points; throws HIPIE_NETWORK_NOT_READ on anything malformed)
size_t serialize_graph(const hipie_graph& g, uint8_t* dst);
hipie_graph* deserialize_graph(const uint8_t* bytes, size_t size);
}  // namespace hipie
