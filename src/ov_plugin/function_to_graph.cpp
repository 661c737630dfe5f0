#include "function_to_graph.hpp"

#include <map>

#include <ngraph/opsets/opset1.hpp>
#include <ngraph/opsets/opset2.hpp>
#include <ngraph/opsets/opset6.hpp>
#include <ngraph/opsets/opset7.hpp>

namespace HipPlugin {
namespace {

int element_type(const ngraph::element::Type& t, const ngraph::Node& node) {
    if (t == ngraph::element::f32) return HIPIE_F32;
    if (t == ngraph::element::u8) return HIPIE_U8;
    if (t == ngraph::element::i8) return HIPIE_I8;
    if (t == ngraph::element::i32) return HIPIE_I32;
    IE_THROW(NotImplemented) << "HIP plugin: element type " << t << " of node " << node.get_friendly_name();
}

std::vector<int64_t> dims_of(const ngraph::Node& node) {
    const ngraph::PartialShape& ps = node.get_output_partial_shape(0);
    if (ps.is_dynamic()) IE_THROW(NotImplemented) << "HIP plugin: dynamic shape at " << node.get_friendly_name();
    const ngraph::Shape shape = ps.to_shape();
    return std::vector<int64_t>(shape.begin(), shape.end());
}

template <typename T>
std::vector<int64_t> as_i64(const T& v) {
    return std::vector<int64_t>(v.begin(), v.end());
}

// integer attribute carried by a Constant input (MVN axes, Transpose order, Gather axis)
std::vector<int64_t> constant_i64(const ngraph::Output<ngraph::Node>& value, const ngraph::Node& user) {
    const auto c = ngraph::as_type_ptr<ngraph::opset1::Constant>(value.get_node_shared_ptr());
    if (!c) IE_THROW(NotImplemented) << "HIP plugin: " << user.get_friendly_name() << " needs a constant attribute input";
    return c->cast_vector<int64_t>();
}

struct Translator {
    hipie_graph* g;
    TranslatedGraph& out;
    std::unordered_map<const ngraph::Node*, int> id_of;
    // a node with several outputs (Split, VariadicSplit) is one Slice per output: (node, output index) -> id;
    // id_of holds its first output's
    std::map<std::pair<const ngraph::Node*, size_t>, int> output_id;

    // An i64 / u64 Constant is skipped when it is met (most are attributes their users read: axes, orders, target
    // shapes).  One that a node takes as DATA - Gather indices, an integer table - is described here, on first use, as
    // the i32 constant the engine's integer inputs are (values that do not fit are refused).
    int in(const ngraph::Node& n, size_t i) {
        const ngraph::Node* producer = n.get_input_node_ptr(i);
        if (producer->get_output_size() > 1) {
            const auto part = output_id.find({producer, n.input_value(i).get_index()});
            if (part != output_id.end()) return part->second;
        }
        const auto it = id_of.find(producer);
        if (it != id_of.end()) return it->second;
        const auto c = ngraph::as_type_ptr<ngraph::opset1::Constant>(n.input_value(i).get_node_shared_ptr());
        if (c && (c->get_element_type() == ngraph::element::i64 || c->get_element_type() == ngraph::element::u64)) {
            const std::vector<int64_t> wide = c->cast_vector<int64_t>();
            std::vector<int32_t> narrow(wide.size());
            for (size_t k = 0; k < wide.size(); ++k) {
                if (wide[k] < INT32_MIN || wide[k] > INT32_MAX)
                    IE_THROW(NotImplemented) << "HIP plugin: 64-bit constant " << c->get_friendly_name() << " does not fit 32-bit integers";
                narrow[k] = static_cast<int32_t>(wide[k]);
            }
            const auto d = as_i64(c->get_shape());
            int id = -1;
            check(hipie_graph_constant(g, HIPIE_I32, d.data(), static_cast<int>(d.size()), narrow.data(), &id), "hipie_graph_constant");
            done(*c, id);
            return id;
        }
        IE_THROW(NotImplemented) << "HIP plugin: input " << i << " of " << n.get_friendly_name() << " was not translated";
    }
    void done(const ngraph::Node& n, int id) {
        id_of[&n] = id;
        check(hipie_graph_set_name(g, id, n.get_friendly_name().c_str()), "hipie_graph_set_name");
        if (out.node_names.size() <= static_cast<size_t>(id)) out.node_names.resize(id + 1);
        out.node_names[id] = n.get_friendly_name();
    }

    // returns false when there is no call for this node type
    bool node(const std::shared_ptr<ngraph::Node>& node) {
        const ngraph::Node& n = *node;
        int id = -1;
        if (const auto p = ngraph::as_type_ptr<ngraph::opset1::Parameter>(node)) {
            const auto d = dims_of(n);
            check(hipie_graph_parameter(g, n.get_friendly_name().c_str(), element_type(p->get_element_type(), n), d.data(),
                                        static_cast<int>(d.size()), &id), "hipie_graph_parameter");
        } else if (const auto c = ngraph::as_type_ptr<ngraph::opset1::Constant>(node)) {
            const auto& t = c->get_element_type();
            if (t == ngraph::element::i64 || t == ngraph::element::u64) return true;   // attribute inputs: read by their users
            const auto d = as_i64(c->get_shape());
            check(hipie_graph_constant(g, element_type(t, n), d.data(), static_cast<int>(d.size()), c->get_data_ptr(), &id),
                  "hipie_graph_constant");
        } else if (const auto fq = ngraph::as_type_ptr<ngraph::opset1::FakeQuantize>(node)) {
            // TypeRelaxed<FakeQuantize> keeps the type_info of FakeQuantize; its output type says u8 / i8 / f32
            check(hipie_graph_fake_quantize(g, in(n, 0), in(n, 1), in(n, 2), in(n, 3), in(n, 4), static_cast<int64_t>(fq->get_levels()),
                                            element_type(n.get_output_element_type(0), n), &id), "hipie_graph_fake_quantize");
        } else if (const auto conv = ngraph::as_type_ptr<ngraph::opset1::Convolution>(node)) {
            const auto s = as_i64(conv->get_strides()), dl = as_i64(conv->get_dilations());
            const auto pb = as_i64(conv->get_pads_begin()), pe = as_i64(conv->get_pads_end());
            if (s.size() < 1 || s.size() > 3) IE_THROW(NotImplemented) << "HIP plugin: " << n.get_friendly_name() << " is a convolution over " << s.size() << " spatial dimensions";
            check(hipie_graph_convolution(g, in(n, 0), in(n, 1), s.data(), dl.data(), pb.data(), pe.data(), &id), "hipie_graph_convolution");
        } else if (const auto gconv = ngraph::as_type_ptr<ngraph::opset1::GroupConvolution>(node)) {
            const auto s = as_i64(gconv->get_strides()), dl = as_i64(gconv->get_dilations());
            const auto pb = as_i64(gconv->get_pads_begin()), pe = as_i64(gconv->get_pads_end());
            if (s.size() < 1 || s.size() > 3) IE_THROW(NotImplemented) << "HIP plugin: " << n.get_friendly_name() << " is a convolution over " << s.size() << " spatial dimensions";
            check(hipie_graph_group_convolution(g, in(n, 0), in(n, 1), s.data(), dl.data(), pb.data(), pe.data(), &id),
                  "hipie_graph_group_convolution");
        } else if (const auto mm = ngraph::as_type_ptr<ngraph::opset1::MatMul>(node)) {
            check(hipie_graph_matmul(g, in(n, 0), in(n, 1), mm->get_transpose_a(), mm->get_transpose_b(), &id), "hipie_graph_matmul");
        } else if (ngraph::is_type<ngraph::opset1::Add>(node)) {
            check(hipie_graph_eltwise(g, HIPIE_OP_ADD, in(n, 0), in(n, 1), &id), "hipie_graph_eltwise");
        } else if (ngraph::is_type<ngraph::opset1::Multiply>(node)) {
            check(hipie_graph_eltwise(g, HIPIE_OP_MULTIPLY, in(n, 0), in(n, 1), &id), "hipie_graph_eltwise");
        } else if (ngraph::is_type<ngraph::opset1::Subtract>(node)) {
            check(hipie_graph_eltwise(g, HIPIE_OP_SUBTRACT, in(n, 0), in(n, 1), &id), "hipie_graph_eltwise");
        } else if (ngraph::is_type<ngraph::opset1::Sigmoid>(node)) {
            check(hipie_graph_activation(g, HIPIE_OP_SIGMOID, in(n, 0), 1.0f, &id), "hipie_graph_activation");
        } else if (ngraph::is_type<ngraph::opset7::HSwish>(node)) {
            check(hipie_graph_activation(g, HIPIE_OP_HSWISH, in(n, 0), 1.0f, &id), "hipie_graph_activation");
        } else if (ngraph::is_type<ngraph::opset7::HSigmoid>(node)) {
            check(hipie_graph_activation(g, HIPIE_OP_HSIGMOID, in(n, 0), 1.0f, &id), "hipie_graph_activation");
        } else if (ngraph::is_type<ngraph::opset7::Swish>(node)) {
            float beta = 1.0f;
            if (n.get_input_size() > 1) {
                const auto b = ngraph::as_type_ptr<ngraph::opset1::Constant>(n.input_value(1).get_node_shared_ptr());
                if (!b || ngraph::shape_size(b->get_shape()) != 1)
                    IE_THROW(NotImplemented) << "HIP plugin: " << n.get_friendly_name() << ": Swish with a beta that is not a constant scalar";
                beta = b->cast_vector<float>().at(0);
            }
            check(hipie_graph_activation(g, HIPIE_OP_SWISH, in(n, 0), beta, &id), "hipie_graph_activation");
        } else if (ngraph::is_type<ngraph::opset1::PRelu>(node)) {
            check(hipie_graph_eltwise(g, HIPIE_OP_PRELU, in(n, 0), in(n, 1), &id), "hipie_graph_eltwise");
        } else if (ngraph::is_type<ngraph::opset1::Relu>(node)) {
            check(hipie_graph_relu(g, in(n, 0), &id), "hipie_graph_relu");
        } else if (const auto cl = ngraph::as_type_ptr<ngraph::opset1::Clamp>(node)) {
            check(hipie_graph_clamp(g, in(n, 0), static_cast<float>(cl->get_min()), static_cast<float>(cl->get_max()), &id), "hipie_graph_clamp");
        } else if (ngraph::is_type<ngraph::opset1::Convert>(node)) {
            check(hipie_graph_convert(g, in(n, 0), element_type(n.get_output_element_type(0), n), &id), "hipie_graph_convert");
        } else if (const auto mp = ngraph::as_type_ptr<ngraph::opset1::MaxPool>(node)) {
            const auto k = as_i64(mp->get_kernel()), s = as_i64(mp->get_strides());
            const auto pb = as_i64(mp->get_pads_begin()), pe = as_i64(mp->get_pads_end());
            if (k.size() != 2 && k.size() != 1) IE_THROW(NotImplemented) << "HIP plugin: " << n.get_friendly_name() << " is a pooling over three spatial dimensions";
            check(hipie_graph_max_pool(g, in(n, 0), k.data(), s.data(), pb.data(), pe.data(),
                                       mp->get_rounding_type() == ngraph::op::RoundingType::CEIL, &id), "hipie_graph_max_pool");
        } else if (const auto ap = ngraph::as_type_ptr<ngraph::opset1::AvgPool>(node)) {
            const auto k = as_i64(ap->get_kernel()), s = as_i64(ap->get_strides());
            const auto pb = as_i64(ap->get_pads_begin()), pe = as_i64(ap->get_pads_end());
            if (k.size() != 2 && k.size() != 1) IE_THROW(NotImplemented) << "HIP plugin: " << n.get_friendly_name() << " is a pooling over three spatial dimensions";
            check(hipie_graph_avg_pool(g, in(n, 0), k.data(), s.data(), pb.data(), pe.data(), ap->get_exclude_pad(),
                                       ap->get_rounding_type() == ngraph::op::RoundingType::CEIL,
                                       element_type(n.get_output_element_type(0), n), &id), "hipie_graph_avg_pool");
        } else if (ngraph::is_type<ngraph::opset1::Reshape>(node) || ngraph::is_type<ngraph::opset1::Squeeze>(node) ||
                   ngraph::is_type<ngraph::opset1::Unsqueeze>(node)) {
            const auto d = dims_of(n);
            check(hipie_graph_reshape(g, in(n, 0), d.data(), static_cast<int>(d.size()), &id), "hipie_graph_reshape");
        } else if (const auto sm = ngraph::as_type_ptr<ngraph::opset1::Softmax>(node)) {
            check(hipie_graph_softmax(g, in(n, 0), static_cast<int64_t>(sm->get_axis()), &id), "hipie_graph_softmax");
        } else if (const auto mvn = ngraph::as_type_ptr<ngraph::opset6::MVN>(node)) {
            const auto axes = constant_i64(n.input_value(1), n);
            check(hipie_graph_mvn(g, in(n, 0), axes.data(), static_cast<int>(axes.size()), mvn->get_normalize_variance(), mvn->get_eps(),
                                  mvn->get_eps_mode() == ngraph::op::MVNEpsMode::INSIDE_SQRT, &id), "hipie_graph_mvn");
        } else if (const auto gelu7 = ngraph::as_type_ptr<ngraph::opset7::Gelu>(node)) {
            if (gelu7->get_approximation_mode() != ngraph::op::GeluApproximationMode::ERF)
                IE_THROW(NotImplemented) << "HIP plugin: " << n.get_friendly_name() << ": only the ERF form of Gelu";
            check(hipie_graph_gelu(g, in(n, 0), &id), "hipie_graph_gelu");
        } else if (ngraph::is_type<ngraph::opset2::Gelu>(node)) {
            check(hipie_graph_gelu(g, in(n, 0), &id), "hipie_graph_gelu");
        } else if (ngraph::is_type<ngraph::opset1::Transpose>(node)) {
            const auto order = constant_i64(n.input_value(1), n);
            check(hipie_graph_transpose(g, in(n, 0), order.data(), static_cast<int>(order.size()), &id), "hipie_graph_transpose");
        } else if (ngraph::is_type<ngraph::opset1::Gather>(node)) {
            const auto axis = constant_i64(n.input_value(2), n);
            check(hipie_graph_gather(g, in(n, 0), in(n, 1), axis.at(0), &id), "hipie_graph_gather");
        } else if (ngraph::is_type<ngraph::opset1::Split>(node) || ngraph::is_type<ngraph::opset1::VariadicSplit>(node)) {
            // every output is the box reference::split takes for it: consecutive extents along the axis
            const auto axis_c = constant_i64(n.input_value(1), n);
            const int64_t rank = static_cast<int64_t>(n.get_input_shape(0).size());
            const int64_t axis = axis_c.at(0) < 0 ? axis_c.at(0) + rank : axis_c.at(0);
            const int x = in(n, 0);
            int64_t begin = 0;
            for (size_t k = 0; k < n.get_output_size(); ++k) {
                const int64_t extent = static_cast<int64_t>(n.get_output_shape(k).at(static_cast<size_t>(axis)));
                int part = -1;
                check(hipie_graph_slice(g, x, axis, begin, begin + extent, &part), "hipie_graph_slice");
                output_id[{&n, k}] = part;
                const std::string name = n.get_friendly_name() + '.' + std::to_string(k);
                check(hipie_graph_set_name(g, part, name.c_str()), "hipie_graph_set_name");
                if (out.node_names.size() <= static_cast<size_t>(part)) out.node_names.resize(part + 1);
                out.node_names[part] = n.get_friendly_name();
                if (k == 0) id_of[&n] = part;
                begin += extent;
            }
            return true;
        } else if (const auto concat = ngraph::as_type_ptr<const ngraph::opset1::Concat>(node)) {
            std::vector<int> inputs;
            for (size_t i = 0; i < n.get_input_size(); ++i) inputs.push_back(in(n, i));
            check(hipie_graph_concat(g, inputs.data(), static_cast<int>(inputs.size()), concat->get_axis(), &id), "hipie_graph_concat");
        } else if (ngraph::is_type<ngraph::opset1::Result>(node)) {
            // the request's output is named after the producer (template_executable_network.cpp:100-110)
            const auto producer = n.input_value(0);
            std::string name = producer.get_node()->get_friendly_name();
            if (producer.get_node()->get_output_size() > 1) name += '.' + std::to_string(producer.get_index());
            check(hipie_graph_result(g, in(n, 0), name.c_str()), "hipie_graph_result");
            return true;
        } else {
            return false;
        }
        done(n, id);
        return true;
    }
};

}  // namespace

TranslatedGraph translate(const std::shared_ptr<const ngraph::Function>& function, bool tolerate_unknown) {
    TranslatedGraph out;
    hipie_graph* raw = nullptr;
    check(hipie_graph_create(&raw), "hipie_graph_create");
    out.graph.reset(raw);
    Translator t{raw, out, {}};
    for (const auto& node : function->get_ordered_ops()) {
        bool usable = true;
        for (size_t i = 0; usable && i < node->get_input_size(); ++i) {
            const ngraph::Node* producer = node->get_input_node_ptr(i);
            const bool attribute = ngraph::is_type<ngraph::opset1::Constant>(producer) &&
                                   (producer->get_output_element_type(0) == ngraph::element::i64 ||
                                    producer->get_output_element_type(0) == ngraph::element::u64);
            usable = attribute || t.id_of.count(producer) != 0;
        }
        if (usable) {
            // QueryNetwork (tolerate_unknown) wants a verdict per node, as the template plugin gives one
            // (template_plugin.cpp:117-195): a node the helpers refuse - an element type, a dynamic shape, a 3-D
            // convolution, an attribute that is not constant, a description hipie_graph_* rejects - is reported
            // untranslated like a node of an unknown type, and so is everything that reads it
            if (!tolerate_unknown) {
                if (t.node(node)) continue;
            } else {
                try {
                    if (t.node(node)) continue;
                } catch (const InferenceEngine::Exception&) {
                }
            }
        }
        if (!tolerate_unknown)
            IE_THROW(NotImplemented) << "HIP plugin: no kernel for node " << node->get_friendly_name() << " (" << node->get_type_name() << ")";
        out.untranslated.push_back(node->get_friendly_name());
    }
    return out;
}

}  // namespace HipPlugin
