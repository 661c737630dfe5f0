// ngraph::Function (after CommonOptimizations and the low-precision transformations) -> hipie_graph: one
// hipie_graph_* call per node of Function::get_ordered_ops().
#pragma once

#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include <ngraph/function.hpp>

#include "hip_common.hpp"

namespace HipPlugin {

struct TranslatedGraph {
    GraphPtr graph;
    // graph node id -> friendly name of the ngraph node it stands for (for QueryNetwork), in id order
    std::vector<std::string> node_names;
    // nodes the translator itself has no call for (their friendly names); the graph then lacks them and what they feed
    std::vector<std::string> untranslated;
};

// throws NotImplemented for a node without a hipie_graph_* counterpart unless `tolerate_unknown` (QueryNetwork)
TranslatedGraph translate(const std::shared_ptr<const ngraph::Function>& function, bool tolerate_unknown);

}  // namespace HipPlugin
