#include "hip_plugin.hpp"

#include <ie_metric_helpers.hpp>
#include <ie_plugin_config.hpp>
#include <threading/ie_executor_manager.hpp>

#include <sstream>
#include <unordered_set>

#include <ngraph/graph_util.hpp>
#include <ngraph/opsets/opset1.hpp>
#include <ngraph/pass/manager.hpp>
#include <low_precision/low_precision.hpp>
#include <transformations/common_optimizations/common_optimizations.hpp>
#include <transformations/rt_info/fused_names_attribute.hpp>

#include "function_to_graph.hpp"
#include "hip_executable_network.hpp"

using namespace HipPlugin;

namespace {

std::vector<std::string> split_words(const std::string& text) {
    std::istringstream in(text);
    std::vector<std::string> words;
    for (std::string w; in >> w;) words.push_back(w);
    return words;
}

std::string device_metric(int device, const char* name) {
    char buf[2048];
    check(hipie_get_metric(device, name, buf, sizeof buf), name);
    return buf;
}

}  // namespace

Plugin::Plugin() {
    _pluginName = "HIP";
    _waitExecutor = InferenceEngine::ExecutorManager::getInstance()->getIdleCPUStreamsExecutor({"HipWaitExecutor"});
}

Plugin::~Plugin() {
    // executors are cached process-wide by name: give them back (template_plugin.cpp:46-52)
    InferenceEngine::ExecutorManager::getInstance()->clear("HipStreamsExecutor");
    InferenceEngine::ExecutorManager::getInstance()->clear("HipWaitExecutor");
}

std::shared_ptr<ngraph::Function> HipPlugin::transform_network(const std::shared_ptr<const ngraph::Function>& function) {
    auto clone = ngraph::clone_function(*function);   // never mutate the caller's Function (template_plugin.cpp:60)
    ngraph::pass::Manager common;
    common.register_pass<ngraph::pass::CommonOptimizations>();
    common.run_passes(clone);

    using namespace ngraph::pass::low_precision;
    // the integer kernels multiply u8 (or zero-point-shifted u8) activations by i8 weights (mkldnn_plugin.cpp:316-338 sets
    // the same restrictions for the CPU plugin, which is why the post-LPT graphs of both devices look alike)
    const auto precisions = std::vector<OperationPrecisionRestriction>({
        OperationPrecisionRestriction::create<ngraph::opset1::Convolution>({{0, {ngraph::element::u8}}, {1, {ngraph::element::i8}}}),
        OperationPrecisionRestriction::create<ngraph::opset1::GroupConvolution>({{0, {ngraph::element::u8}}, {1, {ngraph::element::i8}}}),
    });
    const auto per_tensor = std::vector<OperationPerTensorQuantizationRestriction>({
        OperationPerTensorQuantizationRestriction::create<ngraph::opset1::Convolution>({0}),
    });
    ngraph::pass::Manager lpt;
    lpt.register_pass<LowPrecision>(precisions, per_tensor);
    lpt.run_passes(clone);
    return clone;
}

ConfigMap Plugin::merged(const ConfigMap& config) const {
    ConfigMap all = _cfg;
    for (const auto& kv : config) all[kv.first] = kv.second;
    return all;
}

int Plugin::device_of(const ConfigMap& config) {
    const auto it = config.find(CONFIG_KEY(DEVICE_ID));
    return it == config.end() || it->second.empty() ? 0 : std::stoi(it->second);
}

void Plugin::SetConfig(const ConfigMap& config) {
    // validated by compiling nothing: every key must be one the engine lists (template_config.cpp:16-39 throws NotFound)
    const auto known = split_words(device_metric(0, METRIC_KEY(SUPPORTED_CONFIG_KEYS)));
    for (const auto& kv : config)
        if (std::find(known.begin(), known.end(), kv.first) == known.end()) IE_THROW(NotFound) << "HIP plugin: unsupported config key " << kv.first;
    _cfg = merged(config);
}

InferenceEngine::Parameter Plugin::GetConfig(const std::string& name, const std::map<std::string, InferenceEngine::Parameter>&) const {
    const auto it = _cfg.find(name);
    if (it != _cfg.end()) return it->second;
    const auto known = split_words(device_metric(0, METRIC_KEY(SUPPORTED_CONFIG_KEYS)));
    if (std::find(known.begin(), known.end(), name) == known.end()) IE_THROW(NotFound) << "HIP plugin: unsupported config key " << name;
    return std::string();
}

InferenceEngine::Parameter Plugin::GetMetric(const std::string& name, const std::map<std::string, InferenceEngine::Parameter>& options) const {
    int device = device_of(_cfg);
    const auto id = options.find(CONFIG_KEY(DEVICE_ID));
    if (id != options.end()) device = std::stoi(id->second.as<std::string>());
    if (METRIC_KEY(SUPPORTED_METRICS) == name) {
        IE_SET_METRIC_RETURN(SUPPORTED_METRICS, split_words(device_metric(device, name.c_str())));
    } else if (METRIC_KEY(SUPPORTED_CONFIG_KEYS) == name) {
        IE_SET_METRIC_RETURN(SUPPORTED_CONFIG_KEYS, split_words(device_metric(device, name.c_str())));
    } else if (METRIC_KEY(AVAILABLE_DEVICES) == name) {
        IE_SET_METRIC_RETURN(AVAILABLE_DEVICES, split_words(device_metric(device, name.c_str())));
    } else if (METRIC_KEY(FULL_DEVICE_NAME) == name) {
        IE_SET_METRIC_RETURN(FULL_DEVICE_NAME, device_metric(device, name.c_str()));
    } else if (METRIC_KEY(IMPORT_EXPORT_SUPPORT) == name) {
        IE_SET_METRIC_RETURN(IMPORT_EXPORT_SUPPORT, device_metric(device, name.c_str()) == "YES");
    } else if (METRIC_KEY(DEVICE_ARCHITECTURE) == name) {
        IE_SET_METRIC_RETURN(DEVICE_ARCHITECTURE, device_metric(device, name.c_str()));
    } else if (METRIC_KEY(OPTIMIZATION_CAPABILITIES) == name) {
        IE_SET_METRIC_RETURN(OPTIMIZATION_CAPABILITIES, split_words(device_metric(device, name.c_str())));
    } else if (METRIC_KEY(RANGE_FOR_ASYNC_INFER_REQUESTS) == name) {
        const auto r = split_words(device_metric(device, name.c_str()));
        using uint = unsigned int;
        IE_SET_METRIC_RETURN(RANGE_FOR_ASYNC_INFER_REQUESTS,
                             std::make_tuple(uint(std::stoul(r.at(0))), uint(std::stoul(r.at(1))), uint(std::stoul(r.at(2)))));
    } else if (METRIC_KEY(RANGE_FOR_STREAMS) == name) {
        const auto r = split_words(device_metric(device, name.c_str()));
        using uint = unsigned int;
        IE_SET_METRIC_RETURN(RANGE_FOR_STREAMS, std::make_tuple(uint(std::stoul(r.at(0))), uint(std::stoul(r.at(1)))));
    }
    IE_THROW(NotFound) << "HIP plugin: unsupported metric " << name;
}

InferenceEngine::IExecutableNetworkInternal::Ptr Plugin::LoadExeNetworkImpl(const InferenceEngine::CNNNetwork& network, const ConfigMap& config) {
    const auto function = network.getFunction();
    if (!function) IE_THROW(NotImplemented) << "HIP plugin: only ngraph-based networks";
    return std::make_shared<ExecutableNetwork>(function, merged(config), std::static_pointer_cast<Plugin>(shared_from_this()));
}

InferenceEngine::IExecutableNetworkInternal::Ptr Plugin::ImportNetwork(std::istream& model, const ConfigMap& config) {
    return std::make_shared<ExecutableNetwork>(model, merged(config), std::static_pointer_cast<Plugin>(shared_from_this()));
}

InferenceEngine::QueryNetworkResult Plugin::QueryNetwork(const InferenceEngine::CNNNetwork& network, const ConfigMap&) const {
    InferenceEngine::QueryNetworkResult res;
    const auto function = network.getFunction();
    if (!function) IE_THROW(NotImplemented) << "HIP plugin: only ngraph-based networks";
    std::unordered_set<std::string> original;
    for (const auto& node : function->get_ops()) original.insert(node->get_friendly_name());

    // the same transformations as at load, then the engine's own answer per node of the transformed graph
    const auto transformed = transform_network(function);
    TranslatedGraph t = translate(transformed, true);
    std::vector<int> ok(t.node_names.size(), 0);
    if (!ok.empty()) check(hipie_query(t.graph.get(), ok.data(), static_cast<int>(ok.size()), nullptr), "hipie_query");
    std::unordered_set<std::string> bad_names(t.untranslated.begin(), t.untranslated.end());
    for (size_t i = 0; i < ok.size(); ++i)
        if (!ok[i]) bad_names.insert(t.node_names[i]);

    // a transformed node stands for the original nodes fused into it (template_plugin.cpp:139-152): an original node is
    // supported when every transformed node that carries its name is
    std::unordered_set<std::string> supported, unsupported;
    for (const auto& node : transformed->get_ops())
        for (const auto& fused : ngraph::getFusedNamesVector(node)) {
            if (!original.count(fused)) continue;
            (bad_names.count(node->get_friendly_name()) ? unsupported : supported).insert(fused);
        }
    for (const auto& name : unsupported) supported.erase(name);
    for (const auto& name : supported) res.supportedLayersMap.emplace(name, GetName());
    return res;
}

void Plugin::AddExtension(const std::shared_ptr<InferenceEngine::IExtension>&) {
    IE_THROW(NotImplemented);   // Core tolerates this (ie_core.cpp:697-719)
}

static const InferenceEngine::Version version = {{2, 1}, "hipie", "hipPlugin"};
IE_DEFINE_PLUGIN_CREATE_FUNCTION(Plugin, version)
