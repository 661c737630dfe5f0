#include "hip_executable_network.hpp"

#include <exec_graph_info.hpp>
#include <ie_metric_helpers.hpp>
#include <ie_plugin_config.hpp>
#include <threading/ie_executor_manager.hpp>

#include <ngraph/function.hpp>
#include <ngraph/op/parameter.hpp>
#include <ngraph/op/result.hpp>
#include <ngraph/variant.hpp>

#include <sstream>

#include "function_to_graph.hpp"
#include "hip_async_infer_request.hpp"
#include "hip_infer_request.hpp"

using namespace HipPlugin;

namespace {

// any failure of the compilation library leaves as an InferenceEngine exception (template_executable_network.cpp:29-39)
template <typename F>
void as_ie_exception(F&& body) {
    try {
        body();
    } catch (const InferenceEngine::Exception&) {
        throw;
    } catch (const std::exception& e) {
        IE_THROW(Unexpected) << "HIP plugin: " << e.what();
    } catch (...) {
        IE_THROW(Unexpected) << "HIP plugin: unknown exception";
    }
}

}  // namespace

ExecutableNetwork::ExecutableNetwork(const std::shared_ptr<const ngraph::Function>& function, const ConfigMap& config, const Plugin::Ptr& plugin)
    : InferenceEngine::ExecutableNetworkThreadSafeDefault(nullptr, nullptr), _cfg(config), _device(Plugin::device_of(config)), _hipPlugin(plugin) {
    as_ie_exception([&] {
        const auto transformed = transform_network(function);
        TranslatedGraph t = translate(transformed, false);
        ConfigMap cfg = _cfg;
        cfg["NETWORK_NAME"] = function->get_friendly_name();
        const ConfigArrays arrays(cfg);
        hipie_plan* raw = nullptr;
        check(hipie_compile_opts(t.graph.get(), _device, arrays.keys.data(), arrays.values.data(), static_cast<int>(arrays.keys.size()), &raw),
              "hipie_compile_opts");
        _plan.reset(raw);
        init_executor();
    });
}

ExecutableNetwork::ExecutableNetwork(std::istream& model, const ConfigMap& config, const Plugin::Ptr& plugin)
    : InferenceEngine::ExecutableNetworkThreadSafeDefault(nullptr, nullptr), _cfg(config), _device(Plugin::device_of(config)), _hipPlugin(plugin) {
    as_ie_exception([&] {
        // the stream holds one exported plan behind its byte count (Export below)
        std::uint64_t size = 0;
        model.read(reinterpret_cast<char*>(&size), sizeof size);
        std::string bytes(static_cast<size_t>(size), '\0');
        model.read(&bytes[0], static_cast<std::streamsize>(size));
        if (!model) IE_THROW(NetworkNotRead) << "HIP plugin: truncated model stream";
        hipie_plan* raw = nullptr;
        check(hipie_plan_import(bytes.data(), bytes.size(), _device, &raw), "hipie_plan_import");
        _plan.reset(raw);
        // the request blobs are described by the plan itself
        InferenceEngine::InputsDataMap inputs;
        InferenceEngine::OutputsDataMap outputs;
        for (int is_out = 0; is_out < 2; ++is_out) {
            const int n = is_out ? hipie_plan_num_outputs(raw) : hipie_plan_num_inputs(raw);
            for (int i = 0; i < n; ++i) {
                char name[256];
                int dtype = 0, rank = 0;
                int64_t dims[8];
                check(hipie_plan_io_desc(raw, is_out, i, name, sizeof name, &dtype, dims, &rank), "hipie_plan_io_desc");
                const InferenceEngine::SizeVector shape(dims, dims + rank);
                const auto precision = dtype == HIPIE_F32 ? InferenceEngine::Precision::FP32
                                                          : (dtype == HIPIE_I32 ? InferenceEngine::Precision::I32 : InferenceEngine::Precision::U8);
                const auto data = std::make_shared<InferenceEngine::Data>(
                    name, InferenceEngine::TensorDesc(precision, shape, InferenceEngine::TensorDesc::getLayoutByDims(shape)));
                if (is_out) {
                    outputs[name] = data;
                } else {
                    auto info = std::make_shared<InferenceEngine::InputInfo>();
                    info->setInputData(data);
                    inputs[name] = info;
                }
            }
        }
        setNetworkInputs(inputs);
        setNetworkOutputs(outputs);
        SetPointerToPlugin(_hipPlugin->shared_from_this());
        init_executor();
    });
}

void ExecutableNetwork::init_executor() {
    // one executor thread per request in flight: the threads only enqueue work and hand over to the wait executor
    auto cfg = InferenceEngine::IStreamsExecutor::Config::MakeDefaultMultiThreaded(InferenceEngine::IStreamsExecutor::Config {});
    cfg._name = "HipStreamsExecutor";
    cfg._streams = std::stoi(plan_text(true, METRIC_KEY(OPTIMAL_NUMBER_OF_INFER_REQUESTS)));
    _taskExecutor = InferenceEngine::ExecutorManager::getInstance()->getIdleCPUStreamsExecutor(cfg);
}

std::string ExecutableNetwork::plan_text(bool metric, const std::string& name) const {
    char buf[2048];
    check(metric ? hipie_plan_get_metric(_plan.get(), name.c_str(), buf, sizeof buf) : hipie_plan_get_config(_plan.get(), name.c_str(), buf, sizeof buf),
          name.c_str());
    return buf;
}

InferenceEngine::IInferRequestInternal::Ptr ExecutableNetwork::CreateInferRequestImpl(InferenceEngine::InputsDataMap networkInputs,
                                                                                      InferenceEngine::OutputsDataMap networkOutputs) {
    return std::make_shared<InferRequest>(networkInputs, networkOutputs, std::static_pointer_cast<ExecutableNetwork>(shared_from_this()));
}

InferenceEngine::IInferRequestInternal::Ptr ExecutableNetwork::CreateInferRequest() {
    auto sync = std::static_pointer_cast<InferRequest>(CreateInferRequestImpl(_networkInputs, _networkOutputs));
    return std::make_shared<AsyncInferRequest>(sync, _taskExecutor, _hipPlugin->waitExecutor(), _callbackExecutor);
}

InferenceEngine::Parameter ExecutableNetwork::GetMetric(const std::string& name) const {
    auto words = [&](const std::string& text) {
        std::istringstream in(text);
        std::vector<std::string> out;
        for (std::string w; in >> w;) out.push_back(w);
        return out;
    };
    if (EXEC_NETWORK_METRIC_KEY(SUPPORTED_METRICS) == name) {
        IE_SET_METRIC_RETURN(SUPPORTED_METRICS, words(plan_text(true, name)));
    } else if (EXEC_NETWORK_METRIC_KEY(SUPPORTED_CONFIG_KEYS) == name) {
        IE_SET_METRIC_RETURN(SUPPORTED_CONFIG_KEYS, words(plan_text(true, name)));
    } else if (EXEC_NETWORK_METRIC_KEY(NETWORK_NAME) == name) {
        IE_SET_METRIC_RETURN(NETWORK_NAME, plan_text(true, name));
    } else if (EXEC_NETWORK_METRIC_KEY(OPTIMAL_NUMBER_OF_INFER_REQUESTS) == name) {
        IE_SET_METRIC_RETURN(OPTIMAL_NUMBER_OF_INFER_REQUESTS, static_cast<unsigned int>(std::stoul(plan_text(true, name))));
    }
    IE_THROW(NotFound) << "HIP plugin: unsupported ExecutableNetwork metric " << name;
}

InferenceEngine::Parameter ExecutableNetwork::GetConfig(const std::string& name) const {
    return plan_text(false, name);
}

// The executed graph (ie_iexecutable_network_internal.hpp:87, exec_graph_info.hpp:34-76): one ExecutionNode per step of
// the plan - a fused kernel - carrying the attributes of hipie_plan_step_rt_info under the reference's keys, wired by
// hipie_plan_step_sources; graph inputs are Parameters, steps of layer type "Result" become Results.  The CPU plugin
// builds its own the same way (mkldnn_plugin/mkldnn_graph_dumper.cpp:115-213).
InferenceEngine::CNNNetwork ExecutableNetwork::GetExecGraphInfo() {
    namespace info = ExecGraphInfoSerialization;
    hipie_plan* plan = _plan.get();
    auto text = [&](int step, const char* key) {
        char buf[4096];
        check(hipie_plan_step_rt_info(plan, step, key, buf, sizeof buf), key);
        return std::string(buf);
    };
    auto precision_of = [](const std::string& p) {
        if (p == "U8") return ngraph::element::u8;
        if (p == "I8") return ngraph::element::i8;
        if (p == "I32") return ngraph::element::i32;
        return ngraph::element::f32;
    };
    auto dims_of = [](const std::string& csv) {
        ngraph::Shape shape;
        std::istringstream in(csv);
        for (std::string d; std::getline(in, d, ',');) shape.push_back(static_cast<size_t>(std::stoull(d)));
        return shape;
    };
    ngraph::ParameterVector params;
    for (int i = 0; i < hipie_plan_num_inputs(plan); ++i) {
        char name[256];
        int dtype = 0, rank = 0;
        int64_t dims[8];
        check(hipie_plan_io_desc(plan, 0, i, name, sizeof name, &dtype, dims, &rank), "hipie_plan_io_desc");
        const auto et = dtype == HIPIE_F32 ? ngraph::element::f32 : (dtype == HIPIE_I32 ? ngraph::element::i32 : ngraph::element::u8);
        auto p = std::make_shared<ngraph::op::Parameter>(et, ngraph::Shape(dims, dims + rank));
        p->set_friendly_name(name);
        params.push_back(p);
    }
    ngraph::ResultVector results;
    std::vector<std::shared_ptr<ngraph::Node>> nodes;
    const int n_steps = hipie_plan_num_steps(plan);
    for (int s = 0; s < n_steps; ++s) {
        int count = 0;
        check(hipie_plan_step_sources(plan, s, nullptr, 0, &count), "hipie_plan_step_sources");
        std::vector<int> src(static_cast<size_t>(count));
        if (count > 0) check(hipie_plan_step_sources(plan, s, src.data(), count, &count), "hipie_plan_step_sources");
        ngraph::OutputVector inputs;
        for (int from : src) inputs.push_back(from >= 0 ? nodes[static_cast<size_t>(from)]->output(0) : params[static_cast<size_t>(-1 - from)]->output(0));
        char name[256], type[64];
        int64_t macs = 0, bytes = 0;
        check(hipie_plan_step_info(plan, s, name, sizeof name, type, sizeof type, &macs, &bytes), "hipie_plan_step_info");
        std::shared_ptr<ngraph::Node> node;
        if (std::string(type) == "Result" && !inputs.empty()) {
            results.push_back(std::make_shared<ngraph::op::Result>(inputs.back()));
            node = results.back();
        } else {
            node = std::make_shared<info::ExecutionNode>(inputs, 1);
            node->set_output_type(0, precision_of(text(s, info::OUTPUT_PRECISIONS)), ngraph::PartialShape(dims_of(text(s, "outputDims"))));
        }
        for (const char* key : {info::ORIGINAL_NAMES, info::IMPL_TYPE, info::OUTPUT_PRECISIONS, info::OUTPUT_LAYOUTS, info::EXECUTION_ORDER,
                                info::LAYER_TYPE, info::RUNTIME_PRECISION})
            node->get_rt_info()[key] = std::make_shared<ngraph::VariantWrapper<std::string>>(text(s, key));
        // (execTimeMcs belongs to a request's counters, GetPerformanceCounts; a plan that has not run reports none)
        node->get_rt_info()[info::PERF_COUNTER] = std::make_shared<ngraph::VariantWrapper<std::string>>("not_executed");
        node->set_friendly_name(name);
        nodes.push_back(node);
    }
    if (results.empty()) IE_THROW() << "HIP plugin: the plan has no Result step";
    return InferenceEngine::CNNNetwork(std::make_shared<ngraph::Function>(results, params, plan_text(true, EXEC_NETWORK_METRIC_KEY(NETWORK_NAME))));
}

void ExecutableNetwork::Export(std::ostream& model) {
    size_t size = 0;
    check(hipie_plan_export(_plan.get(), nullptr, 0, &size), "hipie_plan_export");
    std::string bytes(size, '\0');
    check(hipie_plan_export(_plan.get(), &bytes[0], bytes.size(), &size), "hipie_plan_export");
    const std::uint64_t n = size;
    model.write(reinterpret_cast<const char*>(&n), sizeof n);
    model.write(bytes.data(), static_cast<std::streamsize>(size));
}
