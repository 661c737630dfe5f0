#include "hip_executable_network.hpp"

#include <ie_metric_helpers.hpp>
#include <ie_plugin_config.hpp>
#include <threading/ie_executor_manager.hpp>

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

void ExecutableNetwork::Export(std::ostream& model) {
    size_t size = 0;
    check(hipie_plan_export(_plan.get(), nullptr, 0, &size), "hipie_plan_export");
    std::string bytes(size, '\0');
    check(hipie_plan_export(_plan.get(), &bytes[0], bytes.size(), &size), "hipie_plan_export");
    const std::uint64_t n = size;
    model.write(reinterpret_cast<const char*>(&n), sizeof n);
    model.write(bytes.data(), static_cast<std::streamsize>(size));
}
