// The plugin object: IInferencePlugin for the device name "HIP" (ie_iplugin_internal.hpp:86-302).
#pragma once

#include <cpp_interfaces/interface/ie_iexecutable_network_internal.hpp>
#include <cpp_interfaces/interface/ie_iplugin_internal.hpp>
#include <threading/ie_itask_executor.hpp>

#include "hip_common.hpp"

namespace HipPlugin {

class Plugin : public InferenceEngine::IInferencePlugin {
public:
    using Ptr = std::shared_ptr<Plugin>;

    Plugin();
    ~Plugin();

    void SetConfig(const std::map<std::string, std::string>& config) override;
    InferenceEngine::Parameter GetConfig(const std::string& name, const std::map<std::string, InferenceEngine::Parameter>& options) const override;
    InferenceEngine::Parameter GetMetric(const std::string& name, const std::map<std::string, InferenceEngine::Parameter>& options) const override;
    InferenceEngine::QueryNetworkResult QueryNetwork(const InferenceEngine::CNNNetwork& network,
                                                     const std::map<std::string, std::string>& config) const override;
    InferenceEngine::IExecutableNetworkInternal::Ptr LoadExeNetworkImpl(const InferenceEngine::CNNNetwork& network,
                                                                        const std::map<std::string, std::string>& config) override;
    InferenceEngine::IExecutableNetworkInternal::Ptr ImportNetwork(std::istream& model, const std::map<std::string, std::string>& config) override;
    void AddExtension(const std::shared_ptr<InferenceEngine::IExtension>& extension) override;

    // the plugin-wide config merged with a per-call one; DEVICE_ID picks the device (default 0)
    ConfigMap merged(const ConfigMap& config) const;
    static int device_of(const ConfigMap& config);

    InferenceEngine::ITaskExecutor::Ptr waitExecutor() const { return _waitExecutor; }

private:
    ConfigMap _cfg;
    InferenceEngine::ITaskExecutor::Ptr _waitExecutor;   // blocks in hipie_request_wait so that the stream executors do not
};

// CommonOptimizations, then the stock low-precision transformations with this device's restrictions (u8 activations,
// i8 weights, per-tensor activation quantization in front of convolutions): what LoadExeNetworkImpl and QueryNetwork
// both hand to the translator
std::shared_ptr<ngraph::Function> transform_network(const std::shared_ptr<const ngraph::Function>& function);

}  // namespace HipPlugin
