// ExecutableNetwork: owns the compiled plan (hipie_plan) and creates requests over it
// (ie_iexecutable_network_internal.hpp:30-151, impl/ie_executable_network_thread_safe_default.hpp:23-69).
#pragma once

#include <cpp_interfaces/impl/ie_executable_network_thread_safe_default.hpp>

#include "hip_common.hpp"
#include "hip_plugin.hpp"

namespace HipPlugin {

class ExecutableNetwork : public InferenceEngine::ExecutableNetworkThreadSafeDefault {
public:
    ExecutableNetwork(const std::shared_ptr<const ngraph::Function>& function, const ConfigMap& config, const Plugin::Ptr& plugin);
    ExecutableNetwork(std::istream& model, const ConfigMap& config, const Plugin::Ptr& plugin);

    InferenceEngine::IInferRequestInternal::Ptr CreateInferRequestImpl(InferenceEngine::InputsDataMap networkInputs,
                                                                       InferenceEngine::OutputsDataMap networkOutputs) override;
    InferenceEngine::IInferRequestInternal::Ptr CreateInferRequest() override;
    InferenceEngine::Parameter GetMetric(const std::string& name) const override;
    InferenceEngine::Parameter GetConfig(const std::string& name) const override;
    void Export(std::ostream& model) override;
    InferenceEngine::CNNNetwork GetExecGraphInfo() override;

    hipie_plan* plan() const { return _plan.get(); }
    int device() const { return _device; }

private:
    void init_executor();
    std::string plan_text(bool metric, const std::string& name) const;

    PlanPtr _plan;
    ConfigMap _cfg;
    int _device = 0;
    Plugin::Ptr _hipPlugin;
};

}  // namespace HipPlugin
