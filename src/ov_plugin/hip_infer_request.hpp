// InferRequest: the blobs of one request and one hipie_request (own stream, own activation arena) behind them
// (ie_iinfer_request_internal.hpp:28-240).
#pragma once

#include <cpp_interfaces/interface/ie_iinfer_request_internal.hpp>

#include "hip_common.hpp"

namespace HipPlugin {

class ExecutableNetwork;

class InferRequest : public InferenceEngine::IInferRequestInternal {
public:
    using Ptr = std::shared_ptr<InferRequest>;

    InferRequest(const InferenceEngine::InputsDataMap& networkInputs, const InferenceEngine::OutputsDataMap& networkOutputs,
                 const std::shared_ptr<ExecutableNetwork>& network);

    void InferImpl() override;
    void Cancel() override;
    std::map<std::string, InferenceEngine::InferenceEngineProfileInfo> GetPerformanceCounts() const override;

    // the stages of the asynchronous pipeline (hip_async_infer_request.cpp)
    void inferPreprocess();    // user blobs -> page-locked blobs of the plan's own types, in plan order
    void startPipeline();      // hipie_request_start: copies and kernels queued on the request's stream
    void waitPipeline();       // hipie_request_wait: blocks until the stream has drained
    void inferPostprocess();   // page-locked results -> user blobs of another precision

private:
    struct Port {
        std::string name;
        int dtype = 0;
        InferenceEngine::Blob::Ptr staged;   // page-locked, of the plan's type and dense NCHW
    };

    void describe_ports(bool outputs);

    std::shared_ptr<ExecutableNetwork> _network;
    RequestPtr _request;
    std::vector<Port> _in, _out;
    std::vector<const void*> _in_ptrs;
    std::vector<void*> _out_ptrs;
};

}  // namespace HipPlugin
