// AsyncInferRequest: StartAsync / Wait / Cancel over a three-stage pipeline
// (impl/ie_infer_async_request_thread_safe_default.hpp:42-267).
#pragma once

#include <cpp_interfaces/impl/ie_infer_async_request_thread_safe_default.hpp>

#include "hip_infer_request.hpp"

namespace HipPlugin {

class AsyncInferRequest : public InferenceEngine::AsyncInferRequestThreadSafeDefault {
public:
    AsyncInferRequest(const InferRequest::Ptr& request, const InferenceEngine::ITaskExecutor::Ptr& taskExecutor,
                      const InferenceEngine::ITaskExecutor::Ptr& waitExecutor, const InferenceEngine::ITaskExecutor::Ptr& callbackExecutor);
    ~AsyncInferRequest();

    void Cancel() override;

private:
    InferRequest::Ptr _request;
    InferenceEngine::ITaskExecutor::Ptr _waitExecutor;
};

}  // namespace HipPlugin
