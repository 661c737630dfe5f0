#include "hip_async_infer_request.hpp"

using namespace HipPlugin;

AsyncInferRequest::AsyncInferRequest(const InferRequest::Ptr& request, const InferenceEngine::ITaskExecutor::Ptr& taskExecutor,
                                     const InferenceEngine::ITaskExecutor::Ptr& waitExecutor, const InferenceEngine::ITaskExecutor::Ptr& callbackExecutor)
    : AsyncInferRequestThreadSafeDefault(request, taskExecutor, callbackExecutor), _request(request), _waitExecutor(waitExecutor) {
    // the device runs asynchronously to the host, so the stage that blocks has threads of its own: a stream executor
    // thread is free for the next request as soon as this one's work is queued
    // (template_async_infer_request.cpp:17-41 describes this split for remote devices)
    _pipeline = {
        {taskExecutor, [this] { _request->inferPreprocess(); _request->startPipeline(); }},
        {_waitExecutor, [this] { _request->waitPipeline(); }},
        {taskExecutor, [this] { _request->inferPostprocess(); }},
    };
}

AsyncInferRequest::~AsyncInferRequest() {
    // no stage may run on a destroyed request (template_async_infer_request.cpp:45-47)
    InferenceEngine::AsyncInferRequestThreadSafeDefault::StopAndWait();
}

void AsyncInferRequest::Cancel() {
    // marks the device-side request first, so that the wait stage ends with InferCancelled whichever stage is running
    _request->Cancel();
    InferenceEngine::AsyncInferRequestThreadSafeDefault::Cancel();
}
