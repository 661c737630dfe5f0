// "HIP" device plugin for the OpenVINO 2021.4 Inference Engine: the thin adapter between the plugin API
// (inference-engine/src/plugin_api) and the engine's C ABI (include/hipie.h).  Everything that computes lives
// behind that ABI in libhipie.so; these files translate types, errors and lifetimes.
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include <ie_common.h>

#include "hipie.h"

namespace HipPlugin {

// hipie_status -> the InferenceEngine exception of the same meaning (ie_common.h:231-249, 317-365): no status
// code ever leaves the plugin as an integer
[[noreturn]] inline void throw_status(int status, const std::string& what) {
    const std::string text = what + ": " + hipie_last_error();
    switch (status) {
    case HIPIE_NOT_IMPLEMENTED: IE_THROW(NotImplemented) << text;
    case HIPIE_NETWORK_NOT_LOADED: IE_THROW(NetworkNotLoaded) << text;
    case HIPIE_PARAMETER_MISMATCH: IE_THROW(ParameterMismatch) << text;
    case HIPIE_NOT_FOUND: IE_THROW(NotFound) << text;
    case HIPIE_OUT_OF_BOUNDS: IE_THROW(OutOfBounds) << text;
    case HIPIE_UNEXPECTED: IE_THROW(Unexpected) << text;
    case HIPIE_REQUEST_BUSY: IE_THROW(RequestBusy) << text;
    case HIPIE_RESULT_NOT_READY: IE_THROW(ResultNotReady) << text;
    case HIPIE_NOT_ALLOCATED: IE_THROW(NotAllocated) << text;
    case HIPIE_INFER_NOT_STARTED: IE_THROW(InferNotStarted) << text;
    case HIPIE_NETWORK_NOT_READ: IE_THROW(NetworkNotRead) << text;
    case HIPIE_INFER_CANCELLED: IE_THROW(InferCancelled) << text;
    default: IE_THROW(GeneralError) << text;
    }
}

inline void check(int status, const char* what) {
    if (status != HIPIE_OK) throw_status(status, what);
}

using ConfigMap = std::map<std::string, std::string>;

// key / value arrays for hipie_compile_opts over a config map that outlives them
struct ConfigArrays {
    std::vector<const char*> keys, values;
    explicit ConfigArrays(const ConfigMap& cfg) {
        for (const auto& kv : cfg) {
            keys.push_back(kv.first.c_str());
            values.push_back(kv.second.c_str());
        }
    }
};

struct GraphDeleter { void operator()(hipie_graph* g) const { hipie_graph_destroy(g); } };
struct PlanDeleter { void operator()(hipie_plan* p) const { hipie_plan_destroy(p); } };
struct RequestDeleter { void operator()(hipie_request* r) const { hipie_request_destroy(r); } };
using GraphPtr = std::unique_ptr<hipie_graph, GraphDeleter>;
using PlanPtr = std::unique_ptr<hipie_plan, PlanDeleter>;
using RequestPtr = std::unique_ptr<hipie_request, RequestDeleter>;

}  // namespace HipPlugin
