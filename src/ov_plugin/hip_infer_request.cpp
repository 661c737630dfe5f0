#include "hip_infer_request.hpp"

#include <algorithm>
#include <cstring>

#include <blob_factory.hpp>
#include <ie_allocator.hpp>
#include <precision_utils.h>

#include "hip_executable_network.hpp"

using namespace HipPlugin;

namespace {

// page-locked host memory from the engine, so that StartAsync returns once the copies are queued
class PinnedAllocator final : public InferenceEngine::IAllocator {
public:
    void* lock(void* handle, InferenceEngine::LockOp) noexcept override { return handle; }
    void unlock(void*) noexcept override {}
    void* alloc(size_t size) noexcept override {
        void* p = nullptr;
        return hipie_host_alloc(std::max<size_t>(size, 1), &p) == HIPIE_OK ? p : nullptr;
    }
    bool free(void* handle) noexcept override { return hipie_host_free(handle) == HIPIE_OK; }
};

InferenceEngine::Precision precision_of(int dtype) {
    switch (dtype) {
    case HIPIE_F32: return InferenceEngine::Precision::FP32;
    case HIPIE_I32: return InferenceEngine::Precision::I32;
    case HIPIE_U8: return InferenceEngine::Precision::U8;
    case HIPIE_I8: return InferenceEngine::Precision::I8;
    default: IE_THROW(NotImplemented) << "HIP plugin: port type " << dtype;
    }
}

template <typename From, typename To>
void convert(const InferenceEngine::Blob& from, InferenceEngine::Blob& to) {
    const From* src = from.cbuffer().as<const From*>();
    To* dst = to.buffer().as<To*>();
    std::transform(src, src + from.size(), dst, [](From v) { return static_cast<To>(v); });
}

// dense copies between the precisions users set on ports (U8 images into FP32 networks, FP32 results read as they are):
// the same small set the template plugin converts between (template_infer_request.cpp:176-229)
void copy_blob(const InferenceEngine::Blob& from, InferenceEngine::Blob& to) {
    using P = InferenceEngine::Precision;
    if (from.size() != to.size()) IE_THROW(ParameterMismatch) << "HIP plugin: blob sizes differ";
    const auto a = from.getTensorDesc().getPrecision(), b = to.getTensorDesc().getPrecision();
    if (a == b) {
        std::memcpy(to.buffer().as<void*>(), from.cbuffer().as<const void*>(), from.byteSize());
    } else if (a == P::U8 && b == P::FP32) {
        convert<std::uint8_t, float>(from, to);
    } else if (a == P::I8 && b == P::FP32) {
        convert<std::int8_t, float>(from, to);
    } else if (a == P::I32 && b == P::FP32) {
        convert<std::int32_t, float>(from, to);
    } else if (a == P::FP32 && b == P::I32) {
        convert<float, std::int32_t>(from, to);
    } else if (a == P::U8 && b == P::I32) {
        convert<std::uint8_t, std::int32_t>(from, to);
    } else {
        IE_THROW(NotImplemented) << "HIP plugin: no conversion from " << a << " to " << b;
    }
}

}  // namespace

InferRequest::InferRequest(const InferenceEngine::InputsDataMap& networkInputs, const InferenceEngine::OutputsDataMap& networkOutputs,
                           const std::shared_ptr<ExecutableNetwork>& network)
    : IInferRequestInternal(networkInputs, networkOutputs), _network(network) {
    hipie_request* raw = nullptr;
    check(hipie_request_create(_network->plan(), -1, &raw), "hipie_request_create");
    _request.reset(raw);
    describe_ports(false);
    describe_ports(true);
}

void InferRequest::describe_ports(bool outputs) {
    static const auto pinned = std::make_shared<PinnedAllocator>();
    const hipie_plan* plan = _network->plan();
    const int n = outputs ? hipie_plan_num_outputs(plan) : hipie_plan_num_inputs(plan);
    auto& ports = outputs ? _out : _in;
    for (int i = 0; i < n; ++i) {
        char name[256];
        int dtype = 0, rank = 0;
        int64_t dims[8];
        check(hipie_plan_io_desc(plan, outputs, i, name, sizeof name, &dtype, dims, &rank), "hipie_plan_io_desc");
        Port port;
        port.name = name;
        port.dtype = dtype;
        const InferenceEngine::SizeVector shape(dims, dims + rank);
        const InferenceEngine::TensorDesc dense(precision_of(dtype), shape, InferenceEngine::TensorDesc::getLayoutByDims(shape));
        port.staged = make_blob_with_precision(dense, pinned);
        port.staged->allocate();

        // the blob the user sees: the staged one itself when the port's precision and layout are the plan's, else a
        // plain blob of the user's description that the pre / post stage converts
        InferenceEngine::TensorDesc user = dense;
        if (outputs) {
            const auto it = _networkOutputs.find(port.name);
            if (it == _networkOutputs.end()) IE_THROW(NotFound) << "HIP plugin: the plan's output " << port.name << " is not a network output";
            user = it->second->getTensorDesc();
        } else {
            const auto it = _networkInputs.find(port.name);
            if (it == _networkInputs.end()) IE_THROW(NotFound) << "HIP plugin: the plan's input " << port.name << " is not a network input";
            user = it->second->getTensorDesc();
        }
        InferenceEngine::Blob::Ptr seen = port.staged;
        if (user.getPrecision() != dense.getPrecision() || user.getLayout() != dense.getLayout()) {
            seen = make_blob_with_precision(user);
            seen->allocate();
        }
        if (outputs) {
            _outputs[port.name] = seen;
        } else {
            _inputs[port.name] = seen;
            _deviceInputs[port.name] = port.staged;
        }
        ports.push_back(std::move(port));
    }
}

void InferRequest::inferPreprocess() {
    // resize / colour conversion / layout of user blobs into _deviceInputs where the user asked for it (ie_preprocess_data.hpp)
    execDataPreprocessing(_deviceInputs);
    _in_ptrs.clear();
    for (auto& port : _in) {
        const auto& user = _inputs.at(port.name);
        const bool preprocessed = _preProcData.count(port.name) != 0;
        if (!preprocessed && user != port.staged) {
            if (user->getTensorDesc().getLayout() != port.staged->getTensorDesc().getLayout() && user->getTensorDesc().getDims().size() > 2)
                IE_THROW(NotImplemented) << "HIP plugin: input " << port.name << " in a layout other than the network's needs a preprocessing step";
            copy_blob(*user, *port.staged);
        }
        _in_ptrs.push_back(port.staged->cbuffer().as<const void*>());
    }
    _out_ptrs.clear();
    for (auto& port : _out) {
        // a user blob of the plan's own type receives the copy from the device directly
        const auto& user = _outputs.at(port.name);
        const bool direct = user->getTensorDesc().getPrecision() == port.staged->getTensorDesc().getPrecision() &&
                            user->getTensorDesc().getLayout() == port.staged->getTensorDesc().getLayout();
        _out_ptrs.push_back(direct ? user->buffer().as<void*>() : port.staged->buffer().as<void*>());
    }
}

void InferRequest::startPipeline() {
    check(hipie_request_start(_request.get(), _in_ptrs.data(), _out_ptrs.data(), 0), "hipie_request_start");
}

void InferRequest::waitPipeline() {
    check(hipie_request_wait(_request.get()), "hipie_request_wait");   // InferCancelled after Cancel()
}

void InferRequest::inferPostprocess() {
    for (size_t i = 0; i < _out.size(); ++i) {
        const auto& user = _outputs.at(_out[i].name);
        if (_out_ptrs[i] != user->buffer().as<void*>()) copy_blob(*_out[i].staged, *user);
    }
}

void InferRequest::InferImpl() {
    inferPreprocess();
    startPipeline();
    waitPipeline();
    inferPostprocess();
}

void InferRequest::Cancel() {
    check(hipie_request_cancel(_request.get()), "hipie_request_cancel");
}

std::map<std::string, InferenceEngine::InferenceEngineProfileInfo> InferRequest::GetPerformanceCounts() const {
    std::map<std::string, InferenceEngine::InferenceEngineProfileInfo> perf;
    const hipie_plan* plan = _network->plan();
    const int steps = hipie_plan_num_steps(plan);
    for (int i = 0; i < steps; ++i) {
        char name[256], type[64];
        int64_t macs = 0, bytes = 0;
        check(hipie_plan_step_info(plan, i, name, sizeof name, type, sizeof type, &macs, &bytes), "hipie_plan_step_info");
        float ms = 0.f;
        check(hipie_request_perf(_request.get(), i, &ms), "hipie_request_perf");   // PERF_COUNT=NO: NotFound, as nothing was measured
        InferenceEngine::InferenceEngineProfileInfo info;
        info.status = InferenceEngine::InferenceEngineProfileInfo::EXECUTED;
        info.realTime_uSec = info.cpu_uSec = static_cast<long long>(ms * 1000.f);
        info.execution_index = static_cast<unsigned>(i);
        // exec_type as the CPU plugin writes it: "<primitive>_<runtime precision>" (mkldnn_node.cpp getPrimitiveDescriptorType)
        char primitive[64] = "", precision[16] = "";
        check(hipie_plan_step_rt_info(plan, i, "primitiveType", primitive, sizeof primitive), "hipie_plan_step_rt_info");
        check(hipie_plan_step_rt_info(plan, i, "runtimePrecision", precision, sizeof precision), "hipie_plan_step_rt_info");
        std::snprintf(info.exec_type, sizeof info.exec_type, "%s_%s", primitive, precision);
        std::snprintf(info.layer_type, sizeof info.layer_type, "%s", type);
        perf[name] = info;
    }
    return perf;
}
