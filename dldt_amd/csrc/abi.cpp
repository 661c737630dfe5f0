// Library-wide C-ABI entry points: error text, version, device enumeration.
#include "common.h"

namespace hipie {
static thread_local std::string g_last_error;
void set_last_error(const char* msg) { g_last_error = msg ? msg : ""; }
}  // namespace hipie

using namespace hipie;

extern "C" {

const char* hipie_last_error(void) { return g_last_error.c_str(); }

const char* hipie_version(void) { return "0.1 gfx950"; }

int hipie_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int hipie_device_name(int device, char* buf, size_t buf_len) {
    return guarded([&] {
        HIPIE_REQUIRE(buf && buf_len > 0, HIPIE_PARAMETER_MISMATCH, "hipie_device_name: no buffer");
        hipDeviceProp_t prop;
        HIPIE_CHECK_HIP(hipGetDeviceProperties(&prop, device));
        snprintf(buf, buf_len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName,
                 prop.multiProcessorCount);
    });
}

int hipie_memcpy(void* dst, const void* src, size_t bytes, int to_device) {
    return guarded([&] {
        HIPIE_REQUIRE((dst && src) || bytes == 0, HIPIE_PARAMETER_MISMATCH, "hipie_memcpy: null argument");
        if (bytes)
            HIPIE_CHECK_HIP(hipMemcpy(dst, src, bytes, to_device ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost));
    });
}

int hipie_host_alloc(size_t bytes, void** ptr) {
    return guarded([&] {
        HIPIE_REQUIRE(ptr, HIPIE_PARAMETER_MISMATCH, "hipie_host_alloc: null argument");
        *ptr = nullptr;
        HIPIE_CHECK_HIP(hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault));
    });
}

int hipie_host_free(void* ptr) {
    return guarded([&] {
        if (ptr) HIPIE_CHECK_HIP(hipHostFree(ptr));
    });
}

}  // extern "C"
