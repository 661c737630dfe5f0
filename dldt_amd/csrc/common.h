// Shared host-side plumbing of the engine: status + thread-local error text, HIP error
// translation, and small RAII helpers for device constants.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <algorithm>
#include <string>
#include <thread>
#include <vector>

#include "../../include/hipie.h"
#include "../../include/hipie_diag.h"

namespace hipie {

// Thrown inside the library; converted to a hipie_status + message at the C boundary so that no
// C++ exception and no raw hipError_t ever crosses it.
struct Error : std::runtime_error {
    hipie_status code;
    Error(hipie_status c, const std::string& m) : std::runtime_error(m), code(c) {}
};

[[noreturn]] inline void fail(hipie_status code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    throw Error(code, buf);
}

#define HIPIE_CHECK_HIP(expr)                                                              \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess)                                                              \
            ::hipie::fail(HIPIE_GENERAL_ERROR, "%s failed: %s (%s:%d)", #expr,            \
                          hipGetErrorString(e_), __FILE__, __LINE__);                      \
    } while (0)

#define HIPIE_REQUIRE(cond, code, ...)                                                     \
    do {                                                                                   \
        if (!(cond)) ::hipie::fail(code, __VA_ARGS__);                                     \
    } while (0)

void set_last_error(const char* msg);

// Runs `body`, mapping exceptions to status codes (the C-ABI trampoline).
template <typename F>
int guarded(F&& body) noexcept {
    try {
        body();
        return HIPIE_OK;
    } catch (const Error& e) {
        set_last_error(e.what());
        return e.code;
    } catch (const std::exception& e) {
        set_last_error(e.what());
        return HIPIE_GENERAL_ERROR;
    } catch (...) {
        set_last_error("unknown exception");
        return HIPIE_UNEXPECTED;
    }
}

// Selects a device for the current scope (calls may arrive on any executor thread).
struct DeviceGuard {
    int prev = -1;
    explicit DeviceGuard(int dev) {
        HIPIE_CHECK_HIP(hipGetDevice(&prev));
        if (prev != dev) HIPIE_CHECK_HIP(hipSetDevice(dev));
        else prev = -1;
    }
    ~DeviceGuard() {
        if (prev >= 0) (void)hipSetDevice(prev);
    }
};

// Device buffer owned by a load-time object (weights, per-channel tables).
struct DeviceBuffer {
    void* ptr = nullptr;
    size_t bytes = 0;
    int device = 0;
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    DeviceBuffer(DeviceBuffer&& o) noexcept { *this = std::move(o); }
    DeviceBuffer& operator=(DeviceBuffer&& o) noexcept {
        release();
        ptr = o.ptr; bytes = o.bytes; device = o.device;
        o.ptr = nullptr; o.bytes = 0;
        return *this;
    }
    void alloc(int dev, size_t n) {
        release();
        device = dev;
        DeviceGuard g(dev);
        HIPIE_CHECK_HIP(hipMalloc(&ptr, n ? n : 1));
        bytes = n;
    }
    void upload(int dev, const void* host, size_t n) {
        alloc(dev, n);
        if (n) HIPIE_CHECK_HIP(hipMemcpy(ptr, host, n, hipMemcpyHostToDevice));
    }
    void release() {
        if (ptr) {
            (void)hipFree(ptr);
            ptr = nullptr;
        }
    }
    ~DeviceBuffer() { release(); }
    template <typename T> T* as() const { return static_cast<T*>(ptr); }
};

// Load-time host loops (per-channel checks, weight packing) spread over a few threads.
template <typename F>
void parallel_for(int64_t n, F&& body) {
    const int64_t nt = std::min<int64_t>(std::max<int64_t>(1, std::thread::hardware_concurrency()),
                                         std::min<int64_t>(16, (n + 63) / 64));
    if (nt <= 1) {
        for (int64_t i = 0; i < n; ++i) body(i);
        return;
    }
    std::vector<std::thread> pool;
    for (int64_t t = 0; t < nt; ++t)
        pool.emplace_back([&, t] {
            for (int64_t i = t; i < n; i += nt) body(i);
        });
    for (auto& th : pool) th.join();
}

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

}  // namespace hipie
