// Diagnostics: what the device's matrix pipe delivers with nothing else in the way.  The published dense int8 peak
// is a clock times a count of units; the rate a kernel can reach is what the device sustains with every SIMD issuing
// matrix instructions back to back from registers - no memory, no LDS, no epilogue.  Roofline fractions read against
// this number say how much of the gap to the published peak belongs to the kernels.
#include <hip/hip_runtime.h>

#include "common.h"
#include "hipie_diag.h"

namespace hipie {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// four independent accumulators per wave, so that consecutive matrix instructions never wait for each other
__global__ __launch_bounds__(256) void mfma_rate_kernel(int iters, int* sink) {
    const int lane = threadIdx.x & 63;
    v4i a = {lane, lane + 1, lane + 2, lane + 3}, b = {lane ^ 5, lane ^ 9, lane ^ 17, lane ^ 33};
    v16i acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    if (s == 0x7fffffff) sink[0] = s;       // keeps the products alive; not taken for these operands
}

// LDS read rate: every wave reads 1 KB per ds_read_b128 (lane l the 16 bytes at 16 l of a 1 KB row: no bank conflict),
// eight rows per iteration, into one of two register sets; MFMA: the eight matrix instructions of a 64 x 64 wave tile
// whose operands both come from LDS run on the other set meanwhile (reads issued a step ahead, one wait per step).
// The first wave of the first workgroup reports its loop in core clocks and in ticks of the constant 100 MHz clock,
// which gives the core clock the launch ran at.
#define HIPIE_PROBE_READ8(R)                                                                                               \
    asm volatile("ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:1024\n\tds_read_b128 %2, %8 offset:2048\n\t"            \
                 "ds_read_b128 %3, %8 offset:3072\n\tds_read_b128 %4, %8 offset:4096\n\tds_read_b128 %5, %8 offset:5120\n\t" \
                 "ds_read_b128 %6, %8 offset:6144\n\tds_read_b128 %7, %8 offset:7168"                                         \
                 : "=&v"(R[0]), "=&v"(R[1]), "=&v"(R[2]), "=&v"(R[3]), "=&v"(R[4]), "=&v"(R[5]), "=&v"(R[6]), "=&v"(R[7])  \
                 : "v"(addr))
#define HIPIE_PROBE_WAIT8(R)                                                                                               \
    asm volatile("s_waitcnt lgkmcnt(0)"                                                                                    \
                 : "+v"(R[0]), "+v"(R[1]), "+v"(R[2]), "+v"(R[3]), "+v"(R[4]), "+v"(R[5]), "+v"(R[6]), "+v"(R[7]))

template <bool MFMA>
__global__ __launch_bounds__(256) void lds_rate_kernel(int iters, long long* cycles, int* sink) {
    __shared__ __attribute__((aligned(16))) int8_t buf[32768];
    const int tid = threadIdx.x, lane = tid & 63;
    for (int i = tid; i < 32768 / 16; i += 256) reinterpret_cast<v4i*>(buf)[i] = v4i{i, i + 1, i + 2, i + 3};
    __syncthreads();
    const uint32_t addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) int8_t*)(buf + (tid >> 6) * 8192 + lane * 16)));
    v4i ra[8], rb[8];
    v16i acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[i][q] = 0;
    int s = 0;
    const long long w0 = wall_clock64();
    const long long t0 = clock64();
    HIPIE_PROBE_READ8(ra);
    HIPIE_PROBE_WAIT8(ra);
    for (int it = 0; it < iters; it += 2) {
        HIPIE_PROBE_READ8(rb);
        __builtin_amdgcn_sched_barrier(0);            // reads first: they run under the matrix instructions below
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (MFMA) acc[i & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ra[i], ra[(i + 1) & 7], acc[i & 3], 0, 0, 0);
            else s ^= ra[i].x;
        }
        __builtin_amdgcn_sched_barrier(0);
        HIPIE_PROBE_WAIT8(rb);
        HIPIE_PROBE_READ8(ra);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (MFMA) acc[i & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(rb[i], rb[(i + 1) & 7], acc[i & 3], 0, 0, 0);
            else s ^= rb[i].x;
        }
        __builtin_amdgcn_sched_barrier(0);
        HIPIE_PROBE_WAIT8(ra);
    }
    const long long t1 = clock64();
    const long long w1 = wall_clock64();
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int q = 0; q < 16; ++q) s += acc[i][q];
    if (blockIdx.x == 0 && tid == 0) {
        cycles[0] = t1 - t0;
        cycles[1] = w1 - w0;
    }
    if (s == 0x7fffffff) sink[0] = s;
}

}  // namespace
}  // namespace hipie

using namespace hipie;

extern "C" int hipie_probe_lds_rate(int device, int iterations, int waves_per_simd, int with_mfma, double* bytes_per_clock_per_cu,
                                    double* gigabytes_per_second) {
    return guarded([&] {
        HIPIE_REQUIRE(bytes_per_clock_per_cu && iterations > 0 && iterations <= (1 << 20) && iterations % 2 == 0 &&
                          waves_per_simd >= 1 && waves_per_simd <= 4,
                      HIPIE_PARAMETER_MISMATCH, "hipie_probe_lds_rate: iterations %d (even), waves per SIMD %d", iterations, waves_per_simd);
        DeviceGuard g(device);
        hipDeviceProp_t prop;
        HIPIE_CHECK_HIP(hipGetDeviceProperties(&prop, device));
        long long* cycles = nullptr;
        HIPIE_CHECK_HIP(hipMalloc(&cycles, 32));
        int* sink = reinterpret_cast<int*>(cycles + 2);
        const int blocks = prop.multiProcessorCount * waves_per_simd;      // four waves each: one per SIMD
        auto launch = [&](int iters) {
            if (with_mfma) hipLaunchKernelGGL(lds_rate_kernel<true>, dim3(blocks), dim3(256), 0, nullptr, iters, cycles, sink);
            else hipLaunchKernelGGL(lds_rate_kernel<false>, dim3(blocks), dim3(256), 0, nullptr, iters, cycles, sink);
        };
        hipEvent_t e0, e1;
        HIPIE_CHECK_HIP(hipEventCreate(&e0));
        HIPIE_CHECK_HIP(hipEventCreate(&e1));
        launch(16);                                                        // warm-up
        HIPIE_CHECK_HIP(hipEventRecord(e0, nullptr));
        launch(iterations);
        HIPIE_CHECK_HIP(hipEventRecord(e1, nullptr));
        HIPIE_CHECK_HIP(hipEventSynchronize(e1));
        float ms = 0.f;
        HIPIE_CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
        long long host_cycles[2] = {0, 0};
        HIPIE_CHECK_HIP(hipMemcpy(host_cycles, cycles, sizeof host_cycles, hipMemcpyDeviceToHost));
        HIPIE_CHECK_HIP(hipEventDestroy(e0));
        HIPIE_CHECK_HIP(hipEventDestroy(e1));
        HIPIE_CHECK_HIP(hipFree(cycles));
        // bytes all compute units read over the launch's duration, in core clocks of the rate the first wave saw
        const double total = 8.0 * 1024.0 * (iterations + 1) * 4.0 * blocks;
        const double core_hz = host_cycles[1] > 0 ? 1e8 * static_cast<double>(host_cycles[0]) / static_cast<double>(host_cycles[1]) : 0.0;
        const double per_second = total / (ms * 1e-3);
        *bytes_per_clock_per_cu = core_hz > 0 ? per_second / prop.multiProcessorCount / core_hz : 0.0;
        if (gigabytes_per_second) *gigabytes_per_second = per_second / 1e9;
    });
}

extern "C" int hipie_probe_mfma_rate(int device, int iterations, int waves_per_simd, double* tops, double* milliseconds) {
    return guarded([&] {
        HIPIE_REQUIRE(tops && iterations > 0 && iterations <= (1 << 20) && waves_per_simd >= 1 && waves_per_simd <= 8,
                      HIPIE_PARAMETER_MISMATCH, "hipie_probe_mfma_rate: iterations %d, waves per SIMD %d", iterations, waves_per_simd);
        DeviceGuard g(device);
        hipDeviceProp_t prop;
        HIPIE_CHECK_HIP(hipGetDeviceProperties(&prop, device));
        int* sink = nullptr;
        HIPIE_CHECK_HIP(hipMalloc(&sink, 16));
        const int blocks = prop.multiProcessorCount * waves_per_simd;      // four waves each: one per SIMD
        hipEvent_t e0, e1;
        HIPIE_CHECK_HIP(hipEventCreate(&e0));
        HIPIE_CHECK_HIP(hipEventCreate(&e1));
        hipLaunchKernelGGL(mfma_rate_kernel, dim3(blocks), dim3(256), 0, nullptr, 16, sink);      // warm-up
        HIPIE_CHECK_HIP(hipEventRecord(e0, nullptr));
        hipLaunchKernelGGL(mfma_rate_kernel, dim3(blocks), dim3(256), 0, nullptr, iterations, sink);
        HIPIE_CHECK_HIP(hipEventRecord(e1, nullptr));
        HIPIE_CHECK_HIP(hipEventSynchronize(e1));
        float ms = 0.f;
        HIPIE_CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
        HIPIE_CHECK_HIP(hipEventDestroy(e0));
        HIPIE_CHECK_HIP(hipEventDestroy(e1));
        HIPIE_CHECK_HIP(hipFree(sink));
        const double ops = 2.0 * 32 * 32 * 32 * 4.0 * iterations * 4.0 * blocks;     // per instruction x 4 per iteration x 4 waves
        *tops = ops / (ms * 1e-3) / 1e12;
        if (milliseconds) *milliseconds = ms;
    });
}
