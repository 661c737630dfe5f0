#include "div2.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>

#include "common.h"
#include "fq.h"

namespace hipie {
namespace {

constexpr int kBlocksPerDivisor = 32, kThreads = 256;

// fail[i] != 0 when fma(n, zh[i], n * zl[i]) != n / d[i] for some significand of n
__global__ __launch_bounds__(kThreads) void div2_check(const float* d, const float* zh, const float* zl, int* fail) {
    const int i = blockIdx.y;
    const float dd = d[i], h = zh[i], l = zl[i];
    bool bad = false;
    const uint32_t stride = kBlocksPerDivisor * kThreads;
    for (uint32_t m = blockIdx.x * kThreads + threadIdx.x; m < (1u << 23); m += stride) {
        const float n = __uint_as_float(0x3f800000u | m);
        const float lo = n * l;
        const float fast = fmaf(n, h, lo);
        const float ref = n / dd;
        bad = bad || !(fast == ref);
    }
    if (bad) atomicOr(&fail[i], 1);
}

float next_float(float x, int k) {
    // k units in the last place away from x (x finite; zero stays zero)
    if (x == 0.f) return x;
    int32_t b;
    std::memcpy(&b, &x, 4);
    b += (b >= 0) ? k : -k;
    float y;
    std::memcpy(&y, &b, 4);
    return y;
}

}  // namespace

bool fq_div2_constants(int device, const std::vector<float>& d, std::vector<float>& zh, std::vector<float>& zl) {
    zh.assign(d.size(), 0.f);
    zl.assign(d.size(), 0.f);
    if (device < 0 || d.empty()) return false;
    // distinct divisors only (a per-tensor range repeats one value for every channel)
    std::map<uint32_t, int> index;
    std::vector<float> ud;
    for (float v : d) {
        if (!(v > 0.f) || !std::isfinite(v)) return false;
        uint32_t b;
        std::memcpy(&b, &v, 4);
        if (index.emplace(b, static_cast<int>(ud.size())).second) ud.push_back(v);
    }
    const size_t n = ud.size();
    std::vector<float> uh(n), ul(n);
    std::vector<double> inv(n);
    for (size_t i = 0; i < n; ++i) {
        inv[i] = 1.0 / static_cast<double>(ud[i]);
        const float h = static_cast<float>(inv[i]);
        const float l = static_cast<float>(inv[i] - static_cast<double>(h));
        if (!std::isnormal(h) || !(l == 0.f || std::isnormal(l))) return false;   // l == 0: d is a power of two
    }
    DeviceGuard g(device);
    // divisors the calling thread's table of earlier verdicts already answers need no run on the device
    FqVerdicts* table = FqVerdicts::current();
    auto bits_of = [](float v) {
        uint32_t b;
        std::memcpy(&b, &v, 4);
        return b;
    };
    std::vector<int> todo;
    for (size_t i = 0; i < n; ++i) {
        if (table) {
            const auto it = table->div2.find(bits_of(ud[i]));
            if (it != table->div2.end()) {
                if (!it->second.ok) return false;
                uh[i] = it->second.zh;
                ul[i] = it->second.zl;
                continue;
            }
        }
        todo.push_back(static_cast<int>(i));
    }
    const std::vector<int> asked = todo;
    // candidates: zh = RN(1/d) moved by hs units in the last place, zl = RN(1/d - zh) moved by ls
    static const int kShift[] = {0, 1, -1, 2, -2, 3, -3, 4, -4};
    DeviceBuffer bd, bh, bl, bf;
    for (int hs : {0, 1, -1}) {
        for (int ls : kShift) {
            if (todo.empty()) break;
            const size_t m = todo.size();
            std::vector<float> cd(m), ch(m), cl(m);
            for (size_t j = 0; j < m; ++j) {
                const int i = todo[j];
                cd[j] = ud[i];
                ch[j] = next_float(static_cast<float>(inv[i]), hs);
                cl[j] = next_float(static_cast<float>(inv[i] - static_cast<double>(ch[j])), ls);
            }
            std::vector<int> fail(m, 0);
            bd.upload(device, cd.data(), m * sizeof(float));
            bh.upload(device, ch.data(), m * sizeof(float));
            bl.upload(device, cl.data(), m * sizeof(float));
            bf.upload(device, fail.data(), m * sizeof(int));
            for (size_t off = 0; off < m; off += 32768) {   // grid.y limit
                const size_t cnt = std::min<size_t>(32768, m - off);
                hipLaunchKernelGGL(div2_check, dim3(kBlocksPerDivisor, static_cast<unsigned>(cnt)), dim3(kThreads), 0,
                                   nullptr, bd.as<float>() + off, bh.as<float>() + off, bl.as<float>() + off,
                                   bf.as<int>() + off);
            }
            HIPIE_CHECK_HIP(hipGetLastError());
            HIPIE_CHECK_HIP(hipMemcpy(fail.data(), bf.as<int>(), m * sizeof(int), hipMemcpyDeviceToHost));
            std::vector<int> still;
            for (size_t j = 0; j < m; ++j) {
                if (fail[j]) {
                    still.push_back(todo[j]);
                } else {
                    uh[todo[j]] = ch[j];
                    ul[todo[j]] = cl[j];
                }
            }
            todo.swap(still);
            if (std::getenv("HIPIE_TUNE_LOG"))
                std::fprintf(stderr, "hipie div2: %zu divisors, zh%+d zl%+d ulp: %zu unmatched\n", n, hs, ls, todo.size());
        }
    }
    if (table) {
        for (int i : asked) table->div2[bits_of(ud[i])] = FqVerdicts::Div2{uh[i], ul[i], 1u};
        for (int i : todo) table->div2[bits_of(ud[i])] = FqVerdicts::Div2{0.f, 0.f, 0u};
    }
    if (!todo.empty()) {
        if (std::getenv("HIPIE_TUNE_LOG"))
            for (int i : todo) std::fprintf(stderr, "hipie div2: no constants for d = %a (%.9g)\n", ud[i], ud[i]);
        return false;
    }
    for (size_t c = 0; c < d.size(); ++c) {
        uint32_t b;
        std::memcpy(&b, &d[c], 4);
        const int i = index[b];
        zh[c] = uh[i];
        zl[c] = ul[i];
    }
    return true;
}

}  // namespace hipie

extern "C" int hipie_fq_div2_constants(int device, const float* d, int64_t n, float* zh, float* zl, int* verified) {
    return hipie::guarded([&] {
        HIPIE_REQUIRE(d && zh && zl && verified && n > 0, HIPIE_PARAMETER_MISMATCH, "hipie_fq_div2_constants: null argument");
        HIPIE_REQUIRE(device >= 0, HIPIE_PARAMETER_MISMATCH, "hipie_fq_div2_constants: needs a device");
        std::vector<float> dv(d, d + n), h, l;
        *verified = hipie::fq_div2_constants(device, dv, h, l) ? 1 : 0;
        std::copy(h.begin(), h.end(), zh);
        std::copy(l.begin(), l.end(), zl);
    });
}
