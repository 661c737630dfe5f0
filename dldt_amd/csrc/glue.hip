// fp32 glue of the transformer path (HBM-bound): Softmax and MVN over the last axis, GELU(erf).
// Reference semantics (tolerance only; libm exp/erf are not bit-reproducible on a GPU):
//   softmax.hpp (subtract the row maximum, exp, sum, divide),
//   mvn.hpp mvn_6 (mean, centre, mean of squares, sqrt(var + eps) | sqrt(var) + eps, divide),
//   gelu.hpp ERF mode (0.5 * x * (1 + erf(x / sqrt(2))) evaluated in double).
// One wavefront owns one row: coalesced 256-byte row segments, reductions by cross-lane shuffles.
#include "common.h"

namespace hipie {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

__global__ __launch_bounds__(kThreads) void softmax_rows(const float* __restrict__ x, float* __restrict__ y,
                                                         int64_t rows, int axis) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const float* p = x + row * axis;
    float* q = y + row * axis;
    float m = -INFINITY;
    for (int i = lane; i < axis; i += 64) m = fmaxf(m, p[i]);
    m = wave_max(m);
    float s = 0.f;
    for (int i = lane; i < axis; i += 64) {
        const float e = expf(p[i] - m);
        q[i] = e;
        s += e;
    }
    s = wave_sum(s);
    for (int i = lane; i < axis; i += 64) q[i] = q[i] / s;
}

__global__ __launch_bounds__(kThreads) void mvn_rows(const float* __restrict__ x, float* __restrict__ y,
                                                     int64_t rows, int axis, int normalize_variance, float eps,
                                                     int eps_inside, const float* __restrict__ gamma,
                                                     const float* __restrict__ beta) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const float* p = x + row * axis;
    float* q = y + row * axis;
    float s = 0.f;
    for (int i = lane; i < axis; i += 64) s += p[i];
    const float mean = wave_sum(s) / static_cast<float>(axis);
    float v = 0.f;
    for (int i = lane; i < axis; i += 64) {
        const float c = p[i] - mean;
        v += c * c;
    }
    float denom = 1.f;
    if (normalize_variance) {
        const float var = wave_sum(v) / static_cast<float>(axis);
        denom = eps_inside ? sqrtf(var + eps) : sqrtf(var) + eps;
    }
    for (int i = lane; i < axis; i += 64) {
        float o = p[i] - mean;
        if (normalize_variance) o = o / denom;
        if (gamma) o = o * gamma[i];
        if (beta) o = o + beta[i];
        q[i] = o;
    }
}

__global__ __launch_bounds__(kThreads) void gelu_erf(const float* __restrict__ x, float* __restrict__ y, int64_t n) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
        const double v = static_cast<double>(x[i]);
        y[i] = static_cast<float>(0.5 * v * (1.0 + erf(v / 1.4142135623730951)));
    }
}

// Batched 2-D transpose of bytes through a 64 x 64 LDS tile (row stride 65 words would not help
// bytes: rows are read as 16-byte pieces and written back byte-wise from a 64 x 65 tile).
// dst[b][c][r] = src[b][r][c]; the two inner dimensions of a Transpose node on an i8 tensor
// (reference::transpose, transpose.hpp:20-25, moves elements only).
__global__ __launch_bounds__(256) void transpose_bytes_kernel(const int8_t* __restrict__ src, int64_t ld_src,
                                                              int64_t bs_src, int64_t os_src, int8_t* __restrict__ dst,
                                                              int64_t ld_dst, int64_t bs_dst, int64_t os_dst, int rows,
                                                              int cols, int batch_inner) {
    __shared__ int8_t tile[64][65];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int bo = blockIdx.z / batch_inner, bi = blockIdx.z - bo * batch_inner;
    const int8_t* s = src + bo * os_src + bi * bs_src;
    int8_t* d = dst + bo * os_dst + bi * bs_dst;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int r = r0 + ty * 16 + i, c = c0 + tx;
        tile[ty * 16 + i][tx] = (r < rows && c < cols) ? s[static_cast<int64_t>(r) * ld_src + c] : int8_t(0);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int c = c0 + ty * 16 + i, r = r0 + tx;
        if (c < cols && r < rows) d[static_cast<int64_t>(c) * ld_dst + r] = tile[tx][ty * 16 + i];
    }
}

}  // namespace
}  // namespace hipie

using namespace hipie;

extern "C" {

int hipie_softmax_f32(const float* x, float* y, int64_t rows, int64_t axis, void* stream) {
    return guarded([&] {
        if (rows == 0 || axis == 0) return;
        HIPIE_REQUIRE(x && y && rows > 0 && axis > 0 && axis < (1ll << 31), HIPIE_PARAMETER_MISMATCH,
                      "hipie_softmax_f32: bad argument");
        hipLaunchKernelGGL(softmax_rows, dim3(static_cast<uint32_t>(ceil_div(rows, kThreads / 64))), dim3(kThreads), 0,
                           as_stream(stream), x, y, rows, static_cast<int>(axis));
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_mvn_f32(const float* x, float* y, int64_t rows, int64_t axis, int normalize_variance, float eps,
                  int eps_inside_sqrt, const float* gamma, const float* beta, void* stream) {
    return guarded([&] {
        if (rows == 0 || axis == 0) return;
        HIPIE_REQUIRE(x && y && rows > 0 && axis > 0 && axis < (1ll << 31), HIPIE_PARAMETER_MISMATCH,
                      "hipie_mvn_f32: bad argument");
        hipLaunchKernelGGL(mvn_rows, dim3(static_cast<uint32_t>(ceil_div(rows, kThreads / 64))), dim3(kThreads), 0,
                           as_stream(stream), x, y, rows, static_cast<int>(axis), normalize_variance, eps,
                           eps_inside_sqrt, gamma, beta);
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_gelu_f32(const float* x, float* y, int64_t n, void* stream) {
    return guarded([&] {
        if (n == 0) return;
        HIPIE_REQUIRE(x && y && n > 0, HIPIE_PARAMETER_MISMATCH, "hipie_gelu_f32: bad argument");
        const int64_t blocks = std::min<int64_t>(ceil_div(n, kThreads), 256 * 16);
        hipLaunchKernelGGL(gelu_erf, dim3(static_cast<uint32_t>(blocks)), dim3(kThreads), 0, as_stream(stream), x, y, n);
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_transpose_bytes(const void* src, int64_t ld_src, int64_t batch_stride_src, void* dst, int64_t ld_dst,
                          int64_t batch_stride_dst, int32_t rows, int32_t cols, int32_t batch, void* stream) {
    return hipie_transpose_bytes_nested(src, ld_src, batch_stride_src, 0, dst, ld_dst, batch_stride_dst, 0, rows, cols,
                                        batch, 1, stream);
}

int hipie_transpose_bytes_nested(const void* src, int64_t ld_src, int64_t stride_src, int64_t outer_src, void* dst,
                                 int64_t ld_dst, int64_t stride_dst, int64_t outer_dst, int32_t rows, int32_t cols,
                                 int32_t batch, int32_t batch_outer, void* stream) {
    return guarded([&] {
        if (rows == 0 || cols == 0 || batch == 0 || batch_outer == 0) return;
        HIPIE_REQUIRE(src && dst && rows > 0 && cols > 0 && batch > 0 && batch_outer > 0 &&
                          static_cast<int64_t>(batch) * batch_outer < 65536 && ld_src >= cols && ld_dst >= rows,
                      HIPIE_PARAMETER_MISMATCH, "hipie_transpose_bytes: bad argument");
        const dim3 grid(static_cast<uint32_t>(ceil_div(cols, 64)), static_cast<uint32_t>(ceil_div(rows, 64)),
                        static_cast<uint32_t>(batch * batch_outer));
        hipLaunchKernelGGL(transpose_bytes_kernel, grid, dim3(256), 0, as_stream(stream), static_cast<const int8_t*>(src),
                           ld_src, stride_src, outer_src, static_cast<int8_t*>(dst), ld_dst, stride_dst, outer_dst, rows,
                           cols, batch);
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

}  // extern "C"
