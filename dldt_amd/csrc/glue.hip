// fp32 glue of the transformer path (HBM-bound): Softmax and MVN over the last axis, GELU(erf).
// Reference semantics (tolerance only; libm exp/erf are not bit-reproducible on a GPU):
//   softmax.hpp (subtract the row maximum, exp, sum, divide),
//   mvn.hpp mvn_6 (mean, centre, mean of squares, sqrt(var + eps) | sqrt(var) + eps, divide),
//   gelu.hpp ERF mode (0.5 * x * (1 + erf(x / sqrt(2))) evaluated in double there).
// One wavefront owns one row and holds it in registers: the row is read once and written once,
// reductions by cross-lane shuffles.  The per-tensor FakeQuantize that follows each of them in a
// post-LPT encoder can be fused in (i8 levels written beside or instead of the f32 result).
#include "gelu.h"
#include "requant.h"

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

// Row kernels: one wavefront owns one row and keeps it in registers (NCH float4 per lane, lane l holds
// elements 4 l .. 4 l + 3 of every 256-element chunk), so a row is read once in 1 KB wave loads and
// written once; y and/or q may be null.
template <int NCH>
__global__ __launch_bounds__(kThreads) void softmax_rows_reg(const float* __restrict__ x, float* __restrict__ y,
                                                             int8_t* __restrict__ q, int64_t rows, int axis, Requant fq) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const float* p = x + row * axis;
    float4 v[NCH];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int i = 256 * j + 4 * lane;
        v[j] = i < axis ? *reinterpret_cast<const float4*>(p + i) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        m = fmaxf(fmaxf(m, fmaxf(v[j].x, v[j].y)), fmaxf(v[j].z, v[j].w));
    }
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        v[j].x = expf(v[j].x - m); v[j].y = expf(v[j].y - m); v[j].z = expf(v[j].z - m); v[j].w = expf(v[j].w - m);
        s += (v[j].x + v[j].y) + (v[j].z + v[j].w);    // exp(-inf) = 0 in the padding
    }
    s = wave_sum(s);
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int i = 256 * j + 4 * lane;
        if (i >= axis) continue;
        const float4 o = make_float4(v[j].x / s, v[j].y / s, v[j].z / s, v[j].w / s);
        if (y) *reinterpret_cast<float4*>(y + row * axis + i) = o;
        if (q) *reinterpret_cast<uint32_t*>(q + row * axis + i) = requant4(fq, o);
    }
}

template <int NCH>
__global__ __launch_bounds__(kThreads) void mvn_rows_reg(const float* __restrict__ x, float* __restrict__ y,
                                                         int8_t* __restrict__ q, int64_t rows, int axis,
                                                         int normalize_variance, float eps, int eps_inside,
                                                         const float* __restrict__ gamma, const float* __restrict__ beta,
                                                         Requant fq) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (kThreads / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const float* p = x + row * axis;
    float4 v[NCH];
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int i = 256 * j + 4 * lane;
        v[j] = i < axis ? *reinterpret_cast<const float4*>(p + i) : make_float4(0.f, 0.f, 0.f, 0.f);
        s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
    }
    const float mean = wave_sum(s) / static_cast<float>(axis);
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int i = 256 * j + 4 * lane;
        v[j].x -= mean; v[j].y -= mean; v[j].z -= mean; v[j].w -= mean;
        if (i < axis) sq += (v[j].x * v[j].x + v[j].y * v[j].y) + (v[j].z * v[j].z + v[j].w * v[j].w);
    }
    float denom = 1.f;
    if (normalize_variance) {
        const float var = wave_sum(sq) / static_cast<float>(axis);
        denom = eps_inside ? sqrtf(var + eps) : sqrtf(var) + eps;
    }
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
        const int i = 256 * j + 4 * lane;
        if (i >= axis) continue;
        float4 o = v[j];
        if (normalize_variance) { o.x = o.x / denom; o.y = o.y / denom; o.z = o.z / denom; o.w = o.w / denom; }
        if (gamma) {
            const float4 gm = *reinterpret_cast<const float4*>(gamma + i);
            o.x = o.x * gm.x; o.y = o.y * gm.y; o.z = o.z * gm.z; o.w = o.w * gm.w;
        }
        if (beta) {
            const float4 bt = *reinterpret_cast<const float4*>(beta + i);
            o.x = o.x + bt.x; o.y = o.y + bt.y; o.z = o.z + bt.z; o.w = o.w + bt.w;
        }
        if (y) *reinterpret_cast<float4*>(y + row * axis + i) = o;
        if (q) *reinterpret_cast<uint32_t*>(q + row * axis + i) = requant4(fq, o);
    }
}

// rows of any length (not a multiple of 4, or longer than 4096): three passes over the row
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

// four elements per lane and step (n4 = n / 4 full groups), then the tail one by one
__global__ __launch_bounds__(kThreads) void gelu_erf(const float* __restrict__ x, float* __restrict__ y,
                                                     int8_t* __restrict__ q, int64_t n, Requant fq) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int64_t n4 = n >> 2;
    for (int64_t i = t; i < n4; i += stride) {
        const float4 v = reinterpret_cast<const float4*>(x)[i];
        const float4 o = make_float4(gelu_one(v.x), gelu_one(v.y), gelu_one(v.z), gelu_one(v.w));
        if (y) reinterpret_cast<float4*>(y)[i] = o;
        if (q) reinterpret_cast<uint32_t*>(q)[i] = requant4(fq, o);
    }
    for (int64_t i = 4 * n4 + t; i < n; i += stride) {
        const float o = gelu_one(x[i]);
        if (y) y[i] = o;
        if (q) q[i] = static_cast<int8_t>(requant_level(fq, o));
    }
}

// y = x + m over a dense value of up to four dimensions d[0..3]; m has stride ms[k] along dimension k (0 where it
// has one element and is repeated).  One element per thread and step, the last dimension fastest.
__global__ __launch_bounds__(kThreads) void add_broadcast(const float* __restrict__ x, const float* __restrict__ m,
                                                          float* __restrict__ y, int64_t n, int32_t d1, int32_t d2, int32_t d3,
                                                          int64_t ms0, int64_t ms1, int64_t ms2, int64_t ms3) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
        const int64_t r2 = i / d3, r1 = r2 / d2, i0 = r1 / d1;
        const int64_t i3 = i - r2 * d3, i2 = r2 - r1 * d2, i1 = r1 - i0 * d1;
        y[i] = x[i] + m[i0 * ms0 + i1 * ms1 + i2 * ms2 + i3 * ms3];
    }
}

// dst (dense, dimensions d[0..4], the last fastest) = the elements of src at strides st[0..4]
template <typename T>
__global__ __launch_bounds__(kThreads) void copy_strided(const T* __restrict__ src, T* __restrict__ dst, int64_t n, int32_t d1, int32_t d2,
                                                         int32_t d3, int32_t d4, int64_t s0, int64_t s1, int64_t s2, int64_t s3, int64_t s4) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
        const int64_t r3 = i / d4, r2 = r3 / d3, r1 = r2 / d2, i0 = r1 / d1;
        const int64_t i4 = i - r3 * d4, i3 = r3 - r2 * d3, i2 = r2 - r1 * d2, i1 = r1 - i0 * d1;
        dst[i] = src[i0 * s0 + i1 * s1 + i2 * s2 + i3 * s3 + i4 * s4];
    }
}

// plain per-tensor requantisation of a dense f32 array (behind the long-row fallbacks)
__global__ __launch_bounds__(kThreads) void requant_flat(const float* __restrict__ x, int8_t* __restrict__ q, int64_t n,
                                                         Requant fq) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride)
        q[i] = static_cast<int8_t>(requant_level(fq, x[i]));
}

template <template <int> class Launch, typename... A>
bool dispatch_chunks(int axis, A&&... a) {
    if (axis % 4 != 0 || axis > 4096) return false;
    const int nch = static_cast<int>(ceil_div(axis, 256));
    switch (nch) {
    case 1: Launch<1>::go(a...); break;
    case 2: Launch<2>::go(a...); break;
    case 3: Launch<3>::go(a...); break;
    case 4: Launch<4>::go(a...); break;
    case 5: case 6: Launch<6>::go(a...); break;
    case 7: case 8: Launch<8>::go(a...); break;
    case 9: case 10: case 11: case 12: Launch<12>::go(a...); break;
    default: Launch<16>::go(a...); break;
    }
    return true;
}

template <int NCH>
struct LaunchSoftmax {
    static void go(const float* x, float* y, int8_t* q, int64_t rows, int axis, const Requant& fq, hipStream_t s) {
        hipLaunchKernelGGL(softmax_rows_reg<NCH>, dim3(static_cast<uint32_t>(ceil_div(rows, kThreads / 64))), dim3(kThreads), 0,
                           s, x, y, q, rows, axis, fq);
    }
};
template <int NCH>
struct LaunchMvn {
    static void go(const float* x, float* y, int8_t* q, int64_t rows, int axis, int nv, float eps, int inside,
                   const float* gamma, const float* beta, const Requant& fq, hipStream_t s) {
        hipLaunchKernelGGL(mvn_rows_reg<NCH>, dim3(static_cast<uint32_t>(ceil_div(rows, kThreads / 64))), dim3(kThreads), 0, s,
                           x, y, q, rows, axis, nv, eps, inside, gamma, beta, fq);
    }
};

void launch_requant_flat(const float* x, int8_t* q, int64_t n, const Requant& fq, hipStream_t s) {
    const int64_t blocks = std::min<int64_t>(ceil_div(n, kThreads), 256 * 16);
    hipLaunchKernelGGL(requant_flat, dim3(static_cast<uint32_t>(blocks)), dim3(kThreads), 0, s, x, q, n, fq);
}

void run_softmax(const float* x, float* y, int8_t* q, int64_t rows, int64_t axis, const hipie_requant* r, void* stream,
                 const char* what) {
    if (rows == 0 || axis == 0) return;
    HIPIE_REQUIRE(x && (y || q) && rows > 0 && axis > 0 && axis < (1ll << 31), HIPIE_PARAMETER_MISMATCH, "%s: bad argument", what);
    HIPIE_REQUIRE(!q || r, HIPIE_PARAMETER_MISMATCH, "%s: quantized output without a requantisation", what);
    const Requant fq = q ? make_requant(r, what) : Requant{};
    hipStream_t s = as_stream(stream);
    const bool aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(q) % 4 == 0;
    if (!(aligned && dispatch_chunks<LaunchSoftmax>(static_cast<int>(axis), x, y, q, rows, static_cast<int>(axis), fq, s))) {
        HIPIE_REQUIRE(y, HIPIE_NOT_IMPLEMENTED, "%s: rows of %lld elements need the f32 output as well", what, (long long)axis);
        hipLaunchKernelGGL(softmax_rows, dim3(static_cast<uint32_t>(ceil_div(rows, kThreads / 64))), dim3(kThreads), 0, s, x, y,
                           rows, static_cast<int>(axis));
        if (q) launch_requant_flat(y, q, rows * axis, fq, s);
    }
    HIPIE_CHECK_HIP(hipGetLastError());
}

void run_mvn(const float* x, float* y, int8_t* q, int64_t rows, int64_t axis, int normalize_variance, float eps,
             int eps_inside_sqrt, const float* gamma, const float* beta, const hipie_requant* r, void* stream,
             const char* what) {
    if (rows == 0 || axis == 0) return;
    HIPIE_REQUIRE(x && (y || q) && rows > 0 && axis > 0 && axis < (1ll << 31), HIPIE_PARAMETER_MISMATCH, "%s: bad argument", what);
    HIPIE_REQUIRE(!q || r, HIPIE_PARAMETER_MISMATCH, "%s: quantized output without a requantisation", what);
    const Requant fq = q ? make_requant(r, what) : Requant{};
    hipStream_t s = as_stream(stream);
    const bool aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(q) % 4 == 0 && reinterpret_cast<uintptr_t>(gamma) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(beta) % 16 == 0;
    if (!(aligned && dispatch_chunks<LaunchMvn>(static_cast<int>(axis), x, y, q, rows, static_cast<int>(axis),
                                                normalize_variance, eps, eps_inside_sqrt, gamma, beta, fq, s))) {
        HIPIE_REQUIRE(y, HIPIE_NOT_IMPLEMENTED, "%s: rows of %lld elements need the f32 output as well", what, (long long)axis);
        hipLaunchKernelGGL(mvn_rows, dim3(static_cast<uint32_t>(ceil_div(rows, kThreads / 64))), dim3(kThreads), 0, s, x, y, rows,
                           static_cast<int>(axis), normalize_variance, eps, eps_inside_sqrt, gamma, beta);
        if (q) launch_requant_flat(y, q, rows * axis, fq, s);
    }
    HIPIE_CHECK_HIP(hipGetLastError());
}

void run_gelu(const float* x, float* y, int8_t* q, int64_t n, const hipie_requant* r, void* stream, const char* what) {
    if (n == 0) return;
    HIPIE_REQUIRE(x && (y || q) && n > 0, HIPIE_PARAMETER_MISMATCH, "%s: bad argument", what);
    HIPIE_REQUIRE(!q || r, HIPIE_PARAMETER_MISMATCH, "%s: quantized output without a requantisation", what);
    HIPIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(q) % 4 == 0, HIPIE_PARAMETER_MISMATCH, "%s: buffers must be 16-byte aligned", what);
    const Requant fq = q ? make_requant(r, what) : Requant{};
    const int64_t blocks = std::min<int64_t>(ceil_div(ceil_div(n, 4), kThreads), 256 * 32);
    hipLaunchKernelGGL(gelu_erf, dim3(static_cast<uint32_t>(blocks)), dim3(kThreads), 0, as_stream(stream), x, y, q, n, fq);
    HIPIE_CHECK_HIP(hipGetLastError());
}

// Embedding lookup: one wavefront per token copies its table row (float4 per lane and step) and adds
// up to two addends in the graph's order.
__global__ __launch_bounds__(kThreads) void embedding_rows(const float* __restrict__ table, int64_t vocab, int hidden,
                                                           const int32_t* __restrict__ ids, int64_t tokens, int seq,
                                                           const float* __restrict__ add0, int pos0,
                                                           const float* __restrict__ add1, int pos1, float* __restrict__ out) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * (kThreads / 64) + (threadIdx.x >> 6);
    if (t >= tokens) return;
    const int lane = threadIdx.x & 63;
    int64_t idx = ids[t];
    if (idx < 0) idx += vocab;
    idx = idx < 0 ? 0 : (idx >= vocab ? vocab - 1 : idx);
    const int64_t p = t % seq;
    const float* src = table + idx * hidden;
    const float* a0 = add0 ? add0 + (pos0 ? p * hidden : 0) : nullptr;
    const float* a1 = add1 ? add1 + (pos1 ? p * hidden : 0) : nullptr;
    float* dst = out + t * hidden;
    for (int i = 4 * lane; i < hidden; i += 256) {
        float4 v = *reinterpret_cast<const float4*>(src + i);
        if (a0) {
            const float4 a = *reinterpret_cast<const float4*>(a0 + i);
            v.x = v.x + a.x; v.y = v.y + a.y; v.z = v.z + a.z; v.w = v.w + a.w;
        }
        if (a1) {
            const float4 a = *reinterpret_cast<const float4*>(a1 + i);
            v.x = v.x + a.x; v.y = v.y + a.y; v.z = v.z + a.z; v.w = v.w + a.w;
        }
        *reinterpret_cast<float4*>(dst + i) = v;
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
    return guarded([&] { run_softmax(x, y, nullptr, rows, axis, nullptr, stream, "hipie_softmax_f32"); });
}

int hipie_mvn_f32(const float* x, float* y, int64_t rows, int64_t axis, int normalize_variance, float eps,
                  int eps_inside_sqrt, const float* gamma, const float* beta, void* stream) {
    return guarded([&] {
        run_mvn(x, y, nullptr, rows, axis, normalize_variance, eps, eps_inside_sqrt, gamma, beta, nullptr, stream, "hipie_mvn_f32");
    });
}

int hipie_gelu_f32(const float* x, float* y, int64_t n, void* stream) {
    return guarded([&] { run_gelu(x, y, nullptr, n, nullptr, stream, "hipie_gelu_f32"); });
}

int hipie_add_broadcast_f32(const float* x, const int64_t* dims, const float* addend, const int64_t* addend_dims, int rank,
                            float* y, void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(x && dims && addend && addend_dims && y && rank >= 1 && rank <= 4, HIPIE_PARAMETER_MISMATCH,
                      "hipie_add_broadcast_f32: bad argument");
        int64_t d[4] = {1, 1, 1, 1}, md[4] = {1, 1, 1, 1}, ms[4] = {0, 0, 0, 0};
        for (int k = 0; k < rank; ++k) {
            d[4 - rank + k] = dims[k];
            md[4 - rank + k] = addend_dims[k];
        }
        int64_t n = 1, run = 1;
        for (int k = 3; k >= 0; --k) {
            HIPIE_REQUIRE(d[k] >= 0 && d[k] < (int64_t{1} << 31) && (md[k] == d[k] || md[k] == 1), HIPIE_PARAMETER_MISMATCH,
                          "hipie_add_broadcast_f32: dimension %lld of the addend against %lld", (long long)md[k], (long long)d[k]);
            ms[k] = md[k] == 1 ? 0 : run;
            run *= md[k];
            n *= d[k];
            HIPIE_REQUIRE(n < (int64_t{1} << 40), HIPIE_PARAMETER_MISMATCH, "hipie_add_broadcast_f32: too many elements");
        }
        if (n == 0) return;
        const int64_t blocks = std::min<int64_t>(ceil_div(n, kThreads), 256 * 32);
        hipLaunchKernelGGL(add_broadcast, dim3(static_cast<uint32_t>(blocks)), dim3(kThreads), 0, as_stream(stream), x, addend, y, n,
                           static_cast<int32_t>(d[1]), static_cast<int32_t>(d[2]), static_cast<int32_t>(d[3]), ms[0], ms[1], ms[2], ms[3]);
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_copy_strided(const void* src, const int64_t* dims, const int64_t* strides, int rank, int element_bytes, void* dst,
                       void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(src && dims && strides && dst && rank >= 1 && rank <= 5 && (element_bytes == 1 || element_bytes == 4),
                      HIPIE_PARAMETER_MISMATCH, "hipie_copy_strided: bad argument");
        int64_t d[5] = {1, 1, 1, 1, 1}, st[5] = {0, 0, 0, 0, 0}, n = 1;
        for (int k = 0; k < rank; ++k) {
            d[5 - rank + k] = dims[k];
            st[5 - rank + k] = strides[k];
            HIPIE_REQUIRE(dims[k] >= 0 && dims[k] < (int64_t{1} << 31) && strides[k] >= 0, HIPIE_PARAMETER_MISMATCH,
                          "hipie_copy_strided: dimension %d", k);
            n *= dims[k];
            HIPIE_REQUIRE(n < (int64_t{1} << 40), HIPIE_PARAMETER_MISMATCH, "hipie_copy_strided: too many elements");
        }
        if (n == 0) return;
        const dim3 grid(static_cast<uint32_t>(std::min<int64_t>(ceil_div(n, kThreads), 256 * 32))), block(kThreads);
        hipStream_t s = as_stream(stream);
        const int32_t d1 = static_cast<int32_t>(d[1]), d2 = static_cast<int32_t>(d[2]), d3 = static_cast<int32_t>(d[3]), d4 = static_cast<int32_t>(d[4]);
        if (element_bytes == 4)
            hipLaunchKernelGGL(copy_strided<uint32_t>, grid, block, 0, s, static_cast<const uint32_t*>(src), static_cast<uint32_t*>(dst), n, d1, d2,
                               d3, d4, st[0], st[1], st[2], st[3], st[4]);
        else
            hipLaunchKernelGGL(copy_strided<uint8_t>, grid, block, 0, s, static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), n, d1, d2, d3,
                               d4, st[0], st[1], st[2], st[3], st[4]);
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_softmax_q8(const float* x, float* y, int8_t* q, int64_t rows, int64_t axis, const hipie_requant* requant,
                     void* stream) {
    return guarded([&] { run_softmax(x, y, q, rows, axis, requant, stream, "hipie_softmax_q8"); });
}

int hipie_mvn_q8(const float* x, float* y, int8_t* q, int64_t rows, int64_t axis, int normalize_variance, float eps,
                 int eps_inside_sqrt, const float* gamma, const float* beta, const hipie_requant* requant, void* stream) {
    return guarded([&] {
        run_mvn(x, y, q, rows, axis, normalize_variance, eps, eps_inside_sqrt, gamma, beta, requant, stream, "hipie_mvn_q8");
    });
}

int hipie_gelu_q8(const float* x, float* y, int8_t* q, int64_t n, const hipie_requant* requant, void* stream) {
    return guarded([&] { run_gelu(x, y, q, n, requant, stream, "hipie_gelu_q8"); });
}

int hipie_embedding_f32(const float* table, int64_t vocabulary, int64_t hidden, const int32_t* ids, int64_t tokens,
                        int64_t seq, const float* add0, int add0_per_position, const float* add1, int add1_per_position,
                        float* out, void* stream) {
    return guarded([&] {
        if (tokens == 0) return;
        HIPIE_REQUIRE(table && ids && out && vocabulary > 0 && tokens > 0 && seq > 0 && hidden > 0 && hidden % 4 == 0 &&
                          hidden < (1ll << 31) && seq < (1ll << 31),
                      HIPIE_PARAMETER_MISMATCH, "hipie_embedding_f32: bad argument (hidden must be a multiple of 4)");
        for (const void* p : {static_cast<const void*>(table), static_cast<const void*>(add0), static_cast<const void*>(add1),
                              static_cast<const void*>(out)})
            HIPIE_REQUIRE(reinterpret_cast<uintptr_t>(p) % 16 == 0, HIPIE_PARAMETER_MISMATCH,
                          "hipie_embedding_f32: buffers must be 16-byte aligned");
        hipLaunchKernelGGL(embedding_rows, dim3(static_cast<uint32_t>(ceil_div(tokens, kThreads / 64))), dim3(kThreads), 0,
                           as_stream(stream), table, vocabulary, static_cast<int>(hidden), ids, tokens, static_cast<int>(seq),
                           add0, add0_per_position, add1, add1_per_position, out);
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
