// f32 Convolution / GroupConvolution / MatMul against constants, FakeQuantize with an f32 result, MaxPool / AvgPool of f32
// values, Softmax along one axis: the layers of an INT8 network that the low-precision transformations leave
// unquantized.  See convf.h.
#include "convf.h"

namespace hipie {
namespace {

__device__ __forceinline__ float source_value(const F32Source& s, int n, int c, int h, int w) {
    const int64_t i = n * s.sn + c * s.sc + h * s.sh + w * s.sw;
    if (s.dtype == HIPIE_F32) return static_cast<const float*>(s.p)[i];
    const int level = static_cast<int>(static_cast<const int8_t*>(s.p)[i]) + (s.dtype == HIPIE_U8B ? 128 : 0);
    float v = static_cast<float>(level);            // Convert
    if (s.sub) v = v - s.sub[c];                    // Subtract
    if (s.mul) v = v * s.mul[c];                    // Multiply
    return v;
}

__global__ __launch_bounds__(256) void conv_f32_kernel(const ConvF32Args a) {
    const int64_t total = static_cast<int64_t>(a.N) * a.OD * a.OH * a.OW * a.OC;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int oc = static_cast<int>(i % a.OC);
    int64_t p = i / a.OC;
    const int ow = static_cast<int>(p % a.OW);
    p /= a.OW;
    const int oh = static_cast<int>(p % a.OH);
    p /= a.OH;
    const int od = static_cast<int>(p % a.OD);
    const int n = static_cast<int>(p / a.OD);
    const int cg = a.C / a.groups, ocg = a.OC / a.groups;
    const int c0 = (oc / ocg) * cg;
    const int z0 = od * a.stride_d - a.pad_front, y0 = oh * a.stride_h - a.pad_top, x0 = ow * a.stride_w - a.pad_left;
    const float* w = a.wgt + oc;
    float sum = 0.f;
    for (int c = 0; c < cg; ++c)
        for (int kd = 0; kd < a.KD; ++kd) {
            const int z = z0 + kd * a.dil_d;
            for (int kh = 0; kh < a.KH; ++kh) {
                const int y = y0 + kh * a.dil_h;
                for (int kw = 0; kw < a.KW; ++kw) {
                    const int x = x0 + kw * a.dil_w;
                    if (z < 0 || z >= a.D || y < 0 || y >= a.H || x < 0 || x >= a.W) continue;   // padding cells are skipped, not added as zeros
                    const float prod = source_value(a.in, n, c0 + c, z * a.H + y, x) *
                                       w[static_cast<int64_t>(((c * a.KD + kd) * a.KH + kh) * a.KW + kw) * a.OC];
                    sum = sum + prod;
                }
            }
        }
    a.out[n * a.out_sn + (od * a.OH + oh) * a.out_sh + ow * a.out_sw + oc] = sum;
}

template <bool QUANTIZE>
__global__ __launch_bounds__(256) void fq_f32_kernel(const FqF32Args a) {
    const int64_t total = static_cast<int64_t>(a.N) * a.H * a.W * a.C;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int c = static_cast<int>(i % a.C);
    int64_t p = i / a.C;
    const int w = static_cast<int>(p % a.W);
    p /= a.W;
    const int h = static_cast<int>(p % a.H);
    const int n = static_cast<int>(p / a.H);
    float v = source_value(a.in, n, c, h, w);
    if constexpr (QUANTIZE) v = fq_value<false>(a.ch[a.per_channel ? c : 0], a.lm1, v);
    a.out[n * a.out_sn + h * a.out_sh + w * a.out_sw + c] = v;
}

// one wavefront per row along the axis, its lanes striding over the row: maximum, exp and sum (the exponentials parked
// in the output), quotients
__global__ __launch_bounds__(256) void softmax_f32_kernel(const FqF32Args a) {
    int d[4] = {a.N, a.C, a.H, a.W};
    const int len = d[a.axis];
    d[a.axis] = 1;
    const int64_t rows = static_cast<int64_t>(d[0]) * d[1] * d[2] * d[3];
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    // the row's position on the other axes, channels fastest
    int at[4];
    at[1] = static_cast<int>(row % d[1]);
    int64_t p = row / d[1];
    at[3] = static_cast<int>(p % d[3]);
    p /= d[3];
    at[2] = static_cast<int>(p % d[2]);
    at[0] = static_cast<int>(p / d[2]);
    const int64_t out_stride[4] = {a.out_sn, 1, a.out_sh, a.out_sw};
    float* out = a.out + at[0] * a.out_sn + at[1] + at[2] * a.out_sh + at[3] * a.out_sw;
    const int64_t step = out_stride[a.axis];
    auto value = [&](int i) {
        int q[4] = {at[0], at[1], at[2], at[3]};
        q[a.axis] = i;
        return source_value(a.in, q[0], q[1], q[2], q[3]);
    };
    float m = -INFINITY;
    for (int i = lane; i < len; i += 64) m = fmaxf(m, value(i));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    float sum = 0.f;
    for (int i = lane; i < len; i += 64) {
        const float e = expf(value(i) - m);
        out[i * step] = e;
        sum += e;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    for (int i = lane; i < len; i += 64) out[i * step] = out[i * step] / sum;     // each lane reads back what it wrote itself
}

__global__ __launch_bounds__(256) void pool_f32_kernel(const PoolF32Args a) {
    const int64_t total = static_cast<int64_t>(a.N) * a.OH * a.OW * a.C;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const int c = static_cast<int>(i % a.C);
    int64_t p = i / a.C;
    const int ow = static_cast<int>(p % a.OW);
    p /= a.OW;
    const int oh = static_cast<int>(p % a.OH);
    const int n = static_cast<int>(p / a.OH);
    // window in the coordinates of the padded tensor, cut at its upper bound
    const int y0 = a.sh * oh, x0 = a.sw * ow;
    const int y1 = min(y0 + a.kh, a.H + a.pt + a.pb), x1 = min(x0 + a.kw, a.W + a.pl + a.pr);
    const bool padding_present = a.pt != 0 || a.pl != 0 || a.pb != 0 || a.pr != 0;
    float r = a.avg ? 0.f : -3.402823466e+38f;
    int count = a.avg && a.include_pad && padding_present ? a.kh * a.kw : 0;
    for (int y = y0; y < y1; ++y)
        for (int x = x0; x < x1; ++x) {
            const int iy = y - a.pt, ix = x - a.pl;
            const bool inside = iy >= 0 && iy < a.H && ix >= 0 && ix < a.W;
            if (!a.avg) {
                if (inside) {
                    const float v = source_value(a.in, n, c, iy, ix);
                    r = v > r ? v : r;
                }
            } else if (inside || a.include_pad) {
                const float v = inside ? source_value(a.in, n, c, iy, ix) : 0.0f;
                r = r + v;
                if (!padding_present || (inside && !a.include_pad)) ++count;
            }
        }
    if (a.avg) r = r / static_cast<float>(count);
    a.out[n * a.out_sn + oh * a.out_sh + ow * a.out_sw + c] = r;
}

void check_source(const F32Source& s, const char* what) {
    HIPIE_REQUIRE(s.p && (s.dtype == HIPIE_F32 || s.dtype == HIPIE_U8B || s.dtype == HIPIE_I8), HIPIE_PARAMETER_MISMATCH,
                  "%s: input of type %d", what, s.dtype);
    HIPIE_REQUIRE(s.dtype != HIPIE_F32 || (!s.sub && !s.mul), HIPIE_PARAMETER_MISMATCH, "%s: dequantization constants on an f32 input", what);
}

}  // namespace

void launch_conv_f32(const ConvF32Args& a, hipStream_t s) {
    check_source(a.in, "f32 convolution");
    HIPIE_REQUIRE(a.wgt && a.out && a.N > 0 && a.C > 0 && a.H > 0 && a.W > 0 && a.OC > 0 && a.OH > 0 && a.OW > 0 && a.KH > 0 && a.KW > 0 &&
                      a.stride_h > 0 && a.stride_w > 0 && a.dil_h > 0 && a.dil_w > 0 && a.groups > 0 && a.C % a.groups == 0 &&
                      a.OC % a.groups == 0 && a.D > 0 && a.OD > 0 && a.KD > 0 && a.stride_d > 0 && a.dil_d > 0,
                  HIPIE_PARAMETER_MISMATCH, "f32 convolution: shape");
    const int64_t total = static_cast<int64_t>(a.N) * a.OD * a.OH * a.OW * a.OC;
    const int64_t blocks = ceil_div(total, 256);
    HIPIE_REQUIRE(blocks < (int64_t{1} << 31), HIPIE_PARAMETER_MISMATCH, "f32 convolution: %lld outputs", (long long)total);
    hipLaunchKernelGGL(conv_f32_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s, a);
    HIPIE_CHECK_HIP(hipGetLastError());
}

static void launch_elementwise_f32(const FqF32Args& a, bool quantize, hipStream_t s) {
    const char* what = quantize ? "f32 FakeQuantize" : "f32 copy";
    check_source(a.in, what);
    HIPIE_REQUIRE((a.ch || !quantize) && a.out && a.N > 0 && a.C > 0 && a.H > 0 && a.W > 0 && a.lm1 >= 1.f, HIPIE_PARAMETER_MISMATCH, "%s: shape", what);
    const int64_t total = static_cast<int64_t>(a.N) * a.H * a.W * a.C;
    const int64_t blocks = ceil_div(total, 256);
    HIPIE_REQUIRE(blocks < (int64_t{1} << 31), HIPIE_PARAMETER_MISMATCH, "%s: %lld elements", what, (long long)total);
    if (quantize) hipLaunchKernelGGL(fq_f32_kernel<true>, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(fq_f32_kernel<false>, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s, a);
    HIPIE_CHECK_HIP(hipGetLastError());
}

void launch_pool_f32(const PoolF32Args& a, hipStream_t s) {
    check_source(a.in, "f32 pooling");
    HIPIE_REQUIRE(a.out && a.N > 0 && a.C > 0 && a.H > 0 && a.W > 0 && a.OH > 0 && a.OW > 0 && a.kh > 0 && a.kw > 0 && a.sh > 0 && a.sw > 0 &&
                      a.pt >= 0 && a.pl >= 0 && a.pb >= 0 && a.pr >= 0,
                  HIPIE_PARAMETER_MISMATCH, "f32 pooling: shape");
    const int64_t total = static_cast<int64_t>(a.N) * a.OH * a.OW * a.C;
    const int64_t blocks = ceil_div(total, 256);
    HIPIE_REQUIRE(blocks < (int64_t{1} << 31), HIPIE_PARAMETER_MISMATCH, "f32 pooling: %lld outputs", (long long)total);
    hipLaunchKernelGGL(pool_f32_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s, a);
    HIPIE_CHECK_HIP(hipGetLastError());
}

void launch_softmax_f32(const FqF32Args& a, hipStream_t s) {
    check_source(a.in, "f32 Softmax");
    HIPIE_REQUIRE(a.out && a.N > 0 && a.C > 0 && a.H > 0 && a.W > 0 && a.axis >= 0 && a.axis <= 3, HIPIE_PARAMETER_MISMATCH, "f32 Softmax: shape");
    HIPIE_REQUIRE(static_cast<const void*>(a.out) != a.in.p, HIPIE_PARAMETER_MISMATCH, "f32 Softmax: in place");
    const int len = a.axis == 0 ? a.N : (a.axis == 1 ? a.C : (a.axis == 2 ? a.H : a.W));
    const int64_t rows = static_cast<int64_t>(a.N) * a.C * a.H * a.W / len;
    const int64_t blocks = ceil_div(rows, 4);
    HIPIE_REQUIRE(blocks < (int64_t{1} << 31), HIPIE_PARAMETER_MISMATCH, "f32 Softmax: %lld rows", (long long)rows);
    hipLaunchKernelGGL(softmax_f32_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s, a);
    HIPIE_CHECK_HIP(hipGetLastError());
}

void launch_fq_f32(const FqF32Args& a, hipStream_t s) { launch_elementwise_f32(a, true, s); }
void launch_copy_f32(const FqF32Args& a, hipStream_t s) { launch_elementwise_f32(a, false, s); }

}  // namespace hipie
