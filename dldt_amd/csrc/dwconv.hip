// Depthwise GroupConvolution (groups == channels, one filter per channel): HBM-bound, no MFMA.
// Reference semantics: reference::group_convolution on widened inputs
// (ngraph/core/reference/.../group_convolution.hpp:78-144 looping convolution.hpp:63-146 over
// single-channel slices), then the same fused epilogue as the dense convolution.
//
// A lane owns 32 consecutive channels of two adjacent output pixels: every load is 2 x 16 B of
// one NHWC pixel, consecutive lanes read consecutive channel groups, padding comes from the
// tensor's halo.  Weights are packed [kh*kw][Cp] so a lane's 32 filter bytes of one tap are
// contiguous.  Traffic per output byte: ~1 B read (taps hit L1/L2) + 1 B written.
#include "conv.h"
#include "conv_epilogue.h"

namespace hipie {
namespace {

__device__ __forceinline__ void mac_bytes(uint32_t x, uint32_t w, int& a0, int& a1, int& a2, int& a3) {
    a0 += static_cast<int>(static_cast<int8_t>(x)) * static_cast<int>(static_cast<int8_t>(w));
    a1 += static_cast<int>(static_cast<int8_t>(x >> 8)) * static_cast<int>(static_cast<int8_t>(w >> 8));
    a2 += static_cast<int>(static_cast<int8_t>(x >> 16)) * static_cast<int>(static_cast<int8_t>(w >> 16));
    a3 += static_cast<int>(static_cast<int8_t>(x >> 24)) * static_cast<int>(static_cast<int8_t>(w >> 24));
}

template <uint32_t F>
__global__ __launch_bounds__(256) void dwconv_kernel(const ConvArgs a, int KH, int KW, int dil_h, int dil_w,
                                                     int cgroups, int64_t items) {
    const int64_t item = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (item >= items) return;
    const int cgi = static_cast<int>(item % cgroups);
    const int m0 = static_cast<int>(item / cgroups) * 2;
    const int oc_lane = cgi * 32;
    int32_t base[2];
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
        const int m = min(m0 + pb, a.M - 1);
        const PixelCoord p = decode_pixel(a, m);
        base[pb] = p.n * a.in_sn + p.oh * a.conv_sh * a.in_sh + p.ow * a.conv_sw * a.in_sw + a.in_origin + oc_lane;
    }
    v16i acc[2][2];
    init_acc(a, oc_lane, acc);
    for (int kh = 0; kh < KH; ++kh)
        for (int kw = 0; kw < KW; ++kw) {
            const int8_t* wp = a.wgt + static_cast<int64_t>(kh * KW + kw) * a.OCp + oc_lane;
            const uint4 w0 = *reinterpret_cast<const uint4*>(wp), w1 = *reinterpret_cast<const uint4*>(wp + 16);
            const uint32_t w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
            const int32_t tap = kh * dil_h * a.in_sh + kw * dil_w * a.in_sw;
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) {
                const int8_t* xp = a.in + (base[pb] + tap);
                const uint4 x0 = *reinterpret_cast<const uint4*>(xp), x1 = *reinterpret_cast<const uint4*>(xp + 16);
                const uint32_t x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const int ob = q >> 2, r0 = (q & 3) * 4;
                    int c0 = acc[ob][pb][r0], c1 = acc[ob][pb][r0 + 1], c2 = acc[ob][pb][r0 + 2], c3 = acc[ob][pb][r0 + 3];
                    mac_bytes(x[q], w[q], c0, c1, c2, c3);
                    acc[ob][pb][r0] = c0; acc[ob][pb][r0 + 1] = c1; acc[ob][pb][r0 + 2] = c2; acc[ob][pb][r0 + 3] = c3;
                }
            }
        }
    run_epilogue<F>(a, acc, oc_lane, m0, m0 + 1);
}

}  // namespace

void launch_dwconv(const ConvArgs& a, int KH, int KW, int dil_h, int dil_w, hipStream_t s) {
    const int cgroups = a.OCp / 32;
    const int64_t items = ceil_div(a.M, 2) * cgroups;
    const dim3 grid(static_cast<uint32_t>(ceil_div(items, 256))), block(256);
    const uint32_t core = a.flags & ~CF_OUT_XOR;
    switch (core) {
    case E_PLAIN0: hipLaunchKernelGGL((dwconv_kernel<E_PLAIN0>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items); break;
    case E_CLAMPFQ: hipLaunchKernelGGL((dwconv_kernel<E_CLAMPFQ>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items); break;
    default: hipLaunchKernelGGL((dwconv_kernel<kDyn>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items); break;
    }
}

}  // namespace hipie
