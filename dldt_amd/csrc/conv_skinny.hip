// 1 x 1 convolution / MatMul against constant weights over FEW pixels and many channels (the FC layer of a
// classifier: 64 rows x 2048 -> 1000), as dot products on the vector pipe.
//
// Why not the matrix kernels: 64 pixels are half a pixel tile, so such a layer is 8 tiles of 128 channels - 8 of the
// chip's 256 compute units, each walking K = 2048 alone (19 us in a batch-64 ResNet-50, mostly the latency of its own
// weight stream).  Splitting K over workgroups helps only as far as the tile count allows.  Here a workgroup owns 64
// output channels (a lane per channel) and 8 pixels; its four waves take a quarter of K each, request their whole
// part of the weights at once (K-major packing: the 16 K bytes of 64 neighbouring channels are 1 KiB, one load per
// wave), read the pixels' bytes as broadcasts from LDS (the same for every lane) and meet in LDS for the sum:
// 128 workgroups for the FC layer, one latency instead of a dependent chain of them.
// Reference semantics as for the other kernels: reference::convolution<int32_t> / reference::matmul<int32_t> on
// widened inputs (ngraph/core/reference/include/ngraph/runtime/reference/convolution.hpp:63-146, matmul.hpp:24-57);
// integer sums do not depend on the order of the additions, the f32 tail is evaluated one IEEE operation at a time.
#include "conv.h"
#include "conv_epilogue.h"

namespace hipie {
namespace {

constexpr int kSkinnyPix = 8;      // pixels per workgroup
constexpr int kSkinnyPieces = 32;  // 16-byte weight pieces per lane and round: a quarter of K = 2048

__global__ __launch_bounds__(256) void conv_skinny_kernel(const ConvArgs a) {
    constexpr int P = kSkinnyPix, NP = kSkinnyPieces;
    __shared__ int32_t part[4][P][64];
    extern __shared__ __attribute__((aligned(16))) int8_t rows[];   // [P][Kp]: the workgroup's pixels
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int oc = blockIdx.x * 64 + lane;                       // < OCp: the tables and the packed weights hold it
    const int m0 = blockIdx.y * P;
    // a.wgt2: [Kp / 16][OCp] pieces of 16 K bytes; this wave's quarter of them, requested before anything else
    const int n16 = a.Kp >> 4, quarter = (n16 + 3) >> 2;
    const int k_begin = wave * quarter, k_end = min(k_begin + quarter, n16);
    const uint4* const wk = reinterpret_cast<const uint4*>(a.wgt2) + oc;
    uint4 w[NP];
#pragma unroll
    for (int j = 0; j < NP; ++j) w[j] = wk[static_cast<int64_t>(min(k_begin + j, k_end - 1)) * a.OCp];
    // the pixels' rows into LDS (read back as broadcasts: every lane of a wave needs the same 16 bytes; through the
    // scalar cache the 256 reads of a wave, each awaited before the next batch, were most of the kernel's time)
    for (int i = tid; i < P * n16; i += 256) {
        const int p = i / n16, k = i - p * n16;
        const int m = min(m0 + p, a.M - 1);
        const int off = window_offset(a, m, a.in_sn, a.in_sh, a.in_sw, a.conv_sh, a.conv_sw, a.flat_in != 0) + a.in_origin;
        *reinterpret_cast<uint4*>(rows + (p * n16 + k) * 16) = *reinterpret_cast<const uint4*>(a.in + off + 16 * k);
    }
    __syncthreads();
    int acc[P];
#pragma unroll
    for (int p = 0; p < P; ++p) acc[p] = 0;
    for (int k0 = k_begin; k0 < k_end; k0 += NP) {               // one round for K <= 2048
        if (k0 != k_begin) {
#pragma unroll
            for (int j = 0; j < NP; ++j) w[j] = wk[static_cast<int64_t>(min(k0 + j, k_end - 1)) * a.OCp];
        }
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            if (k0 + j < k_end) {                                // uniform
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    const uint4 xv = *reinterpret_cast<const uint4*>(rows + (p * n16 + k0 + j) * 16);   // uniform address
                    acc[p] = __builtin_amdgcn_sdot4(static_cast<int>(xv.x), static_cast<int>(w[j].x), acc[p], false);
                    acc[p] = __builtin_amdgcn_sdot4(static_cast<int>(xv.y), static_cast<int>(w[j].y), acc[p], false);
                    acc[p] = __builtin_amdgcn_sdot4(static_cast<int>(xv.z), static_cast<int>(w[j].z), acc[p], false);
                    acc[p] = __builtin_amdgcn_sdot4(static_cast<int>(xv.w), static_cast<int>(w[j].w), acc[p], false);
                }
            }
        }
    }
#pragma unroll
    for (int p = 0; p < P; ++p) part[wave][p][lane] = acc[p];
    __syncthreads();
    // wave w finishes pixels w and w + 4
    const uint32_t fl = a.flags;
#pragma unroll
    for (int q = 0; q < P / 4; ++q) {
        const int p = wave + 4 * q, m = m0 + p;
        const int sum = part[0][p][lane] + part[1][p][lane] + part[2][p][lane] + part[3][p][lane] + a.corr[oc];
        if (m >= a.M || oc >= a.out_sw) continue;                // (out_sw: the output pixel's stride = its padded channels)
        const PixelCoord c = decode_pixel(a, m);
        const int64_t off = static_cast<int64_t>(c.n) * a.out_sn + c.oh * a.out_sh + c.ow * a.out_sw + oc;
        if (fl & CF_OUT_I32) {
            static_cast<int32_t*>(a.out)[off] = sum;
            continue;
        }
        float v = static_cast<float>(sum);
        if (fl & CF_BIAS) v = v + a.bias[oc];
        if (fl & CF_SCALE) v = v * a.scale[oc];
        if (fl & CF_RELU) v = v > 0.f ? v : 0.f;
        static_cast<float*>(a.out)[off] = v;
    }
}

}  // namespace

// the epilogues the kernel evaluates: raw sums, or bias / scale / ReLU to f32
bool skinny_epilogue_fits(uint32_t flags) {
    const uint32_t core = flags & ~CF_OUT_XOR;
    return core == CF_OUT_I32 || (core & ~(CF_BIAS | CF_SCALE | CF_RELU)) == 0;
}

void launch_skinny(const ConvArgs& a, hipStream_t s) {
    const dim3 grid(static_cast<uint32_t>(a.OCp / 64), static_cast<uint32_t>(ceil_div(a.M, kSkinnyPix)));
    hipLaunchKernelGGL(conv_skinny_kernel, grid, dim3(256), static_cast<size_t>(kSkinnyPix) * a.Kp, s, a);
}

}  // namespace hipie
