// Layers the low-precision transformations leave in f32 (no FakeQuantize in front of them, or intervals the
// transformation does not take): Convolution, GroupConvolution and MatMul against f32 constants, and FakeQuantize with
// an f32 result.  One thread per output element, every sum in the order of the reference loops, one IEEE f32 operation per
// operation of the graph - a correct path for the few unquantized layers of an INT8 network, not a fast one.
#pragma once
#include "common.h"
#include "fq_math.h"

namespace hipie {

// A 4-D value [N, C, H, W] wherever it lives: element (n, c, h, w) at p + n sn + c sc + h sh + w sw (in elements).
// f32, or the bytes of a quantized tensor behind their dequantization (float(level) - sub[c]) * mul[c]: Convert,
// Subtract, Multiply as three operations, like the graph's nodes.
struct F32Source {
    const void* p = nullptr;
    int32_t dtype = HIPIE_F32;        // HIPIE_F32, HIPIE_U8B (level - 128 stored) or HIPIE_I8
    int64_t sn = 0, sc = 0, sh = 0, sw = 0;
    const float* sub = nullptr;       // one per channel, or null
    const float* mul = nullptr;
};

// reference::convolution<float> / reference::group_convolution<float> (convolution.hpp:63-146, group_convolution.hpp:78-144):
// sum = 0; for every input channel of the group, filter plane, filter row, filter column that is not padding: sum += x * w
// (convolve_3D_channels; one and two spatial dimensions are the same loops with unit extents in front).
// MatMul against a constant (matmul.hpp:24-57, sum over k ascending from 0) is the 1 x 1 case.
struct ConvF32Args {
    F32Source in;
    const float* wgt = nullptr;       // [C / G][KH][KW][OC]: the lanes of a wave read consecutive output channels
    float* out = nullptr;             // NHWC
    int64_t out_sn = 0, out_sh = 0, out_sw = 0;
    int32_t N = 0, C = 0, H = 0, W = 0, OC = 0, OH = 0, OW = 0;
    int32_t KH = 1, KW = 1, stride_h = 1, stride_w = 1, dil_h = 1, dil_w = 1, pad_top = 0, pad_left = 0;
    int32_t groups = 1;
    // three spatial dimensions: the values are [N, C, D * H, W] / [N, OC, OD * OH, OW] (depth and rows merged into the
    // row axis), filters [C / G][KD][KH][KW][OC]; D = 1 otherwise
    int32_t D = 1, OD = 1, KD = 1, stride_d = 1, dil_d = 1, pad_front = 0;
};
void launch_conv_f32(const ConvF32Args& a, hipStream_t s);

// reference::fake_quantize<float> (fake_quantize.hpp:175-194) with an f32 result; ch: one entry, or one per channel
struct FqF32Args {
    F32Source in;
    const FqChannel* ch = nullptr;
    int32_t per_channel = 0;
    float lm1 = 255.f;                // levels - 1
    float* out = nullptr;             // NHWC
    int64_t out_sn = 0, out_sh = 0, out_sw = 0;
    int32_t N = 0, C = 0, H = 0, W = 0;
    int32_t axis = 1;                 // Softmax only: 0 .. 3 of [N, C, H, W]
};
void launch_fq_f32(const FqF32Args& a, hipStream_t s);
// the same walk without the FakeQuantize (ch unused): a graph input as the NHWC f32 tensor the elementwise kernels read
void launch_copy_f32(const FqF32Args& a, hipStream_t s);
// reference::softmax (softmax.hpp:20-50) along `axis` of the same walk (ch, lm1 unused): for every position of the other
// three axes the maximum along the axis, exp(x - max), their sum, the quotients.  One wavefront per such row (over the
// channels, the usual case, its lanes read consecutive elements); exp is the device's, so the result agrees with the
// reference's to rounding, not bit for bit.
void launch_softmax_f32(const FqF32Args& a, hipStream_t s);


// reference::max_pool<float> / avg_pool<float> (max_pool.hpp, avg_pool.hpp:114-265): the window runs over the padded
// tensor and ends at its upper bound, padding cells are skipped (a maximum starts from lowest()); the mean adds the
// window's cells row by row - zeros for padding cells when they count - and divides by the cell count of the
// reference's rules (kernel area when padding counts and there is any, else the cells taken)
struct PoolF32Args {
    F32Source in;
    float* out = nullptr;             // NHWC
    int64_t out_sn = 0, out_sh = 0, out_sw = 0;
    int32_t N = 0, C = 0, H = 0, W = 0, OH = 0, OW = 0;
    int32_t kh = 1, kw = 1, sh = 1, sw = 1, pt = 0, pl = 0, pb = 0, pr = 0;
    int32_t avg = 0, include_pad = 0;
};
void launch_pool_f32(const PoolF32Args& a, hipStream_t s);

}  // namespace hipie
