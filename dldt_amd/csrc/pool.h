// Argument blocks and launchers of the pooling / layout kernels.
#pragma once
#include "common.h"
#include "fq_math.h"

namespace hipie {

struct PoolArgs {
    const void* in;
    void* out;
    int32_t M, OW, OHOW;           // output pixels, output width, OH * OW
    int32_t H, W;                  // input spatial dims
    int32_t cs;                    // channels processed (padded channel count of the output)
    int32_t in_sn, in_sh, in_sw;   // element strides
    int32_t out_sn, out_sh, out_sw;
    int32_t kh, kw, sh, sw, pt, pl, pb, pr;
    int32_t include_pad;
    int32_t in_bias;               // 128 for U8B storage, 0 for I8
    int32_t preserve;              // AvgPool whose result has the input's type (precision preserved): 1 = u8 levels, 2 = i8;
                                   // the window sum is kept modulo 256 as the reference's element-typed accumulator keeps it
    // AvgPool tail: optional Multiply and FakeQuantize tables, each [cs]
    const float* mul;
    const float* fq_il;
    const float* fq_ih;
    const float* fq_d;
    const float* fq_r;
    float lm1, out_off;
};

struct ExitArgs {
    const void* in;
    void* out;
    int32_t N, C, HW, W;
    int32_t in_sn, in_sh, in_sw;
    float in_bias;                 // 128 for U8B storage
    const float* sub;              // optional dequantization (x - sub[c]) * mul[c], each [C]
    const float* mul;
    int32_t out_u8;
};

// Concat along the channel axis of byte NHWC tensors: one input's C channels copied to channels [c_off, c_off + C) of
// the output (reference::concat, concat.hpp:17-57, is the same copy in NCHW order).  Along N, H or W the caller moves
// `out` to the first element of the input's box and passes c_off = 0.
struct ConcatArgs {
    const int8_t* in;
    int8_t* out;
    int32_t N, H, W, C;
    int64_t in_sn, in_sh, in_sw, out_sn, out_sh, out_sw;   // bytes
    int32_t c_off;
};

void launch_max_pool(const PoolArgs& a, hipStream_t s);
void launch_concat_channels(const ConcatArgs& a, hipStream_t s);
void launch_avg_pool(const PoolArgs& a, bool rcp, hipStream_t s);
void launch_exit(const ExitArgs& a, int in_dtype, hipStream_t s);

}  // namespace hipie
