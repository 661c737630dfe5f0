// u8/i8 x i8 -> i32 implicit-GEMM convolution on CDNA4 int8 MFMA with a fused f32 epilogue.
//
// Reference semantics: reference::convolution<int32_t> on widened inputs
// (ngraph/core/reference/.../convolution.hpp:63-146) followed by the post-LPT elementwise chain
// (Add bias, Multiply, residual Add, ReLU/Clamp, FakeQuantize) evaluated one IEEE f32 operation
// at a time in graph order, so the u8 levels are the reference's bit for bit.
//
// GEMM view: rows = output channels (MFMA A operand, packed weights [OCp][Kp]), columns = output
// pixels (MFMA B operand, NHWC activations gathered through a per-16-byte offset table),
// K = (kh, kw, ic).  v_mfma_i32_32x32x32_i8: lane l feeds row/col l%32 with the 16 K-bytes
// starting at 16*(l/32); it receives rows 8*(r/4) + 4*(l/32) + r%4 of column l%32.
// Weight rows are stored permuted inside every group of 64 channels (packed row 32*ob + i holds
// channel 32*((i>>2)&1) + 16*ob + 4*(i>>3) + (i&3)), so each lane ends up with 32 CONSECUTIVE
// output channels of one pixel and results leave as 16-byte stores into NHWC.
//
// Two kernels share the epilogue:
//   conv_stream_kernel  channel tile 64, the whole [64][K] weight slab resident in LDS for the
//                       life of a persistent workgroup, activations loaded from global memory
//                       straight into MFMA operand registers (no barrier in the loop, loads of
//                       the next K step / next pixel tile in flight during MFMAs and epilogue).
//                       For the HBM-bound layers (small K * OC).
//   conv_tiled_kernel   (WOC*64) channels x (WPIX*64) pixels per workgroup, both operands staged
//                       through double-buffered LDS (rows 64 B + 16 B pad: conflict-free
//                       ds_read_b128), one barrier per 64-byte K step.  For the MFMA-bound layers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hipie {

enum ConvFlags : uint32_t {
    CF_BIAS = 1u << 0,        // v += bias[c]
    CF_SCALE = 1u << 1,       // v *= scale[c]
    CF_RES = 1u << 2,         // residual operand present
    CF_RES_F32 = 1u << 3,     // residual is f32 (else U8B / I8 bytes converted to float)
    CF_RES_SUB = 1u << 4,     // r -= res_sub[c]
    CF_RES_MUL = 1u << 5,     // r *= res_mul[c]
    CF_POST_SCALE = 1u << 6,  // v *= post_scale[c]   (after the residual add)
    CF_RELU = 1u << 7,        // v = v > 0 ? v : 0
    CF_CLAMP = 1u << 8,       // v = clamp(v, clamp_lo, clamp_hi)
    CF_OUT_FQ = 1u << 9,      // FakeQuantize -> one byte per element
    CF_OUT_I32 = 1u << 10,    // raw accumulators (integer parity tests, MatMul without epilogue)
    CF_FQ_RCP = 1u << 11,     // reciprocal evaluation of the FQ division (proven at load time)
    CF_RES_U8B = 1u << 12,    // residual bytes are level-128 (add 128 after conversion)
    CF_FQ_IL0 = 1u << 13,     // every input_low is +0: x - il == x
    CF_OUT_XOR = 1u << 14,    // packed levels ^ 0x80808080 is the stored byte (offset -128)
    CF_FQ_DIV2 = 1u << 16,    // two-operation division by the channel constant: fma(n, fq_r, n * fq_r2), verified at load time
    CF_GELU = 1u << 17,       // v = gelu(v), ERF mode (after scale / residual, in place of relu / clamp)
    CF_FQ_SAT = 1u << 18,     // 256 levels: the packing conversion's own saturation to 0 .. 255 stands for both saturating branches
    CF_OUT_ADD = 1u << 19,    // stored byte = level + out_off by a bytewise add (offsets other than 0 and -128)
    CF_RES_GEMM = 1u << 15,   // residual = (float(acc2) + bias2[c]) * scale2[c] of a second GEMM run in the same kernel
};

// VALU instructions per output element of the epilogue's f32 chain (each of the graph's f32 operations is one
// instruction here; a byte conversion or bytewise offset of a packed dword counts a quarter per element): what the
// vector pipe has to issue for a layer's results whatever the kernel's shape.
inline double epilogue_valu_ops(uint32_t f) {
    if (f & CF_OUT_I32) return 0.0;
    double n = 1.0;                                         // i32 -> f32 (the integer correction rides in the accumulator)
    if (f & CF_BIAS) n += 1;
    if (f & CF_SCALE) n += 1;
    if (f & CF_RES) {
        if (f & CF_RES_GEMM) n += 3;                        // the second accumulator: conversion, bias, scale
        else if (!(f & CF_RES_F32)) n += (f & CF_RES_U8B) ? 1.25 : 1.0;
        if (f & CF_RES_SUB) n += 1;
        if (f & CF_RES_MUL) n += 1;
        n += 1;                                             // the Add
    }
    if (f & CF_POST_SCALE) n += 1;
    if (f & CF_RELU) n += 1;
    if (f & CF_CLAMP) n += (f & CF_OUT_FQ) ? 1 : 2;
    if (f & CF_GELU) n += 30;                               // erf by its polynomial
    if (f & CF_OUT_FQ) {
        if (!(f & CF_FQ_SAT)) n += 1;                       // median of three for the saturating branches
        if (!(f & CF_FQ_IL0)) n += 1;                       // x - input_low
        n += (f & CF_FQ_DIV2) ? 2 : ((f & CF_FQ_RCP) ? 5 : 10);
        n += 2;                                             // * (levels - 1), rounding conversion into its byte
        if (f & CF_OUT_XOR) n += 0.25;
        if (f & CF_OUT_ADD) n += 1.25;
    }
    return n;
}


struct ConvArgs {
    const int8_t* in;     // element (n=0, h=0, w=0, c=0) of the input tensor
    const int8_t* wgt;    // packed [OCp][Kp]
    void* out;            // element (0,0,0,0) of the output tensor
    const void* res;      // residual tensor or nullptr
    const int32_t* koff;  // [Kp/16] byte offset of every 16-byte K piece relative to the window origin
    // per-channel tables, each [OCp]
    const int32_t* corr;  // 128 * sum_k w[oc][k] for U8B inputs (0 for I8)
    const float* bias;
    const float* scale;
    const float* res_sub;
    const float* res_mul;
    const float* post_scale;
    const float* fq_il;
    const float* fq_ih;
    const float* fq_d;
    const float* fq_r;
    const float* fq_r2;
    int32_t M;            // N * OH * OW
    int32_t OW, OHOW;
    float inv_OW, inv_OHOW;          // for the reciprocal pixel decode (M < 2^24)
    int32_t in_sn, in_sh, in_sw;     // input strides in bytes
    int32_t conv_sh, conv_sw;        // convolution strides
    int32_t in_origin;               // -(pad_top * in_sh + pad_left * in_sw)
    int32_t out_sn, out_sh, out_sw;  // output strides in elements
    int32_t res_sn, res_sh, res_sw;  // residual strides in elements
    int32_t OC, OCp;
    int32_t nk;                      // Kp / 64
    int32_t Kp;
    int32_t p_tiles, t_tiles, p_per_xcd;
    int32_t t_shift;                 // log2(t_tiles) when it is a power of two, else -1 (tile decode by shifts)
    uint32_t flags;
    float lm1, out_off, clamp_lo, clamp_hi;
    // batched MatMul (grid.y = batch): per-batch strides in bytes (operands) / elements (out, res);
    // wgt_ld = row stride of the weight-side operand, wgt_rows = rows that exist (others clamped),
    // wgt_plain = rows are in natural order (activation operand): the loader applies the MFMA
    // row permutation that constant weights carry from packing
    int64_t batch_in, batch_wgt, batch_out, batch_res;
    // two-level batches (sequence, head): batch index y -> (y / batch_inner) * outer stride + (y % batch_inner) * stride;
    // batch_inner = 0 means one level
    int32_t batch_inner;
    int64_t batch_in_o, batch_wgt_o, batch_out_o;
    int32_t batch_corr;              // accumulator corrections per batch element: entries from one batch's row to the next (0: one row for all)
    // batched MatMul with a u8 right operand: one integer per output ROW (pixel), added to every accumulator of the
    // row in front of the epilogue; batch element b's rows start at pix_corr + b * batch_pix_corr.  nullptr: none
    const int32_t* pix_corr;
    int32_t batch_pix_corr;
    int32_t wgt_ld, wgt_rows, wgt_plain;
    // fused shortcut convolution (CF_RES_GEMM): a second operand set accumulated first; its
    // dequantised result stays in registers as the residual of the main convolution
    const int8_t* in2;
    const int8_t* wgt2;
    const int32_t* koff2;
    const int32_t* corr2;
    const float* bias2;
    const float* scale2;
    int32_t in2_sn, in2_sh, in2_sw, conv2_sh, conv2_sw, in2_origin, nk2, Kp2;
    // the input / output / residual tensor is dense in (n, h, w) for this convolution: no pixel decode
    int32_t flat_in, flat_out, flat_res;
    // the K pieces of the convolution (of the fused shortcut) lie one behind the other in memory: koff[p] == 16 p
    int32_t k_linear, k_linear2;
    // grouped convolution in its own form: channel tile t (64 channels) reads its K offsets at koff + t * koff_tile
    int32_t koff_tile;
    // row-tile kernel (3 x 3, stride 1): output rows per tile, tiles per image, patch width OW + 2 and its reciprocal
    int32_t rows_per_tile, tiles_per_image, patch_w;
    float inv_patch_w;
    // first-layer kernel (few channels, one 32-byte K slice per filter row): filter rows, patch rows, padding
    int32_t stem_kh, stem_patch_rows, stem_pad_top, stem_pad_left;
    // K split over workgroups (pipelined kernel, grid.z = ksplit): partial accumulators of tile i, part z at
    // ws_part + (i * ksplit + z) * 64 * threads dwords, arrival counter of tile i at ws_count[i] (zero between launches)
    int32_t ksplit;
    int32_t* ws_part;
    uint32_t* ws_count;
};

}  // namespace hipie
