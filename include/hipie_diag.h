/* hipie_diag.h - tuning knobs and diagnostics of libhipie.so.
 *
 * Nothing here replaces an interface of the reference: these entry points choose among kernel variants that all compute
 * the same bits (what hipie_compile does by measurement at load time), expose constants the library derives, or measure
 * what the device itself delivers so that a kernel's roofline fraction can be read against it.  The interfaces the
 * library stands in for are in hipie.h. */
#ifndef HIPIE_DIAG_H
#define HIPIE_DIAG_H

#include "hipie.h"

#ifdef __cplusplus
extern "C" {
#endif

/* kernel variant: 0 = LDS-tiled 128 channels x 128 pixels, 1 = 64 x 256, 2 = 64 x 64, 3 = streaming
 * (weights resident in LDS), 4 / 5 = 128 x 128 / 64 x 256 with a multi-stage direct-to-LDS K pipeline,
 * 6 / 7 = the same two with eight waves that split the K steps between two wave groups (for layers
 * with fewer tiles than compute units; needs an even number of 64-byte K steps), 8 / 9 = 128 x 128 /
 * 64 x 256 persistent workgroups that prefetch the next pixel tile during the epilogue (small K; byte
 * outputs with a byte residual or none), 10 / 11 = 128 x 128 / 64 x 256 requesting the operands of two K
 * steps together (whole 128-byte lines per row), 12 = whole output rows of one image x 64 channels per
 * workgroup with the input patch and the nine weight slices staged once in LDS (3 x 3, stride 1, pad 1,
 * undilated, input channels a multiple of 64; rows too wide for a patch run variant 0), 13 = the same idea for
 * a first layer (4-byte pixels, filter rows of 5 to 8 taps, undilated: one 32-byte K slice per filter row; a
 * patch that would overhang the tensor's halo runs variant 1), 14 to 17 = variant 4 with the K steps of a tile
 * split over 2 / 4 / 8 / 16 workgroups (for launches with fewer tiles than compute units; at least two K steps per
 * part; launches of more than 2048 workgroups run variant 4).  The partial sums of variants 14 to 17 pass through a
 * workspace that the library keeps per (device, stream): it is allocated by the first such launch on a stream
 * (which therefore must not be under graph capture) and kept until the process ends.  18 to 22 = 128 x 128 tiles
 * whose K step is a whole cache line of every operand row, 23 = the few-pixel kernel (unpadded 1 x 1 over pixels of
 * a multiple of 64 bytes, raw sums or a bias / scale / ReLU tail to f32: a lane per output channel on the vector
 * pipe, K split over the waves of a workgroup; the FC layer of a classifier), 24 = whole output rows of one image x
 * all 64, 128 or 256 output channels per workgroup, the input patch (every channel) staged once in LDS and the
 * weights streamed through an LDS ring (3 x 3, stride 1, pad 1, undilated, dense pixels of a multiple of 64 channels,
 * bias + 256-level FakeQuantize from 0; rows too wide for a tile run variant 0).  A default is chosen
 * from the shape; hipie_compile times the variants on the device and keeps the fastest.  Every
 * variant produces the same bits.
 * A depthwise convolution (group_convolution.hpp:78-144 with one filter per channel) has three variants of its own:
 * 0 = every lane computes its outputs from registers loaded straight from memory, 1 = the input rows under seven
 * output rows of a strip of columns are staged once in LDS and a lane slides the 3 x 3 window over them in registers
 * (3 x 3, undilated, stride 1 or 2, pixels of at most 1024 bytes, FakeQuantize epilogue without residual), 2 = the
 * taps' diagonal weight matrices on the matrix pipe, 256 pixels x 64 channels per workgroup from an input patch staged
 * once in LDS (3 x 3, undilated, stride 1 or 2, padding 1 on the top and left, input with a border of one pixel;
 * an output row wider than 256 pixels runs variant 0). */
int hipie_conv_set_tile(hipie_conv* conv, int tile);
int hipie_conv_get_tile(const hipie_conv* conv, int* tile);
/* diagnostics: the epilogue's step flags (conv_kernel.h ConvFlags) and whether a kernel instance with
 * these steps compiled in exists (otherwise the generic, slower instance runs) */
int hipie_conv_epilogue_flags(const hipie_conv* conv, uint32_t* flags, int* specialised);
/* ring depth of the pipelined variants: 3, 4, 6 or 8 K steps in LDS (other values round down, and to
 * what fits 144 KB); 0 = the variant's default (4 for tile 4, else 3).  Variant 24 and hipie_conv_run_pair (the
 * setting of its first layer): 6 and more = nine steps of weights in flight in a wave's registers and one workgroup
 * per compute unit (for a launch that runs alone), else three steps and two workgroups; hipie_conv_run_pair only:
 * 7 = eight waves in two groups that split the first layer's input channels and take the second layer's passes in
 * turn (where hipie_conv_pair_fits reports bit 1; HIPIE_NOT_IMPLEMENTED elsewhere) */
int hipie_conv_set_stages(hipie_conv* conv, int stages);

/* Constants of the convolution epilogue's two-operation division: for each divisor d[i] a pair with
 * fma(x, zh[i], x * zl[i]) == x / d[i] for every float x, checked on the device against IEEE division
 * over all 2^23 significands.  *verified = 1 when every divisor has a pair (otherwise the epilogue
 * keeps the reciprocal-with-corrections sequence and zh, zl are unspecified). */
int hipie_fq_div2_constants(int device, const float* d, int64_t n, float* zh, float* zl, int* verified);

/* Diagnostics, no counterpart in the reference: the int8 rate (TOP/s) the device sustains when every SIMD issues
 * v_mfma_i32_32x32x32_i8 back to back from registers (waves_per_simd waves of 4 x iterations independent instructions,
 * no memory traffic) - the ceiling a kernel's roofline fraction can be read against beside the published peak. */
int hipie_probe_mfma_rate(int device, int iterations, int waves_per_simd, double* tops, double* milliseconds);
/* The LDS read rate the device sustains: waves_per_simd (1 .. 4) waves on every SIMD read 1 KB per ds_read_b128 from
 * conflict-free rows, eight reads per iteration (an even count), issued a step ahead of their use; with_mfma = 1 runs
 * one v_mfma_i32_32x32x32_i8 per read meanwhile (the mix of a 64 x 64 wave tile fed from LDS on both sides).
 * gigabytes_per_second (may be NULL) is the whole device by HIP events; bytes_per_clock_per_cu divides it by the
 * compute units and by the core clock a wave measured during the launch (its cycle counter against the constant
 * 100 MHz clock). */
int hipie_probe_lds_rate(int device, int iterations, int waves_per_simd, int with_mfma, double* bytes_per_clock_per_cu,
                         double* gigabytes_per_second);

#ifdef __cplusplus
}
#endif

#endif /* HIPIE_DIAG_H */
