// Host-side pieces of the MFMA convolution shared with MatMul and the graph planner.
#pragma once
#include <atomic>

#include "common.h"
#include "conv_kernel.h"
#include "fq.h"

namespace hipie {

// Packed convolution operands as the host produced them, in the order hipie_conv_create produced them.  A thread
// that builds a plan installs a tape for a scope: recording keeps every packed matrix and correction vector; a tape
// in playback hands them back to the same sequence of calls, which then upload instead of packing (a blob of another
// size than the call expects means the tape belongs to other layers: HIPIE_NETWORK_NOT_READ).  Only values travel on
// the tape, never offsets or sizes the kernels index with.
struct PackTape {
    std::vector<std::vector<uint8_t>> blobs;
    size_t next = 0;
    bool playing = false;
    struct Scope {
        explicit Scope(PackTape* t);
        ~Scope();
        Scope(const Scope&) = delete;
        Scope& operator=(const Scope&) = delete;
        PackTape* previous;
    };
    static PackTape* current();
    bool take(void* dst, size_t bytes);          // playback: the next blob into dst; false when not playing
    void give(const void* src, size_t bytes);    // recording: append; nothing while playing
};


// Per-channel epilogue tables on the device (padded to the packed channel count) + flags.
struct Epilogue {
    int device = 0;
    uint32_t flags = 0;
    int out_dtype = HIPIE_F32;
    float lm1 = 0, out_off = 0, clamp_lo = 0, clamp_hi = 0;
    DeviceBuffer bias, scale, res_sub, res_mul, post_scale, fq_il, fq_ih, fq_d, fq_r, fq_r2;
    std::vector<float> host_bias;
    void build(int device, const hipie_epilogue& e, int64_t oc, int64_t ocp);
    void fill(ConvArgs& a) const;
};

// cache-line kernels (conv_line.hip): shape 0 .. 4 = (wave groups, ring stages, K-step bytes) (1, 3, 128), (2, 3, 128),
// (1, 4, 128), (2, 4, 128), (1, 4, 64)
void launch_line(const ConvArgs& a, int shape, hipStream_t s);
int line_row_bytes(int shape);

// few pixels, many channels (conv_skinny.hip): 1 x 1 over a dense input, weights packed K-major ([Kp / 16][OCp] pieces of
// 16 K bytes, passed as ConvArgs::wgt2), epilogues as skinny_epilogue_fits says
bool skinny_epilogue_fits(uint32_t flags);
void launch_skinny(const ConvArgs& a, hipStream_t s);

// bottleneck-tail kernel (conv_block.hip): a 3 x 3 stride-1 pad-1 convolution over all of its 64, 128 or 256 output
// channels per workgroup, input patch staged once in LDS; alone (b == nullptr) or with the 1 x 1 convolution behind it
// run from the tile in LDS.  block_geometry: the tiling for an output of oh x ow pixels (ok = false: the kernel does
// not take the layer); block_epilogues_fit: the epilogues the kernel is instantiated for
struct BlockGeometry {
    bool ok;
    int nwc, rows, tiles_per_image, patch_w, csa, ppix;
    size_t lds;
    bool ok2;        // the fused form with two wave groups takes the layer too, with lds2 bytes of LDS
    size_t lds2;
};
BlockGeometry block_geometry(int oc_a, int ic_a, int oh, int ow);
bool block_epilogues_fit(uint32_t flags_a, bool fused, uint32_t flags_b);
// form 0: three steps of weights in flight per wave, two workgroups per compute unit; 1: nine steps, one workgroup;
// 2 (with b, where geo.ok2): eight waves in two groups that split the first layer's input slabs and take the second
// layer's passes in turn
void launch_block(const ConvArgs& a, const ConvArgs* b, const BlockGeometry& geo, int images, int form, hipStream_t s);
// the same kernel as a depthwise 3 x 3 convolution (stride 1 or 2, pad 1 on the top and left, a.wgt = [tap][OCp] bytes):
// the taps' diagonal weight matrices on the matrix pipe, 256 pixels x one 64-channel slab per workgroup
bool block_dw_epilogue_fits(uint32_t flags);
BlockGeometry block_dw_geometry(int oh, int ow, int stride);
void launch_block_dw(const ConvArgs& a, const BlockGeometry& geo, int images, hipStream_t s);

// depthwise kernels (dwconv.hip).  variant 0: a lane computes its outputs from registers loaded straight from memory;
// variant 1: 3 x 3 through an LDS patch with the window sliding in registers (dwconv_strip_fits says which layers)
struct DwGeometry {
    int in_h, in_w, halo;     // interior size of the input tensor and its readable border
    int pad_top, pad_left;
};
bool dwconv_strip_fits(int KH, int KW, int dil_h, int dil_w, int stride_h, int stride_w, int in_c_stride, int ocp, uint32_t flags);
void launch_dwconv(const ConvArgs& a, int KH, int KW, int dil_h, int dil_w, int variant, const DwGeometry& g, hipStream_t s);

// frees the split-K workspace kept for this stream, if any (for the owner of a stream, before it destroys
// the stream and after the stream's work has finished)
void release_split_workspace(int device, hipStream_t s);

}  // namespace hipie
