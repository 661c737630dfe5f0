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

// Workgroups are handed to the eight XCDs in turn (blockIdx mod 8), and each XCD has its own L2.  Items run
// along a row, then down the rows of an image: in launch order vertically adjacent output rows - which share
// one (stride 2) or two (stride 1) of their three input rows - land on different XCDs, and every XCD fetches
// the shared rows from memory for itself (FETCH_SIZE read 1.4 to 3.1 times the input).  With per_xcd > 0 the
// grid has 8 * per_xcd workgroups and XCD x works through the contiguous range [x * per_xcd, (x + 1) * per_xcd)
// of them, so neighbouring rows meet in one L2; indices past the last item fall out at the caller's bound check.
__device__ __forceinline__ int64_t workgroup_index(int per_xcd) {
    if (per_xcd <= 0) return blockIdx.x;
    return static_cast<int64_t>(blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
}

__device__ __forceinline__ void mac_bytes(uint32_t x, uint32_t w, int& a0, int& a1, int& a2, int& a3) {
    a0 += static_cast<int>(static_cast<int8_t>(x)) * static_cast<int>(static_cast<int8_t>(w));
    a1 += static_cast<int>(static_cast<int8_t>(x >> 8)) * static_cast<int>(static_cast<int8_t>(w >> 8));
    a2 += static_cast<int>(static_cast<int8_t>(x >> 16)) * static_cast<int>(static_cast<int8_t>(w >> 16));
    a3 += static_cast<int>(static_cast<int8_t>(x >> 24)) * static_cast<int>(static_cast<int8_t>(w >> 24));
}

template <uint32_t F>
__global__ __launch_bounds__(256) void dwconv_kernel(const ConvArgs a, int KH, int KW, int dil_h, int dil_w,
                                                     int cgroups, int64_t items, int per_xcd) {
    const int64_t item = workgroup_index(per_xcd) * 256 + threadIdx.x;
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


// 3x3, dilation 1, stride 1 or 2: a lane owns 16 channels of two horizontally adjacent output
// pixels.  All 9 weight pieces and the 12 (stride 1) or 15 (stride 2) input pieces the two windows
// cover are requested before the first multiply, so a wave waits for memory once instead of once
// per tap, and the two windows share their overlapping input columns in registers.
template <uint32_t F, int STRIDE>
__global__ __launch_bounds__(256) void dwconv3x3_kernel(const ConvArgs a, int cgroups, int pairs_per_row, int64_t items,
                                                        int per_xcd) {
    const int64_t item = workgroup_index(per_xcd) * 256 + threadIdx.x;
    if (item >= items) return;
    const int cgi = static_cast<int>(item % cgroups);
    const int pair = static_cast<int>(item / cgroups);
    const int oc_lane = cgi * 16;
    // pair -> (n, oh, ow0): pairs never straddle a row
    const int OH = a.OHOW / a.OW;
    const int rowi = pair / pairs_per_row, ow0 = (pair - rowi * pairs_per_row) * 2;
    const int n = rowi / OH, oh = rowi - n * OH;
    constexpr int COLS = 3 + STRIDE;   // input columns under the two windows
    const int8_t* xp = a.in + (static_cast<int64_t>(n) * a.in_sn + oh * STRIDE * a.in_sh + ow0 * STRIDE * a.in_sw +
                               a.in_origin + oc_lane);
    // a.wgt2: [kh][OCp] dwords, the three taps of a filter row of one channel in bytes 0..2
    uint4 x[3][COLS], wr[3][4];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            wr[r][q] = *reinterpret_cast<const uint4*>(a.wgt2 + (static_cast<int64_t>(r) * a.OCp + oc_lane + 4 * q) * 4);
    // the last pair of an odd row has one pixel: its second window's extra columns are clamped onto
    // existing ones (the results are discarded)
    const bool two = ow0 + 1 < a.OW;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            const int cc = (c < 3 || two) ? c : 2;
            x[r][c] = *reinterpret_cast<const uint4*>(xp + r * a.in_sh + cc * a.in_sw);
        }
    v16i acc[2][2];
    {
        const int4 c0 = *reinterpret_cast<const int4*>(a.corr + oc_lane), c1 = *reinterpret_cast<const int4*>(a.corr + oc_lane + 4);
        const int4 c2 = *reinterpret_cast<const int4*>(a.corr + oc_lane + 8), c3 = *reinterpret_cast<const int4*>(a.corr + oc_lane + 12);
        const int cv[16] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w, c2.x, c2.y, c2.z, c2.w, c3.x, c3.y, c3.z, c3.w};
#pragma unroll
        for (int pb = 0; pb < 2; ++pb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                acc[0][pb][r] = cv[r];
                acc[1][pb][r] = 0;
            }
    }
    // Four pixels x four channels of bytes are transposed with 8 v_perm_b32 into one dword per
    // channel holding that channel's byte of four consecutive pixels; a filter row is then one
    // v_dot4_i32_i8 per channel and output pixel against (w0, w1, w2, 0) - shifted by one byte for the
    // second pixel of a stride-1 pair, whose window starts one column later.
#pragma unroll
    for (int kh = 0; kh < 3; ++kh)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            auto dw = [&](const uint4& v) { return q == 0 ? v.x : (q == 1 ? v.y : (q == 2 ? v.z : v.w)); };
            auto transpose4 = [&](uint32_t p0, uint32_t p1, uint32_t p2, uint32_t p3, uint32_t (&t)[4]) {
                const uint32_t lo01 = __builtin_amdgcn_perm(p1, p0, 0x05010400u), hi01 = __builtin_amdgcn_perm(p1, p0, 0x07030602u);
                const uint32_t lo23 = __builtin_amdgcn_perm(p3, p2, 0x05010400u), hi23 = __builtin_amdgcn_perm(p3, p2, 0x07030602u);
                t[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
                t[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
                t[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
                t[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
            };
            const uint32_t wq[4] = {wr[kh][q].x, wr[kh][q].y, wr[kh][q].z, wr[kh][q].w};
            uint32_t t0[4];
            transpose4(dw(x[kh][0]), dw(x[kh][1]), dw(x[kh][2]), dw(x[kh][3]), t0);
            if (STRIDE == 1) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    acc[0][0][4 * q + c] = __builtin_amdgcn_sdot4(static_cast<int>(t0[c]), static_cast<int>(wq[c]), acc[0][0][4 * q + c], false);
                    acc[0][1][4 * q + c] = __builtin_amdgcn_sdot4(static_cast<int>(t0[c]), static_cast<int>(wq[c] << 8), acc[0][1][4 * q + c], false);
                }
            } else {   // second window: columns 2, 3, 4
                uint32_t t1[4];
                transpose4(dw(x[kh][2]), dw(x[kh][3]), dw(x[kh][4]), dw(x[kh][4]), t1);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    acc[0][0][4 * q + c] = __builtin_amdgcn_sdot4(static_cast<int>(t0[c]), static_cast<int>(wq[c]), acc[0][0][4 * q + c], false);
                    acc[0][1][4 * q + c] = __builtin_amdgcn_sdot4(static_cast<int>(t1[c]), static_cast<int>(wq[c]), acc[0][1][4 * q + c], false);
                }
            }
        }
    bool valid[2] = {true, two};
    int64_t out_off[2], res_off[2];
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
        const int ow = two || pb == 0 ? ow0 + pb : ow0;
        out_off[pb] = static_cast<int64_t>(n) * a.out_sn + oh * a.out_sh + ow * a.out_sw + oc_lane;
        res_off[pb] = static_cast<int64_t>(n) * a.res_sn + oh * a.res_sh + ow * a.res_sw + oc_lane;
    }
    v16f none[2][2];
    epilogue<F, 1>(a, acc, oc_lane, valid, out_off, res_off, none, nullptr, 0, 0);
}

}  // namespace

// grid of a launch of `workgroups` workgroups: XCD-contiguous order from 64 workgroups up (8 per XCD), the
// plain order below that, where spreading the few workgroups matters more than sharing rows
struct XcdGrid {
    uint32_t blocks;
    int per_xcd;
    explicit XcdGrid(int64_t workgroups) {
        per_xcd = workgroups >= 64 ? static_cast<int>(ceil_div(workgroups, 8)) : 0;
        blocks = static_cast<uint32_t>(per_xcd > 0 ? 8 * static_cast<int64_t>(per_xcd) : workgroups);
    }
};

void launch_dwconv(const ConvArgs& a, int KH, int KW, int dil_h, int dil_w, hipStream_t s) {
    const uint32_t core = a.flags & ~CF_OUT_XOR;
    const bool known = core == E_PLAIN0 || core == E_CLAMPFQ || core == E_SCALEFQ0;
    if (KH == 3 && KW == 3 && dil_h == 1 && dil_w == 1 && a.conv_sh == a.conv_sw && (a.conv_sh == 1 || a.conv_sh == 2) &&
        known && !(a.flags & CF_RES)) {
        const int cgroups = std::min(a.OCp, a.in_sw) / 16;   // groups of 16 channels that exist in the tensors
        const int pairs_per_row = (a.OW + 1) / 2;
        const int64_t items = static_cast<int64_t>(a.M / a.OW) * pairs_per_row * cgroups;
        const XcdGrid xg(ceil_div(items, 256));
        const dim3 grid(xg.blocks), block(256);
        const int per_xcd = xg.per_xcd;
#define HIPIE_LAUNCH_DW3(FLAGS, STRIDE) \
    hipLaunchKernelGGL((dwconv3x3_kernel<FLAGS, STRIDE>), grid, block, 0, s, a, cgroups, pairs_per_row, items, per_xcd)
        if (core == E_PLAIN0) {
            if (a.conv_sh == 1) HIPIE_LAUNCH_DW3(E_PLAIN0, 1); else HIPIE_LAUNCH_DW3(E_PLAIN0, 2);
        } else if (core == E_SCALEFQ0) {
            if (a.conv_sh == 1) HIPIE_LAUNCH_DW3(E_SCALEFQ0, 1); else HIPIE_LAUNCH_DW3(E_SCALEFQ0, 2);
        } else {
            if (a.conv_sh == 1) HIPIE_LAUNCH_DW3(E_CLAMPFQ, 1); else HIPIE_LAUNCH_DW3(E_CLAMPFQ, 2);
        }
#undef HIPIE_LAUNCH_DW3
        return;
    }
    const int cgroups = a.OCp / 32;
    const int64_t items = ceil_div(a.M, 2) * cgroups;
    const XcdGrid xg(ceil_div(items, 256));
    const dim3 grid(xg.blocks), block(256);
    const int per_xcd = xg.per_xcd;
    switch (core) {
    case E_PLAIN0: hipLaunchKernelGGL((dwconv_kernel<E_PLAIN0>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items, per_xcd); break;
    case E_CLAMPFQ: hipLaunchKernelGGL((dwconv_kernel<E_CLAMPFQ>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items, per_xcd); break;
    case E_SCALEFQ0: hipLaunchKernelGGL((dwconv_kernel<E_SCALEFQ0>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items, per_xcd); break;
    default: hipLaunchKernelGGL((dwconv_kernel<kDyn>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items, per_xcd); break;
    }
}

}  // namespace hipie
