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

// reciprocals for the decode of a lane's item index; inv_cgroups = 0 says "too many items for them"
struct ItemDecode {
    float inv_cgroups, inv_pairs, inv_oh;
};

__device__ __forceinline__ void mac_bytes(uint32_t x, uint32_t w, int& a0, int& a1, int& a2, int& a3) {
    a0 += static_cast<int>(static_cast<int8_t>(x)) * static_cast<int>(static_cast<int8_t>(w));
    a1 += static_cast<int>(static_cast<int8_t>(x >> 8)) * static_cast<int>(static_cast<int8_t>(w >> 8));
    a2 += static_cast<int>(static_cast<int8_t>(x >> 16)) * static_cast<int>(static_cast<int8_t>(w >> 16));
    a3 += static_cast<int>(static_cast<int8_t>(x >> 24)) * static_cast<int>(static_cast<int8_t>(w >> 24));
}

template <uint32_t F>
__global__ __launch_bounds__(256) void dwconv_kernel(const ConvArgs a, int KH, int KW, int dil_h, int dil_w,
                                                     int cgroups, int64_t items, int per_xcd, ItemDecode dec) {
    const int64_t item = workgroup_index(per_xcd) * 256 + threadIdx.x;
    if (item >= items) return;
    int cgi, m_pair;
    if (dec.inv_cgroups > 0.f) {
        fast_divmod(static_cast<int>(item), cgroups, dec.inv_cgroups, m_pair, cgi);
    } else {
        cgi = static_cast<int>(item % cgroups);
        m_pair = static_cast<int>(item / cgroups);
    }
    const int m0 = m_pair * 2;
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
                                                        int per_xcd, ItemDecode dec) {
    // The filter rows of all channels ([3][channels] dwords, three taps each) go through LDS: read from memory they
    // are twelve more 16-byte vector loads per lane beside the fifteen of the input, and the kernel is bound by the
    // rate at which the texture addresser takes those (its busy counter reads 80 % of the kernel's time).
    // The epilogue's per-channel tables and the accumulator corrections take the same way (another twenty loads).
    extern __shared__ __attribute__((aligned(16))) uint32_t sFilt[];
    const int cs = cgroups * 16;
    float* const sTab = reinterpret_cast<float*>(sFilt + 3 * cs);
    for (int r = 0; r < 3; ++r)
        for (int q = threadIdx.x; q < cs / 4; q += 256)
            *reinterpret_cast<uint4*>(&sFilt[r * cs + 4 * q]) =
                *reinterpret_cast<const uint4*>(a.wgt2 + (static_cast<int64_t>(r) * a.OCp + 4 * q) * 4);
    stage_params<F>(a, 0, (lds_float_ptr)sTab, cs, static_cast<int>(threadIdx.x), 256);
    __syncthreads();
    const int64_t item = workgroup_index(per_xcd) * 256 + threadIdx.x;
    if (item >= items) return;
    // item -> (channel group, pair) -> (n, oh, ow0): pairs never straddle a row.  Below 2^24 items the quotients come
    // from reciprocals (exact there); 64-bit and 32-bit integer divisions per lane cost more than the lane's multiplies.
    const int OH = a.OHOW / a.OW;
    int cgi, pair, rowi, ow0, n, oh;
    if (dec.inv_cgroups > 0.f) {
        fast_divmod(static_cast<int>(item), cgroups, dec.inv_cgroups, pair, cgi);
        fast_divmod(pair, pairs_per_row, dec.inv_pairs, rowi, ow0);
        fast_divmod(rowi, OH, dec.inv_oh, n, oh);
        ow0 *= 2;
    } else {
        cgi = static_cast<int>(item % cgroups);
        pair = static_cast<int>(item / cgroups);
        rowi = pair / pairs_per_row;
        ow0 = (pair - rowi * pairs_per_row) * 2;
        n = rowi / OH;
        oh = rowi - n * OH;
    }
    const int oc_lane = cgi * 16;
    constexpr int COLS = 3 + STRIDE;   // input columns under the two windows
    const int8_t* xp = a.in + (static_cast<int64_t>(n) * a.in_sn + oh * STRIDE * a.in_sh + ow0 * STRIDE * a.in_sw +
                               a.in_origin + oc_lane);
    // a.wgt2: [kh][OCp] dwords, the three taps of a filter row of one channel in bytes 0..2
    uint4 x[3][COLS], wr[3][4];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            wr[r][q] = *reinterpret_cast<const uint4*>(&sFilt[r * cs + oc_lane + 4 * q]);
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
        const int32_t* const corr = reinterpret_cast<const int32_t*>(sTab) + PT_COUNT * cs + oc_lane;
        const int4 c0 = *reinterpret_cast<const int4*>(corr), c1 = *reinterpret_cast<const int4*>(corr + 4);
        const int4 c2 = *reinterpret_cast<const int4*>(corr + 8), c3 = *reinterpret_cast<const int4*>(corr + 12);
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
    epilogue<F, 1>(a, acc, oc_lane, valid, out_off, res_off, none, (lds_cfloat_ptr)sTab, cs, 0);
}


// 3x3, dilation 1, stride 1 or 2, through LDS: a workgroup stages the input rows under R output rows of a strip of
// columns (all channels, halo included) in LDS once, with 16-byte loads of whole pixels.  A lane owns FOUR channels
// (one dword of a pixel) of four horizontally adjacent output pixels and walks down the R output rows: every input
// row is read from LDS once per lane (6 dwords at stride 1, 9 at stride 2), transposed once (v_perm_b32) into one
// dword per channel holding four consecutive pixels, and used for all three filter rows it belongs to, so the
// 3 x 3 window slides in registers in both directions.  Per output: 4 VALU instructions of multiply work at stride 1
// (7 at stride 2) plus the epilogue's 7 or 8; address arithmetic is per lane and per row, not per output.
struct DwStrip {
    int32_t cpb;              // dwords (groups of four channels) per pixel = in_sw / 4
    float inv_cpb;
    int32_t strips;           // strips of four output columns per workgroup
    int32_t col_tiles, row_tiles;
    int32_t cols_in;          // input columns staged per workgroup
    int32_t pad_top, pad_left;
    int32_t in_h_end, in_w_end;   // one past the last readable input row / column (interior + halo)
    int32_t OH;
    int32_t cgroups_out;      // groups of four channels that exist in the output tensor
    int64_t tiles;
    int32_t per_xcd;
};

constexpr int kDwRows = 7;    // output rows per workgroup: 7, 14, 28, 56, 112 are all multiples of it

template <uint32_t F, int STRIDE>
__global__ __launch_bounds__(256) void dwconv3x3_lds_kernel(const ConvArgs a, const DwStrip t) {
    constexpr int R = kDwRows, ROWS_IN = (R - 1) * STRIDE + 3, NPX = 3 * STRIDE + 3;
    extern __shared__ __attribute__((aligned(16))) int8_t patch[];
    const int64_t wg = workgroup_index(t.per_xcd);
    if (wg >= t.tiles) return;                        // whole workgroup, before the barrier
    const int col_tile = static_cast<int>(wg % t.col_tiles);
    const int64_t rest = wg / t.col_tiles;
    const int row_tile = static_cast<int>(rest % t.row_tiles), n = static_cast<int>(rest / t.row_tiles);
    const int oh0 = row_tile * R, ow0 = col_tile * 4 * t.strips;
    const int ih0 = oh0 * STRIDE - t.pad_top, iw0 = ow0 * STRIDE - t.pad_left;
    const int tid = threadIdx.x, nt = blockDim.x;

    // ---- stage: rows_eff x cols_eff whole pixels, each row one contiguous run in memory and in LDS
    // (holding the loads of the lower rows in registers until the first output rows are done was slower: the 32
    // registers cost more occupancy than the overlap returned)
    const int rows_eff = min(ROWS_IN, t.in_h_end - ih0), cols_eff = min(t.cols_in, t.in_w_end - iw0);
    const int chunks_row = cols_eff * (a.in_sw >> 4), total = rows_eff * chunks_row;
    const float inv_chunks_row = 1.0f / static_cast<float>(chunks_row);
    const int8_t* const src = a.in + (static_cast<int64_t>(n) * a.in_sn + static_cast<int64_t>(ih0) * a.in_sh +
                                      static_cast<int64_t>(iw0) * a.in_sw);
    const int lds_row = t.cols_in * a.in_sw;
    constexpr int NJ = 8;                             // loads in flight per thread and round
    for (int base = 0; base < total; base += NJ * nt) {
        uint4 v[NJ];
        int dst[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int idx = base + j * nt + tid;
            int row, ch;
            fast_divmod(min(idx, total - 1), chunks_row, inv_chunks_row, row, ch);
            dst[j] = idx < total ? row * lds_row + ch * 16 : -1;
            v[j] = *reinterpret_cast<const uint4*>(src + static_cast<int64_t>(row) * a.in_sh + ch * 16);
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            if (dst[j] >= 0) *reinterpret_cast<uint4*>(patch + dst[j]) = v[j];
    }

    // ---- lane role
    int strip, cg;
    fast_divmod(tid, t.cpb, t.inv_cpb, strip, cg);
    const bool lane_on = strip < t.strips;
    if (!lane_on) { strip = 0; cg = 0; }
    const int oc = 4 * cg;
    uint32_t w[3][4], ws[3][4];                       // (w0, w1, w2, 0) of a filter row and the same one byte up
#pragma unroll
    for (int kh = 0; kh < 3; ++kh) {
        const uint4 q = *reinterpret_cast<const uint4*>(a.wgt2 + (static_cast<int64_t>(kh) * a.OCp + oc) * 4);
        w[kh][0] = q.x; w[kh][1] = q.y; w[kh][2] = q.z; w[kh][3] = q.w;
#pragma unroll
        for (int c = 0; c < 4; ++c) ws[kh][c] = w[kh][c] << 8;
    }
    const int4 corr = *reinterpret_cast<const int4*>(a.corr + oc);
    const int corr_[4] = {corr.x, corr.y, corr.z, corr.w};
    float bias_[4], scale_[4], ih_[4], r_[4], r2_[4];
    f4_to_array(ld4f(a.bias + oc), bias_);
    if (F & CF_SCALE) f4_to_array(ld4f(a.scale + oc), scale_);
    f4_to_array(ld4f(a.fq_ih + oc), ih_);
    f4_to_array(ld4f(a.fq_r + oc), r_);
    f4_to_array(ld4f(a.fq_r2 + oc), r2_);
    const uint32_t xmask = (a.flags & CF_OUT_XOR) ? 0x80808080u : 0u;
    const int ow_lane = ow0 + 4 * strip;
    const bool store_on = lane_on && cg < t.cgroups_out;
    int8_t* const out_lane = static_cast<int8_t*>(a.out) + (static_cast<int64_t>(n) * a.out_sn + static_cast<int64_t>(ow_lane) * a.out_sw + oc);

    __syncthreads();

    int acc[3][4][4];                                 // [output row mod 3][pixel][channel]
#pragma unroll
    for (int s = 0; s < 3; ++s)
#pragma unroll
        for (int px = 0; px < 4; ++px)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[s][px][c] = corr_[c];

    auto transpose4 = [&](uint32_t p0, uint32_t p1, uint32_t p2, uint32_t p3, uint32_t (&o)[4]) {
        const uint32_t lo01 = __builtin_amdgcn_perm(p1, p0, 0x05010400u), hi01 = __builtin_amdgcn_perm(p1, p0, 0x07030602u);
        const uint32_t lo23 = __builtin_amdgcn_perm(p3, p2, 0x05010400u), hi23 = __builtin_amdgcn_perm(p3, p2, 0x07030602u);
        o[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
        o[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
        o[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
        o[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
    };
    const int8_t* lds_lane = patch + (4 * strip * STRIDE) * a.in_sw + oc;
#pragma unroll
    for (int i = 0; i < ROWS_IN; ++i) {
        uint32_t p[NPX];
#pragma unroll
        for (int j = 0; j < NPX; ++j) p[j] = *reinterpret_cast<const uint32_t*>(lds_lane + i * lds_row + j * a.in_sw);
        // T[g][c]: channel c of the four pixels under output pixel pair / pixel g
        uint32_t T[STRIDE == 1 ? 2 : 4][4];
        if (STRIDE == 1) {
            transpose4(p[0], p[1], p[2], p[3], T[0]);
            transpose4(p[2], p[3], p[4], p[5], T[1]);
        } else {
            transpose4(p[0], p[1], p[2], p[3], T[0]);
            transpose4(p[2], p[3], p[4], p[5], T[1]);
            transpose4(p[4], p[5], p[6], p[7], T[2]);
            transpose4(p[6], p[7], p[8], p[8], T[3]);
        }
#pragma unroll
        for (int kh = 0; kh < 3; ++kh) {
            if ((i - kh) % STRIDE != 0 || i - kh < 0 || (i - kh) / STRIDE >= R) continue;
            const int s = ((i - kh) / STRIDE) % 3;
#pragma unroll
            for (int px = 0; px < 4; ++px)
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint32_t x = STRIDE == 1 ? T[px >> 1][c] : T[px][c];
                    const uint32_t wv = (STRIDE == 1 && (px & 1)) ? ws[kh][c] : w[kh][c];
                    acc[s][px][c] = __builtin_amdgcn_sdot4(static_cast<int>(x), static_cast<int>(wv), acc[s][px][c], false);
                }
        }
        // output row r is complete behind input row r * STRIDE + 2
        if (i >= 2 && (i - 2) % STRIDE == 0 && (i - 2) / STRIDE < R) {
            const int r = (i - 2) / STRIDE, s = r % 3;
            const int oh = oh0 + r;
            uint32_t packed[4];
#pragma unroll
            for (int px = 0; px < 4; ++px) {
                packed[px] = 0;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float x = static_cast<float>(acc[s][px][c]);
                    x = x + bias_[c];
                    if (F & CF_SCALE) x = x * scale_[c];
                    if (F & CF_CLAMP) x = __builtin_amdgcn_fmed3f(x, a.clamp_lo, a.clamp_hi);
                    const float lv = fq_level_fast<2, true, true>(x, 0.f, ih_[c], ih_[c], r_[c], r2_[c], a.lm1);
                    packed[px] = __builtin_amdgcn_cvt_pk_u8_f32(lv, c, packed[px]);
                    acc[s][px][c] = corr_[c];
                }
            }
            if (store_on && oh < t.OH) {
                int8_t* const o = out_lane + static_cast<int64_t>(oh) * a.out_sh;
#pragma unroll
                for (int px = 0; px < 4; ++px)
                    if (ow_lane + px < a.OW) *reinterpret_cast<uint32_t*>(o + px * a.out_sw) = packed[px] ^ xmask;
            }
        }
    }
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

// the LDS strip kernel takes 3 x 3, undilated, stride 1 or 2 (the same both ways) with one of the specialised epilogues,
// pixels of at most 1024 bytes (a lane per four channels, at most 256 lanes) and no residual
bool dwconv_strip_fits(int KH, int KW, int dil_h, int dil_w, int stride_h, int stride_w, int in_c_stride, int ocp, uint32_t flags) {
    const uint32_t core = flags & ~CF_OUT_XOR;
    const bool known = core == E_PLAIN0 || core == E_CLAMPFQ || core == E_SCALEFQ0;
    // (a lane reads the weights and tables of the channels its pixel slice holds: the padded channel count must cover the stride)
    return KH == 3 && KW == 3 && dil_h == 1 && dil_w == 1 && stride_h == stride_w && (stride_h == 1 || stride_h == 2) && known &&
           in_c_stride % 16 == 0 && in_c_stride <= 1024 && in_c_stride <= ocp;
}

static void launch_dwconv_strip(const ConvArgs& a, const DwGeometry& g, hipStream_t s) {
    const int stride = a.conv_sh;
    DwStrip t;
    t.cpb = a.in_sw / 4;
    t.inv_cpb = 1.0f / static_cast<float>(t.cpb);
    const int OH = a.OHOW / a.OW;
    const int rows_in = (kDwRows - 1) * stride + 3;
    // as many strips as fit 256 lanes, the row's width and 48 KB of LDS (three workgroups per compute unit)
    int strips = std::max(1, 256 / t.cpb);
    strips = std::min(strips, static_cast<int>(ceil_div(a.OW, 4)));
    // (measured from 12 to 64 KB on the MobileNetV2 layers: smaller patches lose more to halo columns and idle lanes
    // than the extra workgroups per compute unit return)
    while (strips > 1 && static_cast<int64_t>(rows_in) * ((4 * strips - 1) * stride + 3) * a.in_sw > 48 * 1024) --strips;
    t.strips = strips;
    t.cols_in = (4 * strips - 1) * stride + 3;
    t.col_tiles = static_cast<int>(ceil_div(a.OW, 4 * strips));
    t.row_tiles = static_cast<int>(ceil_div(OH, kDwRows));
    t.pad_top = g.pad_top;
    t.pad_left = g.pad_left;
    t.in_h_end = g.in_h + g.halo;
    t.in_w_end = g.in_w + g.halo;
    t.OH = OH;
    t.cgroups_out = std::min(a.out_sw, a.in_sw) / 4;
    t.tiles = static_cast<int64_t>(a.M / a.OHOW) * t.row_tiles * t.col_tiles;
    const XcdGrid xg(t.tiles);
    t.per_xcd = xg.per_xcd;
    const size_t lds = static_cast<size_t>(rows_in) * t.cols_in * a.in_sw;
    const int threads = static_cast<int>(round_up(strips * t.cpb, 64));
    HIPIE_REQUIRE(lds <= 160 * 1024, HIPIE_GENERAL_ERROR, "depthwise strip kernel: %zu bytes of LDS", lds);
    const dim3 grid(xg.blocks), block(static_cast<uint32_t>(threads));
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_DWS(FLAGS, STRIDE)                                                                                     \
    do {                                                                                                                    \
        static bool attr_set = false;                                                                                       \
        if (!attr_set) {                                                                                                    \
            HIPIE_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&dwconv3x3_lds_kernel<FLAGS, STRIDE>),         \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));                   \
            attr_set = true;                                                                                                \
        }                                                                                                                   \
        hipLaunchKernelGGL((dwconv3x3_lds_kernel<FLAGS, STRIDE>), grid, block, lds, s, a, t);                               \
    } while (0)
    if (core == E_PLAIN0) {
        if (stride == 1) HIPIE_LAUNCH_DWS(E_PLAIN0, 1); else HIPIE_LAUNCH_DWS(E_PLAIN0, 2);
    } else if (core == E_SCALEFQ0) {
        if (stride == 1) HIPIE_LAUNCH_DWS(E_SCALEFQ0, 1); else HIPIE_LAUNCH_DWS(E_SCALEFQ0, 2);
    } else {
        if (stride == 1) HIPIE_LAUNCH_DWS(E_CLAMPFQ, 1); else HIPIE_LAUNCH_DWS(E_CLAMPFQ, 2);
    }
#undef HIPIE_LAUNCH_DWS
}

void launch_dwconv(const ConvArgs& a, int KH, int KW, int dil_h, int dil_w, int variant, const DwGeometry& g, hipStream_t s) {
    const uint32_t core = a.flags & ~CF_OUT_XOR;
    const bool known = core == E_PLAIN0 || core == E_CLAMPFQ || core == E_SCALEFQ0;
    if (variant == 1) {
        HIPIE_REQUIRE(dwconv_strip_fits(KH, KW, dil_h, dil_w, a.conv_sh, a.conv_sw, a.in_sw, a.OCp, a.flags) && !(a.flags & CF_RES),
                      HIPIE_GENERAL_ERROR, "depthwise strip kernel chosen for a layer it does not take");
        launch_dwconv_strip(a, g, s);
        return;
    }
    if (KH == 3 && KW == 3 && dil_h == 1 && dil_w == 1 && a.conv_sh == a.conv_sw && (a.conv_sh == 1 || a.conv_sh == 2) &&
        known && !(a.flags & CF_RES) && std::min(a.OCp, a.in_sw) * (3 + PT_ROWS) * 4 <= 60 * 1024) {   // (filter rows and tables fit their LDS)
        const int cgroups = std::min(a.OCp, a.in_sw) / 16;   // groups of 16 channels that exist in the tensors
        const int pairs_per_row = (a.OW + 1) / 2;
        const int64_t items = static_cast<int64_t>(a.M / a.OW) * pairs_per_row * cgroups;
        const XcdGrid xg(ceil_div(items, 256));
        const dim3 grid(xg.blocks), block(256);
        const int per_xcd = xg.per_xcd;
        const size_t filt_lds = static_cast<size_t>(cgroups) * 16 * (3 + PT_ROWS) * 4;   // filter rows and tables: 60 bytes per channel
        ItemDecode dec{0.f, 0.f, 0.f};
        if (items < (1 << 24))
            dec = ItemDecode{1.0f / static_cast<float>(cgroups), 1.0f / static_cast<float>(pairs_per_row),
                             1.0f / static_cast<float>(a.OHOW / a.OW)};
#define HIPIE_LAUNCH_DW3(FLAGS, STRIDE)                                                                                     \
    do {                                                                                                                    \
        static bool attr_set = false;                                                                                       \
        if (!attr_set) {                                                                                                    \
            HIPIE_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&dwconv3x3_kernel<FLAGS, STRIDE>),            \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));                    \
            attr_set = true;                                                                                                \
        }                                                                                                                   \
        hipLaunchKernelGGL((dwconv3x3_kernel<FLAGS, STRIDE>), grid, block, filt_lds, s, a, cgroups, pairs_per_row, items,   \
                           per_xcd, dec);                                                                                   \
    } while (0)
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
    ItemDecode dec{0.f, 0.f, 0.f};
    if (items < (1 << 24)) dec.inv_cgroups = 1.0f / static_cast<float>(cgroups);
    switch (core) {
    case E_PLAIN0: hipLaunchKernelGGL((dwconv_kernel<E_PLAIN0>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items, per_xcd, dec); break;
    case E_CLAMPFQ: hipLaunchKernelGGL((dwconv_kernel<E_CLAMPFQ>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items, per_xcd, dec); break;
    case E_SCALEFQ0: hipLaunchKernelGGL((dwconv_kernel<E_SCALEFQ0>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items, per_xcd, dec); break;
    default: hipLaunchKernelGGL((dwconv_kernel<kDyn>), grid, block, 0, s, a, KH, KW, dil_h, dil_w, cgroups, items, per_xcd, dec); break;
    }
}

}  // namespace hipie
