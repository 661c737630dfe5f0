// Convolution / MatMul on int8 MFMA: kernel instantiations, load-time packing, launcher.
#include "conv.h"

#include <cmath>
#include <memory>

namespace hipie {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

constexpr int kRow = 80;  // LDS row stride: 64 K-bytes + 16 pad

__device__ __forceinline__ float res_byte_to_float(uint32_t dw, int j, float add) {
    const int b = static_cast<int>(static_cast<int8_t>((dw >> (8 * j)) & 0xffu));
    return static_cast<float>(b) + add;
}

template <int WOC, int WPIX>
__global__ __launch_bounds__(WOC* WPIX * 64) void conv_mfma_kernel(const ConvArgs a) {
    constexpr int NT = WOC * WPIX * 64;
    constexpr int BOC = WOC * 64, BPIX = WPIX * 64;
    constexpr int A_PIECES = BOC * 4 / NT, B_PIECES = BPIX * 4 / NT;
    __shared__ __attribute__((aligned(16))) int8_t sA[2][BOC * kRow];
    __shared__ __attribute__((aligned(16))) int8_t sB[2][BPIX * kRow];
    extern __shared__ int32_t s_koff[];  // [Kp / 16]

    // ---- block -> (pixel tile, channel tile): consecutive pixel tiles stay on one XCD ----------
    const int xcd = blockIdx.x & 7, y = blockIdx.x >> 3;
    const int t_tile = y % a.t_tiles, p_local = y / a.t_tiles;
    const int p_tile = xcd * a.p_per_xcd + p_local;
    if (p_tile >= a.p_tiles) return;  // whole block leaves before any barrier
    const int pix0 = p_tile * BPIX, oc0 = t_tile * BOC;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int woc = wave % WOC, wpix = wave / WOC;
    const int l32 = lane & 31, h = lane >> 5;

    for (int i = tid; i < a.nk * 4; i += NT) s_koff[i] = a.koff[i];

    // ---- this thread's global->LDS pieces ------------------------------------------------------
    int32_t b_base[B_PIECES];
    const int8_t* a_ptr[A_PIECES];
    const int chunk = tid & 3;
#pragma unroll
    for (int i = 0; i < B_PIECES; ++i) {
        const int row = (tid + i * NT) >> 2;
        int m = pix0 + row;
        m = m < a.M ? m : a.M - 1;
        const int n = m / a.OHOW, rem = m - n * a.OHOW;
        const int oh = rem / a.OW, ow = rem - oh * a.OW;
        b_base[i] = n * a.in_sn + oh * a.conv_sh * a.in_sh + ow * a.conv_sw * a.in_sw + a.in_origin;
    }
#pragma unroll
    for (int i = 0; i < A_PIECES; ++i) {
        const int row = (tid + i * NT) >> 2;
        a_ptr[i] = a.wgt + static_cast<int64_t>(oc0 + row) * a.Kp + chunk * 16;
    }
    __syncthreads();  // s_koff visible

    v4i ga[A_PIECES], gb[B_PIECES];
    auto load_global = [&](int k) {
        const int32_t off = s_koff[k * 4 + chunk];
#pragma unroll
        for (int i = 0; i < A_PIECES; ++i) ga[i] = *reinterpret_cast<const v4i*>(a_ptr[i] + k * 64);
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i)
            gb[i] = *reinterpret_cast<const v4i*>(a.in + (b_base[i] + off));
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_PIECES; ++i)
            *reinterpret_cast<v4i*>(&sA[buf][((tid + i * NT) >> 2) * kRow + chunk * 16]) = ga[i];
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i)
            *reinterpret_cast<v4i*>(&sB[buf][((tid + i * NT) >> 2) * kRow + chunk * 16]) = gb[i];
    };

    // weight rows are read permuted so that the lane's results are 32 consecutive channels
    const int perm0 = 32 * ((l32 >> 2) & 1) + 4 * (l32 >> 3) + (l32 & 3);
    const int a_row[2] = {woc * 64 + perm0, woc * 64 + perm0 + 16};
    const int b_row[2] = {wpix * 64 + l32, wpix * 64 + 32 + l32};

    v16i acc[2][2];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int pb = 0; pb < 2; ++pb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ob][pb][r] = 0;

    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int k = 0; k < a.nk; ++k) {
        const int buf = k & 1;
        if (k + 1 < a.nk) load_global(k + 1);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v4i af[2], bf[2];
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
                af[ob] = *reinterpret_cast<const v4i*>(&sA[buf][a_row[ob] * kRow + ks * 32 + h * 16]);
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
                bf[pb] = *reinterpret_cast<const v4i*>(&sB[buf][b_row[pb] * kRow + ks * 32 + h * 16]);
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
                    acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ob], bf[pb], acc[ob][pb], 0, 0, 0);
        }
        if (k + 1 < a.nk) store_lds(buf ^ 1);
        __syncthreads();
    }

    // ---- fused epilogue -----------------------------------------------------------------------
    // acc[ob][pb][r] = channel oc_lane + 16*ob + r of pixel pix0 + wpix*64 + pb*32 + l32
    const int oc_lane = oc0 + woc * 64 + 32 * h;
    const uint32_t fl = a.flags;
    bool valid[2];
    int64_t out_off[2], res_off[2];
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
        const int m = pix0 + wpix * 64 + pb * 32 + l32;
        valid[pb] = m < a.M;
        const int mm = valid[pb] ? m : a.M - 1;
        const int n = mm / a.OHOW, rem = mm - n * a.OHOW;
        const int oh = rem / a.OW, ow = rem - oh * a.OW;
        out_off[pb] = static_cast<int64_t>(n) * a.out_sn + oh * a.out_sh + ow * a.out_sw + oc_lane;
        res_off[pb] = static_cast<int64_t>(n) * a.res_sn + oh * a.res_sh + ow * a.res_sw + oc_lane;
    }
    const int out_cs = a.out_sw;  // NHWC: pixel stride == channel stride of the output tensor

    uint32_t res_dw[2][8];
    if ((fl & CF_RES) && !(fl & CF_RES_F32)) {
#pragma unroll
        for (int pb = 0; pb < 2; ++pb)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint4 v = make_uint4(0, 0, 0, 0);
                if (valid[pb] && oc_lane + 16 * j < a.res_sw)
                    v = *reinterpret_cast<const uint4*>(static_cast<const int8_t*>(a.res) + res_off[pb] + 16 * j);
                res_dw[pb][4 * j + 0] = v.x;
                res_dw[pb][4 * j + 1] = v.y;
                res_dw[pb][4 * j + 2] = v.z;
                res_dw[pb][4 * j + 3] = v.w;
            }
    }
    const float res_add = (fl & CF_RES_U8B) ? 128.0f : 0.0f;

    uint32_t out_dw[2][8];
#pragma unroll
    for (int e4 = 0; e4 < 8; ++e4) {
        const int oc = oc_lane + 4 * e4;
        const int ob = e4 >> 2, r0 = (e4 & 3) * 4;
        const int4 corr = *reinterpret_cast<const int4*>(a.corr + oc);
        const int corr_[4] = {corr.x, corr.y, corr.z, corr.w};
        float bias_[4], scale_[4], rsub_[4], rmul_[4], post_[4], il_[4], ih_[4], d_[4], rr_[4];
        auto ld4 = [&](const float* p, float* dst) {
            const float4 v = *reinterpret_cast<const float4*>(p + oc);
            dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
        };
        if (fl & CF_BIAS) ld4(a.bias, bias_);
        if (fl & CF_SCALE) ld4(a.scale, scale_);
        if (fl & CF_RES_SUB) ld4(a.res_sub, rsub_);
        if (fl & CF_RES_MUL) ld4(a.res_mul, rmul_);
        if (fl & CF_POST_SCALE) ld4(a.post_scale, post_);
        if (fl & CF_OUT_FQ) {
            ld4(a.fq_il, il_);
            ld4(a.fq_ih, ih_);
            ld4(a.fq_d, d_);
            ld4(a.fq_r, rr_);
        }
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) {
            int ai[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) ai[j] = acc[ob][pb][r0 + j] + corr_[j];
            if (fl & CF_OUT_I32) {
                if (valid[pb] && oc + 4 <= out_cs)
                    *reinterpret_cast<int4*>(static_cast<int32_t*>(a.out) + out_off[pb] + 4 * e4) =
                        make_int4(ai[0], ai[1], ai[2], ai[3]);
                continue;
            }
            float rv[4] = {0.f, 0.f, 0.f, 0.f};
            if (fl & CF_RES) {
                if (fl & CF_RES_F32) {
                    float4 r4 = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (valid[pb] && oc + 4 <= a.res_sw)
                        r4 = *reinterpret_cast<const float4*>(static_cast<const float*>(a.res) + res_off[pb] + 4 * e4);
                    rv[0] = r4.x; rv[1] = r4.y; rv[2] = r4.z; rv[3] = r4.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) rv[j] = res_byte_to_float(res_dw[pb][e4], j, res_add);
                }
            }
            float v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float x = static_cast<float>(ai[j]);
                if (fl & CF_BIAS) x = x + bias_[j];
                if (fl & CF_SCALE) x = x * scale_[j];
                if (fl & CF_RES) {
                    float r = rv[j];
                    if (fl & CF_RES_SUB) r = r - rsub_[j];
                    if (fl & CF_RES_MUL) r = r * rmul_[j];
                    x = x + r;
                }
                if (fl & CF_POST_SCALE) x = x * post_[j];
                if (fl & CF_RELU) x = x > 0.0f ? x : 0.0f;
                if (fl & CF_CLAMP) x = x < a.clamp_lo ? a.clamp_lo : (x > a.clamp_hi ? a.clamp_hi : x);
                v[j] = x;
            }
            if (fl & CF_OUT_FQ) {
                uint32_t packed = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    FqChannel p;
                    p.il = il_[j]; p.ih = ih_[j]; p.d = d_[j]; p.r = rr_[j];
                    const float kf = (fl & CF_FQ_RCP) ? fq_level_clamped<true>(p, a.lm1, v[j])
                                                     : fq_level_clamped<false>(p, a.lm1, v[j]);
                    packed |= (static_cast<uint32_t>(static_cast<int>(kf + a.out_off)) & 0xffu) << (8 * j);
                }
                out_dw[pb][e4] = packed;
            } else {
                if (valid[pb] && oc + 4 <= out_cs)
                    *reinterpret_cast<float4*>(static_cast<float*>(a.out) + out_off[pb] + 4 * e4) =
                        make_float4(v[0], v[1], v[2], v[3]);
            }
        }
    }
    if (fl & CF_OUT_FQ) {
#pragma unroll
        for (int pb = 0; pb < 2; ++pb)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if (valid[pb] && oc_lane + 16 * j < out_cs)
                    *reinterpret_cast<uint4*>(static_cast<int8_t*>(a.out) + out_off[pb] + 16 * j) =
                        make_uint4(out_dw[pb][4 * j], out_dw[pb][4 * j + 1], out_dw[pb][4 * j + 2],
                                   out_dw[pb][4 * j + 3]);
    }
}

template <int WOC, int WPIX>
void launch(const ConvArgs& a, hipStream_t s) {
    const int grid = 8 * a.p_per_xcd * a.t_tiles;
    const size_t dyn = static_cast<size_t>(a.nk) * 4 * sizeof(int32_t);
    hipLaunchKernelGGL((conv_mfma_kernel<WOC, WPIX>), dim3(grid), dim3(WOC * WPIX * 64), dyn, s, a);
}

}  // namespace

// ------------------------------------------------------------------------------------------------
void Epilogue::build(int device_, const hipie_epilogue& e, int64_t oc, int64_t ocp) {
    device = device_;
    flags = 0;
    auto vec = [&](const float* p, int64_t n, float pad, const char* what, std::vector<float>& dst) {
        HIPIE_REQUIRE(n == 1 || n == oc, HIPIE_PARAMETER_MISMATCH,
                      "epilogue: %s has %lld values, expected 1 or %lld", what, (long long)n, (long long)oc);
        dst.assign(ocp, pad);
        for (int64_t c = 0; c < oc; ++c) dst[c] = p[n == 1 ? 0 : c];
    };
    std::vector<float> h;
    auto up = [&](DeviceBuffer& b, const std::vector<float>& v) {
        if (device >= 0) b.upload(device, v.data(), v.size() * sizeof(float));
    };
    if (e.bias) { vec(e.bias, e.n_bias, 0.f, "bias", h); up(bias, h); host_bias = h; flags |= CF_BIAS; }
    if (e.scale) { vec(e.scale, e.n_scale, 1.f, "scale", h); up(scale, h); flags |= CF_SCALE; }
    switch (e.residual_dtype) {
    case 0: break;
    case HIPIE_F32: flags |= CF_RES | CF_RES_F32; break;
    case HIPIE_U8B: flags |= CF_RES | CF_RES_U8B; break;
    case HIPIE_I8: flags |= CF_RES; break;
    default: fail(HIPIE_PARAMETER_MISMATCH, "epilogue: residual dtype %d", e.residual_dtype);
    }
    if (flags & CF_RES) {
        if (e.res_sub) { vec(e.res_sub, e.n_res_sub, 0.f, "res_sub", h); up(res_sub, h); flags |= CF_RES_SUB; }
        if (e.res_mul) { vec(e.res_mul, e.n_res_mul, 1.f, "res_mul", h); up(res_mul, h); flags |= CF_RES_MUL; }
    }
    if (e.post_scale) { vec(e.post_scale, e.n_post_scale, 1.f, "post_scale", h); up(post_scale, h); flags |= CF_POST_SCALE; }
    if (e.activation == 1) flags |= CF_RELU;
    else if (e.activation == 2) { flags |= CF_CLAMP; clamp_lo = e.clamp_lo; clamp_hi = e.clamp_hi; }
    else HIPIE_REQUIRE(e.activation == 0, HIPIE_PARAMETER_MISMATCH, "epilogue: activation %d", e.activation);
    out_dtype = e.out_dtype;
    switch (e.out_dtype) {
    case HIPIE_F32: break;
    case HIPIE_I32:
        HIPIE_REQUIRE(flags == 0, HIPIE_PARAMETER_MISMATCH, "epilogue: i32 output takes no other step");
        flags |= CF_OUT_I32;
        break;
    case HIPIE_U8B: case HIPIE_I8: {
        HIPIE_REQUIRE(e.fq_in_low && e.fq_in_high, HIPIE_PARAMETER_MISMATCH,
                      "epilogue: 8-bit output needs FakeQuantize bounds");
        HIPIE_REQUIRE(e.fq_levels >= 2 && e.fq_levels <= 256, HIPIE_PARAMETER_MISMATCH,
                      "epilogue: levels=%lld", (long long)e.fq_levels);
        lm1 = static_cast<float>(static_cast<size_t>(e.fq_levels - 1));
        std::vector<float> il, ih;
        vec(e.fq_in_low, e.n_fq_in_low, 0.f, "fq_in_low", il);
        vec(e.fq_in_high, e.n_fq_in_high, 1.f, "fq_in_high", ih);
        const float ol = e.fq_out_low, oh = e.fq_out_high;
        bool ok = ol == std::nearbyintf(ol) && oh == ol + lm1;
        for (int k = 0; ok && k < e.fq_levels; ++k)
            ok = (static_cast<float>(k) / lm1 * (oh - ol) + ol) == ol + static_cast<float>(k);
        HIPIE_REQUIRE(ok, HIPIE_NOT_IMPLEMENTED,
                      "epilogue: output range [%g, %g] with %lld levels is not consecutive integers",
                      ol, oh, (long long)e.fq_levels);
        if (e.out_dtype == HIPIE_U8B) {
            HIPIE_REQUIRE(ol >= 0 && oh <= 255, HIPIE_PARAMETER_MISMATCH, "epilogue: levels do not fit u8");
            out_off = ol - 128.0f;
        } else {
            HIPIE_REQUIRE(ol >= -128 && oh <= 127, HIPIE_PARAMETER_MISMATCH, "epilogue: levels do not fit i8");
            out_off = ol;
        }
        std::vector<float> d(ocp), r(ocp);
        std::atomic<bool> exact{true};
        for (int64_t c = 0; c < ocp; ++c) {
            HIPIE_REQUIRE(il[c] < ih[c], HIPIE_NOT_IMPLEMENTED,
                          "epilogue: FakeQuantize needs input_low < input_high (channel %lld)", (long long)c);
            d[c] = ih[c] - il[c];
        }
        parallel_for(ocp, [&](int64_t c) {
            FqChannel p{};
            p.il = il[c]; p.ih = ih[c]; p.lo = il[c]; p.hi = ih[c]; p.d = d[c];
            p.r = fq_rounded_reciprocal(p.d);
            r[c] = p.r;
            if (!fq_reciprocal_exact_on_boundaries(p, lm1)) exact = false;
        });
        up(fq_il, il); up(fq_ih, ih); up(fq_d, d); up(fq_r, r);
        flags |= CF_OUT_FQ;
        if (exact) flags |= CF_FQ_RCP;
        break;
    }
    default: fail(HIPIE_PARAMETER_MISMATCH, "epilogue: out dtype %d", e.out_dtype);
    }
}

void Epilogue::fill(ConvArgs& a) const {
    a.bias = bias.as<float>(); a.scale = scale.as<float>();
    a.res_sub = res_sub.as<float>(); a.res_mul = res_mul.as<float>();
    a.post_scale = post_scale.as<float>();
    a.fq_il = fq_il.as<float>(); a.fq_ih = fq_ih.as<float>();
    a.fq_d = fq_d.as<float>(); a.fq_r = fq_r.as<float>();
    a.flags = flags; a.lm1 = lm1; a.out_off = out_off; a.clamp_lo = clamp_lo; a.clamp_hi = clamp_hi;
}

}  // namespace hipie

using namespace hipie;

struct hipie_conv {
    int device = 0;
    hipie_conv_desc d{};
    int64_t K = 0, Kp = 0, OCp = 0;
    int tile = 0;  // 0: 128 ch x 128 px (2x2 waves), 1: 64 ch x 256 px (1x4), 2: 64 ch x 64 px (1 wave)
    DeviceBuffer wgt, koff, corr;
    Epilogue epi;
};

extern "C" {

int hipie_conv_create(int device, const hipie_conv_desc* desc, const int8_t* weights,
                      const hipie_epilogue* epilogue, hipie_conv** out) {
    return guarded([&] {
        HIPIE_REQUIRE(desc && weights && epilogue && out, HIPIE_PARAMETER_MISMATCH, "hipie_conv_create: null argument");
        const hipie_conv_desc& d = *desc;
        HIPIE_REQUIRE(d.in_dtype == HIPIE_U8B || d.in_dtype == HIPIE_I8, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_create: input dtype %d (U8B or I8 expected)", d.in_dtype);
        HIPIE_REQUIRE(d.ic > 0 && d.oc > 0 && d.kh > 0 && d.kw > 0 && d.stride_h > 0 && d.stride_w > 0 &&
                          d.dil_h > 0 && d.dil_w > 0 && d.pad_top >= 0 && d.pad_left >= 0 &&
                          d.pad_bottom >= 0 && d.pad_right >= 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_conv_create: bad geometry");
        HIPIE_REQUIRE(d.groups == 1, HIPIE_NOT_IMPLEMENTED,
                      "hipie_conv_create: groups=%d (depthwise has its own entry point)", d.groups);
        HIPIE_REQUIRE(d.in_c_stride >= d.ic && d.in_c_stride % 4 == 0, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_create: in_c_stride=%d must be a multiple of 4 >= ic=%d", d.in_c_stride, d.ic);
        auto c = std::make_unique<hipie_conv>();
        c->device = device;
        c->d = d;
        // K order (kh, kw, ic) over the padded channel stride.  A 16-byte piece must not straddle
        // two filter taps unless consecutive taps are contiguous in memory (in_stride_w == c stride).
        const bool row_contig = d.in_stride_w == d.in_c_stride && d.dil_w == 1;
        HIPIE_REQUIRE(d.in_c_stride % 16 == 0 || row_contig, HIPIE_NOT_IMPLEMENTED,
                      "hipie_conv_create: channel stride %d needs a multiple of 16", d.in_c_stride);
        const int64_t cs = d.in_c_stride;
        int64_t row_k = d.kw * cs;             // bytes of one filter row when taps are contiguous
        int64_t row_kp = round_up(row_k, 16);
        const bool per_row = cs % 16 != 0;      // small-channel first layer: pad every filter row
        c->K = per_row ? d.kh * row_kp : static_cast<int64_t>(d.kh) * d.kw * cs;
        c->Kp = round_up(c->K, 64);
        c->OCp = round_up(d.oc, 128);
        // offsets of every 16-byte K piece
        std::vector<int32_t> koff(c->Kp / 16, 0);
        for (int64_t p = 0; p < c->K / 16; ++p) {
            const int64_t k = p * 16;
            if (per_row) {
                const int64_t kh = k / row_kp, within = k % row_kp;
                koff[p] = static_cast<int32_t>(kh * d.dil_h * d.in_stride_h + within);
            } else {
                const int64_t tap = k / cs, ic0 = k % cs;
                const int64_t kh = tap / d.kw, kw = tap % d.kw;
                koff[p] = static_cast<int32_t>(kh * d.dil_h * d.in_stride_h + kw * d.dil_w * d.in_stride_w + ic0);
            }
        }
        // pack weights OIHW -> [OCp][Kp]
        std::vector<int8_t> w(static_cast<size_t>(c->OCp) * c->Kp, 0);
        std::vector<int32_t> corr(c->OCp, 0);
        parallel_for(d.oc, [&](int64_t oc) {
            int64_t sum = 0;
            for (int kh = 0; kh < d.kh; ++kh)
                for (int kw = 0; kw < d.kw; ++kw)
                    for (int ic = 0; ic < d.ic; ++ic) {
                        const int8_t v = weights[((oc * d.ic + ic) * d.kh + kh) * d.kw + kw];
                        const int64_t k = per_row ? kh * row_kp + kw * cs + ic
                                                  : (static_cast<int64_t>(kh) * d.kw + kw) * cs + ic;
                        w[oc * c->Kp + k] = v;
                        sum += v;
                    }
            corr[oc] = d.in_dtype == HIPIE_U8B ? static_cast<int32_t>(128 * sum) : 0;
        });
        c->epi.build(device, *epilogue, d.oc, c->OCp);
        // tile choice: wide channel tiles when there are enough channels, else all waves on pixels
        c->tile = d.oc > 64 ? 0 : 1;
        if (device >= 0) {
            c->wgt.upload(device, w.data(), w.size());
            c->koff.upload(device, koff.data(), koff.size() * sizeof(int32_t));
            c->corr.upload(device, corr.data(), corr.size() * sizeof(int32_t));
        }
        *out = c.release();
    });
}

void hipie_conv_destroy(hipie_conv* c) { delete c; }

int hipie_conv_set_tile(hipie_conv* c, int tile) {
    return guarded([&] {
        HIPIE_REQUIRE(c && tile >= 0 && tile <= 2, HIPIE_PARAMETER_MISMATCH, "hipie_conv_set_tile: tile=%d", tile);
        c->tile = tile;
    });
}

int hipie_conv_out_dims(const hipie_conv* c, int32_t h, int32_t w, int32_t* oh, int32_t* ow) {
    return guarded([&] {
        HIPIE_REQUIRE(c && oh && ow, HIPIE_PARAMETER_MISMATCH, "hipie_conv_out_dims: null argument");
        const hipie_conv_desc& d = c->d;
        *oh = (h + d.pad_top + d.pad_bottom - (d.dil_h * (d.kh - 1) + 1)) / d.stride_h + 1;
        *ow = (w + d.pad_left + d.pad_right - (d.dil_w * (d.kw - 1) + 1)) / d.stride_w + 1;
    });
}

int hipie_conv_run(const hipie_conv* c, const hipie_tensor* in, const hipie_tensor* residual,
                   const hipie_tensor* out, void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(c && in && out, HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: null argument");
        HIPIE_REQUIRE(c->wgt.ptr, HIPIE_NOT_ALLOCATED, "hipie_conv_run: host-only object");
        const hipie_conv_desc& d = c->d;
        HIPIE_REQUIRE(in->dtype == d.in_dtype && in->c == d.ic && in->stride_w == d.in_stride_w &&
                          in->stride_h == d.in_stride_h,
                      HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_run: input (dtype %d, c %d, strides %lld/%lld) does not match the "
                      "geometry the weights were packed for (dtype %d, c %d, strides %d/%d)",
                      in->dtype, in->c, (long long)in->stride_h, (long long)in->stride_w, d.in_dtype, d.ic,
                      d.in_stride_h, d.in_stride_w);
        const int need_halo = std::max(std::max(d.pad_top, d.pad_bottom), std::max(d.pad_left, d.pad_right));
        HIPIE_REQUIRE(in->halo >= need_halo, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_run: input halo %d < padding %d (the engine reads padding from the "
                      "tensor's own border)", in->halo, need_halo);
        int32_t oh, ow;
        oh = (in->h + d.pad_top + d.pad_bottom - (d.dil_h * (d.kh - 1) + 1)) / d.stride_h + 1;
        ow = (in->w + d.pad_left + d.pad_right - (d.dil_w * (d.kw - 1) + 1)) / d.stride_w + 1;
        HIPIE_REQUIRE(out->n == in->n && out->h == oh && out->w == ow && out->c == d.oc,
                      HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: output is [%d,%d,%d,%d], expected [%d,%d,%d,%d]",
                      out->n, out->h, out->w, out->c, in->n, oh, ow, d.oc);
        HIPIE_REQUIRE(out->dtype == c->epi.out_dtype, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_run: output dtype %d, epilogue produces %d", out->dtype, c->epi.out_dtype);
        const bool byte_out = out->dtype == HIPIE_U8B || out->dtype == HIPIE_I8;
        HIPIE_REQUIRE(out->stride_w % (byte_out ? 16 : 4) == 0 && out->stride_w >= d.oc &&
                          reinterpret_cast<uintptr_t>(out->data) % 16 == 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: output channel stride/alignment");
        HIPIE_REQUIRE(reinterpret_cast<uintptr_t>(in->data) % 4 == 0 &&
                          (d.in_c_stride % 16 != 0 || reinterpret_cast<uintptr_t>(in->data) % 16 == 0),
                      HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: input alignment");
        const int64_t M = static_cast<int64_t>(in->n) * oh * ow;
        if (M == 0) return;
        const int64_t in_span = static_cast<int64_t>(in->n) * in->stride_n;
        HIPIE_REQUIRE(in_span < (1ll << 31) && M < (1ll << 31), HIPIE_OUT_OF_BOUNDS,
                      "hipie_conv_run: tensor too large for 32-bit offsets");
        ConvArgs a{};
        a.in = static_cast<const int8_t*>(in->data);
        a.wgt = c->wgt.as<int8_t>();
        a.out = out->data;
        a.koff = c->koff.as<int32_t>();
        a.corr = c->corr.as<int32_t>();
        c->epi.fill(a);
        if (a.flags & CF_RES) {
            HIPIE_REQUIRE(residual && residual->data, HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: residual missing");
            const int want = (a.flags & CF_RES_F32) ? HIPIE_F32 : ((a.flags & CF_RES_U8B) ? HIPIE_U8B : HIPIE_I8);
            HIPIE_REQUIRE(residual->dtype == want && residual->n == out->n && residual->h == oh &&
                              residual->w == ow && residual->c == d.oc,
                          HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: residual shape/dtype mismatch");
            HIPIE_REQUIRE(residual->stride_w % ((a.flags & CF_RES_F32) ? 4 : 16) == 0 &&
                              reinterpret_cast<uintptr_t>(residual->data) % 16 == 0,
                          HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: residual channel stride/alignment");
            a.res = residual->data;
            a.res_sn = static_cast<int32_t>(residual->stride_n);
            a.res_sh = static_cast<int32_t>(residual->stride_h);
            a.res_sw = static_cast<int32_t>(residual->stride_w);
        }
        a.M = static_cast<int32_t>(M);
        a.OW = ow;
        a.OHOW = oh * ow;
        a.in_sn = static_cast<int32_t>(in->stride_n);
        a.in_sh = static_cast<int32_t>(in->stride_h);
        a.in_sw = static_cast<int32_t>(in->stride_w);
        a.conv_sh = d.stride_h;
        a.conv_sw = d.stride_w;
        a.in_origin = -(d.pad_top * a.in_sh + d.pad_left * a.in_sw);
        a.out_sn = static_cast<int32_t>(out->stride_n);
        a.out_sh = static_cast<int32_t>(out->stride_h);
        a.out_sw = static_cast<int32_t>(out->stride_w);
        a.OC = d.oc;
        a.OCp = static_cast<int32_t>(c->OCp);
        a.Kp = static_cast<int32_t>(c->Kp);
        a.nk = static_cast<int32_t>(c->Kp / 64);
        const int boc = c->tile == 0 ? 128 : 64;
        const int bpix = c->tile == 0 ? 128 : (c->tile == 1 ? 256 : 64);
        a.p_tiles = static_cast<int32_t>(ceil_div(M, bpix));
        a.t_tiles = static_cast<int32_t>(ceil_div(d.oc, boc));
        a.p_per_xcd = static_cast<int32_t>(ceil_div(a.p_tiles, 8));
        DeviceGuard g(c->device);
        hipStream_t s = as_stream(stream);
        switch (c->tile) {
        case 0: launch<2, 2>(a, s); break;
        case 1: launch<1, 4>(a, s); break;
        default: launch<1, 1>(a, s); break;
        }
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

}  // extern "C"
