// Precision-preserved ops on the engine's NHWC byte tensors (HBM-bound): MaxPool, AvgPool with an
// optional fused requantize, and the exit conversion back to the reference's NCHW layout.
// Reference semantics: ngraph/core/reference/.../max_pool.hpp, avg_pool.hpp:114-265.
#include "pool.h"

namespace hipie {
namespace {

constexpr int kThreads = 256;

// Bytewise max on four packed bytes in the order-preserving unsigned domain (byte ^ 0x80 for signed
// storage): even and odd bytes are compared as the low / high byte of 16-bit lanes (v_pk_max_u16).
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

struct ByteMax {
    uint32_t even = 0, odd = 0;   // running maxima, unsigned domain; 0 is the identity
    __device__ __forceinline__ void take(uint32_t stored) {
        const uint32_t x = stored ^ 0x80808080u;
        const uint32_t e = x & 0x00ff00ffu, o = x & 0xff00ff00u;
        even = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, even), __builtin_bit_cast(u16x2, e)));
        odd = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, odd), __builtin_bit_cast(u16x2, o)));
    }
    __device__ __forceinline__ uint32_t stored() const { return (even | odd) ^ 0x80808080u; }
};

// One thread = 16 channels of one output pixel.  The reference skips padding cells and starts from the
// type's lowest value (max_pool.hpp); max is idempotent, so a window coordinate that falls into the
// padding is moved onto the nearest cell of the tensor instead (every window holds at least one: the
// graph refuses the others) and nothing is read from the tensor's border, whatever it holds.
// K3 = true: a 3 x 3 window, all nine loads requested up front.  VEC = dwords per thread: 4 (16 channels), or 1
// for tensors whose pixels hold four channels (image inputs).
template <int VEC> struct PoolWord;
template <> struct PoolWord<4> { typedef uint4 type; };
template <> struct PoolWord<1> { typedef uint32_t type; };
__device__ __forceinline__ void take_word(ByteMax (&r)[4], const uint4& v) { r[0].take(v.x); r[1].take(v.y); r[2].take(v.z); r[3].take(v.w); }
__device__ __forceinline__ void take_word(ByteMax (&r)[1], const uint32_t& v) { r[0].take(v); }
__device__ __forceinline__ uint4 stored_word(const ByteMax (&r)[4]) { return make_uint4(r[0].stored(), r[1].stored(), r[2].stored(), r[3].stored()); }
__device__ __forceinline__ uint32_t stored_word(const ByteMax (&r)[1]) { return r[0].stored(); }

template <bool K3, int VEC>
__global__ __launch_bounds__(kThreads) void max_pool_nhwc_i8(PoolArgs a) {
    typedef typename PoolWord<VEC>::type Word;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int cg = a.cs / (4 * VEC);
    if (t >= static_cast<int64_t>(a.M) * cg) return;
    const int m = static_cast<int>(t / cg), c = static_cast<int>(t % cg) * (4 * VEC);
    const int n = m / a.OHOW, rem = m - n * a.OHOW, oh = rem / a.OW, ow = rem - oh * a.OW;
    const int y0 = oh * a.sh - a.pt, x0 = ow * a.sw - a.pl;
    const int8_t* base = static_cast<const int8_t*>(a.in) + static_cast<int64_t>(n) * a.in_sn + c;
    ByteMax r[VEC];
    if (K3) {
        Word v[3][3];
#pragma unroll
        for (int y = 0; y < 3; ++y)
#pragma unroll
            for (int x = 0; x < 3; ++x) {
                const int yy = min(max(y0 + y, 0), a.H - 1), xx = min(max(x0 + x, 0), a.W - 1);
                v[y][x] = *reinterpret_cast<const Word*>(base + static_cast<int64_t>(yy) * a.in_sh + xx * a.in_sw);
            }
#pragma unroll
        for (int y = 0; y < 3; ++y)
#pragma unroll
            for (int x = 0; x < 3; ++x) take_word(r, v[y][x]);
    } else {
        const int ya = max(y0, 0), xa = max(x0, 0);
        const int yb = min(min(y0 + a.kh, a.H + a.pb), a.H), xb = min(min(x0 + a.kw, a.W + a.pr), a.W);
        for (int y = ya; y < yb; ++y)
            for (int x = xa; x < xb; ++x)
                take_word(r, *reinterpret_cast<const Word*>(base + static_cast<int64_t>(y) * a.in_sh + x * a.in_sw));
    }
    *reinterpret_cast<Word*>(static_cast<int8_t*>(a.out) + static_cast<int64_t>(n) * a.out_sn +
                             oh * a.out_sh + ow * a.out_sw + c) = stored_word(r);
}

// One thread = 4 channels of one output pixel.  Integer window sum (exact; equals the
// reference's float accumulation of integer levels below 2^24), float(sum) / n as in
// avg_pool.hpp:236-262, then optional Multiply and FakeQuantize.
template <bool RCP>
__global__ __launch_bounds__(kThreads) void avg_pool_nhwc_i8(PoolArgs a) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    const int cg = a.cs / 4;
    if (t >= static_cast<int64_t>(a.M) * cg) return;
    const int m = static_cast<int>(t / cg), c = static_cast<int>(t % cg) * 4;
    const int n = m / a.OHOW, rem = m - n * a.OHOW, oh = rem / a.OW, ow = rem - oh * a.OW;
    const int y0 = oh * a.sh - a.pt, x0 = ow * a.sw - a.pl;
    const int y1 = min(y0 + a.kh, a.H + a.pb), x1 = min(x0 + a.kw, a.W + a.pr);
    const bool padding_present = a.pt || a.pl || a.pb || a.pr;
    int sum[4] = {0, 0, 0, 0};
    // the in-bounds part of the window, walked two rows x eight columns at a time with all sixteen
    // loads requested before the first add (a global 7x7 pool is 49 dependent round trips otherwise)
    const int ya = max(y0, 0), yb = min(y1, a.H), xa = max(x0, 0), xb = min(x1, a.W);
    const int cells = max(yb - ya, 0) * max(xb - xa, 0);
    int count = padding_present ? cells : (y1 - y0) * (x1 - x0);
    const int8_t* base = static_cast<const int8_t*>(a.in) + static_cast<int64_t>(n) * a.in_sn + c;
    for (int y = ya; y < yb; y += 2)
        for (int x = xa; x < xb; x += 8) {
            uint32_t v[2][8];
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const bool ok = y + r < yb && x + i < xb;
                    const int yy = ok ? y + r : ya, xx = ok ? x + i : xa;   // clamped onto an existing cell
                    const uint32_t t = *reinterpret_cast<const uint32_t*>(base + static_cast<int64_t>(yy) * a.in_sh + xx * a.in_sw);
                    v[r][i] = ok ? t : 0u;
                }
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) sum[j] += static_cast<int8_t>(v[r][i] >> (8 * j));
        }
    if (a.include_pad && padding_present) count = a.kh * a.kw;
    const float nf = static_cast<float>(count);
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float x = static_cast<float>(sum[j] + a.in_bias * cells) / nf;
        if (a.mul) x = x * a.mul[c + j];
        v[j] = x;
    }
    const int64_t o = static_cast<int64_t>(n) * a.out_sn + oh * a.out_sh + ow * a.out_sw + c;
    if (a.preserve) {
        // avg_pool.hpp:236-262 for T = uint8_t / int8_t: T result (the sum wraps like the type), then
        // static_cast<T>(nearbyint(float(result) / n)); stored as the tensor stores levels (u8: level - 128)
        uint32_t packed = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int total = sum[j] + a.in_bias * cells;
            const int r = a.preserve == 1 ? (total & 0xff) : static_cast<int>(static_cast<int8_t>(total & 0xff));
            const int level = static_cast<int>(__builtin_rintf(static_cast<float>(r) / nf));
            packed |= (static_cast<uint32_t>(level - (a.preserve == 1 ? 128 : 0)) & 0xffu) << (8 * j);
        }
        *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(a.out) + o) = packed;
    } else if (a.fq_il) {
        uint32_t packed = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            FqChannel p;
            p.il = a.fq_il[c + j]; p.ih = a.fq_ih[c + j]; p.d = a.fq_d[c + j]; p.r = a.fq_r[c + j];
            const float k = fq_level_clamped<RCP>(p, a.lm1, v[j]);
            packed |= (static_cast<uint32_t>(static_cast<int>(k + a.out_off)) & 0xffu) << (8 * j);
        }
        *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(a.out) + o) = packed;
    } else {
        *reinterpret_cast<float4*>(static_cast<float*>(a.out) + o) = make_float4(v[0], v[1], v[2], v[3]);
    }
}

// NHWC engine tensor -> dense NCHW f32 (optionally (x - sub[c]) * mul[c]) or NCHW u8 levels.
// A block transposes 64 pixels x 64 channels through LDS: channel-contiguous reads, pixel-
// contiguous writes.
template <typename TIn>
__global__ __launch_bounds__(kThreads) void exit_nhwc_to_nchw(ExitArgs a) {
    __shared__ float tile[64][65];
    const int n = blockIdx.z, p0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int i = ty; i < 64; i += 4) {   // pixel p0 + i, channel c0 + tx
        const int p = p0 + i, c = c0 + tx;
        float v = 0.f;
        if (p < a.HW && c < a.C) {
            const int h = p / a.W, w = p - h * a.W;
            const TIn raw = static_cast<const TIn*>(a.in)[static_cast<int64_t>(n) * a.in_sn + h * a.in_sh + w * a.in_sw + c];
            v = static_cast<float>(raw) + a.in_bias;
            if (a.sub) v = v - a.sub[c];
            if (a.mul) v = v * a.mul[c];
        }
        tile[i][tx] = v;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {   // channel c0 + i, pixel p0 + tx
        const int p = p0 + tx, c = c0 + i;
        if (p < a.HW && c < a.C) {
            const int64_t o = (static_cast<int64_t>(n) * a.C + c) * a.HW + p;
            if (a.out_u8) static_cast<uint8_t*>(a.out)[o] = static_cast<uint8_t>(static_cast<int>(tile[tx][i]));
            else static_cast<float*>(a.out)[o] = tile[tx][i];
        }
    }
}

}  // namespace

void launch_max_pool(const PoolArgs& a, hipStream_t s) {
    const int vec = a.cs % 16 == 0 ? 4 : 1;
    const int64_t threads = static_cast<int64_t>(a.M) * (a.cs / (4 * vec));
    // no 3 x 3 window is trimmed at the padded upper bound: the last one ends at (OH-1)*s - pad + 3 <= H + pad_end
    // (a trimmed cell inside the tensor would have to be left out; cells in the padding never count)
    const int OH = a.OHOW / a.OW;
    const bool k3 = a.kh == 3 && a.kw == 3 && (OH - 1) * a.sh - a.pt + 3 <= a.H + a.pb &&
                    (a.OW - 1) * a.sw - a.pl + 3 <= a.W + a.pr;
    const dim3 grid(static_cast<uint32_t>(ceil_div(threads, kThreads)));
    if (k3 && vec == 4) hipLaunchKernelGGL((max_pool_nhwc_i8<true, 4>), grid, dim3(kThreads), 0, s, a);
    else if (vec == 4) hipLaunchKernelGGL((max_pool_nhwc_i8<false, 4>), grid, dim3(kThreads), 0, s, a);
    else if (k3) hipLaunchKernelGGL((max_pool_nhwc_i8<true, 1>), grid, dim3(kThreads), 0, s, a);
    else hipLaunchKernelGGL((max_pool_nhwc_i8<false, 1>), grid, dim3(kThreads), 0, s, a);
}

void launch_avg_pool(const PoolArgs& a, bool rcp, hipStream_t s) {
    const int64_t threads = static_cast<int64_t>(a.M) * (a.cs / 4);
    auto k = rcp ? avg_pool_nhwc_i8<true> : avg_pool_nhwc_i8<false>;
    hipLaunchKernelGGL(k, dim3(static_cast<uint32_t>(ceil_div(threads, kThreads))), dim3(kThreads), 0, s, a);
}

void launch_exit(const ExitArgs& a, int in_dtype, hipStream_t s) {
    dim3 grid(static_cast<uint32_t>(ceil_div(a.HW, 64)), static_cast<uint32_t>(ceil_div(a.C, 64)),
              static_cast<uint32_t>(a.N));
    if (in_dtype == HIPIE_F32) hipLaunchKernelGGL(exit_nhwc_to_nchw<float>, grid, dim3(kThreads), 0, s, a);
    else if (in_dtype == HIPIE_I32) hipLaunchKernelGGL(exit_nhwc_to_nchw<int32_t>, grid, dim3(kThreads), 0, s, a);
    else hipLaunchKernelGGL(exit_nhwc_to_nchw<int8_t>, grid, dim3(kThreads), 0, s, a);
}

namespace {

// VEC bytes per thread and copy: 16 when the slice starts and ends on 16-byte boundaries of the output pixel, 4 on
// 4-byte boundaries, else single bytes.  Consecutive threads take consecutive pieces of one pixel, then the next pixel.
template <int VEC>
__global__ __launch_bounds__(256) void concat_channels_kernel(const ConcatArgs a, int32_t pieces, float inv_pieces,
                                                              float inv_W, float inv_HW, int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    // idx -> (pixel, piece) -> (n, h, w): float reciprocals give an estimate of each quotient (the host keeps every
    // quotient below 2^24), the remainder corrects it exactly
    auto divmod = [](int64_t v, int32_t d, float inv, int32_t& q, int32_t& r) {
        q = static_cast<int32_t>(static_cast<float>(v) * inv);
        int64_t rem = v - static_cast<int64_t>(q) * d;
        // the dividend may exceed 2^24 (only the quotient is below it): its conversion, the reciprocal and the product
        // each round, so the estimate can be off by a few units - corrected until the remainder is in range
        while (rem < 0) { --q; rem += d; }
        while (rem >= d) { ++q; rem -= d; }
        r = static_cast<int32_t>(rem);
    };
    int32_t pix, piece, n, hw, h, w;
    divmod(idx, pieces, inv_pieces, pix, piece);
    divmod(pix, a.H * a.W, inv_HW, n, hw);
    divmod(hw, a.W, inv_W, h, w);
    const int8_t* src = a.in + n * a.in_sn + h * a.in_sh + w * a.in_sw + piece * VEC;
    int8_t* dst = a.out + n * a.out_sn + h * a.out_sh + w * a.out_sw + a.c_off + piece * VEC;
    if (VEC == 16) *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(src);
    else if (VEC == 4) *reinterpret_cast<uint32_t*>(dst) = *reinterpret_cast<const uint32_t*>(src);
    else *dst = *src;
}

}  // namespace

void launch_concat_channels(const ConcatArgs& a, hipStream_t s) {
    const int64_t pixels = static_cast<int64_t>(a.N) * a.H * a.W;
    if (pixels == 0 || a.C == 0) return;
    auto aligned = [&](int v) {
        return a.C % v == 0 && a.c_off % v == 0 && reinterpret_cast<uintptr_t>(a.out) % v == 0 && reinterpret_cast<uintptr_t>(a.in) % v == 0 &&
               a.out_sw % v == 0 && a.out_sh % v == 0 && a.out_sn % v == 0 && a.in_sw % v == 0 && a.in_sh % v == 0 && a.in_sn % v == 0;
    };
    const bool al16 = aligned(16), al4 = aligned(4);
    const int vec = al16 ? 16 : (al4 ? 4 : 1);
    const int32_t pieces = a.C / vec;
    const int64_t total = pixels * pieces;
    HIPIE_REQUIRE(pixels < (1 << 24) && total < (int64_t(1) << 31) * 256, HIPIE_OUT_OF_BOUNDS, "Concat: %lld pixels", (long long)pixels);
    // the piece quotient must stay exact too: idx / pieces < 2^24 holds because it is the pixel index
    const dim3 grid(static_cast<uint32_t>(ceil_div(total, 256))), block(256);
    const float ip = 1.0f / static_cast<float>(pieces), iw = 1.0f / static_cast<float>(a.W), ihw = 1.0f / static_cast<float>(a.H * a.W);
    if (vec == 16) hipLaunchKernelGGL(concat_channels_kernel<16>, grid, block, 0, s, a, pieces, ip, iw, ihw, total);
    else if (vec == 4) hipLaunchKernelGGL(concat_channels_kernel<4>, grid, block, 0, s, a, pieces, ip, iw, ihw, total);
    else hipLaunchKernelGGL(concat_channels_kernel<1>, grid, block, 0, s, a, pieces, ip, iw, ihw, total);
}

}  // namespace hipie
