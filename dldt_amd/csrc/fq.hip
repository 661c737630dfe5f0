// FakeQuantize / requantize kernels (HBM-bound) and their load-time object.
// Reference semantics: ngraph/core/reference/.../fake_quantize.hpp:175-265.
//
// Traffic per element: 4 B read + 1 B written (q8 forms) or + 4 B written (f32 op form).
// One wave reads 64 x 16 B = 1 KiB contiguous per load instruction; the per-channel table
// (32 B per channel) stays in L1/L2.
#include "fq.h"

#include <algorithm>
#include <atomic>
#include <cmath>

namespace hipie {

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ uint32_t pack_levels(float k0, float k1, float k2, float k3, float off) {
    // levels are small integers held exactly in floats; off shifts them into the output type
    const uint32_t b0 = static_cast<uint32_t>(static_cast<int>(k0 + off)) & 0xffu;
    const uint32_t b1 = static_cast<uint32_t>(static_cast<int>(k1 + off)) & 0xffu;
    const uint32_t b2 = static_cast<uint32_t>(static_cast<int>(k2 + off)) & 0xffu;
    const uint32_t b3 = static_cast<uint32_t>(static_cast<int>(k3 + off)) & 0xffu;
    return b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
}

// [N, C, HW] f32 -> same layout, one byte per element.  hw4 = HW / 4 (HW % 4 == 0).
template <bool RCP>
__global__ __launch_bounds__(kThreads) void fq_nchw_q8_vec4(const float4* __restrict__ x,
                                                             uint32_t* __restrict__ y,
                                                             const FqChannel* __restrict__ tab,
                                                             float lm1, float off, int64_t n4,
                                                             uint32_t hw4, uint32_t C) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n4; i += stride) {
        const uint32_t plane = static_cast<uint32_t>(i / hw4);
        const FqChannel p = tab[plane % C];
        const float4 v = x[i];
        y[i] = pack_levels(fq_level_clamped<RCP>(p, lm1, v.x), fq_level_clamped<RCP>(p, lm1, v.y),
                           fq_level_clamped<RCP>(p, lm1, v.z), fq_level_clamped<RCP>(p, lm1, v.w),
                           off);
    }
}

// any HW: one element per thread-iteration
template <bool RCP>
__global__ __launch_bounds__(kThreads) void fq_nchw_q8_scalar(const float* __restrict__ x,
                                                               uint8_t* __restrict__ y,
                                                               const FqChannel* __restrict__ tab,
                                                               float lm1, float off, int64_t n,
                                                               uint32_t hw, uint32_t C) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
        const FqChannel p = tab[static_cast<uint32_t>(i / hw) % C];
        y[i] = static_cast<uint8_t>(static_cast<int>(fq_level_clamped<RCP>(p, lm1, x[i]) + off));
    }
}

// f32 op form, same layout
template <bool RCP>
__global__ __launch_bounds__(kThreads) void fq_nchw_f32(const float* __restrict__ x,
                                                         float* __restrict__ y,
                                                         const FqChannel* __restrict__ tab,
                                                         float lm1, int64_t n, uint32_t hw,
                                                         uint32_t C) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
        const FqChannel p = tab[static_cast<uint32_t>(i / hw) % C];
        y[i] = fq_value<RCP>(p, lm1, x[i]);
    }
}

template <bool RCP>
__global__ __launch_bounds__(kThreads) void fq_nchw_f32_vec4(const float4* __restrict__ x,
                                                              float4* __restrict__ y,
                                                              const FqChannel* __restrict__ tab,
                                                              float lm1, int64_t n4, uint32_t hw4,
                                                              uint32_t C) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n4; i += stride) {
        const FqChannel p = tab[static_cast<uint32_t>(i / hw4) % C];
        const float4 v = x[i];
        float4 o;
        o.x = fq_value<RCP>(p, lm1, v.x);
        o.y = fq_value<RCP>(p, lm1, v.y);
        o.z = fq_value<RCP>(p, lm1, v.z);
        o.w = fq_value<RCP>(p, lm1, v.w);
        y[i] = o;
    }
}

// [N, C, HW] f32 -> [N, HW, c_stride] bytes.  A block transposes 64 pixels x 64 channels
// through LDS so that both the f32 reads (256 B per channel row) and the byte writes (16 B per
// thread, whole pixels contiguous) are coalesced.  grid = (N * ceil(HW/64), ceil(c_stride/64)).
template <bool RCP, typename TIn = float>
__global__ __launch_bounds__(kThreads) void fq_nchw_to_nhwc_q8(const TIn* __restrict__ x,
                                                                uint8_t* __restrict__ y,
                                                                const FqChannel* __restrict__ tab,
                                                                float lm1, float off, uint32_t hw,
                                                                uint32_t C, uint32_t c_stride,
                                                                uint32_t tiles_per_image, uint32_t W,
                                                                int64_t out_sn, int64_t out_sh) {
    __shared__ uint32_t tile[64][17];  // [pixel][16 dwords = 64 channel bytes] + 1 pad
    const uint32_t n = blockIdx.x / tiles_per_image;
    const uint32_t p0 = (blockIdx.x % tiles_per_image) * 64;
    const uint32_t c0 = blockIdx.y * 64;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t pix = p0 + lane;
    // each wave quantises 16 channels of the 64; a lane owns one pixel and packs 4 channels/dword
    for (uint32_t cc = 0; cc < 16; cc += 4) {
        float k[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t c = c0 + wave * 16 + cc + j;
            if (c < C && pix < hw) {
                const FqChannel p = tab[c];
                k[j] = fq_level_clamped<RCP>(p, lm1, static_cast<float>(x[(static_cast<int64_t>(n) * C + c) * hw + pix]));
            } else {
                k[j] = 0.0f;
            }
        }
        tile[lane][wave * 4 + cc / 4] = pack_levels(k[0], k[1], k[2], k[3], off);
    }
    __syncthreads();
    // 256 threads x 16 B: thread t writes channels [16*(t%4), +16) of pixel t/4
    const uint32_t op = threadIdx.x >> 2, oq = threadIdx.x & 3;
    const uint32_t cbyte = c0 + oq * 16;
    if (p0 + op < hw && cbyte < c_stride) {
        uint4 v;
        v.x = tile[op][oq * 4 + 0];
        v.y = tile[op][oq * 4 + 1];
        v.z = tile[op][oq * 4 + 2];
        v.w = tile[op][oq * 4 + 3];
        const uint32_t ph = (p0 + op) / W, pw = (p0 + op) - ph * W;
        uint8_t* dst = y + static_cast<int64_t>(n) * out_sn + ph * out_sh + static_cast<int64_t>(pw) * c_stride + cbyte;
        if (cbyte + 16 <= c_stride && c_stride % 16 == 0) {
            *reinterpret_cast<uint4*>(dst) = v;
        } else {  // c_stride is a multiple of 4
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
            for (uint32_t j = 0; j < 4 && cbyte + 4 * j < c_stride; ++j)
                reinterpret_cast<uint32_t*>(dst)[j] = w[j];
        }
    }
}

__device__ __forceinline__ float4 load4_as_float(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4_as_float(const uint8_t* p) {   // convert<uint8_t, float>: exact
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    return make_float4(static_cast<float>(w & 0xffu), static_cast<float>((w >> 8) & 0xffu),
                       static_cast<float>((w >> 16) & 0xffu), static_cast<float>(w >> 24));
}

// The same transposition for HW % 4 == 0, 256 pixels x 64 channels per workgroup.  A lane reads float4s (four
// consecutive pixels of one channel; a wave's load instruction is 1 KB contiguous) of four consecutive channels at a
// time, sixteen loads in flight per lane, and packs each pixel's four channels into one dword.  LDS holds the tile as
// [16 channel dwords][256 pixels + 4]: the four dwords a lane produces per step are one conflict-free 16-byte write, and
// the write-out reads (four lanes per pixel, 64 contiguous bytes per pixel and wave instruction) meet two-way at most.
template <bool RCP, typename TIn = float>
__global__ __launch_bounds__(kThreads) void fq_nchw_to_nhwc_q8_wide(const TIn* __restrict__ x, uint8_t* __restrict__ y,
                                                                     const FqChannel* __restrict__ tab, float lm1, float off,
                                                                     uint32_t hw, uint32_t C, uint32_t c_stride,
                                                                     uint32_t tiles_per_image, uint32_t W, float inv_W,
                                                                     int64_t out_sn, int64_t out_sh) {
    constexpr uint32_t kRow = 256 + 4;
    __shared__ __attribute__((aligned(16))) uint32_t tile[16 * kRow];
    __shared__ __attribute__((aligned(16))) FqChannel chan[64];        // the tile's channels (from memory: two more vector
                                                                         // loads per channel and lane)
    const uint32_t n = blockIdx.x / tiles_per_image;
    const uint32_t p0 = (blockIdx.x - n * tiles_per_image) * 256;
    const uint32_t c0 = blockIdx.y * 64;
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t pix = p0 + 4 * lane;
    const bool pix_on = pix < hw;                      // HW % 4 == 0: a group of four is inside or outside as a whole
    if (threadIdx.x < 64) chan[threadIdx.x] = tab[min(c0 + threadIdx.x, C - 1)];
    float4 v[4][4];                                    // [step][channel of the quad]
#pragma unroll
    for (uint32_t it = 0; it < 4; ++it)
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t c = c0 + 4 * (wave + 4 * it) + j;
            v[it][j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (pix_on && c < C) v[it][j] = load4_as_float(x + (static_cast<int64_t>(n) * C + c) * hw + pix);
        }
    __syncthreads();
#pragma unroll
    for (uint32_t it = 0; it < 4; ++it) {
        const uint32_t cq = wave + 4 * it;
        float k[4][4];                                 // [channel][pixel]
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t c = c0 + 4 * cq + j;
            if (pix_on && c < C) {
                const FqChannel p = chan[4 * cq + j];
                k[j][0] = fq_level_clamped<RCP>(p, lm1, v[it][j].x);
                k[j][1] = fq_level_clamped<RCP>(p, lm1, v[it][j].y);
                k[j][2] = fq_level_clamped<RCP>(p, lm1, v[it][j].z);
                k[j][3] = fq_level_clamped<RCP>(p, lm1, v[it][j].w);
            } else {
                k[j][0] = k[j][1] = k[j][2] = k[j][3] = 0.0f;
            }
        }
        uint4 o;
        o.x = pack_levels(k[0][0], k[1][0], k[2][0], k[3][0], off);
        o.y = pack_levels(k[0][1], k[1][1], k[2][1], k[3][1], off);
        o.z = pack_levels(k[0][2], k[1][2], k[2][2], k[3][2], off);
        o.w = pack_levels(k[0][3], k[1][3], k[2][3], k[3][3], off);
        *reinterpret_cast<uint4*>(&tile[cq * kRow + 4 * lane]) = o;
    }
    __syncthreads();
    // thread t writes channels [16 * (t % 4), + 16) of pixels t / 4 + 64 * i
    const uint32_t oq = threadIdx.x & 3;
    const uint32_t cbyte = c0 + oq * 16;
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t op = (threadIdx.x >> 2) + 64 * i;
        if (p0 + op >= hw || cbyte >= c_stride) continue;
        uint4 o;
        o.x = tile[(4 * oq + 0) * kRow + op];
        o.y = tile[(4 * oq + 1) * kRow + op];
        o.z = tile[(4 * oq + 2) * kRow + op];
        o.w = tile[(4 * oq + 3) * kRow + op];
        // pixel -> (row, column) through the reciprocal: exact below 2^24 after one correction
        uint32_t ph = static_cast<uint32_t>(static_cast<float>(p0 + op) * inv_W);
        int32_t pw = static_cast<int32_t>(p0 + op) - static_cast<int32_t>(ph * W);
        if (pw < 0) { --ph; pw += static_cast<int32_t>(W); }
        else if (pw >= static_cast<int32_t>(W)) { ++ph; pw -= static_cast<int32_t>(W); }
        uint8_t* dst = y + static_cast<int64_t>(n) * out_sn + ph * out_sh + static_cast<int64_t>(pw) * c_stride + cbyte;
        if (cbyte + 16 <= c_stride && c_stride % 16 == 0) {
            *reinterpret_cast<uint4*>(dst) = o;
        } else {  // c_stride is a multiple of 4
            const uint32_t w[4] = {o.x, o.y, o.z, o.w};
            for (uint32_t j = 0; j < 4 && cbyte + 4 * j < c_stride; ++j)
                reinterpret_cast<uint32_t*>(dst)[j] = w[j];
        }
    }
}

// The same transposition for tensors of 128 channels and more: a workgroup takes 32 pixels x 256 channels, so that it
// writes whole pixels (256 contiguous bytes each, 8 KB per tile where the row continues) instead of 64-byte quarters
// of 256 pixels, and holds 32 KB of input in flight instead of 64: eight workgroups per compute unit pass through
// load, quantise and store at different times.  Loads are 128 contiguous bytes per channel (8 lanes x 16 B).
// (Measured beside it: 64 pixels x 256 channels 29.7 us, 64 x 128 26.1, 16 x 256 - half cache lines per channel -
// 34.0, and a persistent form that requests the next tile before it quantises the current one 27.7 - 32.3 us, against
// 26.0 us for this one on [32, 256, 56, 56].)
template <bool RCP, typename TIn = float>
__global__ __launch_bounds__(kThreads) void fq_nchw_to_nhwc_q8_lines(const TIn* __restrict__ x, uint8_t* __restrict__ y,
                                                                       const FqChannel* __restrict__ tab, float lm1, float off,
                                                                       uint32_t hw, uint32_t C, uint32_t c_stride,
                                                                       uint32_t tiles_per_image, uint32_t W, float inv_W,
                                                                       int64_t out_sn, int64_t out_sh) {
    constexpr uint32_t kPix = 64 + 4;                  // dwords per pixel row of the tile: 64 channel quads + padding
    __shared__ __attribute__((aligned(16))) uint32_t tile[32 * kPix];
    __shared__ __attribute__((aligned(16))) FqChannel chan[256];       // the tile's channels: read from memory they are two
                                                                         // more vector loads per channel and lane
    const uint32_t n = blockIdx.x / tiles_per_image;
    const uint32_t p0 = (blockIdx.x - n * tiles_per_image) * 32;
    const uint32_t c0 = blockIdx.y * 256;
    const uint32_t pg = threadIdx.x & 7, cq_lo = threadIdx.x >> 3;
    const uint32_t pix = p0 + 4 * pg;
    const bool pix_on = pix < hw;                      // HW % 4 == 0: a group of four is inside or outside as a whole
    chan[threadIdx.x] = tab[min(c0 + threadIdx.x, C - 1)];
    float4 v[2][4];                                    // [step][channel of the quad]
#pragma unroll
    for (uint32_t it = 0; it < 2; ++it)
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t c = c0 + 4 * (cq_lo + 32 * it) + j;
            v[it][j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (pix_on && c < C) v[it][j] = load4_as_float(x + (static_cast<int64_t>(n) * C + c) * hw + pix);
        }
    __syncthreads();
#pragma unroll
    for (uint32_t it = 0; it < 2; ++it) {
        const uint32_t cq = cq_lo + 32 * it;
        float k[4][4];                                 // [channel][pixel]
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t c = c0 + 4 * cq + j;
            if (pix_on && c < C) {
                const FqChannel p = chan[4 * cq + j];
                k[j][0] = fq_level_clamped<RCP>(p, lm1, v[it][j].x);
                k[j][1] = fq_level_clamped<RCP>(p, lm1, v[it][j].y);
                k[j][2] = fq_level_clamped<RCP>(p, lm1, v[it][j].z);
                k[j][3] = fq_level_clamped<RCP>(p, lm1, v[it][j].w);
            } else {
                k[j][0] = k[j][1] = k[j][2] = k[j][3] = 0.0f;
            }
        }
#pragma unroll
        for (uint32_t e = 0; e < 4; ++e) tile[(4 * pg + e) * kPix + cq] = pack_levels(k[0][e], k[1][e], k[2][e], k[3][e], off);
    }
    __syncthreads();
    // thread t writes channels [16 * (t % 16), + 16) of pixels t / 16 and t / 16 + 16
    const uint32_t chunk = threadIdx.x & 15;
    const uint32_t cbyte = c0 + chunk * 16;
#pragma unroll
    for (uint32_t i = 0; i < 2; ++i) {
        const uint32_t op = (threadIdx.x >> 4) + 16 * i;
        if (p0 + op >= hw || cbyte >= c_stride) continue;
        const uint4 o = *reinterpret_cast<const uint4*>(&tile[op * kPix + 4 * chunk]);
        // pixel -> (row, column) through the reciprocal: exact below 2^24 after one correction
        uint32_t ph = static_cast<uint32_t>(static_cast<float>(p0 + op) * inv_W);
        int32_t pw = static_cast<int32_t>(p0 + op) - static_cast<int32_t>(ph * W);
        if (pw < 0) { --ph; pw += static_cast<int32_t>(W); }
        else if (pw >= static_cast<int32_t>(W)) { ++ph; pw -= static_cast<int32_t>(W); }
        uint8_t* dst = y + static_cast<int64_t>(n) * out_sn + ph * out_sh + static_cast<int64_t>(pw) * c_stride + cbyte;
        if (cbyte + 16 <= c_stride && c_stride % 16 == 0) {
            *reinterpret_cast<uint4*>(dst) = o;
        } else {  // c_stride is a multiple of 4
            const uint32_t w[4] = {o.x, o.y, o.z, o.w};
            for (uint32_t j = 0; j < 4 && cbyte + 4 * j < c_stride; ++j)
                reinterpret_cast<uint32_t*>(dst)[j] = w[j];
        }
    }
}

// Image-like inputs (C <= 4) -> pixels of 4 bytes: a thread quantises 4 consecutive pixels of one
// row from C coalesced float4 reads and writes 16 contiguous bytes.  W % 4 == 0.

template <bool RCP, typename TIn = float>
__global__ __launch_bounds__(kThreads) void fq_nchw_to_nhwc4_q8(const TIn* __restrict__ x,
                                                                 uint8_t* __restrict__ y,
                                                                 const FqChannel* __restrict__ tab,
                                                                 float lm1, float off, uint32_t C,
                                                                 uint32_t H, uint32_t W, float inv_w4, int64_t out_sn,
                                                                 int64_t out_sh) {
    // grid: (groups of four pixels of one image / (256 * kItems), images); 32-bit index arithmetic, the row by a
    // reciprocal (exact below 2^24 after one correction; the host passes inv_w4 = 0 -> integer division above that).
    // A thread takes kItems groups a workgroup's width apart and requests all their planes before it quantises the
    // first.  One group per thread is the fastest for a batch of 64 images of 224 x 224 (12 544 waves; with four
    // groups the 3136 waves left do not fill the chip and the kernel takes 22 us instead of 15).
    constexpr uint32_t kItems = 1;
    const uint32_t w4 = W / 4, n = blockIdx.y, items = H * w4;
    uint32_t h[kItems], wq[kItems];
    bool on[kItems];
    float4 v[kItems][4];
#pragma unroll
    for (uint32_t t = 0; t < kItems; ++t) {
        const uint32_t i = (blockIdx.x * kItems + t) * kThreads + threadIdx.x;
        on[t] = i < items;
        const uint32_t ii = on[t] ? i : 0;
        if (inv_w4 > 0.0f) {
            uint32_t hh = static_cast<uint32_t>(static_cast<float>(ii) * inv_w4);
            int32_t ww = static_cast<int32_t>(ii) - static_cast<int32_t>(hh * w4);
            if (ww < 0) { --hh; ww += static_cast<int32_t>(w4); }
            else if (ww >= static_cast<int32_t>(w4)) { ++hh; ww -= static_cast<int32_t>(w4); }
            h[t] = hh;
            wq[t] = static_cast<uint32_t>(ww);
        } else {
            h[t] = ii / w4;
            wq[t] = ii - h[t] * w4;
        }
#pragma unroll
        for (uint32_t c = 0; c < 4; ++c)
            if (c < C) v[t][c] = load4_as_float(x + ((static_cast<int64_t>(n) * C + c) * H + h[t]) * W + wq[t] * 4);
    }
#pragma unroll
    for (uint32_t t = 0; t < kItems; ++t) {
        float k[4][4];   // [pixel][channel]
#pragma unroll
        for (uint32_t c = 0; c < 4; ++c) {
            if (c < C) {
                const FqChannel p = tab[c];
                k[0][c] = fq_level_clamped<RCP>(p, lm1, v[t][c].x);
                k[1][c] = fq_level_clamped<RCP>(p, lm1, v[t][c].y);
                k[2][c] = fq_level_clamped<RCP>(p, lm1, v[t][c].z);
                k[3][c] = fq_level_clamped<RCP>(p, lm1, v[t][c].w);
            } else {
                k[0][c] = k[1][c] = k[2][c] = k[3][c] = 0.0f;
            }
        }
        if (!on[t]) continue;
        // a row of a tensor with a halo starts on a 4-byte boundary only: four dword stores (exchanging the wave's 256
        // dwords between the lanes first, so that every store instruction writes 64 consecutive dwords, was slower:
        // 14.2 against 11.3 us in the network)
        uint32_t* dst = reinterpret_cast<uint32_t*>(y + static_cast<int64_t>(n) * out_sn + h[t] * out_sh + static_cast<int64_t>(wq[t]) * 16);
#pragma unroll
        for (uint32_t p = 0; p < 4; ++p) dst[p] = pack_levels(k[p][0], k[p][1], k[p][2], k[p][3], off);
    }
}

int grid_for(int64_t work_items) {
    // enough blocks to fill 256 CUs several times over, capped so the grid-stride loop amortises
    const int64_t blocks = ceil_div(work_items, kThreads);
    return static_cast<int>(std::min<int64_t>(blocks, 256 * 16));
}

// r = correctly rounded 1/d: pick among the neighbours of (float)(1.0/d) the one whose exact
// residual |1 - d*r| (a product of two floats is exact in double) is smallest.
}  // namespace

float fq_rounded_reciprocal(float d) {
    float r = static_cast<float>(1.0 / static_cast<double>(d));
    float best = r;
    double best_err = std::fabs(1.0 - static_cast<double>(d) * r);
    for (float cand : {std::nextafterf(r, INFINITY), std::nextafterf(r, -INFINITY)}) {
        const double err = std::fabs(1.0 - static_cast<double>(d) * cand);
        if (err < best_err) { best = cand; best_err = err; }
    }
    return best;
}

namespace {

// monotone map float <-> ordered int, for bisection over floats
int32_t ordered(float f) {
    int32_t i;
    std::memcpy(&i, &f, 4);
    return i < 0 ? static_cast<int32_t>(0x80000000u - static_cast<uint32_t>(i)) : i;
}
float unordered(int32_t o) {
    int32_t i = o < 0 ? static_cast<int32_t>(0x80000000u - static_cast<uint32_t>(o)) : o;
    float f;
    std::memcpy(&f, &i, 4);
    return f;
}

}  // namespace

namespace {

thread_local FqVerdicts* t_verdicts = nullptr;

std::array<uint32_t, 5> rcp_key(const FqChannel& p, float lm1) {
    std::array<uint32_t, 5> k;
    const float v[5] = {p.il, p.ih, p.d, p.r, lm1};
    std::memcpy(k.data(), v, sizeof v);
    return k;
}

bool check_boundaries(const FqChannel& p, float lm1) {
    if (!(p.il < p.ih)) return false;
    if (!(std::fabs(p.d) > 0x1p-60f && std::fabs(p.d) < 0x1p60f)) return false;
    uint32_t bits;
    std::memcpy(&bits, &p.d, 4);
    if ((bits & 0x7fffffu) == 0x7fffffu) return false;  // all-ones significand: excluded by the theorem
    const int levels = static_cast<int>(lm1) + 1;
    const int32_t o_lo = ordered(p.il), o_hi = ordered(p.ih);
    for (int k = 1; k < levels; ++k) {
        // smallest x in (il, ih] whose reference level is >= k (the level is monotone in x)
        // (64-bit: the ordered images of il <= -2 and ih >= 2 are 2^31 or more apart)
        int64_t a = o_lo, b = o_hi;  // level(a) < k <= level(b)
        if (fq_level_div(p, lm1, p.ih) < k) break;
        while (b - a > 1) {
            const int64_t m = a + (b - a) / 2;
            if (fq_level_div(p, lm1, unordered(static_cast<int32_t>(m))) >= k) b = m; else a = m;
        }
        for (int64_t o : {a, b, b + 1 <= o_hi ? b + 1 : b, a - 1 >= o_lo ? a - 1 : a}) {
            const float x = unordered(static_cast<int32_t>(o));
            if (fq_level_rcp(p, lm1, x) != fq_level_div(p, lm1, x)) return false;
        }
    }
    return true;
}


}  // namespace

FqVerdicts::Scope::Scope(FqVerdicts* v) : previous(t_verdicts) { t_verdicts = v; }
FqVerdicts::Scope::~Scope() { t_verdicts = previous; }
FqVerdicts* FqVerdicts::current() { return t_verdicts; }

bool fq_reciprocal_exact_on_boundaries(const FqChannel& p, float lm1) { return fq_reciprocal_exact_on_all(&p, 1, lm1); }

bool fq_reciprocal_exact_on_all(const FqChannel* p, int64_t n, float lm1) {
    FqVerdicts* table = t_verdicts;
    std::map<std::array<uint32_t, 5>, uint32_t> local;
    std::map<std::array<uint32_t, 5>, uint32_t>& known = table ? table->rcp : local;
    std::vector<int64_t> open;                                  // first channel of every key not answered yet
    {
        std::map<std::array<uint32_t, 5>, int> asked;
        for (int64_t c = 0; c < n; ++c) {
            const auto key = rcp_key(p[c], lm1);
            const auto it = known.find(key);
            if (it != known.end()) {
                if (!it->second) return false;
            } else if (asked.emplace(key, 0).second) {
                open.push_back(c);
            }
        }
    }
    std::vector<uint32_t> verdict(open.size());
    parallel_for(static_cast<int64_t>(open.size()), [&](int64_t i) { verdict[i] = check_boundaries(p[open[i]], lm1) ? 1u : 0u; });
    bool all = true;
    for (size_t i = 0; i < open.size(); ++i) {
        known[rcp_key(p[open[i]], lm1)] = verdict[i];
        all = all && verdict[i];
    }
    return all;
}

}  // namespace hipie

using namespace hipie;

struct hipie_fq {
    int device = 0;
    int64_t C = 0;
    int64_t levels = 0;
    float lm1 = 0;
    bool rcp = false;           // reciprocal path proven on every boundary of every channel
    bool clamp_ok = false;      // il < ih everywhere (q8 kernels fold the saturating branches)
    bool q8_ok = false;         // op results are the integers out_low + k
    float q8_base = 0;          // out_low (integer valued) when q8_ok
    std::vector<FqChannel> host;
    DeviceBuffer table;
};

template <typename TIn>
void run_q8_tensor(const hipie_fq* fq, const TIn* x, const hipie_tensor* out, void* stream) {
    {
        HIPIE_REQUIRE(fq && out, HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8_tensor: null argument");
        HIPIE_REQUIRE(fq->table.ptr, HIPIE_NOT_ALLOCATED, "hipie_fq_run_q8_tensor: host-only object");
        const int64_t hw = static_cast<int64_t>(out->h) * out->w;
        if (out->n == 0 || hw == 0) return;
        HIPIE_REQUIRE(x && out->data, HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8_tensor: null data");
        HIPIE_REQUIRE(out->c == fq->C, HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8_tensor: %d channels, expected %lld",
                      out->c, (long long)fq->C);
        HIPIE_REQUIRE(fq->q8_ok && fq->clamp_ok, HIPIE_NOT_IMPLEMENTED,
                      "hipie_fq_run_q8_tensor: needs input_low < input_high and consecutive integer output levels");
        float off;
        if (out->dtype == HIPIE_U8B) off = fq->q8_base - 128.0f;
        else if (out->dtype == HIPIE_I8) off = fq->q8_base;
        else fail(HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8_tensor: output dtype %d", out->dtype);
        HIPIE_REQUIRE(out->dtype == HIPIE_U8B ? fq->q8_base >= 0 : fq->q8_base + fq->lm1 <= 127.0f,
                      HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8_tensor: levels do not fit the output type");
        const int64_t cs = out->stride_w;
        HIPIE_REQUIRE(cs >= fq->C && cs % 4 == 0 && reinterpret_cast<uintptr_t>(out->data) % 4 == 0 &&
                          (cs % 16 != 0 || reinterpret_cast<uintptr_t>(out->data) % 16 == 0),
                      HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8_tensor: channel stride / alignment");
        DeviceGuard g(fq->device);
        if (fq->C <= 4 && cs == 4 && out->w % 4 == 0) {
            auto k4 = fq->rcp ? fq_nchw_to_nhwc4_q8<true, TIn> : fq_nchw_to_nhwc4_q8<false, TIn>;
            const int64_t per_image = static_cast<int64_t>(out->h) * (out->w / 4);
            HIPIE_REQUIRE(per_image < (1ll << 31) && out->n <= 65535, HIPIE_OUT_OF_BOUNDS, "hipie_fq_run_q8_tensor: image too large");
            const float inv_w4 = per_image < (1 << 24) ? 1.0f / static_cast<float>(out->w / 4) : 0.0f;
            hipLaunchKernelGGL(k4, dim3(static_cast<uint32_t>(ceil_div(per_image, kThreads)), static_cast<uint32_t>(out->n)),
                               dim3(kThreads), 0, as_stream(stream), x, static_cast<uint8_t*>(out->data),
                               fq->table.as<FqChannel>(), fq->lm1, off, static_cast<uint32_t>(fq->C),
                               static_cast<uint32_t>(out->h), static_cast<uint32_t>(out->w), inv_w4, out->stride_n,
                               out->stride_h);
            HIPIE_CHECK_HIP(hipGetLastError());
            return;
        }
        if (hw % 4 == 0 && hw < (1 << 24) && cs >= 128) {   // whole float4s per lane, whole cache lines per pixel
            const uint32_t tiles = static_cast<uint32_t>(ceil_div(hw, 32));
            HIPIE_REQUIRE(static_cast<int64_t>(out->n) * tiles < (1ll << 31), HIPIE_OUT_OF_BOUNDS, "hipie_fq_run_q8_tensor: grid too large");
            auto kl = fq->rcp ? fq_nchw_to_nhwc_q8_lines<true, TIn> : fq_nchw_to_nhwc_q8_lines<false, TIn>;
            hipLaunchKernelGGL(kl, dim3(static_cast<uint32_t>(out->n * tiles), static_cast<uint32_t>(ceil_div(cs, 256))),
                               dim3(kThreads), 0, as_stream(stream), x, static_cast<uint8_t*>(out->data),
                               fq->table.as<FqChannel>(), fq->lm1, off, static_cast<uint32_t>(hw),
                               static_cast<uint32_t>(fq->C), static_cast<uint32_t>(cs), tiles,
                               static_cast<uint32_t>(out->w), 1.0f / static_cast<float>(out->w), out->stride_n, out->stride_h);
            HIPIE_CHECK_HIP(hipGetLastError());
            return;
        }
        if (hw % 4 == 0 && hw < (1 << 24)) {   // whole float4s per lane
            const uint32_t tiles = static_cast<uint32_t>(ceil_div(hw, 256));
            auto kw = fq->rcp ? fq_nchw_to_nhwc_q8_wide<true, TIn> : fq_nchw_to_nhwc_q8_wide<false, TIn>;
            hipLaunchKernelGGL(kw, dim3(static_cast<uint32_t>(out->n * tiles), static_cast<uint32_t>(ceil_div(cs, 64))),
                               dim3(kThreads), 0, as_stream(stream), x, static_cast<uint8_t*>(out->data),
                               fq->table.as<FqChannel>(), fq->lm1, off, static_cast<uint32_t>(hw),
                               static_cast<uint32_t>(fq->C), static_cast<uint32_t>(cs), tiles,
                               static_cast<uint32_t>(out->w), 1.0f / static_cast<float>(out->w), out->stride_n, out->stride_h);
            HIPIE_CHECK_HIP(hipGetLastError());
            return;
        }
        const uint32_t tiles = static_cast<uint32_t>(ceil_div(hw, 64));
        auto k = fq->rcp ? fq_nchw_to_nhwc_q8<true, TIn> : fq_nchw_to_nhwc_q8<false, TIn>;
        hipLaunchKernelGGL(k, dim3(static_cast<uint32_t>(out->n * tiles), static_cast<uint32_t>(ceil_div(cs, 64))),
                           dim3(kThreads), 0, as_stream(stream), x, static_cast<uint8_t*>(out->data),
                           fq->table.as<FqChannel>(), fq->lm1, off, static_cast<uint32_t>(hw),
                           static_cast<uint32_t>(fq->C), static_cast<uint32_t>(cs), tiles,
                           static_cast<uint32_t>(out->w), out->stride_n, out->stride_h);
        HIPIE_CHECK_HIP(hipGetLastError());
    }
}

namespace {

__device__ __forceinline__ void elt_load4(const EltOperand& o, int64_t pix_off, int c0, float (&v)[4]) {
    if (o.konst) {
        const float4 k = *reinterpret_cast<const float4*>(o.konst + c0);
        v[0] = k.x; v[1] = k.y; v[2] = k.z; v[3] = k.w;
        return;
    }
    if (o.dtype == HIPIE_F32) {
        const float4 k = *reinterpret_cast<const float4*>(static_cast<const float*>(o.p) + pix_off + c0);
        v[0] = k.x; v[1] = k.y; v[2] = k.z; v[3] = k.w;
    } else {
        const uint32_t w = *reinterpret_cast<const uint32_t*>(static_cast<const int8_t*>(o.p) + pix_off + c0);
        const int bias = o.dtype == HIPIE_U8B ? 128 : 0;   // stored byte = level - 128
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = static_cast<float>(static_cast<int>(static_cast<int8_t>(w >> (8 * j))) + bias);   // Convert
    }
    if (o.sub) {
        const float4 k = *reinterpret_cast<const float4*>(o.sub + c0);
        v[0] = v[0] - k.x; v[1] = v[1] - k.y; v[2] = v[2] - k.z; v[3] = v[3] - k.w;
    }
    if (o.mul) {
        const float4 k = *reinterpret_cast<const float4*>(o.mul + c0);
        v[0] = v[0] * k.x; v[1] = v[1] * k.y; v[2] = v[2] * k.z; v[3] = v[3] * k.w;
    }
}

// a thread computes four consecutive channels of one pixel
template <bool RCP>
__global__ __launch_bounds__(kThreads) void eltwise_nhwc_kernel(const EltArgs a, const FqChannel* __restrict__ tab, float lm1, float off,
                                                                int32_t groups, float inv_groups, float inv_W, float inv_HW,
                                                                int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (idx >= total) return;
    auto divmod = [](int64_t v, int32_t d, float inv, int32_t& q, int32_t& r) {   // estimate by reciprocal, exact by the remainder
        q = static_cast<int32_t>(static_cast<float>(v) * inv);
        int64_t rem = v - static_cast<int64_t>(q) * d;
        // the dividend may exceed 2^24 (only the quotient is below it): its conversion, the reciprocal and the product
        // each round, so the estimate can be off by a few units - corrected until the remainder is in range
        while (rem < 0) { --q; rem += d; }
        while (rem >= d) { ++q; rem -= d; }
        r = static_cast<int32_t>(rem);
    };
    int32_t pix, g, n, hw, h, w;
    divmod(idx, groups, inv_groups, pix, g);
    divmod(pix, a.H * a.W, inv_HW, n, hw);
    divmod(hw, a.W, inv_W, h, w);
    const int c0 = 4 * g;
    float v[4], u[4];
    elt_load4(a.a, n * a.a.sn + h * a.a.sh + w * a.a.sw, c0, v);
    if (a.op != 0) {
        elt_load4(a.b, n * a.b.sn + h * a.b.sh + w * a.b.sw, c0, u);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            v[j] = a.op == 1 ? v[j] + u[j] : (a.op == 2 ? v[j] - u[j] : (a.op == 3 ? v[j] * u[j] : (v[j] < 0.0f ? v[j] * u[j] : v[j])));   // 4: prelu.hpp:43
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (a.act == 1) v[j] = v[j] > 0.0f ? v[j] : 0.0f;                                    // relu.hpp
        else if (a.act == 2) v[j] = v[j] < a.lo ? a.lo : (v[j] > a.hi ? a.hi : v[j]);        // clamp.hpp
        else if (a.act == 3) v[j] = 1.0f / (1.0f + expf(-v[j]));                             // sigmoid.hpp
        else if (a.act == 4) v[j] = v[j] * fminf(fmaxf(v[j] + 3.0f, 0.0f), 6.0f) / 6.0f;     // hswish.hpp: (x * clamped) / 6
        else if (a.act == 5) v[j] = fminf(fmaxf(v[j] + 3.0f, 0.0f), 6.0f) / 6.0f;            // hsigmoid.hpp
        else if (a.act == 6) v[j] = static_cast<float>(static_cast<double>(v[j]) / (1.0 + static_cast<double>(expf(-v[j] * a.lo))));   // swish.hpp: the sum and the quotient in double
    }
    const int64_t o = n * a.out_sn + h * a.out_sh + w * a.out_sw + c0;
    if (tab) {
        float k[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) k[j] = c0 + j < a.C ? fq_level_clamped<RCP>(tab[c0 + j], lm1, v[j]) : 0.0f;
        *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(a.out) + o) = pack_levels(k[0], k[1], k[2], k[3], off);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = c0 + j < a.C ? v[j] : 0.0f;
        *reinterpret_cast<float4*>(static_cast<float*>(a.out) + o) = make_float4(v[0], v[1], v[2], v[3]);
    }
}

}  // namespace

bool hipie::fq_gives_levels(const hipie_fq* fq) { return fq && fq->q8_ok && fq->clamp_ok; }

void hipie::run_eltwise(const hipie_fq* fq, const EltArgs& a, hipStream_t s) {
    const int64_t pixels = static_cast<int64_t>(a.N) * a.H * a.W;
    if (pixels == 0 || a.C == 0) return;
    const int32_t groups = static_cast<int32_t>(ceil_div(a.C, 4));
    HIPIE_REQUIRE(pixels < (1 << 24), HIPIE_OUT_OF_BOUNDS, "elementwise step: %lld pixels", (long long)pixels);
    const int64_t total = pixels * groups;
    float lm1 = 0.f, off = 0.f;
    const FqChannel* tab = nullptr;
    bool rcp = false;
    if (a.out_dtype != HIPIE_F32) {
        HIPIE_REQUIRE(fq_gives_levels(fq) && fq->table.ptr && fq->C == a.C, HIPIE_NOT_IMPLEMENTED,
                      "elementwise step: the FakeQuantize behind it must give consecutive integer levels");
        HIPIE_REQUIRE(a.out_dtype == HIPIE_U8B ? fq->q8_base >= 0 : fq->q8_base + fq->lm1 <= 127.0f, HIPIE_PARAMETER_MISMATCH,
                      "elementwise step: levels do not fit the output type");
        tab = fq->table.as<FqChannel>();
        lm1 = fq->lm1;
        off = a.out_dtype == HIPIE_U8B ? fq->q8_base - 128.0f : fq->q8_base;
        rcp = fq->rcp;
    }
    DeviceGuard g(fq ? fq->device : a.device);
    const dim3 grid(static_cast<uint32_t>(ceil_div(total, kThreads))), block(kThreads);
    const float ig = 1.0f / static_cast<float>(groups), iw = 1.0f / static_cast<float>(a.W), ihw = 1.0f / static_cast<float>(a.H * a.W);
    if (rcp) hipLaunchKernelGGL(eltwise_nhwc_kernel<true>, grid, block, 0, s, a, tab, lm1, off, groups, ig, iw, ihw, total);
    else hipLaunchKernelGGL(eltwise_nhwc_kernel<false>, grid, block, 0, s, a, tab, lm1, off, groups, ig, iw, ihw, total);
    HIPIE_CHECK_HIP(hipGetLastError());
}

extern "C" {

int hipie_fq_create(int device, int64_t channels, int64_t levels, const float* in_low,
                    int64_t n_in_low, const float* in_high, int64_t n_in_high,
                    const float* out_low, int64_t n_out_low, const float* out_high,
                    int64_t n_out_high, hipie_fq** out) {
    return guarded([&] {
        HIPIE_REQUIRE(out && in_low && in_high && out_low && out_high, HIPIE_PARAMETER_MISMATCH,
                      "hipie_fq_create: null argument");
        HIPIE_REQUIRE(channels > 0 && levels >= 2 && levels <= 65536, HIPIE_PARAMETER_MISMATCH,
                      "hipie_fq_create: channels=%lld levels=%lld", (long long)channels,
                      (long long)levels);
        for (int64_t n : {n_in_low, n_in_high, n_out_low, n_out_high})
            HIPIE_REQUIRE(n == 1 || n == channels, HIPIE_PARAMETER_MISMATCH,
                          "hipie_fq_create: a bound has %lld values, expected 1 or %lld",
                          (long long)n, (long long)channels);
        auto fq = std::make_unique<hipie_fq>();
        fq->device = device;
        fq->C = channels;
        fq->levels = levels;
        fq->lm1 = static_cast<float>(static_cast<size_t>(levels - 1));
        fq->host.resize(channels);
        fq->rcp = true;
        fq->clamp_ok = true;
        for (int64_t c = 0; c < channels; ++c) {
            FqChannel& p = fq->host[c];
            p.il = in_low[n_in_low == 1 ? 0 : c];
            p.ih = in_high[n_in_high == 1 ? 0 : c];
            p.ol = out_low[n_out_low == 1 ? 0 : c];
            p.oh = out_high[n_out_high == 1 ? 0 : c];
            p.lo = std::min(p.il, p.ih);
            p.hi = std::max(p.il, p.ih);
            p.d = p.ih - p.il;
            p.r = (p.d != 0.0f && std::isfinite(p.d)) ? fq_rounded_reciprocal(p.d) : 0.0f;
            if (!(p.il < p.ih)) fq->clamp_ok = false;
        }
        fq->rcp = fq_reciprocal_exact_on_all(fq->host.data(), channels, fq->lm1);
        // integer output forms: scalar out range whose op results are out_low + k exactly
        if (n_out_low == 1 && n_out_high == 1 && levels <= 256) {
            const float ol = out_low[0], oh = out_high[0];
            bool ok = ol == std::nearbyintf(ol) && ol >= -128.0f && ol + fq->lm1 <= 255.0f;
            for (int k = 0; ok && k < levels; ++k)
                ok = (static_cast<float>(k) / fq->lm1 * (oh - ol) + ol) == ol + static_cast<float>(k);
            // x > max(il, ih) returns out_high itself, which must be the last level
            ok = ok && oh == ol + fq->lm1;
            fq->q8_ok = ok;
            fq->q8_base = ol;
        }
        // device < 0: host-only object for load-time checks without a GPU; it cannot run
        if (device >= 0) fq->table.upload(device, fq->host.data(), sizeof(FqChannel) * channels);
        *out = fq.release();
    });
}

void hipie_fq_destroy(hipie_fq* fq) { delete fq; }

int hipie_fq_uses_reciprocal(const hipie_fq* fq) { return fq && fq->rcp ? 1 : 0; }

float hipie_fq_host_eval(const hipie_fq* fq, int64_t channel, float x) {
    if (!fq || channel < 0 || channel >= fq->C) return NAN;
    return fq->rcp ? fq_value<true>(fq->host[channel], fq->lm1, x)
                   : fq_value<false>(fq->host[channel], fq->lm1, x);
}

int hipie_fq_run_f32(const hipie_fq* fq, const float* x, float* y, int64_t n, int64_t hw,
                     void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(fq, HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_f32: null handle");
        if (n == 0 || hw == 0) return;  // empty tensor: nothing to do, pointers may be null
        HIPIE_REQUIRE(x && y, HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_f32: null argument");
        HIPIE_REQUIRE(fq->table.ptr, HIPIE_NOT_ALLOCATED, "hipie_fq_run_f32: host-only object");
        HIPIE_REQUIRE(n >= 0 && hw >= 0 && hw < (1ll << 31), HIPIE_PARAMETER_MISMATCH,
                      "hipie_fq_run_f32: n=%lld hw=%lld", (long long)n, (long long)hw);
        const int64_t total = n * fq->C * hw;
        if (total == 0) return;
        DeviceGuard g(fq->device);
        const FqChannel* tab = fq->table.as<FqChannel>();
        const uint32_t C = static_cast<uint32_t>(fq->C);
        const bool vec = hw % 4 == 0 && (reinterpret_cast<uintptr_t>(x) % 16 == 0) &&
                         (reinterpret_cast<uintptr_t>(y) % 16 == 0);
        hipStream_t s = as_stream(stream);
        if (vec) {
            const int64_t n4 = total / 4;
            auto k = fq->rcp ? fq_nchw_f32_vec4<true> : fq_nchw_f32_vec4<false>;
            hipLaunchKernelGGL(k, dim3(grid_for(n4)), dim3(kThreads), 0, s,
                               reinterpret_cast<const float4*>(x), reinterpret_cast<float4*>(y),
                               tab, fq->lm1, n4, static_cast<uint32_t>(hw / 4), C);
        } else {
            auto k = fq->rcp ? fq_nchw_f32<true> : fq_nchw_f32<false>;
            hipLaunchKernelGGL(k, dim3(grid_for(total)), dim3(kThreads), 0, s, x, y, tab, fq->lm1,
                               total, static_cast<uint32_t>(hw), C);
        }
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_fq_run_q8(const hipie_fq* fq, const float* x, void* y, int64_t n, int64_t hw,
                    hipie_dtype out_dtype, hipie_layout out_layout, int64_t c_stride,
                    void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(fq, HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8: null handle");
        if (n == 0 || hw == 0) return;  // empty tensor: nothing to do, pointers may be null
        HIPIE_REQUIRE(x && y, HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8: null argument");
        HIPIE_REQUIRE(fq->table.ptr, HIPIE_NOT_ALLOCATED, "hipie_fq_run_q8: host-only object");
        HIPIE_REQUIRE(n >= 0 && hw >= 0 && hw < (1ll << 31), HIPIE_PARAMETER_MISMATCH,
                      "hipie_fq_run_q8: n=%lld hw=%lld", (long long)n, (long long)hw);
        HIPIE_REQUIRE(fq->q8_ok && fq->clamp_ok, HIPIE_NOT_IMPLEMENTED,
                      "hipie_fq_run_q8: needs input_low < input_high and a scalar output range "
                      "whose %lld values are consecutive integers in [-128, 255]",
                      (long long)fq->levels);
        float off;
        switch (out_dtype) {
        case HIPIE_U8:
            HIPIE_REQUIRE(fq->q8_base >= 0, HIPIE_PARAMETER_MISMATCH,
                          "hipie_fq_run_q8: negative levels do not fit u8");
            off = fq->q8_base;
            break;
        case HIPIE_U8B:
            HIPIE_REQUIRE(fq->q8_base >= 0, HIPIE_PARAMETER_MISMATCH,
                          "hipie_fq_run_q8: negative levels do not fit u8");
            off = fq->q8_base - 128.0f;
            break;
        case HIPIE_I8:
            HIPIE_REQUIRE(fq->q8_base + fq->lm1 <= 127.0f, HIPIE_PARAMETER_MISMATCH,
                          "hipie_fq_run_q8: levels do not fit i8");
            off = fq->q8_base;
            break;
        default:
            fail(HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8: out_dtype %d", (int)out_dtype);
        }
        const int64_t total = n * fq->C * hw;
        if (total == 0) return;
        DeviceGuard g(fq->device);
        const FqChannel* tab = fq->table.as<FqChannel>();
        const uint32_t C = static_cast<uint32_t>(fq->C);
        hipStream_t s = as_stream(stream);
        if (out_layout == HIPIE_NCHW) {
            const bool vec = hw % 4 == 0 && (reinterpret_cast<uintptr_t>(x) % 16 == 0) &&
                             (reinterpret_cast<uintptr_t>(y) % 4 == 0);
            if (vec) {
                const int64_t n4 = total / 4;
                auto k = fq->rcp ? fq_nchw_q8_vec4<true> : fq_nchw_q8_vec4<false>;
                hipLaunchKernelGGL(k, dim3(grid_for(n4)), dim3(kThreads), 0, s,
                                   reinterpret_cast<const float4*>(x),
                                   static_cast<uint32_t*>(y), tab, fq->lm1, off, n4,
                                   static_cast<uint32_t>(hw / 4), C);
            } else {
                auto k = fq->rcp ? fq_nchw_q8_scalar<true> : fq_nchw_q8_scalar<false>;
                hipLaunchKernelGGL(k, dim3(grid_for(total)), dim3(kThreads), 0, s, x,
                                   static_cast<uint8_t*>(y), tab, fq->lm1, off, total,
                                   static_cast<uint32_t>(hw), C);
            }
        } else if (out_layout == HIPIE_NHWC) {
            HIPIE_REQUIRE(c_stride >= fq->C && c_stride % 4 == 0, HIPIE_PARAMETER_MISMATCH,
                          "hipie_fq_run_q8: c_stride=%lld must be a multiple of 4 >= C=%lld",
                          (long long)c_stride, (long long)fq->C);
            HIPIE_REQUIRE(reinterpret_cast<uintptr_t>(y) % 16 == 0 || c_stride % 16 != 0,
                          HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8: output must be 16 B aligned");
            if (hw % 4 == 0 && hw < (1 << 24) && reinterpret_cast<uintptr_t>(x) % 16 == 0 && c_stride >= 128) {
                const uint32_t tiles = static_cast<uint32_t>(ceil_div(hw, 32));
                const int64_t gx = n * tiles;
                HIPIE_REQUIRE(gx < (1ll << 31), HIPIE_OUT_OF_BOUNDS, "hipie_fq_run_q8: grid too large");
                auto kl = fq->rcp ? fq_nchw_to_nhwc_q8_lines<true> : fq_nchw_to_nhwc_q8_lines<false>;
                // a dense [N, HW, c_stride] result: one "row" of HW pixels per image
                hipLaunchKernelGGL(kl, dim3(static_cast<uint32_t>(gx), static_cast<uint32_t>(ceil_div(c_stride, 256))),
                                   dim3(kThreads), 0, s, x, static_cast<uint8_t*>(y), tab, fq->lm1, off,
                                   static_cast<uint32_t>(hw), C, static_cast<uint32_t>(c_stride), tiles,
                                   static_cast<uint32_t>(hw), 1.0f / static_cast<float>(hw), hw * c_stride, hw * c_stride);
                HIPIE_CHECK_HIP(hipGetLastError());
                return;
            }
            if (hw % 4 == 0 && hw < (1 << 24) && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
                const uint32_t tiles = static_cast<uint32_t>(ceil_div(hw, 256));
                const int64_t gx = n * tiles;
                HIPIE_REQUIRE(gx < (1ll << 31), HIPIE_OUT_OF_BOUNDS, "hipie_fq_run_q8: grid too large");
                auto kw = fq->rcp ? fq_nchw_to_nhwc_q8_wide<true> : fq_nchw_to_nhwc_q8_wide<false>;
                // a dense [N, HW, c_stride] result: one "row" of HW pixels per image
                hipLaunchKernelGGL(kw, dim3(static_cast<uint32_t>(gx), static_cast<uint32_t>(ceil_div(c_stride, 64))),
                                   dim3(kThreads), 0, s, x, static_cast<uint8_t*>(y), tab, fq->lm1, off,
                                   static_cast<uint32_t>(hw), C, static_cast<uint32_t>(c_stride), tiles,
                                   static_cast<uint32_t>(hw), 1.0f / static_cast<float>(hw), hw * c_stride, hw * c_stride);
                HIPIE_CHECK_HIP(hipGetLastError());
                return;
            }
            const uint32_t tiles = static_cast<uint32_t>(ceil_div(hw, 64));
            const int64_t gx = n * tiles;
            HIPIE_REQUIRE(gx < (1ll << 31), HIPIE_OUT_OF_BOUNDS, "hipie_fq_run_q8: grid too large");
            auto k = fq->rcp ? fq_nchw_to_nhwc_q8<true> : fq_nchw_to_nhwc_q8<false>;
            hipLaunchKernelGGL(k, dim3(static_cast<uint32_t>(gx),
                                       static_cast<uint32_t>(ceil_div(c_stride, 64))),
                               dim3(kThreads), 0, s, x, static_cast<uint8_t*>(y), tab, fq->lm1, off,
                               static_cast<uint32_t>(hw), C, static_cast<uint32_t>(c_stride), tiles,
                               static_cast<uint32_t>(hw), hw * c_stride, hw * c_stride);
        } else {
            fail(HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8: out_layout %d", (int)out_layout);
        }
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_fq_run_q8_tensor(const hipie_fq* fq, const float* x, const hipie_tensor* out, void* stream) {
    return guarded([&] { run_q8_tensor(fq, x, out, stream); });
}

int hipie_fq_run_q8_tensor_u8(const hipie_fq* fq, const uint8_t* x, const hipie_tensor* out, void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 4 == 0, HIPIE_PARAMETER_MISMATCH, "hipie_fq_run_q8_tensor_u8: unaligned input");
        run_q8_tensor(fq, x, out, stream);
    });
}

}  // extern "C"
