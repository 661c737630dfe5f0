// Bottleneck tail in one launch: a 3 x 3, stride-1, pad-1 convolution whose requantised output tile never leaves the
// compute unit, and the 1 x 1 convolution (with its residual add and FakeQuantize) that consumes it.
//
// A workgroup of four waves owns P output pixels of one image (whole output rows) and ALL CM channels of the 3 x 3
// convolution (CM x P = 16384: 64 x 256, 128 x 128 or 256 x 64, a wave 64 x 64 each).
//  * The input patch under the tile ((rows + 2) x (OW + 2) pixels, every channel, the tensor's own halo where the
//    filter overhangs) is brought into LDS once, so an input byte crosses the L2 -> compute-unit path once instead of
//    once per filter tap; the nine taps read their B fragments from the patch at shifted positions.
//  * Weights stream through a ring of S steps filled by `buffer_load ... lds` (a step = 64 K bytes of every one of
//    the CM weight rows: one tap of one 64-channel slab), first the 3 x 3 convolution's, then - without a break -
//    the 1 x 1 convolution's.
//  * The first epilogue (bias, FakeQuantize) writes the level bytes of the tile into LDS in the layout of an operand
//    tile; the second convolution runs passes of CM output channels over it, each ending in the ordinary epilogue
//    (bias, scale, residual, FakeQuantize) and stores to memory.
// FB == 0: the 3 x 3 convolution alone (its epilogue stores to memory).
// NG == 2 (fused only): eight waves, two groups of four, for layers that give a compute unit one workgroup - a wave alone
// on its SIMD runs the epilogues' dependent vector instructions at half the rate two waves reach together.  The groups
// split the 3 x 3 convolution's input slabs (group 1 hands its partial sums to group 0 through LDS, group 0 requantises
// the tile) and take the 1 x 1 convolution's passes in turn (group g: passes g, g + 2, ...).
// DW: a depthwise 3 x 3 convolution (stride 1 or 2) on the matrix pipe, which such a layer otherwise leaves idle: a
// workgroup takes 256 pixels x the 64 channels of slab blockIdx.y; the weight operand of tap t is the 64 x 64 diagonal
// matrix diag(w[t][c]), built in registers from the lane's two weight bytes per tap (a lane's 16-byte fragment holds
// one diagonal element or none), and only the two diagonal 32 x 32 blocks are multiplied: 36 matrix instructions per
// 64 x 64 outputs where the vector pipe needs 13 or more instructions per output
// (reference::group_convolution, group_convolution.hpp:78-144, with one filter per channel).
//
// Reference semantics, as for every kernel here: reference::convolution<int32_t> on widened inputs
// (ngraph/core/reference/include/ngraph/runtime/reference/convolution.hpp:63-146) for both convolutions, the elementwise
// chains one IEEE f32 operation at a time; the intermediate tensor holds the same bytes the separate kernels would
// have stored.  The CPU plugin fuses two consecutive convolutions into one primitive the same way
// (inference-engine/src/mkldnn_plugin/mkldnn_graph_optimizer.cpp, FuseConvolutionAndDWConvolution).
#include "conv.h"
#include "conv_dispatch.h"

#include <utility>

namespace hipie {
namespace {

constexpr int block_waitcnt_vm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }        // vmcnt <= n
constexpr int block_waitcnt_vm_lds(int n) { return 0x0070 | (n & 15) | ((n >> 4) << 14); }    // and every LDS operation done

// LDS writes of this wave are done and visible, then the workgroup meets; no memory access moves across
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#define HIPIE_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

struct BlockArgs {
    ConvArgs a;          // the 3 x 3 convolution (rows_per_tile, tiles_per_image, patch_w, p_tiles filled)
    ConvArgs b;          // the 1 x 1 convolution behind it (FB != 0)
    int32_t csa;         // 64-byte slabs of the 3 x 3 convolution's input channels
    int32_t ppix;        // patch pixels, padded to a multiple of 16
    int32_t passes;      // output channels of the 1 x 1 convolution / CM
    int32_t p_per_xcd;   // pixel tiles per XCD (neighbouring tiles share halo rows in that XCD's L2), 0: plain order
#ifdef HIPIE_BLOCK_STAMPS
    long long* stamps;   // probe builds only: eight cycle stamps per workgroup
#endif
};

#ifdef HIPIE_BLOCK_STAMPS
long long* g_block_stamps = nullptr;
#define HIPIE_STAMP(i) do { if (g.stamps && tid == 0) g.stamps[blockIdx.x * 8 + (i)] = clock64(); } while (0)
#define HIPIE_STAMP_ADD(i, v) do { if (g.stamps && tid == 0) g.stamps[blockIdx.x * 8 + (i)] = (v); } while (0)
#else
#define HIPIE_STAMP(i)
#define HIPIE_STAMP_ADD(i, v)
#endif

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <uint32_t FA, uint32_t FB, int NWC, bool DEEP, int NG = 1, bool DW = false>
__global__ __launch_bounds__(256 * NG, (DEEP || NG == 2) ? 1 : 2) void conv_block_kernel(const BlockArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr bool kFused = FB != 0;
    static_assert(!DW || (!kFused && NWC == 1 && NG == 1 && !DEEP), "depthwise: one 64-channel slab per workgroup, alone");
    static_assert(NG == 1 || (NG == 2 && kFused && !DEEP), "two wave groups: the fused form, three steps in flight");
    constexpr int NW = 4, NWP = NW / NWC;
    constexpr int CM = NWC * 64, P = NWP * 64;
    constexpr int CSB = CM / 64;                // 64-byte slabs of the intermediate tile
    constexpr int WSTEP = NWC * 4096;           // weight bytes of one step: every wave row block's four fragments
    // steps of weight fragments in flight (registers; a divisor of nine, so that a tap always finds its step in the same
    // registers).  With 256 channels a workgroup is alone on its compute unit and the stream is bound by latency:
    // 36 KB per wave in flight run a step in 350 cycles where 12 KB take 490
    // (DEEP: nine steps and one workgroup per compute unit, for a launch of no more workgroups than compute units; else
    // three and two workgroups, which share the unit when several requests are in flight)
    constexpr int D = DEEP ? 9 : 3;
    constexpr int D0 = 3;                       // of them requested in front of the first barrier
    extern __shared__ __attribute__((aligned(16))) int8_t lds[];
    // (not at LDS offset 0: the epilogue takes LDS pointers whose null value, zero, means "none")
    int8_t* const mid = lds + 256;                                         // [CSB][P][64 bytes]: 16 KB
    float* const sPB0 = reinterpret_cast<float*>(mid + P * CM);            // tables of the 1 x 1 convolution, even passes
    float* const sPA = sPB0 + PT_ROWS * CM;                                // tables of the 3 x 3 convolution; odd passes later
    // (NG == 2: four table buffers - group 0 alternates between the first two, group 1 between the other two)
    int8_t* const patch = reinterpret_cast<int8_t*>(sPA + (NG == 2 ? 3 : 1) * PT_ROWS * CM);   // [csa][ppix][64]; later the stores' staging space
    // NG == 2: group 1's partial sums on their way to group 0, [register quad][wave][lane][16 bytes], behind the patch
    int8_t* const xch = patch + max(g.csa * g.ppix * 64, NG * 16384);

    const ConvArgs& a = g.a;
    const ConvArgs& b = g.b;
    int p_tile = blockIdx.x;
    if (g.p_per_xcd > 0) {
        const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
        p_tile = xcd * g.p_per_xcd + local;
        if (local >= g.p_per_xcd || p_tile >= a.p_tiles) return;           // whole block leaves before any barrier
    }
    const int tid = threadIdx.x, lane = tid & 63;
    HIPIE_STAMP(0);
    const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = NG == 1 ? 0 : wave_all >> 2, wave = wave_all & 3;     // wave group, wave inside it
    const int gtid = tid & 255;
    const int woc = wave % NWC, wpix = wave / NWC;
    const int l32 = lane & 31, h = lane >> 5;

    const int n = p_tile / a.tiles_per_image, ty = p_tile - n * a.tiles_per_image;
    const int OH = a.OHOW / a.OW;
    const int y0 = ty * a.rows_per_tile;                                   // first output row of the tile
    const int rows = min(a.rows_per_tile, OH - y0);
    const int count = rows * a.OW;                                         // pixels of this tile
    const int pix0 = n * a.OHOW + y0 * a.OW;
    const int PW = a.patch_w;
    const int cb = DW ? static_cast<int>(blockIdx.y) * 64 : 0;            // first channel of the workgroup (depthwise: its slab)
    const int cs_ = DW ? a.conv_sh : 1;                                    // stride (the dense form is built for 1)
    // the slabs of the 3 x 3 convolution's input channels this wave group multiplies
    const int c_begin = NG == 1 ? 0 : grp * (g.csa >> 1), c_end = NG == 1 ? g.csa : c_begin + (g.csa >> 1);
    const int NA = 9 * c_end;                                              // one behind the group's last step

    // tables of both convolutions: requested first, stored to LDS behind the operand requests
    StagedParams spa, spb;
    stage_params_load<FA>(a, cb, CM, tid, spa);
    if (kFused) stage_params_load<FB>(b, grp * CM, CM, gtid, spb);          // the group's first pass

    // ---- the patch: 1 KB loads of 16 pixels x 64 bytes, chunk c of pixel q in slot c ^ ((q >> 2) & 3) -------------
    {
        const int8_t* in0 = a.in + (static_cast<int64_t>(n) * a.in_sn + (y0 * cs_ - 1) * a.in_sh - a.in_sw + cb);   // patch pixel (0, 0), in the halo
        const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(in0), 0, 0x7fffffff, 0x00020000);
        const int npix = ((a.rows_per_tile - 1) * cs_ + 3) * PW, ngroups = g.ppix >> 4;
        for (int grp16 = wave_all; grp16 < ngroups; grp16 += NW * NG) {
            const int q_lds = grp16 * 16 + (lane >> 2);
            const int chunk = (lane & 3) ^ ((q_lds >> 2) & 3);
            const int q = min(q_lds, npix - 1);
            int py, px;
            fast_divmod(q, PW, a.inv_patch_w, py, px);
            py = min(py, (rows - 1) * cs_ + 2);                            // rows under a short last tile: never multiplied into a stored pixel
            // (depthwise: a slab that ends behind the pixel's channels re-reads the pixel's first bytes there instead of its
            // neighbour's - those channels meet zero weights, and no byte behind the tensor is touched)
            const int32_t vo = py * a.in_sh + px * a.in_sw + ((DW && cb + chunk * 16 >= a.in_sw) ? -cb : chunk * 16);
            for (int c = 0; c < g.csa; ++c)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rp, HIPIE_LDS_PTR(patch + (c * g.ppix + grp16 * 16) * 64), 16, vo, c * 64, 0, 0);
        }
    }

    // ---- weights: straight from memory into matrix operand registers --------------------------------------------------
    // Packed in the order they are used (pack_fragments in conv.hip): step, wave row block, fragment (ks, ob), lane - a
    // load instruction of a wave is 1 KB of contiguous memory, a step 4 KB per wave.  The 3 x 3 convolution's steps are
    // (slab, tap), tap fastest; D of them are in flight in registers.
    typedef v4i WFrag[4];                                                  // [ks * 2 + ob]
    const int8_t* const wa_lane = a.wgt + (woc * 4096 + lane * 16);
    auto load_wa = [&](int step, WFrag& r) {
        const int8_t* const p = wa_lane + static_cast<int64_t>(step) * WSTEP;
#pragma unroll
        for (int f = 0; f < 4; ++f) r[f] = *reinterpret_cast<const v4i*>(p + f * 1024);
    };
    WFrag wreg[D];
    if constexpr (!DW) {
#pragma unroll
        for (int s0 = 0; s0 < D0; ++s0) load_wa(9 * c_begin + s0, wreg[s0]);   // a group has at least nine steps >= D
    }
    // depthwise: the lane's diagonal elements under every tap ([tap][OCp] bytes).  Row l32 of row block ob is channel
    // 32 ((l32 >> 2) & 1) + 16 ob + 4 (l32 >> 3) + (l32 & 3) of the slab: the order in which the epilogue finds a lane's
    // sixteen results of a block on consecutive channels (packed_row in conv.hip)
    const int dw_c = 32 * ((l32 >> 2) & 1) + 4 * (l32 >> 3) + (l32 & 3);
    uint32_t wdiag[2][9];
    if constexpr (DW) {
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int t = 0; t < 9; ++t)
                wdiag[ob][t] = static_cast<uint8_t>(a.wgt[static_cast<int64_t>(t) * a.OCp + cb + 16 * ob + dw_c]);
    }

    stage_params_store<FA>(a, (lds_float_ptr)sPA, CM, tid, spa);           // (threads tid < CM: of group 0)
    if (kFused) stage_params_store<FB>(b, (lds_float_ptr)(sPB0 + 2 * grp * PT_ROWS * CM), CM, gtid, spb);

    // ---- fragment addresses -----------------------------------------------------------------------------------------
    // pixel rows of 64 bytes, K chunk 2 ks + h in slot (2 ks + h) ^ ((row >> 2) & 3): ks = 1 flips bit 5
    const int mfo = (wpix * 64 + l32) * 64 + ((h ^ ((l32 >> 2) & 3)) << 4);   // rows of the intermediate tile
    int poff[9][2];                                                        // patch position of the lane's two pixels under every tap
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
        const int p = min(wpix * 64 + pb * 32 + l32, count - 1);
        int r, x;
        fast_divmod(p, a.OW, a.inv_OW, r, x);
        const int idx0 = r * cs_ * PW + x * cs_;
#pragma unroll
        for (int kh = 0; kh < 3; ++kh)
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const int idx = idx0 + kh * PW + kw;
                // (depthwise: the half-waves read the chunks 2 h and 2 h + 1 - see the matrix instructions below)
                poff[kh * 3 + kw][pb] = idx * 64 + (((DW ? 2 * h : h) ^ ((idx >> 2) & 3)) << 4);
            }
    }
    typedef v4i BFrag[4];                                                  // [ks * 2 + pb]
    auto read_b_patch = [&](const int8_t* slab, const int (&po)[2], BFrag& bf) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) bf[ks * 2 + pb] = *reinterpret_cast<const v4i*>(slab + (ks ? (po[pb] ^ 32) : po[pb]));
    };
    auto read_b_mid = [&](int c, BFrag& bf) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int8_t* const sb = mid + c * (P * 64) + (ks ? (mfo ^ 32) : mfo);
            bf[ks * 2 + 0] = *reinterpret_cast<const v4i*>(sb);
            bf[ks * 2 + 1] = *reinterpret_cast<const v4i*>(sb + 32 * 64);
        }
    };
    v16i acc[2][2];
    auto mfma8 = [&](const WFrag& af, const BFrag& bf) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
                    acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks * 2 + ob], bf[ks * 2 + pb], acc[ob][pb], 0, 0, 0);
    };

    // this wave's part of the patch has landed and its tables are written (every load: the compiler may have moved
    // table or weight loads behind the patch requests, so no smaller count is safe; the first weights are needed at
    // once anyway); the barrier makes every wave's part visible
    __builtin_amdgcn_s_waitcnt(block_waitcnt_vm_lds(0));
    __builtin_amdgcn_s_barrier();
    if constexpr (!DW) {
#pragma unroll
        for (int s0 = D0; s0 < D; ++s0) load_wa(9 * c_begin + s0, wreg[s0]);
    }
    if (grp == 0) {
        init_acc_lds((lds_cfloat_ptr)sPA, CM, woc * 64 + 32 * h, acc);
    } else {
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ob][pb][r] = 0;
    }
    HIPIE_STAMP(1);

    // ---- the 3 x 3 convolution: no barrier, no LDS traffic but the patch reads ------------------------------------------
    BFrag bset[2];
    if constexpr (DW) {
        // Row block ob holds the channels 16 ob .. 16 ob + 15 and 32 + 16 ob .. 47 + 16 ob, i.e. the 16-byte chunks ob and
        // ob + 2 of a pixel: one matrix instruction per block multiplies exactly those 32 input channels when the lower
        // half-wave reads chunk ob and the upper one chunk ob + 2.  A lane's A fragment then holds its row's diagonal
        // element in byte 4 (l32 >> 3) + (l32 & 3) if its half is the one that carries the row's channel, zeros else.
        const bool has = ((l32 >> 2) & 1) == h;
        const int dsel = l32 >> 3, sh = (l32 & 3) * 8;
        const uint32_t m0_ = has && dsel == 0 ? 0xffffffffu : 0u, m1_ = has && dsel == 1 ? 0xffffffffu : 0u,
                       m2_ = has && dsel == 2 ? 0xffffffffu : 0u, m3_ = has && dsel == 3 ? 0xffffffffu : 0u;
        auto read_b_dw = [&](const int (&po)[2], BFrag& bf) {                // [ob * 2 + pb]
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb) bf[ob * 2 + pb] = *reinterpret_cast<const v4i*>(patch + (ob ? (po[pb] ^ 16) : po[pb]));
        };
        if (wpix * 64 < count) {                                           // (a wave without pixels only meets the others)
            read_b_dw(poff[0], bset[0]);
            static_for<9>([&](auto tap_c) {
                constexpr int T = decltype(tap_c)::value;
                constexpr int cur = T & 1, nxt = cur ^ 1;
                if (T < 8) read_b_dw(poff[T + 1 < 9 ? T + 1 : 0], bset[nxt]);
#pragma unroll
                for (int ob = 0; ob < 2; ++ob) {
                    const uint32_t w = wdiag[ob][T] << sh;
                    v4i af;
                    af.x = static_cast<int>(w & m0_); af.y = static_cast<int>(w & m1_); af.z = static_cast<int>(w & m2_); af.w = static_cast<int>(w & m3_);
#pragma unroll
                    for (int pb = 0; pb < 2; ++pb)
                        acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bset[cur][ob * 2 + pb], acc[ob][pb], 0, 0, 0);
                }
            });
        }
    } else {
    read_b_patch(patch + c_begin * (g.ppix * 64), poff[0], bset[0]);
    for (int c = c_begin; c < c_end; ++c) {
        const int8_t* const slab = patch + c * (g.ppix * 64);
        const int step0 = c * 9;
        static_for<9>([&](auto tap_c) {
            constexpr int T = decltype(tap_c)::value;
            constexpr int cur = T & 1, nxt = cur ^ 1;
            if (T < 8) read_b_patch(slab, poff[(T + 1) % 9], bset[nxt]);
            else if (c + 1 < c_end) read_b_patch(slab + g.ppix * 64, poff[0], bset[nxt]);
            mfma8(wreg[T % D], bset[cur]);
            if (step0 + T + D < NA) load_wa(step0 + T + D, wreg[T % D]);
        });
        // nine taps: the next slab starts on set 0 again
#pragma unroll
        for (int f = 0; f < 4; ++f) bset[0][f] = bset[1][f];
    }
    }
    HIPIE_STAMP(2);

    v16f rres[2][2];
    const int m0 = pix0 + wpix * 64 + l32;
    if (!kFused) {
        __builtin_amdgcn_s_barrier();                                      // every wave is done with the patch: it becomes the stores' staging space
        if (DW && wpix * 64 >= count) return;
        ConvArgs e = a;
        e.M = min(a.M, pix0 + count);                                      // pixels behind the tile's rows belong to the next tile
        EpiAddr ea;
        epilogue_addresses(e, cb + woc * 64 + 32 * h, m0, m0 + 32, 0, ea);
        epilogue<FA, 2, false, true, true, true>(e, acc, cb + woc * 64 + 32 * h, ea.valid, ea.out_off, ea.res_off, rres, (lds_cfloat_ptr)sPA, CM, cb, nullptr,
                                     (lds_float_ptr)patch + wave * 1024);
        HIPIE_STAMP(4);
        return;
    }
    typedef __attribute__((address_space(3))) v4i* lds_v4i_ptr;
    if (NG == 2 && grp == 1) {                                             // partial sums over this group's slabs: to group 0
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    v4i v;
                    v.x = acc[ob][pb][4 * q]; v.y = acc[ob][pb][4 * q + 1]; v.z = acc[ob][pb][4 * q + 2]; v.w = acc[ob][pb][4 * q + 3];
                    *(lds_v4i_ptr)(xch + ((((ob * 2 + pb) * 4 + q) * 4 + wave) * 64 + lane) * 16) = v;
                }
    }

    // ---- the 1 x 1 convolution's weights of a pass: requested while an epilogue runs ----------------------------------
    const int8_t* const wb_lane = b.wgt + (woc * 4096 + lane * 16);
    WFrag wb[CSB];
    auto load_wb = [&](int pass) {
#pragma unroll
        for (int c = 0; c < CSB; ++c) {
            const int8_t* const p = wb_lane + static_cast<int64_t>(pass * CSB + c) * WSTEP;
#pragma unroll
            for (int f = 0; f < 4; ++f) wb[c][f] = *reinterpret_cast<const v4i*>(p + f * 1024);
        }
    };
    load_wb(grp);                                                          // (NG == 1: grp is 0)
    // where the lane's two pixels live in the output and residual tensors (channel 0 of the wave's part of pass 0), and
    // the residual bytes of a pass: requested a pass ahead, like the weights
    ConvArgs e = b;
    e.M = min(b.M, pix0 + count);
    EpiAddr ea;
    epilogue_addresses(e, woc * 64 + 32 * h, m0, m0 + 32, 0, ea);
    constexpr bool kByteRes = (FB & CF_RES) && !(FB & (CF_RES_F32 | CF_RES_GEMM));
    // (requested as raw 16-byte pieces; the zeroing of pieces that do not exist waits until the pass consumes them - done
    // at once it would wait for the loads the moment they are issued)
    uint4 res_raw[2][2];
    uint32_t res_cur[2][8];
    auto res_exists = [&](int pass, int pb, int j) { return ea.valid[pb] && pass * CM + woc * 64 + 32 * h + 16 * j < e.res_sw; };
    auto request_res = [&](int pass) {
#pragma unroll
        for (int pb = 0; pb < 2; ++pb)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                // a lane without an element reads its (clamped, existing) pixel's first 16 bytes: no load hides in a branch
                const int64_t off = res_exists(pass, pb, j) ? ea.res_off[pb] + pass * CM + 16 * j : ea.res_off[pb] - (woc * 64 + 32 * h);
                res_raw[pb][j] = *reinterpret_cast<const uint4*>(static_cast<const int8_t*>(e.res) + off);
            }
    };
    auto take_res = [&](int pass) {
#pragma unroll
        for (int pb = 0; pb < 2; ++pb)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const bool ok = res_exists(pass, pb, j);
                res_cur[pb][4 * j + 0] = ok ? res_raw[pb][j].x : 0u;
                res_cur[pb][4 * j + 1] = ok ? res_raw[pb][j].y : 0u;
                res_cur[pb][4 * j + 2] = ok ? res_raw[pb][j].z : 0u;
                res_cur[pb][4 * j + 3] = ok ? res_raw[pb][j].w : 0u;
            }
    };
    if (kByteRes) request_res(grp);

    if (NG == 2) {
        lds_barrier();                                                     // group 1's sums are in LDS; everyone has left the patch
        if (grp == 0) {
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const v4i v = *(lds_v4i_ptr)(xch + ((((ob * 2 + pb) * 4 + q) * 4 + wave) * 64 + lane) * 16);
                        acc[ob][pb][4 * q] += v.x; acc[ob][pb][4 * q + 1] += v.y; acc[ob][pb][4 * q + 2] += v.z; acc[ob][pb][4 * q + 3] += v.w;
                    }
        }
    }

    // ---- first epilogue: the tile's level bytes -> LDS, in the layout of an operand tile ------------------------------
    if (grp == 0) {
        const bool valid[2] = {true, true};
        const int64_t none[2] = {0, 0};
        epilogue<FA, 2, true, true, true, true>(a, acc, woc * 64 + 32 * h, valid, none, none, rres, (lds_cfloat_ptr)sPA, CM, 0, nullptr,
                              (lds_float_ptr)(mid + woc * (P * 64) + wpix * (64 * 64)));
    }
    HIPIE_STAMP(3);

    // ---- the 1 x 1 convolution: passes of CM output channels over the tile --------------------------------------------
#ifdef HIPIE_BLOCK_STAMPS
    long long t_bar = 0, t_mma = 0, t_epi = 0;
#endif
    for (int it = 0; it * NG < g.passes; ++it) {
        const int pass = it * NG + grp;                                    // (NG == 2: the groups take the passes in turn)
#ifdef HIPIE_BLOCK_STAMPS
        const long long q0 = clock64();
#endif
        // first pass: the tile is complete and the patch is free; later passes: everyone has left the previous epilogue
        // (whose tables the next store below overwrites)
        lds_barrier();
        if (NG == 2 && pass >= g.passes) continue;                         // an odd number of passes: group 1 only meets the others
#ifdef HIPIE_BLOCK_STAMPS
        const long long q1 = clock64();
#endif
        float* const tab_a = NG == 1 ? sPB0 : sPB0 + 2 * grp * PT_ROWS * CM;
        float* const tab_b = NG == 1 ? sPA : tab_a + PT_ROWS * CM;
        lds_float_ptr const tables = (lds_float_ptr)((it & 1) ? tab_b : tab_a);
        lds_float_ptr const tables_next = (lds_float_ptr)((it & 1) ? tab_a : tab_b);
        const bool more = pass + NG < g.passes;
        if (more) stage_params_load<FB>(b, (pass + NG) * CM, CM, gtid, spb);
        init_acc_lds((lds_cfloat_ptr)tables, CM, woc * 64 + 32 * h, acc);
        read_b_mid(0, bset[0]);
        static_for<CSB>([&](auto c_c) {
            constexpr int C = decltype(c_c)::value;
            if (C + 1 < CSB) read_b_mid(C + 1, bset[(C + 1) & 1]);
            mfma8(wb[C], bset[C & 1]);
        });
#ifdef HIPIE_BLOCK_STAMPS
        const long long q2 = clock64();
#endif
        if (kByteRes) take_res(pass);
        if (more) {
            load_wb(pass + NG);
            if (kByteRes) request_res(pass + NG);
            stage_params_store<FB>(b, tables_next, CM, gtid, spb);
        }
        const int oc0 = pass * CM;
        const int64_t oo[2] = {ea.out_off[0] + oc0, ea.out_off[1] + oc0}, ro[2] = {ea.res_off[0] + oc0, ea.res_off[1] + oc0};
#ifdef HIPIE_BLOCK_NOSTORE
        const bool vv[2] = {false, false};
#else
        const bool vv[2] = {ea.valid[0], ea.valid[1]};
#endif
        epilogue<FB, 2, false, true, true, true>(e, acc, oc0 + woc * 64 + 32 * h, vv, oo, ro, rres, (lds_cfloat_ptr)tables, CM, oc0,
                     kByteRes ? res_cur : nullptr, (lds_float_ptr)patch + wave_all * 1024);
#ifdef HIPIE_BLOCK_STAMPS
        const long long q3 = clock64();
        t_bar += q1 - q0; t_mma += q2 - q1; t_epi += q3 - q2;
#endif
    }
    HIPIE_STAMP(4);
    HIPIE_STAMP_ADD(5, t_bar);
    HIPIE_STAMP_ADD(6, t_mma);
    HIPIE_STAMP_ADD(7, t_epi);
#endif
}

// ng = 2: the layout of the form with two wave groups (four table buffers, staging space for eight waves, 64 KB for
// the partial sums that change groups)
size_t block_lds_bytes(int nwc, int csa, int ppix, int ng) {
    const size_t cm = static_cast<size_t>(nwc) * 64;
    return 256 + 16384 + 2 * ng * PT_ROWS * cm * 4 + std::max<size_t>(static_cast<size_t>(csa) * ppix * 64, ng * 16384) +
           (ng == 2 ? 65536 : 0);
}

template <uint32_t FA, uint32_t FB, int NWC, bool DEEP, int NG = 1>
void launch_block_instance(const BlockArgs& g, size_t lds, hipStream_t s) {
    static bool attr_set = false;
    if (!attr_set) {
        HIPIE_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_block_kernel<FA, FB, NWC, DEEP, NG>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        attr_set = true;
    }
    const dim3 grid(g.p_per_xcd > 0 ? 8 * g.p_per_xcd : g.a.p_tiles), block(256 * NG);
    hipLaunchKernelGGL((conv_block_kernel<FA, FB, NWC, DEEP, NG>), grid, block, lds, s, g);
}

// form: 0 three steps of weights in flight and two workgroups per compute unit, 1 nine steps and one workgroup,
// 2 (fused only) eight waves in two groups
template <uint32_t FA, uint32_t FB>
void launch_block_shape(const BlockArgs& g, int nwc, int form, size_t lds, hipStream_t s) {
    if constexpr (FB != 0) {
        if (form == 2) {
            switch (nwc) {
            case 2: launch_block_instance<FA, FB, 2, false, 2>(g, lds, s); return;
            case 4: launch_block_instance<FA, FB, 4, false, 2>(g, lds, s); return;
            default: fail(HIPIE_GENERAL_ERROR, "block kernel: two wave groups with %d channel waves", nwc);
            }
        }
    }
    switch (nwc * 2 + (form == 1 ? 1 : 0)) {
    case 2: case 3: launch_block_instance<FA, FB, 1, false>(g, lds, s); break;   // 64 channels: nine steps in all
    case 4: launch_block_instance<FA, FB, 2, false>(g, lds, s); break;
    case 5: launch_block_instance<FA, FB, 2, true>(g, lds, s); break;
    case 8: launch_block_instance<FA, FB, 4, false>(g, lds, s); break;
    case 9: launch_block_instance<FA, FB, 4, true>(g, lds, s); break;
    default: fail(HIPIE_GENERAL_ERROR, "block kernel: %d channel waves", nwc);
    }
}

}  // namespace

// the epilogues the kernel is instantiated for: bias + 256-level FakeQuantize from 0 behind the 3 x 3 convolution,
// bias, scale, byte residual with a multiplier and the same FakeQuantize behind the 1 x 1 convolution; each with the
// division in its two-operation form, as reciprocal with corrections, or as a division
constexpr uint32_t kBlockFirst[3] = {E_PLAIN0, E_PLAIN0 & ~CF_FQ_DIV2, E_PLAIN0 & ~(CF_FQ_DIV2 | CF_FQ_RCP)};
constexpr uint32_t kBlockSecond[3] = {E_RESU8, E_RESU8 & ~CF_FQ_DIV2, E_RESU8 & ~(CF_FQ_DIV2 | CF_FQ_RCP)};

static int block_index(const uint32_t (&table)[3], uint32_t flags) {
    for (int i = 0; i < 3; ++i)
        if ((flags & ~CF_OUT_XOR) == table[i]) return i;
    return -1;
}

bool block_epilogues_fit(uint32_t flags_a, bool fused, uint32_t flags_b) {
    return block_index(kBlockFirst, flags_a) >= 0 && (!fused || block_index(kBlockSecond, flags_b) >= 0);
}

BlockGeometry block_geometry(int oc_a, int ic_a, int oh, int ow) {
    BlockGeometry r{};
    if (!(oc_a == 64 || oc_a == 128 || oc_a == 256) || ic_a % 64 != 0 || ow < 1 || oh < 1) return r;
    r.nwc = oc_a / 64;
    const int P = 16384 / oc_a;
    if (ow > P) return r;
    r.rows = std::min(P / ow, oh);
    r.tiles_per_image = static_cast<int>(ceil_div(oh, r.rows));
    r.patch_w = ow + 2;
    r.csa = ic_a / 64;
    r.ppix = static_cast<int>(round_up(static_cast<int64_t>(r.rows + 2) * r.patch_w, 16));
    r.lds = block_lds_bytes(r.nwc, r.csa, r.ppix, 1);
    r.ok = r.lds <= 160 * 1024;
    r.lds2 = block_lds_bytes(r.nwc, r.csa, r.ppix, 2);
    r.ok2 = r.ok && r.nwc >= 2 && r.csa % 2 == 0 && r.lds2 <= 160 * 1024;   // (64 channels: the four waves already split the pixels)
    return r;
}

void launch_block(const ConvArgs& a, const ConvArgs* b, const BlockGeometry& geo, int images, int form, hipStream_t s) {
    BlockArgs g{};
    g.a = a;
    g.a.rows_per_tile = geo.rows;
    g.a.tiles_per_image = geo.tiles_per_image;
    g.a.patch_w = geo.patch_w;
    g.a.inv_patch_w = 1.0f / static_cast<float>(geo.patch_w);
    g.a.p_tiles = images * geo.tiles_per_image;
    g.csa = geo.csa;
    g.ppix = geo.ppix;
    g.p_per_xcd = g.a.p_tiles >= 16 ? static_cast<int32_t>(ceil_div(g.a.p_tiles, 8)) : 0;
#ifdef HIPIE_BLOCK_STAMPS
    g.stamps = g_block_stamps;
#endif
    const int cm = geo.nwc * 64;
    if (b) {
        g.b = *b;
        g.passes = b->OC / cm;
        HIPIE_REQUIRE(b->OC % cm == 0 && 9 * geo.csa + g.passes * geo.nwc < (1 << 20), HIPIE_GENERAL_ERROR, "block kernel: channel counts");
    }
    HIPIE_REQUIRE(form != 2 || (b && geo.ok2 && g.passes >= 2), HIPIE_NOT_IMPLEMENTED,
                  "block kernel: the form with two wave groups takes a fused pair with an even number of input slabs, 128 or 256 "
                  "channels between the layers and at least two passes");
    const size_t lds = form == 2 ? geo.lds2 : geo.lds;
    const int ia = block_index(kBlockFirst, a.flags), ib = b ? block_index(kBlockSecond, b->flags) : 3;
    HIPIE_REQUIRE(ia >= 0 && ib >= 0, HIPIE_GENERAL_ERROR, "block kernel: no instance for epilogues %#x / %#x", a.flags, b ? b->flags : 0u);
#define HIPIE_BLOCK_CASE(IA, IB, FB) \
    case (IA) * 4 + (IB): launch_block_shape<kBlockFirst[IA], FB>(g, geo.nwc, form, lds, s); break;
    switch (ia * 4 + ib) {
        HIPIE_BLOCK_CASE(0, 0, kBlockSecond[0]) HIPIE_BLOCK_CASE(0, 1, kBlockSecond[1]) HIPIE_BLOCK_CASE(0, 2, kBlockSecond[2]) HIPIE_BLOCK_CASE(0, 3, 0u)
        HIPIE_BLOCK_CASE(1, 0, kBlockSecond[0]) HIPIE_BLOCK_CASE(1, 1, kBlockSecond[1]) HIPIE_BLOCK_CASE(1, 2, kBlockSecond[2]) HIPIE_BLOCK_CASE(1, 3, 0u)
        HIPIE_BLOCK_CASE(2, 0, kBlockSecond[0]) HIPIE_BLOCK_CASE(2, 1, kBlockSecond[1]) HIPIE_BLOCK_CASE(2, 2, kBlockSecond[2]) HIPIE_BLOCK_CASE(2, 3, 0u)
    }
#undef HIPIE_BLOCK_CASE
}

// ---- depthwise 3 x 3 on the matrix pipe -------------------------------------------------------------------------------
constexpr uint32_t kBlockDepthwise[3] = {E_PLAIN0, E_SCALEFQ0, E_CLAMPFQ};

bool block_dw_epilogue_fits(uint32_t flags) { return block_index(kBlockDepthwise, flags) >= 0; }

BlockGeometry block_dw_geometry(int oh, int ow, int stride) {
    BlockGeometry r{};
    if (ow < 1 || oh < 1 || ow > 256 || (stride != 1 && stride != 2)) return r;
    r.nwc = 1;
    r.rows = std::min(256 / ow, oh);
    r.tiles_per_image = static_cast<int>(ceil_div(oh, r.rows));
    r.patch_w = (ow - 1) * stride + 3;
    r.csa = 1;
    r.ppix = static_cast<int>(round_up(static_cast<int64_t>((r.rows - 1) * stride + 3) * r.patch_w, 16));
    r.lds = block_lds_bytes(1, 1, r.ppix, 1);
    r.ok = r.lds <= 160 * 1024;
    return r;
}

template <uint32_t FA>
static void launch_block_dw_instance(const BlockArgs& g, int slabs, size_t lds, hipStream_t s) {
    static bool attr_set = false;
    if (!attr_set) {
        HIPIE_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_block_kernel<FA, 0u, 1, false, 1, true>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        attr_set = true;
    }
    const dim3 grid(g.p_per_xcd > 0 ? 8 * g.p_per_xcd : g.a.p_tiles, slabs), block(256);
    hipLaunchKernelGGL((conv_block_kernel<FA, 0u, 1, false, 1, true>), grid, block, lds, s, g);
}

void launch_block_dw(const ConvArgs& a, const BlockGeometry& geo, int images, hipStream_t s) {
    BlockArgs g{};
    g.a = a;
    g.a.rows_per_tile = geo.rows;
    g.a.tiles_per_image = geo.tiles_per_image;
    g.a.patch_w = geo.patch_w;
    g.a.inv_patch_w = 1.0f / static_cast<float>(geo.patch_w);
    g.a.p_tiles = images * geo.tiles_per_image;
    g.csa = 1;
    g.ppix = geo.ppix;
    g.p_per_xcd = g.a.p_tiles >= 16 ? static_cast<int32_t>(ceil_div(g.a.p_tiles, 8)) : 0;
#ifdef HIPIE_BLOCK_STAMPS
    g.stamps = nullptr;
#endif
    const int slabs = static_cast<int>(ceil_div(a.OC, 64));
    HIPIE_REQUIRE(slabs >= 1 && slabs <= 65535 && a.OCp >= slabs * 64, HIPIE_GENERAL_ERROR, "depthwise block kernel: %d channels", a.OC);
    switch (block_index(kBlockDepthwise, a.flags)) {
    case 0: launch_block_dw_instance<kBlockDepthwise[0]>(g, slabs, geo.lds, s); break;
    case 1: launch_block_dw_instance<kBlockDepthwise[1]>(g, slabs, geo.lds, s); break;
    case 2: launch_block_dw_instance<kBlockDepthwise[2]>(g, slabs, geo.lds, s); break;
    default: fail(HIPIE_GENERAL_ERROR, "depthwise block kernel: no instance for epilogue %#x", a.flags);
    }
}

#ifdef HIPIE_BLOCK_STAMPS
extern "C" void hipie_debug_block_stamps(long long* p) { g_block_stamps = p; }
#endif

}  // namespace hipie
