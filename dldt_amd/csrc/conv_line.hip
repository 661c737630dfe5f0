// Implicit-GEMM convolution on int8 MFMA whose K loop moves whole cache lines: a K step is RB = 128
// bytes of every operand row (64 where a pixel holds 64 channels), brought into an LDS ring by buffer
// loads that write LDS directly.
//
// Why this form (measured on the device with operand-load-only and full-loop probes):
//  * An L2 channel serves one request per clock whatever its size.  With 64-byte K steps every operand
//    row is a 64-byte request, half a 128-byte line, and 256 compute units together get 29 B/clk each;
//    with 128-byte steps they get 46 B/clk.  A 128 x 128 tile needs 64 B/clk at the matrix peak, so the
//    operand stream, not the matrix pipe, is what a K loop of such tiles runs at.
//  * `global_load ... lds` is a FLAT-encoded instruction to the compiler: with one in flight it no longer
//    counts LDS operations in order and puts `s_waitcnt lgkmcnt(0)` in front of every group of matrix
//    instructions, which exposes the whole LDS latency once per 32 bytes of K.  The MUBUF form
//    (`buffer_load ... lds`) keeps the in-order counting (`lgkmcnt(4)`: wait for the older fragment set
//    only), takes the K step's offset as a scalar and needs no address arithmetic per load.
//  * KS = 2: eight waves; both groups of four read the same ring, group g multiplies the 32-byte
//    sub-steps [2 g, 2 g + 2) of every step and group 1 hands its partial sums over through LDS at the
//    end.  Two waves per SIMD fill each other's waits (barrier, LDS latency) without more operand traffic.
// Reference semantics as for the other kernels: reference::convolution<int32_t> on widened inputs
// (ngraph/core/reference/include/ngraph/runtime/reference/convolution.hpp:63-146); integer sums do not
// depend on the order, so every variant gives the same bits.
#include "conv.h"
#include "conv_dispatch.h"

namespace hipie {
namespace {

constexpr int line_waitcnt_vm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

#define HIPIE_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

template <uint32_t F, int KS, int S, int RB>
__global__ __launch_bounds__(256 * KS, RB == 64 ? 2 : 1) void conv_line_kernel(const ConvArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int NW = 4 * KS, NT = NW * 64;
    constexpr int BOC = 128, BPIX = 128;
    constexpr int CH = RB / 16;                        // 16-byte chunks of an LDS row
    constexpr int RPG = 1024 / RB;                     // rows of one 1 KB load
    constexpr int AG = BOC / RPG / NW, BG = BPIX / RPG / NW;
    constexpr int LPS = AG + BG;                       // loads per wave per K step
    constexpr int STAGE = (BOC + BPIX) * RB;
    constexpr int NSUB = RB / 32 / KS;                 // 32-byte sub-steps one wave group multiplies
    static_assert(NSUB >= 2 && NSUB % 2 == 0, "the two fragment register sets alternate with a fixed phase");
    static_assert((S - 1) * LPS < 64 && S >= 3, "vmcnt is a 6-bit counter; the ring keeps a step between reader and writer");
    extern __shared__ __attribute__((aligned(16))) int8_t ring[];

    int t_tile, p_tile;
    if (a.p_per_xcd > 0) {
        const int xcd = blockIdx.x & 7, y = blockIdx.x >> 3;
        int p_local;
        split_tile_index(a, y, p_local, t_tile);
        p_tile = xcd * a.p_per_xcd + p_local;
        if (p_local >= a.p_per_xcd || p_tile >= a.p_tiles) return;   // whole block leaves before any barrier
    } else {
        split_tile_index(a, blockIdx.x, p_tile, t_tile);
    }
    const int pix0 = p_tile * BPIX, oc0 = t_tile * BOC;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: LDS bases of the loads stay scalar
    const int grp = KS == 1 ? 0 : wave_all >> 2, wave = wave_all & 3;
    const int woc = wave & 1, wpix = wave >> 1;
    const int l32 = lane & 31, h = lane >> 5;
    const int oc_lane = oc0 + woc * 64 + 32 * h;
    // chunk c of row r is kept in slot c ^ swz(r): sixteen consecutive rows of one chunk fall on sixteen
    // different 16-byte bank groups, for the fragment reads and for the 1 KB rows a load writes
    auto swz = [](int row) { return RB == 64 ? ((row >> 2) & 3) : ((row >> 1) & 7); };

    float* const sP = reinterpret_cast<float*>(ring + S * STAGE);
    stage_params<F>(a, oc0, (lds_float_ptr)sP, BOC, tid, NT);
    // byte offset of every K step relative to the window origin: a step never straddles two filter taps
    // (the channel stride is a multiple of RB), so its first 16-byte piece places all of it
    int32_t* const kt = reinterpret_cast<int32_t*>(ring + S * STAGE + PT_ROWS * BOC * 4);
    const int nk = a.Kp / RB;
    for (int i = tid; i < nk; i += NT) kt[i] = a.koff[i * CH];

    // load roles: wave w fetches the 1 KB groups [w AG, (w + 1) AG) of the weight rows and the same of the pixels
    const int dma_row = lane / CH, dma_slot = lane % CH;
    int32_t a_vo[AG], b_vo[BG];
#pragma unroll
    for (int i = 0; i < AG; ++i) {
        const int row = (wave_all * AG + i) * RPG + dma_row;
        const int chunk = dma_slot ^ swz(row);
        a_vo[i] = min(oc0 + row, a.wgt_rows - 1) * a.wgt_ld + chunk * 16;
    }
#pragma unroll
    for (int i = 0; i < BG; ++i) {
        const int row = (wave_all * BG + i) * RPG + dma_row;
        const int chunk = dma_slot ^ swz(row);
        int m = pix0 + row;
        m = m < a.M ? m : a.M - 1;
        b_vo[i] = window_offset(a, m, a.in_sn, a.in_sh, a.in_sw, a.conv_sh, a.conv_sw, a.flat_in != 0) + chunk * 16;
    }
    // raw buffers (no stride, no swizzle) that start at the lowest byte any lane reads: offsets stay non-negative
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.wgt), 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.in + a.in_origin), 0, 0x7fffffff, 0x00020000);
    auto issue = [&](int slot, int k, int32_t off_b) {
        int8_t* const sa = ring + slot * STAGE;
        int8_t* const sb = sa + BOC * RB;
#pragma unroll
        for (int i = 0; i < AG; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, HIPIE_LDS_PTR(sa + (wave_all * AG + i) * 1024), 16, a_vo[i], k * RB, 0, 0);
#pragma unroll
        for (int i = 0; i < BG; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, HIPIE_LDS_PTR(sb + (wave_all * BG + i) * 1024), 16, b_vo[i], off_b, 0, 0);
    };
    auto step_offset = [&](int k) { return __builtin_amdgcn_readfirstlane(kt[k]); };

    // fragment of sub-step j: rows l32 (+ 32), logical chunk 2 (grp NSUB + j) + h
    int frag_off[NSUB];
#pragma unroll
    for (int j = 0; j < NSUB; ++j) frag_off[j] = l32 * RB + (((2 * (grp * NSUB + j) + h) ^ swz(l32)) * 16);
    auto read_frags = [&](int slot, int j, v4i (&af)[2], v4i (&bf)[2]) {
        const int8_t* const sa = ring + slot * STAGE + (woc * 64) * RB;
        const int8_t* const sb = ring + slot * STAGE + BOC * RB + (wpix * 64) * RB;
#pragma unroll
        for (int i = 0; i < 2; ++i) af[i] = *reinterpret_cast<const v4i*>(sa + i * 32 * RB + frag_off[j]);
#pragma unroll
        for (int i = 0; i < 2; ++i) bf[i] = *reinterpret_cast<const v4i*>(sb + i * 32 * RB + frag_off[j]);
    };
    v16i acc[2][2];
    auto mfma4 = [&](const v4i (&af)[2], const v4i (&bf)[2]) {
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
                acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ob], bf[pb], acc[ob][pb], 0, 0, 0);
    };

    __syncthreads();                                   // tables and K offsets are in LDS
    if (grp == 0) {
        init_acc_lds((lds_cfloat_ptr)sP, BOC, oc_lane - oc0, acc);
    } else {
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ob][pb][r] = 0;
    }

    // Ring of S steps.  Iteration k multiplies step k one sub-step at a time, reading the fragments of the
    // next sub-step before the matrix instructions of the current one; behind the first group of matrix
    // instructions a wave waits for its own loads of step k + 1, the barrier makes every wave's part of
    // that step visible and proves that nobody reads step k - 1 any more, and step k + S - 1 is requested
    // into that slot.  The fences keep the compiler from interleaving reads and matrix instructions (the
    // wait in front of a group would then cover the reads just issued).
    const int ahead = min(S - 1, nk);
    for (int s0 = 0; s0 < ahead; ++s0) issue(s0, s0, step_offset(s0));
    if (ahead == S - 1) __builtin_amdgcn_s_waitcnt(line_waitcnt_vm((S - 2) * LPS));
    else __builtin_amdgcn_s_waitcnt(line_waitcnt_vm(0));
    __builtin_amdgcn_s_barrier();
    int rd = 0, wr = ahead == S - 1 ? S - 1 : 0;
    v4i fa[2][2], fb[2][2];
    read_frags(0, 0, fa[0], fb[0]);
    auto step = [&](int k, auto requests, auto last_step) {
        constexpr bool kRequests = decltype(requests)::value;   // step k + S - 1 exists and is requested here
        constexpr bool kLast = decltype(last_step)::value;      // k == nk - 1: no later step to wait for or read
        int32_t off_req = 0;
        if (kRequests) off_req = step_offset(k + S - 1);
        const int nrd = rd + 1 == S ? 0 : rd + 1;
#pragma unroll
        for (int j = 0; j < NSUB; ++j) {
            __builtin_amdgcn_sched_barrier(0);
            if (j + 1 < NSUB) read_frags(rd, j + 1, fa[(j + 1) & 1], fb[(j + 1) & 1]);
            else if (!kLast) read_frags(nrd, 0, fa[0], fb[0]);
            __builtin_amdgcn_sched_barrier(0);
            mfma4(fa[j & 1], fb[j & 1]);
            if (j == 0 && !kLast) {
                __builtin_amdgcn_sched_barrier(0);
                // outstanding before the wait: steps k + 1 .. k + S - 2 (all of them in the last iterations)
                if (kRequests) __builtin_amdgcn_s_waitcnt(line_waitcnt_vm((S - 3) * LPS));
                else __builtin_amdgcn_s_waitcnt(line_waitcnt_vm(0));
                __builtin_amdgcn_s_barrier();
                if (kRequests) {
                    issue(wr, k + S - 1, off_req);
                    wr = wr + 1 == S ? 0 : wr + 1;
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        rd = nrd;
    };
    int k = 0;
    for (; k + S - 1 < nk; ++k) step(k, std::true_type{}, std::false_type{});
    for (; k + 1 < nk; ++k) step(k, std::false_type{}, std::false_type{});
    step(k, std::false_type{}, std::true_type{});
    __builtin_amdgcn_s_barrier();                      // every wave is done reading: the ring becomes scratch space

    if (KS == 2) {
        // partial sums of group 1 -> LDS (register r of thread t at dword r * 256 + t), added by group 0
        int32_t* const red = reinterpret_cast<int32_t*>(ring);
        const int t = tid & 255;
        if (grp == 1) {
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) red[((ob * 2 + pb) * 16 + r) * 256 + t] = acc[ob][pb][r];
        }
        __syncthreads();
        if (grp == 1) return;
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ob][pb][r] += red[((ob * 2 + pb) * 16 + r) * 256 + t];
    }
    // stores leave through 8 KB of LDS per wave, behind the 64 KB of partial sums where there are any
    static_assert(S * STAGE >= (KS == 2 ? 65536 : 0) + 4 * 8192, "staging space inside the ring");
    lds_float_ptr stage = (lds_float_ptr)(ring + (KS == 2 ? 65536 : 0)) + wave * 2048;
    v16f rres[2][2];
    const int m0 = pix0 + wpix * 64 + l32;
    run_epilogue<F, true, true>(a, acc, oc_lane, m0, m0 + 32, 0, rres, (lds_cfloat_ptr)sP, BOC, oc0, stage);   // both in (dynamic) LDS
#endif
}

template <int KS, int S, int RB>
void launch_line_shape(const ConvArgs& a, hipStream_t s) {
    const dim3 grid(a.p_per_xcd > 0 ? 8 * a.p_per_xcd * a.t_tiles : a.p_tiles * a.t_tiles), block(256 * KS);
    const size_t lds = static_cast<size_t>(S) * 256 * RB + PT_ROWS * 128 * 4 + 4 * static_cast<size_t>(a.Kp / RB) + 16;
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_LINE(FLAGS, ...)                                                                        \
    do {                                                                                                     \
        if constexpr ((FLAGS) != kDyn && ((FLAGS) & CF_RES_GEMM)) break;   /* the second GEMM exists in the tiled kernel only */ \
        else {                                                                                               \
            static bool attr_set = false;                                                                    \
            if (!attr_set) {                                                                                 \
                HIPIE_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_line_kernel<FLAGS, KS, S, RB>), \
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); \
                attr_set = true;                                                                             \
            }                                                                                                \
            hipLaunchKernelGGL((conv_line_kernel<FLAGS, KS, S, RB>), grid, block, lds, s, a);                \
        }                                                                                                    \
    } while (0)
    HIPIE_FOR_EACH_EPILOGUE(HIPIE_LAUNCH_LINE, 0)
#undef HIPIE_LAUNCH_LINE
}

}  // namespace

int line_row_bytes(int shape) { return shape == 4 ? 64 : 128; }

void launch_line(const ConvArgs& a, int shape, hipStream_t s) {
    switch (shape) {
    case 0: launch_line_shape<1, 3, 128>(a, s); break;
    case 1: launch_line_shape<2, 3, 128>(a, s); break;
    case 2: launch_line_shape<1, 4, 128>(a, s); break;
    case 3: launch_line_shape<2, 4, 128>(a, s); break;
    case 4: launch_line_shape<1, 4, 64>(a, s); break;
    default: fail(HIPIE_GENERAL_ERROR, "line kernel: shape %d", shape);
    }
}

}  // namespace hipie
