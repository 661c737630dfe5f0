// Convolution / MatMul on int8 MFMA: kernel instantiations, load-time packing, launcher.
#include "conv.h"
#include "div2.h"
#include "conv_epilogue.h"
#include "conv_dispatch.h"

#include <cmath>
#include <map>
#include <memory>
#include <mutex>

namespace hipie {

namespace {

constexpr int kRow = 64;  // LDS rows of the tiled kernels: 64 K-bytes, chunk c of row r in slot c ^ ((r >> 2) & 3)

// ------------------------------------------------------------------------------------------------
// LDS-tiled kernel
// PAIR: the operands of two 64-byte K steps are requested together, eight lanes per row, so that a row's
// 128-byte cache line crosses the L2 -> L1 path once instead of once per step (with four workgroups on a
// compute unit the lines of one step, 128 KB, do not survive in the 32 KB L1 until the next step asks
// for their other half: the operand loads alone run 1.4 times faster this way).  The two LDS buffers
// then hold the two steps of a pair instead of alternating.
// PIXC: one integer per output row (ConvArgs::pix_corr) is added to the row's accumulators in front of the epilogue
// (MatMul between activations with a u8 right operand).  A template constant: as a run-time branch its registers
// pushed the 128-register instances of every convolution into spills.
template <int WOC, int WPIX, uint32_t F, bool PAIR = false, bool PIXC = false>
__global__ __launch_bounds__(WOC* WPIX * 64, (WOC * WPIX >= 4 && !(F != kDyn && (F & CF_RES_GEMM))) ? ((F == kDyn || PAIR || PIXC) ? 3 : 4) : 2) void conv_tiled_kernel(const ConvArgs a) {
    constexpr int NT = WOC * WPIX * 64;
    constexpr int BOC = WOC * 64, BPIX = WPIX * 64;
    constexpr int A_PIECES = BOC * 4 / NT, B_PIECES = BPIX * 4 / NT;
    // PAIR: eight neighbouring lanes of a store instruction write one row of both buffers (the two steps
    // of a pair).  The second buffer sits 128 bytes further and holds row r at position r ^ 1, so those
    // two 64-byte pieces, and the four of sixteen lanes, fall on different LDS banks
    constexpr int kBufPad = PAIR ? 128 : 0;
    __shared__ __attribute__((aligned(256))) int8_t sA[2][BOC * kRow + kBufPad];
    __shared__ __attribute__((aligned(256))) int8_t sB[2][BPIX * kRow + kBufPad];
    __shared__ __attribute__((aligned(16))) float sP[PT_ROWS * BOC];

    // block -> (pixel tile, channel tile): consecutive pixel tiles stay on one XCD
    int t_tile, p_tile;
    if (a.p_per_xcd > 0) {
        const int xcd = blockIdx.x & 7, y = blockIdx.x >> 3;
        int p_local;
        split_tile_index(a, y, p_local, t_tile);
        p_tile = xcd * a.p_per_xcd + p_local;
        if (p_local >= a.p_per_xcd || p_tile >= a.p_tiles) return;  // whole block leaves before any barrier
    } else {   // few pixel tiles: plain order, consecutive workgroups land on consecutive XCDs
        split_tile_index(a, blockIdx.x, p_tile, t_tile);
    }
    const int pix0 = p_tile * BPIX, oc0 = t_tile * BOC;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int woc = wave % WOC, wpix = wave / WOC;
    const int l32 = lane & 31, h = lane >> 5;
    const int chunk = tid & 3;
    const PiecePick pick(chunk);
    // XOR swizzle instead of row padding: the thread that stages (row, chunk) and the lanes that read
    // fragments (rows l32 + 32 i, chunk 2 ks + h) agree on slot = chunk ^ ((row >> 2) & 3); rows that
    // differ by a multiple of 16 share the swizzle, so (tid + i NT) >> 2 and l32 + 32 i need one value each
    const int lds_slot = (chunk ^ ((tid >> 4) & 3)) * 16;
    const int frag_slot[2] = {((0 + h) ^ ((l32 >> 2) & 3)) * 16, ((2 + h) ^ ((l32 >> 2) & 3)) * 16};

    const int batch = blockIdx.y;
    static_assert(BOC <= NT, "one table element per thread");
    StagedParams staged;
    // (a batched MatMul with a u8 left operand has one row of accumulator corrections per batch element)
    stage_params_load<F>(a, oc0, BOC, tid, staged, static_cast<int64_t>(batch) * a.batch_corr);   // awaited only after the first K step has been requested
    const int a_row[2] = {woc * 64 + l32, woc * 64 + 32 + l32};
    const int b_row[2] = {wpix * 64 + l32, wpix * 64 + 32 + l32};
    const int oc_lane = oc0 + woc * 64 + 32 * h;

    // one implicit GEMM over an operand set (activation tensor, packed weights, K-offset table)
    auto gemm = [&](const int8_t* in_base, int in_sn, int in_sh, int in_sw, int csh, int csw, int origin,
                    const int8_t* wgt_base, int wgt_ld, int wgt_rows, bool wgt_plain, const int32_t* koff, int nk,
                    v16i (&acc)[2][2], bool first, bool acc_from_lds, bool flat, bool linear) {
        int32_t b_base[B_PIECES];
        uint32_t a_off[A_PIECES];                          // unsigned: added to the uniform base by the load itself
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i) {
            int m = pix0 + ((tid + i * NT) >> 2);
            m = m < a.M ? m : a.M - 1;
            b_base[i] = window_offset(a, m, in_sn, in_sh, in_sw, csh, csw, flat) + origin;
        }
#pragma unroll
        for (int i = 0; i < A_PIECES; ++i) {
            int row = (tid + i * NT) >> 2;                 // row of the LDS tile
            if (wgt_plain) {                               // natural row order in memory: LDS row 32*ob + j
                const int j = row & 31;                    // must hold channel 32*((j>>2)&1) + 16*ob + 4*(j>>3) + (j&3)
                row = (row & ~63) + 32 * ((j >> 2) & 1) + 16 * ((row >> 5) & 1) + 4 * (j >> 3) + (j & 3);
            }
            row = min(oc0 + row, wgt_rows - 1);
            a_off[i] = static_cast<uint32_t>(row) * static_cast<uint32_t>(wgt_ld) + chunk * 16;
        }
        auto mfma_step = [&](int buf) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                v4i af[2], bf[2];
#pragma unroll
                for (int ob = 0; ob < 2; ++ob)
                    af[ob] = *reinterpret_cast<const v4i*>(&sA[buf][(a_row[ob] ^ (PAIR ? buf : 0)) * kRow + frag_slot[ks]]);
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
                    bf[pb] = *reinterpret_cast<const v4i*>(&sB[buf][(b_row[pb] ^ (PAIR ? buf : 0)) * kRow + frag_slot[ks]]);
#pragma unroll
                for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                    for (int pb = 0; pb < 2; ++pb)
                        acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ob], bf[pb], acc[ob][pb], 0, 0, 0);
            }
        };
        if constexpr (PAIR) {
            static_assert(NT == 256, "eight lanes per row, 32 rows per load instruction");
            constexpr int RPI = NT / 8, A_P2 = BOC / RPI, B_P2 = BPIX / RPI;
            const int sub = (tid >> 2) & 1, row0 = tid >> 3;          // chunk tid & 3 of step 2 j + sub, rows row0 + i RPI
            const int slot2 = (chunk ^ ((tid >> 5) & 3)) * 16;        // RPI is a multiple of 16: one swizzle per thread
            int32_t b_base2[B_P2];
            const int8_t* a_ptr2[A_P2];
#pragma unroll
            for (int i = 0; i < B_P2; ++i) {
                int m = pix0 + row0 + i * RPI;
                m = m < a.M ? m : a.M - 1;
                b_base2[i] = window_offset(a, m, in_sn, in_sh, in_sw, csh, csw, flat) + origin;
            }
#pragma unroll
            for (int i = 0; i < A_P2; ++i) {
                int row = row0 + i * RPI;
                if (wgt_plain) {
                    const int j = row & 31;
                    row = (row & ~63) + 32 * ((j >> 2) & 1) + 16 * ((row >> 5) & 1) + 4 * (j >> 3) + (j & 3);
                }
                row = min(oc0 + row, wgt_rows - 1);
                a_ptr2[i] = wgt_base + static_cast<int64_t>(row) * wgt_ld + chunk * 16;
            }
            v4i ga2[A_P2], gb2[B_P2];
            auto load_pair = [&](int j) {
                // an odd step count leaves the last pair half empty: its second half re-reads the last step
                // (in bounds, never multiplied)
                const int k0 = 2 * j, k1 = min(2 * j + 1, nk - 1);
                const int4 ko0 = load_uniform_int4(koff + 4 * k0), ko1 = load_uniform_int4(koff + 4 * k1);
                const int32_t off0 = pick(ko0), off1 = pick(ko1);
                const int32_t off = sub ? off1 : off0;
                const int kk = sub ? k1 : k0;
#pragma unroll
                for (int i = 0; i < A_P2; ++i) ga2[i] = *reinterpret_cast<const v4i*>(a_ptr2[i] + kk * 64);
#pragma unroll
                for (int i = 0; i < B_P2; ++i) gb2[i] = *reinterpret_cast<const v4i*>(in_base + (b_base2[i] + off));
            };
            auto store_pair = [&]() {
#pragma unroll
                for (int i = 0; i < A_P2; ++i)
                    *reinterpret_cast<v4i*>(&sA[sub][((row0 + i * RPI) ^ sub) * kRow + slot2]) = ga2[i];
#pragma unroll
                for (int i = 0; i < B_P2; ++i)
                    *reinterpret_cast<v4i*>(&sB[sub][((row0 + i * RPI) ^ sub) * kRow + slot2]) = gb2[i];
            };
            const int npairs = (nk + 1) >> 1;
            load_pair(0);
            store_pair();
            if (first) stage_params_store<F>(a, (lds_float_ptr)sP, BOC, tid, staged);
            __syncthreads();
            if (acc_from_lds) init_acc_lds((lds_cfloat_ptr)sP, BOC, oc_lane - oc0, acc);
            for (int j = 0; j < npairs; ++j) {
                const bool more = j + 1 < npairs;
                if (more) load_pair(j + 1);
                mfma_step(0);
                if (2 * j + 1 < nk) mfma_step(1);
                __syncthreads();             // every wave has read this pair
                if (more) {
                    store_pair();
                    __syncthreads();
                }
            }
            return;
        }
        v4i ga[A_PIECES], gb[B_PIECES];
        if constexpr (F != kDyn && (F & CF_RES_GEMM)) {
            // the kernel with two GEMMs keeps the shortcut's dequantised result in 64 registers next to the accumulators:
            // plain loads through pointers here - the two buffer descriptors and the second copy of the loop below cost it
            // registers it does not have (200 bytes of scratch per lane when tried)
            auto load_global = [&](int k) {
                const int32_t off = pick(load_uniform_int4(koff + 4 * k));   // one scalar load of the step's four offsets
                const int8_t* wk = wgt_base + k * 64;                        // uniform part of the weight address
#pragma unroll
                for (int i = 0; i < A_PIECES; ++i) ga[i] = *reinterpret_cast<const v4i*>(wk + a_off[i]);
#pragma unroll
                for (int i = 0; i < B_PIECES; ++i) gb[i] = *reinterpret_cast<const v4i*>(in_base + (b_base[i] + off));
            };
            auto store_lds = [&](int buf) {
#pragma unroll
                for (int i = 0; i < A_PIECES; ++i)
                    *reinterpret_cast<v4i*>(&sA[buf][((tid + i * NT) >> 2) * kRow + lds_slot]) = ga[i];
#pragma unroll
                for (int i = 0; i < B_PIECES; ++i)
                    *reinterpret_cast<v4i*>(&sB[buf][((tid + i * NT) >> 2) * kRow + lds_slot]) = gb[i];
            };
            load_global(0);
            store_lds(0);
            if (first) stage_params_store<F>(a, (lds_float_ptr)sP, BOC, tid, staged);
            __syncthreads();
            if (acc_from_lds) init_acc_lds((lds_cfloat_ptr)sP, BOC, oc_lane - oc0, acc);
            for (int k = 0; k < nk; ++k) {
                const int buf = k & 1;
                if (k + 1 < nk) load_global(k + 1);
                mfma_step(buf);
                if (k + 1 < nk) store_lds(buf ^ 1);
                __syncthreads();
            }
            return;
        }
        // Both operands through buffer loads: a lane's offset in a register that does not change from step to step, the
        // step's part in a scalar register - no 64-bit address arithmetic per load.  The activations' buffer starts at
        // the window origin of pixel 0 (the tensor's element (0, 0, 0, 0) moved back by the padding), so that every
        // offset is non-negative.  linear: the K pieces lie one behind the other in memory (a 1 x 1 convolution, a
        // MatMul): step k is 64 k bytes behind step 0 and no table is read; else the lane adds its piece's entry of the
        // step's four offsets.
        const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(wgt_base), 0, 0x7fffffff, 0x00020000);
        const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(in_base + origin), 0, 0x7fffffff, 0x00020000);
        int32_t b_vo[B_PIECES];
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i) b_vo[i] = b_base[i] - origin + (linear ? chunk * 16 : 0);
        auto store_lds = [&](int buf) {
#pragma unroll
            for (int i = 0; i < A_PIECES; ++i)
                *reinterpret_cast<v4i*>(&sA[buf][((tid + i * NT) >> 2) * kRow + lds_slot]) = ga[i];
#pragma unroll
            for (int i = 0; i < B_PIECES; ++i)
                *reinterpret_cast<v4i*>(&sB[buf][((tid + i * NT) >> 2) * kRow + lds_slot]) = gb[i];
        };
        // (two copies of the loop behind a uniform branch: with the form as a run-time value inside one loop the
        // compiler evaluates the table path for every step and selects)
        auto k_loop = [&](auto linear_c) {
            constexpr bool LINEAR = decltype(linear_c)::value;
            auto load_global = [&](int k) {
                const int32_t sk = k * 64;
                // the step's four offsets: one scalar load, issued and awaited here, in front of the vector loads that
                // need it (requested a step ahead it would be in flight during the LDS reads of the matrix
                // instructions, whose partial waits then all become waits for everything)
                const int32_t off = LINEAR ? 0 : pick(load_uniform_int4(koff + 4 * k));
#pragma unroll
                for (int i = 0; i < A_PIECES; ++i) ga[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, static_cast<int32_t>(a_off[i]), sk, 0);
#pragma unroll
                for (int i = 0; i < B_PIECES; ++i) gb[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_vo[i] + off, LINEAR ? sk : 0, 0);
            };
            load_global(0);
            store_lds(0);
            if (first) stage_params_store<F>(a, (lds_float_ptr)sP, BOC, tid, staged);
            __syncthreads();
            if (acc_from_lds) init_acc_lds((lds_cfloat_ptr)sP, BOC, oc_lane - oc0, acc);
            for (int k = 0; k < nk; ++k) {
                const int buf = k & 1;
                if (k + 1 < nk) load_global(k + 1);
                mfma_step(buf);
                if (k + 1 < nk) store_lds(buf ^ 1);
                __syncthreads();
            }
        };
        if (linear) k_loop(std::true_type{});
        else k_loop(std::false_type{});
    };

    v16i acc[2][2];
    v16f rres[2][2];
    constexpr bool kFused = F != kDyn && (F & CF_RES_GEMM);
    static_assert(!(kFused && PAIR), "the second GEMM keeps the single-step loop");
    if (kFused) {
        // shortcut convolution first: (float(acc2) + bias2[c]) * scale2[c] stays in registers
        ConvArgs a2 = a;
        a2.corr = a.corr2;
        init_acc(a2, oc_lane, acc);
        gemm(a.in2, a.in2_sn, a.in2_sh, a.in2_sw, a.conv2_sh, a.conv2_sw, a.in2_origin, a.wgt2, a.Kp2, a.OCp, false,
             a.koff2, a.nk2, acc, true, false, false, a.k_linear2 != 0);
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 b4 = ld4f(a.bias2 + oc_lane + 16 * ob + 4 * q);
                const float4 s4 = ld4f(a.scale2 + oc_lane + 16 * ob + 4 * q);
                const float bb[4] = {b4.x, b4.y, b4.z, b4.w}, ss[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float x = static_cast<float>(acc[ob][pb][4 * q + j]) + bb[j];
                        rres[ob][pb][4 * q + j] = x * ss[j];
                    }
            }
    }
    if (kFused) init_acc_lds((lds_cfloat_ptr)sP, BOC, oc_lane - oc0, acc);   // published by the shortcut GEMM's first barrier
    gemm(a.in + batch_offset(a, batch, a.batch_in, a.batch_in_o), a.in_sn, a.in_sh, a.in_sw, a.conv_sh, a.conv_sw, a.in_origin,
         a.wgt + batch_offset(a, batch, a.batch_wgt, a.batch_wgt_o), a.wgt_ld, a.wgt_rows, a.wgt_plain != 0, a.koff + t_tile * a.koff_tile, a.nk, acc, !kFused, !kFused, a.flat_in != 0, a.k_linear != 0);
    const int m0 = pix0 + wpix * 64 + l32;
    if constexpr (PIXC) {   // MatMul between activations whose right operand is stored as level - 128
        const int32_t* pc = a.pix_corr + static_cast<int64_t>(batch) * a.batch_pix_corr;
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) {
            const int32_t v = pc[min(m0 + 32 * pb, a.M - 1)];
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ob][pb][r] += v;
        }
    }
    // the K loop ends with a barrier, so the operand tiles are free: every wave takes 8 KB of them as
    // the staging buffer of its f32 stores (2 (BOC + BPIX) 64 bytes cover 8 KB per wave for all shapes)
    constexpr int kStageWavesA = 2 * BOC * kRow / 8192;
    static_assert(2 * (BOC + BPIX) * kRow >= (NT / 64) * 8192 && 2 * BOC * kRow % 8192 == 0, "staging space");
    lds_float_ptr stage = wave < kStageWavesA ? (lds_float_ptr)&sA[0][0] + wave * 2048
                                              : (lds_float_ptr)&sB[0][0] + (wave - kStageWavesA) * 2048;
    run_epilogue<F>(a, acc, oc_lane, m0, m0 + 32, batch, rres, (lds_cfloat_ptr)sP, BOC, oc0, stage);
}

// Persistent LDS-tiled kernel for the layers whose time is the epilogue and the memory latency
// around it (small K): a workgroup keeps its channel tile and walks pixel tiles.  The operands of
// the next tile's first K step and the next tile's residual bytes are requested before the
// epilogue of the current tile, so memory latency, the matrix pipe and the epilogue's VALU work of
// one wave overlap by construction instead of by occupancy.  Grid: 8 XCDs x channel tiles x n_per
// workgroups, workgroup (xcd, t_tile, i) takes the XCD's pixel tiles i, i + n_per, ...
template <int WOC, int WPIX, uint32_t F>
__global__ __launch_bounds__(WOC* WPIX * 64, 2) void conv_persist_kernel(const ConvArgs a, const int n_per) {
    constexpr int NT = WOC * WPIX * 64;
    constexpr int BOC = WOC * 64, BPIX = WPIX * 64;
    constexpr int A_PIECES = BOC * 4 / NT, B_PIECES = BPIX * 4 / NT;
    constexpr bool kByteRes = (F & CF_RES) && !(F & (CF_RES_F32 | CF_RES_GEMM));
    __shared__ __attribute__((aligned(16))) int8_t sA[2][BOC * kRow];
    __shared__ __attribute__((aligned(16))) int8_t sB[2][BPIX * kRow];
    __shared__ __attribute__((aligned(16))) float sP[PT_ROWS * BOC];

    const int xcd = blockIdx.x & 7, y = blockIdx.x >> 3;
    int t_tile, p_local;           // p_local < n_per
    split_tile_index(a, y, p_local, t_tile);
    auto tile_exists = [&](int pl) { return pl < a.p_per_xcd && xcd * a.p_per_xcd + pl < a.p_tiles; };
    if (!tile_exists(p_local)) return;   // uniform over the workgroup
    const int oc0 = t_tile * BOC;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int woc = wave % WOC, wpix = wave / WOC;
    const int l32 = lane & 31, h = lane >> 5;
    const int chunk = tid & 3;
    const PiecePick pick(chunk);
    // XOR swizzle instead of row padding: the thread that stages (row, chunk) and the lanes that read
    // fragments (rows l32 + 32 i, chunk 2 ks + h) agree on slot = chunk ^ ((row >> 2) & 3); rows that
    // differ by a multiple of 16 share the swizzle, so (tid + i NT) >> 2 and l32 + 32 i need one value each
    const int lds_slot = (chunk ^ ((tid >> 4) & 3)) * 16;
    const int frag_slot[2] = {((0 + h) ^ ((l32 >> 2) & 3)) * 16, ((2 + h) ^ ((l32 >> 2) & 3)) * 16};
    static_assert(BOC <= NT, "one table element per thread");
    StagedParams staged;
    stage_params_load<F>(a, oc0, BOC, tid, staged);
    bool first = true;
    const int a_row[2] = {woc * 64 + l32, woc * 64 + 32 + l32};
    const int b_row[2] = {wpix * 64 + l32, wpix * 64 + 32 + l32};
    const int oc_lane = oc0 + woc * 64 + 32 * h;
    const int nk = a.nk;

    const int8_t* a_ptr[A_PIECES];
#pragma unroll
    for (int i = 0; i < A_PIECES; ++i) {
        const int row = min(oc0 + ((tid + i * NT) >> 2), a.wgt_rows - 1);
        a_ptr[i] = a.wgt + static_cast<int64_t>(row) * a.wgt_ld + chunk * 16;
    }
    int32_t b_base[B_PIECES];
    auto pixel_bases = [&](int pl) {
        const int pix0 = (xcd * a.p_per_xcd + pl) * BPIX;
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i) {
            int m = pix0 + ((tid + i * NT) >> 2);
            m = m < a.M ? m : a.M - 1;
            b_base[i] = window_offset(a, m, a.in_sn, a.in_sh, a.in_sw, a.conv_sh, a.conv_sw, a.flat_in != 0) + a.in_origin;
        }
    };
    v4i ga[A_PIECES], gb[B_PIECES];
    auto load_global = [&](int k) {
        const int32_t off = pick(load_uniform_int4(a.koff + 4 * k));
#pragma unroll
        for (int i = 0; i < A_PIECES; ++i) ga[i] = *reinterpret_cast<const v4i*>(a_ptr[i] + k * 64);
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i) gb[i] = *reinterpret_cast<const v4i*>(a.in + (b_base[i] + off));
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_PIECES; ++i)
            *reinterpret_cast<v4i*>(&sA[buf][((tid + i * NT) >> 2) * kRow + lds_slot]) = ga[i];
#pragma unroll
        for (int i = 0; i < B_PIECES; ++i)
            *reinterpret_cast<v4i*>(&sB[buf][((tid + i * NT) >> 2) * kRow + lds_slot]) = gb[i];
    };
    auto addresses = [&](int pl, EpiAddr& e) {
        const int m0 = (xcd * a.p_per_xcd + pl) * BPIX + wpix * 64 + l32;
        epilogue_addresses(a, oc_lane, m0, m0 + 32, 0, e);
    };

    EpiAddr cur, nxt;
    uint32_t res_cur[2][8], res_nxt[2][8];
    pixel_bases(p_local);
    load_global(0);
    addresses(p_local, cur);
    if (kByteRes) load_residual_bytes(a, oc_lane, cur.valid, cur.res_off, res_cur);
    v16f none[2][2];
    while (true) {
        v16i acc[2][2];
        store_lds(0);
        if (first) stage_params_store<F>(a, (lds_float_ptr)sP, BOC, tid, staged);
        first = false;
        __syncthreads();
        init_acc_lds((lds_cfloat_ptr)sP, BOC, oc_lane - oc0, acc);
        const int next_p = p_local + n_per;
        const bool has_next = tile_exists(next_p);
        for (int k = 0; k < nk; ++k) {
            const int buf = k & 1;
            if (k + 1 < nk) {
                load_global(k + 1);
            } else if (has_next) {   // first K step of the next tile, in flight during the epilogue
                pixel_bases(next_p);
                load_global(0);
            }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                v4i af[2], bf[2];
#pragma unroll
                for (int ob = 0; ob < 2; ++ob)
                    af[ob] = *reinterpret_cast<const v4i*>(&sA[buf][a_row[ob] * kRow + frag_slot[ks]]);
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
                    bf[pb] = *reinterpret_cast<const v4i*>(&sB[buf][b_row[pb] * kRow + frag_slot[ks]]);
#pragma unroll
                for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                    for (int pb = 0; pb < 2; ++pb)
                        acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ob], bf[pb], acc[ob][pb], 0, 0, 0);
            }
            if (k + 1 < nk) {
                store_lds(buf ^ 1);
                __syncthreads();
            }
        }
        if (has_next) {
            addresses(next_p, nxt);
            if (kByteRes) load_residual_bytes(a, oc_lane, nxt.valid, nxt.res_off, res_nxt);
        }
        epilogue<F>(a, acc, oc_lane, cur.valid, cur.out_off, cur.res_off, none, (lds_cfloat_ptr)sP, BOC, oc0, kByteRes ? res_cur : nullptr);
        if (!has_next) break;
        cur = nxt;
        if (kByteRes) {
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int q = 0; q < 8; ++q) res_cur[pb][q] = res_nxt[pb][q];
        }
        p_local = next_p;
        __syncthreads();   // every wave has read the last K step before the buffers are refilled
    }
}

// ------------------------------------------------------------------------------------------------
// Pipelined LDS-tiled kernel: a ring of `stages` K steps in LDS filled by direct global->LDS loads
// (global_load_lds_dwordx4: no staging registers, so many K steps can be in flight), one raw
// s_barrier per step.  Rows are 64 bytes without padding; the 16-byte chunk c of row r sits in
// slot c ^ ((r >> 2) & 3), which makes both the DMA writes (lane t -> byte 16 t of a 1 KiB group)
// and the ds_read_b128 fragment reads (16 consecutive rows, one logical chunk) conflict-free.
// Hazards are ordered by hand: a wave waits for its own loads of the step it is about to read
// (s_waitcnt vmcnt(n) with the younger stages still in flight), then the barrier makes every
// wave's part of that step visible and proves that the stage about to be refilled is no longer read.
constexpr int waitcnt_vm(int n) {
    // s_waitcnt immediate: vmcnt in bits [3:0] and [15:14]; expcnt / lgkmcnt left at "no wait"
    return 0x0F70 | (n & 15) | ((n >> 4) << 14);
}

// KS = 2: eight waves; wave group g (four waves, own ring) multiplies the K steps k = g mod 2 and
// group 1 hands its partial sums to group 0 through LDS.  Twice the waves per compute unit keep
// twice the loads in flight, which is what bounds the layers with fewer tiles than compute units.
template <int WOC, int WPIX, uint32_t F, int KS>
__global__ __launch_bounds__(WOC* WPIX * 64 * KS, KS == 2 ? 1 : 2)
void conv_pipe_kernel(const ConvArgs a, const int stages) {
    constexpr int NT = WOC * WPIX * 64;          // threads of one wave group
    constexpr int NT_ALL = NT * KS;
    constexpr int BOC = WOC * 64, BPIX = WPIX * 64;
    constexpr int A_GROUPS = BOC / 16 / (NT / 64), B_GROUPS = BPIX / 16 / (NT / 64);   // 1 KiB groups per wave
    constexpr int LPS = A_GROUPS + B_GROUPS;   // loads per wave per stage
    static_assert(6 * LPS < 64, "vmcnt is a 6-bit counter");
    constexpr int STAGE = (BOC + BPIX) * 64;
    extern __shared__ __attribute__((aligned(16))) int8_t ring[];

    int t_tile, p_tile;
    if (a.p_per_xcd > 0) {
        const int xcd = blockIdx.x & 7, y = blockIdx.x >> 3;
        int p_local;
        split_tile_index(a, y, p_local, t_tile);
        p_tile = xcd * a.p_per_xcd + p_local;
        if (p_local >= a.p_per_xcd || p_tile >= a.p_tiles) return;
    } else {   // few pixel tiles: plain order, consecutive workgroups land on consecutive XCDs
        split_tile_index(a, blockIdx.x, p_tile, t_tile);
    }
    const int pix0 = p_tile * BPIX, oc0 = t_tile * BOC;

    const int tid = threadIdx.x, lane = tid & 63;
    // wave-uniform by construction; said so, or the LDS base of every DMA load goes through a VGPR
    const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = KS == 1 ? 0 : wave_all / (NT / 64), wave = wave_all % (NT / 64);
    const int woc = wave % WOC, wpix = wave / WOC;
    int8_t* const gring = ring + grp * stages * STAGE;
    const int l32 = lane & 31, h = lane >> 5;
    const int batch = blockIdx.y;
    const int oc_lane = oc0 + woc * 64 + 32 * h;
    // DMA role of this lane inside a 16-row group: row lane>>2, logical chunk (lane&3) ^ ((lane>>4)&3)
    const int dma_row = lane >> 2, dma_chunk = (lane & 3) ^ ((lane >> 4) & 3);
    // fragment reads: row l32 (+32 ob / pb), logical chunk 2*ks + h -> slot
    const int swz = (l32 >> 2) & 3;
    const int frag_off[2] = {l32 * 64 + ((0 + h) ^ swz) * 16, l32 * 64 + ((2 + h) ^ swz) * 16};
    // epilogue tables behind the rings; visible after the barrier that follows the K-offset table fill
    float* const sP = reinterpret_cast<float*>(ring + KS * stages * STAGE);
    stage_params<F>(a, oc0, (lds_float_ptr)sP, BOC, tid, NT_ALL);

    auto gemm = [&](const int8_t* in_base, int in_sn, int in_sh, int in_sw, int csh, int csw, int origin,
                    const int8_t* wgt_base, int wgt_ld, int wgt_rows, bool wgt_plain, const int32_t* koff, int nk_all,
                    v16i (&acc)[2][2], bool flat) {
        const int nk = nk_all / KS;   // steps of this wave group: local step j is global step j * KS + grp
        const int8_t* a_ptr[A_GROUPS];
        int32_t b_base[B_GROUPS];
#pragma unroll
        for (int i = 0; i < A_GROUPS; ++i) {
            int row = (wave * A_GROUPS + i) * 16 + dma_row;
            if (wgt_plain) {
                const int j = row & 31;
                row = (row & ~63) + 32 * ((j >> 2) & 1) + 16 * ((row >> 5) & 1) + 4 * (j >> 3) + (j & 3);
            }
            row = min(oc0 + row, wgt_rows - 1);
            a_ptr[i] = wgt_base + static_cast<int64_t>(row) * wgt_ld + dma_chunk * 16;
        }
#pragma unroll
        for (int i = 0; i < B_GROUPS; ++i) {
            int m = pix0 + (wave * B_GROUPS + i) * 16 + dma_row;
            m = m < a.M ? m : a.M - 1;
            b_base[i] = window_offset(a, m, in_sn, in_sh, in_sw, csh, csw, flat) + origin;
        }
        // The K-offset table lives in LDS behind the ring: a vector-memory load of it would have to
        // be awaited with vmcnt(0), which drains every DMA load in flight and serialises the ring.
        int32_t* kt = reinterpret_cast<int32_t*>(ring + KS * stages * STAGE + PT_ROWS * BOC * 4);
        for (int i = tid; i < 4 * nk_all; i += NT_ALL) kt[i] = koff[i];
        __syncthreads();
        auto issue = [&](int stage, int j, int32_t off) {
            int8_t* sa = gring + stage * STAGE;
            int8_t* sb = sa + BOC * 64;
            const int k = j * KS + grp;
#pragma unroll
            for (int i = 0; i < A_GROUPS; ++i)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(a_ptr[i] + k * 64),
                                                 (__attribute__((address_space(3))) void*)(sa + (wave * A_GROUPS + i) * 1024),
                                                 16, 0, 0);
#pragma unroll
            for (int i = 0; i < B_GROUPS; ++i)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(in_base + (b_base[i] + off)),
                                                 (__attribute__((address_space(3))) void*)(sb + (wave * B_GROUPS + i) * 1024),
                                                 16, 0, 0);
        };
        // Software pipeline over a ring of 3 to 8 stages.  Iteration k multiplies step k in two halves of
        // 32 K bytes; the fragments of each half are read from LDS while the other half is in the matrix
        // pipe, and the barrier sits between the halves:
        //   read (k, half 1) | mfma (k, half 0) | wait own loads of step k+1, barrier |
        //   refill the slot of step k-1 with step k+stages-1 | read (k+1, half 0) | mfma (k, half 1)
        // After barrier k every wave's part of step k+1 has landed and every wave has consumed
        // step k-1, whose slot is the one refilled.  A layer with no more workgroups than compute
        // units has ONE wave per SIMD, and whatever that wave waits for between two matrix
        // instructions is time the matrix pipe idles: the loop body is straight-line code (last
        // iteration peeled, the K offset of the step to request read at the top, the ring depth a
        // constant of the loop so that its wait is one instruction), and a deep ring keeps the
        // slowest of a step's 256 cache lines (an L2 miss among them, most steps) off the critical path.
        v4i fa[2][2], fb[2][2];
        auto read_frags = [&](int slot, int ks, v4i (&af)[2], v4i (&bf)[2]) {
            const int8_t* sa = gring + slot * STAGE + (woc * 64) * 64;
            const int8_t* sb = gring + slot * STAGE + BOC * 64 + (wpix * 64) * 64;
#pragma unroll
            for (int ob = 0; ob < 2; ++ob) af[ob] = *reinterpret_cast<const v4i*>(sa + ob * 32 * 64 + frag_off[ks]);
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) bf[pb] = *reinterpret_cast<const v4i*>(sb + pb * 32 * 64 + frag_off[ks]);
        };
        auto mfma4 = [&](const v4i (&af)[2], const v4i (&bf)[2]) {
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
                    acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ob], bf[pb], acc[ob][pb], 0, 0, 0);
        };
        static_assert(5 * LPS < 64, "vmcnt is a 6-bit counter");
        const int ahead = min(stages - 1, nk);
        for (int s0 = 0; s0 < ahead; ++s0) issue(s0, s0, kt[4 * (s0 * KS + grp) + dma_chunk]);
        // the loop for a ring of Y + 3 stages: in the steady state Y younger steps stay in flight behind
        // step k+1; towards the end the wait is for everything (what is left in flight is due next anyway)
        auto loop = [&](auto depth) {
            constexpr int Y = decltype(depth)::value;
            if (ahead - 1 >= Y + 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm((Y + 1) * LPS));   // step 0 of a full ring
            else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            __builtin_amdgcn_s_barrier();
            int rd = 0, wr = ahead % stages;
            read_frags(0, 0, fa[0], fb[0]);
            for (int k = 0; k + 1 < nk; ++k) {
                const int kn = k + Y + 2;                                        // the step requested in this iteration
                const int32_t off_req = kt[4 * (min(kn, nk - 1) * KS + grp) + dma_chunk];
                read_frags(rd, 1, fa[1], fb[1]);
                mfma4(fa[0], fb[0]);
                const int nrd = rd + 1 == Y + 3 ? 0 : rd + 1;
                // outstanding: steps k+1 .. min(k + Y + 1, nk - 1)
                if (k + Y + 1 < nk) __builtin_amdgcn_s_waitcnt(waitcnt_vm(Y * LPS));
                else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
                __builtin_amdgcn_s_barrier();
                if (kn < nk) {
                    issue(wr, kn, off_req);
                    wr = wr + 1 == Y + 3 ? 0 : wr + 1;
                }
                read_frags(nrd, 0, fa[0], fb[0]);
                mfma4(fa[1], fb[1]);
                rd = nrd;
            }
            read_frags(rd, 1, fa[1], fb[1]);                                     // last step: nothing left to request
            mfma4(fa[0], fb[0]);
            mfma4(fa[1], fb[1]);
        };
        switch (stages) {                                                        // uniform
        case 3: loop(std::integral_constant<int, 0>{}); break;
        case 4: loop(std::integral_constant<int, 1>{}); break;
        case 6: loop(std::integral_constant<int, 3>{}); break;
        default: loop(std::integral_constant<int, 5>{}); break;                  // 8
        }
        __builtin_amdgcn_s_barrier();   // every wave is done reading before the ring is refilled
    };

    v16i acc[2][2];
    v16f rres[2][2];
    constexpr bool kFused = F != kDyn && (F & CF_RES_GEMM);
    if (kFused) {
        ConvArgs a2 = a;
        a2.corr = a.corr2;
        init_acc(a2, oc_lane, acc);
        gemm(a.in2, a.in2_sn, a.in2_sh, a.in2_sw, a.conv2_sh, a.conv2_sw, a.in2_origin, a.wgt2, a.Kp2, a.OCp, false,
             a.koff2, a.nk2, acc, false);
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 b4 = ld4f(a.bias2 + oc_lane + 16 * ob + 4 * q);
                const float4 s4 = ld4f(a.scale2 + oc_lane + 16 * ob + 4 * q);
                const float bb[4] = {b4.x, b4.y, b4.z, b4.w}, ss[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float x = static_cast<float>(acc[ob][pb][4 * q + j]) + bb[j];
                        rres[ob][pb][4 * q + j] = x * ss[j];
                    }
            }
    }
    // K split over workgroups: part z of S multiplies the K steps [nk z / S, nk (z + 1) / S)
    const int S = KS == 1 ? a.ksplit : 1, z = S > 1 ? static_cast<int>(blockIdx.z) : 0;
    const int k_first = S > 1 ? (a.nk * z) / S : 0;
    const int nk_part = S > 1 ? (a.nk * (z + 1)) / S - k_first : a.nk;
    if (grp == 0 && z == 0) {
        init_acc(a, oc_lane, acc);
    } else {
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ob][pb][r] = 0;
    }
    gemm(a.in + batch * a.batch_in, a.in_sn, a.in_sh, a.in_sw, a.conv_sh, a.conv_sw, a.in_origin,
         a.wgt + batch * a.batch_wgt + k_first * 64, a.wgt_ld, a.wgt_rows, a.wgt_plain != 0, a.koff + 4 * k_first, nk_part, acc,
         a.flat_in != 0);
    if (KS == 1 && S > 1) {
        // Every part stores its accumulators (register r of thread t at dword r * NT + t: whole cache lines per
        // wave) and takes a ticket; the workgroup that draws the last ticket of its tile adds the other parts to
        // its own registers and runs the epilogue, the others are done.  Integer sums do not depend on the order.
        // No workgroup waits for another.  The partial sums cross between compute dies, whose L2 caches are not
        // coherent with each other: they are written and read with device-scope accesses (which go through to
        // memory) instead of fences, because a device-scope fence writes back or invalidates a die's whole L2
        // and costs more than the split saves.
        const int tile_id = t_tile * a.p_tiles + p_tile;
        int32_t* const parts = a.ws_part + static_cast<int64_t>(tile_id) * S * (64 * NT);
        int32_t* const mine = parts + z * (64 * NT) + tid;
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    __hip_atomic_store(&mine[((ob * 2 + pb) * 16 + r) * NT], acc[ob][pb][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));                            // the stores have reached device-wide memory
        __syncthreads();
        uint32_t* const ticket = reinterpret_cast<uint32_t*>(ring);          // the ring is no longer read
        if (tid == 0) {
            const uint32_t t = atomicAdd(a.ws_count + tile_id, 1u);
            if (t == static_cast<uint32_t>(S - 1)) atomicExch(a.ws_count + tile_id, 0u);   // zero again for the next launch
            *ticket = t;
        }
        __syncthreads();
        const uint32_t drawn = *ticket;
        __syncthreads();                                                     // read by every wave before the epilogue stages its stores here
        if (drawn != static_cast<uint32_t>(S - 1)) return;
        for (int zz = 0; zz < S; ++zz) {
            if (zz == z) continue;
            const int32_t* const other = parts + zz * (64 * NT) + tid;
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc[ob][pb][r] += __hip_atomic_load(&other[((ob * 2 + pb) * 16 + r) * NT], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (KS == 2) {
        // partial sums of group 1 -> LDS (register r of thread t at dword r * NT + t), added by group 0
        int32_t* red = reinterpret_cast<int32_t*>(ring);
        const int t = tid % NT;
        if (grp == 1) {
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) red[((ob * 2 + pb) * 16 + r) * NT + t] = acc[ob][pb][r];
        }
        __syncthreads();
        if (grp == 1) return;
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[ob][pb][r] += red[((ob * 2 + pb) * 16 + r) * NT + t];
    }
    const int m0 = pix0 + wpix * 64 + l32;
    run_epilogue<F, true, false>(a, acc, oc_lane, m0, m0 + 32, batch, rres, (lds_cfloat_ptr)sP, BOC, oc0);   // tables in (dynamic) LDS, no staging
}

// ------------------------------------------------------------------------------------------------
// Row-tile kernel for 3 x 3, stride 1, pad 1 convolutions: the implicit GEMM above fetches every input
// pixel once per filter tap (nine times), and the path from L2 into the compute unit is what bounds
// these layers.  Here a workgroup takes whole output rows of one image (R rows, R * OW <= 256 pixels)
// and 64 output channels; per 64 input channels it stages the input patch ((R + 2) x (OW + 2) pixels,
// read from the tensor's own halo where the filter overhangs) and the nine 64-byte weight slices ONCE
// in LDS, and the nine taps read their B fragments from the patch at shifted positions.  No barrier
// inside the 72 matrix instructions of a chunk.  LDS rows are 64 bytes (patch pixels) and 576 bytes
// (weights: 64 mod 256, so the same bank picture), chunk c of row r in slot c ^ ((r >> 2) & 3).
constexpr int kPatchRows = 384;   // 24 KB: three waves' staging space later
template <uint32_t F>
__global__ __launch_bounds__(256, 2) void conv_rows_kernel(const ConvArgs a) {
    __shared__ __attribute__((aligned(16))) int8_t sPatch[kPatchRows * 64];
    __shared__ __attribute__((aligned(16))) int8_t sW[64 * 576];
    __shared__ __attribute__((aligned(16))) float sP[PT_ROWS * 64];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    int p_tile, t_tile;
    split_tile_index(a, blockIdx.x, p_tile, t_tile);
    const int oc0 = t_tile * 64;
    const int n = p_tile / a.tiles_per_image, ty = p_tile - n * a.tiles_per_image;
    const int OH = a.OHOW / a.OW;
    const int y0 = ty * a.rows_per_tile;                                  // first output row of the tile
    const int rows = min(a.rows_per_tile, OH - y0);
    const int count = rows * a.OW;                                        // pixels of this tile
    const int pix0 = n * a.OHOW + y0 * a.OW;
    const int PW = a.patch_w, patch_rows = (rows + 2) * PW;
    const int oc_lane = oc0 + 32 * h;
    stage_params<F>(a, oc0, (lds_float_ptr)sP, 64, tid, 256);

    // patch position of the lane's two pixels at tap (0, 0)
    int idx0[2];
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
        const int p = min(wave * 64 + pb * 32 + l32, count - 1);
        int r, x;
        fast_divmod(p, a.OW, a.inv_OW, r, x);
        idx0[pb] = r * PW + x;
    }
    // input element (n, y0 - 1, -1, 0): the patch's first pixel (in the halo)
    const int8_t* in0 = a.in + (static_cast<int64_t>(n) * a.in_sn + (y0 - 1) * a.in_sh - a.in_sw);
    const int8_t* w0 = a.wgt + static_cast<int64_t>(oc0) * a.wgt_ld;

    v16i acc[2][2];
    v16f rres[2][2];
    init_acc(a, oc_lane, acc);
    const int chunks = a.Kp / 576;                                        // 64-channel slices of the input
    for (int c = 0; c < chunks; ++c) {
        if (c > 0) __syncthreads();                                       // everyone is done with the previous slice
        // all requests of the slice go out before the first of them is awaited
        constexpr int PP = kPatchRows * 4 / 256;                          // patch pieces per thread, at most
        v4i pv[PP], wv[9];
#pragma unroll
        for (int j = 0; j < PP; ++j) {
            const int i = min(tid + j * 256, patch_rows * 4 - 1);
            const int row = i >> 2, ch = i & 3;
            int py, px;
            fast_divmod(row, PW, a.inv_patch_w, py, px);
            pv[j] = *reinterpret_cast<const v4i*>(in0 + (py * a.in_sh + px * a.in_sw + c * 64 + ch * 16));
        }
#pragma unroll
        for (int j = 0; j < 9; ++j) {                                     // 64 rows x 9 taps x 4 chunks = 9 x 256 pieces
            const int i = tid + j * 256;
            const int row = i / 36, rem = i - row * 36, tap = rem >> 2, ch = rem & 3;
            const int wrow = min(oc0 + row, a.wgt_rows - 1) - oc0;
            wv[j] = *reinterpret_cast<const v4i*>(w0 + (static_cast<int64_t>(wrow) * a.wgt_ld + tap * (chunks * 64) + c * 64 + ch * 16));
        }
#pragma unroll
        for (int j = 0; j < PP; ++j) {
            const int i = tid + j * 256;
            const int row = i >> 2, ch = i & 3;
            if (i < patch_rows * 4) *reinterpret_cast<v4i*>(&sPatch[row * 64 + ((ch ^ ((row >> 2) & 3)) << 4)]) = pv[j];
        }
#pragma unroll
        for (int j = 0; j < 9; ++j) {
            const int i = tid + j * 256;
            const int row = i / 36, rem = i - row * 36, tap = rem >> 2, ch = rem & 3;
            *reinterpret_cast<v4i*>(&sW[row * 576 + tap * 64 + ((ch ^ ((row >> 2) & 3)) << 4)]) = wv[j];
        }
        __syncthreads();
#pragma unroll
        for (int kh = 0; kh < 3; ++kh)
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const int tap = kh * 3 + kw;
                int idx[2];
#pragma unroll
                for (int pb = 0; pb < 2; ++pb) idx[pb] = idx0[pb] + kh * PW + kw;
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    v4i af[2], bf[2];
#pragma unroll
                    for (int ob = 0; ob < 2; ++ob) {
                        const int row = ob * 32 + l32;
                        af[ob] = *reinterpret_cast<const v4i*>(&sW[row * 576 + tap * 64 + (((2 * ks + h) ^ ((row >> 2) & 3)) << 4)]);
                    }
#pragma unroll
                    for (int pb = 0; pb < 2; ++pb)
                        bf[pb] = *reinterpret_cast<const v4i*>(&sPatch[idx[pb] * 64 + (((2 * ks + h) ^ ((idx[pb] >> 2) & 3)) << 4)]);
#pragma unroll
                    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                        for (int pb = 0; pb < 2; ++pb)
                            acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ob], bf[pb], acc[ob][pb], 0, 0, 0);
                }
            }
    }
    __syncthreads();                                                      // the patch becomes the stores' staging space
    ConvArgs e = a;
    e.M = min(a.M, pix0 + count);                                         // pixels behind the tile's rows belong to the next tile
    const int m0 = pix0 + wave * 64 + l32;
    lds_float_ptr stage = wave < 3 ? (lds_float_ptr)&sPatch[0] + wave * 2048 : (lds_float_ptr)&sW[0];
    run_epilogue<F>(e, acc, oc_lane, m0, m0 + 32, 0, rres, (lds_cfloat_ptr)sP, 64, oc0, stage);
}

// ------------------------------------------------------------------------------------------------
// First-layer kernel: few input channels (pixel = 4 bytes), one 32-byte K slice per filter row (the
// packing of such layers: kw * 4 <= 32 bytes of taps, zero-padded).  As an implicit GEMM the 7 x 7
// stride-2 stem fetches every input byte about twelve times; here a workgroup takes R whole output rows
// of one image x 64 channels, stages the input patch ((R - 1) stride + kh rows, 8 KB) and the weights
// (64 x kh x 32 bytes) once, and a lane's B fragment of filter row kh is the 32 contiguous patch bytes
// that start at its pixel's window (8-byte aligned: two ds_read_b64).  Bytes of the slice behind the
// last tap meet zero weights.  Weight rows are 240 bytes apart in LDS (16 x 15: conflict-free b128 reads).
constexpr int kStemPatch = 12288, kStemWRow = 240, kStemLds = 36864;
template <uint32_t F>
__global__ __launch_bounds__(256, 2) void conv_stem_kernel(const ConvArgs a) {
    __shared__ __attribute__((aligned(16))) int8_t lds[kStemLds];          // patch | weights; later 4 x 8 KB of staging
    __shared__ __attribute__((aligned(16))) float sP[PT_ROWS * 64];
    int8_t* const sPatch = lds;
    int8_t* const sW = lds + kStemPatch;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    int p_tile, t_tile;
    split_tile_index(a, blockIdx.x, p_tile, t_tile);
    const int oc0 = t_tile * 64;
    const int n = p_tile / a.tiles_per_image, ty = p_tile - n * a.tiles_per_image;
    const int R = a.rows_per_tile, y0 = ty * R;
    const int count = R * a.OW, pix0 = n * a.OHOW + y0 * a.OW;
    const int PWb = a.patch_w * 4;                                          // patch row in bytes
    const int oc_lane = oc0 + 32 * h;
    stage_params<F>(a, oc0, (lds_float_ptr)sP, 64, tid, 256);

    // patch: input rows y0 * stride - pad_top .., columns -pad_left ..; dword by dword (rows start 4-byte aligned)
    const int8_t* in0 = a.in + (static_cast<int64_t>(n) * a.in_sn + (y0 * a.conv_sh - a.stem_pad_top) * a.in_sh - a.stem_pad_left * 4);
    const int row_dw = a.patch_w, total_dw = a.stem_patch_rows * row_dw;
    constexpr int PD = kStemPatch / 4 / 256;                                // dwords per thread, at most
    uint32_t pv[PD];
#pragma unroll
    for (int j = 0; j < PD; ++j) {
        const int i = min(tid + j * 256, total_dw - 1);
        int py, px;
        fast_divmod(i, row_dw, a.inv_patch_w, py, px);
        pv[j] = *reinterpret_cast<const uint32_t*>(in0 + (py * a.in_sh + px * 4));
    }
    // weights: the packed rows' kh * 32 bytes, 16 bytes at a time
    const int w_pieces = 64 * a.stem_kh * 2;
    const int8_t* w0 = a.wgt + static_cast<int64_t>(oc0) * a.wgt_ld;
    v4i wv[4];
    int w_at[4];                                                            // where the piece goes in LDS
    const int ppr = a.stem_kh * 2;                                          // 16-byte pieces per weight row
    const float inv_ppr = 1.0f / static_cast<float>(ppr);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int i = min(tid + j * 256, w_pieces - 1);
        int row, pc;
        fast_divmod(i, ppr, inv_ppr, row, pc);
        wv[j] = *reinterpret_cast<const v4i*>(w0 + (static_cast<int64_t>(row) * a.wgt_ld + pc * 16));
        w_at[j] = row * kStemWRow + pc * 16;
    }
#pragma unroll
    for (int j = 0; j < PD; ++j) {
        const int i = tid + j * 256;
        if (i < total_dw) *reinterpret_cast<uint32_t*>(&sPatch[i * 4]) = pv[j];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (tid + j * 256 < w_pieces) *reinterpret_cast<v4i*>(&sW[w_at[j]]) = wv[j];
    // window start of the lane's two pixels in the patch (bytes), filter row 0
    int b0[2];
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
        const int p = min(wave * 64 + pb * 32 + l32, count - 1);
        int r, x;
        fast_divmod(p, a.OW, a.inv_OW, r, x);
        b0[pb] = r * a.conv_sh * PWb + x * a.conv_sw * 4 + 16 * h;
    }
    v16i acc[2][2];
    v16f rres[2][2];
    init_acc(a, oc_lane, acc);
    __syncthreads();
    typedef int v2i __attribute__((ext_vector_type(2)));
    for (int kh = 0; kh < a.stem_kh; ++kh) {
        v4i af[2], bf[2];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob) af[ob] = *reinterpret_cast<const v4i*>(&sW[(ob * 32 + l32) * kStemWRow + kh * 32 + 16 * h]);
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) {
            const int8_t* q = &sPatch[b0[pb] + kh * PWb];
            const v2i lo = *reinterpret_cast<const v2i*>(q), hi = *reinterpret_cast<const v2i*>(q + 8);
            bf[pb].x = lo.x; bf[pb].y = lo.y; bf[pb].z = hi.x; bf[pb].w = hi.y;
        }
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
                acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ob], bf[pb], acc[ob][pb], 0, 0, 0);
    }
    __syncthreads();                                                       // patch and weights become the stores' staging space
    ConvArgs e = a;
    e.M = min(a.M, pix0 + count);
    const int m0 = pix0 + wave * 64 + l32;
    run_epilogue<F>(e, acc, oc_lane, m0, m0 + 32, 0, rres, (lds_cfloat_ptr)sP, 64, oc0, (lds_float_ptr)lds + wave * 2048);
}

// ------------------------------------------------------------------------------------------------
// Streaming kernel: grid (x, channel tiles of 64); a workgroup of 4 waves walks pixel tiles of 256
// (64 per wave) with stride gridDim.x.  Dynamic LDS: 64 rows of (Kp + 16) weight bytes.
template <uint32_t F>
__global__ __launch_bounds__(256, 2) void conv_stream_kernel(const ConvArgs a) {
    extern __shared__ __attribute__((aligned(16))) int8_t sW[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int oc0 = blockIdx.y * 64;
    const int wrow = a.Kp + 16;   // 16 * odd: 16 consecutive rows hit distinct bank groups

    {   // the channel tile's whole weight slab -> LDS, once
        const int pieces_per_row = a.Kp >> 4, total = 64 * pieces_per_row;
        const int8_t* src = a.wgt + static_cast<int64_t>(oc0) * a.Kp;
        for (int i = tid; i < total; i += 256) {
            const int row = i / pieces_per_row, pc = i - row * pieces_per_row;
            *reinterpret_cast<v4i*>(&sW[row * wrow + pc * 16]) =
                *reinterpret_cast<const v4i*>(src + static_cast<int64_t>(row) * a.Kp + pc * 16);
        }
    }
    float* const sP = reinterpret_cast<float*>(sW + 64 * wrow);
    stage_params<F>(a, oc0, (lds_float_ptr)sP, 64, tid, 256);
    const int oc_lane = oc0 + 32 * h;
    const int a_row[2] = {l32 * wrow + h * 16, (32 + l32) * wrow + h * 16};

    int tile = blockIdx.x;
    const int n_tiles = a.p_tiles;
    int32_t base[2];
    auto pixel_base = [&](int t, int32_t (&b)[2]) {
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) {
            int m = t * 256 + wave * 64 + pb * 32 + l32;
            m = m < a.M ? m : a.M - 1;
            b[pb] = window_offset(a, m, a.in_sn, a.in_sh, a.in_sw, a.conv_sh, a.conv_sw, a.flat_in != 0) + a.in_origin;
        }
    };
    auto load_b = [&](const int32_t (&b)[2], int k, v4i (&f)[2][2]) {
        const int4 ko = load_uniform_int4(a.koff + 4 * k);
        const int32_t o0 = h ? ko.y : ko.x, o1 = h ? ko.w : ko.z;
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) {
            f[0][pb] = *reinterpret_cast<const v4i*>(a.in + (b[pb] + o0));
            f[1][pb] = *reinterpret_cast<const v4i*>(a.in + (b[pb] + o1));
        }
    };
    // Work items are (tile, k) pairs in order; item i+1 is loaded while item i is multiplied.
    // Two register sets alternate (no copies: a copy would wait for the load it copies).
    v4i bset[2][2][2];
    int k = 0;
    bool have = tile < n_tiles;
    if (have) {
        pixel_base(tile, base);
        load_b(base, 0, bset[0]);
    }
    __syncthreads();   // weights resident; no barrier after this point
    v16i acc[2][2];
    init_acc(a, oc_lane, acc);
    auto compute = [&](const v4i (&b)[2][2], int kk) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v4i af[2];
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
                af[ob] = *reinterpret_cast<const v4i*>(&sW[a_row[ob] + kk * 64 + ks * 32]);
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
                    acc[ob][pb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ob], b[ks][pb], acc[ob][pb], 0, 0, 0);
        }
    };
    // one pipeline stage: prefetch the next item into `nxt`, multiply `cur`, finish the tile if
    // this was its last K step.  Returns false when there is no next item.
    auto stage = [&](const v4i (&cur)[2][2], v4i (&nxt)[2][2]) -> bool {
        const int cur_tile = tile, cur_k = k;
        bool more = true;
        if (k + 1 < a.nk) {
            ++k;
            load_b(base, k, nxt);
        } else {
            k = 0;
            tile += gridDim.x;
            more = tile < n_tiles;
            if (more) {
                pixel_base(tile, base);
                load_b(base, 0, nxt);
            }
        }
        compute(cur, cur_k);
        if (cur_k + 1 == a.nk) {
            const int m0 = cur_tile * 256 + wave * 64 + l32;
            run_epilogue<F, true>(a, acc, oc_lane, m0, m0 + 32, 0, (lds_cfloat_ptr)sP, 64, oc0);
            init_acc(a, oc_lane, acc);
        }
        return more;
    };
    while (have) {
        if (!stage(bset[0], bset[1])) break;
        if (!stage(bset[1], bset[0])) break;
    }
}

template <int WOC, int WPIX>
void launch_tiled(const ConvArgs& a, hipStream_t s, int batches = 1) {
    const dim3 grid(a.p_per_xcd > 0 ? 8 * a.p_per_xcd * a.t_tiles : a.p_tiles * a.t_tiles, batches), block(WOC * WPIX * 64);
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_TILED(FLAGS, ...) \
    hipLaunchKernelGGL((conv_tiled_kernel<WOC, WPIX, FLAGS>), grid, block, 0, s, a)
    HIPIE_FOR_EACH_EPILOGUE(HIPIE_LAUNCH_TILED, 0)
#undef HIPIE_LAUNCH_TILED
}

// the same tiles with one accumulator correction per output row (ConvArgs::pix_corr): the epilogues a MatMul between
// activations ends in as template constants, any other through the instance that reads its flags at run time
template <int WOC, int WPIX>
void launch_tiled_pixc(const ConvArgs& a, hipStream_t s, int batches) {
    const dim3 grid(a.p_tiles * a.t_tiles, batches), block(WOC * WPIX * 64);
    switch (a.flags & ~CF_OUT_XOR) {
    case E_SCALE: hipLaunchKernelGGL((conv_tiled_kernel<WOC, WPIX, E_SCALE, false, true>), grid, block, 0, s, a); break;
    case E_DEQFQ: hipLaunchKernelGGL((conv_tiled_kernel<WOC, WPIX, E_DEQFQ, false, true>), grid, block, 0, s, a); break;
    default: hipLaunchKernelGGL((conv_tiled_kernel<WOC, WPIX, kDyn, false, true>), grid, block, 0, s, a); break;
    }
}

template <int WOC, int WPIX, int KS>
void launch_pipe(const ConvArgs& a, int stages, hipStream_t s, int batches = 1) {
    const dim3 grid(a.p_per_xcd > 0 ? 8 * a.p_per_xcd * a.t_tiles : a.p_tiles * a.t_tiles, batches, a.ksplit > 1 ? a.ksplit : 1),
        block(WOC * WPIX * 64 * KS);
    const size_t lds = static_cast<size_t>(KS) * stages * (WOC + WPIX) * 64 * 64 + PT_ROWS * WOC * 64 * 4 +
                       16 * static_cast<size_t>(std::max(a.nk, a.nk2));
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_PIPE(FLAGS, ...)                                                                       \
    do {                                                                                                    \
        if constexpr ((FLAGS) != kDyn && ((FLAGS) & CF_RES_GEMM)) break;   /* the second GEMM exists in the tiled kernel only */ \
        else {                                                                                              \
            static bool attr_set = false;                                                                   \
            if (!attr_set) {                                                                                \
                HIPIE_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_pipe_kernel<WOC, WPIX, FLAGS, KS>), \
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); \
                attr_set = true;                                                                            \
            }                                                                                               \
            hipLaunchKernelGGL((conv_pipe_kernel<WOC, WPIX, FLAGS, KS>), grid, block, lds, s, a, stages);   \
        }                                                                                                   \
    } while (0)
    HIPIE_FOR_EACH_EPILOGUE(HIPIE_LAUNCH_PIPE, 0)
#undef HIPIE_LAUNCH_PIPE
}

// Workspace of the kernels that split K over workgroups: partial accumulators and arrival counters, one
// per (device, stream).  Launches on one stream run one after another, so they can share it; launches on
// different streams (several requests in flight) get their own.  It is created, or replaced by a larger
// one after the stream has drained, on the first launch that needs it; the counters start at zero and every
// launch leaves them at zero.  Kept until the process ends.
struct SplitWorkspace {
    DeviceBuffer part, count;
    size_t tiles = 0;
};
struct SplitPool {
    std::mutex mu;
    std::map<std::pair<int, hipStream_t>, SplitWorkspace> of_stream;
};
SplitPool& split_pool() {
    static auto* pool = new SplitPool();   // never destroyed: the HIP runtime may be gone before static destructors run
    return *pool;
}
// The caller holds `lock` (on the pool's mutex) until its kernel is enqueued: another host thread that
// launches on the same stream and needs a larger workspace waits, and its stream synchronisation then
// covers that kernel before the old buffers are freed.
SplitWorkspace& split_workspace(std::unique_lock<std::mutex>& lock, int device, hipStream_t s, size_t part_bytes, size_t tiles) {
    SplitPool& pool = split_pool();
    lock = std::unique_lock<std::mutex>(pool.mu);
    SplitWorkspace& w = pool.of_stream[std::make_pair(device, s)];
    if (w.part.bytes < part_bytes || w.tiles < tiles) {
        DeviceGuard g(device);
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        HIPIE_CHECK_HIP(hipStreamIsCapturing(s, &capturing));
        HIPIE_REQUIRE(capturing == hipStreamCaptureStatusNone, HIPIE_NOT_ALLOCATED,
                      "the split-K workspace of this stream is created by the first launch: run once before capturing");
        HIPIE_CHECK_HIP(hipStreamSynchronize(s));
        if (w.part.bytes < part_bytes) w.part.alloc(device, part_bytes);
        if (w.tiles < tiles) {
            w.count.alloc(device, tiles * sizeof(uint32_t));
            // on the launching stream: a memset on the null stream is not ordered before work on a non-blocking stream
            HIPIE_CHECK_HIP(hipMemsetAsync(w.count.ptr, 0, tiles * sizeof(uint32_t), s));
            w.tiles = tiles;
        }
    }
    return w;
}

// Scratch memory of the entry point that allocates nothing (hipie_conv_run_static): the partial sums and the
// arrival counters of the K split in a device array of fixed size instead of an allocated workspace.  Every
// device the library runs on holds its own copy until the process ends; all calls on a device share it.
constexpr size_t kStaticParts = 256;                                          // 64 KB blocks of partial sums: 16 MB
constexpr size_t kStaticPartBytes = kStaticParts * 64 * 256 * sizeof(int32_t);
constexpr size_t kStaticTiles = 1024;                                         // arrival counters
constexpr size_t kStaticScratchBytes = kStaticPartBytes + kStaticTiles * sizeof(uint32_t);
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

// The array's name is a host-side handle, not a device address: the address is asked for once per device, with
// that device current, and only that pointer is ever passed to a kernel.
struct StaticScratch {
    std::mutex mu;
    std::map<int, uint8_t*> of_device;
};
uint8_t* static_scratch(int device) {
    static auto* table = new StaticScratch();   // never destroyed, like the workspace pool
    std::lock_guard<std::mutex> lock(table->mu);
    auto it = table->of_device.find(device);
    if (it != table->of_device.end()) return it->second;
    DeviceGuard g(device);
    uint8_t* ptr = nullptr;
    HIPIE_CHECK_HIP(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
    HIPIE_REQUIRE(ptr != nullptr, HIPIE_GENERAL_ERROR, "no device address for the static scratch array on device %d", device);
    table->of_device[device] = ptr;
    return ptr;
}

// arrival counters start at zero: a fill kernel (a memset node in a captured graph gave wrong replays here)
__global__ void clear_counters_kernel(uint32_t* counters, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) counters[i] = 0u;
}

// parts of the K split of variants 14 to 17: 2, 4, 8, 16
int split_parts(int tile) { return 2 << (tile - 14); }

bool rows_kernel_fits(const hipie_conv_desc& d) {
    return d.groups == 1 && d.kh == 3 && d.kw == 3 && d.stride_h == 1 && d.stride_w == 1 && d.dil_h == 1 && d.dil_w == 1 &&
           d.pad_top == 1 && d.pad_bottom == 1 && d.pad_left == 1 && d.pad_right == 1 && d.ic % 64 == 0;
}

// output rows per tile: at most 256 pixels, and a patch of (R + 2) x (OW + 2) pixels within the LDS buffer; 0: none fits
int rows_per_tile(int oh, int ow) {
    const int r = std::min(std::min(256 / ow, kPatchRows / (ow + 2) - 2), oh);
    return r >= 1 ? r : 0;
}

// the bottleneck-tail kernel's first convolution: 3 x 3, stride 1, pad 1 over dense pixels of a multiple of 64 channels,
// 64, 128 or 256 output channels, 32-bit buffer offsets
bool block_first_fits(const hipie_conv_desc& d, int64_t Kp, int64_t OCp) {
    return rows_kernel_fits(d) && d.in_c_stride == d.ic && d.in_stride_w == d.ic && Kp == 9 * static_cast<int64_t>(d.ic) &&
           (d.oc == 64 || d.oc == 128 || d.oc == 256) && OCp * Kp < (int64_t(1) << 31);
}

// its second convolution: 1 x 1, stride 1, unpadded, over dense pixels of exactly 64, 128 or 256 channels, output
// channels a multiple of that
bool block_second_fits(const hipie_conv_desc& d, int64_t Kp, int64_t OCp) {
    return d.groups == 1 && d.kh == 1 && d.kw == 1 && d.stride_h == 1 && d.stride_w == 1 && d.pad_top == 0 && d.pad_bottom == 0 &&
           d.pad_left == 0 && d.pad_right == 0 && (d.ic == 64 || d.ic == 128 || d.ic == 256) && d.in_c_stride == d.ic &&
           d.in_stride_w == d.ic && Kp == d.ic && d.oc % d.ic == 0 && OCp * Kp < (int64_t(1) << 31);
}

// the cache-line kernels: a K step of `rb` bytes must stay inside one filter tap, and 32-bit buffer offsets
bool line_kernel_fits(const hipie_conv_desc& d, int64_t Kp, int64_t OCp, int rb) {
    return d.groups == 1 && d.in_c_stride % rb == 0 && Kp % rb == 0 && OCp * Kp < (int64_t(1) << 31);
}

// the first-layer kernel's geometry: 4-byte pixels, one 32-byte slice per filter row, undilated
bool stem_kernel_fits(const hipie_conv_desc& d) {
    return d.groups == 1 && d.in_c_stride == 4 && d.in_stride_w == 4 && d.dil_h == 1 && d.dil_w == 1 && d.kw * 4 > 16 && d.kw * 4 <= 32 &&
           d.kh <= 8 && (d.stride_w * 4) % 8 == 0;
}

void launch_stem(const ConvArgs& a, hipStream_t s) {
    const dim3 grid(a.p_tiles * a.t_tiles), block(256);
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_STEM(FLAGS, ...)                                                    \
    do {                                                                                 \
        if constexpr ((FLAGS) != kDyn && ((FLAGS) & CF_RES_GEMM)) break;                  \
        else hipLaunchKernelGGL((conv_stem_kernel<FLAGS>), grid, block, 0, s, a);        \
    } while (0)
    HIPIE_FOR_EACH_EPILOGUE(HIPIE_LAUNCH_STEM, 0)
#undef HIPIE_LAUNCH_STEM
}

void launch_rows(const ConvArgs& a, hipStream_t s) {
    const dim3 grid(a.p_tiles * a.t_tiles), block(256);
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_ROWS(FLAGS, ...)                                                    \
    do {                                                                                 \
        if constexpr ((FLAGS) != kDyn && ((FLAGS) & CF_RES_GEMM)) break;                  \
        else hipLaunchKernelGGL((conv_rows_kernel<FLAGS>), grid, block, 0, s, a);        \
    } while (0)
    HIPIE_FOR_EACH_EPILOGUE(HIPIE_LAUNCH_ROWS, 0)
#undef HIPIE_LAUNCH_ROWS
}

// the template instances of the persistent kernel: byte outputs and byte / no residual
bool persist_available(uint32_t flags) {
    switch (flags & ~CF_OUT_XOR) {
    case E_PLAIN0: case E_PLAIN: case E_RESU8: case E_CLAMPFQ: case E_SCALEFQ0: return true;
    default: return false;
    }
}

template <int WOC, int WPIX>
void launch_persist(const ConvArgs& a, hipStream_t s) {
    // two workgroups per compute unit, a whole number of them per (XCD, channel tile)
    const int n_per = std::max(1, std::min<int>(a.p_per_xcd, 512 / (8 * a.t_tiles)));
    const dim3 grid(8 * a.t_tiles * n_per), block(WOC * WPIX * 64);
    switch (a.flags & ~CF_OUT_XOR) {
    case E_PLAIN0: hipLaunchKernelGGL((conv_persist_kernel<WOC, WPIX, E_PLAIN0>), grid, block, 0, s, a, n_per); break;
    case E_PLAIN: hipLaunchKernelGGL((conv_persist_kernel<WOC, WPIX, E_PLAIN>), grid, block, 0, s, a, n_per); break;
    case E_RESU8: hipLaunchKernelGGL((conv_persist_kernel<WOC, WPIX, E_RESU8>), grid, block, 0, s, a, n_per); break;
    case E_CLAMPFQ: hipLaunchKernelGGL((conv_persist_kernel<WOC, WPIX, E_CLAMPFQ>), grid, block, 0, s, a, n_per); break;
    case E_SCALEFQ0: hipLaunchKernelGGL((conv_persist_kernel<WOC, WPIX, E_SCALEFQ0>), grid, block, 0, s, a, n_per); break;
    default: fail(HIPIE_GENERAL_ERROR, "persistent convolution kernel: no instance for epilogue %#x", a.flags);
    }
}

// the same tiles with the operands of two K steps requested together
template <int WOC, int WPIX>
void launch_tiled_pair(const ConvArgs& a, hipStream_t s, int batches = 1) {
    const dim3 grid(a.p_per_xcd > 0 ? 8 * a.p_per_xcd * a.t_tiles : a.p_tiles * a.t_tiles, batches), block(WOC * WPIX * 64);
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_PAIR(FLAGS, ...)                                                                  \
    do {                                                                                               \
        if constexpr ((FLAGS) != kDyn && ((FLAGS) & CF_RES_GEMM)) break;                                \
        else hipLaunchKernelGGL((conv_tiled_kernel<WOC, WPIX, FLAGS, true>), grid, block, 0, s, a);    \
    } while (0)
    HIPIE_FOR_EACH_EPILOGUE(HIPIE_LAUNCH_PAIR, 0)
#undef HIPIE_LAUNCH_PAIR
}

void launch_tiled_small(const ConvArgs& a, hipStream_t s) {   // 64 x 64 tile, one wave per workgroup
    const dim3 grid(a.p_per_xcd > 0 ? 8 * a.p_per_xcd * a.t_tiles : a.p_tiles * a.t_tiles), block(64);
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_SMALL(FLAGS, ...) \
    hipLaunchKernelGGL((conv_tiled_kernel<1, 1, FLAGS>), grid, block, 0, s, a)
    HIPIE_FOR_EACH_EPILOGUE(HIPIE_LAUNCH_SMALL, 0)
#undef HIPIE_LAUNCH_SMALL
}

void launch_stream(const ConvArgs& a, int grid_x, hipStream_t s) {
    const dim3 grid(grid_x, a.t_tiles), block(256);
    const size_t lds = static_cast<size_t>(64) * (a.Kp + 16) + PT_ROWS * 64 * 4;
    const uint32_t core = a.flags & ~CF_OUT_XOR;
#define HIPIE_LAUNCH_STREAM(FLAGS, ...) \
    hipLaunchKernelGGL((conv_stream_kernel<FLAGS>), grid, block, lds, s, a)
    HIPIE_FOR_EACH_EPILOGUE(HIPIE_LAUNCH_STREAM, 0)
#undef HIPIE_LAUNCH_STREAM
}

}  // namespace

void release_split_workspace(int device, hipStream_t s) {
    SplitPool& pool = split_pool();
    std::lock_guard<std::mutex> lock(pool.mu);
    pool.of_stream.erase(std::make_pair(device, s));
}

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
    case HIPIE_RESIDUAL_SHORTCUT_CONV: flags |= CF_RES | CF_RES_GEMM; break;
    default: fail(HIPIE_PARAMETER_MISMATCH, "epilogue: residual dtype %d", e.residual_dtype);
    }
    if (flags & CF_RES) {
        if (e.res_sub) { vec(e.res_sub, e.n_res_sub, 0.f, "res_sub", h); up(res_sub, h); flags |= CF_RES_SUB; }
        if (e.res_mul) { vec(e.res_mul, e.n_res_mul, 1.f, "res_mul", h); up(res_mul, h); flags |= CF_RES_MUL; }
    }
    if (e.post_scale) { vec(e.post_scale, e.n_post_scale, 1.f, "post_scale", h); up(post_scale, h); flags |= CF_POST_SCALE; }
    if (e.activation == 1) flags |= CF_RELU;
    else if (e.activation == 2) {
        HIPIE_REQUIRE(e.clamp_lo <= e.clamp_hi, HIPIE_PARAMETER_MISMATCH, "epilogue: clamp range [%g, %g]", e.clamp_lo, e.clamp_hi);
        flags |= CF_CLAMP; clamp_lo = e.clamp_lo; clamp_hi = e.clamp_hi;
    }
    else if (e.activation == 3) flags |= CF_GELU;
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
        for (int64_t c = 0; c < ocp; ++c) {
            HIPIE_REQUIRE(il[c] < ih[c], HIPIE_NOT_IMPLEMENTED,
                          "epilogue: FakeQuantize needs input_low < input_high (channel %lld)", (long long)c);
            d[c] = ih[c] - il[c];
        }
        std::vector<FqChannel> ch(ocp);
        for (int64_t c = 0; c < ocp; ++c) {
            FqChannel& p = ch[c];
            p.il = il[c]; p.ih = ih[c]; p.lo = il[c]; p.hi = ih[c]; p.d = d[c];
            p.r = r[c] = fq_rounded_reciprocal(p.d);
        }
        const bool exact = fq_reciprocal_exact_on_all(ch.data(), ocp, lm1);
        up(fq_il, il); up(fq_ih, ih); up(fq_d, d); up(fq_r, r);
        flags |= CF_OUT_FQ;
        if (exact) flags |= CF_FQ_RCP;
        std::vector<float> zh, zl;
        if (exact && device < 0) {
            flags |= CF_FQ_DIV2;   // dry run: nothing executes, plan as if the constants verify
        } else if (exact && fq_div2_constants(device, d, zh, zl)) {
            up(fq_r, zh);
            up(fq_r2, zl);
            flags |= CF_FQ_DIV2;
        }
        bool il0 = true;
        for (int64_t c = 0; c < ocp; ++c) il0 = il0 && il[c] == 0.0f && !std::signbit(il[c]);
        if (il0) flags |= CF_FQ_IL0;
        if (out_off == -128.0f) flags |= CF_OUT_XOR;
        else if (out_off != 0.0f) flags |= CF_OUT_ADD;
        if (lm1 == 255.0f) {
            flags |= CF_FQ_SAT;
            // a Clamp whose range holds every channel's FakeQuantize range changes no level: what it cuts off
            // lies in the FakeQuantize's own saturating branches (clamp.hpp maps x to the bound, which the
            // FakeQuantize maps to the same end level as any value beyond it)
            bool covered = (flags & CF_CLAMP) != 0;
            for (int64_t c = 0; covered && c < ocp; ++c) covered = clamp_lo <= il[c] && clamp_hi >= ih[c];
            if (covered) flags &= ~CF_CLAMP;
        }
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
    a.fq_d = fq_d.as<float>(); a.fq_r = fq_r.as<float>(); a.fq_r2 = fq_r2.as<float>();
    a.flags = flags; a.lm1 = lm1; a.out_off = out_off; a.clamp_lo = clamp_lo; a.clamp_hi = clamp_hi;
}

}  // namespace hipie

using namespace hipie;

// row of the packed weight matrix that holds logical channel oc: inside every group of 64 the rows
// are in MFMA order so that a lane's 16 results per tile are consecutive channels
static int64_t packed_row(int64_t oc) {
    const int64_t e = oc & 63;
    const int64_t hh = e >> 5, ob = (e >> 4) & 1, q = (e >> 2) & 3, t = e & 3;
    return (oc & ~int64_t(63)) + 32 * ob + 8 * q + 4 * hh + t;
}

// Dense convolution operand set packed for the MFMA kernels: weights [OCp][Kp] (rows in MFMA
// order), byte offset of every 16-byte K piece, per-channel integer correction.
struct PackedGemm {
    int64_t K = 0, Kp = 0, OCp = 0;
    bool linear = false;           // koff[p] == 16 p for every piece: the K bytes of a pixel's window are contiguous
    DeviceBuffer wgt, koff, corr;
    // `keep`: receives the packed matrix ([OCp][Kp], rows in MFMA order) for a second packing derived from it
    void pack(int device, const hipie_conv_desc& d, const int8_t* weights, std::vector<int8_t>* keep = nullptr);
    // A grouped convolution (weights [oc][ic / groups][kh][kw]) whose 64-channel output tiles each read one contiguous
    // span of `span` input channels: K holds the span only (taps x span bytes), and every tile has a K-offset table of
    // its own that starts at its span (koff_tile entries from one tile's table to the next)
    static bool grouped_fits(const hipie_conv_desc& d, int64_t* span);
    void pack_grouped(int device, const hipie_conv_desc& d, const int8_t* weights, int64_t span);
    int64_t koff_tile = 0;
};

struct hipie_conv {
    int device = 0;
    hipie_conv_desc d{};
    int64_t K = 0, Kp = 0, OCp = 0;
    bool k_linear = false;         // PackedGemm::linear of the main convolution
    int64_t koff_tile = 0;         // grouped convolution in its own form: entries from one 64-channel tile's K offsets to the next
    // fused shortcut convolution (second operand set + its bias / scale tables)
    bool fused = false;
    hipie_conv_desc sd{};
    PackedGemm sg;
    DeviceBuffer s_bias, s_scale;
    bool depthwise = false;
    int tile = 0;  // 0: tiled 128 ch x 128 px, 1: tiled 64 x 256, 2: tiled 64 x 64, 3: streaming (64 ch, weights
                   // in LDS), 4: pipelined 128 x 128, 5: pipelined 64 x 256
    int stages = 0;  // ring depth of the pipelined kernels (0 = choose from K)
    DeviceBuffer wgt, koff, corr;
    DeviceBuffer wgt_rows;   // depthwise 3 x 3: [kh][OCp] dwords, bytes (w[kh][0], w[kh][1], w[kh][2], 0) of a channel
    DeviceBuffer wgt_k16;    // 1 x 1 with an epilogue the few-pixel kernel evaluates: [Kp / 16][OCp] pieces of 16 K bytes
    DeviceBuffer wgt_steps;  // the bottleneck-tail kernel's packing (pack_fragments), where the layer can be one of its two
    int steps_role = 0;      // 1: its 3 x 3 layer, 2: its 1 x 1 layer, 0: neither
    bool few_pixel_ok = false;   // the layer is one the few-pixel kernel takes (also known for a host-only object)
    Epilogue epi;
};

// corr[b][n] = factor * sum_k Bt[b][n][k] + addend for the rows n < N of every batch element b (0 for the padded
// rows up to Np): a thread per row, 16 bytes a step, v_dot4_i32_i8 against four ones
__global__ __launch_bounds__(256) void row_sums_kernel(const int8_t* bt, int64_t ldb, int64_t stride_b, int64_t outer_b,
                                                       int32_t batch_inner, int32_t N, int32_t Np, int32_t K, int32_t factor,
                                                       int32_t addend, int32_t* corr, int64_t rows) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (row >= rows) return;
    const int b = static_cast<int>(row / Np), n = static_cast<int>(row - static_cast<int64_t>(b) * Np);
    int32_t sum = 0;
    if (n < N) {
        int64_t base = static_cast<int64_t>(b) * stride_b;
        if (batch_inner > 0) {
            const int o = b / batch_inner;
            base = o * outer_b + static_cast<int64_t>(b - o * batch_inner) * stride_b;
        }
        const int8_t* p = bt + base + static_cast<int64_t>(n) * ldb;
        for (int k = 0; k < K; k += 16) {
            const uint4 v = *reinterpret_cast<const uint4*>(p + k);
            sum = __builtin_amdgcn_sdot4(static_cast<int>(v.x), 0x01010101, sum, false);
            sum = __builtin_amdgcn_sdot4(static_cast<int>(v.y), 0x01010101, sum, false);
            sum = __builtin_amdgcn_sdot4(static_cast<int>(v.z), 0x01010101, sum, false);
            sum = __builtin_amdgcn_sdot4(static_cast<int>(v.w), 0x01010101, sum, false);
        }
    }
    corr[row] = n < N ? sum * factor + addend : 0;
}

static void launch_row_sums(const int8_t* bt, int64_t ldb, int64_t stride_b, int64_t outer_b, int32_t batch_inner, int32_t N,
                            int32_t Np, int32_t K, int32_t factor, int32_t addend, int32_t* corr, int32_t batches,
                            hipStream_t s) {
    const int64_t rows = static_cast<int64_t>(batches) * Np;
    hipLaunchKernelGGL(row_sums_kernel, dim3(static_cast<uint32_t>(ceil_div(rows, 256))), dim3(256), 0, s, bt, ldb, stride_b,
                       outer_b, batch_inner, N, Np, K, factor, addend, corr, rows);
}

struct hipie_matmul {
    int device = 0;
    hipie_matmul_desc d{};
    int64_t Np = 0;
    DeviceBuffer koff, corr;
    Epilogue epi;
};

// the zero point of input channel ic
static inline int zero_point_of(const hipie_conv_desc& d, int ic) { return d.in_zero_points ? d.in_zero_points[ic] : d.in_zero_point; }

namespace hipie {
namespace {
thread_local PackTape* t_tape = nullptr;
}
PackTape::Scope::Scope(PackTape* t) : previous(t_tape) { t_tape = t; }
PackTape::Scope::~Scope() { t_tape = previous; }
PackTape* PackTape::current() { return t_tape; }
bool PackTape::take(void* dst, size_t bytes) {
    if (!playing) return false;
    HIPIE_REQUIRE(next < blobs.size() && blobs[next].size() == bytes, HIPIE_NETWORK_NOT_READ,
                  "packed operands of the stream do not belong to this graph (blob %zu)", next);
    std::memcpy(dst, blobs[next].data(), bytes);
    ++next;
    return true;
}
void PackTape::give(const void* src, size_t bytes) {
    if (playing) return;
    const uint8_t* b = static_cast<const uint8_t*>(src);
    blobs.emplace_back(b, b + bytes);
}
}  // namespace hipie

bool PackedGemm::grouped_fits(const hipie_conv_desc& d, int64_t* span) {
    if (d.groups <= 1 || d.ic % d.groups || d.oc % d.groups || d.oc % 64 || d.in_c_stride % 16) return false;
    const int64_t icg = d.ic / d.groups, ocg = d.oc / d.groups;
    int64_t s = 0;
    if (64 % ocg == 0) s = (64 / ocg) * icg;          // a tile holds whole groups: their input channels, side by side
    else if (ocg % 64 == 0) s = icg;                   // a tile lies inside one group
    else return false;
    // a tile's span starts at a multiple of 16 bytes and is whole 16-byte pieces; and it must be a real part of the
    // input (a layer whose every tile reads every channel gains nothing over the dense form)
    if (s % 16 != 0 || s >= d.ic) return false;
    *span = s;
    return true;
}

void PackedGemm::pack_grouped(int device, const hipie_conv_desc& d, const int8_t* weights, int64_t span) {
    const int64_t icg = d.ic / d.groups, ocg = d.oc / d.groups, taps = static_cast<int64_t>(d.kh) * d.kw;
    K = taps * span;
    Kp = round_up(K, 64);
    OCp = round_up(d.oc, 128);
    linear = false;
    const int64_t tiles = d.oc / 64;
    koff_tile = Kp / 16;
    auto span_start = [&](int64_t tile) { return ((tile * 64) / ocg) * icg; };   // first input channel a tile reads
    std::vector<int32_t> off(static_cast<size_t>(round_up(d.oc, 128) / 64 * koff_tile), 0);   // (a padding tile reads its neighbour's span: zero weights)
    for (int64_t t = 0; t < static_cast<int64_t>(off.size()) / koff_tile; ++t)
        for (int64_t p = 0; p < K / 16; ++p) {
            const int64_t k = p * 16, tap = k / span, ic0 = k % span, kh = tap / d.kw, kw = tap % d.kw;
            off[static_cast<size_t>(t * koff_tile + p)] = static_cast<int32_t>(kh * d.dil_h * d.in_stride_h + kw * d.dil_w * d.in_stride_w +
                                                                                  span_start(std::min(t, tiles - 1)) + ic0);
        }
    std::vector<int8_t> w(static_cast<size_t>(OCp) * Kp, 0);
    std::vector<int32_t> cr(OCp, 0);
    const int stored_zero = d.in_dtype == HIPIE_U8B ? 128 : 0;
    PackTape* tape = PackTape::current();
    const bool played = tape && tape->take(w.data(), w.size()) && tape->take(cr.data(), cr.size() * sizeof(int32_t));
    if (!played) parallel_for(d.oc, [&](int64_t oc) {
        const int64_t first = (oc / ocg) * icg, base = span_start(oc / 64);   // the group's channels inside the tile's span
        int64_t corr = 0;
        for (int64_t t = 0; t < taps; ++t)
            for (int64_t i = 0; i < icg; ++i) {
                const int8_t v = weights[(oc * icg + i) * taps + t];
                w[static_cast<size_t>(packed_row(oc) * Kp + t * span + (first - base) + i)] = v;
                corr += static_cast<int64_t>(stored_zero - zero_point_of(d, static_cast<int>(first + i))) * v;
            }
        cr[oc] = static_cast<int32_t>(corr - (d.acc_sub ? d.acc_sub[oc] : 0));
    });
    if (tape && !played) {
        tape->give(w.data(), w.size());
        tape->give(cr.data(), cr.size() * sizeof(int32_t));
    }
    if (device >= 0) {
        wgt.upload(device, w.data(), w.size());
        koff.upload(device, off.data(), off.size() * sizeof(int32_t));
        corr.upload(device, cr.data(), cr.size() * sizeof(int32_t));
    }
}

void PackedGemm::pack(int device, const hipie_conv_desc& d, const int8_t* weights, std::vector<int8_t>* keep) {
    // K order (kh, kw, ic) over the padded channel stride.  A 16-byte piece must not straddle
    // two filter taps unless consecutive taps are contiguous in memory (in_stride_w == c stride).
    const bool row_contig = d.in_stride_w == d.in_c_stride && d.dil_w == 1;
    HIPIE_REQUIRE(d.in_c_stride % 16 == 0 || row_contig, HIPIE_NOT_IMPLEMENTED,
                  "convolution: channel stride %d needs a multiple of 16", d.in_c_stride);
    const int64_t cs = d.in_c_stride;
    const int64_t row_kp = round_up(d.kw * cs, 16);   // bytes of one filter row when taps are contiguous
    const bool per_row = cs % 16 != 0;                // small-channel first layer: pad every filter row
    K = per_row ? d.kh * row_kp : static_cast<int64_t>(d.kh) * d.kw * cs;
    Kp = round_up(K, 64);
    OCp = round_up(d.oc, 128);
    std::vector<int32_t> off(Kp / 16, 0);
    for (int64_t p = 0; p < K / 16; ++p) {
        const int64_t k = p * 16;
        if (per_row) {
            const int64_t kh = k / row_kp, within = k % row_kp;
            off[p] = static_cast<int32_t>(kh * d.dil_h * d.in_stride_h + within);
        } else {
            const int64_t tap = k / cs, ic0 = k % cs;
            const int64_t kh = tap / d.kw, kw = tap % d.kw;
            off[p] = static_cast<int32_t>(kh * d.dil_h * d.in_stride_h + kw * d.dil_w * d.in_stride_w + ic0);
        }
    }
    linear = true;
    for (size_t p = 0; p < off.size(); ++p) linear = linear && off[p] == static_cast<int32_t>(16 * p);
    std::vector<int8_t> w(static_cast<size_t>(OCp) * Kp, 0);
    std::vector<int32_t> cr(OCp, 0);
    const int stored_zero = d.in_dtype == HIPIE_U8B ? 128 : 0;
    PackTape* tape = PackTape::current();
    const bool played = tape && tape->take(w.data(), w.size()) && tape->take(cr.data(), cr.size() * sizeof(int32_t));
    if (!played) parallel_for(d.oc, [&](int64_t oc) {
        int64_t corr = 0;
        for (int kh = 0; kh < d.kh; ++kh)
            for (int kw = 0; kw < d.kw; ++kw)
                for (int ic = 0; ic < d.ic; ++ic) {
                    const int8_t v = weights[((oc * d.ic + ic) * d.kh + kh) * d.kw + kw];
                    const int64_t k = per_row ? kh * row_kp + kw * cs + ic
                                              : (static_cast<int64_t>(kh) * d.kw + kw) * cs + ic;
                    w[packed_row(oc) * Kp + k] = v;
                    // stored byte = level - 128 (U8B) or level (I8); the product wanted is (level - zero point) * w
                    corr += static_cast<int64_t>(stored_zero - zero_point_of(d, ic)) * v;
                }
        cr[oc] = static_cast<int32_t>(corr - (d.acc_sub ? d.acc_sub[oc] : 0));
    });
    if (tape && !played) {
        tape->give(w.data(), w.size());
        tape->give(cr.data(), cr.size() * sizeof(int32_t));
    }
    if (device >= 0) {
        wgt.upload(device, w.data(), w.size());
        koff.upload(device, off.data(), off.size() * sizeof(int32_t));
        corr.upload(device, cr.data(), cr.size() * sizeof(int32_t));
    }
    if (keep) *keep = std::move(w);
}

// The bottleneck-tail kernel's weight stream: the matrix in the order the kernel's waves use it, so that a wave's load
// instruction is 1 KB of contiguous memory that lands in matrix operand registers as it is.  A step is 64 K bytes of `cm`
// rows; inside a step come the row blocks of 64 (one per wave), inside a block the four fragments (ks, ob) - K bytes
// [32 ks, 32 ks + 32) of rows [32 ob, 32 ob + 32) - and inside a fragment lane l's 16 bytes: row l % 32, K bytes
// 16 (l / 32) onwards.  `first`: steps ordered (64-channel slab, filter tap) over all cm = OC rows of a 3 x 3 layer with
// `ic` dense input channels; else (row block of cm = K rows, slab) of a 1 x 1 layer.
static std::vector<int8_t> pack_fragments(const std::vector<int8_t>& w, int64_t Kp, bool first, int64_t cm, int64_t ic, int64_t oc) {
    const int64_t step = cm * 64;
    const int64_t slabs = first ? ic / 64 : cm / 64;
    const int64_t n_steps = first ? 9 * slabs : (oc / cm) * slabs;
    std::vector<int8_t> out(static_cast<size_t>(n_steps * step));
    parallel_for(n_steps, [&](int64_t st) {
        int64_t row0, k0;
        if (first) {
            const int64_t c = st / 9, tap = st % 9;
            row0 = 0;
            k0 = tap * ic + c * 64;
        } else {
            const int64_t pass = st / slabs, c = st % slabs;
            row0 = pass * cm;
            k0 = c * 64;
        }
        for (int64_t blk = 0; blk < cm / 64; ++blk)
            for (int64_t f = 0; f < 4; ++f)
                for (int64_t l = 0; l < 64; ++l) {
                    const int64_t ks = f >> 1, ob = f & 1;
                    std::memcpy(&out[static_cast<size_t>(st * step + ((blk * 4 + f) * 64 + l) * 16)],
                                &w[static_cast<size_t>((row0 + blk * 64 + ob * 32 + (l & 31)) * Kp + k0 + ks * 32 + (l >> 5) * 16)], 16);
                }
    });
    return out;
}

static void check_conv_desc(const hipie_conv_desc& d, const char* what) {
    HIPIE_REQUIRE(d.in_dtype == HIPIE_U8B || d.in_dtype == HIPIE_I8, HIPIE_PARAMETER_MISMATCH,
                  "%s: input dtype %d (U8B or I8 expected)", what, d.in_dtype);
    HIPIE_REQUIRE(d.ic > 0 && d.oc > 0 && d.kh > 0 && d.kw > 0 && d.stride_h > 0 && d.stride_w > 0 && d.dil_h > 0 &&
                      d.dil_w > 0 && d.pad_top >= 0 && d.pad_left >= 0 && d.pad_bottom >= 0 && d.pad_right >= 0,
                  HIPIE_PARAMETER_MISMATCH, "%s: bad geometry", what);
    HIPIE_REQUIRE(d.in_c_stride >= d.ic && d.in_c_stride % 4 == 0, HIPIE_PARAMETER_MISMATCH,
                  "%s: in_c_stride=%d must be a multiple of 4 >= ic=%d", what, d.in_c_stride, d.ic);
    const int lo = d.in_dtype == HIPIE_U8B ? 0 : -128;
    for (int ic = 0; ic < (d.in_zero_points ? d.ic : 1); ++ic)
        HIPIE_REQUIRE(zero_point_of(d, ic) >= lo && zero_point_of(d, ic) <= lo + 255, HIPIE_PARAMETER_MISMATCH,
                      "%s: zero point %d is not a level of the input type", what, zero_point_of(d, ic));
}

static void conv_out_hw(const hipie_conv_desc& d, int h, int w, int& oh, int& ow) {
    oh = (h + d.pad_top + d.pad_bottom - (d.dil_h * (d.kh - 1) + 1)) / d.stride_h + 1;
    ow = (w + d.pad_left + d.pad_right - (d.dil_w * (d.kw - 1) + 1)) / d.stride_w + 1;
}

extern "C" {

int hipie_matmul_create(int device, const hipie_matmul_desc* desc, const hipie_epilogue* epilogue,
                        hipie_matmul** out) {
    return guarded([&] {
        HIPIE_REQUIRE(desc && epilogue && out, HIPIE_PARAMETER_MISMATCH, "hipie_matmul_create: null argument");
        const hipie_matmul_desc& d = *desc;
        HIPIE_REQUIRE((d.a_dtype == HIPIE_I8 || d.a_dtype == HIPIE_U8B) && (d.b_dtype == HIPIE_I8 || d.b_dtype == HIPIE_U8B),
                      HIPIE_NOT_IMPLEMENTED, "hipie_matmul_create: operand dtypes %d, %d (i8 or u8 expected)", d.a_dtype,
                      d.b_dtype);
        HIPIE_REQUIRE(d.a_dtype == HIPIE_U8B ? (d.a_zero_point >= 0 && d.a_zero_point <= 255) : d.a_zero_point == 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_matmul_create: zero point %d of the left operand", d.a_zero_point);
        HIPIE_REQUIRE(d.b_dtype == HIPIE_U8B ? (d.b_zero_point >= 0 && d.b_zero_point <= 255) : d.b_zero_point == 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_matmul_create: zero point %d of the right operand", d.b_zero_point);
        HIPIE_REQUIRE(d.k > 0 && d.n > 0 && d.k % 64 == 0, HIPIE_NOT_IMPLEMENTED,
                      "hipie_matmul_create: K=%d must be a positive multiple of 64", d.k);
        auto m = std::make_unique<hipie_matmul>();
        m->device = device;
        m->d = d;
        m->Np = round_up(d.n, 128);
        std::vector<int32_t> koff(d.k / 16), corr(m->Np, 0);
        for (size_t p = 0; p < koff.size(); ++p) koff[p] = static_cast<int32_t>(16 * p);
        m->epi.build(device, *epilogue, d.n, m->Np);
        if (device >= 0) {
            m->koff.upload(device, koff.data(), koff.size() * sizeof(int32_t));
            m->corr.upload(device, corr.data(), corr.size() * sizeof(int32_t));
        }
        *out = m.release();
    });
}

void hipie_matmul_destroy(hipie_matmul* m) { delete m; }

int hipie_matmul_run(const hipie_matmul* mm, const void* a_ptr, int64_t lda, int64_t stride_a, const void* bt_ptr,
                     int64_t ldb, int64_t stride_b, void* out, int64_t ldo, int64_t stride_o, int32_t m,
                     int32_t batch, void* stream) {
    return hipie_matmul_run_nested(mm, a_ptr, lda, stride_a, 0, bt_ptr, ldb, stride_b, 0, out, ldo, stride_o, 0, m, batch,
                                   1, stream);
}

int hipie_matmul_run_nested(const hipie_matmul* mm, const void* a_ptr, int64_t lda, int64_t stride_a, int64_t outer_a,
                            const void* bt_ptr, int64_t ldb, int64_t stride_b, int64_t outer_b, void* out, int64_t ldo,
                            int64_t stride_o, int64_t outer_o, int32_t m, int32_t batch, int32_t batch_outer,
                            void* stream) {
    return hipie_matmul_run_nested_ws(mm, a_ptr, lda, stride_a, outer_a, bt_ptr, ldb, stride_b, outer_b, out, ldo, stride_o,
                                      outer_o, m, batch, batch_outer, nullptr, 0, stream);
}

// workspace layout: [batches][Np] sums over the right operand's rows (u8 left operand), then [batches][round_up(m, 4)]
// sums over the left operand's rows (u8 right operand)
static size_t matmul_ws_left(const hipie_matmul* mm, int64_t batches) {
    return mm->d.a_dtype == HIPIE_U8B ? static_cast<size_t>(batches * mm->Np) * sizeof(int32_t) : 0;
}
static size_t matmul_ws_right(const hipie_matmul* mm, int64_t m, int64_t batches) {
    return mm->d.b_dtype == HIPIE_U8B ? static_cast<size_t>(batches * round_up(m, 4)) * sizeof(int32_t) : 0;
}

int hipie_matmul_workspace_size(const hipie_matmul* mm, int32_t m, int32_t batch, int32_t batch_outer, size_t* bytes) {
    return guarded([&] {
        HIPIE_REQUIRE(mm && bytes && m >= 0 && batch >= 0 && batch_outer >= 0, HIPIE_PARAMETER_MISMATCH,
                      "hipie_matmul_workspace_size: argument");
        const int64_t batches = static_cast<int64_t>(batch) * batch_outer;
        *bytes = matmul_ws_left(mm, batches) + matmul_ws_right(mm, m, batches);
    });
}

int hipie_matmul_run_nested_ws(const hipie_matmul* mm, const void* a_ptr, int64_t lda, int64_t stride_a, int64_t outer_a,
                               const void* bt_ptr, int64_t ldb, int64_t stride_b, int64_t outer_b, void* out, int64_t ldo,
                               int64_t stride_o, int64_t outer_o, int32_t m, int32_t batch, int32_t batch_outer,
                               void* workspace, size_t workspace_bytes, void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(mm, HIPIE_PARAMETER_MISMATCH, "hipie_matmul_run: null handle");
        HIPIE_REQUIRE(mm->koff.ptr, HIPIE_NOT_ALLOCATED, "hipie_matmul_run: host-only object");
        if (m == 0 || batch == 0 || batch_outer == 0) return;
        HIPIE_REQUIRE(a_ptr && bt_ptr && out && m > 0 && batch > 0 && batch_outer > 0 &&
                          static_cast<int64_t>(batch) * batch_outer < 65536 && outer_a % 16 == 0 && outer_b % 16 == 0,
                      HIPIE_PARAMETER_MISMATCH,
                      "hipie_matmul_run: null operand or negative size");
        const hipie_matmul_desc& d = mm->d;
        const bool byte_out = mm->epi.out_dtype == HIPIE_U8B || mm->epi.out_dtype == HIPIE_I8;
        const int gran = byte_out ? 16 : 4;
        const int64_t n_pad = round_up(d.n, gran);
        HIPIE_REQUIRE(lda >= d.k && ldb >= d.k && lda % 16 == 0 && ldb % 16 == 0 && ldo >= n_pad && ldo % gran == 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_matmul_run: leading dimensions (lda %lld, ldb %lld, ldo %lld)",
                      (long long)lda, (long long)ldb, (long long)ldo);
        HIPIE_REQUIRE(reinterpret_cast<uintptr_t>(a_ptr) % 16 == 0 && reinterpret_cast<uintptr_t>(bt_ptr) % 16 == 0 &&
                          reinterpret_cast<uintptr_t>(out) % 16 == 0 && stride_a % 16 == 0 && stride_b % 16 == 0 &&
                          stride_o % gran == 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_matmul_run: operands must be 16-byte aligned");
        HIPIE_REQUIRE(static_cast<int64_t>(m) * lda < (1ll << 31) && m < (1 << 24), HIPIE_OUT_OF_BOUNDS,
                      "hipie_matmul_run: matrix too large for 32-bit offsets");
        HIPIE_REQUIRE(!(mm->epi.flags & CF_RES), HIPIE_NOT_IMPLEMENTED, "hipie_matmul_run: residual operand");
        ConvArgs a{};
        a.in = static_cast<const int8_t*>(a_ptr);
        a.wgt = static_cast<const int8_t*>(bt_ptr);
        a.out = out;
        a.koff = mm->koff.as<int32_t>();
        a.k_linear = 1;
        a.corr = mm->corr.as<int32_t>();
        mm->epi.fill(a);
        a.M = m;
        a.OW = 1;
        a.OHOW = m;
        a.inv_OW = 1.0f;
        a.inv_OHOW = 1.0f / static_cast<float>(m);
        a.in_sh = static_cast<int32_t>(lda);
        a.conv_sh = a.conv_sw = 1;
        a.out_sh = static_cast<int32_t>(ldo);
        a.out_sw = static_cast<int32_t>(n_pad);
        a.OC = d.n;
        a.OCp = static_cast<int32_t>(mm->Np);
        a.Kp = d.k;
        a.nk = d.k / 64;
        a.wgt_ld = static_cast<int32_t>(ldb);
        a.wgt_rows = d.n;
        a.wgt_plain = 1;
        a.batch_in = stride_a;
        a.batch_wgt = stride_b;
        a.batch_out = stride_o;
        a.batch_inner = batch_outer > 1 ? batch : 0;
        a.batch_in_o = outer_a;
        a.batch_wgt_o = outer_b;
        a.batch_out_o = outer_o;
        DeviceGuard g(mm->device);
        // Operands stored as level - 128 (u8): with a' = a - 128, b' = b - 128 the stored bytes and za, zb the levels that
        // stand for 0.0,
        //   sum_k (a_k - za)(b_k - zb) = sum_k a'_k b'_k + (128 - za) sum_k b'_k + (128 - zb) (sum_k a'_k + K (128 - za)).
        // The second term is one number per output column and batch element (sums over the right operand's rows), the
        // third one per output row (sums over the left operand's rows); both are computed on the same stream in front
        // of the product.  An i8 operand is its own a' with "128 - z" = 0.
        const int64_t batches = static_cast<int64_t>(batch) * batch_outer;
        const size_t ws_left = matmul_ws_left(mm, batches), ws_right = matmul_ws_right(mm, m, batches);
        if (ws_left + ws_right > 0)
            HIPIE_REQUIRE(workspace && workspace_bytes >= ws_left + ws_right && reinterpret_cast<uintptr_t>(workspace) % 16 == 0,
                          HIPIE_PARAMETER_MISMATCH,
                          "hipie_matmul_run: a u8 operand needs a workspace of %zu bytes (hipie_matmul_workspace_size)",
                          ws_left + ws_right);
        const int32_t fa = d.a_dtype == HIPIE_U8B ? 128 - d.a_zero_point : 0;
        const int32_t fb = d.b_dtype == HIPIE_U8B ? 128 - d.b_zero_point : 0;
        if (d.a_dtype == HIPIE_U8B) {
            launch_row_sums(static_cast<const int8_t*>(bt_ptr), ldb, stride_b, outer_b, batch_outer > 1 ? batch : 0, d.n,
                            static_cast<int32_t>(mm->Np), d.k, fa, 0, static_cast<int32_t*>(workspace),
                            batch * batch_outer, as_stream(stream));
            a.corr = static_cast<const int32_t*>(workspace);
            a.batch_corr = static_cast<int32_t>(mm->Np);
        }
        if (d.b_dtype == HIPIE_U8B) {
            int32_t* rows = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + ws_left);
            const int32_t mp = static_cast<int32_t>(round_up(m, 4));
            launch_row_sums(static_cast<const int8_t*>(a_ptr), lda, stride_a, outer_a, batch_outer > 1 ? batch : 0, m, mp,
                            d.k, fb, fb * fa * d.k, rows, batch * batch_outer, as_stream(stream));
            a.pix_corr = rows;
            a.batch_pix_corr = mp;
        }
        const bool wide = d.n > 64;
        const int boc = wide ? 128 : 64, bpix = wide ? 128 : 256;
        a.p_tiles = static_cast<int32_t>(ceil_div(m, bpix));
        a.t_tiles = static_cast<int32_t>(ceil_div(d.n, boc));
        a.t_shift = (a.t_tiles & (a.t_tiles - 1)) == 0 ? __builtin_ctz(a.t_tiles) : -1;
        a.p_per_xcd = 0;   // plain order: batches are spread over the XCDs by their launch order
        if (a.pix_corr) {
            if (wide) launch_tiled_pixc<2, 2>(a, as_stream(stream), batch * batch_outer);
            else launch_tiled_pixc<1, 4>(a, as_stream(stream), batch * batch_outer);
        } else if (wide) {
            launch_tiled<2, 2>(a, as_stream(stream), batch * batch_outer);
        } else {
            launch_tiled<1, 4>(a, as_stream(stream), batch * batch_outer);
        }
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

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
        HIPIE_REQUIRE(d.groups >= 1 && d.ic % d.groups == 0 && d.oc % d.groups == 0, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_create: groups=%d does not divide ic=%d and oc=%d", d.groups, d.ic, d.oc);
        int64_t group_span = 0;
        const bool grouped_own = d.groups > 1 && !(d.groups == d.ic && d.ic == d.oc) && PackedGemm::grouped_fits(d, &group_span);
        if (d.groups > 1 && !grouped_own && (!(d.groups == d.ic && d.ic == d.oc) || d.in_c_stride % 16 != 0)) {
            // A grouped convolution that is not depthwise (weights [oc][ic / groups][kh][kw]) is the dense convolution
            // with block-diagonal weights: reference::group_convolution (group_convolution.hpp:78-144) convolves every
            // slice on its own, and the products added here are zeros.  So is a depthwise one over pixels that are
            // not a multiple of 16 bytes (an image-like input of up to four channels), which the depthwise kernels,
            // reading 16 channels per lane, do not take.
            const int64_t icg = d.ic / d.groups, ocg = d.oc / d.groups, taps = static_cast<int64_t>(d.kh) * d.kw;
            std::vector<int8_t> dense(static_cast<size_t>(d.oc) * d.ic * taps, 0);
            for (int64_t oc = 0; oc < d.oc; ++oc)
                for (int64_t i = 0; i < icg; ++i)
                    for (int64_t t = 0; t < taps; ++t)
                        dense[static_cast<size_t>((oc * d.ic + (oc / ocg) * icg + i) * taps + t)] = weights[(oc * icg + i) * taps + t];
            hipie_conv_desc dd = d;
            dd.groups = 1;
            const int st = hipie_conv_create(device, &dd, dense.data(), epilogue, out);
            if (st != HIPIE_OK) fail(static_cast<hipie_status>(st), "%s", std::string(hipie_last_error()).c_str());
            return;
        }
        const bool depthwise = d.groups > 1 && !grouped_own;
        HIPIE_REQUIRE(d.in_c_stride >= d.ic && d.in_c_stride % 4 == 0, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_create: in_c_stride=%d must be a multiple of 4 >= ic=%d", d.in_c_stride, d.ic);
        {
            const int lo = d.in_dtype == HIPIE_U8B ? 0 : -128;
            for (int ic = 0; ic < (d.in_zero_points ? d.ic : 1); ++ic)
                HIPIE_REQUIRE(zero_point_of(d, ic) >= lo && zero_point_of(d, ic) <= lo + 255, HIPIE_PARAMETER_MISMATCH,
                              "hipie_conv_create: zero point %d is not a level of the input type", zero_point_of(d, ic));
        }
        auto c = std::make_unique<hipie_conv>();
        c->device = device;
        c->d = d;
        c->d.in_zero_points = nullptr;   // the caller's arrays are read during this call only
        c->d.acc_sub = nullptr;
        HIPIE_REQUIRE(!(depthwise && d.acc_sub), HIPIE_NOT_IMPLEMENTED, "hipie_conv_create: acc_sub on a depthwise convolution");
        if (depthwise) {
            // weights [C][kh][kw] -> [kh*kw][OCp]; corr = 128 * sum of the channel's taps
            HIPIE_REQUIRE(d.in_c_stride % 16 == 0, HIPIE_NOT_IMPLEMENTED,
                          "hipie_conv_create: depthwise needs a channel stride multiple of 16");
            c->depthwise = true;
            c->OCp = round_up(d.oc, 128);
            const int taps = d.kh * d.kw;
            std::vector<int8_t> w(static_cast<size_t>(taps) * c->OCp, 0);
            std::vector<int32_t> corr(c->OCp, 0);
            for (int ch = 0; ch < d.oc; ++ch) {
                int sum = 0;
                for (int t = 0; t < taps; ++t) {
                    w[static_cast<size_t>(t) * c->OCp + ch] = weights[ch * taps + t];
                    sum += weights[ch * taps + t];
                }
                corr[ch] = ((d.in_dtype == HIPIE_U8B ? 128 : 0) - zero_point_of(d, ch)) * sum;
            }
            c->epi.build(device, *epilogue, d.oc, c->OCp);
            std::vector<uint32_t> rows;
            if (d.kh == 3 && d.kw == 3) {
                rows.assign(static_cast<size_t>(3) * c->OCp, 0u);
                for (int ch = 0; ch < d.oc; ++ch)
                    for (int kh = 0; kh < 3; ++kh) {
                        uint32_t v = 0;
                        for (int kw = 0; kw < 3; ++kw)
                            v |= static_cast<uint32_t>(static_cast<uint8_t>(weights[ch * 9 + kh * 3 + kw])) << (8 * kw);
                        rows[static_cast<size_t>(kh) * c->OCp + ch] = v;
                    }
            }
            if (device >= 0) {
                c->wgt.upload(device, w.data(), w.size());
                c->corr.upload(device, corr.data(), corr.size() * sizeof(int32_t));
                if (!rows.empty()) c->wgt_rows.upload(device, rows.data(), rows.size() * sizeof(uint32_t));
            }
            *out = c.release();
            return;
        }
        if (grouped_own) {
            // the grouped form: tiles of 64 output channels over the K bytes of their own groups, in the tiled kernels
            // whose channel tile is 64 wide (variants 1 and 2)
            PackedGemm g;
            g.pack_grouped(device, d, weights, group_span);
            c->K = g.K; c->Kp = g.Kp; c->OCp = g.OCp;
            c->wgt = std::move(g.wgt); c->koff = std::move(g.koff); c->corr = std::move(g.corr);
            c->koff_tile = g.koff_tile;
            c->epi.build(device, *epilogue, d.oc, c->OCp);
            c->tile = 1;
            *out = c.release();
            return;
        }
        PackedGemm g;
        std::vector<int8_t> packed;
        g.pack(device, d, weights, &packed);
        c->K = g.K; c->Kp = g.Kp; c->OCp = g.OCp;
        c->wgt = std::move(g.wgt); c->koff = std::move(g.koff); c->corr = std::move(g.corr);
        c->k_linear = g.linear;
        c->epi.build(device, *epilogue, d.oc, c->OCp);
        if (block_first_fits(d, c->Kp, c->OCp)) c->steps_role = 1;
        else if (block_second_fits(d, c->Kp, c->OCp)) c->steps_role = 2;
        if (device >= 0 && c->steps_role) {
            const std::vector<int8_t> steps = pack_fragments(packed, c->Kp, c->steps_role == 1, c->steps_role == 1 ? d.oc : d.ic, d.ic, d.oc);
            c->wgt_steps.upload(device, steps.data(), steps.size());
        }
        packed.clear();
        packed.shrink_to_fit();
        c->few_pixel_ok = d.kh == 1 && d.kw == 1 && d.in_c_stride % 64 == 0 && c->Kp == d.in_c_stride && !d.acc_sub &&
                          d.stride_h == 1 && d.stride_w == 1 && d.pad_top == 0 && d.pad_left == 0 && d.pad_bottom == 0 &&
                          d.pad_right == 0 && skinny_epilogue_fits(c->epi.flags) && c->Kp * c->OCp <= (16 << 20) &&
                          c->Kp <= 7168;   // (8 pixels x Kp bytes of LDS)
        if (device >= 0 && c->few_pixel_ok) {
            // the few-pixel kernel's packing (variant 23): piece k16 of channel oc at (k16 * OCp + oc) * 16
            std::vector<int8_t> k16(static_cast<size_t>(c->Kp) * c->OCp, 0);
            parallel_for(d.oc, [&](int64_t oc) {
                for (int64_t k = 0; k < d.ic; ++k)
                    k16[static_cast<size_t>(((k >> 4) * c->OCp + oc) * 16 + (k & 15))] = weights[oc * d.ic + k];
            });
            c->wgt_k16.upload(device, k16.data(), k16.size());
        }
        // default: wide channel tiles when there are enough channels, else all waves on pixels
        // (the planner may override this after timing the candidates)
        c->tile = d.oc > 64 ? 0 : 1;
        *out = c.release();
    });
}

int hipie_conv_create_fused(int device, const hipie_conv_desc* desc, const int8_t* weights,
                            const hipie_epilogue* epilogue, const hipie_conv_desc* shortcut_desc,
                            const int8_t* shortcut_weights, const float* shortcut_bias, int64_t n_bias,
                            const float* shortcut_scale, int64_t n_scale, hipie_conv** out) {
    return guarded([&] {
        HIPIE_REQUIRE(desc && weights && epilogue && shortcut_desc && shortcut_weights && shortcut_bias &&
                          shortcut_scale && out,
                      HIPIE_PARAMETER_MISMATCH, "hipie_conv_create_fused: null argument");
        HIPIE_REQUIRE(epilogue->residual_dtype == HIPIE_RESIDUAL_SHORTCUT_CONV, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_create_fused: the epilogue's residual must be HIPIE_RESIDUAL_SHORTCUT_CONV");
        const hipie_conv_desc& sd = *shortcut_desc;
        check_conv_desc(sd, "hipie_conv_create_fused (shortcut)");
        HIPIE_REQUIRE(sd.groups == 1 && desc->groups == 1 && sd.oc == desc->oc, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_create_fused: both convolutions must be dense with the same output channels");
        for (int64_t n : {n_bias, n_scale})
            HIPIE_REQUIRE(n == 1 || n == sd.oc, HIPIE_PARAMETER_MISMATCH, "hipie_conv_create_fused: table length");
        hipie_conv* c = nullptr;
        const int st = hipie_conv_create(device, desc, weights, epilogue, &c);
        if (st != HIPIE_OK) fail(static_cast<hipie_status>(st), "%s", hipie_last_error());
        std::unique_ptr<hipie_conv> guard(c);
        HIPIE_REQUIRE((c->epi.flags & ~(CF_OUT_XOR | CF_FQ_DIV2)) == (E_RESGEMM & ~CF_FQ_DIV2), HIPIE_NOT_IMPLEMENTED,
                      "hipie_conv_create_fused: the fused form needs bias, scale, FakeQuantize with input_low 0");
        c->fused = true;
        c->sd = sd;
        c->sd.in_zero_points = nullptr;
        c->sd.acc_sub = nullptr;
        c->sg.pack(device, sd, shortcut_weights);
        std::vector<float> b(c->OCp, 0.f), s(c->OCp, 1.f);
        for (int oc = 0; oc < sd.oc; ++oc) {
            b[oc] = shortcut_bias[n_bias == 1 ? 0 : oc];
            s[oc] = shortcut_scale[n_scale == 1 ? 0 : oc];
        }
        if (device >= 0) {
            c->s_bias.upload(device, b.data(), b.size() * sizeof(float));
            c->s_scale.upload(device, s.data(), s.size() * sizeof(float));
        }
        c->tile = 0;
        *out = guard.release();
    });
}

void hipie_conv_destroy(hipie_conv* c) { delete c; }

int hipie_conv_set_tile(hipie_conv* c, int tile) {
    return guarded([&] {
        HIPIE_REQUIRE(c && tile >= 0 && tile <= 24, HIPIE_PARAMETER_MISMATCH, "hipie_conv_set_tile: tile=%d", tile);
        if (c->depthwise) {   // 0: registers only, 1: 3 x 3 through an LDS patch, 2: 3 x 3 on the matrix pipe
            const hipie_conv_desc& dd = c->d;
            const bool matrix_ok = dd.kh == 3 && dd.kw == 3 && dd.dil_h == 1 && dd.dil_w == 1 && dd.stride_h == dd.stride_w &&
                                   (dd.stride_h == 1 || dd.stride_h == 2) && dd.pad_top == 1 && dd.pad_left == 1 &&
                                   block_dw_epilogue_fits(c->epi.flags);
            HIPIE_REQUIRE(tile == 0 || (tile == 1 && !(c->epi.flags & CF_RES) &&
                                        dwconv_strip_fits(c->d.kh, c->d.kw, c->d.dil_h, c->d.dil_w, c->d.stride_h, c->d.stride_w,
                                                          c->d.in_c_stride, static_cast<int>(c->OCp), c->epi.flags)) ||
                              (tile == 2 && matrix_ok),
                          HIPIE_PARAMETER_MISMATCH, "hipie_conv_set_tile: depthwise variant %d does not take this layer", tile);
            c->tile = tile;
            return;
        }
        if (c->koff_tile) {   // a grouped convolution in its own form: the tiled kernels with 64-channel tiles
            HIPIE_REQUIRE(tile == 1 || tile == 2, HIPIE_PARAMETER_MISMATCH,
                          "hipie_conv_set_tile: a grouped convolution runs in the tiled kernels with 64-channel tiles (variants 1, 2)");
            c->tile = tile;
            return;
        }
        if (c->fused && tile != 0) return;      // the second GEMM exists in the 128 x 128 tiled kernel
        HIPIE_REQUIRE(tile < 8 || tile > 9 || (!c->fused && persist_available(c->epi.flags)), HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: the persistent kernels exist for byte outputs with a byte residual or none");
        HIPIE_REQUIRE(tile < 6 || tile > 7 || (c->Kp / 64) % 2 == 0, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: the split-K kernels need an even number of 64-byte K steps (K=%lld)", (long long)c->Kp);
        HIPIE_REQUIRE(tile < 18 || tile > 22 || line_kernel_fits(c->d, c->Kp, c->OCp, line_row_bytes(tile - 18)), HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: the cache-line kernels need a channel stride (%d) and K (%lld) that are multiples of their %d-byte K step",
                      c->d.in_c_stride, (long long)c->Kp, line_row_bytes(tile - 18));
        HIPIE_REQUIRE(tile < 14 || tile > 17 || c->Kp / 64 >= 2 * split_parts(tile), HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: the K split over workgroups needs two 64-byte K steps per part (K=%lld)", (long long)c->Kp);
        HIPIE_REQUIRE(tile != 13 || stem_kernel_fits(c->d), HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: the first-layer kernel takes 4-byte pixels and filter rows of 5 to 8 taps, undilated");
        HIPIE_REQUIRE(tile != 12 || rows_kernel_fits(c->d), HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: the row-tile kernel takes 3 x 3, stride 1, pad 1, undilated convolutions over a multiple of 64 input channels");
        HIPIE_REQUIRE(tile != 23 || c->few_pixel_ok, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: the few-pixel kernel takes unpadded 1 x 1 convolutions over pixels of a multiple of 64 "
                      "bytes with raw sums or a bias / scale / ReLU tail to f32");
        HIPIE_REQUIRE(tile != 24 || (!c->fused && c->steps_role == 1 && block_epilogues_fit(c->epi.flags, false, 0)),
                      HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: the patch-staged kernel takes 3 x 3, stride 1, pad 1 convolutions over a multiple of 64 dense "
                      "input channels with 64, 128 or 256 output channels, bias and a 256-level FakeQuantize from 0");
        HIPIE_REQUIRE(tile != 3 || 64 * (c->Kp + 16) + PT_ROWS * 64 * 4 <= 160 * 1024, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_set_tile: K=%lld does not fit the streaming kernel's LDS", (long long)c->Kp);
        c->tile = tile;
    });
}

int hipie_conv_get_tile(const hipie_conv* c, int* tile) {
    return guarded([&] {
        HIPIE_REQUIRE(c && tile, HIPIE_PARAMETER_MISMATCH, "hipie_conv_get_tile: null argument");
        *tile = c->tile;
    });
}

int hipie_conv_epilogue_flags(const hipie_conv* c, uint32_t* flags, int* specialised) {
    return guarded([&] {
        HIPIE_REQUIRE(c && flags && specialised, HIPIE_PARAMETER_MISMATCH, "hipie_conv_epilogue_flags: null argument");
        *flags = c->epi.flags;
        const uint32_t core = c->epi.flags & ~CF_OUT_XOR;
        bool generic = false;
#define HIPIE_IS_GENERIC(FLAGS, ...) generic = (FLAGS) == kDyn
        HIPIE_FOR_EACH_EPILOGUE(HIPIE_IS_GENERIC, 0)
#undef HIPIE_IS_GENERIC
        *specialised = generic ? 0 : 1;
    });
}

int hipie_conv_set_stages(hipie_conv* c, int stages) {
    return guarded([&] {
        HIPIE_REQUIRE(c && stages >= 0 && stages <= 8, HIPIE_PARAMETER_MISMATCH, "hipie_conv_set_stages: %d", stages);
        c->stages = stages;
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

// Checks the tensors of one launch against the layer and fills the kernel arguments every variant shares; returns the
// number of output pixels (0: nothing to do)
static int64_t fill_conv_args(const hipie_conv* c, const hipie_tensor* in, const hipie_tensor* residual,
                              const hipie_tensor* out, ConvArgs& a, int32_t& oh, int32_t& ow) {
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
    if (M == 0) return 0;
    const int64_t in_span = static_cast<int64_t>(in->n) * in->stride_n;
    HIPIE_REQUIRE(in_span < (1ll << 31) && M < (1ll << 24), HIPIE_OUT_OF_BOUNDS,
                  "hipie_conv_run: tensor too large (32-bit byte offsets, < 2^24 output pixels)");
    a = ConvArgs{};
    a.in = static_cast<const int8_t*>(in->data);
    a.wgt = c->wgt.as<int8_t>();
    a.wgt2 = c->wgt_rows.as<int8_t>();   // depthwise only; a fused shortcut overwrites it below
    a.out = out->data;
    a.koff = c->koff.as<int32_t>();
    a.k_linear = c->k_linear ? 1 : 0;
    a.koff_tile = static_cast<int32_t>(c->koff_tile);
    a.corr = c->corr.as<int32_t>();
    c->epi.fill(a);
    if (a.flags & CF_RES_GEMM) {
        // `residual` is the INPUT of the fused shortcut convolution
        HIPIE_REQUIRE(c->fused && residual && residual->data, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_run: shortcut input missing");
        const hipie_conv_desc& sd = c->sd;
        HIPIE_REQUIRE(residual->dtype == sd.in_dtype && residual->c == sd.ic && residual->n == in->n &&
                          residual->stride_w == sd.in_stride_w && residual->stride_h == sd.in_stride_h,
                      HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: shortcut input does not match its packing");
        int soh, sow;
        conv_out_hw(sd, residual->h, residual->w, soh, sow);
        HIPIE_REQUIRE(soh == oh && sow == ow, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_run: shortcut convolution yields %dx%d, main %dx%d", soh, sow, oh, ow);
        HIPIE_REQUIRE(residual->halo >= std::max(std::max(sd.pad_top, sd.pad_bottom), std::max(sd.pad_left, sd.pad_right)),
                      HIPIE_PARAMETER_MISMATCH, "hipie_conv_run: shortcut input halo");
        HIPIE_REQUIRE(static_cast<int64_t>(residual->n) * residual->stride_n < (1ll << 31), HIPIE_OUT_OF_BOUNDS,
                      "hipie_conv_run: shortcut tensor too large");
        a.in2 = static_cast<const int8_t*>(residual->data);
        a.wgt2 = c->sg.wgt.as<int8_t>();
        a.koff2 = c->sg.koff.as<int32_t>();
        a.k_linear2 = c->sg.linear ? 1 : 0;
        a.corr2 = c->sg.corr.as<int32_t>();
        a.bias2 = c->s_bias.as<float>();
        a.scale2 = c->s_scale.as<float>();
        a.in2_sn = static_cast<int32_t>(residual->stride_n);
        a.in2_sh = static_cast<int32_t>(residual->stride_h);
        a.in2_sw = static_cast<int32_t>(residual->stride_w);
        a.conv2_sh = sd.stride_h;
        a.conv2_sw = sd.stride_w;
        a.in2_origin = -(sd.pad_top * a.in2_sh + sd.pad_left * a.in2_sw);
        a.Kp2 = static_cast<int32_t>(c->sg.Kp);
        a.nk2 = static_cast<int32_t>(c->sg.Kp / 64);
    } else if (a.flags & CF_RES) {
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
    a.inv_OW = 1.0f / static_cast<float>(ow);
    a.inv_OHOW = 1.0f / static_cast<float>(oh * ow);
    a.in_sn = static_cast<int32_t>(in->stride_n);
    a.in_sh = static_cast<int32_t>(in->stride_h);
    a.in_sw = static_cast<int32_t>(in->stride_w);
    a.conv_sh = d.stride_h;
    a.conv_sw = d.stride_w;
    a.in_origin = -(d.pad_top * a.in_sh + d.pad_left * a.in_sw);
    a.out_sn = static_cast<int32_t>(out->stride_n);
    a.out_sh = static_cast<int32_t>(out->stride_h);
    a.out_sw = static_cast<int32_t>(out->stride_w);
    // tensors that are dense in (n, h, w) for this convolution: pixel m sits at m * pixel stride
    a.flat_in = static_cast<int64_t>(d.stride_h) * a.in_sh == static_cast<int64_t>(ow) * d.stride_w * a.in_sw &&
                a.in_sn == static_cast<int64_t>(oh) * ow * d.stride_w * a.in_sw;
    a.flat_out = a.out_sh == static_cast<int64_t>(ow) * a.out_sw && a.out_sn == static_cast<int64_t>(oh) * ow * a.out_sw;
    a.flat_res = a.res != nullptr && a.res_sh == static_cast<int64_t>(ow) * a.res_sw &&
                 a.res_sn == static_cast<int64_t>(oh) * ow * a.res_sw;
    a.OC = d.oc;
    a.OCp = static_cast<int32_t>(c->OCp);
    a.Kp = static_cast<int32_t>(c->Kp);
    a.nk = static_cast<int32_t>(c->Kp / 64);
    a.wgt_ld = a.Kp;
    a.wgt_rows = static_cast<int32_t>(c->OCp);
    a.wgt_plain = 0;
    return M;
}

static int conv_run(const hipie_conv* c, const hipie_tensor* in, const hipie_tensor* residual,
                    const hipie_tensor* out, void* stream, bool static_scratch_only) {
    return guarded([&] {
        ConvArgs a;
        int32_t oh, ow;
        const int64_t M = fill_conv_args(c, in, residual, out, a, oh, ow);
        if (M == 0) return;
        const hipie_conv_desc& d = c->d;
        if (c->depthwise) {
            HIPIE_REQUIRE(in->stride_w >= d.ic && in->stride_w % 16 == 0, HIPIE_PARAMETER_MISMATCH,
                          "hipie_conv_run: depthwise input channel stride");
            DeviceGuard g(c->device);
            if (c->tile == 2) {
                // the matrix-pipe form reads a border of one pixel around the tensor; an output too wide for its tile, or a
                // tensor without that border, runs the general kernel
                const BlockGeometry bg = block_dw_geometry(oh, ow, d.stride_h);
                if (bg.ok && in->halo >= 1 && (oh - 1) * d.stride_h + 1 <= in->h && (ow - 1) * d.stride_w + 1 <= in->w) {
                    launch_block_dw(a, bg, in->n, as_stream(stream));
                    HIPIE_CHECK_HIP(hipGetLastError());
                    return;
                }
            }
            const DwGeometry geo{in->h, in->w, in->halo, d.pad_top, d.pad_left};
            launch_dwconv(a, d.kh, d.kw, d.dil_h, d.dil_w, c->tile == 2 ? 0 : c->tile, geo, as_stream(stream));
            HIPIE_CHECK_HIP(hipGetLastError());
            return;
        }
        int tile = c->tile;
        if (tile == 13) {
            // R whole output rows per tile (R divides OH): at most 256 pixels, the patch within its LDS buffer,
            // and every byte the patch reads inside the tensor's halo
            const int patch_w = (ow - 1) * d.stride_w + 8;
            int R = 0;
            for (int r = std::min(oh, 256 / std::max(ow, 1)); r >= 1 && R == 0; --r)
                if (oh % r == 0 && ((r - 1) * d.stride_h + d.kh) * patch_w * 4 + 16 <= kStemPatch) R = r;
            const bool inside = in->halo >= d.pad_top && in->halo >= d.pad_left &&
                                (oh - 1) * d.stride_h - d.pad_top + d.kh - 1 <= in->h - 1 + in->halo &&
                                (ow - 1) * d.stride_w - d.pad_left + 7 <= in->w - 1 + in->halo;
            if (R == 0 || !inside || ow > 256) {
                tile = 1;                     // the general kernel
            } else {
                a.rows_per_tile = R;
                a.tiles_per_image = oh / R;
                a.patch_w = patch_w;
                a.inv_patch_w = 1.0f / static_cast<float>(patch_w);
                a.stem_kh = d.kh;
                a.stem_patch_rows = (R - 1) * d.stride_h + d.kh;
                a.stem_pad_top = d.pad_top;
                a.stem_pad_left = d.pad_left;
                a.p_tiles = in->n * a.tiles_per_image;
                a.t_tiles = static_cast<int32_t>(ceil_div(d.oc, 64));
                a.t_shift = (a.t_tiles & (a.t_tiles - 1)) == 0 ? __builtin_ctz(a.t_tiles) : -1;
                DeviceGuard g(c->device);
                launch_stem(a, as_stream(stream));
                HIPIE_CHECK_HIP(hipGetLastError());
                return;
            }
        }
        if (tile == 12) {
            const int R = rows_per_tile(oh, ow);
            if (R == 0 || in->halo < 1) {
                tile = 0;                     // rows too wide for a patch: the general kernel
            } else {
                a.rows_per_tile = R;
                a.tiles_per_image = static_cast<int32_t>(ceil_div(oh, R));
                a.patch_w = ow + 2;
                a.inv_patch_w = 1.0f / static_cast<float>(ow + 2);
                a.p_tiles = in->n * a.tiles_per_image;
                a.t_tiles = static_cast<int32_t>(ceil_div(d.oc, 64));
                a.t_shift = (a.t_tiles & (a.t_tiles - 1)) == 0 ? __builtin_ctz(a.t_tiles) : -1;
                DeviceGuard g(c->device);
                launch_rows(a, as_stream(stream));
                HIPIE_CHECK_HIP(hipGetLastError());
                return;
            }
        }
        if (tile == 24) {
            const BlockGeometry geo = block_geometry(d.oc, d.ic, oh, ow);
            if (!geo.ok || in->halo < 1) {
                tile = 0;                     // rows too wide for a tile: the general kernel
            } else {
                DeviceGuard g(c->device);
                a.wgt = c->wgt_steps.as<int8_t>();
                launch_block(a, nullptr, geo, in->n, c->stages >= 6 ? 1 : 0, as_stream(stream));
                HIPIE_CHECK_HIP(hipGetLastError());
                return;
            }
        }
        const bool square = tile == 0 || tile == 4 || tile == 6 || tile == 8 || tile == 10 || tile >= 14;
        const int boc = square ? 128 : 64;
        const int bpix = square ? 128 : (tile == 2 ? 64 : 256);
        a.p_tiles = static_cast<int32_t>(ceil_div(M, bpix));
        a.t_tiles = static_cast<int32_t>(ceil_div(d.oc, boc));
        a.t_shift = (a.t_tiles & (a.t_tiles - 1)) == 0 ? __builtin_ctz(a.t_tiles) : -1;
        // XCD-aware tile order (neighbouring pixel tiles share an L2) once every XCD gets at least two
        // pixel tiles; below that the plain order, which spreads what few tiles there are over all XCDs
        const bool xcd_order = a.p_tiles >= 16 || tile == 3 || tile == 8 || tile == 9;
        a.p_per_xcd = xcd_order ? static_cast<int32_t>(ceil_div(a.p_tiles, 8)) : 0;
        DeviceGuard g(c->device);
        hipStream_t s = as_stream(stream);
        // ring depth: enough K steps in flight to cover the load latency, within 160 KB of LDS
        const int stage_bytes = (square ? 256 : 320) * 64 * (tile == 6 || tile == 7 ? 2 : 1);
        // ring depth: 3, 4, 6 or 8 K steps (the depths the kernel has loops for), within 160 KB of LDS
        const int max_stages = (144 * 1024) / stage_bytes;
        int stages = c->stages > 0 ? c->stages : (tile == 4 || tile >= 14 ? 4 : 3);
        stages = stages >= 8 && max_stages >= 8 ? 8 : (stages >= 6 && max_stages >= 6 ? 6 : (stages >= 4 && max_stages >= 4 ? 4 : 3));
        // the K split pays where a launch has fewer tiles than the device has compute units; with many tiles
        // (more than 2048 workgroups, a 128 MB workspace) the plain pipelined kernel runs instead
        if (tile >= 14 && tile <= 17 && static_cast<int64_t>(a.p_tiles) * a.t_tiles * split_parts(tile) > 2048) tile = 4;
        std::unique_lock<std::mutex> workspace_lock;   // held across the launch below
        if (tile >= 14 && tile <= 17) {
            a.ksplit = split_parts(tile);
            const size_t tiles = static_cast<size_t>(a.p_tiles) * a.t_tiles;
            if (static_scratch_only) {
                // the device's fixed array instead of an allocated workspace: nothing is allocated, larger launches are refused
                HIPIE_REQUIRE(tiles * a.ksplit <= kStaticParts && tiles <= kStaticTiles, HIPIE_OUT_OF_BOUNDS,
                              "hipie_conv_run_static: %zu tiles x %d parts need %zu KB of partial sums, the static scratch holds %zu KB "
                              "(use hipie_conv_run, which allocates its workspace)",
                              tiles, a.ksplit, tiles * a.ksplit * 64, kStaticParts * 64);
                uint8_t* const base = static_scratch(c->device);
                a.ws_part = reinterpret_cast<int32_t*>(base);
                a.ws_count = reinterpret_cast<uint32_t*>(base + kStaticPartBytes);
                // the array keeps what the last call left (a launch that was cut short could have left counters behind)
                hipLaunchKernelGGL(clear_counters_kernel, dim3(static_cast<uint32_t>(ceil_div(tiles, 256))), dim3(256), 0, s,
                                   a.ws_count, static_cast<int>(tiles));
            } else {
                SplitWorkspace& w = split_workspace(workspace_lock, c->device, s, tiles * a.ksplit * 64 * 256 * sizeof(int32_t), tiles);
                a.ws_part = w.part.as<int32_t>();
                a.ws_count = w.count.as<uint32_t>();
            }
        }
        switch (tile) {
        case 23:
            a.wgt2 = c->wgt_k16.as<int8_t>();
            launch_skinny(a, s);
            break;
        case 18: case 19: case 20: case 21: case 22: launch_line(a, tile - 18, s); break;
        case 14:
        case 15:
        case 16:
        case 17:
        case 4: launch_pipe<2, 2, 1>(a, stages, s); break;
        case 5: launch_pipe<1, 4, 1>(a, stages, s); break;
        case 8: launch_persist<2, 2>(a, s); break;
        case 9: launch_persist<1, 4>(a, s); break;
        case 6: launch_pipe<2, 2, 2>(a, stages, s); break;
        case 7: launch_pipe<1, 4, 2>(a, stages, s); break;
        case 0: launch_tiled<2, 2>(a, s); break;
        case 1: launch_tiled<1, 4>(a, s); break;
        case 2: launch_tiled_small(a, s); break;
        case 10: launch_tiled_pair<2, 2>(a, s); break;
        case 11: launch_tiled_pair<1, 4>(a, s); break;
        default: {
            // persistent workgroups: as many as fit per CU by LDS (at most 4), spread over the
            // channel tiles; a multiple of 8 so that sibling channel tiles share an XCD
            const int64_t lds = 64 * (c->Kp + 16) + PT_ROWS * 64 * 4;
            const int per_cu = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(4, (160 * 1024) / lds)));
            int64_t gx = std::max<int64_t>(8, (256 * per_cu) / a.t_tiles);
            gx = std::min<int64_t>(round_up(gx, 8), round_up(a.p_tiles, 8));
            launch_stream(a, static_cast<int>(gx), s);
            break;
        }
        }
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_conv_run(const hipie_conv* c, const hipie_tensor* in, const hipie_tensor* residual,
                   const hipie_tensor* out, void* stream) {
    return conv_run(c, in, residual, out, stream, false);
}

int hipie_conv_pair_fits(const hipie_conv* first, const hipie_conv* second, int32_t h, int32_t w, int* fits) {
    return guarded([&] {
        HIPIE_REQUIRE(first && second && fits, HIPIE_PARAMETER_MISMATCH, "hipie_conv_pair_fits: null argument");
        const hipie_conv_desc& da = first->d;
        const hipie_conv_desc& db = second->d;
        *fits = 0;
        if (first->depthwise || second->depthwise || first->fused || second->fused) return;
        if (first->steps_role != 1 || second->steps_role != 2 || db.ic != da.oc || db.in_dtype != first->epi.out_dtype) return;
        if (!block_epilogues_fit(first->epi.flags, true, second->epi.flags)) return;
        int oh, ow;
        conv_out_hw(da, h, w, oh, ow);
        const BlockGeometry geo = block_geometry(da.oc, da.ic, oh, ow);
        // bit 0: the pair runs as one kernel; bit 1: also in the form with two wave groups (hipie_conv_set_stages 7)
        *fits = geo.ok ? (1 | ((geo.ok2 && db.oc / da.oc >= 2) ? 2 : 0)) : 0;
    });
}

int hipie_conv_run_pair(const hipie_conv* first, const hipie_conv* second, const hipie_tensor* in, const hipie_tensor* residual,
                        const hipie_tensor* out, void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(first && second && in && out, HIPIE_PARAMETER_MISMATCH, "hipie_conv_run_pair: null argument");
        int fits = 0;
        const int st = hipie_conv_pair_fits(first, second, in->h, in->w, &fits);
        if (st != HIPIE_OK) fail(static_cast<hipie_status>(st), "%s", std::string(hipie_last_error()).c_str());
        HIPIE_REQUIRE(fits && in->halo >= 1, HIPIE_PARAMETER_MISMATCH,
                      "hipie_conv_run_pair: the fused kernel takes a 3 x 3, stride 1, pad 1 convolution (bias, FakeQuantize) over dense "
                      "pixels with 64, 128 or 256 output channels followed by a 1 x 1 convolution over exactly those channels with a "
                      "byte residual (ask hipie_conv_pair_fits first)");
        HIPIE_REQUIRE(first->device == second->device, HIPIE_PARAMETER_MISMATCH, "hipie_conv_run_pair: layers of two devices");
        // the intermediate tensor exists in LDS only: a descriptor of the shape the second layer was packed for,
        // whose bytes nobody touches
        hipie_tensor mid = *out;
        mid.dtype = first->epi.out_dtype;
        mid.c = first->d.oc;
        mid.stride_w = second->d.in_stride_w;
        mid.stride_h = second->d.in_stride_h;
        mid.stride_n = static_cast<int64_t>(out->h) * mid.stride_h;
        mid.halo = 0;
        ConvArgs a, b;
        int32_t oh, ow, oh2, ow2;
        const int64_t M = fill_conv_args(first, in, nullptr, &mid, a, oh, ow);
        if (M == 0) return;
        (void)fill_conv_args(second, &mid, residual, out, b, oh2, ow2);
        const BlockGeometry geo = block_geometry(first->d.oc, first->d.ic, oh, ow);
        a.wgt = first->wgt_steps.as<int8_t>();
        b.wgt = second->wgt_steps.as<int8_t>();
        DeviceGuard g(first->device);
        launch_block(a, &b, geo, in->n, first->stages == 7 ? 2 : (first->stages >= 6 ? 1 : 0), as_stream(stream));
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

int hipie_conv_run_static(const hipie_conv* c, const hipie_tensor* in, const hipie_tensor* residual,
                          const hipie_tensor* out, void* stream) {
    return conv_run(c, in, residual, out, stream, true);
}

}  // extern "C"
