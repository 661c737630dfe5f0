// Self-attention core of a post-LPT encoder in one kernel:
//     scores = MatMul'(q, k^T) * s1 [+ mask] -> Softmax -> FakeQuantize (i8) -> MatMul'(., v) * s2 [-> FakeQuantize]
// (mat_mul.cpp:81-171 leaves the two TypeRelaxed MatMuls with their dequantization Multiply; softmax.hpp,
// fake_quantize.hpp).  The f32 scores and probabilities of one encoder layer are 2 x 113 MB at
// batch 16 x 12 heads x 384^2; here they never leave the registers.
//
// One workgroup (4 waves) takes 128 queries of one (sequence, head); a wave takes 32 of them against
// all S keys.  Keys are the rows of the first MFMA operand and queries its columns, so a lane ends up
// with S / 2 scores of ONE query (column l % 32; rows 8 (r / 4) + 4 (l / 32) + r % 4 of every 32-key
// tile): the softmax reductions are a loop over the lane's registers plus one exchange with lane
// l ^ 32.  The requantised probabilities of a tile, packed in register order, are already the second
// MFMA's column operand for "32 keys in the order (r, l / 32)"; V is transposed into LDS in exactly
// that key order, so the probabilities go from the accumulators of the first product into the
// second without touching memory.  Integer sums are exact, every f32 step is one IEEE operation in
// the graph's order; Softmax has tolerance parity like the stand-alone kernel.
#include "conv_epilogue.h"
#include "div2.h"
#include "requant.h"

namespace hipie {
namespace {

constexpr int kMaxSeq = 384;   // S / 2 accumulator registers per lane
constexpr int kHeadDim = 64;

struct AttentionArgs {
    const int8_t *q, *k, *v;
    int64_t ldq, sq, oq, ldk, sk, ok, ldv, sv, ov;   // row pitch, inner / outer batch stride (bytes)
    void* out;
    int64_t ldo, so, oo;                              // elements
    const float* mask;                                // optional additive mask row [S] per batch element, or null
    int64_t mask_inner, mask_outer;                   // its batch strides (elements)
    float* scores;                                    // optional [batch][S][S] dumps (inspection), or null
    float* probs;
    int S, batch_inner;
    float scale1, scale2;
    Requant fq_p, fq_o;                               // fq_o.levels == 0: f32 output
    float p_zh, p_zl;                                 // probabilities: two-operation division by fq_p.p.d
    int p_div2;                                       // ... verified against IEEE division on the device
    int p_sat;                                        // input_low of the probabilities' FakeQuantize is +0 and it has 256 levels
    int p_inside;                                     // ... or input_low <= 0 and input_high >= 1: a probability never leaves the interval
    int qblocks;                                      // blocks of 128 queries per batch element
    int xcd_groups;                                   // 1: a one-dimensional grid that keeps the blocks of two neighbouring batch elements on one XCD
#ifdef HIPIE_ATT_STAMPS
    long long* stamps;                                // probe builds only: cycle stamps per workgroup
#endif
    uint32_t p_xor, p_add;                            // stored byte = level + out_low (mod 256): XOR 0x80 per byte, or bytewise add
    int p_bias;                                       // 128 when the probabilities are u8 levels (stored as level - 128), else 0
};

// level index k of four probabilities as four unsigned bytes (rounded to nearest-even and packed by
// v_cvt_pk_u8_f32), then the output offset applied bytewise
// PFORM 2: input_low is +0 and there are 256 levels - a probability is never below input_low, and the packing
// conversion's saturation at 255 is the branch for values above input_high: no clamp, no subtraction.
// PFORM 1: input_low <= 0 and input_high >= 1 - a probability (0 <= e / sum <= 1: the largest e is 2^0 and counted in
// the sum) takes neither of the reference's saturating branches: no clamp.  PFORM 0: any interval.
template <bool DIV2, int PFORM>
__device__ __forceinline__ uint32_t prob_levels4(const AttentionArgs& a, float p0, float p1, float p2, float p3) {
    const FqChannel& c = a.fq_p.p;
    constexpr int M = DIV2 ? 2 : 1;
    constexpr bool IL0 = PFORM == 2, NOCLAMP = PFORM != 0;
    uint32_t w = 0;
    w = __builtin_amdgcn_cvt_pk_u8_f32(fq_level_fast<M, IL0, NOCLAMP>(p0, c.il, c.ih, c.d, DIV2 ? a.p_zh : c.r, a.p_zl, a.fq_p.lm1), 0, w);
    w = __builtin_amdgcn_cvt_pk_u8_f32(fq_level_fast<M, IL0, NOCLAMP>(p1, c.il, c.ih, c.d, DIV2 ? a.p_zh : c.r, a.p_zl, a.fq_p.lm1), 1, w);
    w = __builtin_amdgcn_cvt_pk_u8_f32(fq_level_fast<M, IL0, NOCLAMP>(p2, c.il, c.ih, c.d, DIV2 ? a.p_zh : c.r, a.p_zl, a.fq_p.lm1), 2, w);
    w = __builtin_amdgcn_cvt_pk_u8_f32(fq_level_fast<M, IL0, NOCLAMP>(p3, c.il, c.ih, c.d, DIV2 ? a.p_zh : c.r, a.p_zl, a.fq_p.lm1), 3, w);
    return a.p_add ? add_bytes(w, a.p_add) : (w ^ a.p_xor);
}

template <int NT, bool DIV2, bool MASK, int PFORM>   // NT = S / 32 key tiles
__global__ __launch_bounds__(256, 2) void attention_kernel(const AttentionArgs a) {
    constexpr int S = NT * 32;
    constexpr int VT_LD = S + 16;                     // odd number of 16-byte groups per row: conflict-free
    __shared__ __attribute__((aligned(16))) int8_t sK[S * 64];       // [key][d], chunk c of row r in slot c ^ ((r >> 2) & 3)
    __shared__ __attribute__((aligned(16))) int8_t sVT[64 * VT_LD];  // [d][tile][half][j]: key 32 t + 8 (j / 4) + 4 half + j % 4
    __shared__ __attribute__((aligned(16))) float sMask[MASK ? S : 4];    // the sequence's mask row
    // u8 probabilities q are multiplied as q - 128: sum_k q_k v_k = sum_k (q_k - 128) v_k + 128 sum_k v_k, and the
    // sums of V over the keys, one per d, start the accumulators of the second product
    __shared__ __attribute__((aligned(16))) int32_t sVsum[64];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    // Which queries of which batch element: plain (x = query block, y = batch element), or - consecutive workgroups go
    // to consecutive XCDs, each with its own L2 - the blocks of a pair of neighbouring heads on one XCD: they stage the
    // same K and V rows, and two neighbouring heads' 64-byte rows share the 128-byte lines of a [tokens, 3 hidden] tensor
    int qblk = blockIdx.x, b = blockIdx.y;
    if (a.xcd_groups) {
        const int id = blockIdx.x, per = 2 * a.qblocks, k = id >> 3, sub = k % per;
        b = ((k / per) * 8 + (id & 7)) * 2 + sub / a.qblocks;
        qblk = sub % a.qblocks;
    }
    const int bo = b / a.batch_inner, bi = b - bo * a.batch_inner;
#ifdef HIPIE_ATT_STAMPS
#define ATT_STAMP(i) do { if (a.stamps && tid == 0) a.stamps[(b * a.qblocks + qblk) * 8 + (i)] = clock64(); } while (0)
#else
#define ATT_STAMP(i)
#endif
    ATT_STAMP(0);
    const int8_t* qp = a.q + bo * a.oq + bi * a.sq;
#ifdef HIPIE_ATT_NOSTAGE   // timing probe: every workgroup stages the same K and V (wrong results, no memory traffic to speak of)
    const int8_t* kp = a.k;
    const int8_t* vp = a.v;
#else
    const int8_t* kp = a.k + bo * a.ok + bi * a.sk;
    const int8_t* vp = a.v + bo * a.ov + bi * a.sv;
#endif

    // ---- K into LDS (rows of 64 bytes), V transposed into LDS ------------------------------------
    // Every load of the staging is requested before the first is used: a round trip to memory in all, where a loop of
    // load-and-store iterations pays one per iteration (a third of the kernel's time at S = 384).
    constexpr int KI = (S * 4 + 255) / 256;           // 16-byte pieces of K per thread; and groups of 4 keys x 4 d of V
    v4i kx[KI];
    uint32_t vw[KI][4];
#pragma unroll
    for (int j = 0; j < KI; ++j) {
        const int i = min(tid + j * 256, S * 4 - 1);
        kx[j] = *reinterpret_cast<const v4i*>(kp + (i >> 2) * a.ldk + (i & 3) * 16);
    }
#pragma unroll
    for (int j = 0; j < KI; ++j) {
        const int i = min(tid + j * 256, S * 4 - 1);
        const int d4 = i & 15, kq = i >> 4;            // 4 consecutive keys x 4 consecutive d
#pragma unroll
        for (int q = 0; q < 4; ++q) vw[j][q] = *reinterpret_cast<const uint32_t*>(vp + (4 * kq + q) * a.ldv + 4 * d4);
    }
    // ---- this wave's queries: the column operand of the first product, straight from memory ------
    const int q_row = qblk * 128 + wave * 32 + l32;
    const bool q_ok = q_row < a.S;
    const int8_t* qrow = qp + static_cast<int64_t>(q_ok ? q_row : a.S - 1) * a.ldq;
    const v4i qf[2] = {*reinterpret_cast<const v4i*>(qrow + 16 * h), *reinterpret_cast<const v4i*>(qrow + 32 + 16 * h)};
    if (a.p_bias) {
        if (tid < 64) sVsum[tid] = 0;
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < KI; ++j) {
        const int i = tid + j * 256;
        if (i < S * 4) {
            const int r = i >> 2, c = i & 3;
            *reinterpret_cast<v4i*>(&sK[r * 64 + ((c ^ ((r >> 2) & 3)) * 16)]) = kx[j];
        }
    }
    int32_t vsum[4] = {0, 0, 0, 0};                     // this thread's share of the sums (d4 = tid % 16 in every round)
#pragma unroll
    for (int j = 0; j < KI; ++j) {
        const int i = tid + j * 256;
        if (i >= S * 4) continue;
        const int d4 = i & 15, kq = i >> 4;
        const uint32_t* w = vw[j];
        // 4 x 4 byte transpose: t[e] = bytes e of w[0..3]
        const uint32_t lo01 = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u);   // w0.b0 w1.b0 w0.b1 w1.b1
        const uint32_t hi01 = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);   // w0.b2 w1.b2 w0.b3 w1.b3
        const uint32_t lo23 = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u);
        const uint32_t hi23 = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
        const uint32_t t[4] = {__builtin_amdgcn_perm(lo23, lo01, 0x05040100u), __builtin_amdgcn_perm(lo23, lo01, 0x07060302u),
                               __builtin_amdgcn_perm(hi23, hi01, 0x05040100u), __builtin_amdgcn_perm(hi23, hi01, 0x07060302u)};
        const int key = 4 * kq, tile = key >> 5, in = key & 31;               // in = 8 a + 4 half
        const int col = tile * 32 + ((in >> 2) & 1) * 16 + (in >> 3) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            *reinterpret_cast<uint32_t*>(&sVT[(4 * d4 + e) * VT_LD + col]) = t[e];
            vsum[e] = __builtin_amdgcn_sdot4(static_cast<int>(t[e]), 0x01010101, vsum[e], false);
        }
    }
    if (a.p_bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e) atomicAdd(&sVsum[4 * (tid & 15) + e], vsum[e]);
    }

    if constexpr (MASK) {
        const float* mrow = a.mask + bo * a.mask_outer + bi * a.mask_inner;
        for (int i = tid; i < S; i += 256) sMask[i] = mrow[i];
    }

    ATT_STAMP(1);
    __syncthreads();
    ATT_STAMP(2);

    const int slot[2] = {((0 + h) ^ ((l32 >> 2) & 3)) * 16, ((2 + h) ^ ((l32 >> 2) & 3)) * 16};
    v16i ctx[2] = {{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}};
    const int64_t dump_row = (static_cast<int64_t>(b) * a.S + q_row) * a.S;   // [batch][query][key]
    constexpr float kLog2e = 1.4426950408889634f;
    auto init_ctx = [&]() {
        if (a.p_bias) {     // register r of block db holds d = 32 db + 8 (r / 4) + 4 h + r % 4
#pragma unroll
            for (int db = 0; db < 2; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const v4i sv = *reinterpret_cast<const v4i*>(&sVsum[32 * db + 8 * g + 4 * h]);
#pragma unroll
                    for (int j = 0; j < 4; ++j) ctx[db][4 * g + j] = sv[j] * a.p_bias;
                }
        }
    };
    // the integer scores of key tile t, and from them the f32 scores (Multiply by the scale, then the mask's Add)
    auto raw_scores = [&](int t) {
        v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const v4i kf = *reinterpret_cast<const v4i*>(&sK[(32 * t + l32) * 64 + slot[ks]]);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf, qf[ks], acc, 0, 0, 0);
        }
        return acc;
    };
    auto f32_scores = [&](int t, const v16i& acc, float (&v)[16]) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float mv[4] = {0.f, 0.f, 0.f, 0.f};
            if constexpr (MASK) {
                const float4 mk = *reinterpret_cast<const float4*>(&sMask[32 * t + 8 * g + 4 * h]);
                mv[0] = mk.x; mv[1] = mk.y; mv[2] = mk.z; mv[3] = mk.w;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float x = static_cast<float>(acc[4 * g + j]) * a.scale1;
                if constexpr (MASK) x = x + mv[j];       // the mask Add between the Multiply and the Softmax
                v[4 * g + j] = x;
            }
        }
    };
    // probabilities of a tile -> levels -> second product
    auto finish_tile = [&](int t, const float (&e)[16], float inv) {
        v4i pf;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 p4 = make_float4(e[4 * g] * inv, e[4 * g + 1] * inv, e[4 * g + 2] * inv, e[4 * g + 3] * inv);
            if (a.probs && q_ok)
                *reinterpret_cast<float4*>(a.probs + dump_row + 32 * t + 8 * g + 4 * h) = p4;
            pf[g] = static_cast<int>(prob_levels4<DIV2, PFORM>(a, p4.x, p4.y, p4.z, p4.w));
        }
#pragma unroll
        for (int db = 0; db < 2; ++db) {
            const v4i vf = *reinterpret_cast<const v4i*>(&sVT[(32 * db + l32) * VT_LD + 32 * t + 16 * h]);
            ctx[db] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf, pf, ctx[db], 0, 0, 0);
        }
    };
    float x[NT][16];
    float m = -INFINITY;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        f32_scores(t, raw_scores(t), x[t]);
#pragma unroll
        for (int r = 0; r < 16; ++r) m = fmaxf(m, x[t][r]);
        if constexpr (MASK) __builtin_amdgcn_sched_barrier(0);   // keep the mask reads next to their tile
    }
    if (a.scores && q_ok) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) a.scores[dump_row + 32 * t + 8 * (r >> 2) + 4 * h + (r & 3)] = x[t][r];
    }
    // Softmax over the keys of this lane's query (softmax.hpp: subtract the maximum, exp, sum, divide).
    // exp(x - m) as 2^((x - m) log2 e) on the hardware's exp2, the division as a multiplication by the
    // reciprocal of the sum: within the tolerance the stand-alone kernel is held to.
    m = fmaxf(m, __shfl_xor(m, 32, 64));
    const float mL = -m * kLog2e;
    float s = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            x[t][r] = __builtin_amdgcn_exp2f(fmaf(x[t][r], kLog2e, mL));
            s += x[t][r];
        }
    s += __shfl_xor(s, 32, 64);
    const float inv = 1.0f / s;
    // probabilities -> i8 levels -> second product, one 32-key tile at a time
    init_ctx();
#pragma unroll
    for (int t = 0; t < NT; ++t) finish_tile(t, x[t], inv);

    ATT_STAMP(5);
    // ---- context of query q_row: d = 32 db + 8 (r / 4) + 4 h + r % 4 --------------------------------
    if (!q_ok) return;
    const int64_t orow = bo * a.oo + bi * a.so + static_cast<int64_t>(q_row) * a.ldo;
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d = 32 * db + 8 * g + 4 * h;
            const float4 o = make_float4(static_cast<float>(ctx[db][4 * g]) * a.scale2, static_cast<float>(ctx[db][4 * g + 1]) * a.scale2,
                                         static_cast<float>(ctx[db][4 * g + 2]) * a.scale2, static_cast<float>(ctx[db][4 * g + 3]) * a.scale2);
            if (a.fq_o.levels) *reinterpret_cast<uint32_t*>(static_cast<int8_t*>(a.out) + orow + d) = requant4(a.fq_o, o);
            else *reinterpret_cast<float4*>(static_cast<float*>(a.out) + orow + d) = o;
        }
}

template <int NT>
void launch(const AttentionArgs& a_in, int batches, hipStream_t s) {
    AttentionArgs a = a_in;
    a.qblocks = static_cast<int>(ceil_div(a.S, 128));
    a.xcd_groups = batches % 16 == 0 ? 1 : 0;         // pairs of batch elements, eight pairs at a time
    const dim3 grid = a.xcd_groups ? dim3(static_cast<uint32_t>(a.qblocks) * batches) : dim3(a.qblocks, static_cast<uint32_t>(batches));
    // (the forms without clamp: compiled for the usual division only)
    const int pform = !a.p_div2 ? 0 : (a.p_sat ? 2 : (a.p_inside ? 1 : 0));
    const int form = (a.mask ? 8 : 0) + (a.p_div2 ? 4 : 0) + pform;
#define HIPIE_ATT_LAUNCH(D, M, P) hipLaunchKernelGGL((attention_kernel<NT, D, M, P>), grid, dim3(256), 0, s, a)
    switch (form) {
    case 0: HIPIE_ATT_LAUNCH(false, false, 0); break;
    case 4: HIPIE_ATT_LAUNCH(true, false, 0); break;
    case 5: HIPIE_ATT_LAUNCH(true, false, 1); break;
    case 6: HIPIE_ATT_LAUNCH(true, false, 2); break;
    case 8: HIPIE_ATT_LAUNCH(false, true, 0); break;
    case 12: HIPIE_ATT_LAUNCH(true, true, 0); break;
    case 13: HIPIE_ATT_LAUNCH(true, true, 1); break;
    default: HIPIE_ATT_LAUNCH(true, true, 2); break;
    }
#undef HIPIE_ATT_LAUNCH
}

}  // namespace
}  // namespace hipie

using namespace hipie;

#ifdef HIPIE_ATT_STAMPS
static long long* g_att_stamps = nullptr;
extern "C" void hipie_debug_attention_stamps(long long* p) { g_att_stamps = p; }
#endif

struct hipie_attention {
    int device = 0;
    hipie_attention_desc d{};
    AttentionArgs proto{};   // everything but the operands
};

extern "C" {

int hipie_attention_supported(int32_t seq, int32_t head_dim) {
    return seq > 0 && seq % 32 == 0 && seq <= kMaxSeq && head_dim == kHeadDim;
}

int hipie_attention_create(int device, const hipie_attention_desc* desc, hipie_attention** out) {
    return guarded([&] {
        HIPIE_REQUIRE(desc && out, HIPIE_PARAMETER_MISMATCH, "hipie_attention_create: null argument");
        HIPIE_REQUIRE(hipie_attention_supported(desc->seq, desc->head_dim), HIPIE_NOT_IMPLEMENTED,
                      "hipie_attention_create: sequence length %d (multiple of 32 up to %d) / head dimension %d (%d)", desc->seq,
                      kMaxSeq, desc->head_dim, kHeadDim);
        HIPIE_REQUIRE(desc->out_dtype == HIPIE_I8 || desc->out_dtype == HIPIE_F32, HIPIE_PARAMETER_MISMATCH,
                      "hipie_attention_create: output type %d", desc->out_dtype);
        HIPIE_REQUIRE(desc->prob_dtype == 0 || desc->prob_dtype == HIPIE_I8 || desc->prob_dtype == HIPIE_U8B, HIPIE_PARAMETER_MISMATCH,
                      "hipie_attention_create: probabilities of type %d", desc->prob_dtype);
        auto att = std::make_unique<hipie_attention>();
        att->device = device;
        att->d = *desc;
        AttentionArgs& a = att->proto;
        a.S = desc->seq;
        a.scale1 = desc->score_scale;
        a.scale2 = desc->context_scale;

        a.fq_p = make_requant(&desc->prob_fq, "hipie_attention_create (probabilities)");
        if (desc->out_dtype == HIPIE_I8) a.fq_o = make_requant(&desc->out_fq, "hipie_attention_create (output)");
        // the probabilities' level index: two-operation division when the device confirms it against IEEE
        // division for this divisor, else the reciprocal sequence when the host proved it on every level
        // boundary; a divisor that has neither is left to the separate kernels
        std::vector<float> zh, zl;
        a.p_div2 = fq_div2_constants(device, std::vector<float>(1, a.fq_p.p.d), zh, zl) ? 1 : 0;
        if (a.p_div2) { a.p_zh = zh[0]; a.p_zl = zl[0]; }
        HIPIE_REQUIRE(a.p_div2 || a.fq_p.rcp || device < 0, HIPIE_NOT_IMPLEMENTED,
                      "hipie_attention_create: no exact fast division for the probabilities' FakeQuantize range");
        a.p_sat = a.fq_p.p.il == 0.f && !std::signbit(a.fq_p.p.il) && a.fq_p.lm1 == 255.f;
        a.p_inside = a.fq_p.p.il <= 0.f && a.fq_p.p.ih >= 1.f;
        a.p_bias = desc->prob_dtype == HIPIE_U8B ? 128 : 0;
        const int off = static_cast<int>(a.fq_p.p.ol) & 0xff;
        a.p_xor = off == 0x80 ? 0x80808080u : 0u;
        a.p_add = (off == 0x80 || off == 0) ? 0u : static_cast<uint32_t>(off) * 0x01010101u;
        *out = att.release();
    });
}

void hipie_attention_destroy(hipie_attention* att) { delete att; }

int hipie_attention_run(const hipie_attention* att, const void* q, int64_t ldq, int64_t stride_q, int64_t outer_q,
                        const void* k, int64_t ldk, int64_t stride_k, int64_t outer_k, const void* v, int64_t ldv,
                        int64_t stride_v, int64_t outer_v, void* out, int64_t ldo, int64_t stride_o, int64_t outer_o,
                        int32_t batch, int32_t batch_outer, const float* mask, int64_t mask_stride, int64_t mask_outer,
                        float* scores, float* probs, void* stream) {
    return guarded([&] {
        HIPIE_REQUIRE(att && q && k && v && out, HIPIE_PARAMETER_MISMATCH, "hipie_attention_run: null argument");
        HIPIE_REQUIRE(reinterpret_cast<uintptr_t>(mask) % 16 == 0 && mask_stride % 4 == 0 && mask_outer % 4 == 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_attention_run: mask rows must be 16-byte aligned");
        HIPIE_REQUIRE(att->device >= 0, HIPIE_NOT_ALLOCATED, "hipie_attention_run: host-only object");
        if (batch == 0 || batch_outer == 0) return;
        HIPIE_REQUIRE(batch > 0 && batch_outer > 0 && static_cast<int64_t>(batch) * batch_outer < 65536, HIPIE_PARAMETER_MISMATCH,
                      "hipie_attention_run: batch %d x %d", batch, batch_outer);
        auto aligned = [](const void* p, int64_t a, int64_t b, int64_t c, int64_t g) {
            return reinterpret_cast<uintptr_t>(p) % g == 0 && a % g == 0 && b % g == 0 && c % g == 0;
        };
        HIPIE_REQUIRE(ldq >= kHeadDim && ldk >= kHeadDim && ldv >= kHeadDim && ldo >= kHeadDim && aligned(q, ldq, stride_q, outer_q, 16) &&
                          aligned(k, ldk, stride_k, outer_k, 16) && aligned(v, ldv, stride_v, outer_v, 4) &&
                          aligned(out, ldo, stride_o, outer_o, 4) && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                          reinterpret_cast<uintptr_t>(probs) % 16 == 0,
                      HIPIE_PARAMETER_MISMATCH, "hipie_attention_run: pitches and strides must keep 16-byte rows aligned");
        AttentionArgs a = att->proto;
        a.q = static_cast<const int8_t*>(q); a.k = static_cast<const int8_t*>(k); a.v = static_cast<const int8_t*>(v);
        a.ldq = ldq; a.sq = stride_q; a.oq = outer_q;
        a.ldk = ldk; a.sk = stride_k; a.ok = outer_k;
        a.ldv = ldv; a.sv = stride_v; a.ov = outer_v;
        a.out = out; a.ldo = ldo; a.so = stride_o; a.oo = outer_o;
        a.scores = scores; a.probs = probs;
        a.mask = mask; a.mask_inner = mask_stride; a.mask_outer = mask_outer;
        a.batch_inner = batch;
#ifdef HIPIE_ATT_STAMPS
        a.stamps = g_att_stamps;
#endif
        DeviceGuard dg(att->device);
        hipStream_t s = as_stream(stream);
        const int batches = batch * batch_outer;
        switch (a.S / 32) {
        case 1: launch<1>(a, batches, s); break;
        case 2: launch<2>(a, batches, s); break;
        case 3: launch<3>(a, batches, s); break;
        case 4: launch<4>(a, batches, s); break;
        case 5: launch<5>(a, batches, s); break;
        case 6: launch<6>(a, batches, s); break;
        case 7: launch<7>(a, batches, s); break;
        case 8: launch<8>(a, batches, s); break;
        case 9: launch<9>(a, batches, s); break;
        case 10: launch<10>(a, batches, s); break;
        case 11: launch<11>(a, batches, s); break;
        default: launch<12>(a, batches, s); break;
        }
        HIPIE_CHECK_HIP(hipGetLastError());
    });
}

}  // extern "C"
