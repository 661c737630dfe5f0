// Device-side pieces shared by the MFMA convolution kernels and the depthwise kernel: pixel
// decode, accumulator initialisation and the fused f32 epilogue.  A lane always owns 32
// consecutive output channels (oc_lane ...) of two pixels, held as acc[ob][pb][r] = channel
// oc_lane + 16*ob + r of pixel pb.
#pragma once
#include "conv_kernel.h"
#include "gelu.h"
#include "fq_math.h"

namespace hipie {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// m -> (m / d, m % d) for m < 2^24 through a float reciprocal (exact after one correction step)
__device__ __forceinline__ void fast_divmod(int m, int d, float inv_d, int& q, int& r) {
    q = static_cast<int>(static_cast<float>(m) * inv_d);
    r = m - q * d;
    // branch-free correction by one in either direction (selects, no divergent flow)
    const int lo = r < 0 ? 1 : 0, hi = r >= d ? 1 : 0;
    q += hi - lo;
    r += (lo - hi) * d;
}

// y -> (y / t_tiles, y % t_tiles) of a workgroup index: shifts when the channel tile count is a power of two
__device__ __forceinline__ void split_tile_index(const ConvArgs& a, int y, int& p_local, int& t_tile) {
    if (a.t_shift >= 0) {
        p_local = y >> a.t_shift;
        t_tile = y & (a.t_tiles - 1);
    } else {
        p_local = y / a.t_tiles;
        t_tile = y - p_local * a.t_tiles;
    }
}

struct PixelCoord { int n, oh, ow; };

// offset of batch element `batch` for an operand with inner stride `stride` and outer stride `outer`
__device__ __forceinline__ int64_t batch_offset(const ConvArgs& a, int batch, int64_t stride, int64_t outer) {
    if (a.batch_inner <= 0) return batch * stride;
    const int o = batch / a.batch_inner;
    return o * outer + (batch - o * a.batch_inner) * stride;
}

__device__ __forceinline__ PixelCoord decode_pixel(const ConvArgs& a, int m) {
    PixelCoord p;
    int rem;
    fast_divmod(m, a.OHOW, a.inv_OHOW, p.n, rem);
    fast_divmod(rem, a.OW, a.inv_OW, p.oh, p.ow);
    return p;
}

// offset of output pixel m's window origin (padding not counted) in a tensor with strides sn, sh, sw under
// convolution strides csh, csw; `flat`: the offset is linear in m (uniform flag computed on the host)
__device__ __forceinline__ int window_offset(const ConvArgs& a, int m, int sn, int sh, int sw, int csh, int csw, bool flat) {
    if (flat) return m * (csw * sw);
    const PixelCoord p = decode_pixel(a, m);
    return p.n * sn + p.oh * csh * sh + p.ow * csw * sw;
}

__device__ __forceinline__ float4 ld4f(const float* p) { return *reinterpret_cast<const float4*>(p); }

// Four consecutive dwords of a table no kernel writes, at an address every lane of the wave shares: read through the
// constant address space, so that the load is a scalar one (one request per wave, waited for on the scalar / LDS counter).
// As an ordinary global load behind a barrier the compiler issues it as a vector load - every lane asks - and waits for
// it with vmcnt(0), i.e. for every vector load of the wave that is still on its way, in front of the loads that need it.
__device__ __forceinline__ int4 load_uniform_int4(const int32_t* p) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef int dwords4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(4))) const dwords4 constant_dwords4;
    const dwords4 v = *reinterpret_cast<constant_dwords4*>(reinterpret_cast<uintptr_t>(p));
    return make_int4(v.x, v.y, v.z, v.w);
#else
    return *reinterpret_cast<const int4*>(p);
#endif
}

// A thread's piece (0 .. 3) of four such values, taken with masks: written as a chain of selects on scalar registers
// it becomes divergent branches, each with a scalar load and a wait of its own.
struct PiecePick {
    int32_t m0, m1, m2, m3;
    __device__ __forceinline__ explicit PiecePick(int piece)
        : m0(piece == 0 ? -1 : 0), m1(piece == 1 ? -1 : 0), m2(piece == 2 ? -1 : 0), m3(piece == 3 ? -1 : 0) {}
    __device__ __forceinline__ int32_t operator()(const int4& v) const { return (v.x & m0) | (v.y & m1) | (v.z & m2) | (v.w & m3); }
};

// Accumulators start from the per-channel integer correction, so the epilogue begins with the
// exact u8 x i8 sum.  acc[ob][pb][r] = channel oc_lane + 16*ob + r of pixel pb.
__device__ __forceinline__ void init_acc(const ConvArgs& a, int oc_lane, v16i (&acc)[2][2]) {
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int4 c = *reinterpret_cast<const int4*>(a.corr + oc_lane + 16 * ob + 4 * q);
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) {
                acc[ob][pb][4 * q + 0] = c.x;
                acc[ob][pb][4 * q + 1] = c.y;
                acc[ob][pb][4 * q + 2] = c.z;
                acc[ob][pb][4 * q + 3] = c.w;
            }
        }
}

// level index of one value; the clamp folds both saturating branches of the reference
// MODE 0: IEEE division, 1: reciprocal with two correction rounds, 2: fma(n, r, n * r2)
// SAT (256 levels only): no clamp.  x <= il gives n <= 0 and a product <= 0, x > ih gives n > d, a quotient
// >= 1 (every form of the division is the correctly rounded one, which is monotone) and a product >= 255:
// the packing conversion saturates both to the levels 0 and 255 the reference's branches name.
template <int MODE, bool IL0, bool SAT = false>
__device__ __forceinline__ float fq_level_fast(float x, float il, float ih, float d, float r, float r2, float lm1) {
    const float xc = SAT ? x : __builtin_amdgcn_fmed3f(x, il, ih);
    const float n = IL0 ? xc : xc - il;
    float q;
    if (MODE == 2) {
        const float lo = n * r2;
        q = fmaf(n, r, lo);
    } else if (MODE == 1) {
        const float q0 = n * r;
        const float e0 = fmaf(-d, q0, n);
        const float q1 = fmaf(e0, r, q0);
        const float e1 = fmaf(-d, q1, n);
        q = fmaf(e1, r, q1);
    } else {
        q = n / d;
    }
    return q * lm1;   // rounded to nearest-even by the packing conversion
}

// bytewise (a + b) mod 256 on four packed bytes
__device__ __forceinline__ uint32_t add_bytes(uint32_t a, uint32_t b) {
    return ((a & 0x7f7f7f7fu) + (b & 0x7f7f7f7fu)) ^ ((a ^ b) & 0x80808080u);
}

// ---- fused epilogue ---------------------------------------------------------------------------
// One lane owns 32 consecutive channels (oc_lane ...) of two pixels.  The step list is a flag
// word; the hot combinations are instantiated with the flags as a template constant so that
// unused steps vanish, kDyn reads them from the kernel arguments.  Per-channel constants are
// fetched one group of four channels ahead of their use, and each group's results are pinned
// with an empty asm: otherwise the compiler sinks the arithmetic into the store predicates and
// hoists every table load of the epilogue to its top, which costs an occupancy step.
constexpr uint32_t kDyn = 0xffffffffu;
constexpr uint32_t E_FQ = CF_OUT_FQ | CF_FQ_RCP | CF_FQ_DIV2 | CF_FQ_SAT;   // 256 levels, the division every verified layer uses
constexpr uint32_t E_PLAIN0 = CF_BIAS | E_FQ | CF_FQ_IL0;
constexpr uint32_t E_PLAIN = CF_BIAS | E_FQ;
constexpr uint32_t E_RESU8 = CF_BIAS | CF_SCALE | CF_RES | CF_RES_U8B | CF_RES_MUL | E_FQ | CF_FQ_IL0;
constexpr uint32_t E_RESF32 = CF_BIAS | CF_SCALE | CF_RES | CF_RES_F32 | E_FQ | CF_FQ_IL0;
constexpr uint32_t E_RESGEMM = CF_BIAS | CF_SCALE | CF_RES | CF_RES_GEMM | E_FQ | CF_FQ_IL0;
constexpr uint32_t E_F32 = CF_BIAS | CF_SCALE;
constexpr uint32_t E_SCALE = CF_SCALE;
constexpr uint32_t E_RESI8 = CF_BIAS | CF_SCALE | CF_RES | CF_RES_MUL | E_FQ;   // linear bottleneck + i8 residual (MobileNetV2)
constexpr uint32_t E_SCALEFQ = CF_BIAS | CF_SCALE | E_FQ;              // linear layer requantised to symmetric i8
constexpr uint32_t E_F32RES = CF_BIAS | CF_SCALE | CF_RES | CF_RES_F32;   // linear layer + f32 residual, f32 out                      // MatMul' -> Multiply(s_a * s_b)
constexpr uint32_t E_F32RELU = CF_BIAS | CF_SCALE | CF_RELU;
constexpr uint32_t E_GELUFQ = CF_BIAS | CF_SCALE | CF_GELU | E_FQ;       // FFN up projection: Gelu and the next FakeQuantize in the GEMM
constexpr uint32_t E_DEQFQ = CF_SCALE | E_FQ;                           // MatMul between activations, requantised (attention context)
constexpr uint32_t E_CLAMPFQ = CF_BIAS | CF_SCALE | CF_CLAMP | E_FQ | CF_FQ_IL0;
constexpr uint32_t E_SCALEFQ0 = CF_BIAS | CF_SCALE | E_FQ | CF_FQ_IL0;   // the same behind a Clamp that holds the FakeQuantize's range (ReLU6 -> FQ(0, 6))

// Per-channel tables of the epilogue staged in LDS, one row of `stride` floats per table.  Every
// lane of a half-wave needs the same four channels at a time: read from global memory that is a
// 64-lane vector load whose address processing costs as much as a real gather (the convolution
// kernels spent most of their texture-addresser cycles there); read from LDS it is a broadcast.
typedef const __attribute__((address_space(3))) float* lds_cfloat_ptr;   // keeps ds_read (a generic pointer makes them FLAT loads)
typedef __attribute__((address_space(3))) float* lds_float_ptr;

enum ParamTable { PT_BIAS, PT_SCALE, PT_RSUB, PT_RMUL, PT_POST, PT_IL, PT_IH, PT_D, PT_R, PT_R2, PT_COUNT };
constexpr int PT_ROWS = PT_COUNT + 1;   // plus the row of integer accumulator corrections

// Two phases so that the caller can put its operand loads between them: the table loads must not
// be awaited (for the LDS writes) before the first K step has been requested.
struct StagedParams {
    float v[PT_COUNT];
    int32_t corr;
};

template <uint32_t F>
__device__ __forceinline__ void stage_params_load(const ConvArgs& a, int oc0, int stride, int tid, StagedParams& r,
                                                  int64_t corr_shift = 0) {
    const uint32_t fl = F == kDyn ? a.flags : F;
    const int c = oc0 + (tid < stride ? tid : 0);
    auto get = [&](int t, const float* src) { r.v[t] = src[c]; };
    r.corr = a.corr[corr_shift + c];
    if (fl & CF_BIAS) get(PT_BIAS, a.bias);
    if (fl & CF_SCALE) get(PT_SCALE, a.scale);
    if (fl & CF_RES_SUB) get(PT_RSUB, a.res_sub);
    if (fl & CF_RES_MUL) get(PT_RMUL, a.res_mul);
    if (fl & CF_POST_SCALE) get(PT_POST, a.post_scale);
    if (fl & CF_OUT_FQ) {
        get(PT_IH, a.fq_ih);
        if (fl & CF_FQ_RCP) get(PT_R, a.fq_r);
        if (fl & CF_FQ_DIV2) get(PT_R2, a.fq_r2);
        if (!(fl & CF_FQ_IL0)) {
            get(PT_IL, a.fq_il);
            get(PT_D, a.fq_d);
        }
    }
}

// rows PT_BIAS .. PT_R2 of `stride` floats, then one row of the integer accumulator corrections
template <uint32_t F>
__device__ __forceinline__ void stage_params_store(const ConvArgs& a, lds_float_ptr sp, int stride, int tid,
                                                   const StagedParams& r) {
    const uint32_t fl = F == kDyn ? a.flags : F;
    if (tid >= stride) return;
    auto put = [&](int t) { sp[t * stride + tid] = r.v[t]; };
    ((__attribute__((address_space(3))) int32_t*)sp)[PT_COUNT * stride + tid] = r.corr;
    if (fl & CF_BIAS) put(PT_BIAS);
    if (fl & CF_SCALE) put(PT_SCALE);
    if (fl & CF_RES_SUB) put(PT_RSUB);
    if (fl & CF_RES_MUL) put(PT_RMUL);
    if (fl & CF_POST_SCALE) put(PT_POST);
    if (fl & CF_OUT_FQ) {
        put(PT_IH);
        if (fl & CF_FQ_RCP) put(PT_R);
        if (fl & CF_FQ_DIV2) put(PT_R2);
        if (!(fl & CF_FQ_IL0)) {
            put(PT_IL);
            put(PT_D);
        }
    }
}

// single-phase form (threads tid, tid + nt, ... of a workgroup of nt threads)
template <uint32_t F>
__device__ __forceinline__ void stage_params(const ConvArgs& a, int oc0, lds_float_ptr sp, int stride, int tid, int nt) {
    for (int t0 = 0; t0 < stride; t0 += nt) {
        StagedParams r;
        const int t = t0 + tid;
        if (t < stride) {   // uniform for all but the last round
            stage_params_load<F>(a, oc0 + t0, stride - t0, tid, r);
            // rows are indexed by the channel inside the tile
            lds_float_ptr base = sp + t0;
            const uint32_t fl = F == kDyn ? a.flags : F;
            auto put = [&](int tb) { base[tb * stride + tid] = r.v[tb]; };
            ((__attribute__((address_space(3))) int32_t*)sp)[PT_COUNT * stride + t] = r.corr;
            if (fl & CF_BIAS) put(PT_BIAS);
            if (fl & CF_SCALE) put(PT_SCALE);
            if (fl & CF_RES_SUB) put(PT_RSUB);
            if (fl & CF_RES_MUL) put(PT_RMUL);
            if (fl & CF_POST_SCALE) put(PT_POST);
            if (fl & CF_OUT_FQ) {
                put(PT_IH);
                if (fl & CF_FQ_RCP) put(PT_R);
                if (fl & CF_FQ_DIV2) put(PT_R2);
                if (!(fl & CF_FQ_IL0)) {
                    put(PT_IL);
                    put(PT_D);
                }
            }
        }
    }
}

// accumulators from the staged corrections (after the barrier that publishes them)
__device__ __forceinline__ void init_acc_lds(lds_cfloat_ptr sp, int stride, int oc_local, v16i (&acc)[2][2]) {
    const __attribute__((address_space(3))) int32_t* corr =
        (const __attribute__((address_space(3))) int32_t*)sp + PT_COUNT * stride + oc_local;
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            // one LDS read per accumulator tile (volatile: not merged into one read and four register copies per
            // tile - the reads are broadcasts that cost no vector-ALU issue, the copies would)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) {
                const v4i c = *(const volatile __attribute__((address_space(3))) v4i*)(corr + 16 * ob + 4 * q);
                acc[ob][pb][4 * q + 0] = c.x;
                acc[ob][pb][4 * q + 1] = c.y;
                acc[ob][pb][4 * q + 2] = c.z;
                acc[ob][pb][4 * q + 3] = c.w;
            }
        }
}

struct EpiParams {
    float4 bias, scale, rsub, rmul, post, il, ih, d, r, r2;
    float4 res[2];   // f32 residual of the two pixels
};

// residual level as float: signed bytes as they are; level-128 bytes through a sign-bit flip of the
// whole dword and the unsigned byte conversion (v_cvt_f32_ubyteN), the same exact integer value
template <bool U8B>
__device__ __forceinline__ float res_byte_to_float(uint32_t dw, int j) {
    if (U8B) return static_cast<float>(((dw ^ 0x80808080u) >> (8 * j)) & 0xffu);
    return static_cast<float>(static_cast<int>(static_cast<int8_t>((dw >> (8 * j)) & 0xffu)));
}

__device__ __forceinline__ void f4_to_array(const float4& v, float (&o)[4]) {
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}

// The 32 residual bytes of each of a lane's two pixels (zero where the pixel or channel does not
// exist).  The loads are unconditional - a lane without a valid element reads the first 16 bytes
// of its (clamped, existing) pixel and discards them - so that all four are in flight together;
// a load inside a divergent branch is awaited at the end of its branch.
__device__ __forceinline__ void load_residual_bytes(const ConvArgs& a, int oc_lane, const bool (&valid)[2],
                                                    const int64_t (&res_off)[2], uint32_t (&res_dw)[2][8]) {
    uint4 v[2][2];
    bool ok[2][2];
#pragma unroll
    for (int pb = 0; pb < 2; ++pb)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ok[pb][j] = valid[pb] && oc_lane + 16 * j < a.res_sw;
            const int64_t off = ok[pb][j] ? res_off[pb] + 16 * j : res_off[pb] - oc_lane;
            v[pb][j] = *reinterpret_cast<const uint4*>(static_cast<const int8_t*>(a.res) + off);
        }
#pragma unroll
    for (int pb = 0; pb < 2; ++pb)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            res_dw[pb][4 * j + 0] = ok[pb][j] ? v[pb][j].x : 0u;
            res_dw[pb][4 * j + 1] = ok[pb][j] ? v[pb][j].y : 0u;
            res_dw[pb][4 * j + 2] = ok[pb][j] ? v[pb][j].z : 0u;
            res_dw[pb][4 * j + 3] = ok[pb][j] ? v[pb][j].w : 0u;
        }
}

// sp: the tile's staged tables (stage_params) with local channel 0 = channel oc0, or nullptr to
// read the tables from global memory
// NOB = 2: a lane owns 32 channels (acc[0..1]); NOB = 1: 16 channels (acc[0] only)
// LDS_ONLY (byte outputs): the wave's 64 pixels x 64 channels stay in `stage` (row r = pixel, chunk c of 16 bytes in slot
// c ^ ((r >> 2) & 3): the layout of an operand tile) and nothing is stored to memory - the tile is the next
// convolution's operand
// IN_LDS: the caller vouches that `sp` is set, STAGED that `stage` is (a pointer into dynamically sized LDS does not tell
// the compiler, which then keeps both forms of every table read behind a run-time test and waits for all memory and
// LDS operations in front of each group of channels)
// ILP: for a kernel whose waves run one or two to a SIMD - the eight values of a group of channels advance through the
// FakeQuantize together, operation by operation (pinned, or the compiler folds them back into eight serial chains to
// save registers), so that the wave's own independent instructions stand between an operation and its consumer
#define HIPIE_PIN8(x) asm volatile("" : "+v"(x[0][0]), "+v"(x[0][1]), "+v"(x[0][2]), "+v"(x[0][3]), "+v"(x[1][0]), "+v"(x[1][1]), "+v"(x[1][2]), "+v"(x[1][3]))
template <uint32_t F, int NOB = 2, bool LDS_ONLY = false, bool IN_LDS = false, bool STAGED = IN_LDS, bool ILP = false>
__device__ __forceinline__ void epilogue(const ConvArgs& a, const v16i (&acc)[2][2], int oc_lane,
                                         const bool (&valid)[2], const int64_t (&out_off)[2],
                                         const int64_t (&res_off)[2], const v16f (&rres)[2][2],
                                         lds_cfloat_ptr sp, int sp_stride, int oc0,
                                         const uint32_t (*pre_res)[8] = nullptr, lds_float_ptr stage = nullptr) {
    const uint32_t fl = F == kDyn ? a.flags : F;
    // f32 results leave through a wave-private 8 KB LDS buffer (`stage`, when the kernel has one): a
    // lane owns 32 channels of two pixels, so direct stores put 16-byte pieces of 32 different rows in
    // one instruction; staged, 16 lanes store the 256 contiguous bytes of one pixel's 64 channels.
    // One pixel block (32 pixels) at a time, rows of 16 chunks with chunk c of row r kept in slot
    // c ^ (r & 15): conflict-free for the writes (rows r .. r + 7, one chunk) and the reads (one row).
    constexpr bool kCanStage = F != kDyn && !(F & (CF_OUT_FQ | CF_OUT_I32)) && NOB == 2;
    const bool staged_out = kCanStage && (STAGED || stage != nullptr);
    constexpr bool kCanStageBytes = F != kDyn && (F & CF_OUT_FQ) && NOB == 2;
    // an f32 residual that is the last operation in front of the store is added where the staged rows
    // are read back: there a lane's residual piece is as contiguous as its store
    constexpr bool kLateRes = kCanStage && (F & CF_RES) && (F & CF_RES_F32) &&
                              !(F & (CF_RES_SUB | CF_RES_MUL | CF_POST_SCALE | CF_RELU | CF_CLAMP | CF_GELU | CF_RES_GEMM));
    const bool late_res = kLateRes && staged_out;
    const int lane_id = static_cast<int>(threadIdx.x) & 63;
    auto tab = [&](int t, const float* g, int oc) {
        if (IN_LDS || sp) {
            typedef float v4f __attribute__((ext_vector_type(4)));
            const v4f v = *(const __attribute__((address_space(3))) v4f*)(sp + t * sp_stride + (oc - oc0));
            return make_float4(v.x, v.y, v.z, v.w);
        }
        return ld4f(g + oc);
    };
    const int out_cs = a.out_sw;

    if (fl & CF_OUT_I32) {   // raw accumulators
#pragma unroll
        for (int e4 = 0; e4 < 4 * NOB; ++e4)
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
                if (valid[pb] && oc_lane + 4 * e4 + 4 <= out_cs) {
                    const int ob = e4 >> 2, r0 = (e4 & 3) * 4;
                    *reinterpret_cast<int4*>(static_cast<int32_t*>(a.out) + out_off[pb] + 4 * e4) =
                        make_int4(acc[ob][pb][r0], acc[ob][pb][r0 + 1], acc[ob][pb][r0 + 2], acc[ob][pb][r0 + 3]);
                }
        return;
    }

    uint32_t res_dw[2][8];
    if ((fl & CF_RES) && !(fl & (CF_RES_F32 | CF_RES_GEMM))) {
        if (pre_res) {
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int q = 0; q < 8; ++q) res_dw[pb][q] = pre_res[pb][q];
        } else {
            load_residual_bytes(a, oc_lane, valid, res_off, res_dw);
        }
    }

    int pass_now = 0;   // pixel block of the current pass over the channels (staged f32 output only)
    auto load = [&](int e4, EpiParams& p) {
        const int oc = oc_lane + 4 * e4;
        if (fl & CF_BIAS) p.bias = tab(PT_BIAS, a.bias, oc);
        if (fl & CF_SCALE) p.scale = tab(PT_SCALE, a.scale, oc);
        if (fl & CF_RES_SUB) p.rsub = tab(PT_RSUB, a.res_sub, oc);
        if (fl & CF_RES_MUL) p.rmul = tab(PT_RMUL, a.res_mul, oc);
        if (fl & CF_POST_SCALE) p.post = tab(PT_POST, a.post_scale, oc);
        if (fl & CF_OUT_FQ) {
            p.ih = tab(PT_IH, a.fq_ih, oc);
            if (fl & CF_FQ_RCP) p.r = tab(PT_R, a.fq_r, oc);
            if (fl & CF_FQ_DIV2) p.r2 = tab(PT_R2, a.fq_r2, oc);
            if (!(fl & CF_FQ_IL0)) {
                p.il = tab(PT_IL, a.fq_il, oc);
                p.d = tab(PT_D, a.fq_d, oc);
            }
        }
        if ((fl & CF_RES) && (fl & CF_RES_F32) && !late_res) {
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) {
                if (staged_out && pb != pass_now) continue;
                p.res[pb] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (valid[pb] && oc + 4 <= a.res_sw)
                    p.res[pb] = ld4f(static_cast<const float*>(a.res) + res_off[pb] + 4 * e4);
            }
        }
    };

    uint32_t out_dw[2][8];
#pragma unroll
    for (int pass = 0; pass < (kCanStage ? 2 : 1); ++pass) {
    if (pass == 1 && !staged_out) break;
    pass_now = pass;
    EpiParams cur, nxt;
    load(0, cur);
#pragma unroll
    for (int e4 = 0; e4 < 4 * NOB; ++e4) {
        if (e4 + 1 < 4 * NOB) load(e4 + 1, nxt);
        const int ob = e4 >> 2, r0 = (e4 & 3) * 4;
        float bias_[4], scale_[4], rsub_[4], rmul_[4], post_[4], il_[4], ih_[4], d_[4], rr_[4], r2_[4];
        f4_to_array(cur.bias, bias_);
        f4_to_array(cur.scale, scale_);
        f4_to_array(cur.rsub, rsub_);
        f4_to_array(cur.rmul, rmul_);
        f4_to_array(cur.post, post_);
        f4_to_array(cur.ih, ih_);
        f4_to_array(cur.r, rr_);
        f4_to_array(cur.r2, r2_);
        if (fl & CF_FQ_IL0) {   // input_low == +0: x - il == x and d == ih
            il_[0] = il_[1] = il_[2] = il_[3] = 0.f;
            f4_to_array(cur.ih, d_);
        } else {
            f4_to_array(cur.il, il_);
            f4_to_array(cur.d, d_);
        }
        float v[2][4];
#pragma unroll
        for (int pb = 0; pb < 2; ++pb) {
            if (staged_out && pb != pass) continue;   // staged: pixel block `pass` only
            float rv[4];
            if ((fl & CF_RES) && !late_res) {
                if (fl & CF_RES_GEMM) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) rv[j] = rres[ob][pb][r0 + j];
                } else if (fl & CF_RES_F32) f4_to_array(cur.res[pb], rv);
                else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        rv[j] = (fl & CF_RES_U8B) ? res_byte_to_float<true>(res_dw[pb][e4], j) : res_byte_to_float<false>(res_dw[pb][e4], j);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float x = static_cast<float>(acc[ob][pb][r0 + j]);
                if (fl & CF_BIAS) x = x + bias_[j];
                if (fl & CF_SCALE) x = x * scale_[j];
                if ((fl & CF_RES) && !late_res) {
                    float r = rv[j];
                    if (fl & CF_RES_SUB) r = r - rsub_[j];
                    if (fl & CF_RES_MUL) r = r * rmul_[j];
                    x = x + r;
                }
                if (fl & CF_POST_SCALE) x = x * post_[j];
                if (fl & CF_RELU) x = x > 0.0f ? x : 0.0f;
                // clamp.hpp: x < lo ? lo : (x > hi ? hi : x).  In front of a FakeQuantize the median of three gives
                // the same level in one instruction (x is finite; the two differ only in the sign of a zero,
                // and both zeros are level 0 or the same distance from every level boundary)
                if ((fl & CF_CLAMP) && (fl & CF_OUT_FQ)) x = __builtin_amdgcn_fmed3f(x, a.clamp_lo, a.clamp_hi);
                else if (fl & CF_CLAMP) x = x < a.clamp_lo ? a.clamp_lo : (x > a.clamp_hi ? a.clamp_hi : x);
                if (fl & CF_GELU) x = gelu_one(x);
                v[pb][j] = x;
            }
        }
        if (fl & CF_OUT_FQ) {
            // the eight values of a group advance together, operation by operation, and the two dwords are packed in
            // turn: a wave that runs alone on its SIMD has nothing but its own independent instructions to put
            // between an operation and the one that needs its result
            uint32_t packed[2] = {0, 0};
            float t[2][4];
            if (ILP && (fl & CF_FQ_DIV2) && (fl & CF_FQ_SAT)) {
                float n[2][4], lo[2][4];
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        n[pb][j] = (fl & CF_FQ_IL0) ? v[pb][j] : v[pb][j] - il_[j];
                        lo[pb][j] = n[pb][j] * r2_[j];
                    }
                HIPIE_PIN8(lo);
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int j = 0; j < 4; ++j) lo[pb][j] = fmaf(n[pb][j], rr_[j], lo[pb][j]);
                HIPIE_PIN8(lo);
#pragma unroll
                for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                    for (int j = 0; j < 4; ++j) t[pb][j] = lo[pb][j] * a.lm1;
                HIPIE_PIN8(t);
            } else
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if ((fl & CF_FQ_DIV2) && (fl & CF_FQ_SAT)) {
                        t[pb][j] = (fl & CF_FQ_IL0) ? fq_level_fast<2, true, true>(v[pb][j], 0.f, ih_[j], d_[j], rr_[j], r2_[j], a.lm1)
                                                    : fq_level_fast<2, false, true>(v[pb][j], il_[j], ih_[j], d_[j], rr_[j], r2_[j], a.lm1);
                    } else if (fl & CF_FQ_DIV2) {
                        t[pb][j] = (fl & CF_FQ_IL0) ? fq_level_fast<2, true>(v[pb][j], 0.f, ih_[j], d_[j], rr_[j], r2_[j], a.lm1)
                                                    : fq_level_fast<2, false>(v[pb][j], il_[j], ih_[j], d_[j], rr_[j], r2_[j], a.lm1);
                    } else if ((fl & CF_FQ_RCP) && (fl & CF_FQ_SAT)) {
                        t[pb][j] = (fl & CF_FQ_IL0) ? fq_level_fast<1, true, true>(v[pb][j], 0.f, ih_[j], d_[j], rr_[j], 0.f, a.lm1)
                                                    : fq_level_fast<1, false, true>(v[pb][j], il_[j], ih_[j], d_[j], rr_[j], 0.f, a.lm1);
                    } else if (fl & CF_FQ_RCP) {
                        t[pb][j] = (fl & CF_FQ_IL0) ? fq_level_fast<1, true>(v[pb][j], 0.f, ih_[j], d_[j], rr_[j], 0.f, a.lm1)
                                                    : fq_level_fast<1, false>(v[pb][j], il_[j], ih_[j], d_[j], rr_[j], 0.f, a.lm1);
                    } else {
                        t[pb][j] = fq_level_fast<0, false>(v[pb][j], il_[j], ih_[j], d_[j], 0.f, 0.f, a.lm1);
                    }
                }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int pb = 0; pb < 2; ++pb) packed[pb] = __builtin_amdgcn_cvt_pk_u8_f32(t[pb][j], j, packed[pb]);
            asm volatile("" : "+v"(packed[0]), "+v"(packed[1]) : : "memory");
            out_dw[0][e4] = packed[0];
            out_dw[1][e4] = packed[1];
        } else if (staged_out) {
            typedef float v4f __attribute__((ext_vector_type(4)));
            const int row = lane_id & 31, c = ((lane_id >> 5) * 8 + e4) ^ (row & 15);
            v4f o;
            o.x = v[pass][0]; o.y = v[pass][1]; o.z = v[pass][2]; o.w = v[pass][3];
            *(__attribute__((address_space(3))) v4f*)(stage + row * 64 + c * 4) = o;
        } else {
            asm volatile("" : "+v"(v[0][0]), "+v"(v[0][1]), "+v"(v[0][2]), "+v"(v[0][3]), "+v"(v[1][0]),
                         "+v"(v[1][1]), "+v"(v[1][2]), "+v"(v[1][3]) : : "memory");
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
                if (valid[pb] && oc_lane + 4 * e4 + 4 <= out_cs)
                    *reinterpret_cast<float4*>(static_cast<float*>(a.out) + out_off[pb] + 4 * e4) =
                        make_float4(v[pb][0], v[pb][1], v[pb][2], v[pb][3]);
        }
        cur = nxt;
    }
    if (staged_out) {
        // LDS operations of one wave complete in order; the waits only keep the compiler from moving
        // accesses across the two phases
        typedef float v4f __attribute__((ext_vector_type(4)));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const int oc_wave = oc_lane - 32 * (lane_id >> 5);          // first channel of the wave's 64
        const int c = lane_id & 15;
        const int64_t own = out_off[pass] - 32 * (lane_id >> 5);    // lanes 0 .. 31 hold rows 0 .. 31
        const int64_t own_res = res_off[pass] - 32 * (lane_id >> 5);
        auto from_row = [&](int64_t v, int row) {
            const uint32_t lo = __shfl(static_cast<uint32_t>(v), row, 64);
            const uint32_t hi = __shfl(static_cast<uint32_t>(static_cast<uint64_t>(v) >> 32), row, 64);
            return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
        };
        float4 late[8];
        bool ok[8];
        int64_t off[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = 4 * i + (lane_id >> 4);
            off[i] = from_row(own, row);
            ok[i] = __shfl(static_cast<int>(valid[pass]), row, 64) != 0;
            if (late_res) {   // all eight loads in flight together
                late[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                const int64_t roff = from_row(own_res, row);
                if (ok[i] && oc_wave + 4 * c + 4 <= a.res_sw) late[i] = ld4f(static_cast<const float*>(a.res) + roff + 4 * c);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = 4 * i + (lane_id >> 4);
            const v4f o = *(const __attribute__((address_space(3))) v4f*)(stage + row * 64 + ((c ^ (row & 15)) * 4));
            float4 r = make_float4(o.x, o.y, o.z, o.w);
            if (late_res) { r.x = r.x + late[i].x; r.y = r.y + late[i].y; r.z = r.z + late[i].z; r.w = r.w + late[i].w; }
            if (ok[i] && oc_wave + 4 * c + 4 <= out_cs)
                *reinterpret_cast<float4*>(static_cast<float*>(a.out) + off[i] + 4 * c) = r;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    }
    if (fl & CF_OUT_FQ) {
        // stored byte = level + out_off (mod 256); -128 is a sign-bit flip, 0 nothing: one XOR mask
        // covers both, anything else goes through the bytewise add (one uniform branch for all stores)
        const bool flip = a.flags & CF_OUT_XOR;
        if (fl & CF_OUT_ADD) {   // run-time flags only: no specialised instance carries this step
            const uint32_t off4 = (static_cast<uint32_t>(static_cast<int>(a.out_off)) & 0xffu) * 0x01010101u;
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int q = 0; q < 4 * NOB; ++q) out_dw[pb][q] = add_bytes(out_dw[pb][q], off4);
        }
        const uint32_t xmask = flip ? 0x80808080u : 0u;
        if (kCanStageBytes && (STAGED || stage != nullptr)) {
            // Bytes leave through the wave's LDS buffer as well: 64 rows (pixels) of the wave's 64
            // channels, chunk c (16 bytes) of row r in slot c ^ ((r >> 2) & 3); four lanes then store
            // the 64 contiguous bytes of one pixel instead of 16-byte pieces of 32 different pixels.
            typedef uint32_t v4u __attribute__((ext_vector_type(4)));
            typedef __attribute__((address_space(3))) v4u* lds_v4u_ptr;
            const lds_v4u_ptr st = (lds_v4u_ptr)stage;
            const int h = lane_id >> 5;
#pragma unroll
            for (int pb = 0; pb < 2; ++pb)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int row = 32 * pb + (lane_id & 31);
                    v4u o;
                    o.x = out_dw[pb][4 * j] ^ xmask; o.y = out_dw[pb][4 * j + 1] ^ xmask;
                    o.z = out_dw[pb][4 * j + 2] ^ xmask; o.w = out_dw[pb][4 * j + 3] ^ xmask;
                    st[row * 4 + ((2 * h + j) ^ ((row >> 2) & 3))] = o;
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (LDS_ONLY) return;
            const int oc_wave = oc_lane - 32 * h;
            const int c = lane_id & 3;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 16 * i + (lane_id >> 2), pb = i >> 1, src = row & 31;
                const v4u o = st[row * 4 + (c ^ ((row >> 2) & 3))];
                const int64_t own = out_off[pb] - 32 * h;
                const uint32_t lo = __shfl(static_cast<uint32_t>(own), src, 64);
                const uint32_t hi = __shfl(static_cast<uint32_t>(static_cast<uint64_t>(own) >> 32), src, 64);
                const int ok = __shfl(static_cast<int>(valid[pb]), src, 64);
                const int64_t off = static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
                if (ok && oc_wave + 16 * c < out_cs)
                    *reinterpret_cast<uint4*>(static_cast<int8_t*>(a.out) + off + 16 * c) = make_uint4(o.x, o.y, o.z, o.w);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            return;
        }
#pragma unroll
        for (int pb = 0; pb < 2; ++pb)
#pragma unroll
            for (int j = 0; j < NOB; ++j)
                if (valid[pb] && oc_lane + 16 * j < out_cs)
                    *reinterpret_cast<uint4*>(static_cast<int8_t*>(a.out) + out_off[pb] + 16 * j) =
                        make_uint4(out_dw[pb][4 * j] ^ xmask, out_dw[pb][4 * j + 1] ^ xmask,
                                   out_dw[pb][4 * j + 2] ^ xmask, out_dw[pb][4 * j + 3] ^ xmask);
    }
}

// where a lane's two pixels live in the output and residual tensors
struct EpiAddr {
    bool valid[2];
    int64_t out_off[2], res_off[2];
};

__device__ __forceinline__ void epilogue_addresses(const ConvArgs& a, int oc_lane, int m0, int m1, int batch, EpiAddr& e) {
    const int m[2] = {m0, m1};
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
        e.valid[pb] = m[pb] < a.M;
        const int mm = e.valid[pb] ? m[pb] : a.M - 1;
        if (a.flat_out && (a.flat_res || !a.res)) {   // uniform: dense tensors, no decode
            e.out_off[pb] = batch_offset(a, batch, a.batch_out, a.batch_out_o) + static_cast<int64_t>(mm) * a.out_sw + oc_lane;
            e.res_off[pb] = batch * a.batch_res + static_cast<int64_t>(mm) * a.res_sw + oc_lane;
            continue;
        }
        const PixelCoord p = decode_pixel(a, mm);
        e.out_off[pb] = batch_offset(a, batch, a.batch_out, a.batch_out_o) + static_cast<int64_t>(p.n) * a.out_sn + p.oh * a.out_sh +
                        p.ow * a.out_sw + oc_lane;
        e.res_off[pb] = batch * a.batch_res + static_cast<int64_t>(p.n) * a.res_sn + p.oh * a.res_sh +
                        p.ow * a.res_sw + oc_lane;
    }
}

template <uint32_t F, bool IN_LDS = false, bool STAGED = false>
__device__ __forceinline__ void run_epilogue(const ConvArgs& a, const v16i (&acc)[2][2], int oc_lane,
                                             int m0, int m1, int batch, const v16f (&rres)[2][2],
                                             lds_cfloat_ptr sp = nullptr, int sp_stride = 0, int oc0 = 0,
                                             lds_float_ptr stage = nullptr) {
    EpiAddr e;
    epilogue_addresses(a, oc_lane, m0, m1, batch, e);
    epilogue<F, 2, false, IN_LDS, STAGED>(a, acc, oc_lane, e.valid, e.out_off, e.res_off, rres, sp, sp_stride, oc0, nullptr, stage);
}

template <uint32_t F, bool IN_LDS = false>
__device__ __forceinline__ void run_epilogue(const ConvArgs& a, const v16i (&acc)[2][2], int oc_lane,
                                             int m0, int m1, int batch = 0, lds_cfloat_ptr sp = nullptr,
                                             int sp_stride = 0, int oc0 = 0) {
    v16f none[2][2];
    run_epilogue<F, IN_LDS, false>(a, acc, oc_lane, m0, m1, batch, none, sp, sp_stride, oc0);
}

}  // namespace hipie
