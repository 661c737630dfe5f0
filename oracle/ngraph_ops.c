/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement of the nGraph reference kernels that define the
 * INT8 hot path.  Nothing in the shipped library links, loads or calls this file; it exists so
 * that tests, the smoke check and the CPU-baseline leg of the benchmark have an independent
 * checker.  Every function names the reference file:line it follows
 * (paths relative to ngraph/core/reference/include/ngraph/runtime/reference/).
 *
 * Tensors are dense row-major in the reference's own layouts (NCHW data, OIHW / GOIHW filters).
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (no fast-math: float op order is part
 * of the contract).
 *
 * Pinning status (what fixes each function besides this text):
 *   fake_quantize      reference goldens fake_quantize.in.cpp + compiled reference (_ref) fuzz
 *   convolution        27 reference goldens convolution.in.cpp + _ref fuzz + int64 brute force
 *   group_convolution  reference goldens group_convolution.in.cpp + _ref fuzz
 *   matmul             reference goldens matmul.in.cpp + numpy integer matmul + _ref fuzz
 *   add/mul/sub/relu/clamp/convert   numpy closed forms + _ref fuzz
 *   prelu              36 reference goldens prelu.in.cpp (every literal vector there) + _ref fuzz
 *   hswish/hsigmoid    _ref fuzz (bit-exact) + the points the definition fixes (0 below -3, x or 1 above 3, hswish(1) = 4/6)
 *   sigmoid/swish      _ref fuzz + scipy closed forms (expit) on the inputs of sigmoid.in.cpp / swish.in.cpp, whose
 *                      expected values are formulas, not vectors (tolerance only; libm-dependent)
 *   max_pool/avg_pool  reference goldens + _ref fuzz
 *   softmax/mvn/gelu   _ref fuzz + scipy closed forms (tolerance only; libm-dependent)
 */
#include <fenv.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAX_RANK 8

static int64_t shape_size(const int64_t* s, int rank) {
    int64_t n = 1;
    for (int i = 0; i < rank; ++i) n *= s[i];
    return n;
}

/* ---------------------------------------------------------------------------------------
 * numpy-style broadcast strides of `shape` (rank r) against `target` (rank tr).
 * axis == -2 : NUMPY (right-aligned); axis >= -1 : PDPD placement as in
 * fake_quantize.hpp:64-98 (align_shape_sizes).
 * ------------------------------------------------------------------------------------- */
static void bcast_strides(const int64_t* shape, int r, const int64_t* target, int tr, int axis,
                          int64_t* strides /* [tr] */) {
    int64_t aligned[ORC_MAX_RANK];
    for (int i = 0; i < tr; ++i) aligned[i] = 1;
    if (axis == -2) {
        for (int i = 0; i < r; ++i) aligned[tr - r + i] = shape[i];
    } else {
        int a = axis == -1 ? tr - r : axis;
        int ncopy = tr - a;
        if (ncopy > r) ncopy = r;
        for (int i = 0; i < ncopy; ++i) aligned[a + i] = shape[i];
    }
    int64_t st = 1;
    for (int i = tr - 1; i >= 0; --i) {
        strides[i] = aligned[i] == 1 ? 0 : st;
        st *= aligned[i];
    }
    (void)target;
}

/* fake_quantize.hpp:175-194 (fake_quantize_details::quantize) */
static inline float fq_quantize(float arg, float in_low, float in_high, float out_low,
                                float out_high, size_t levels) {
    float lo = in_low < in_high ? in_low : in_high;   /* std::min(in_low, in_high) */
    float hi = in_low < in_high ? in_high : in_low;   /* std::max(in_low, in_high) */
    if (arg <= lo) return out_low;
    else if (arg > hi) return out_high;
    /* (levels - 1) is size_t in the reference; float op size_t converts the integer to float */
    float lm1 = (float)(levels - 1);
    return nearbyintf((arg - in_low) / (in_high - in_low) * lm1) / lm1 * (out_high - out_low) +
           out_low;
}

/* fake_quantize.hpp:199-265 (v0::fake_quantize) with the bounds broadcast to the data shape. */
void orc_fake_quantize_f32(const float* x, const int64_t* xshape, int xrank,
                           const float* il, const int64_t* il_shape, int il_rank,
                           const float* ih, const int64_t* ih_shape, int ih_rank,
                           const float* ol, const int64_t* ol_shape, int ol_rank,
                           const float* oh, const int64_t* oh_shape, int oh_rank,
                           int64_t levels, int bcast_axis, float* out) {
    int64_t s_il[ORC_MAX_RANK], s_ih[ORC_MAX_RANK], s_ol[ORC_MAX_RANK], s_oh[ORC_MAX_RANK];
    bcast_strides(il_shape, il_rank, xshape, xrank, bcast_axis, s_il);
    bcast_strides(ih_shape, ih_rank, xshape, xrank, bcast_axis, s_ih);
    bcast_strides(ol_shape, ol_rank, xshape, xrank, bcast_axis, s_ol);
    bcast_strides(oh_shape, oh_rank, xshape, xrank, bcast_axis, s_oh);
    int old = fegetround();
    fesetround(FE_TONEAREST);
    int64_t n = shape_size(xshape, xrank);
    int64_t idx[ORC_MAX_RANK] = {0};
    for (int64_t i = 0; i < n; ++i) {
        int64_t a = 0, b = 0, c = 0, d = 0;
        for (int k = 0; k < xrank; ++k) {
            a += idx[k] * s_il[k];
            b += idx[k] * s_ih[k];
            c += idx[k] * s_ol[k];
            d += idx[k] * s_oh[k];
        }
        out[i] = fq_quantize(x[i], il[a], ih[b], ol[c], oh[d], (size_t)levels);
        for (int k = xrank - 1; k >= 0; --k) { /* fake_quantize.hpp:100-113 */
            if (++idx[k] < xshape[k]) break;
            idx[k] = 0;
        }
    }
    fesetround(old);
}

/* ---------------------------------------------------------------------------------------
 * convolution.hpp:63-146 (convolve_3D_channels), :148-167 (extend_to_3D), :245-293 (driver).
 * in: [N, C, spatial...], f: [OC, C, k...], rank 3..5; padding cells are skipped, the
 * accumulator has the element type (float: sequential order c, z, y, x).
 * ------------------------------------------------------------------------------------- */
typedef struct {
    int N, C, D, H, W, OC, KD, KH, KW;
    int sd, sh, sw, dd, dh, dw, pbd, pbh, pbw, ped, peh, pew;
    int OD, OH, OW;
} conv3d_t;

static void conv_setup(conv3d_t* p, const int64_t* in_shape, const int64_t* f_shape, int rank,
                       const int64_t* strides, const int64_t* dil, const int64_t* pb,
                       const int64_t* pe, int f_off /* 0: OIHW, 1: skip group axis */) {
    int sp = rank - 2;
    int ins[3] = {1, 1, 1}, ks[3] = {1, 1, 1}, st[3] = {1, 1, 1}, di[3] = {1, 1, 1};
    int b[3] = {0, 0, 0}, e[3] = {0, 0, 0};
    for (int i = 0; i < sp; ++i) {
        int j = 3 - sp + i;
        ins[j] = (int)in_shape[2 + i];
        ks[j] = (int)f_shape[f_off + 2 + i];
        st[j] = (int)strides[i];
        di[j] = (int)dil[i];
        b[j] = (int)pb[i];
        e[j] = (int)pe[i];
    }
    p->N = (int)in_shape[0];
    p->C = (int)in_shape[1];
    p->OC = (int)f_shape[f_off + 0];
    p->D = ins[0]; p->H = ins[1]; p->W = ins[2];
    p->KD = ks[0]; p->KH = ks[1]; p->KW = ks[2];
    p->sd = st[0]; p->sh = st[1]; p->sw = st[2];
    p->dd = di[0]; p->dh = di[1]; p->dw = di[2];
    p->pbd = b[0]; p->pbh = b[1]; p->pbw = b[2];
    p->ped = e[0]; p->peh = e[1]; p->pew = e[2];
    /* loop bounds of convolution.hpp:89-103: i from -pb while i <= pe + in - dilated_k */
    int dkd = p->KD + (p->KD - 1) * (p->dd - 1);
    int dkh = p->KH + (p->KH - 1) * (p->dh - 1);
    int dkw = p->KW + (p->KW - 1) * (p->dw - 1);
    p->OD = (p->ped + p->D - dkd + p->pbd) / p->sd + 1;
    p->OH = (p->peh + p->H - dkh + p->pbh) / p->sh + 1;
    p->OW = (p->pew + p->W - dkw + p->pbw) / p->sw + 1;
}

#define DEFINE_CONV(NAME, T)                                                                    \
    /* one (batch, filter) plane: convolve_3D_channels, convolution.hpp:63-146 */              \
    static void NAME##_plane(const conv3d_t* p, int Cg, const T* batch, const T* filter,       \
                             T* out) {                                                          \
        const int64_t in_ch = (int64_t)p->D * p->H * p->W;                                      \
        const int64_t f_ch = (int64_t)p->KD * p->KH * p->KW;                                    \
        for (int oz = 0; oz < p->OD; ++oz)                                                      \
            for (int oy = 0; oy < p->OH; ++oy)                                                  \
                for (int ox = 0; ox < p->OW; ++ox) {                                            \
                    const int iz = -p->pbd + oz * p->sd, iy = -p->pbh + oy * p->sh,             \
                              ix = -p->pbw + ox * p->sw;                                        \
                    T sum = 0;                                                                  \
                    for (int c = 0; c < Cg; ++c)                                                \
                        for (int fz = 0; fz < p->KD; ++fz)                                      \
                            for (int fy = 0; fy < p->KH; ++fy)                                  \
                                for (int fx = 0; fx < p->KW; ++fx) {                            \
                                    int rz = iz + fz * p->dd, ry = iy + fy * p->dh,             \
                                        rx = ix + fx * p->dw;                                   \
                                    if (rx < 0 || rx >= p->W || ry < 0 || ry >= p->H ||         \
                                        rz < 0 || rz >= p->D)                                   \
                                        continue;                                               \
                                    sum += batch[c * in_ch + ((int64_t)rz * p->H + ry) * p->W + \
                                                 rx] *                                          \
                                           filter[c * f_ch + (fz * p->KH + fy) * p->KW + fx];   \
                                }                                                               \
                    out[((int64_t)oz * p->OH + oy) * p->OW + ox] = sum;                         \
                }                                                                               \
    }                                                                                           \
    /* convolution.hpp:245-293 */                                                               \
    void NAME(const T* in, const T* f, T* out, const int64_t* in_shape, const int64_t* f_shape, \
              int rank, const int64_t* strides, const int64_t* dil, const int64_t* pb,          \
              const int64_t* pe) {                                                              \
        conv3d_t p;                                                                             \
        conv_setup(&p, in_shape, f_shape, rank, strides, dil, pb, pe, 0);                       \
        const int64_t batch_size = (int64_t)p.C * p.D * p.H * p.W;                              \
        const int64_t filter_size = (int64_t)p.C * p.KD * p.KH * p.KW;                          \
        const int64_t out_plane = (int64_t)p.OD * p.OH * p.OW;                                  \
        _Pragma("omp parallel for collapse(2) schedule(static)")                                \
        for (int n = 0; n < p.N; ++n)                                                           \
            for (int oc = 0; oc < p.OC; ++oc)                                                   \
                NAME##_plane(&p, p.C, in + n * batch_size, f + oc * filter_size,                \
                             out + ((int64_t)n * p.OC + oc) * out_plane);                       \
    }                                                                                           \
    /* group_convolution.hpp:78-144: f is [G, OC/G, C/G, k...]; loops batch x group and    */   \
    /* convolves channel slices.                                                            */   \
    void NAME##_group(const T* in, const T* f, T* out, const int64_t* in_shape,                 \
                      const int64_t* f_shape, int rank, const int64_t* strides,                 \
                      const int64_t* dil, const int64_t* pb, const int64_t* pe) {               \
        conv3d_t p;                                                                             \
        conv_setup(&p, in_shape, f_shape, rank, strides, dil, pb, pe, 1);                       \
        const int G = (int)f_shape[0];                                                          \
        const int Cg = p.C / G, OCg = p.OC; /* f_shape[1] = OC/G */                             \
        const int64_t in_plane = (int64_t)p.D * p.H * p.W;                                      \
        const int64_t filter_size = (int64_t)Cg * p.KD * p.KH * p.KW;                           \
        const int64_t out_plane = (int64_t)p.OD * p.OH * p.OW;                                  \
        _Pragma("omp parallel for collapse(2) schedule(static)")                                \
        for (int n = 0; n < p.N; ++n)                                                           \
            for (int g = 0; g < G; ++g)                                                         \
                for (int oc = 0; oc < OCg; ++oc)                                                \
                    NAME##_plane(&p, Cg, in + ((int64_t)n * p.C + (int64_t)g * Cg) * in_plane,  \
                                 f + ((int64_t)g * OCg + oc) * filter_size,                     \
                                 out + ((int64_t)n * G * OCg + (int64_t)g * OCg + oc) *         \
                                           out_plane);                                          \
    }

DEFINE_CONV(orc_convolution_f32, float)
DEFINE_CONV(orc_convolution_i32, int32_t)
DEFINE_CONV(orc_convolution_i64, int64_t)

/* output spatial dims as the reference's loop bounds produce them (convolution.hpp:89-103) */
void orc_conv_out_spatial(const int64_t* in_shape, const int64_t* f_shape, int rank, int grouped,
                          const int64_t* strides, const int64_t* dil, const int64_t* pb,
                          const int64_t* pe, int64_t* out_spatial) {
    conv3d_t p;
    conv_setup(&p, in_shape, f_shape, rank, strides, dil, pb, pe, grouped ? 1 : 0);
    int o[3] = {p.OD, p.OH, p.OW};
    int sp = rank - 2;
    for (int i = 0; i < sp; ++i) out_spatial[i] = o[3 - sp + i];
}

/* ---------------------------------------------------------------------------------------
 * matmul.hpp:24-57 (details::dot, loop order i, k, j), :75-247 (transpose last two dims,
 * numpy batch broadcast, batched dot).  out_shape must come from orc_matmul_out_shape.
 * ------------------------------------------------------------------------------------- */
int orc_matmul_out_shape(const int64_t* a_shape, int ar, const int64_t* b_shape, int br, int ta,
                         int tb, int64_t* out_shape) {
    /* shape rules of ngraph/core/src/op/matmul.cpp (evaluate_matmul / validate_matmul_output_shape) */
    int64_t A[ORC_MAX_RANK], B[ORC_MAX_RANK];
    int r0 = ar, r1 = br;
    memcpy(A, a_shape, sizeof(int64_t) * ar);
    memcpy(B, b_shape, sizeof(int64_t) * br);
    if (ta && ar > 1) { int64_t t = A[ar - 1]; A[ar - 1] = A[ar - 2]; A[ar - 2] = t; }
    if (tb && br > 1) { int64_t t = B[br - 1]; B[br - 1] = B[br - 2]; B[br - 2] = t; }
    if (r0 == 1 && r1 == 1) { out_shape[0] = 1; return 0; /* scalar */ }
    if (r0 == 1) { A[1] = A[0]; A[0] = 1; r0 = 2; }          /* {K} -> {1,K} */
    if (r1 == 1) { B[1] = 1; r1 = 2; }                        /* {K} -> {K,1} */
    int mr = r0 > r1 ? r0 : r1;
    int64_t O[ORC_MAX_RANK];
    for (int i = 0; i < mr - 2; ++i) {
        int ia = i - (mr - r0), ib = i - (mr - r1);
        int64_t da = ia >= 0 ? A[ia] : 1, db = ib >= 0 ? B[ib] : 1;
        O[i] = da > db ? da : db;
    }
    O[mr - 2] = A[r0 - 2];
    O[mr - 1] = B[r1 - 1];
    int orank = mr;
    /* 1-D operands drop their temporary axis */
    if (ar == 1) { for (int i = mr - 2; i < mr - 1; ++i) O[i] = O[i + 1]; orank--; }
    else if (br == 1) { orank--; }
    for (int i = 0; i < orank; ++i) out_shape[i] = O[i];
    return orank;
}

#define DEFINE_MATMUL(NAME, T)                                                                  \
    static void NAME##_dot(const T* a, const T* b, T* out, int64_t I, int64_t K, int64_t J) {   \
        for (int64_t i = 0; i < I * J; ++i) out[i] = 0;                                         \
        for (int64_t i = 0; i < I; ++i)                                                         \
            for (int64_t k = 0; k < K; ++k)                                                     \
                for (int64_t j = 0; j < J; ++j) out[i * J + j] += a[i * K + k] * b[k * J + j];  \
    }                                                                                           \
    static T* NAME##_tr(const T* x, const int64_t* s, int r) { /* swap last two dims */         \
        int64_t R = s[r - 2], Cc = s[r - 1], nb = shape_size(s, r - 2);                         \
        T* t = (T*)malloc(sizeof(T) * (size_t)(nb * R * Cc + 1));                               \
        for (int64_t bb = 0; bb < nb; ++bb)                                                     \
            for (int64_t i = 0; i < R; ++i)                                                     \
                for (int64_t j = 0; j < Cc; ++j)                                                \
                    t[bb * R * Cc + j * R + i] = x[bb * R * Cc + i * Cc + j];                   \
        return t;                                                                               \
    }                                                                                           \
    void NAME(const T* a, const T* b, T* out, const int64_t* a_shape, int ar,                   \
              const int64_t* b_shape, int br, int ta, int tb) {                                 \
        int64_t A[ORC_MAX_RANK], B[ORC_MAX_RANK];                                               \
        memcpy(A, a_shape, sizeof(int64_t) * ar);                                               \
        memcpy(B, b_shape, sizeof(int64_t) * br);                                               \
        T *fa = NULL, *fb = NULL;                                                               \
        if (ta && ar > 1) {                                                                     \
            fa = NAME##_tr(a, A, ar); a = fa;                                                   \
            int64_t t = A[ar - 1]; A[ar - 1] = A[ar - 2]; A[ar - 2] = t;                        \
        }                                                                                       \
        if (tb && br > 1) {                                                                     \
            fb = NAME##_tr(b, B, br); b = fb;                                                   \
            int64_t t = B[br - 1]; B[br - 1] = B[br - 2]; B[br - 2] = t;                        \
        }                                                                                       \
        const int64_t I = ar == 1 ? 1 : A[ar - 2];                                              \
        const int64_t K = br == 1 ? B[0] : B[br - 2];                                           \
        const int64_t J = br == 1 ? 1 : B[br - 1];                                              \
        if (ar <= 2 && br <= 2) {                                                               \
            NAME##_dot(a, b, out, I, K, J);                                                     \
        } else {                                                                                \
            /* numpy broadcast over the batch dims (matmul.hpp:148-201) */                      \
            int bra = ar > 2 ? ar - 2 : 0, brb = br > 2 ? br - 2 : 0;                           \
            int mr = bra > brb ? bra : brb;                                                     \
            int64_t ob[ORC_MAX_RANK], sa[ORC_MAX_RANK], sb[ORC_MAX_RANK];                       \
            int64_t sta = 1, stb = 1;                                                           \
            for (int i = mr - 1; i >= 0; --i) {                                                 \
                int ia = i - (mr - bra), ib = i - (mr - brb);                                   \
                int64_t da = ia >= 0 ? A[ia] : 1, db = ib >= 0 ? B[ib] : 1;                     \
                ob[i] = da > db ? da : db;                                                      \
                sa[i] = da == 1 ? 0 : sta; sta *= da;                                           \
                sb[i] = db == 1 ? 0 : stb; stb *= db;                                           \
            }                                                                                   \
            int64_t nb = shape_size(ob, mr);                                                    \
            for (int64_t q = 0; q < nb; ++q) {                                                  \
                int64_t rem = q, oa = 0, obb = 0;                                               \
                for (int i = mr - 1; i >= 0; --i) {                                             \
                    int64_t c = rem % ob[i]; rem /= ob[i];                                      \
                    oa += c * sa[i]; obb += c * sb[i];                                          \
                }                                                                               \
                if (ar <= 2) oa = 0;                                                            \
                if (br <= 2) obb = 0;                                                           \
                NAME##_dot(a + oa * I * K, b + obb * K * J, out + q * I * J, I, K, J);          \
            }                                                                                   \
        }                                                                                       \
        free(fa);                                                                               \
        free(fb);                                                                               \
    }

DEFINE_MATMUL(orc_matmul_f32, float)
DEFINE_MATMUL(orc_matmul_i32, int32_t)
DEFINE_MATMUL(orc_matmul_i64, int64_t)

/* ---------------------------------------------------------------------------------------
 * Elementwise with numpy broadcast: autobroadcast_binop.hpp (add.hpp, multiply.hpp,
 * subtract.hpp, divide.hpp); relu.hpp; clamp.hpp; convert.hpp (static_cast).
 * The output shape is the numpy broadcast of both inputs and must be given by the caller.
 * ------------------------------------------------------------------------------------- */
#define DEFINE_BINOP(NAME, EXPR)                                                                \
    void NAME(const float* a, const int64_t* a_shape, int ar, const float* b,                   \
              const int64_t* b_shape, int br, const int64_t* o_shape, int orank, float* out) {  \
        int64_t sa[ORC_MAX_RANK], sb[ORC_MAX_RANK], idx[ORC_MAX_RANK] = {0};                    \
        bcast_strides(a_shape, ar, o_shape, orank, -2, sa);                                     \
        bcast_strides(b_shape, br, o_shape, orank, -2, sb);                                     \
        int64_t n = shape_size(o_shape, orank);                                                 \
        for (int64_t i = 0; i < n; ++i) {                                                       \
            int64_t oa = 0, ob = 0;                                                             \
            for (int k = 0; k < orank; ++k) { oa += idx[k] * sa[k]; ob += idx[k] * sb[k]; }     \
            const float x = a[oa], y = b[ob];                                                   \
            out[i] = (EXPR);                                                                    \
            for (int k = orank - 1; k >= 0; --k) {                                              \
                if (++idx[k] < o_shape[k]) break;                                               \
                idx[k] = 0;                                                                     \
            }                                                                                   \
        }                                                                                       \
    }
DEFINE_BINOP(orc_add_f32, x + y)
DEFINE_BINOP(orc_subtract_f32, x - y)
DEFINE_BINOP(orc_multiply_f32, x * y)
DEFINE_BINOP(orc_divide_f32, x / y)

/* prelu.hpp:22-47: a one-dimensional slope with as many elements as the argument has channels (axis 1, axis 0 for a
 * one-dimensional argument) is taken per channel; any other slope broadcasts numpy-style; x < 0 ? x * slope : x */
DEFINE_BINOP(orc_prelu_binop_f32, x < 0.0f ? x * y : x)
void orc_prelu_f32(const float* a, const int64_t* a_shape, int ar, const float* slope, const int64_t* s_shape, int sr,
                   float* out) {
    int64_t channel_shape[ORC_MAX_RANK];
    const int channel_axis = ar > 1 ? 1 : 0;
    if (sr == 1 && a_shape[channel_axis] == s_shape[0]) {
        for (int k = 0; k < ar; ++k) channel_shape[k] = 1;
        channel_shape[channel_axis] = s_shape[0];
        s_shape = channel_shape;
        sr = ar;
    }
    orc_prelu_binop_f32(a, a_shape, ar, slope, s_shape, sr, a_shape, ar, out);
}

/* sigmoid.hpp: 1 / (1 + exp(-x)) in float; hswish.hpp: x * min(max(x + 3, 0), 6) / 6; hsigmoid.hpp: min(max(x + 3, 0), 6) / 6;
 * swish.hpp: x / (1.0 + exp(-x * beta)) with the sum and the quotient in double (the literal 1.0) */
void orc_sigmoid_f32(const float* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        const float e = expf(-x[i]);
        out[i] = 1 / (1 + e);
    }
}
void orc_hswish_f32(const float* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = x[i] * fminf(fmaxf(x[i] + 3.0f, 0.0f), 6.0f) / 6.0f;
}
void orc_hsigmoid_f32(const float* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = fminf(fmaxf(x[i] + 3.0f, 0.0f), 6.0f) / 6.0f;
}
void orc_swish_f32(const float* x, float beta, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (float)(x[i] / (1.0 + expf(-x[i] * beta)));
}

/* relu.hpp: arg > 0 ? arg : 0 */
void orc_relu_f32(const float* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = x[i] > 0.0f ? x[i] : 0.0f;
}
/* clamp.hpp */
void orc_clamp_f32(const float* x, float* out, float mn, float mx, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = x[i] < mn ? mn : (x[i] > mx ? mx : x[i]);
}
/* convert.hpp: out[i] = static_cast<TO>(arg[i]) */
void orc_convert_i32_f32(const int32_t* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (float)x[i];
}
void orc_convert_u8_f32(const uint8_t* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (float)x[i];
}
void orc_convert_i8_f32(const int8_t* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (float)x[i];
}
void orc_convert_f32_u8(const float* x, uint8_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (uint8_t)x[i];
}
void orc_convert_f32_i8(const float* x, int8_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (int8_t)x[i];
}
void orc_convert_u8_i32(const uint8_t* x, int32_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (int32_t)x[i];
}
void orc_convert_i8_i32(const int8_t* x, int32_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = (int32_t)x[i];
}

/* ---------------------------------------------------------------------------------------
 * max_pool.hpp (window max, padding cells skipped, window trimmed at the padded upper bound,
 * init numeric_limits<T>::lowest()); avg_pool.hpp:114-265 (sum / n with the include-padding
 * rules; for 8-bit T the result is nearbyint(float(sum) / n)).  2-D spatial, NCHW.
 * ------------------------------------------------------------------------------------- */
#define DEFINE_MAXPOOL(NAME, T, LOWEST)                                                         \
    void NAME(const T* x, T* out, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh,       \
              int64_t kw, int64_t sh, int64_t sw, int64_t pbh, int64_t pbw, int64_t peh,        \
              int64_t pew, int64_t OH, int64_t OW) {                                            \
        for (int64_t nc = 0; nc < N * C; ++nc)                                                  \
            for (int64_t oy = 0; oy < OH; ++oy)                                                 \
                for (int64_t ox = 0; ox < OW; ++ox) {                                           \
                    int64_t y0 = sh * oy, y1 = y0 + kh, x0 = sw * ox, x1 = x0 + kw;             \
                    if (y1 > H + pbh + peh) y1 = H + pbh + peh;                                 \
                    if (x1 > W + pbw + pew) x1 = W + pbw + pew;                                 \
                    T r = LOWEST;                                                               \
                    for (int64_t y = y0; y < y1; ++y)                                           \
                        for (int64_t xx = x0; xx < x1; ++xx) {                                  \
                            int64_t iy = y - pbh, ix = xx - pbw;                                \
                            if (iy < 0 || iy >= H || ix < 0 || ix >= W) continue;               \
                            T v = x[(nc * H + iy) * W + ix];                                    \
                            r = v > r ? v : r;                                                  \
                        }                                                                       \
                    out[(nc * OH + oy) * OW + ox] = r;                                          \
                }                                                                               \
    }
DEFINE_MAXPOOL(orc_max_pool_f32, float, -3.402823466e+38f)
DEFINE_MAXPOOL(orc_max_pool_u8, uint8_t, 0)
DEFINE_MAXPOOL(orc_max_pool_i8, int8_t, -128)
DEFINE_MAXPOOL(orc_max_pool_i32, int32_t, INT32_MIN)

/* avg_pool.hpp:114-265, T = float */
void orc_avg_pool_f32(const float* x, float* out, int64_t N, int64_t C, int64_t H, int64_t W,
                      int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t pbh, int64_t pbw,
                      int64_t peh, int64_t pew, int64_t OH, int64_t OW, int include_pad) {
    const int padding_present = pbh != 0 || pbw != 0 || peh != 0 || pew != 0;
    for (int64_t nc = 0; nc < N * C; ++nc)
        for (int64_t oy = 0; oy < OH; ++oy)
            for (int64_t ox = 0; ox < OW; ++ox) {
                int64_t y0 = sh * oy, y1 = y0 + kh, x0 = sw * ox, x1 = x0 + kw;
                if (y1 > H + pbh + peh) y1 = H + pbh + peh;
                if (x1 > W + pbw + pew) x1 = W + pbw + pew;
                float r = 0;
                size_t n = 0;
                if (include_pad && padding_present) n = (size_t)(kh * kw);
                for (int64_t y = y0; y < y1; ++y)
                    for (int64_t xx = x0; xx < x1; ++xx) {
                        int64_t iy = y - pbh, ix = xx - pbw;
                        int in_bounds = !(iy < 0 || iy >= H || ix < 0 || ix >= W);
                        if (in_bounds || include_pad) {
                            float v = in_bounds ? x[(nc * H + iy) * W + ix] : 0.0f;
                            r += v;
                            if (!padding_present || (in_bounds && !include_pad)) n++;
                        }
                    }
                out[(nc * OH + oy) * OW + ox] = r / n; /* float / size_t -> float division */
            }
}

/* avg_pool.hpp:114-265, T = uint8_t: the accumulator is uint8_t too (wraps), then
 * static_cast<uint8_t>(nearbyint(float(sum) / n)). */
void orc_avg_pool_u8(const uint8_t* x, uint8_t* out, int64_t N, int64_t C, int64_t H, int64_t W,
                     int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t pbh, int64_t pbw,
                     int64_t peh, int64_t pew, int64_t OH, int64_t OW, int include_pad) {
    const int padding_present = pbh != 0 || pbw != 0 || peh != 0 || pew != 0;
    int old = fegetround();
    fesetround(FE_TONEAREST);
    for (int64_t nc = 0; nc < N * C; ++nc)
        for (int64_t oy = 0; oy < OH; ++oy)
            for (int64_t ox = 0; ox < OW; ++ox) {
                int64_t y0 = sh * oy, y1 = y0 + kh, x0 = sw * ox, x1 = x0 + kw;
                if (y1 > H + pbh + peh) y1 = H + pbh + peh;
                if (x1 > W + pbw + pew) x1 = W + pbw + pew;
                uint8_t r = 0;
                size_t n = 0;
                if (include_pad && padding_present) n = (size_t)(kh * kw);
                for (int64_t y = y0; y < y1; ++y)
                    for (int64_t xx = x0; xx < x1; ++xx) {
                        int64_t iy = y - pbh, ix = xx - pbw;
                        int in_bounds = !(iy < 0 || iy >= H || ix < 0 || ix >= W);
                        if (in_bounds || include_pad) {
                            uint8_t v = in_bounds ? x[(nc * H + iy) * W + ix] : 0;
                            r = (uint8_t)(r + v);
                            if (!padding_present || (in_bounds && !include_pad)) n++;
                        }
                    }
                out[(nc * OH + oy) * OW + ox] = (uint8_t)nearbyintf((float)r / n);
            }
    fesetround(old);
}

/* avg_pool.hpp:114-265, T = int8_t: as for uint8_t, the accumulator has the element type (the sum is kept modulo 256
 * in two's complement), then static_cast<int8_t>(nearbyint(float(sum) / n)). */
void orc_avg_pool_i8(const int8_t* x, int8_t* out, int64_t N, int64_t C, int64_t H, int64_t W,
                     int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t pbh, int64_t pbw,
                     int64_t peh, int64_t pew, int64_t OH, int64_t OW, int include_pad) {
    const int padding_present = pbh != 0 || pbw != 0 || peh != 0 || pew != 0;
    int old = fegetround();
    fesetround(FE_TONEAREST);
    for (int64_t nc = 0; nc < N * C; ++nc)
        for (int64_t oy = 0; oy < OH; ++oy)
            for (int64_t ox = 0; ox < OW; ++ox) {
                int64_t y0 = sh * oy, y1 = y0 + kh, x0 = sw * ox, x1 = x0 + kw;
                if (y1 > H + pbh + peh) y1 = H + pbh + peh;
                if (x1 > W + pbw + pew) x1 = W + pbw + pew;
                int8_t r = 0;
                size_t n = 0;
                if (include_pad && padding_present) n = (size_t)(kh * kw);
                for (int64_t y = y0; y < y1; ++y)
                    for (int64_t xx = x0; xx < x1; ++xx) {
                        int64_t iy = y - pbh, ix = xx - pbw;
                        int in_bounds = !(iy < 0 || iy >= H || ix < 0 || ix >= W);
                        if (in_bounds || include_pad) {
                            int8_t v = in_bounds ? x[(nc * H + iy) * W + ix] : 0;
                            r = (int8_t)(uint8_t)((uint8_t)r + (uint8_t)v);
                            if (!padding_present || (in_bounds && !include_pad)) n++;
                        }
                    }
                out[(nc * OH + oy) * OW + ox] = (int8_t)nearbyintf((float)r / n);
            }
    fesetround(old);
}

/* ---------------------------------------------------------------------------------------
 * fp32 glue: softmax.hpp (one axis: subtract max, exp, sum, divide), mvn.hpp (mvn_6:
 * mean, centre, mean of squares, sqrt(var + eps) or sqrt(var) + eps, divide), gelu.hpp
 * (ERF mode evaluated in double: 0.5 * x * (1 + erf(x / sqrt(2.0)))).
 * x is viewed as [outer, axis, inner].
 * ------------------------------------------------------------------------------------- */
void orc_softmax_f32(const float* x, float* out, int64_t outer, int64_t axis, int64_t inner) {
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t i = 0; i < inner; ++i) {
            const float* p = x + o * axis * inner + i;
            float* q = out + o * axis * inner + i;
            float m = p[0];                       /* max.hpp: starts from lowest, takes max */
            for (int64_t a = 1; a < axis; ++a) m = p[a * inner] > m ? p[a * inner] : m;
            for (int64_t a = 0; a < axis; ++a) q[a * inner] = expf(p[a * inner] - m);
            float s = 0;                          /* sum.hpp: Kahan-compensated for floats */
            float c = 0;
            for (int64_t a = 0; a < axis; ++a) {
                float y = q[a * inner] - c;
                float t = s + y;
                c = (t - s) - y;
                s = t;
            }
            for (int64_t a = 0; a < axis; ++a) q[a * inner] /= s;
        }
}

static float kahan_mean(const float* p, int64_t n) { /* mean.hpp: Kahan sum / count */
    float s = 0, c = 0;
    for (int64_t a = 0; a < n; ++a) {
        float y = p[a] - c;
        float t = s + y;
        c = (t - s) - y;
        s = t;
    }
    return s / (float)n;
}

/* mvn.hpp mvn_6 over the last axis of [outer, axis]; eps_inside: INSIDE_SQRT else OUTSIDE_SQRT */
void orc_mvn_last_axis_f32(const float* x, float* out, int64_t outer, int64_t axis,
                           int normalize_variance, double eps, int eps_inside) {
    float* tmp = (float*)malloc(sizeof(float) * (size_t)(axis + 1));
    for (int64_t o = 0; o < outer; ++o) {
        const float* p = x + o * axis;
        float* q = out + o * axis;
        float mean = kahan_mean(p, axis);
        for (int64_t a = 0; a < axis; ++a) q[a] = p[a] - mean;
        if (normalize_variance) {
            for (int64_t a = 0; a < axis; ++a) tmp[a] = q[a] * q[a];
            float var = kahan_mean(tmp, axis);
            float d = eps_inside ? sqrtf(var + (float)eps) : sqrtf(var) + (float)eps;
            for (int64_t a = 0; a < axis; ++a) q[a] = q[a] / d;
        }
    }
    free(tmp);
}

void orc_gelu_erf_f32(const float* x, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i)
        out[i] = (float)(0.5 * x[i] * (1 + erf(x[i] / sqrt(2.0))));
}
