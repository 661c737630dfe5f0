/*
 * hipie — C ABI of the MI355X (gfx950) INT8 execution engine.
 *
 * This is the boundary an OpenVINO 2021.4 device plugin binds: plain pointers, sizes and opaque
 * handles, no C++ types, no exceptions.  Every call returns a hipie_status (0 = OK) that mirrors
 * InferenceEngine::StatusCode (inference-engine/include/ie_common.h:231-249); the message of the
 * last failure on the calling thread is available from hipie_last_error().
 *
 * Two levels are exported:
 *   1. operator level  — one "create" (load time: validates, packs constants, uploads them) and
 *      one "run" (enqueue on a HIP stream; allocates nothing, never synchronises) per reference
 *      kernel of the INT8 path.  Each declaration cites the reference function it replaces.
 *   2. graph level     — the post-LPT nGraph Function described node by node, compiled into a
 *      plan over one static HBM arena, and executed by infer requests; this is what
 *      IInferencePlugin::LoadExeNetworkImpl / IInferRequestInternal::InferImpl bind
 *      (inference-engine/src/plugin_api/cpp_interfaces/interface/ie_iplugin_internal.hpp:270,
 *       ie_iinfer_request_internal.hpp:57).
 *
 * Device pointers are raw HIP device addresses; `stream` is a hipStream_t passed as void*
 * (NULL = the null stream).  Unless stated otherwise tensors are dense, row-major.
 *
 * Activation storage inside the engine ("U8B"): a u8 quantisation level q is stored as the
 * signed byte q - 128 (bit pattern q ^ 0x80), NHWC, channels padded to a multiple of 16 with
 * level 0.  CDNA4 int8 MFMA multiplies signed bytes only; the constant 128 * sum(w) is folded
 * into the per-channel bias at load time, which keeps the integer sum exactly the u8 x i8 one.
 */
#ifndef HIPIE_H
#define HIPIE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ie_common.h:231-249 (StatusCode) */
typedef enum hipie_status {
    HIPIE_OK = 0,
    HIPIE_GENERAL_ERROR = -1,
    HIPIE_NOT_IMPLEMENTED = -2,
    HIPIE_NETWORK_NOT_LOADED = -3,
    HIPIE_PARAMETER_MISMATCH = -4,
    HIPIE_NOT_FOUND = -5,
    HIPIE_OUT_OF_BOUNDS = -6,
    HIPIE_UNEXPECTED = -7,
    HIPIE_REQUEST_BUSY = -8,
    HIPIE_RESULT_NOT_READY = -9,
    HIPIE_NOT_ALLOCATED = -10,
    HIPIE_INFER_NOT_STARTED = -11,
    HIPIE_NETWORK_NOT_READ = -12,
    HIPIE_INFER_CANCELLED = -13
} hipie_status;

/* element types (numbering of InferenceEngine::Precision::ePrecision, ie_precision.hpp:27-48,
 * plus the engine's internal biased-u8 storage) */
typedef enum hipie_dtype {
    HIPIE_F32 = 10,
    HIPIE_U8 = 40,
    HIPIE_I8 = 50,
    HIPIE_I32 = 70,
    HIPIE_U8B = 41 /* u8 level stored as (level - 128); engine-internal */
} hipie_dtype;

typedef enum hipie_layout { HIPIE_NCHW = 1, HIPIE_NHWC = 2 } hipie_layout; /* ie_common.h:70-100 */

const char* hipie_last_error(void);
/* "major.minor gfx950" build string */
const char* hipie_version(void);
/* number of visible HIP devices, their names (AVAILABLE_DEVICES / FULL_DEVICE_NAME metrics) */
int hipie_device_count(void);
int hipie_device_name(int device, char* buf, size_t buf_len);
/* synchronous copy between host and device memory (to_device = 1: host -> device) */
int hipie_memcpy(void* dst, const void* src, size_t bytes, int to_device);
/* Page-locked host memory for the blobs of an infer request (the allocator a plugin gives its
 * input / output blobs in InferRequest::allocateBlobs, template_infer_request.cpp:63-101): from such
 * buffers hipie_request_start returns as soon as the copies and kernels are queued, and the copies run
 * at the link's rate (pageable buffers are copied through the runtime's own staging, about 40 % slower
 * and synchronously).  Allocated fresh (never registered over existing memory); free with
 * hipie_host_free before the process ends. */
int hipie_host_alloc(size_t bytes, void** ptr);
int hipie_host_free(void* ptr);

/* ======================================================================================
 * Activation tensors handed to the engine's kernels: NHWC, channel stride 1, with a readable
 * border ("halo") of `halo` pixels around every image plane that holds quantisation level 0.
 * Convolution and pooling padding is read from that border instead of being bounds-checked, so
 * a consumer with padding p needs halo >= p.  `data` addresses element (n=0,h=0,w=0,c=0).
 * ==================================================================================== */
typedef struct hipie_tensor {
    void* data;
    int32_t dtype;                        /* hipie_dtype */
    int32_t n, h, w, c;                   /* logical dims */
    int64_t stride_n, stride_h, stride_w; /* in elements; stride_w is the (padded) channel count */
    int32_t halo;
} hipie_tensor;

/* ======================================================================================
 * 1a. FakeQuantize — ngraph/core/reference/.../fake_quantize.hpp:175-194 (quantize),
 *     :199-265 (broadcast driver).  Data is [N, C, HW] (NCHW with the spatial dims flattened);
 *     each bound is a host array of length 1 (scalar) or C (per channel, shape [1,C,1,1] or
 *     [C,1,1] in the reference).  Bit-exact with the reference expression
 *         x <= min(il,ih) ? ol : x > max(il,ih) ? oh
 *           : nearbyint((x-il)/(ih-il)*(L-1))/(L-1)*(oh-ol)+ol        (float, ties-to-even).
 * ==================================================================================== */
typedef struct hipie_fq hipie_fq;

/* device < 0 builds a host-only object (load-time checks without a GPU); its run calls return
 * HIPIE_NOT_ALLOCATED. */
int hipie_fq_create(int device, int64_t channels, int64_t levels,
                    const float* in_low, int64_t n_in_low, const float* in_high, int64_t n_in_high,
                    const float* out_low, int64_t n_out_low, const float* out_high,
                    int64_t n_out_high, hipie_fq** fq);
void hipie_fq_destroy(hipie_fq* fq);

/* op form: f32 in, f32 out, same layout (what reference::fake_quantize<float> returns) */
int hipie_fq_run_f32(const hipie_fq* fq, const float* x, float* y, int64_t n, int64_t hw,
                     void* stream);
/* post-LPT form (network_helper.cpp:943-1087: FQ with out range [0, L-1] and u8 output):
 * writes static_cast<uint8_t>(op result).  Requires scalar out_low/out_high whose op results are
 * the integers out_low + k; HIPIE_NOT_IMPLEMENTED otherwise. out_layout NCHW keeps the layout;
 * NHWC writes [N, HW, c_stride] (c_stride >= C, multiple of 16, padding = level 0).
 * out_dtype: HIPIE_U8 (plain level), HIPIE_U8B (level - 128), HIPIE_I8 (signed levels). */
int hipie_fq_run_q8(const hipie_fq* fq, const float* x, void* y, int64_t n, int64_t hw,
                    hipie_dtype out_dtype, hipie_layout out_layout, int64_t c_stride,
                    void* stream);

/* same as hipie_fq_run_q8 with NHWC output, but into an engine tensor (any strides / halo);
 * this is how a graph input enters the arena */
int hipie_fq_run_q8_tensor(const hipie_fq* fq, const float* x, const hipie_tensor* out, void* stream);
/* the same for an input blob of precision U8 (what benchmark_app feeds image inputs): the u8 -> f32
 * Convert in front of the FakeQuantize (reference::convert<uint8_t, float>, as the template plugin's
 * blobCopy does, docs/template_plugin/src/template_infer_request.cpp:115-129) happens in the kernel */
int hipie_fq_run_q8_tensor_u8(const hipie_fq* fq, const uint8_t* x, const hipie_tensor* out, void* stream);

/* host evaluation of exactly the arithmetic the device kernel uses (reciprocal multiply with
 * two FMA corrections); the planner checks it against IEEE division at every level boundary of
 * every channel and falls back to the dividing kernel if any differs. */
float hipie_fq_host_eval(const hipie_fq* fq, int64_t channel, float x);
/* 1 when the reciprocal path was proven equal to division on all boundaries of all channels */
int hipie_fq_uses_reciprocal(const hipie_fq* fq);

/* ======================================================================================
 * 1b. Fused f32 epilogue applied to i32 accumulators, in this fixed order (each step one IEEE
 *     f32 operation, as the post-LPT graph evaluates them with reference::add / multiply /
 *     subtract / relu / clamp / fake_quantize):
 *        v = float(acc)                     convert.hpp
 *        v = v + bias[c]                    Add after swapMultiplyAndAdd (network_helper.cpp:216-292)
 *        v = v * scale[c]                   dequantization Multiply (convolution.cpp:249-258)
 *        r = float(residual); r -= res_sub[c]; r *= res_mul[c]; v = v + r     (add.cpp:154-218)
 *        v = v * post_scale[c]
 *        relu | clamp(lo, hi) | gelu        relu.hpp, clamp.hpp, gelu.hpp (same float as hipie_gelu_f32)
 *        FakeQuantize(in_low[c], in_high[c], out_low, out_high, levels) -> 8-bit     or f32 store
 *     Arrays are host pointers with 1 (broadcast) or OC values; NULL skips the step.
 * ==================================================================================== */
#define HIPIE_RESIDUAL_SHORTCUT_CONV 1

typedef struct hipie_epilogue {
    const float* bias;        int64_t n_bias;
    const float* scale;       int64_t n_scale;
    int32_t residual_dtype;   /* 0 = none, HIPIE_F32, HIPIE_U8B (value = level), HIPIE_I8, or
                                 HIPIE_RESIDUAL_SHORTCUT_CONV (hipie_conv_create_fused) */
    const float* res_sub;     int64_t n_res_sub;
    const float* res_mul;     int64_t n_res_mul;
    const float* post_scale;  int64_t n_post_scale;
    int32_t activation;       /* 0 none, 1 relu, 2 clamp, 3 gelu (ERF mode; tolerance parity like hipie_gelu_f32) */
    float clamp_lo, clamp_hi;
    int32_t out_dtype;        /* HIPIE_F32, HIPIE_U8B, HIPIE_I8, or HIPIE_I32 (raw accumulators) */
    int64_t fq_levels;
    const float* fq_in_low;   int64_t n_fq_in_low;
    const float* fq_in_high;  int64_t n_fq_in_high;
    float fq_out_low, fq_out_high;
} hipie_epilogue;

/* ======================================================================================
 * 1c. Convolution — reference::convolution<int32_t> on widened u8/i8 inputs
 *     (ngraph/core/reference/.../convolution.hpp:63-146, 245-293; dispatched by
 *     ngraph/test/runtime/interpreter/evaluates_map.cpp:193-216), i.e. the TypeRelaxed
 *     Convolution LPT emits (low_precision_transformations/src/convolution.cpp:201-259), plus
 *     the fused epilogue above.  Weights are i8 OIHW (host); they are packed for the input
 *     tensor's strides at creation.  i32 accumulators are exact.
 * ==================================================================================== */
typedef struct hipie_conv_desc {
    int32_t in_dtype;                     /* HIPIE_U8B or HIPIE_I8 */
    int32_t ic, oc, kh, kw;
    int32_t stride_h, stride_w, dil_h, dil_w;
    int32_t pad_top, pad_left, pad_bottom, pad_right;
    int32_t groups;                       /* 1 = dense (weights [oc][ic][kh][kw]); > 1: weights [oc][ic / groups][kh][kw]
                                             (group_convolution.hpp:78-144); groups == ic == oc (depthwise) has kernels of
                                             its own; groups whose input channels lie in 16-byte-aligned spans under tiles
                                             of 64 output channels (oc a multiple of 64; 64 a multiple of oc / groups with
                                             (64 / (oc / groups)) * (ic / groups) a multiple of 16 and less than ic, or
                                             oc / groups a multiple of 64 with ic / groups a multiple of 16) multiply the
                                             K bytes of their own groups only (variants 1 and 2 of hipie_conv_set_tile);
                                             any other grouping runs as the dense convolution with block-diagonal
                                             weights that it equals */
    int32_t in_c_stride;                  /* channel stride of the input tensor (>= ic) */
    int32_t in_stride_h, in_stride_w;     /* element strides of the input tensor */
    int32_t in_zero_point;                /* integer level subtracted from every input element: the
                                             TypeRelaxed Subtract(u8 data, u8 shift) that
                                             ConvolutionTransformation leaves in front of the convolution
                                             (convolution.cpp:84-120, optimizeSubtract network_helper.cpp:1479-1521).
                                             Padding is applied after the Subtract, so the halo of the
                                             input tensor must hold this level (not level 0). */
    const int32_t* in_zero_points;        /* NULL, or one level per input channel [ic] in place of in_zero_point
                                             (a per-channel Subtract constant: what the transformation's explicit
                                             broadcast, convolution.cpp:97-120, holds when the activations in front of a
                                             grouped convolution are quantized per channel); the halo then holds
                                             channel c's level in channel c.  Read during the create call only. */
    const int32_t* acc_sub;               /* NULL, or one integer per output channel [oc] subtracted from the accumulator:
                                             the DequantizationSubtract that MatMulTransformation puts BEHIND a MatMul whose
                                             activations have a zero point (mat_mul.cpp:95-121: the zero point broadcast
                                             along K and multiplied by the weights, i.e. zp * sum_k w[k][oc]).  Read during
                                             the create call only. */
} hipie_conv_desc;

typedef struct hipie_conv hipie_conv;

int hipie_conv_create(int device, const hipie_conv_desc* desc, const int8_t* weights_oihw,
                      const hipie_epilogue* epilogue, hipie_conv** conv);
/* Residual block tail with a projection shortcut in ONE kernel: the shortcut convolution
 * (Conv' -> Add(bias) -> Multiply(scale), f32, consumed only by the residual Add) is accumulated
 * first and its dequantised value stays in registers as the residual operand of the main
 * convolution's epilogue, instead of an f32 round trip through HBM.  Same arithmetic, same order,
 * same bits as running the two convolutions separately.  The epilogue must be bias, scale,
 * residual = HIPIE_RESIDUAL_SHORTCUT_CONV, FakeQuantize with input_low 0.  hipie_conv_run takes the
 * shortcut convolution's INPUT tensor in its `residual` argument. */
int hipie_conv_create_fused(int device, const hipie_conv_desc* desc, const int8_t* weights_oihw,
                            const hipie_epilogue* epilogue, const hipie_conv_desc* shortcut_desc,
                            const int8_t* shortcut_weights_oihw, const float* shortcut_bias, int64_t n_bias,
                            const float* shortcut_scale, int64_t n_scale, hipie_conv** conv);
void hipie_conv_destroy(hipie_conv* conv);
/* output spatial dims for an input of h x w (convolution.hpp:168-183) */
int hipie_conv_out_dims(const hipie_conv* conv, int32_t h, int32_t w, int32_t* oh, int32_t* ow);
/* (the choice among the kernel variants that compute a layer - hipie_conv_set_tile and its companions - is in
 * hipie_diag.h: hipie_compile makes it by measurement, a caller of the operator-level entry points may make it itself) */
int hipie_conv_run(const hipie_conv* conv, const hipie_tensor* in, const hipie_tensor* residual,
                   const hipie_tensor* out, void* stream);
/* Two consecutive convolutions in ONE kernel - the tail of a bottleneck block: `first` (3 x 3, stride 1, pad 1, bias,
 * FakeQuantize to bytes) is computed for whole output rows of one image over all of its 64, 128 or 256 output
 * channels, its level bytes stay in LDS in operand layout, and `second` (1 x 1 over exactly those channels, with its
 * bias, scale, byte residual and FakeQuantize) runs from there: the intermediate tensor is neither written nor read,
 * one launch instead of two.  Same arithmetic in the same order as hipie_conv_run on each layer, hence the same bits.
 * The CPU plugin fuses consecutive convolutions into one primitive the same way
 * (inference-engine/src/mkldnn_plugin/mkldnn_graph_optimizer.cpp:631-759 FuseConvolutionAndDWConvolution, and the
 * sum post-op of :958-1130).  `in` is the first layer's input, `residual` and `out` the second layer's;
 * hipie_conv_pair_fits says whether the kernel takes two layers on an input of h x w pixels (*fits = 0: no; bit 0
 * set: yes; bit 1: also in its form with eight waves per workgroup, see hipie_conv_set_stages in hipie_diag.h). */
int hipie_conv_pair_fits(const hipie_conv* first, const hipie_conv* second, int32_t h, int32_t w, int* fits);
int hipie_conv_run_pair(const hipie_conv* first, const hipie_conv* second, const hipie_tensor* in,
                        const hipie_tensor* residual, const hipie_tensor* out, void* stream);
/* hipie_conv_run for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments, same kernels,
 * same bits; the one piece of device memory hipie_conv_run allocates - the workspace through which variants 14 to
 * 17 pass their partial sums - is a fixed array inside the library instead (16 MB of partial sums = 256 blocks of
 * 64 KB, one per tile and part, and 1024 arrival counters; each device the library runs on holds it until the
 * process ends).  Launches that need more (tiles x parts > 256 or more than 1024 tiles) are refused with
 * HIPIE_OUT_OF_BOUNDS; nothing is allocated or freed.  All calls on one device share the array: calls that overlap
 * on one device (different streams or host threads) race on it and must be serialised by the caller. */
int hipie_conv_run_static(const hipie_conv* conv, const hipie_tensor* in, const hipie_tensor* residual,
                          const hipie_tensor* out, void* stream);

/* ======================================================================================
 * 1d. MatMul between two activations (attention scores and context) — reference::matmul<int32_t>
 *     on widened inputs (ngraph/core/reference/.../matmul.hpp:24-57 dot, :75-247 batching), as the
 *     TypeRelaxed MatMul LPT emits (low_precision_transformations/src/mat_mul.cpp:81-171), plus the
 *     fused epilogue.  out[b][i][j] = sum_k A[b][i][k] * Bt[b][j][k]: the right operand is passed
 *     in its transpose_b = true form ([N][K], K contiguous).  MatMul against constant weights is a
 *     1x1 convolution (hipie_conv_*).  Leading dimensions and batch strides are in elements.
 * ==================================================================================== */
typedef struct hipie_matmul_desc {
    int32_t a_dtype, b_dtype;   /* each HIPIE_I8 or HIPIE_U8B (u8 levels, e.g. a quantized Softmax or ReLU output) */
    int32_t k, n;               /* reduction length (multiple of 64), output columns */
    int32_t a_zero_point;       /* level of a u8 left operand that stands for 0.0 (0 for i8) */
    int32_t b_zero_point;       /* the same for the right operand.  (MatMulTransformation itself only rewrites a MatMul
                                 * between activations whose operands have no zero point, mat_mul.cpp:231-236, :265-267,
                                 * :290-292: 0 is what a transformed graph carries.) */
} hipie_matmul_desc;

typedef struct hipie_matmul hipie_matmul;

int hipie_matmul_create(int device, const hipie_matmul_desc* desc, const hipie_epilogue* epilogue,
                        hipie_matmul** matmul);
void hipie_matmul_destroy(hipie_matmul* matmul);
int hipie_matmul_run(const hipie_matmul* matmul, const void* a, int64_t lda, int64_t stride_a,
                     const void* b_transposed, int64_t ldb, int64_t stride_b, void* out, int64_t ldo,
                     int64_t stride_o, int32_t m, int32_t batch, void* stream);
/* Two-level batch, e.g. (sequence, head) with the heads of one sequence interleaved in a [T, 3H]
 * tensor: element (o, i), o < batch_outer, i < batch, starts at o * outer + i * stride of each operand. */
int hipie_matmul_run_nested(const hipie_matmul* matmul, const void* a, int64_t lda, int64_t stride_a, int64_t outer_a,
                            const void* b_transposed, int64_t ldb, int64_t stride_b, int64_t outer_b, void* out,
                            int64_t ldo, int64_t stride_o, int64_t outer_o, int32_t m, int32_t batch,
                            int32_t batch_outer, void* stream);
/* A u8 operand is stored as level - 128.  With a', b' the stored bytes and za, zb the zero points,
 *   sum_k (a_k - za)(b_k - zb) = sum_k a'_k b'_k + (128 - za) sum_k b'_k + (128 - zb) (sum_k a'_k + K (128 - za)):
 * the sums over K of the right operand's rows (u8 left operand; an activation here, not constant weights as in
 * mat_mul.cpp:95-121) and of the left operand's rows (u8 right operand) are computed on the stream in front of the
 * product, into a workspace of hipie_matmul_workspace_size(m, batch, batch_outer) bytes that the caller owns (one
 * per request in flight; 16-byte aligned; 0 bytes and not needed when both operands are i8). */
int hipie_matmul_workspace_size(const hipie_matmul* matmul, int32_t m, int32_t batch, int32_t batch_outer, size_t* bytes);
int hipie_matmul_run_nested_ws(const hipie_matmul* matmul, const void* a, int64_t lda, int64_t stride_a, int64_t outer_a,
                               const void* b_transposed, int64_t ldb, int64_t stride_b, int64_t outer_b, void* out,
                               int64_t ldo, int64_t stride_o, int64_t outer_o, int32_t m, int32_t batch,
                               int32_t batch_outer, void* workspace, size_t workspace_bytes, void* stream);

/* ======================================================================================
 * 1e. fp32 glue of the transformer path, over the last axis of a dense [rows, axis] f32 matrix
 *     (device pointers).  Tolerance parity only (GPU exp / erf differ from libm in the last ulp).
 *       hipie_softmax_f32  reference::softmax      (.../reference/softmax.hpp:20-50)
 *       hipie_mvn_f32      reference::mvn_6        (.../reference/mvn.hpp:64-117), optionally followed
 *                          by the LayerNorm Multiply(gamma[axis]) and Add(beta[axis]) (device arrays or NULL)
 *       hipie_gelu_f32     reference::gelu, ERF    (.../reference/gelu.hpp:18-28)
 * ==================================================================================== */
int hipie_softmax_f32(const float* x, float* y, int64_t rows, int64_t axis, void* stream);
int hipie_mvn_f32(const float* x, float* y, int64_t rows, int64_t axis, int normalize_variance, float eps,
                  int eps_inside_sqrt, const float* gamma, const float* beta, void* stream);
int hipie_gelu_f32(const float* x, float* y, int64_t n, void* stream);
/* The same three with the per-tensor FakeQuantize that consumes their result in a post-LPT encoder
 * fused in: q receives the i8 levels of FakeQuantize(result, in_low, in_high, out_low,
 * out_low + levels - 1, levels), bit-exact with hipie_fq_run_q8 applied to the f32 result (the
 * level index is evaluated in the reference's operation order, fake_quantize.hpp:175-194); y still
 * receives the f32 result unless it is NULL. */
typedef struct hipie_requant {
    float in_low, in_high, out_low;
    int64_t levels;
} hipie_requant;
int hipie_softmax_q8(const float* x, float* y, int8_t* q, int64_t rows, int64_t axis, const hipie_requant* requant,
                     void* stream);
int hipie_mvn_q8(const float* x, float* y, int8_t* q, int64_t rows, int64_t axis, int normalize_variance, float eps,
                 int eps_inside_sqrt, const float* gamma, const float* beta, const hipie_requant* requant, void* stream);
int hipie_gelu_q8(const float* x, float* y, int8_t* q, int64_t n, const hipie_requant* requant, void* stream);
/* reference::add with numpy broadcasting (ngraph/core/reference/include/ngraph/runtime/reference/add.hpp over
 * autobroadcast_binop.hpp) on the row-major path: y = x + addend for a dense f32 value of `rank` <= 4 dimensions
 * `dims` and an addend of the same rank whose dimensions are the value's or 1 (an attention mask [batch, 1, 1, seq]
 * on scores [batch, heads, seq, seq]).  One IEEE addition per element; x and y may be the same buffer. */
int hipie_add_broadcast_f32(const float* x, const int64_t* dims, const float* addend, const int64_t* addend_dims, int rank,
                            float* y, void* stream);
/* reference::slice with unit steps (ngraph/core/reference/include/ngraph/runtime/reference/slice.hpp; what
 * reference::split takes each of its outputs with): dst, dense, receives the `rank` <= 5 dimensional box `dims` of
 * src whose element (i0, .., i4) lies at sum(i_k * strides[k]) elements from src; elements of 1 or 4 bytes. */
int hipie_copy_strided(const void* src, const int64_t* dims, const int64_t* strides, int rank, int element_bytes, void* dst,
                       void* stream);
/* Embedding front end of an encoder — reference::gather (.../reference/gather.hpp:18-66) of rows of a
 * f32 table [vocabulary, hidden] by i32 token ids, followed by up to two reference::add steps in the
 * graph's order: out[t] = (table[ids[t]] + add0) + add1, each addend (device pointer, or NULL) either
 * one row [hidden] or one row per position [seq, hidden] (position embeddings; token t sits at
 * position t % seq).  Negative ids count from the end like the reference; ids outside the table
 * (undefined behaviour there) read its nearest row. */
int hipie_embedding_f32(const float* table, int64_t vocabulary, int64_t hidden, const int32_t* ids, int64_t tokens,
                        int64_t seq, const float* add0, int add0_per_position, const float* add1, int add1_per_position,
                        float* out, void* stream);
/* Self-attention core of a post-LPT encoder in one kernel, per (sequence, head):
 *     MatMul'(q, k^T) * score_scale [+ mask] -> Softmax -> FakeQuantize(prob_fq) -> MatMul'(., v) * context_scale
 *     [-> FakeQuantize(out_fq) when out_dtype is HIPIE_I8]
 * i.e. the two TypeRelaxed MatMuls low_precision_transformations/src/mat_mul.cpp:81-171 leaves, with
 * reference::softmax (softmax.hpp:20-50) and reference::fake_quantize between them.  q, k, v are i8
 * [seq, head_dim] matrices addressed like the operands of hipie_matmul_run_nested (row pitch, inner and
 * outer batch stride, in bytes); out is [seq, head_dim] f32 or i8 (pitch and strides in elements).
 * The integer products are exact and every f32 step is one IEEE operation in that order; Softmax
 * has tolerance parity.  mask, when not NULL, is the additive attention mask: one f32 row [seq] per
 * batch element (strides in elements; 0 shares a row between the heads of a sequence), added to the
 * scaled scores of every query (reference::add with numpy broadcast).  scores / probs, when not NULL, receive the f32 values in front of and
 * behind the Softmax as dense [batch_outer * batch][seq][seq] arrays (inspection; the kernel is
 * otherwise the same).  Sequence lengths: multiples of 32 up to 384; head_dim 64
 * (hipie_attention_supported). */
typedef struct hipie_attention_desc {
    int32_t seq, head_dim;
    float score_scale, context_scale;
    hipie_requant prob_fq;
    int32_t out_dtype;          /* HIPIE_F32 or HIPIE_I8 */
    hipie_requant out_fq;       /* used when out_dtype is HIPIE_I8 */
    int32_t prob_dtype;         /* HIPIE_I8 (also 0), or HIPIE_U8B: prob_fq gives u8 levels, out_low = first level - 128;
                                 * the context product then starts from 128 x the sums of V over the keys */
} hipie_attention_desc;
typedef struct hipie_attention hipie_attention;
int hipie_attention_supported(int32_t seq, int32_t head_dim);
/* device < 0 builds a host-only object (load-time checks without a GPU) */
int hipie_attention_create(int device, const hipie_attention_desc* desc, hipie_attention** attention);
void hipie_attention_destroy(hipie_attention* attention);
int hipie_attention_run(const hipie_attention* attention, const void* q, int64_t ldq, int64_t stride_q, int64_t outer_q,
                        const void* k, int64_t ldk, int64_t stride_k, int64_t outer_k, const void* v, int64_t ldv,
                        int64_t stride_v, int64_t outer_v, void* out, int64_t ldo, int64_t stride_o, int64_t outer_o,
                        int32_t batch, int32_t batch_outer, const float* mask, int64_t mask_stride, int64_t mask_outer,
                        float* scores, float* probs, void* stream);
/* Transpose of the two inner dimensions of a byte tensor (opset1 Transpose on quantized activations,
 * e.g. V [S, d] -> [d, S] so that the context MatMul finds its reduction axis contiguous;
 * reference::transpose, .../reference/transpose.hpp:20-25): dst[b][c][r] = src[b][r][c], leading
 * dimensions and batch strides in bytes. */
int hipie_transpose_bytes(const void* src, int64_t ld_src, int64_t batch_stride_src, void* dst, int64_t ld_dst,
                          int64_t batch_stride_dst, int32_t rows, int32_t cols, int32_t batch, void* stream);
/* two-level batch as in hipie_matmul_run_nested */
int hipie_transpose_bytes_nested(const void* src, int64_t ld_src, int64_t stride_src, int64_t outer_src, void* dst,
                                 int64_t ld_dst, int64_t stride_dst, int64_t outer_dst, int32_t rows, int32_t cols,
                                 int32_t batch, int32_t batch_outer, void* stream);

/* ======================================================================================
 * 2. Graph level.  The plugin's LoadExeNetworkImpl walks Function::get_ordered_ops()
 *    (ngraph/core/include/ngraph/function.hpp:126) of the post-LPT function and issues one call
 *    per node; value ids are returned in creation order.  Shapes are the reference's (NCHW,
 *    OIHW, [N, C]); element types are the node's output types (TypeRelaxed ops included).
 *    Supported nodes: Parameter(f32; u8 behind a Convert to f32; i32 token ids), Constant, FakeQuantize, Convolution, GroupConvolution,
 *    MatMul, Add, Multiply, Subtract, Relu, Clamp, Convert, MaxPool, AvgPool, Reshape, Result, and
 *    for transformer encoders (rank-3 Parameter [batch, sequence, hidden]): MatMul between two
 *    activations, Softmax, MVN, Gelu, Transpose, and Gather of a constant table by an i32
 *    Parameter [batch, sequence] (the embedding front end).
 * ==================================================================================== */
typedef struct hipie_graph hipie_graph;
typedef struct hipie_plan hipie_plan;
typedef struct hipie_request hipie_request;

/* hipie_graph_eltwise kinds.  PRELU: op::v0::PRelu(a, slope) = a < 0 ? a * slope : a (reference prelu.hpp:22-47; a
 * one-dimensional slope with one element per channel of `a` is taken per channel, any other broadcasts numpy-style) */
enum { HIPIE_OP_ADD = 6, HIPIE_OP_MULTIPLY = 7, HIPIE_OP_SUBTRACT = 8, HIPIE_OP_PRELU = 23 };
/* hipie_graph_activation kinds, f32 in and out (the low-precision transformations leave them in f32): Sigmoid
 * 1 / (1 + exp(-x)) (reference sigmoid.hpp), op::v4::HSwish x * min(max(x + 3, 0), 6) / 6 (hswish.hpp), op::v5::HSigmoid
 * min(max(x + 3, 0), 6) / 6 (hsigmoid.hpp), op::v4::Swish x / (1 + exp(-x * beta)) (swish.hpp; `beta` is read for
 * Swish only).  HSwish and HSigmoid are the reference's f32 operations one by one; Sigmoid and Swish use the device's
 * exp and agree to rounding. */
enum { HIPIE_OP_SIGMOID = 24, HIPIE_OP_HSWISH = 25, HIPIE_OP_HSIGMOID = 26, HIPIE_OP_SWISH = 27 };
int hipie_graph_activation(hipie_graph* g, int kind, int x, float beta, int* id);

int hipie_graph_create(hipie_graph** graph);
void hipie_graph_destroy(hipie_graph* graph);
int hipie_graph_parameter(hipie_graph* g, const char* name, int dtype, const int64_t* dims, int rank, int* id);
int hipie_graph_constant(hipie_graph* g, int dtype, const int64_t* dims, int rank, const void* data, int* id);
/* op::v0::FakeQuantize (TypeRelaxed when out_dtype is HIPIE_U8 / HIPIE_I8) */
int hipie_graph_fake_quantize(hipie_graph* g, int x, int in_low, int in_high, int out_low, int out_high,
                              int64_t levels, int out_dtype, int* id);
/* op::v1::Convolution / GroupConvolution and the pools below: x is [N, C, H, W] or [N, C, W] (a convolution's also
 * [N, C, D, H, W]); every attribute array holds one entry per spatial dimension of x.  A value with one spatial
 * dimension is planned as the same value with H = 1, the way reference::convolution extends its shapes
 * (convolution.hpp:148-167).  Over three spatial dimensions only convolutions with f32 weights are planned
 * (reference::convolution<float>'s loops as they stand, convolution.hpp:63-146); quantized ones and pools are
 * refused (HIPIE_NOT_IMPLEMENTED). */
int hipie_graph_convolution(hipie_graph* g, int x, int weights, const int64_t* strides,
                            const int64_t* dilations, const int64_t* pads_begin, const int64_t* pads_end,
                            int* id);
int hipie_graph_group_convolution(hipie_graph* g, int x, int weights, const int64_t* strides,
                                  const int64_t* dilations, const int64_t* pads_begin,
                                  const int64_t* pads_end, int* id);
int hipie_graph_matmul(hipie_graph* g, int a, int b, int transpose_a, int transpose_b, int* id);
int hipie_graph_eltwise(hipie_graph* g, int kind, int a, int b, int* id);
int hipie_graph_relu(hipie_graph* g, int x, int* id);
int hipie_graph_clamp(hipie_graph* g, int x, float min, float max, int* id);
int hipie_graph_convert(hipie_graph* g, int x, int dtype, int* id);
int hipie_graph_max_pool(hipie_graph* g, int x, const int64_t* kernel, const int64_t* strides,
                         const int64_t* pads_begin, const int64_t* pads_end, int ceil_mode, int* id);
int hipie_graph_avg_pool(hipie_graph* g, int x, const int64_t* kernel, const int64_t* strides,
                         const int64_t* pads_begin, const int64_t* pads_end, int exclude_pad, int ceil_mode,
                         int out_dtype, int* id);
int hipie_graph_reshape(hipie_graph* g, int x, const int64_t* dims, int rank, int* id);
/* op::v1::Softmax, op::v6::MVN (axes as an array), Gelu (ERF), op::v1::Transpose */
int hipie_graph_softmax(hipie_graph* g, int x, int64_t axis, int* id);
int hipie_graph_mvn(hipie_graph* g, int x, const int64_t* axes, int n_axes, int normalize_variance, float eps,
                    int eps_inside_sqrt, int* id);
int hipie_graph_gelu(hipie_graph* g, int x, int* id);
int hipie_graph_transpose(hipie_graph* g, int x, const int64_t* order, int rank, int* id);
/* op::v1::Gather with the axis Constant's value; planned as an embedding lookup: f32 Constant table
 * [vocabulary, hidden], i32 Parameter indices [batch, sequence], axis 0 */
int hipie_graph_gather(hipie_graph* g, int data, int indices, int64_t axis, int* id);
/* op::v0::Concat (ngraph/core/reference/include/ngraph/runtime/reference/concat.hpp:17-57: the inputs' elements copied
 * side by side along `axis`).  After the low-precision transformations a Concat of quantized branches takes their u8 /
 * i8 levels directly (low_precision_transformations/src/concat.cpp:42-190 gives every branch the same interval and
 * moves the dequantization behind the Concat), which is the form the engine runs: byte tensors along the channel axis. */
int hipie_graph_concat(hipie_graph* g, const int* inputs, int n_inputs, int64_t axis, int* id);
/* One output of op::v1::Split / op::v1::VariadicSplit: elements [begin, end) of x along `axis`, every other axis whole
 * (ngraph/core/reference/src/runtime/reference/split.cpp:14-45 takes each output with reference::slice of that box). */
int hipie_graph_slice(hipie_graph* g, int x, int64_t axis, int64_t begin, int64_t end, int* id);
int hipie_graph_result(hipie_graph* g, int x, const char* name);
int hipie_graph_set_name(hipie_graph* g, int id, const char* friendly_name);

/* IInferencePlugin::LoadExeNetworkImpl (ie_iplugin_internal.hpp:270-271): fuse, lay out the static
 * HBM arena, pack and upload constants.  The graph may be destroyed afterwards. */
int hipie_compile(const hipie_graph* graph, int device, hipie_plan** plan);
/* The same with the config map LoadExeNetworkImpl receives (template_plugin.cpp:95-104, template_config.cpp:16-57) as
 * n_opts key / value strings.  Keys: PERF_COUNT (YES | NO: default of hipie_request_create's perf_count = -1),
 * DEVICE_ID (must name `device`), HIP_THROUGHPUT_STREAMS (1 .. 8 or HIP_THROUGHPUT_AUTO: the requests assumed in
 * flight together; the kernel variants are timed that way and OPTIMAL_NUMBER_OF_INFER_REQUESTS reports it),
 * HIP_TUNE (YES | NO: time the kernel variants at load, else shape-based defaults), HIP_TUNE_FILE (cache of the
 * choices, like the reference GPU plugin's KEY_TUNING_FILE), HIP_FUSE_ATTENTION, HIP_MERGE_LINEAR, HIP_KEEP_F32
 * (YES | NO), HIP_FUSE_CONVOLUTIONS (a 3 x 3 convolution and the 1 x 1 convolution that alone reads its result as one
 * kernel, hipie_conv_run_pair: AUTO = where the load-time measurement finds it faster, YES = wherever the kernel takes
 * the pair, NO; the tensor between two layers run that way exists in LDS only and hipie_request_tensor gives
 * HIPIE_NOT_FOUND for it), NETWORK_NAME.  An unknown key gives HIPIE_NOT_FOUND, a value the key does not take
 * HIPIE_PARAMETER_MISMATCH.  The environment variables HIPIE_TUNE, HIPIE_TUNE_FILE, HIPIE_TUNE_STREAMS,
 * HIPIE_FUSE_ATTENTION, HIPIE_MERGE_LINEAR, HIPIE_KEEP_F32, HIPIE_FUSE_CONVS (0 | 1 | 2 = NO | AUTO | YES) are the
 * process-wide defaults of these keys. */
int hipie_compile_opts(const hipie_graph* graph, int device, const char* const* keys, const char* const* values,
                       int n_opts, hipie_plan** plan);
void hipie_plan_destroy(hipie_plan* plan);
/* IInferencePlugin::QueryNetwork (ie_iplugin_internal.hpp:255, template_plugin.cpp:117-195): supported[i] = 1 when
 * the engine can take node i of the graph, 0 when it cannot (every such node, not only the first); n_nodes must be
 * the graph's node count (ids are 0 .. n_nodes - 1 in the order the nodes were added); n_unsupported may be NULL.
 * Needs no device. */
int hipie_query(const hipie_graph* graph, int* supported, int n_nodes, int* n_unsupported);
/* IInferencePlugin::GetMetric (ie_iplugin_internal.hpp:188, template_plugin.cpp:218-259) as text (lists are
 * space-separated): SUPPORTED_METRICS, SUPPORTED_CONFIG_KEYS, AVAILABLE_DEVICES, FULL_DEVICE_NAME,
 * IMPORT_EXPORT_SUPPORT, DEVICE_ARCHITECTURE, OPTIMIZATION_CAPABILITIES, RANGE_FOR_ASYNC_INFER_REQUESTS,
 * RANGE_FOR_STREAMS; an unknown name gives HIPIE_NOT_FOUND, a buffer that is too small HIPIE_OUT_OF_BOUNDS. */
int hipie_get_metric(int device, const char* name, char* buf, size_t buf_len);
/* IExecutableNetworkInternal::GetMetric / GetConfig (template_executable_network.cpp:154-176): NETWORK_NAME,
 * SUPPORTED_METRICS, SUPPORTED_CONFIG_KEYS, OPTIMAL_NUMBER_OF_INFER_REQUESTS (what benchmark_app asks for,
 * samples/benchmark_app/main.cpp:456-472); the config keys of hipie_compile_opts with the values the plan was compiled with */
int hipie_plan_get_metric(const hipie_plan* plan, const char* name, char* buf, size_t buf_len);
int hipie_plan_get_config(const hipie_plan* plan, const char* key, char* buf, size_t buf_len);

/* IExecutableNetworkInternal::Export(std::ostream&) (ie_iexecutable_network_internal.hpp:77-81) and
 * IInferencePlugin::ImportNetwork(std::istream&, config) (ie_iplugin_internal.hpp:213-222), as the
 * template plugin implements them (template_executable_network.cpp:179-201 writes the model,
 * :43-75 reads it back and compiles it again).  The stream holds the graph description with its
 * constants and the kernel variant chosen for every step, so an imported plan skips the timing runs
 * of hipie_compile and runs the same kernels as the exported one; everything else (fusion, arena
 * layout, constant packing) is redone, through the same validation as a newly described graph.
 * hipie_plan_export with buffer == NULL only reports the size.  A stream that is truncated, damaged
 * (checksum), of another format version or not a plan gives HIPIE_NETWORK_NOT_READ. */
int hipie_plan_export(const hipie_plan* plan, void* buffer, size_t capacity, size_t* size);
int hipie_plan_import(const void* stream, size_t size, int device, hipie_plan** plan);
int hipie_plan_num_inputs(const hipie_plan* plan);
int hipie_plan_num_outputs(const hipie_plan* plan);
int hipie_plan_io_desc(const hipie_plan* plan, int is_output, int index, char* name, size_t name_len,
                       int* dtype, int64_t* dims /* [8]: ranks up to 8 */, int* rank);
int64_t hipie_plan_arena_bytes(const hipie_plan* plan);
/* executed (fused) steps, in order: the exec-graph / perf-counter view
 * (exec_graph_info.hpp:34-76, ie_common.h InferenceEngineProfileInfo) */
int hipie_plan_num_steps(const hipie_plan* plan);
int hipie_plan_step_info(const hipie_plan* plan, int index, char* name, size_t name_len, char* type,
                         size_t type_len, int64_t* macs, int64_t* bytes);
/* the kernel variant a step runs (hipie_conv_set_tile numbering), -1 for a step without variants: part
 * of what GetExecGraphInfo reports per executed node (exec_graph_info.hpp:34-76, implementation type) */
int hipie_plan_step_variant(const hipie_plan* plan, int index, int* variant);
/* the attributes GetExecGraphInfo attaches to every executed node (exec_graph_info.hpp:34-76), by their key there:
 * originalLayersNames (comma-separated graph nodes the step stands for), layerType, runtimePrecision (U8 / I8 for the
 * integer kernels: the type of the activations they multiply, as the CPU plugin reports it; FP32 otherwise),
 * outputPrecisions, outputLayouts, execOrder, primitiveType ("hip_int8_v<variant>" | "hip"); execTimeMcs is
 * hipie_request_perf.  HIPIE_NOT_FOUND for another key.  Beside the reference's keys: "kernels" (launches the
 * step enqueues), "outputDims" (the shape of what it stores, comma separated, in the graph's dimension order),
 * "epilogueFlags" (the f32 chain fused behind a convolution as its flag word, 0 for other steps) and "valuOps" (results
 * x vector instructions of that chain: what the step asks of the vector pipe whatever kernel runs it). */
int hipie_plan_step_rt_info(const hipie_plan* plan, int index, const char* key, char* buf, size_t buf_len);
/* The edges of that graph: where the operands of step `index` come from - sources[i] >= 0 is the index of the step that
 * produced one, sources[i] < 0 stands for graph input -(1 + sources[i]).  *count receives their number (at most
 * `capacity` are written).  A step of layerType "Result" is what an output of the plan is read from. */
int hipie_plan_step_sources(const hipie_plan* plan, int index, int* sources, int capacity, int* count);

/* IExecutableNetworkInternal::CreateInferRequestImpl: own stream + own activation arena; weights
 * stay shared in the plan.  perf_count mirrors the PERF_COUNT config key (ie_plugin_config.hpp:277). */
int hipie_request_create(const hipie_plan* plan, int perf_count /* 1, 0, or -1 = the plan's PERF_COUNT */, hipie_request** request);
void hipie_request_destroy(hipie_request* request);
/* IInferRequestInternal::InferImpl (ie_iinfer_request_internal.hpp:57).  inputs / outputs are dense
 * NCHW buffers in plan order: host memory (device_memory = 0: H2D, kernels, D2H on the request's
 * stream) or device memory (device_memory = 1: kernels only). */
int hipie_request_infer(hipie_request* request, const void* const* inputs, void* const* outputs,
                        int device_memory);
/* StartAsync / Wait(RESULT_READY) (ie_infer_async_request_thread_safe_default.hpp:167-214) */
int hipie_request_start(hipie_request* request, const void* const* inputs, void* const* outputs,
                        int device_memory);
int hipie_request_wait(hipie_request* request);
/* Wait(millis_timeout) (ie_infer_async_request_thread_safe_default.hpp:167-204): -1 = RESULT_READY (block; the same
 * as hipie_request_wait), 0 = STATUS_ONLY (ask, do not wait), > 0 = wait at most that many milliseconds.
 * HIPIE_RESULT_NOT_READY: still running, the request stays busy; HIPIE_INFER_NOT_STARTED: nothing was started;
 * HIPIE_INFER_CANCELLED: the inference was cancelled (below), the request is idle again. */
int hipie_request_wait_for(hipie_request* request, int64_t timeout_ms);
/* Cancel (ie_infer_async_request_thread_safe_default.hpp:255-267).  Work that is queued on the request's stream runs
 * to its end (nothing on the device is revoked); the outputs are undefined and the next wait gives
 * HIPIE_INFER_CANCELLED.  On an idle request it does nothing. */
int hipie_request_cancel(hipie_request* request);
/* enqueue the kernels only, on the request's stream, without copies or synchronisation */
int hipie_request_enqueue(hipie_request* request, const void* const* inputs, void* const* outputs);
int hipie_request_stream(hipie_request* request, void** stream);
/* milliseconds of step `index` in the last inference (GetPerformanceCounts) */
int hipie_request_perf(hipie_request* request, int index, float* ms);
/* the arena tensor holding the value of graph node `node_id` (inspection, parity tests) */
int hipie_request_tensor(const hipie_request* request, int node_id, hipie_tensor* tensor);

/* ======================================================================================
 * 3. Load-time arithmetic of the low-precision transformations (host only), for harnesses that
 *    build post-LPT graphs without OpenVINO.  Reference, all under
 *    inference-engine/src/low_precision_transformations/:
 *      src/layer_transformation.cpp:194-273          getPrecisionDetails
 *      include/low_precision/layer_transformation.hpp:63-107   DataPrecision::getMin/MaxValue
 *      src/network_helper.cpp:943-1087               decomposeFakeQuantize (scale, shift, clamp)
 *      src/network_helper.cpp:700-827                foldFakeQuantize (i8 weights)
 *      src/network_helper.cpp:216-292                swapMultiplyAndAdd (bias in front of the dequantization)
 *      src/fake_quantize.cpp:127-183                 fuseElementwise (dequantization folded into the next range)
 *      src/add.cpp:154-218                           AddTransformation, dequantizations on both branches
 *      src/clamp.cpp:71-89                           Clamp bounds in front of a per-tensor dequantization
 * ==================================================================================== */
enum { HIPIE_LPT_MULTIPLY = 1, HIPIE_LPT_SUBTRACT = 2, HIPIE_LPT_ADD = 3 };
int hipie_lpt_precision_details(int64_t levels, const float* out_low, const float* out_high, int64_t n,
                                int* precision, int* has_negative, int* has_zero_point);
int hipie_lpt_data_precision_range(int precision, int64_t levels, float* min, float* max);
int hipie_lpt_decompose_fake_quantize(const float* out_low, const float* out_high, int64_t n, float min,
                                      float max, float* scales, float* shifts, float* new_low,
                                      float* new_high);
int hipie_lpt_fold_fake_quantize(const float* values, int64_t oc, int64_t inner, const float* in_low,
                                 int64_t n_in_low, const float* in_high, int64_t n_in_high,
                                 const float* out_low, int64_t n_out_low, const float* out_high,
                                 int64_t n_out_high, int64_t levels, int round_values, float* out);

int hipie_lpt_swap_multiply_and_add(const float* b, int64_t n_b, const float* a, int64_t n_a, float* b_over_a, int64_t n);
int hipie_lpt_fuse_elementwise(int kind, const float* in_low, const float* in_high, int64_t n_range, const float* value,
                               int64_t n_value, float* new_low, float* new_high, int64_t n, int* fused);
int hipie_lpt_add_both_branches(const float* shift_full, const float* scale_full, const float* shift_empty,
                                const float* scale_empty, int64_t n, float* new_shift_full, float* new_scale_full,
                                float* scale_after);
int hipie_lpt_clamp_bounds(double min, double max, double scale, double shift, double* new_min, double* new_max);

#ifdef __cplusplus
}
#endif
#endif /* HIPIE_H */
