// Planner: post-LPT graph -> fused steps over one static HBM arena -> infer requests.
//
// The matcher walks the graph demand-driven from the Results.  A Convolution / MatMul head
// absorbs the elementwise chain LPT leaves behind it (Add bias, dequantization Multiply, residual
// Add, ReLU/Clamp, FakeQuantize) into one kernel epilogue; Convert/Subtract/Multiply chains over
// byte tensors stay symbolic ("dequantization views") until a consumer fuses or materialises
// them.  Every materialised tensor gets its own arena region (NHWC, padded channels, a halo as
// wide as the largest padding among its consumers, pre-filled with level 0 once); nothing is
// allocated or freed after compilation.
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <map>
#include <mutex>

#include "convf.h"
#include "fq.h"
#include "graph.h"
#include "requant.h"

namespace hipie {
namespace {

struct TensorInfo {
    int dtype = HIPIE_U8B;   // storage type
    int n = 1, h = 1, w = 1, c = 1, cs = 16, halo = 0;
    int64_t offset = 0, bytes = 0;
    int producer = -1;       // graph node whose value it holds
    int alias = -1;          // shares the bytes of this earlier tensor (same element count, other row split)
    int fill_level = 0;      // level held by the halo and the channel padding (a consumer's zero point)
    std::vector<int> fill_levels;   // one level per channel instead (a consumer with per-channel zero points), or empty
    bool fill_fixed = false; // a consumer depends on fill_level / fill_levels
    int64_t esize() const { return dtype == HIPIE_F32 || dtype == HIPIE_I32 ? 4 : 1; }
    int wp() const { return w + 2 * halo; }
    int hp() const { return h + 2 * halo; }
    hipie_tensor desc(uint8_t* arena) const {
        hipie_tensor t;
        t.dtype = dtype; t.n = n; t.h = h; t.w = w; t.c = c;
        t.stride_w = cs;
        t.stride_h = static_cast<int64_t>(wp()) * cs;
        t.stride_n = static_cast<int64_t>(hp()) * wp() * cs;
        t.halo = halo;
        t.data = arena + offset + (static_cast<int64_t>(halo) * wp() + halo) * cs * esize();
        return t;
    }
};

enum ValueKind { VK_NONE = 0, VK_PARAM, VK_CONST, VK_TENSOR, VK_DEQ, VK_FUSED, VK_MAT };

// Row-major strided view of an arena tensor or of a request input buffer: how the values of a
// transformer encoder (rank-3 Parameter [batch, sequence, hidden] and everything computed from it)
// are held.  Memory order is the graph's own dimension order, so Reshape and Transpose are
// arithmetic on shape / stride and move no bytes.
struct View {
    int tensor = -1, param = -1;
    int dtype = HIPIE_F32;
    std::vector<int64_t> shape, stride;   // stride in elements
    int64_t offset = 0;                   // elements
    int64_t esize() const { return dtype == HIPIE_F32 || dtype == HIPIE_I32 ? 4 : 1; }
    int64_t numel() const {
        int64_t n = 1;
        for (auto d : shape) n *= d;
        return n;
    }
    size_t rank() const { return shape.size(); }
    static std::vector<int64_t> dense_strides(const std::vector<int64_t>& shape) {
        std::vector<int64_t> st(shape.size());
        int64_t s = 1;
        for (size_t i = shape.size(); i-- > 0;) {
            st[i] = s;
            s *= shape[i];
        }
        return st;
    }
    bool dense() const {
        int64_t s = 1;
        for (size_t i = shape.size(); i-- > 0;) {
            if (shape[i] != 1 && stride[i] != s) return false;
            s *= shape[i];
        }
        return true;
    }
    uint8_t* ptr(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs) const {
        uint8_t* base = tensor >= 0 ? arena + tensors[tensor].offset : static_cast<uint8_t*>(inputs[param]);
        return base + offset * esize();
    }
};

struct Value {
    int kind = VK_NONE;
    int tensor = -1;
    std::vector<float> sub, mul;   // VK_DEQ: (float(q) - sub) * mul, each empty / 1 / C values
    View view;                     // VK_MAT
    bool flat = false;             // the [N, C, H, W] byte tensor stands for its Reshape to [N, C * H * W] (read by a MatMul)
};

struct EpilogueSpec {
    std::vector<float> bias, scale, res_sub, res_mul, post_scale, fq_il, fq_ih;
    int residual_dtype = 0, activation = 0, out_dtype = HIPIE_F32;
    float clamp_lo = 0, clamp_hi = 0, fq_ol = 0, fq_oh = 0;
    int64_t levels = 0;
    hipie_epilogue c_struct() const {
        hipie_epilogue e{};
        auto set = [](const std::vector<float>& v, const float*& p, int64_t& n) {
            if (!v.empty()) { p = v.data(); n = static_cast<int64_t>(v.size()); }
        };
        set(bias, e.bias, e.n_bias);
        set(scale, e.scale, e.n_scale);
        e.residual_dtype = residual_dtype;
        set(res_sub, e.res_sub, e.n_res_sub);
        set(res_mul, e.res_mul, e.n_res_mul);
        set(post_scale, e.post_scale, e.n_post_scale);
        e.activation = activation;
        e.clamp_lo = clamp_lo;
        e.clamp_hi = clamp_hi;
        e.out_dtype = out_dtype;
        e.fq_levels = levels;
        set(fq_il, e.fq_in_low, e.n_fq_in_low);
        set(fq_ih, e.fq_in_high, e.n_fq_in_high);
        e.fq_out_low = fq_ol;
        e.fq_out_high = fq_oh;
        return e;
    }
};

struct TuneLane {
    uint8_t* arena;
    hipStream_t stream;
    std::vector<void*> inputs;   // the scratch request's input buffers
};

struct Step {
    std::string name, type;
    int64_t macs = 0, bytes = 0;
    int out_node = -1;
    // exec-graph attributes (exec_graph_info.hpp:34-76), filled once the plan is complete: the graph nodes this step
    // stands for, the type it computes in (the CPU plugin reports its kernels' input type there: U8 / I8 for the
    // integer kernels) and the type and layout of what it stores
    std::string original_names, runtime_precision, output_precision, output_layout, output_dims;
    std::vector<int> nodes;      // the graph nodes the step stands for (its own and every node fused into it)
    std::vector<int> sources;    // where its operands come from: a step's index, or -(1 + k) for graph input k
    bool f32_kernel = false;     // computes in f32 whatever type its operand is stored in (an unquantized layer)
    virtual ~Step() = default;
    virtual void create(int device, const std::vector<TensorInfo>& tensors) = 0;
    virtual void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs,
                     void* const* outputs, hipStream_t s) const = 0;
    // pick the fastest kernel variant by timing it on a scratch arena (load time, optional)
    // `lanes`: scratch arenas and streams of as many requests as are expected in flight together; a
    // variant is timed with one copy of the layer running on every lane at once
    virtual void tune(const std::vector<TuneLane>&, const std::vector<TensorInfo>&) {}
    // the chosen variant as an integer (-1: the step has no variants), and its inverse
    virtual int variant() const { return -1; }
    virtual void set_variant(int) {}
    virtual int launches() const { return 1; }   // kernels the step enqueues
    // vector instructions x lanes the step's f32 chain needs per inference (results x epilogue_valu_ops); 0: not counted
    virtual double valu_ops() const { return 0.0; }
    virtual uint32_t epilogue_flags() const { return 0u; }   // the fused f32 chain of a convolution step as its flag word
};

void check_status(int st, const char* what) {
    if (st != HIPIE_OK) fail(static_cast<hipie_status>(st), "%s: %s", what, hipie_last_error());
}

// FakeQuantize on a graph input: f32 NCHW in the request's input buffer -> byte NHWC tensor
struct EntryStep : Step {
    int param_index = 0, out = -1;
    bool u8_in = false;            // the request input holds u8 values (Parameter u8 -> Convert f32 -> FakeQuantize)
    int64_t channels = 0, levels = 0;
    std::vector<float> il, ih, ol, oh;
    hipie_fq* fq = nullptr;
    ~EntryStep() override { hipie_fq_destroy(fq); }
    void create(int device, const std::vector<TensorInfo>&) override {
        check_status(hipie_fq_create(device, channels, levels, il.data(), il.size(), ih.data(), ih.size(),
                                     ol.data(), ol.size(), oh.data(), oh.size(), &fq), name.c_str());
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*,
             hipStream_t s) const override {
        const hipie_tensor d = tensors[out].desc(arena);
        check_status(u8_in ? hipie_fq_run_q8_tensor_u8(fq, static_cast<const uint8_t*>(inputs[param_index]), &d, s)
                           : hipie_fq_run_q8_tensor(fq, static_cast<const float*>(inputs[param_index]), &d, s),
                     name.c_str());
    }
};

struct ConvStep : Step {
    int in = -1, res = -1, out = -1;
    int res_param = -1;            // f32 residual read from this request input instead of the arena
    hipie_conv_desc desc{};
    std::vector<int8_t> weights;   // OIHW
    EpilogueSpec epi;
    std::vector<int32_t> zero_points;   // per input channel (a per-channel Subtract in front of the convolution), or empty
    std::vector<int32_t> acc_sub;       // per output channel (the Subtract behind a MatMul with a zero point), or empty
    hipie_conv* conv = nullptr;
    int64_t results = 0;           // elements of the output tensor
    int64_t in_w_bytes = 0;        // input + weight bytes (what a fused consumer still has to read)
    // projection shortcut (Conv' -> Add -> Multiply, f32, used only by this step's residual Add):
    // run inside this step's kernel when the fused form applies, else right before it
    std::unique_ptr<ConvStep> shortcut;
    bool fused = false;
    float tuned_us = 0.f;          // per launch with every tuning lane busy, of the variant the tuner kept (0: not tuned)
    ~ConvStep() override { hipie_conv_destroy(conv); }
    void fill_desc(const std::vector<TensorInfo>& tensors) {
        const TensorInfo& t = tensors[in];
        desc.in_dtype = t.dtype;
        desc.in_c_stride = t.cs;
        desc.in_stride_w = t.cs;
        desc.in_stride_h = t.wp() * t.cs;
        desc.in_zero_points = zero_points.empty() ? nullptr : zero_points.data();
        desc.acc_sub = acc_sub.empty() ? nullptr : acc_sub.data();
    }
    void create(int device, const std::vector<TensorInfo>& tensors) override {
        fill_desc(tensors);
        if (shortcut) {
            shortcut->fill_desc(tensors);
            EpilogueSpec fe = epi;
            fe.residual_dtype = HIPIE_RESIDUAL_SHORTCUT_CONV;
            const hipie_epilogue e = fe.c_struct();
            const EpilogueSpec& se = shortcut->epi;
            const int st = hipie_conv_create_fused(device, &desc, weights.data(), &e, &shortcut->desc,
                                                   shortcut->weights.data(), se.bias.data(), se.bias.size(),
                                                   se.scale.data(), se.scale.size(), &conv);
            if (st == HIPIE_OK) {
                fused = true;
                type = "Convolution+Shortcut";
            } else if (st == HIPIE_NOT_IMPLEMENTED) {
                shortcut->create(device, tensors);   // run it as its own kernel, f32 through the arena
            } else {
                check_status(st, name.c_str());
            }
        }
        if (!fused) {
            const hipie_epilogue e = epi.c_struct();
            check_status(hipie_conv_create(device, &desc, weights.data(), &e, &conv), name.c_str());
        }
        weights.clear();
        weights.shrink_to_fit();
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const* outputs,
             hipStream_t s) const override {
        const hipie_tensor i = tensors[in].desc(arena), o = tensors[out].desc(arena);
        hipie_tensor r{};
        if (fused) {
            r = tensors[shortcut->in].desc(arena);
        } else {
            if (shortcut) shortcut->run(arena, tensors, inputs, outputs, s);
            if (res >= 0) r = tensors[res].desc(arena);
            else if (res_param >= 0) r = input_residual(o, inputs[res_param]);
        }
        check_status(hipie_conv_run(conv, &i, (fused || res >= 0 || res_param >= 0) ? &r : nullptr, &o, s), name.c_str());
    }
    // a dense f32 [rows, channels] request input as the residual operand of output tensor `o`
    static hipie_tensor input_residual(const hipie_tensor& o, void* data) {
        hipie_tensor r = o;
        r.data = data;
        r.dtype = HIPIE_F32;
        r.stride_w = o.c;
        r.stride_h = static_cast<int64_t>(o.w) * o.c;
        r.stride_n = static_cast<int64_t>(o.h) * r.stride_h;
        r.halo = 0;
        return r;
    }
    int launches() const override { return shortcut && !fused ? 2 : 1; }
    uint32_t epilogue_flags() const override {
        uint32_t flags = 0;
        int specialised = 0;
        return conv && hipie_conv_epilogue_flags(conv, &flags, &specialised) == HIPIE_OK ? flags : 0u;
    }
    double valu_ops() const override {
        uint32_t flags = 0;
        int specialised = 0;
        if (!conv || hipie_conv_epilogue_flags(conv, &flags, &specialised) != HIPIE_OK) return 0.0;
        return static_cast<double>(results) * epilogue_valu_ops(flags) + (shortcut && !fused ? shortcut->valu_ops() : 0.0);
    }
    bool deep = false;             // variant 24 with nine steps of weights in flight (hipie_conv_set_stages)
    // kernel variant (hipie_conv_set_tile) + 32 for `deep`
    int variant() const override {
        int t = -1;
        if (conv) (void)hipie_conv_get_tile(conv, &t);
        return t < 0 ? t : t + (deep ? 32 : 0);
    }
    void set_variant(int v) override {
        if (!conv || v < 0) return;
        check_status(hipie_conv_set_tile(conv, v & 31), name.c_str());
        deep = (v & 32) != 0;
        check_status(hipie_conv_set_stages(conv, deep ? 8 : 0), name.c_str());
    }
    // Every variant computes the same integers, so the choice changes time only.  Variants a layer
    // cannot use are refused by hipie_conv_set_tile and skipped.
    void tune(const std::vector<TuneLane>& lanes, const std::vector<TensorInfo>& tensors) override {
        if (shortcut && !fused) shortcut->tune(lanes, tensors);
        int current = -1;
        check_status(hipie_conv_get_tile(conv, &current), name.c_str());
        if (current < 0) return;
        const size_t nl = lanes.size();
        std::vector<hipie_tensor> ti(nl), to(nl), tr(nl);
        for (size_t l = 0; l < nl; ++l) {
            ti[l] = tensors[in].desc(lanes[l].arena);
            to[l] = tensors[out].desc(lanes[l].arena);
            if (fused) tr[l] = tensors[shortcut->in].desc(lanes[l].arena);
            else if (res >= 0) tr[l] = tensors[res].desc(lanes[l].arena);
            else if (res_param >= 0) tr[l] = input_residual(to[l], lanes[l].inputs[res_param]);
        }
        const bool has_res = fused || res >= 0 || res_param >= 0;
        auto launch_all = [&](int times) {
            for (int w = 0; w < times; ++w)
                for (size_t l = 0; l < nl; ++l)
                    check_status(hipie_conv_run(conv, &ti[l], has_res ? &tr[l] : nullptr, &to[l], lanes[l].stream), name.c_str());
        };
        std::vector<hipEvent_t> e0(nl), e1(nl);
        for (size_t l = 0; l < nl; ++l) {
            HIPIE_CHECK_HIP(hipEventCreate(&e0[l]));
            HIPIE_CHECK_HIP(hipEventCreate(&e1[l]));
        }
        int best = current;
        float best_ms = 0.f, few_ms = -1.f;
        const int candidates[] = {current, 0, 1, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20, 21, 22, 23, 24, 24 + 32};
        for (size_t c = 0; c < sizeof(candidates) / sizeof(candidates[0]); ++c) {
            // (1 stands for 2 as well on a depthwise layer, whose third variant is the matrix-pipe form; the dense variant 2
            // is a tile shape that no layer of a batch wants)
            for (int alt = 0; alt < (desc.groups > 1 && candidates[c] == 1 ? 2 : 1); ++alt) {
            const int tile = alt ? 2 : (candidates[c] & 31);
            if (c > 0 && candidates[c] == current && !alt) continue;
            if (hipie_conv_set_tile(conv, tile) != HIPIE_OK) continue;
            int applied = -1;
            check_status(hipie_conv_get_tile(conv, &applied), name.c_str());
            if (applied != tile) continue;   // not available for this layer (kept its previous variant)
            check_status(hipie_conv_set_stages(conv, (candidates[c] & 32) ? 8 : 0), name.c_str());
            launch_all(2);
            // the fastest of three rounds of five launches: a round disturbed by something else on the
            // device (another plan being compiled, a clock step) does not decide the choice
            float ms = 0.f;
            for (int round = 0; round < 3; ++round) {
                for (size_t l = 0; l < nl; ++l) HIPIE_CHECK_HIP(hipStreamSynchronize(lanes[l].stream));
                for (size_t l = 0; l < nl; ++l) HIPIE_CHECK_HIP(hipEventRecord(e0[l], lanes[l].stream));
                launch_all(5);
                for (size_t l = 0; l < nl; ++l) HIPIE_CHECK_HIP(hipEventRecord(e1[l], lanes[l].stream));
                for (size_t l = 0; l < nl; ++l) HIPIE_CHECK_HIP(hipEventSynchronize(e1[l]));
                float span = 0.f;   // earliest start to latest end
                for (size_t a = 0; a < nl; ++a)
                    for (size_t b = 0; b < nl; ++b) {
                        float t = 0.f;
                        HIPIE_CHECK_HIP(hipEventElapsedTime(&t, e0[a], e1[b]));
                        span = std::max(span, t);
                    }
                ms = round == 0 ? span : std::min(ms, span);
            }
            // a variant has to beat the best so far by more than the timing noise of seven launches,
            // otherwise the choice (and the run-to-run spread of a whole network) follows the noise
            if ((c == 0 && !alt) || ms < 0.97f * best_ms) {
                best_ms = ms;
                best = alt ? 2 : candidates[c];
            }
            if (tile == 23) few_ms = ms;
            }
        }
        // The candidates are timed back to back, their weights hot in the caches; in the network every other layer's
        // weights and tensors pass through between two uses.  A layer of a few pixels is little else than its weight
        // stream: the few-pixel kernel asks for the whole of it at once where the tiled kernels walk it in dependent
        // K steps (the FC layer of a batch-64 ResNet-50 in the network: 13.9 against 19.4 us, timed hot 11.7 against
        // 11.0), so it is taken when it comes within 30 % of the fastest.
        {
            const int64_t pixels = static_cast<int64_t>(to[0].n) * to[0].h * to[0].w;
            if (few_ms > 0.f && best != 23 && pixels <= 256 && few_ms <= 1.3f * best_ms) {
                best = 23;
                best_ms = few_ms;
            }
        }
        for (size_t l = 0; l < nl; ++l) {
            (void)hipEventDestroy(e0[l]);
            (void)hipEventDestroy(e1[l]);
        }
        set_variant(best);
        tuned_us = best_ms * 200.f / static_cast<float>(nl);
        if (std::getenv("HIPIE_TUNE_LOG")) {
            uint32_t fl = 0;
            int spec = 0;
            (void)hipie_conv_epilogue_flags(conv, &fl, &spec);
            std::fprintf(stderr, "hipie tune: %-28s variant %d (%.1f us per launch with %zu in flight; default %d) epilogue %#x%s\n",
                         name.c_str(), best, best_ms * 200.f / static_cast<float>(nl), nl, current, fl, spec ? "" : " GENERIC");
        }
    }
};


// A 3 x 3 convolution and the 1 x 1 convolution that is its only reader (the tail of a bottleneck block), planned as
// two layers and run either one after the other or - where hipie_conv_pair_fits takes them and it is faster - as one
// kernel that keeps the tensor between them in LDS (hipie_conv_run_pair).  Same bits either way.
struct PairStep : Step {
    std::unique_ptr<ConvStep> first, second;
    int mode = 1;                  // PlanConfig::fuse_convs
    bool fits = false, fused = false, fits_groups = false;
    // form of the fused kernel: 0 three steps of weights in flight, 1 nine steps (one workgroup per compute unit),
    // 2 eight waves in two groups (where fits_groups)
    int form = 0;
    static int stages_of(int form) { return form == 1 ? 8 : (form == 2 ? 7 : 0); }
    void create(int, const std::vector<TensorInfo>& tensors) override {   // (the layers exist already)
        name = second->name;
        macs = first->macs + second->macs;
        out_node = second->out_node;
        original_names = first->original_names + "," + second->original_names;
        nodes = first->nodes;
        nodes.insert(nodes.end(), second->nodes.begin(), second->nodes.end());
        output_dims = second->output_dims;
        runtime_precision = first->runtime_precision;
        output_precision = second->output_precision;
        output_layout = second->output_layout;
        const TensorInfo& ti = tensors[first->in];
        int f = 0;
        check_status(hipie_conv_pair_fits(first->conv, second->conv, ti.h, ti.w, &f), name.c_str());
        fits = f != 0 && ti.halo >= 1 && second->res >= 0 && second->res_param < 0;
        fits_groups = fits && (f & 2) != 0;
        const TensorInfo& tm = tensors[first->out];
        mid_bytes = static_cast<int64_t>(tm.n) * tm.h * tm.w * tm.c;
        choose(fits && mode == 2);
    }
    int64_t mid_bytes = 0;         // the tensor between the layers: written and read when they run apart
    void choose(bool one_kernel) {
        fused = one_kernel;
        // the depth is a setting of the first layer's object: the pair's when they run as one kernel, else its own
        if (first->conv) check_status(hipie_conv_set_stages(first->conv, fused ? stages_of(form) : (first->deep ? 8 : 0)), name.c_str());
        type = fused ? "Convolution+Convolution" : "Convolution,Convolution";
        bytes = first->bytes + second->bytes - (fused ? 2 * mid_bytes : 0);
    }
    int launches() const override { return fused ? 1 : first->launches() + second->launches(); }
    double valu_ops() const override { return first->valu_ops() + second->valu_ops(); }
    void run_fused(uint8_t* arena, const std::vector<TensorInfo>& tensors, hipStream_t s) const {
        const hipie_tensor i = tensors[first->in].desc(arena), o = tensors[second->out].desc(arena), r = tensors[second->res].desc(arena);
        check_status(hipie_conv_run_pair(first->conv, second->conv, &i, &r, &o, s), name.c_str());
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const* outputs,
             hipStream_t s) const override {
        if (fused) {
            run_fused(arena, tensors, s);
        } else {
            first->run(arena, tensors, inputs, outputs, s);
            second->run(arena, tensors, inputs, outputs, s);
        }
    }
    void tune(const std::vector<TuneLane>& lanes, const std::vector<TensorInfo>& tensors) override {
        first->tune(lanes, tensors);
        second->tune(lanes, tensors);
        if (!fits || mode == 0) return;
        const size_t nl = lanes.size();
        std::vector<hipEvent_t> e0(nl), e1(nl);
        for (size_t l = 0; l < nl; ++l) {
            HIPIE_CHECK_HIP(hipEventCreate(&e0[l]));
            HIPIE_CHECK_HIP(hipEventCreate(&e1[l]));
        }
        auto launch_all = [&](int times) {
            for (int w = 0; w < times; ++w)
                for (size_t l = 0; l < nl; ++l) run_fused(lanes[l].arena, tensors, lanes[l].stream);
        };
        float best_fused = 0.f;
        for (int d = 0; d < (fits_groups ? 3 : 2); ++d) {
        check_status(hipie_conv_set_stages(first->conv, stages_of(d)), name.c_str());
        launch_all(2);
        float ms = 0.f;   // the same protocol as the layers' own variants: fastest of three rounds of five launches per lane
        for (int round = 0; round < 3; ++round) {
            for (size_t l = 0; l < nl; ++l) HIPIE_CHECK_HIP(hipStreamSynchronize(lanes[l].stream));
            for (size_t l = 0; l < nl; ++l) HIPIE_CHECK_HIP(hipEventRecord(e0[l], lanes[l].stream));
            launch_all(5);
            for (size_t l = 0; l < nl; ++l) HIPIE_CHECK_HIP(hipEventRecord(e1[l], lanes[l].stream));
            for (size_t l = 0; l < nl; ++l) HIPIE_CHECK_HIP(hipEventSynchronize(e1[l]));
            float span = 0.f;
            for (size_t a = 0; a < nl; ++a)
                for (size_t b = 0; b < nl; ++b) {
                    float t = 0.f;
                    HIPIE_CHECK_HIP(hipEventElapsedTime(&t, e0[a], e1[b]));
                    span = std::max(span, t);
                }
            ms = round == 0 ? span : std::min(ms, span);
        }
        if (d == 0 || ms < 0.97f * best_fused) {
            best_fused = ms;
            form = d;
        }
        }
        for (size_t l = 0; l < nl; ++l) {
            (void)hipEventDestroy(e0[l]);
            (void)hipEventDestroy(e1[l]);
        }
        const float fused_us = best_fused * 200.f / static_cast<float>(nl), apart_us = first->tuned_us + second->tuned_us;
        choose(mode == 2 || (apart_us > 0.f && fused_us < 0.97f * apart_us));
        if (std::getenv("HIPIE_TUNE_LOG"))
            std::fprintf(stderr, "hipie tune: %-28s one kernel %.1f us (%s), two %.1f us per launch with %zu in flight: %s\n", name.c_str(),
                         fused_us, form == 2 ? "two wave groups" : (form == 1 ? "nine steps in flight" : "three steps in flight"), apart_us, nl,
                         fused ? "fused" : "apart");
    }
    // the layers' variants and the choice between one kernel and two, in one integer
    int variant() const override { return first->variant() + 64 * second->variant() + (fused ? 4096 : 0) + 8192 * form; }
    void set_variant(int v) override {
        if (v < 0) return;
        first->set_variant(v & 63);
        second->set_variant((v >> 6) & 63);
        form = (v >> 13) & 3;
        if (form == 3 || (form == 2 && !fits_groups)) form = 0;
        choose(fits && (v & 4096) != 0 && mode != 0);
    }
};

struct PoolStep : Step {
    int in = -1, out = -1;
    bool avg = false, rcp = false;
    PoolArgs a{};
    std::vector<float> mul, fq_il, fq_ih;
    float fq_ol = 0, fq_oh = 0;
    int64_t levels = 0;
    DeviceBuffer d_mul, d_il, d_ih, d_d, d_r;
    void create(int device, const std::vector<TensorInfo>& tensors) override {
        const TensorInfo& ti = tensors[in];
        const TensorInfo& to = tensors[out];
        a.M = to.n * to.h * to.w;
        a.OW = to.w;
        a.OHOW = to.h * to.w;
        a.H = ti.h;
        a.W = ti.w;
        a.cs = to.cs;
        a.in_bias = ti.dtype == HIPIE_U8B ? 128 : 0;
        auto expand = [&](const std::vector<float>& v, float pad) {
            std::vector<float> o(to.cs, pad);
            for (int c = 0; c < to.c; ++c) o[c] = v[v.size() == 1 ? 0 : c];
            return o;
        };
        if (!mul.empty()) {
            const auto m = expand(mul, 1.f);
            if (device >= 0) d_mul.upload(device, m.data(), m.size() * 4);
            a.mul = d_mul.as<float>();
        }
        if (!fq_il.empty()) {
            const auto il = expand(fq_il, 0.f), ih = expand(fq_ih, 1.f);
            std::vector<float> d(to.cs), r(to.cs);
            a.lm1 = static_cast<float>(static_cast<size_t>(levels - 1));
            std::vector<FqChannel> ch(to.cs);
            for (int c = 0; c < to.cs; ++c) {
                HIPIE_REQUIRE(il[c] < ih[c], HIPIE_NOT_IMPLEMENTED, "%s: FakeQuantize needs low < high", name.c_str());
                FqChannel& p = ch[c];
                p.il = il[c]; p.ih = ih[c]; p.lo = il[c]; p.hi = ih[c]; p.d = ih[c] - il[c];
                p.r = fq_rounded_reciprocal(p.d);
                d[c] = p.d;
                r[c] = p.r;
            }
            rcp = fq_reciprocal_exact_on_all(ch.data(), to.cs, a.lm1);
            HIPIE_REQUIRE(fq_ol == std::nearbyintf(fq_ol) && fq_oh == fq_ol + a.lm1, HIPIE_NOT_IMPLEMENTED,
                          "%s: output range is not consecutive integers", name.c_str());
            for (int k = 0; k < levels; ++k)
                HIPIE_REQUIRE((static_cast<float>(k) / a.lm1 * (fq_oh - fq_ol) + fq_ol) == fq_ol + k,
                              HIPIE_NOT_IMPLEMENTED, "%s: output levels are not integers", name.c_str());
            a.out_off = to.dtype == HIPIE_U8B ? fq_ol - 128.f : fq_ol;
            if (device >= 0) {
                d_il.upload(device, il.data(), il.size() * 4);
                d_ih.upload(device, ih.data(), ih.size() * 4);
                d_d.upload(device, d.data(), d.size() * 4);
                d_r.upload(device, r.data(), r.size() * 4);
            }
            a.fq_il = d_il.as<float>(); a.fq_ih = d_ih.as<float>();
            a.fq_d = d_d.as<float>(); a.fq_r = d_r.as<float>();
        }
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const*, void* const*,
             hipStream_t s) const override {
        const hipie_tensor i = tensors[in].desc(arena), o = tensors[out].desc(arena);
        PoolArgs b = a;
        b.in = i.data;
        b.out = o.data;
        b.in_sn = static_cast<int32_t>(i.stride_n); b.in_sh = static_cast<int32_t>(i.stride_h);
        b.in_sw = static_cast<int32_t>(i.stride_w);
        b.out_sn = static_cast<int32_t>(o.stride_n); b.out_sh = static_cast<int32_t>(o.stride_h);
        b.out_sw = static_cast<int32_t>(o.stride_w);
        if (avg) launch_avg_pool(b, rcp, s);
        else launch_max_pool(b, s);
        HIPIE_CHECK_HIP(hipGetLastError());
    }
};

// Result: engine tensor -> dense NCHW output buffer of the request (f32, or u8 levels)
// Concat of byte tensors along the channel axis: one strided copy per input into its channel slice
struct ConcatStep : Step {
    std::vector<int> ins, c_off;      // c_off: where the input starts along `axis` of the output
    int out = -1;
    int axis = 1;                     // of [N, C, H, W]
    void create(int, const std::vector<TensorInfo>&) override {}
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const*, void* const*, hipStream_t s) const override {
        const hipie_tensor o = tensors[out].desc(arena);
        for (size_t i = 0; i < ins.size(); ++i) {
            const hipie_tensor x = tensors[ins[i]].desc(arena);
            ConcatArgs a{};
            a.in = static_cast<const int8_t*>(x.data);
            a.out = static_cast<int8_t*>(o.data);
            const int es = static_cast<int>(tensors[out].esize());   // (f32 branches: four bytes per element)
            a.N = x.n; a.H = x.h; a.W = x.w; a.C = x.c * es;
            a.in_sn = x.stride_n * es; a.in_sh = x.stride_h * es; a.in_sw = x.stride_w * es;
            a.out_sn = o.stride_n * es; a.out_sh = o.stride_h * es; a.out_sw = o.stride_w * es;
            // the input copied into its box of the output: first element moved along the axis, same walk
            a.c_off = axis == 1 ? c_off[i] * es : 0;
            if (axis == 0) a.out += c_off[i] * a.out_sn;
            else if (axis == 2) a.out += c_off[i] * a.out_sh;
            else if (axis == 3) a.out += c_off[i] * a.out_sw;
            launch_concat_channels(a, s);
        }
        HIPIE_CHECK_HIP(hipGetLastError());
    }
};

// Elementwise nodes that no other step absorbs (run_eltwise in fq.hip): op(a, b) [-> Relu | Clamp] [-> FakeQuantize]
struct EltwiseStep : Step {
    struct Operand {
        int tensor = -1;                 // arena tensor, or -1: per-channel constant
        bool bn = false, bh = false, bw = false;   // the tensor has one element along N / H / W and is repeated along it
        std::vector<float> sub, mul, konst;
        DeviceBuffer d_sub, d_mul, d_konst;
    };
    Operand a, b;
    int op = 0, act = 0;
    float lo = 0, hi = 0;
    int out = -1;
    // FakeQuantize behind it
    bool quantize = false;
    int64_t levels = 0;
    std::vector<float> il, ih;
    float ol = 0, oh = 0;
    hipie_fq* fq = nullptr;
    int device_ = 0;                     // the plan's device
    ~EltwiseStep() override { hipie_fq_destroy(fq); }
    void create(int device, const std::vector<TensorInfo>& tensors) override {
        device_ = device;
        const int C = tensors[out].c;
        if (quantize) {
            check_status(hipie_fq_create(device, C, levels, il.data(), il.size(), ih.data(), ih.size(), &ol, 1, &oh, 1, &fq), name.c_str());
            HIPIE_REQUIRE(fq_gives_levels(fq), HIPIE_NOT_IMPLEMENTED, "%s: FakeQuantize whose outputs are not consecutive integer levels",
                          name.c_str());
        }
        if (device < 0) return;
        const size_t padded = static_cast<size_t>(round_up(C, 4));
        auto up = [&](const std::vector<float>& v, DeviceBuffer& d, float pad) {
            if (v.empty()) return;
            std::vector<float> o(padded, pad);
            for (int c = 0; c < C; ++c) o[c] = v[v.size() == 1 ? 0 : c];
            d.upload(device, o.data(), o.size() * 4);
        };
        for (Operand* o : {&a, &b}) {
            up(o->sub, o->d_sub, 0.f);
            up(o->mul, o->d_mul, 1.f);
            up(o->konst, o->d_konst, 0.f);
        }
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const*, void* const*, hipStream_t s) const override {
        EltArgs e;
        auto fill = [&](const Operand& o, EltOperand& d) {
            if (o.tensor >= 0) {
                const hipie_tensor t = tensors[o.tensor].desc(arena);
                d.p = t.data;
                d.dtype = t.dtype;
                d.sn = o.bn ? 0 : t.stride_n; d.sh = o.bh ? 0 : t.stride_h; d.sw = o.bw ? 0 : t.stride_w;
            }
            d.sub = o.sub.empty() ? nullptr : o.d_sub.as<float>();
            d.mul = o.mul.empty() ? nullptr : o.d_mul.as<float>();
            d.konst = o.konst.empty() ? nullptr : o.d_konst.as<float>();
        };
        fill(a, e.a);
        if (op != 0) fill(b, e.b);
        e.op = op; e.act = act; e.lo = lo; e.hi = hi;
        const hipie_tensor t = tensors[out].desc(arena);
        e.out = t.data;
        e.out_dtype = t.dtype;
        e.out_sn = t.stride_n; e.out_sh = t.stride_h; e.out_sw = t.stride_w;
        e.N = t.n; e.H = t.h; e.W = t.w; e.C = t.c;
        e.device = device_;
        run_eltwise(fq, e, s);
    }
};

struct ExitStep : Step {
    int in = -1, result_index = 0, C = 0;
    bool out_u8 = false;
    std::vector<float> sub, mul;
    DeviceBuffer d_sub, d_mul;
    void create(int device, const std::vector<TensorInfo>&) override {
        auto expand = [&](const std::vector<float>& v) {
            std::vector<float> o(C);
            for (int c = 0; c < C; ++c) o[c] = v[v.size() == 1 ? 0 : c];
            return o;
        };
        if (device < 0) return;
        if (!sub.empty()) { const auto v = expand(sub); d_sub.upload(device, v.data(), v.size() * 4); }
        if (!mul.empty()) { const auto v = expand(mul); d_mul.upload(device, v.data(), v.size() * 4); }
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const*, void* const* outputs,
             hipStream_t s) const override {
        const TensorInfo& t = tensors[in];
        const hipie_tensor i = t.desc(arena);
        ExitArgs a{};
        a.in = i.data;
        a.out = outputs[result_index];
        a.N = t.n; a.C = t.c; a.HW = t.h * t.w; a.W = t.w;
        a.in_sn = static_cast<int32_t>(i.stride_n); a.in_sh = static_cast<int32_t>(i.stride_h);
        a.in_sw = static_cast<int32_t>(i.stride_w);
        a.in_bias = t.dtype == HIPIE_U8B ? 128.f : 0.f;
        a.sub = sub.empty() ? nullptr : d_sub.as<float>();
        a.mul = mul.empty() ? nullptr : d_mul.as<float>();
        a.out_u8 = out_u8;
        launch_exit(a, t.dtype, s);
        HIPIE_CHECK_HIP(hipGetLastError());
    }
};


// ---- layers left in f32 (convf.hip) --------------------------------------------------------------------------------

// Where such a layer reads its [N, C, H, W] operand: an f32 request input (NCHW), an f32 tensor of the arena (NHWC), or
// the bytes of a quantized tensor behind their dequantization constants
struct F32Input {
    int tensor = -1, param = -1;
    int n = 1, c = 1, h = 1, w = 1;
    std::vector<float> sub, mul;
    DeviceBuffer d_sub, d_mul;
    void upload(int device) {
        auto up = [&](const std::vector<float>& v, DeviceBuffer& d) {
            if (v.empty() || device < 0) return;
            std::vector<float> o(static_cast<size_t>(c));
            for (int i = 0; i < c; ++i) o[i] = v[v.size() == 1 ? 0 : i];
            d.upload(device, o.data(), o.size() * 4);
        };
        up(sub, d_sub);
        up(mul, d_mul);
    }
    F32Source source(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs) const {
        F32Source s;
        if (tensor >= 0) {
            const hipie_tensor t = tensors[tensor].desc(arena);
            s.p = t.data;
            s.dtype = t.dtype;
            s.sn = t.stride_n; s.sc = 1; s.sh = t.stride_h; s.sw = t.stride_w;
        } else {
            s.p = inputs[param];
            s.dtype = HIPIE_F32;
            s.sn = static_cast<int64_t>(c) * h * w; s.sc = static_cast<int64_t>(h) * w; s.sh = w; s.sw = 1;
        }
        s.sub = sub.empty() ? nullptr : d_sub.as<float>();
        s.mul = mul.empty() ? nullptr : d_mul.as<float>();
        return s;
    }
    int64_t bytes(const std::vector<TensorInfo>& tensors) const {
        return static_cast<int64_t>(n) * c * h * w * (tensor >= 0 ? tensors[tensor].esize() : 4);
    }
};

// Convolution / GroupConvolution / MatMul of an f32 value with f32 constant weights
struct ConvF32Step : Step {
    F32Input src;
    int out = -1;
    std::vector<float> weights;        // [C / G][KH][KW][OC]
    DeviceBuffer d_weights;
    ConvF32Args geo{};                 // the shape part
    void create(int device, const std::vector<TensorInfo>&) override {
        if (device < 0) return;
        d_weights.upload(device, weights.data(), weights.size() * 4);
        src.upload(device);
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*, hipStream_t s) const override {
        ConvF32Args a = geo;
        a.in = src.source(arena, tensors, inputs);
        a.wgt = d_weights.as<float>();
        const hipie_tensor t = tensors[out].desc(arena);
        a.out = static_cast<float*>(t.data);
        a.out_sn = t.stride_n; a.out_sh = t.stride_h; a.out_sw = t.stride_w;
        launch_conv_f32(a, s);
    }
};

// MaxPool / AvgPool of an f32 value
struct PoolF32Step : Step {
    F32Input src;
    int out = -1;
    PoolF32Args geo{};
    void create(int device, const std::vector<TensorInfo>&) override { src.upload(device); }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*, hipStream_t s) const override {
        PoolF32Args a = geo;
        a.in = src.source(arena, tensors, inputs);
        const hipie_tensor t = tensors[out].desc(arena);
        a.out = static_cast<float*>(t.data);
        a.out_sn = t.stride_n; a.out_sh = t.stride_h; a.out_sw = t.stride_w;
        launch_pool_f32(a, s);
    }
};

// FakeQuantize with an f32 result; without channels: the operand as an NHWC f32 tensor, nothing else (a graph input
// in front of stand-alone elementwise nodes, which read NHWC)
struct FqF32Step : Step {
    F32Input src;
    int out = -1;
    std::vector<FqChannel> channels;   // one, or one per channel; none: copy
    DeviceBuffer d_channels;
    float lm1 = 255.f;
    void create(int device, const std::vector<TensorInfo>&) override {
        if (device < 0) return;
        if (!channels.empty()) d_channels.upload(device, channels.data(), channels.size() * sizeof(FqChannel));
        src.upload(device);
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*, hipStream_t s) const override {
        FqF32Args a;
        a.in = src.source(arena, tensors, inputs);
        a.ch = d_channels.as<FqChannel>();
        a.per_channel = channels.size() > 1 ? 1 : 0;
        a.lm1 = lm1;
        const hipie_tensor t = tensors[out].desc(arena);
        a.out = static_cast<float*>(t.data);
        a.out_sn = t.stride_n; a.out_sh = t.stride_h; a.out_sw = t.stride_w;
        a.N = src.n; a.C = src.c; a.H = src.h; a.W = src.w;
        if (channels.empty()) launch_copy_f32(a, s);
        else launch_fq_f32(a, s);
    }
};

// Softmax along one axis of an [N, C] or [N, C, H, W] value (over the channels: the classifier's, a detection head's)
struct SoftmaxF32Step : Step {
    F32Input src;
    int out = -1;
    int axis = 1;
    void create(int device, const std::vector<TensorInfo>&) override { src.upload(device); }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*, hipStream_t s) const override {
        FqF32Args a;
        a.in = src.source(arena, tensors, inputs);
        const hipie_tensor t = tensors[out].desc(arena);
        a.out = static_cast<float*>(t.data);
        a.out_sn = t.stride_n; a.out_sh = t.stride_h; a.out_sw = t.stride_w;
        a.N = src.n; a.C = src.c; a.H = src.h; a.W = src.w;
        a.axis = axis;
        launch_softmax_f32(a, s);
    }
};

// ---- steps over row-major views (transformer encoders) ------------------------------------------

// FakeQuantize of a dense f32 value with per-tensor bounds -> i8 levels
struct MatFqStep : Step {
    View in;
    int out = -1;
    int64_t n = 0, levels = 0;
    float il = 0, ih = 0, ol = 0, oh = 0;
    int out_dtype = HIPIE_I8;      // HIPIE_U8B: u8 levels stored as level - 128
    hipie_fq* fq = nullptr;
    ~MatFqStep() override { hipie_fq_destroy(fq); }
    void create(int device, const std::vector<TensorInfo>&) override {
        check_status(hipie_fq_create(device, 1, levels, &il, 1, &ih, 1, &ol, 1, &oh, 1, &fq), name.c_str());
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*,
             hipStream_t s) const override {
        check_status(hipie_fq_run_q8(fq, reinterpret_cast<const float*>(in.ptr(arena, tensors, inputs)),
                                     arena + tensors[out].offset, 1, n, static_cast<hipie_dtype>(out_dtype), HIPIE_NCHW, 0, s), name.c_str());
    }
};

// Softmax / MVN (+ LayerNorm gamma, beta) / Gelu over the last axis of a dense f32 value
struct GlueStep : Step {
    int kind = OP_SOFTMAX;
    View in;
    int out = -1;                  // f32 result (-1: only the quantized one is kept)
    int outq = -1;                 // i8 levels of the FakeQuantize fused behind it (-1: none)
    hipie_requant rq{};
    int64_t rows = 0, axis = 0;
    bool normalize_variance = true, eps_inside_sqrt = true;
    float eps = 0;
    std::vector<float> gamma, beta;
    DeviceBuffer d_gamma, d_beta;
    void create(int device, const std::vector<TensorInfo>&) override {
        if (device < 0) return;
        if (!gamma.empty()) d_gamma.upload(device, gamma.data(), gamma.size() * 4);
        if (!beta.empty()) d_beta.upload(device, beta.data(), beta.size() * 4);
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*,
             hipStream_t s) const override {
        const float* x = reinterpret_cast<const float*>(in.ptr(arena, tensors, inputs));
        float* y = out >= 0 ? reinterpret_cast<float*>(arena + tensors[out].offset) : nullptr;
        int8_t* q = outq >= 0 ? reinterpret_cast<int8_t*>(arena + tensors[outq].offset) : nullptr;
        const hipie_requant* r = outq >= 0 ? &rq : nullptr;
        const float* gm = gamma.empty() ? nullptr : d_gamma.as<float>();
        const float* bt = beta.empty() ? nullptr : d_beta.as<float>();
        int st = HIPIE_OK;
        if (kind == OP_SOFTMAX) st = q ? hipie_softmax_q8(x, y, q, rows, axis, r, s) : hipie_softmax_f32(x, y, rows, axis, s);
        else if (kind == OP_GELU) st = q ? hipie_gelu_q8(x, y, q, rows * axis, r, s) : hipie_gelu_f32(x, y, rows * axis, s);
        else st = q ? hipie_mvn_q8(x, y, q, rows, axis, normalize_variance, eps, eps_inside_sqrt, gm, bt, r, s)
                    : hipie_mvn_f32(x, y, rows, axis, normalize_variance, eps, eps_inside_sqrt, gm, bt, s);
        check_status(st, name.c_str());
    }
};

// Add of a graph input or a constant to a dense f32 value of the row-major path, numpy broadcasting (an attention
// mask on the scores where the attention core runs as separate kernels)
struct MatAddStep : Step {
    View in;
    int out = -1;
    int param = -1;                // the addend: a request input, or ...
    std::vector<float> konst;      // ... a constant
    DeviceBuffer d_konst;
    std::vector<int64_t> dims, addend_dims;
    void create(int device, const std::vector<TensorInfo>&) override {
        if (device >= 0 && !konst.empty()) d_konst.upload(device, konst.data(), konst.size() * 4);
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*, hipStream_t s) const override {
        const float* m = param >= 0 ? static_cast<const float*>(inputs[param]) : d_konst.as<float>();
        check_status(hipie_add_broadcast_f32(reinterpret_cast<const float*>(in.ptr(arena, tensors, inputs)), dims.data(), m, addend_dims.data(),
                                             static_cast<int>(dims.size()), reinterpret_cast<float*>(arena + tensors[out].offset), s),
                     name.c_str());
    }
};

// MatMul between two activations (each i8 or u8), batched over one or two leading dimensions
struct BatchMatMulStep : Step {
    View a, b;                     // b as [.., N, K] with K contiguous
    int out = -1;
    int ws = -1;                   // the sums over K that a u8 operand asks for (hipie_matmul_workspace_size bytes)
    int64_t lda = 0, sa = 0, oa = 0, ldb = 0, sb = 0, ob = 0, ldo = 0, so = 0, oo = 0;
    int32_t m = 0, k = 0, n = 0, batch = 1, outer = 1;
    EpilogueSpec epi;
    hipie_matmul* mm = nullptr;
    ~BatchMatMulStep() override { hipie_matmul_destroy(mm); }
    void create(int device, const std::vector<TensorInfo>&) override {
        hipie_matmul_desc d{};
        d.a_dtype = a.dtype;
        d.b_dtype = b.dtype;
        d.k = k;
        d.n = n;
        const hipie_epilogue e = epi.c_struct();
        check_status(hipie_matmul_create(device, &d, &e, &mm), name.c_str());
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*,
             hipStream_t s) const override {
        check_status(hipie_matmul_run_nested_ws(mm, a.ptr(arena, tensors, inputs), lda, sa, oa, b.ptr(arena, tensors, inputs), ldb,
                                                sb, ob, arena + tensors[out].offset, ldo, so, oo, m, batch, outer,
                                                ws >= 0 ? arena + tensors[ws].offset : nullptr,
                                                ws >= 0 ? static_cast<size_t>(tensors[ws].bytes) : 0, s),
                     name.c_str());
    }
};

// scores, Softmax, requantisation and context product of one attention block in one kernel
struct AttentionStep : Step {
    View q, k, v;
    int64_t ld[3] = {0, 0, 0}, inner[3] = {0, 0, 0}, outer[3] = {0, 0, 0};
    int out = -1, scores = -1, probs = -1;
    int64_t ldo = 0, so = 0, oo = 0;
    int32_t batch = 1, batch_outer = 1;
    // additive mask [batch_outer, 1, 1, S]: a request input or a constant
    bool masked = false;
    int mask_param = -1;
    std::vector<float> mask_const;
    DeviceBuffer d_mask;
    hipie_attention_desc desc{};
    hipie_attention* att = nullptr;
    ~AttentionStep() override { hipie_attention_destroy(att); }
    void create(int device, const std::vector<TensorInfo>&) override {
        check_status(hipie_attention_create(device, &desc, &att), name.c_str());
        if (device >= 0 && !mask_const.empty()) d_mask.upload(device, mask_const.data(), mask_const.size() * 4);
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*,
             hipStream_t s) const override {
        float* sc = scores >= 0 ? reinterpret_cast<float*>(arena + tensors[scores].offset) : nullptr;
        float* pr = probs >= 0 ? reinterpret_cast<float*>(arena + tensors[probs].offset) : nullptr;
        const float* mk = !masked ? nullptr : (mask_param >= 0 ? static_cast<const float*>(inputs[mask_param]) : d_mask.as<float>());
        check_status(hipie_attention_run(att, q.ptr(arena, tensors, inputs), ld[0], inner[0], outer[0],
                                         k.ptr(arena, tensors, inputs), ld[1], inner[1], outer[1],
                                         v.ptr(arena, tensors, inputs), ld[2], inner[2], outer[2], arena + tensors[out].offset,
                                         ldo, so, oo, batch, batch_outer, mk, 0, desc.seq, sc, pr, s), name.c_str());
    }
};

// Gather of a constant f32 table by the i32 token ids of a request input, with the embedding Adds
struct EmbeddingStep : Step {
    int param = 0, out = -1;
    int64_t vocab = 0, hidden = 0, tokens = 0, seq = 0;
    std::vector<float> table, add[2];
    bool per_position[2] = {false, false};
    DeviceBuffer d_table, d_add[2];
    void create(int device, const std::vector<TensorInfo>&) override {
        if (device >= 0) {
            d_table.upload(device, table.data(), table.size() * 4);
            for (int i = 0; i < 2; ++i)
                if (!add[i].empty()) d_add[i].upload(device, add[i].data(), add[i].size() * 4);
        }
        table.clear();
        table.shrink_to_fit();
    }
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*,
             hipStream_t s) const override {
        check_status(hipie_embedding_f32(d_table.as<float>(), vocab, hidden, static_cast<const int32_t*>(inputs[param]), tokens, seq,
                                         add[0].empty() ? nullptr : d_add[0].as<float>(), per_position[0],
                                         add[1].empty() ? nullptr : d_add[1].as<float>(), per_position[1],
                                         reinterpret_cast<float*>(arena + tensors[out].offset), s), name.c_str());
    }
};

// physical transpose of the two inner dimensions of a byte view (the right operand of a MatMul whose
// reduction axis is not contiguous)
struct MatTransposeStep : Step {
    View in;                       // [.., rows, cols], cols contiguous
    int out = -1;                  // dense [.., cols, rows]
    int64_t ld_src = 0, s_src = 0, o_src = 0, ld_dst = 0, s_dst = 0, o_dst = 0;
    int32_t rows = 0, cols = 0, batch = 1, outer = 1;
    void create(int, const std::vector<TensorInfo>&) override {}
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const*,
             hipStream_t s) const override {
        check_status(hipie_transpose_bytes_nested(in.ptr(arena, tensors, inputs), ld_src, s_src, o_src,
                                                  arena + tensors[out].offset, ld_dst, s_dst, o_dst, rows, cols, batch,
                                                  outer, s), name.c_str());
    }
};

// Result of a dense row-major value: its bytes are the output buffer's
struct MatExitStep : Step {
    View in;
    int result_index = 0;
    int64_t nbytes = 0;
    bool strided = false;          // the view is a box inside a larger value (one output of a Split): gathered, not copied whole
    void create(int, const std::vector<TensorInfo>&) override {}
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const* inputs, void* const* outputs,
             hipStream_t s) const override {
        if (strided)
            check_status(hipie_copy_strided(in.ptr(arena, tensors, inputs), in.shape.data(), in.stride.data(), static_cast<int>(in.rank()),
                                            static_cast<int>(in.esize()), outputs[result_index], s),
                         name.c_str());
        else
            HIPIE_CHECK_HIP(hipMemcpyAsync(outputs[result_index], in.ptr(arena, tensors, inputs), static_cast<size_t>(nbytes),
                                           hipMemcpyDeviceToDevice, s));
    }
};

// One output of a Split on a value of the [N, C, H, W] path: its box copied into a tensor of its own (the byte copy of
// ConcatStep, read side and write side exchanged)
struct SliceStep : Step {
    int in = -1, out = -1;
    int axis = 1, begin = 0;       // of [N, C, H, W]
    void create(int, const std::vector<TensorInfo>&) override {}
    void run(uint8_t* arena, const std::vector<TensorInfo>& tensors, void* const*, void* const*, hipStream_t s) const override {
        const hipie_tensor x = tensors[in].desc(arena);
        const hipie_tensor o = tensors[out].desc(arena);
        const int es = static_cast<int>(tensors[out].esize());
        ConcatArgs a{};
        a.in = static_cast<const int8_t*>(x.data);
        a.out = static_cast<int8_t*>(o.data);
        a.N = o.n; a.H = o.h; a.W = o.w; a.C = o.c * es;
        a.in_sn = x.stride_n * es; a.in_sh = x.stride_h * es; a.in_sw = x.stride_w * es;
        a.out_sn = o.stride_n * es; a.out_sh = o.stride_h * es; a.out_sw = o.stride_w * es;
        a.c_off = 0;
        a.in += begin * (axis == 0 ? a.in_sn : (axis == 1 ? es : (axis == 2 ? a.in_sh : a.in_sw)));
        launch_concat_channels(a, s);
        HIPIE_CHECK_HIP(hipGetLastError());
    }
};

// ------------------------------------------------------------------------------------------------
// Per-load configuration (what IInferencePlugin::LoadExeNetworkImpl receives as its config map,
// template_config.cpp:16-57).  The environment variables of the same meaning are the process-wide defaults; a
// key passed to hipie_compile_opts overrides them for that plan.
struct PlanConfig {
    bool perf_count = false;       // PERF_COUNT: requests created with perf_count < 0 time every step
    int streams = 3;               // HIP_THROUGHPUT_STREAMS: requests assumed in flight (tuning lanes, OPTIMAL_NUMBER_OF_INFER_REQUESTS)
    bool tune = true;              // HIP_TUNE: time the kernel variants at load
    std::string tune_file;         // HIP_TUNE_FILE: cache of the choices
    bool keep_f32 = false;         // HIP_KEEP_F32
    bool fuse_attention = true;    // HIP_FUSE_ATTENTION
    bool merge_linear = true;      // HIP_MERGE_LINEAR
    int fuse_convs = 1;            // HIP_FUSE_CONVOLUTIONS: a 3 x 3 convolution and the 1 x 1 behind it in one kernel - NO (0), AUTO
                                   // (1: where the load-time measurement says it is faster), YES (2: wherever the kernel takes the pair)
    int device_id = -1;            // DEVICE_ID (must agree with the device argument when given)
    std::string network_name = "hipie_network";

    static bool env_flag(const char* name, bool dflt) {
        const char* v = std::getenv(name);
        return v ? v[0] != '0' : dflt;
    }
    static PlanConfig from_environment() {
        PlanConfig c;
        c.tune = env_flag("HIPIE_TUNE", true);
        if (const char* f = std::getenv("HIPIE_TUNE_FILE")) c.tune_file = f;
        if (const char* ts = std::getenv("HIPIE_TUNE_STREAMS")) c.streams = std::max(1, std::min(8, std::atoi(ts)));
        c.keep_f32 = env_flag("HIPIE_KEEP_F32", false);
        c.fuse_attention = env_flag("HIPIE_FUSE_ATTENTION", true);
        c.merge_linear = env_flag("HIPIE_MERGE_LINEAR", true);
        if (const char* fc = std::getenv("HIPIE_FUSE_CONVS")) c.fuse_convs = std::max(0, std::min(2, std::atoi(fc)));
        return c;
    }
    static bool yes_no(const char* key, const char* v) {
        if (!std::strcmp(v, "YES")) return true;
        if (!std::strcmp(v, "NO")) return false;
        fail(HIPIE_PARAMETER_MISMATCH, "config key %s takes YES or NO, not '%s'", key, v);
    }
    // unknown key: NOT_FOUND, as template_config.cpp:36-38 throws
    void set(const char* key, const char* value) {
        HIPIE_REQUIRE(key && value, HIPIE_PARAMETER_MISMATCH, "config: null key or value");
        const std::string k = key;
        if (k == "PERF_COUNT") perf_count = yes_no(key, value);
        else if (k == "HIP_THROUGHPUT_STREAMS") {
            if (!std::strcmp(value, "HIP_THROUGHPUT_AUTO")) streams = 3;
            else {
                char* end = nullptr;
                const long n = std::strtol(value, &end, 10);
                HIPIE_REQUIRE(end != value && *end == 0 && n >= 1 && n <= 8, HIPIE_PARAMETER_MISMATCH,
                              "config key HIP_THROUGHPUT_STREAMS takes 1 .. 8 or HIP_THROUGHPUT_AUTO, not '%s'", value);
                streams = static_cast<int>(n);
            }
        } else if (k == "DEVICE_ID") {
            char* end = nullptr;
            const long n = std::strtol(value, &end, 10);
            HIPIE_REQUIRE(end != value && *end == 0 && n >= 0, HIPIE_PARAMETER_MISMATCH, "config key DEVICE_ID: '%s'", value);
            device_id = static_cast<int>(n);
        } else if (k == "HIP_TUNE") tune = yes_no(key, value);
        else if (k == "HIP_TUNE_FILE") tune_file = value;
        else if (k == "HIP_KEEP_F32") keep_f32 = yes_no(key, value);
        else if (k == "HIP_FUSE_ATTENTION") fuse_attention = yes_no(key, value);
        else if (k == "HIP_MERGE_LINEAR") merge_linear = yes_no(key, value);
        else if (k == "HIP_FUSE_CONVOLUTIONS") {
            if (!std::strcmp(value, "AUTO")) fuse_convs = 1;
            else fuse_convs = yes_no(key, value) ? 2 : 0;
        }
        else if (k == "NETWORK_NAME") network_name = value;
        else fail(HIPIE_NOT_FOUND, "config key '%s' is not supported", key);
    }
    bool get(const std::string& k, std::string& v) const {
        auto yn = [](bool b) { return std::string(b ? "YES" : "NO"); };
        if (k == "PERF_COUNT") v = yn(perf_count);
        else if (k == "HIP_THROUGHPUT_STREAMS") v = std::to_string(streams);
        else if (k == "DEVICE_ID") v = std::to_string(device_id);
        else if (k == "HIP_TUNE") v = yn(tune);
        else if (k == "HIP_TUNE_FILE") v = tune_file;
        else if (k == "HIP_KEEP_F32") v = yn(keep_f32);
        else if (k == "HIP_FUSE_ATTENTION") v = yn(fuse_attention);
        else if (k == "HIP_MERGE_LINEAR") v = yn(merge_linear);
        else if (k == "HIP_FUSE_CONVOLUTIONS") v = fuse_convs == 1 ? "AUTO" : yn(fuse_convs == 2);
        else return false;
        return true;
    }
};
constexpr const char* kConfigKeys = "PERF_COUNT DEVICE_ID HIP_THROUGHPUT_STREAMS HIP_TUNE HIP_TUNE_FILE HIP_KEEP_F32 HIP_FUSE_ATTENTION HIP_MERGE_LINEAR HIP_FUSE_CONVOLUTIONS";

// thrown by the planner for a node it cannot take: the status and text of any Error, plus the node
struct UnsupportedNode : Error {
    int node;
    UnsupportedNode(int n, const std::string& m) : Error(HIPIE_NOT_IMPLEMENTED, m), node(n) {}
};

struct Planner {
    const hipie_graph& g;
    std::vector<Value> values;
    std::vector<TensorInfo> tensors;
    std::vector<std::unique_ptr<Step>> steps;
    std::vector<char> visiting;
    // HIPIE_KEEP_F32=1: store the f32 result of Softmax / MVN / Gelu even when only a fused
    // FakeQuantize reads it (inspection of the values behind the tolerance-only operations)
    bool keep_f32 = false;
    // HIPIE_FUSE_ATTENTION=0: plan the attention core as separate MatMul / Softmax kernels
    bool fuse_attention = true;
    // HIPIE_MERGE_LINEAR=0: one GEMM per MatMul node even when several share their input
    bool merge_linear = true;

    Planner(const hipie_graph& graph, const PlanConfig& cfg)
        : g(graph), values(graph.nodes.size()), visiting(graph.nodes.size(), 0), keep_f32(cfg.keep_f32),
          fuse_attention(cfg.fuse_attention), merge_linear(cfg.merge_linear) {}

    const GNode& N(int id) const { return g.nodes[id]; }

    [[noreturn]] void unsupported(int id, const char* why) const {
        char buf[1024];
        snprintf(buf, sizeof buf, "node %d '%s' (%s): %s", id, N(id).name.c_str(), op_name(N(id).op), why);
        throw UnsupportedNode(id, buf);
    }

    // constant broadcastable along the channel axis of an [N, C, ...] value: 1 or C numbers
    bool channel_constant(int id, int64_t C, size_t out_rank, std::vector<float>& v) const {
        const GNode& c = N(id);
        if (c.op != OP_CONSTANT || c.dtype != HIPIE_F32) return false;
        const int64_t n = c.numel();
        if (n == 1) { v.assign(1, c.f32()[0]); return true; }
        if (n != C) return false;
        // the single non-unit axis must align with axis 1 of the output
        const size_t r = c.shape.size();
        for (size_t i = 0; i < r; ++i)
            if (c.shape[i] != 1 && i + out_rank - r != 1) return false;
        v.assign(c.f32(), c.f32() + C);
        return true;
    }

    int new_tensor(int node, int dtype, int n, int h, int w, int c, int cs = 0) {
        TensorInfo t;
        t.dtype = dtype; t.n = n; t.h = h; t.w = w; t.c = c;
        const int gran = (dtype == HIPIE_F32 || dtype == HIPIE_I32) ? 4 : 16;
        t.cs = cs ? cs : static_cast<int>(round_up(c, gran));
        t.producer = node;
        tensors.push_back(t);
        return static_cast<int>(tensors.size()) - 1;
    }

    static void nhwc_dims(const std::vector<int64_t>& s, int& n, int& c, int& h, int& w) {
        n = static_cast<int>(s[0]);
        c = static_cast<int>(s.size() > 1 ? s[1] : 1);
        h = static_cast<int>(s.size() > 2 ? s[2] : 1);
        w = static_cast<int>(s.size() > 3 ? s[3] : 1);
    }

    int storage_type(int graph_dtype) const { return graph_dtype == HIPIE_U8 ? HIPIE_U8B : graph_dtype; }

    const Value& value(int id) {
        if (!visit(id)) unsupported(id, "value depends on a node that is still being planned");
        return values[id];
    }

    bool single_user(int id) const { return N(id).users.size() == 1; }

    // Post-order: producers first, so a Convolution / pooling head is planned before the
    // elementwise nodes behind it and can absorb them.  Returns false when the node (or one of
    // its inputs) is already on the visiting stack, i.e. it cannot be scheduled yet.
    bool visit(int id) {
        if (values[id].kind != VK_NONE) return true;
        if (visiting[id]) return false;
        visiting[id] = 1;
        bool ok = true;
        for (int i : N(id).in) ok = visit(i) && ok;
        if (ok && values[id].kind == VK_NONE) plan_node(id);
        visiting[id] = 0;
        return ok;
    }

    void plan_node(int id) {
        const GNode& n = N(id);
        const bool mat = !n.in.empty() && n.op != OP_CONSTANT && value(n.in[0]).kind == VK_MAT;
        // a flattened feature map keeps its NHWC bytes; only what reads it the way the reference reads [N, C * H * W]
        // may follow: the zero point's Convert and Subtract, and the MatMul (a convolution with an H x W filter)
        for (int in : n.in)
            if (in >= 0 && N(in).op != OP_CONSTANT && values[in].flat && n.op != OP_MATMUL && n.op != OP_CONVERT && n.op != OP_SUBTRACT)
                unsupported(id, "a flattened [N, C, H, W] value is read by a MatMul against constant weights");
        switch (n.op) {
        case OP_PARAMETER: plan_parameter(id); break;
        case OP_CONSTANT: values[id].kind = VK_CONST; break;
        case OP_FAKE_QUANTIZE:
            if (mat) plan_mat_fq(id);
            else if (n.dtype == HIPIE_F32) plan_fq_f32(id);
            else if (value(n.in[0]).kind == VK_PARAM) plan_fake_quantize(id);
            else plan_eltwise(id);
            break;
        case OP_MATMUL: mat ? plan_mat_matmul(id) : plan_conv(id); break;
        case OP_CONVOLUTION: case OP_GROUP_CONVOLUTION: plan_conv(id); break;
        case OP_CONVERT: plan_dequant(id); break;
        case OP_SUBTRACT: case OP_MULTIPLY:
            // the dequantization of a byte tensor stays symbolic; anything else is an elementwise step of its own
            if (value(n.in[0]).kind == VK_DEQ && N(n.in[1]).op == OP_CONSTANT && value(n.in[0]).mul.empty() &&
                (n.op == OP_MULTIPLY || value(n.in[0]).sub.empty()))
                plan_dequant(id);
            else
                plan_eltwise(id);
            break;
        case OP_ADD:
            if (mat || (n.in.size() == 2 && N(n.in[1]).op != OP_CONSTANT && value(n.in[1]).kind == VK_MAT)) plan_mat_add(id);
            else plan_eltwise(id);
            break;
        case OP_RELU: case OP_CLAMP: case OP_PRELU: case OP_SIGMOID: case OP_HSWISH: case OP_HSIGMOID: case OP_SWISH:
            plan_eltwise(id);
            break;
        case OP_MAX_POOL: case OP_AVG_POOL: plan_pool(id); break;
        case OP_RESHAPE: mat ? plan_mat_reshape(id) : plan_reshape(id); break;
        case OP_TRANSPOSE: plan_mat_transpose(id); break;
        case OP_SOFTMAX:
            // an [N, C] / [N, C, H, W] value: the f32 step; else the row-major path's kernel
            if (!mat && (n.shape.size() == 2 || n.shape.size() == 4)) plan_softmax_f32(id);
            else plan_glue(id);
            break;
        case OP_MVN: case OP_GELU: plan_glue(id); break;
        case OP_GATHER: plan_gather(id); break;
        case OP_CONCAT: plan_concat(id); break;
        case OP_SLICE: plan_slice(id); break;
        case OP_RESULT: mat ? plan_mat_result(id) : plan_result(id); values[id].kind = VK_FUSED; break;
        default: unsupported(id, "only planned as part of a fused convolution / pooling chain");
        }
        if (values[id].kind == VK_NONE) unsupported(id, "planner produced no value");
    }


    // ---- row-major world: values of a transformer encoder ---------------------------------------
    // A rank-3 Parameter [batch, sequence, hidden] is read where the request keeps it.
    void plan_parameter(int id) {
        const GNode& n = N(id);
        if (n.shape.size() != 3) {
            values[id].kind = VK_PARAM;
            return;
        }
        HIPIE_REQUIRE(n.dtype == HIPIE_F32, HIPIE_NOT_IMPLEMENTED, "node %d: rank-3 inputs must be f32", id);
        View v;
        for (size_t i = 0; i < g.params.size(); ++i)
            if (g.params[i] == id) v.param = static_cast<int>(i);
        v.dtype = HIPIE_F32;
        v.shape = n.shape;
        v.stride = View::dense_strides(n.shape);
        values[id].kind = VK_MAT;
        values[id].view = v;
    }

    // Embedding front end: Gather(table f32 [V, H], ids i32 Parameter [B, S], axis 0) and the Adds of
    // constants behind it (one row [H], or one row per position [S, H] / [1, S, H])
    void plan_gather(int id) {
        const GNode& n = N(id);
        const GNode& T = N(n.in[0]);
        const GNode& I = N(n.in[1]);
        if (T.op != OP_CONSTANT || T.dtype != HIPIE_F32 || T.shape.size() != 2 || n.axes[0] != 0)
            unsupported(id, "Gather is planned as a lookup in a constant f32 table [vocabulary, hidden] along axis 0");
        if (I.op != OP_PARAMETER || I.dtype != HIPIE_I32 || I.shape.size() != 2)
            unsupported(id, "Gather indices must be an i32 Parameter [batch, sequence]");
        auto st = std::make_unique<EmbeddingStep>();
        for (size_t i = 0; i < g.params.size(); ++i)
            if (g.params[i] == n.in[1]) st->param = static_cast<int>(i);
        st->vocab = T.shape[0];
        st->hidden = T.shape[1];
        st->seq = I.shape[1];
        st->tokens = I.shape[0] * I.shape[1];
        if (st->hidden % 4 != 0) unsupported(id, "hidden size must be a multiple of 4");
        st->table.assign(T.f32(), T.f32() + T.numel());
        int cur = id, k = 0;
        while (k < 2 && single_user(cur)) {
            const int nx = N(cur).users[0];
            const GNode& u = N(nx);
            if (u.op != OP_ADD) break;
            const GNode& c = N(u.in[0] == cur ? u.in[1] : u.in[0]);
            if (c.op != OP_CONSTANT || c.dtype != HIPIE_F32 || c.shape.empty() || c.shape.back() != st->hidden) break;
            const int64_t ne = c.numel();
            const bool row = ne == st->hidden;
            const bool pos = ne == st->seq * st->hidden && c.shape.size() >= 2 && c.shape[c.shape.size() - 2] == st->seq;
            if (!row && !pos) break;
            st->add[k].assign(c.f32(), c.f32() + ne);
            st->per_position[k] = !row;
            ++k;
            cur = nx;
        }
        mark_chain(id, cur);
        st->out = new_matrix(cur, HIPIE_F32, n.shape);
        st->name = N(cur).name;
        st->type = "Gather";
        st->bytes = n.numel() * 8;
        st->out_node = cur;
        set_matrix_value(cur, st->out, HIPIE_F32);
        steps.push_back(std::move(st));
    }

    // constant broadcastable along the last axis: 1 or C numbers
    bool last_axis_constant(int id, int64_t C, std::vector<float>& v) const {
        const GNode& c = N(id);
        if (c.op != OP_CONSTANT || c.dtype != HIPIE_F32) return false;
        const int64_t n = c.numel();
        if (n == 1) { v.assign(1, c.f32()[0]); return true; }
        if (n != C || c.shape.empty() || c.shape.back() != C) return false;
        v.assign(c.f32(), c.f32() + C);
        return true;
    }

    // dense [rows, cols] arena tensor for a value of `shape` (cols = last dimension)
    int new_matrix(int node, int dtype, const std::vector<int64_t>& shape) {
        int64_t numel = 1;
        for (auto d : shape) numel *= d;
        const int64_t cols = shape.back();
        const int gran = dtype == HIPIE_F32 ? 4 : 16;
        if (cols % gran != 0) unsupported(node, "last dimension must be a multiple of 16 (bytes) / 4 (f32)");
        return new_tensor(node, dtype, 1, 1, static_cast<int>(numel / cols), static_cast<int>(cols), static_cast<int>(cols));
    }

    void set_matrix_value(int id, int tensor, int dtype) {
        View v;
        v.tensor = tensor;
        v.dtype = dtype;
        v.shape = N(id).shape;
        v.stride = View::dense_strides(v.shape);
        values[id].kind = VK_MAT;
        values[id].view = v;
    }

    // marks the nodes strictly between a chain's head and its last node as fused away
    void mark_chain(int head, int last) {
        for (int k = head; k != last;) {
            const int nx = N(k).users[0];
            if (nx != last) values[nx].kind = VK_FUSED;
            k = nx;
        }
        if (last != head) values[head].kind = VK_FUSED;
    }

    const View& dense_f32_input(int id, const char* what) {
        const Value& x = value(N(id).in[0]);
        if (x.kind != VK_MAT || x.view.dtype != HIPIE_F32 || !x.view.dense()) unsupported(id, what);
        return x.view;
    }

    void plan_mat_fq(int id) {
        const GNode& n = N(id);
        const View x = dense_f32_input(id, "FakeQuantize input must be a dense f32 value");
        if (n.dtype != HIPIE_I8 && n.dtype != HIPIE_U8) unsupported(id, "activations of the row-major path are i8 or u8 levels");
        auto st = std::make_unique<MatFqStep>();
        st->out_dtype = storage_type(n.dtype);
        float* dst[4] = {&st->il, &st->ih, &st->ol, &st->oh};
        for (int i = 0; i < 4; ++i) {
            std::vector<float> c;
            if (!last_axis_constant(n.in[1 + i], -1, c)) unsupported(id, "FakeQuantize bounds must be per tensor");
            *dst[i] = c[0];
        }
        st->in = x;
        st->n = n.numel();
        st->levels = n.levels;
        st->out = new_matrix(id, st->out_dtype, n.shape);
        st->name = n.name;
        st->type = "FakeQuantize";
        st->bytes = n.numel() * 5;
        st->out_node = id;
        set_matrix_value(id, st->out, st->out_dtype);
        steps.push_back(std::move(st));
    }

    // FakeQuantize node `u` on value `x` with per-tensor bounds whose outputs are the i8 integers
    // out_low + k: can be evaluated inside the kernel that produces x
    // `storage`: where the caller can take u8 levels too, it receives the storage type (HIPIE_I8, or HIPIE_U8B: level - 128);
    // without it only i8 is accepted
    bool fusable_requant(int u, int x, hipie_requant& rq, int* storage = nullptr) const {
        const GNode& f = N(u);
        if (f.op != OP_FAKE_QUANTIZE || f.in[0] != x || (f.dtype != HIPIE_I8 && !(f.dtype == HIPIE_U8 && storage)) || f.levels < 2 ||
            f.levels > 256)
            return false;
        if (storage) *storage = f.dtype == HIPIE_U8 ? HIPIE_U8B : HIPIE_I8;
        float b[4];
        for (int i = 0; i < 4; ++i) {
            std::vector<float> c;
            if (!last_axis_constant(f.in[1 + i], -1, c)) return false;
            b[i] = c[0];
        }
        const float lm1 = static_cast<float>(f.levels - 1);
        const float lo_level = f.dtype == HIPIE_U8 ? 0.f : -128.f;
        if (!(b[0] < b[1]) || b[2] != std::nearbyintf(b[2]) || b[2] < lo_level || b[3] != b[2] + lm1 || b[3] > lo_level + 255.f) return false;
        for (int k = 0; k < f.levels; ++k)
            if (static_cast<float>(k) / lm1 * (b[3] - b[2]) + b[2] != b[2] + static_cast<float>(k)) return false;
        rq.in_low = b[0];
        rq.in_high = b[1];
        rq.out_low = f.dtype == HIPIE_U8 ? b[2] - 128.f : b[2];   // u8 levels are stored as level - 128
        rq.levels = f.levels;
        return true;
    }

    // Add(value of the row-major path, f32 graph input | constant) with numpy broadcasting of the addend
    void plan_mat_add(int id) {
        const GNode& n = N(id);
        const int xi = value(n.in[0]).kind == VK_MAT ? 0 : 1;
        const Value& x = value(n.in[xi]);
        const int other = n.in[1 - xi];
        const GNode& m = N(other);
        const size_t r = n.shape.size();
        if (x.view.dtype != HIPIE_F32 || !x.view.dense() || x.view.shape != n.shape || r > 4)
            unsupported(id, "Add on the row-major path takes a dense f32 value of up to four dimensions");
        if ((m.op != OP_PARAMETER && m.op != OP_CONSTANT) || m.dtype != HIPIE_F32 || m.shape.size() != r)
            unsupported(id, "Add on the row-major path takes an f32 graph input or constant of the value's rank as its addend");
        for (size_t k = 0; k < r; ++k)
            if (m.shape[k] != n.shape[k] && m.shape[k] != 1) unsupported(id, "addend that does not broadcast to the value");
        auto st = std::make_unique<MatAddStep>();
        st->in = x.view;
        st->dims = n.shape;
        st->addend_dims = m.shape;
        if (m.op == OP_PARAMETER) {
            (void)visit(other);
            for (size_t i = 0; i < g.params.size(); ++i)
                if (g.params[i] == other) st->param = static_cast<int>(i);
        } else {
            st->konst.assign(m.f32(), m.f32() + m.numel());
        }
        st->out = new_matrix(id, HIPIE_F32, n.shape);
        set_matrix_value(id, st->out, HIPIE_F32);
        st->name = n.name;
        st->type = "Add";
        st->bytes = n.numel() * 8 + m.numel() * 4;
        st->out_node = id;
        steps.push_back(std::move(st));
    }

    void plan_glue(int id) {
        const GNode& n = N(id);
        const View x = dense_f32_input(id, "Softmax / MVN / Gelu are planned on dense f32 values of the row-major path");
        const int64_t r = static_cast<int64_t>(n.shape.size()), C = n.shape.back();
        auto st = std::make_unique<GlueStep>();
        st->kind = n.op;
        if (n.op == OP_SOFTMAX && n.axes[0] != r - 1) unsupported(id, "Softmax over an axis other than the last");
        if (n.op == OP_MVN && (n.axes.size() != 1 || n.axes[0] != r - 1)) unsupported(id, "MVN over axes other than the last");
        int cur = id;
        if (n.op == OP_MVN) {
            st->normalize_variance = n.normalize_variance;
            st->eps = n.eps;
            st->eps_inside_sqrt = n.eps_inside_sqrt;
            // LayerNorm: Multiply(gamma[C]) then Add(beta[C])
            while (single_user(cur)) {
                const int nx = N(cur).users[0];
                const GNode& u = N(nx);
                if (u.op != OP_MULTIPLY && u.op != OP_ADD) break;
                std::vector<float> c;
                if (!last_axis_constant(u.in[0] == cur ? u.in[1] : u.in[0], C, c)) break;
                if (c.size() == 1) c.assign(static_cast<size_t>(C), c[0]);
                if (u.op == OP_MULTIPLY && st->gamma.empty() && st->beta.empty()) st->gamma = c;
                else if (u.op == OP_ADD && st->beta.empty()) st->beta = c;
                else break;
                cur = nx;
            }
            mark_chain(id, cur);
        }
        st->in = x;
        st->axis = C;
        st->rows = n.numel() / C;
        // A per-tensor FakeQuantize to i8 among the users rides in the same kernel; the f32 result is
        // then only stored when something else reads it too (rows the kernel cannot keep in registers
        // need it as well).
        int fq_node = -1, fq_storage = HIPIE_I8;
        for (int u : N(cur).users)
            if (fq_node < 0 && fusable_requant(u, cur, st->rq, &fq_storage)) fq_node = u;
        const bool keep = fq_node < 0 || N(cur).users.size() > 1 || keep_f32 || C % 4 != 0 || C > 4096;
        if (keep) {
            st->out = new_matrix(cur, HIPIE_F32, n.shape);
            set_matrix_value(cur, st->out, HIPIE_F32);
        } else {
            values[cur].kind = VK_FUSED;
        }
        if (fq_node >= 0) {
            st->outq = new_matrix(fq_node, fq_storage, n.shape);
            set_matrix_value(fq_node, st->outq, fq_storage);
        }
        st->name = N(fq_node >= 0 ? fq_node : cur).name;
        st->type = std::string(op_name(n.op)) + (fq_node >= 0 ? "+FakeQuantize" : "");
        st->bytes = n.numel() * (4 + (keep ? 4 : 0) + (fq_node >= 0 ? 1 : 0));
        st->out_node = fq_node >= 0 ? fq_node : cur;
        steps.push_back(std::move(st));
    }

    // numpy's no-copy reshape: succeeds when every group of merged dimensions is contiguous in itself
    static bool reshape_view(const View& v, const std::vector<int64_t>& ns, View& out) {
        std::vector<int64_t> od, os;
        for (size_t i = 0; i < v.shape.size(); ++i)
            if (v.shape[i] != 1) { od.push_back(v.shape[i]); os.push_back(v.stride[i]); }
        std::vector<int64_t> nstr(ns.size(), 1);
        size_t oi = 0, oj = 1, ni = 0, nj = 1;
        while (ni < ns.size() && oi < od.size()) {
            int64_t np = ns[ni], op = od[oi];
            while (np != op) {
                if (np < op) { if (nj >= ns.size()) return false; np *= ns[nj++]; }
                else { if (oj >= od.size()) return false; op *= od[oj++]; }
            }
            for (size_t k = oi; k + 1 < oj; ++k)
                if (os[k] != od[k + 1] * os[k + 1]) return false;
            nstr[nj - 1] = os[oj - 1];
            for (size_t k = nj - 1; k > ni; --k) nstr[k - 1] = nstr[k] * ns[k];
            ni = nj++;
            oi = oj++;
        }
        for (size_t k = ni; k < ns.size(); ++k) {
            if (ns[k] != 1) return false;
            nstr[k] = 1;
        }
        if (oi < od.size()) return false;
        out = v;
        out.shape = ns;
        out.stride = nstr;
        return true;
    }

    void plan_mat_reshape(int id) {
        const Value& x = value(N(id).in[0]);
        View v;
        if (!reshape_view(x.view, N(id).shape, v)) unsupported(id, "Reshape that would have to move bytes");
        values[id].kind = VK_MAT;
        values[id].view = v;
    }

    void plan_mat_transpose(int id) {
        const GNode& n = N(id);
        const Value& x = value(n.in[0]);
        if (x.kind != VK_MAT) unsupported(id, "Transpose is planned on values of the row-major path");
        View v = x.view;
        for (size_t i = 0; i < n.axes.size(); ++i) {
            v.shape[i] = x.view.shape[n.axes[i]];
            v.stride[i] = x.view.stride[n.axes[i]];
        }
        values[id].kind = VK_MAT;
        values[id].view = v;
    }

    void plan_mat_result(int id) {
        const GNode& n = N(id);
        const Value& x = value(n.in[0]);
        auto st = std::make_unique<MatExitStep>();
        if (!x.view.dense()) {
            // a box of a larger value (strides in the order of the dimensions) is gathered; a transposed view is not taken
            bool ordered = x.view.rank() <= 5;
            for (size_t k = 0; ordered && k + 1 < x.view.rank(); ++k) ordered = x.view.stride[k] >= x.view.stride[k + 1] * x.view.shape[k + 1];
            if (!ordered || x.view.stride.back() != 1) unsupported(id, "Result of a transposed view");
            st->strided = true;
        }
        st->in = x.view;
        st->nbytes = x.view.numel() * x.view.esize();
        for (size_t i = 0; i < g.results.size(); ++i)
            if (g.results[i] == id) st->result_index = static_cast<int>(i);
        st->name = n.name;
        st->type = "Result";
        st->bytes = st->nbytes * 2;
        st->out_node = id;
        steps.push_back(std::move(st));
    }

    void plan_mat_matmul(int id) {
        const GNode& n = N(id);
        const Value a = value(n.in[0]);
        const bool weights = N(n.in[1]).op == OP_CONSTANT;
        if (a.view.dtype != HIPIE_I8 && a.view.dtype != HIPIE_U8B) unsupported(id, "left operand must be quantized (i8 or u8)");
        if (n.ta) unsupported(id, "transpose_a");
        if (weights) plan_linear(id, a.view);
        else plan_batch_matmul(id, a.view);
    }

    // MatMul against constant i8 weights: a 1x1 convolution over [rows, K]
    // the elementwise chain behind a MatMul against constant weights
    struct LinearChain {
        EpilogueSpec e;
        std::vector<int32_t> acc_sub;   // the integer Subtract behind a MatMul whose activations have a zero point
        int cur = -1, res = -1, res_param = -1;
        bool residual = false;
    };

    LinearChain parse_linear_chain(int id, int64_t OC, int64_t T) {
        LinearChain ch;
        EpilogueSpec& e = ch.e;
        int cur = id, stage = 0;
        while (single_user(cur)) {
            const int nx = N(cur).users[0];
            const GNode& u = N(nx);
            if (u.op == OP_SUBTRACT && cur == id && u.in[0] == cur) {
                // DequantizationSubtract right behind the MatMul (mat_mul.cpp:95-121): zero point x column sums of the
                // weights, integers that go into the accumulators' start
                std::vector<float> c;
                if (!last_axis_constant(u.in[1], OC, c)) break;
                for (float v : c)
                    if (v != std::nearbyintf(v) || std::fabs(v) >= 16777216.f) unsupported(nx, "MatMul zero-point correction that is not an integer");
                if (c.size() == 1) c.assign(static_cast<size_t>(OC), c[0]);
                for (float v : c) ch.acc_sub.push_back(static_cast<int32_t>(v));
            } else if (u.op == OP_ADD || u.op == OP_MULTIPLY) {
                const int other = u.in[0] == cur ? u.in[1] : u.in[0];
                std::vector<float> c;
                if (last_axis_constant(other, OC, c)) {
                    if (u.op == OP_ADD && stage < 1) { e.bias = c; stage = 1; }
                    else if (u.op == OP_MULTIPLY && stage < 2) { e.scale = c; stage = 2; }
                    else break;
                } else if (u.op == OP_ADD && stage < 3 && N(other).op != OP_CONSTANT) {
                    if (!visit(other)) break;
                    const Value& r = values[other];
                    if (r.kind != VK_MAT || r.view.dtype != HIPIE_F32 || !r.view.dense() || r.view.offset != 0 ||
                        N(other).shape != u.shape)
                        break;
                    if (r.view.tensor >= 0 && (tensors[r.view.tensor].w != T || tensors[r.view.tensor].c != OC)) break;
                    e.residual_dtype = HIPIE_F32;
                    ch.res = r.view.tensor;
                    ch.res_param = r.view.param;
                    ch.residual = true;
                    stage = 3;
                } else {
                    break;
                }
            } else if (u.op == OP_GELU && stage < 5 && !keep_f32 && single_user(nx) && N(N(nx).users[0]).op == OP_FAKE_QUANTIZE &&
                       (N(N(nx).users[0]).dtype == HIPIE_I8 || N(N(nx).users[0]).dtype == HIPIE_U8)) {
                e.activation = 3;   // Gelu and the FakeQuantize behind it ride in the GEMM: its f32 result is never stored
                stage = 5;
            } else if (u.op == OP_FAKE_QUANTIZE && u.in[0] == cur && (u.dtype == HIPIE_I8 || u.dtype == HIPIE_U8)) {
                std::vector<float> ol, oh;
                if (!last_axis_constant(u.in[1], OC, e.fq_il) || !last_axis_constant(u.in[2], OC, e.fq_ih) ||
                    !last_axis_constant(u.in[3], -1, ol) || !last_axis_constant(u.in[4], -1, oh))
                    break;
                e.fq_ol = ol[0];
                e.fq_oh = oh[0];
                e.levels = u.levels;
                e.out_dtype = storage_type(u.dtype);
                cur = nx;
                break;
            } else {
                break;
            }
            cur = nx;
        }
        ch.cur = cur;
        return ch;
    }

    static void append_rows(std::vector<int8_t>& dst, const GNode& W, bool tb, int64_t OC, int64_t IC) {
        const int8_t* w = reinterpret_cast<const int8_t*>(W.data.data());
        const size_t base = dst.size();
        dst.resize(base + static_cast<size_t>(OC * IC));
        for (int64_t o = 0; o < OC; ++o)
            for (int64_t k = 0; k < IC; ++k) dst[base + o * IC + k] = tb ? w[o * IC + k] : w[k * OC + o];
    }

    static void append_expanded(std::vector<float>& dst, const std::vector<float>& v, int64_t n) {
        for (int64_t i = 0; i < n; ++i) dst.push_back(v[v.size() == 1 ? 0 : static_cast<size_t>(i)]);
    }

    // MatMul against constant i8 weights: a 1x1 convolution over [rows, K].  MatMuls that read the same
    // activation and end in the same kind of requantisation (the Q, K, V projections of an attention
    // block) become ONE GEMM over their concatenated output channels; each one's value is then a
    // column slice of the shared output tensor.
    void plan_linear(int id, const View& av) {
        const GNode& n = N(id);
        const GNode& W = N(n.in[1]);
        if (W.dtype != HIPIE_I8 || W.shape.size() != 2) unsupported(id, "weights must be a rank-2 i8 constant");
        if (!av.dense() || av.tensor < 0 || av.offset != 0) unsupported(id, "left operand must be a whole dense tensor");
        const int64_t IC = n.tb ? W.shape[1] : W.shape[0], OC = n.tb ? W.shape[0] : W.shape[1];
        HIPIE_REQUIRE(av.shape.back() == IC, HIPIE_PARAMETER_MISMATCH, "node %d: inner dimensions %lld vs %lld", id,
                      (long long)av.shape.back(), (long long)IC);
        const int64_t T = av.numel() / IC;
        auto st = std::make_unique<ConvStep>();
        st->in = av.tensor;
        if (tensors[av.tensor].w != T || tensors[av.tensor].c != IC) {   // same bytes, other row split
            if (IC % 16 != 0) unsupported(id, "reduction length must be a multiple of 16");
            st->in = new_tensor(tensors[av.tensor].producer, tensors[av.tensor].dtype, 1, 1, static_cast<int>(T), static_cast<int>(IC),
                                static_cast<int>(IC));
            tensors[st->in].alias = av.tensor;
        }
        LinearChain ch = parse_linear_chain(id, OC, T);

        // siblings to merge with: unplanned MatMuls on the same activation whose chains look the same
        std::vector<int> group(1, id);
        std::vector<LinearChain> chains(1, ch);
        std::vector<int64_t> ocs(1, OC);
        auto mergeable = [](const LinearChain& c) {
            return !c.residual && c.acc_sub.empty() && c.e.out_dtype == HIPIE_I8 && !c.e.bias.empty() && c.e.scale.empty();
        };
        if (merge_linear && mergeable(ch) && OC % 16 == 0) {
            for (int u : N(n.in[0]).users) {
                const GNode& m = N(u);
                if (u == id || values[u].kind != VK_NONE || m.op != OP_MATMUL || m.in[0] != n.in[0] || m.ta || m.tb != n.tb) continue;
                const GNode& W2 = N(m.in[1]);
                if (W2.op != OP_CONSTANT || W2.dtype != HIPIE_I8 || W2.shape.size() != 2) continue;
                const int64_t ic2 = m.tb ? W2.shape[1] : W2.shape[0], oc2 = m.tb ? W2.shape[0] : W2.shape[1];
                if (ic2 != IC || oc2 % 16 != 0 || m.shape.size() != n.shape.size()) continue;
                LinearChain c2 = parse_linear_chain(u, oc2, T);
                if (!mergeable(c2) || c2.e.levels != ch.e.levels || c2.e.fq_ol != ch.e.fq_ol || c2.e.fq_oh != ch.e.fq_oh) continue;
                group.push_back(u);
                chains.push_back(std::move(c2));
                ocs.push_back(oc2);
            }
        }
        int64_t OCt = 0;
        for (auto o : ocs) OCt += o;
        hipie_conv_desc& d = st->desc;
        d.groups = 1;
        d.kh = d.kw = d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1;
        d.ic = static_cast<int>(IC);
        d.oc = static_cast<int>(OCt);
        EpilogueSpec& e = st->epi;
        if (group.size() == 1) {
            e = ch.e;
            append_rows(st->weights, W, n.tb, OC, IC);
        } else {
            e.out_dtype = HIPIE_I8;
            e.levels = ch.e.levels;
            e.fq_ol = ch.e.fq_ol;
            e.fq_oh = ch.e.fq_oh;
            for (size_t i = 0; i < group.size(); ++i) {
                append_rows(st->weights, N(N(group[i]).in[1]), n.tb, ocs[i], IC);
                append_expanded(e.bias, chains[i].e.bias, ocs[i]);
                append_expanded(e.fq_il, chains[i].e.fq_il, ocs[i]);
                append_expanded(e.fq_ih, chains[i].e.fq_ih, ocs[i]);
            }
        }
        st->res = ch.res;
        st->res_param = ch.res_param;
        if (!ch.acc_sub.empty()) {
            // The reference converts the raw u8 x i8 sum to f32 and subtracts there; starting the accumulator from
            // -correction gives the same float exactly when neither the raw sum nor the difference can leave the 24 bits
            // a float holds: 2 * 255 * sum_k |w[k][oc]| < 2^24 for every output channel.
            for (int64_t o = 0; o < OC; ++o) {
                int64_t mag = 0;
                for (int64_t k = 0; k < IC; ++k) mag += std::abs(static_cast<int>(st->weights[o * IC + k]));
                if (510 * mag >= (int64_t(1) << 24))
                    unsupported(id, "MatMul with a zero point whose accumulators may exceed 2^24 (the f32 subtraction would round)");
            }
            st->acc_sub = ch.acc_sub;
        }
        for (size_t i = 0; i < group.size(); ++i) mark_chain(group[i], chains[i].cur);
        std::vector<int64_t> oshape = N(ch.cur).shape;
        oshape.back() = OCt;
        st->out = new_matrix(ch.cur, e.out_dtype, oshape);
        st->name = N(ch.cur).name + (group.size() > 1 ? " (+" + std::to_string(group.size() - 1) + " sharing the input)" : "");
        st->type = "MatMul";
        st->macs = T * OCt * IC;
        st->results = T * OCt;
        st->in_w_bytes = T * IC + OCt * IC;
        st->bytes = st->in_w_bytes + T * OCt * (e.out_dtype == HIPIE_F32 ? 4 : 1) + (ch.residual ? T * OCt * 4 : 0);
        st->out_node = ch.cur;
        if (group.size() == 1) {
            set_matrix_value(ch.cur, st->out, e.out_dtype);
        } else {
            int64_t col = 0;
            for (size_t i = 0; i < group.size(); ++i) {   // column slice [.., ocs[i]] at `col` of [.., OCt]
                View v;
                v.tensor = st->out;
                v.dtype = e.out_dtype;
                v.shape = N(chains[i].cur).shape;
                v.stride.assign(v.shape.size(), 1);
                int64_t pitch = OCt;
                for (size_t k = v.shape.size() - 1; k-- > 0;) {
                    v.stride[k] = pitch;
                    pitch *= v.shape[k];
                }
                v.offset = col;
                col += ocs[i];
                values[chains[i].cur].kind = VK_MAT;
                values[chains[i].cur].view = v;
            }
        }
        steps.push_back(std::move(st));
    }

    // byte strides of the one or two batch dimensions in front of a [.., rows, cols] view
    static void batch_strides(const View& v, int64_t& inner, int64_t& outer) {
        const size_t r = v.rank();
        inner = r >= 3 ? v.stride[r - 3] : 0;
        outer = r >= 4 ? v.stride[r - 4] : 0;
    }

    // What follows a MatMul between activations: the dequantization Multiply(s_a * s_b), then optionally
    // a Transpose that keeps the last axis last (the head merge of attention, written through the
    // output strides), the head-merging Reshape and the next per-tensor FakeQuantize.  Returns the last
    // absorbed node; oshape is the output tensor's (dense) shape, ostride the strides of the MatMul's
    // own dimensions inside it.
    int absorb_matmul_tail(int id, EpilogueSpec& e, std::vector<int64_t>& oshape, std::vector<int64_t>& ostride) {
        const GNode& n = N(id);
        const size_t r = n.shape.size();
        e.out_dtype = HIPIE_F32;
        int cur = id;
        oshape = n.shape;
        ostride = View::dense_strides(oshape);
        hipie_requant rq{};
        while (single_user(cur)) {
            const int nx = N(cur).users[0];
            const GNode& u = N(nx);
            std::vector<float> c;
            if (u.op == OP_MULTIPLY && e.scale.empty() && oshape == n.shape &&
                last_axis_constant(u.in[0] == cur ? u.in[1] : u.in[0], -1, c)) {
                e.scale = c;
            } else if (u.op == OP_TRANSPOSE && u.axes.back() == static_cast<int64_t>(r) - 1 && oshape == n.shape) {
                oshape = u.shape;
                const auto ts = View::dense_strides(oshape);
                for (size_t p = 0; p < r; ++p) ostride[u.axes[p]] = ts[p];
            } else if (u.op == OP_RESHAPE && !keep_f32 && single_user(nx) && u.shape.back() % oshape.back() == 0 &&
                       fusable_requant(N(nx).users[0], nx, rq)) {
                // head merge in front of the FakeQuantize: the output tensor is dense, so the Reshape
                // only renames its dimensions (the last one must stay a multiple of this MatMul's columns)
                oshape = u.shape;
            } else if (!keep_f32 && fusable_requant(nx, cur, rq)) {
                e.levels = rq.levels;
                e.fq_il.assign(1, rq.in_low);
                e.fq_ih.assign(1, rq.in_high);
                e.fq_ol = rq.out_low;
                e.fq_oh = rq.out_low + static_cast<float>(rq.levels - 1);
                e.out_dtype = HIPIE_I8;
                oshape = u.shape;
                cur = nx;
                break;
            } else {
                break;
            }
            cur = nx;
        }
        return cur;
    }

    // MatMul'(q, k^T) -> Multiply -> Softmax -> FakeQuantize -> MatMul'(., v) -> Multiply [-> ...]: one kernel
    // when the shapes fit it (hipie_attention_supported) and every link has a single user
    bool try_plan_attention(int id, const View& qv, const View& kv /* as [.., S, D] */) {
        const GNode& n = N(id);
        const size_t r = qv.rank();
        const int64_t S = qv.shape[r - 2], D = qv.shape[r - 1];
        if (kv.shape[r - 2] != S || !hipie_attention_supported(static_cast<int32_t>(S), static_cast<int32_t>(D))) return false;
        if (qv.stride[r - 1] != 1 || kv.stride[r - 1] != 1) return false;
        if (!single_user(id)) return false;
        const int mul = n.users[0];
        std::vector<float> c1;
        if (N(mul).op != OP_MULTIPLY || !last_axis_constant(N(mul).in[0] == id ? N(mul).in[1] : N(mul).in[0], -1, c1) ||
            !single_user(mul))
            return false;
        // optional attention mask: Add of an f32 Parameter / Constant [batch, 1, 1, S] (rank-4 attention only)
        int pre = mul, mask_node = -1;
        if (N(N(mul).users[0]).op == OP_ADD && r == 4) {
            const int add = N(mul).users[0];
            const int other = N(add).in[0] == mul ? N(add).in[1] : N(add).in[0];
            const GNode& mk = N(other);
            const std::vector<int64_t> want = {qv.shape[0], 1, 1, S};
            if ((mk.op != OP_PARAMETER && mk.op != OP_CONSTANT) || mk.dtype != HIPIE_F32 || mk.shape != want || !single_user(add))
                return false;
            pre = add;
            mask_node = other;
        }
        const int sm = N(pre).users[0];
        if (N(sm).op != OP_SOFTMAX || N(sm).axes[0] != static_cast<int64_t>(r) - 1 || !single_user(sm)) return false;
        const int fq = N(sm).users[0];
        hipie_requant rq{};
        int prob_storage = HIPIE_I8;
        if (!fusable_requant(fq, sm, rq, &prob_storage) || !single_user(fq)) return false;
        Requant host_check{};
        try {
            host_check = make_requant(&rq, "attention");
        } catch (...) {
            return false;
        }
        if (!host_check.rcp) return false;   // an exact fast division is known without asking the device
        const int mm2 = N(fq).users[0];
        const GNode& m2 = N(mm2);
        if (m2.op != OP_MATMUL || m2.in[0] != fq || m2.ta || m2.tb || N(m2.in[1]).op == OP_CONSTANT) return false;
        if (!visit(m2.in[1])) return false;
        const Value& vval = values[m2.in[1]];
        if (vval.kind != VK_MAT || vval.view.dtype != HIPIE_I8 || vval.view.rank() != r) return false;
        const View vv = vval.view;
        if (vv.shape != qv.shape || vv.stride[r - 1] != 1) return false;

        auto st = std::make_unique<AttentionStep>();
        EpilogueSpec tail;
        std::vector<int64_t> oshape, ostride;
        const int cur = absorb_matmul_tail(mm2, tail, oshape, ostride);
        if (tail.scale.empty()) return false;
        st->q = qv; st->k = kv; st->v = vv;
        st->ld[0] = qv.stride[r - 2]; st->ld[1] = kv.stride[r - 2]; st->ld[2] = vv.stride[r - 2];
        batch_strides(qv, st->inner[0], st->outer[0]);
        batch_strides(kv, st->inner[1], st->outer[1]);
        batch_strides(vv, st->inner[2], st->outer[2]);
        st->batch = static_cast<int32_t>(qv.shape[r - 3]);
        st->batch_outer = r == 4 ? static_cast<int32_t>(qv.shape[0]) : 1;
        hipie_attention_desc& d = st->desc;
        d.seq = static_cast<int32_t>(S);
        d.head_dim = static_cast<int32_t>(D);
        d.score_scale = c1[0];
        d.context_scale = tail.scale[0];
        d.prob_fq = rq;
        d.prob_dtype = prob_storage;
        d.out_dtype = tail.out_dtype;
        if (tail.out_dtype == HIPIE_I8) {
            d.out_fq.in_low = tail.fq_il[0];
            d.out_fq.in_high = tail.fq_ih[0];
            d.out_fq.out_low = tail.fq_ol;
            d.out_fq.levels = tail.levels;
        }
        // everything between the two products lives in registers; with HIPIE_KEEP_F32 the kernel also
        // writes the values in front of and behind the Softmax
        values[id].kind = VK_FUSED;
        values[fq].kind = VK_FUSED;
        if (mask_node >= 0) {
            st->masked = true;
            if (N(mask_node).op == OP_PARAMETER) {
                (void)visit(mask_node);
                for (size_t i = 0; i < g.params.size(); ++i)
                    if (g.params[i] == mask_node) st->mask_param = static_cast<int>(i);
            } else {
                st->mask_const.assign(N(mask_node).f32(), N(mask_node).f32() + N(mask_node).numel());
            }
            values[mul].kind = VK_FUSED;
        }
        if (keep_f32) {   // the Softmax input and output
            st->scores = new_matrix(pre, HIPIE_F32, N(pre).shape);
            set_matrix_value(pre, st->scores, HIPIE_F32);
            st->probs = new_matrix(sm, HIPIE_F32, N(sm).shape);
            set_matrix_value(sm, st->probs, HIPIE_F32);
        } else {
            values[pre].kind = VK_FUSED;
            values[sm].kind = VK_FUSED;
        }
        mark_chain(mm2, cur);
        st->out = new_matrix(cur, tail.out_dtype, oshape);
        st->ldo = ostride[r - 2];
        st->so = ostride[r - 3];
        st->oo = r == 4 ? ostride[0] : 0;
        st->name = N(cur).name;
        st->type = "Attention";
        st->macs = 2 * n.numel() * D;
        st->bytes = qv.numel() + kv.numel() + vv.numel() + m2.numel() * (tail.out_dtype == HIPIE_F32 ? 4 : 1);
        st->out_node = cur;
        set_matrix_value(cur, st->out, tail.out_dtype);
        steps.push_back(std::move(st));
        return true;
    }

    void plan_batch_matmul(int id, const View& av) {
        const GNode& n = N(id);
        const Value bval = value(n.in[1]);
        if (bval.kind != VK_MAT || (bval.view.dtype != HIPIE_I8 && bval.view.dtype != HIPIE_U8B))
            unsupported(id, "right operand must be quantized (i8 or u8)");
        View bv = bval.view;
        const size_t r = av.rank();
        if (r < 3 || r > 4 || bv.rank() != r) unsupported(id, "MatMul between activations needs equal ranks of 3 or 4");
        if (!n.tb) {   // bring the right operand to its [.., N, K] form
            std::swap(bv.shape[r - 1], bv.shape[r - 2]);
            std::swap(bv.stride[r - 1], bv.stride[r - 2]);
        }
        const int64_t M = av.shape[r - 2], K = av.shape[r - 1], Nn = bv.shape[r - 2];
        HIPIE_REQUIRE(bv.shape[r - 1] == K, HIPIE_PARAMETER_MISMATCH, "node %d: inner dimensions %lld vs %lld", id,
                      (long long)K, (long long)bv.shape[r - 1]);
        for (size_t i = 0; i + 2 < r; ++i)
            if (av.shape[i] != bv.shape[i]) unsupported(id, "broadcast batch dimensions");
        if (av.stride[r - 1] != 1) unsupported(id, "left operand with a strided reduction axis");
        if (K % 64 != 0) unsupported(id, "reduction length must be a multiple of 64");
        if (fuse_attention && M == Nn && av.dtype == HIPIE_I8 && bv.dtype == HIPIE_I8 && try_plan_attention(id, av, bv))
            return;   // (the scores' operands)
        const int32_t inner = static_cast<int32_t>(av.shape[r - 3]), outer = r == 4 ? static_cast<int32_t>(av.shape[0]) : 1;
        if (bv.stride[r - 1] != 1) {
            // reduction axis not contiguous: transpose the operand's inner dimensions into a new tensor
            if (bv.stride[r - 2] != 1) unsupported(id, "right operand with both inner dimensions strided");
            auto tp = std::make_unique<MatTransposeStep>();
            tp->in = bv;             // as [.., N, K]: in memory K rows of N contiguous bytes
            tp->rows = static_cast<int32_t>(K);
            tp->cols = static_cast<int32_t>(Nn);
            tp->ld_src = bv.stride[r - 1];
            batch_strides(bv, tp->s_src, tp->o_src);
            std::vector<int64_t> tshape(bv.shape);
            tp->out = new_matrix(n.in[1], bv.dtype, tshape);
            const auto ds = View::dense_strides(tshape);
            tp->ld_dst = K;
            tp->s_dst = ds[r - 3];
            tp->o_dst = r == 4 ? ds[0] : 0;
            tp->batch = inner;
            tp->outer = outer;
            tp->name = N(n.in[1]).name + "/transposed";
            tp->type = "Transpose";
            tp->bytes = 2 * bv.numel();
            View nb;
            nb.tensor = tp->out;
            nb.dtype = bv.dtype;
            nb.shape = tshape;
            nb.stride = ds;
            bv = nb;
            steps.push_back(std::move(tp));
        }
        auto st = std::make_unique<BatchMatMulStep>();
        st->a = av;
        st->b = bv;
        st->m = static_cast<int32_t>(M);
        st->k = static_cast<int32_t>(K);
        st->n = static_cast<int32_t>(Nn);
        st->batch = inner;
        st->outer = outer;
        st->lda = av.stride[r - 2];
        batch_strides(av, st->sa, st->oa);
        st->ldb = bv.stride[r - 2];
        batch_strides(bv, st->sb, st->ob);
        EpilogueSpec& e = st->epi;
        std::vector<int64_t> oshape, ostride;
        const int cur = absorb_matmul_tail(id, e, oshape, ostride);
        mark_chain(id, cur);
        st->out = new_matrix(cur, e.out_dtype, oshape);
        // level 0 of a u8 operand stands for 0.0 here: a zero point would arrive as a Subtract, which is not taken (nor
        // does MatMulTransformation rewrite such a MatMul, mat_mul.cpp:231-236, :290-292).  One row of sums per batch
        // element for either u8 operand: over the right operand's rows (u8 left), over the left operand's (u8 right)
        {
            const int64_t per_batch = (av.dtype == HIPIE_U8B ? round_up(Nn, 128) : 0) + (bv.dtype == HIPIE_U8B ? round_up(M, 4) : 0);
            if (per_batch > 0) st->ws = new_tensor(id, HIPIE_I32, 1, 1, inner * outer, static_cast<int>(per_batch));
        }
        st->ldo = ostride[r - 2];
        st->so = ostride[r - 3];
        st->oo = r == 4 ? ostride[0] : 0;
        st->name = N(cur).name;
        st->type = "MatMul";
        st->macs = n.numel() * K;
        st->bytes = av.numel() + bv.numel() + n.numel() * (e.out_dtype == HIPIE_F32 ? 4 : 1);
        st->out_node = cur;
        set_matrix_value(cur, st->out, e.out_dtype);
        steps.push_back(std::move(st));
    }

    void plan_fake_quantize(int id) {
        const GNode& n = N(id);
        const Value& x = value(n.in[0]);
        if (x.kind != VK_PARAM) unsupported(id, "stand-alone FakeQuantize is only planned on graph inputs");
        if (n.dtype == HIPIE_F32) unsupported(id, "FakeQuantize with f32 output (graph was not run through LPT)");
        const int param = N(n.in[0]).op == OP_CONVERT ? N(n.in[0]).in[0] : n.in[0];
        const GNode& p = N(param);
        HIPIE_REQUIRE(p.op == OP_PARAMETER && (p.dtype == HIPIE_F32 || (p.dtype == HIPIE_U8 && param != n.in[0])),
                      HIPIE_NOT_IMPLEMENTED, "node %d: a u8 graph input needs a Convert to f32 in front of its FakeQuantize", id);
        auto st = std::make_unique<EntryStep>();
        st->u8_in = p.dtype == HIPIE_U8;
        int nn, c, h, w;
        nhwc_dims(n.shape, nn, c, h, w);
        st->channels = c;
        st->levels = n.levels;
        std::vector<float>* dst[4] = {&st->il, &st->ih, &st->ol, &st->oh};
        for (int i = 0; i < 4; ++i)
            if (!channel_constant(n.in[1 + i], c, n.shape.size(), *dst[i]))
                unsupported(id, "FakeQuantize bounds must be scalars or per-channel constants");
        for (size_t i = 0; i < g.params.size(); ++i)
            if (g.params[i] == param) st->param_index = static_cast<int>(i);
        // small-channel images keep a 4-byte pixel so the first convolution reads filter rows contiguously
        st->out = new_tensor(id, storage_type(n.dtype), nn, h, w, c, c <= 4 ? 4 : 0);
        st->name = n.name;
        st->type = "FakeQuantize";
        st->bytes = n.numel() * (st->u8_in ? 2 : 5);
        st->out_node = id;
        values[id].kind = VK_TENSOR;
        values[id].tensor = st->out;
        if (param != n.in[0]) values[n.in[0]].kind = VK_FUSED;
        steps.push_back(std::move(st));
    }

    void plan_dequant(int id) {
        const GNode& n = N(id);
        const Value& x = value(n.in[0]);
        Value v;
        if (n.op == OP_CONVERT && x.kind == VK_PARAM && N(n.in[0]).dtype == HIPIE_U8 && n.dtype == HIPIE_F32) {
            values[id].kind = VK_PARAM;   // a u8 graph input seen as f32: read where the FakeQuantize behind it runs
            return;
        }
        if (n.op == OP_CONVERT) {
            if (x.kind != VK_TENSOR || tensors[x.tensor].esize() != 1 || n.dtype != HIPIE_F32)
                unsupported(id, "Convert is planned only as the start of a dequantization (u8/i8 -> f32)");
            v.kind = VK_DEQ;
            v.tensor = x.tensor;
            v.flat = x.flat;
        } else {
            if (x.kind != VK_DEQ) unsupported(id, "stand-alone elementwise op outside a fused chain");
            std::vector<float> c;
            if (!channel_constant(n.in[1], tensors[x.tensor].c, n.shape.size(), c))
                unsupported(id, "dequantization constant must be scalar or per-channel");
            if (x.flat && c.size() != 1) unsupported(id, "a flattened [N, C, H, W] value takes one zero point for all of it");
            v = x;
            if (n.op == OP_SUBTRACT) {
                if (!v.mul.empty() || !v.sub.empty()) unsupported(id, "Subtract after Multiply in a dequantization");
                v.sub = c;
            } else {
                if (!v.mul.empty()) unsupported(id, "two Multiplies in a dequantization");
                v.mul = c;
            }
        }
        values[id] = v;
    }

    // a graph input as a row-major view of the request's own buffer (its memory order is the graph's dimension order)
    bool param_view(int node, View& v) {
        const GNode& src = N(node);
        if (src.op != OP_PARAMETER || (src.dtype != HIPIE_F32 && src.dtype != HIPIE_U8)) return false;
        for (size_t i = 0; i < g.params.size(); ++i)
            if (g.params[i] == node) v.param = static_cast<int>(i);
        v.dtype = src.dtype;
        v.shape = src.shape;
        v.stride = View::dense_strides(src.shape);
        return v.param >= 0;
    }

    // One output of a Split.  On the row-major path (and on a graph input) it is a view: offset and extent change, no
    // byte moves.  On the [N, C, H, W] path the box is copied into a tensor of its own.
    void plan_slice(int id) {
        const GNode& n = N(id);
        const Value& x = value(n.in[0]);
        const size_t ax = static_cast<size_t>(n.axes[0]);
        const int64_t begin = n.axes[1];
        View v;
        if (x.kind == VK_MAT || (x.kind == VK_PARAM && param_view(n.in[0], v))) {
            if (x.kind == VK_MAT) v = x.view;
            v.offset += begin * v.stride[ax];
            v.shape[ax] = n.shape[ax];
            values[id].kind = VK_MAT;
            values[id].view = v;
            return;
        }
        if ((x.kind != VK_TENSOR && x.kind != VK_DEQ) || (n.shape.size() != 4 && n.shape.size() != 2))
            unsupported(id, "Split is planned on graph inputs, values of the row-major path and [N, C, H, W] / [N, C] tensors");
        auto st = std::make_unique<SliceStep>();
        st->in = x.tensor;
        st->axis = static_cast<int>(ax);
        st->begin = static_cast<int>(begin);
        int nn, c, h, w;
        nhwc_dims(n.shape, nn, c, h, w);
        st->out = new_tensor(id, tensors[x.tensor].dtype, nn, h, w, c);
        st->name = n.name;
        st->type = "Split";
        st->bytes = 2 * n.numel() * tensors[x.tensor].esize();
        st->out_node = id;
        values[id] = x;                       // a dequantization in front of the Split stays behind its outputs
        values[id].tensor = st->out;
        if (ax == 1) {
            auto part = [&](std::vector<float>& k) {
                if (k.size() > 1) k = std::vector<float>(k.begin() + begin, k.begin() + begin + c);
            };
            part(values[id].sub);
            part(values[id].mul);
        }
        steps.push_back(std::move(st));
    }

    void plan_reshape(int id) {
        const GNode& n = N(id);
        const Value& x = value(n.in[0]);
        const GNode& src = N(n.in[0]);
        View pv;
        if (x.kind == VK_PARAM && param_view(n.in[0], pv)) {      // the same bytes under other dimensions
            pv.shape = n.shape;
            pv.stride = View::dense_strides(n.shape);
            values[id].kind = VK_MAT;
            values[id].view = pv;
            return;
        }
        // [N, C, 1, 1] <-> [N, C]: same bytes in NHWC
        const bool flatten = src.shape.size() == 4 && n.shape.size() == 2 && src.shape[2] == 1 &&
                             src.shape[3] == 1 && n.shape[0] == src.shape[0] && n.shape[1] == src.shape[1];
        // [N, C, H, W] -> [N, C * H * W] of a byte tensor in front of a fully connected layer: the bytes stay NHWC and
        // the MatMul runs as the convolution with an H x W filter it is equal to (its weights [OC, C * H * W] are that
        // filter in the reference's own order)
        const bool flatten_map = src.shape.size() == 4 && n.shape.size() == 2 && n.shape[0] == src.shape[0] &&
                                 n.shape[1] == src.shape[1] * src.shape[2] * src.shape[3] && (x.kind == VK_TENSOR || x.kind == VK_DEQ) &&
                                 tensors[x.tensor].esize() == 1 && x.mul.empty() && x.sub.size() <= 1;
        if (!flatten && flatten_map) {
            values[id] = x;
            values[id].flat = true;
            return;
        }
        if (!flatten || (x.kind != VK_TENSOR && x.kind != VK_DEQ))
            unsupported(id, "only [N,C,1,1] -> [N,C] reshapes (and [N,C,H,W] -> [N,C*H*W] of quantized values in front of a MatMul) are planned");
        values[id] = x;
    }

    // ---- layers the transformations left in f32 -------------------------------------------------------------
    // the operand of such a layer: an f32 graph input, an f32 tensor, or a byte tensor behind its dequantization
    bool f32_input(int node, F32Input& o) {
        const Value x = value(node);
        const GNode& src = N(node);
        if (src.shape.size() != 4 && src.shape.size() != 2) return false;
        nhwc_dims(src.shape, o.n, o.c, o.h, o.w);
        if (x.kind == VK_PARAM && src.op == OP_PARAMETER && src.dtype == HIPIE_F32) {
            for (size_t i = 0; i < g.params.size(); ++i)
                if (g.params[i] == node) o.param = static_cast<int>(i);
            return o.param >= 0;
        }
        if (x.kind == VK_TENSOR && tensors[x.tensor].dtype == HIPIE_F32) {
            o.tensor = x.tensor;
        } else if (x.kind == VK_DEQ && tensors[x.tensor].esize() == 1) {
            o.tensor = x.tensor;
            o.sub = x.sub;
            o.mul = x.mul;
        } else {
            return false;
        }
        const TensorInfo& t = tensors[o.tensor];
        return t.n == o.n && t.c == o.c && t.h == o.h && t.w == o.w;
    }

    // an f32 graph input ([N, C, H, W] or [N, C], NCHW in the request's buffer) as an NHWC tensor of the arena, for the
    // elementwise nodes that read it directly (mean / scale preprocessing in front of the first FakeQuantize)
    std::map<int, int> param_tensors;
    int param_as_tensor(int node) {
        const auto found = param_tensors.find(node);
        if (found != param_tensors.end()) return found->second;
        auto st = std::make_unique<FqF32Step>();
        const bool ok = f32_input(node, st->src) && st->src.param >= 0;
        HIPIE_REQUIRE(ok, HIPIE_GENERAL_ERROR, "node %d is not an f32 graph input of rank 2 or 4", node);
        st->out = new_tensor(node, HIPIE_F32, st->src.n, st->src.h, st->src.w, st->src.c);
        st->name = N(node).name;
        st->type = "Reorder";
        st->bytes = N(node).numel() * 8;
        param_tensors[node] = st->out;
        const int t = st->out;
        steps.push_back(std::move(st));
        return t;
    }

    // Convolution / GroupConvolution / MatMul whose weights are an f32 constant: no FakeQuantize stood in front of the
    // layer, or the transformations did not take it (convolution.cpp:84-120, weightable_layer_transformation.cpp); the
    // layer runs as the graph says, in f32, and the nodes behind it are planned on their own
    void plan_conv_f32(int id) {
        const GNode& n = N(id);
        const GNode& W = N(n.in[1]);
        const bool is_mm = n.op == OP_MATMUL, grouped = n.op == OP_GROUP_CONVOLUTION;
        auto st = std::make_unique<ConvF32Step>();
        if (!f32_input(n.in[0], st->src))
            unsupported(id, "an f32 layer reads an f32 graph input, an f32 tensor or a dequantized byte tensor of rank 2 or 4");
        ConvF32Args& a = st->geo;
        const float* w = W.f32();
        int64_t G = 1, ocg = 0, icg = 0, KD = 1, KH = 1, KW = 1;
        if (is_mm) {
            if (n.ta || W.shape.size() != 2 || N(n.in[0]).shape.size() != 2)
                unsupported(id, "MatMul is planned for [N,K] x constant [K,OC] / [OC,K]^T");
            icg = n.tb ? W.shape[1] : W.shape[0];
            ocg = n.tb ? W.shape[0] : W.shape[1];
            st->weights.resize(static_cast<size_t>(icg * ocg));
            for (int64_t k = 0; k < icg; ++k)
                for (int64_t o = 0; o < ocg; ++o) st->weights[static_cast<size_t>(k * ocg + o)] = n.tb ? w[o * icg + k] : w[k * ocg + o];
        } else {
            // two spatial dimensions, or three with the values held as [N, C, D * H, W] (GNode::depth)
            const size_t sp = n.strides.size(), b = grouped ? 1 : 0;
            if (N(n.in[0]).shape.size() != 4 || (sp != 2 && sp != 3) || (sp == 3) != (n.depth > 0) || W.shape.size() != sp + 2 + b)
                unsupported(id, "f32 convolutions are planned over one to three spatial dimensions");
            G = grouped ? W.shape[0] : 1;
            ocg = W.shape[b]; icg = W.shape[b + 1];
            KD = sp == 3 ? W.shape[b + 2] : 1; KH = W.shape[b + sp]; KW = W.shape[b + sp + 1];
            const int64_t OCa = G * ocg, taps = KD * KH * KW;
            st->weights.resize(static_cast<size_t>(OCa * icg * taps));
            for (int64_t oc = 0; oc < OCa; ++oc)
                for (int64_t c = 0; c < icg; ++c)
                    for (int64_t t = 0; t < taps; ++t)
                        st->weights[static_cast<size_t>((c * taps + t) * OCa + oc)] = w[(oc * icg + c) * taps + t];
            const size_t o = sp - 2;
            a.stride_h = static_cast<int>(n.strides[o]); a.stride_w = static_cast<int>(n.strides[o + 1]);
            a.dil_h = static_cast<int>(n.dilations[o]); a.dil_w = static_cast<int>(n.dilations[o + 1]);
            a.pad_top = static_cast<int>(n.pads_begin[o]); a.pad_left = static_cast<int>(n.pads_begin[o + 1]);
            if (sp == 3) {
                a.D = static_cast<int>(n.depth);
                a.KD = static_cast<int>(KD);
                a.stride_d = static_cast<int>(n.strides[0]); a.dil_d = static_cast<int>(n.dilations[0]); a.pad_front = static_cast<int>(n.pads_begin[0]);
                a.OD = static_cast<int>((n.depth + n.pads_begin[0] + n.pads_end[0] - (n.dilations[0] * (KD - 1) + 1)) / n.strides[0] + 1);
            }
        }
        const int64_t OC = G * ocg, IC = G * icg;
        HIPIE_REQUIRE(st->src.c == IC, HIPIE_PARAMETER_MISMATCH, "node %d: input has %d channels, weights %lld", id, st->src.c, (long long)IC);
        int nn, c, h, ww;
        nhwc_dims(n.shape, nn, c, h, ww);
        HIPIE_REQUIRE(c == OC && nn == st->src.n, HIPIE_PARAMETER_MISMATCH, "node %d: output shape against the weights", id);
        HIPIE_REQUIRE(st->src.h % a.D == 0 && h % a.OD == 0, HIPIE_UNEXPECTED, "node %d: %d rows for a depth of %d, %d for %d", id, st->src.h, a.D, h, a.OD);
        a.N = nn; a.C = static_cast<int>(IC); a.H = st->src.h / a.D; a.W = st->src.w; a.OC = c; a.OH = h / a.OD; a.OW = ww;
        a.KH = static_cast<int>(KH); a.KW = static_cast<int>(KW); a.groups = static_cast<int>(G);
        st->out = new_tensor(id, HIPIE_F32, nn, h, ww, c);
        st->name = n.name;
        st->type = is_mm ? "MatMul" : (grouped ? "GroupConvolution" : "Convolution");
        st->f32_kernel = true;
        st->macs = n.numel() * icg * KD * KH * KW;
        st->bytes = st->src.bytes(tensors) + static_cast<int64_t>(st->weights.size()) * 4 + n.numel() * 4;
        st->out_node = id;
        values[id].kind = VK_TENSOR;
        values[id].tensor = st->out;
        steps.push_back(std::move(st));
    }

    // FakeQuantize whose result stays f32 (the layer behind it was not transformed): fake_quantize.hpp:175-194 as it stands
    void plan_fq_f32(int id) {
        const GNode& n = N(id);
        auto st = std::make_unique<FqF32Step>();
        if (!f32_input(n.in[0], st->src))
            unsupported(id, "FakeQuantize with an f32 result reads an f32 graph input, an f32 tensor or a dequantized byte tensor of rank 2 or 4");
        std::vector<float> b[4];
        size_t count = 1;
        for (int i = 0; i < 4; ++i) {
            if (!channel_constant(n.in[1 + i], st->src.c, n.shape.size(), b[i]))
                unsupported(id, "FakeQuantize bounds must be scalars or per-channel constants");
            count = std::max(count, b[i].size());
        }
        HIPIE_REQUIRE(n.levels >= 2, HIPIE_PARAMETER_MISMATCH, "node %d: %lld levels", id, (long long)n.levels);
        st->lm1 = static_cast<float>(n.levels - 1);
        st->channels.resize(count);
        for (size_t ch = 0; ch < count; ++ch) {
            auto at = [&](int i) { return b[i][b[i].size() == 1 ? 0 : ch]; };
            FqChannel& f = st->channels[ch];
            f.il = at(0); f.ih = at(1); f.ol = at(2); f.oh = at(3);
            f.lo = std::min(f.il, f.ih); f.hi = std::max(f.il, f.ih);
            f.d = f.ih - f.il;
            f.r = 0.f;
        }
        st->out = new_tensor(id, HIPIE_F32, st->src.n, st->src.h, st->src.w, st->src.c);
        st->name = n.name;
        st->type = "FakeQuantize";
        st->bytes = st->src.bytes(tensors) + n.numel() * 4;
        st->out_node = id;
        values[id].kind = VK_TENSOR;
        values[id].tensor = st->out;
        steps.push_back(std::move(st));
    }

    void plan_softmax_f32(int id) {
        const GNode& n = N(id);
        auto st = std::make_unique<SoftmaxF32Step>();
        if (!f32_input(n.in[0], st->src))
            unsupported(id, "Softmax reads an f32 graph input, an f32 tensor or a dequantized byte tensor of rank 2 or 4");
        st->axis = static_cast<int>(n.axes[0]);
        st->out = new_tensor(id, HIPIE_F32, st->src.n, st->src.h, st->src.w, st->src.c);
        st->name = n.name;
        st->type = "Softmax";
        st->f32_kernel = true;
        st->bytes = st->src.bytes(tensors) + n.numel() * 4 * 3;
        st->out_node = id;
        values[id].kind = VK_TENSOR;
        values[id].tensor = st->out;
        steps.push_back(std::move(st));
    }

    void plan_conv(int id) {
        const GNode& n = N(id);
        if (N(n.in[1]).op == OP_CONSTANT && N(n.in[1]).dtype == HIPIE_F32) {
            plan_conv_f32(id);
            return;
        }
        const bool is_mm = n.op == OP_MATMUL;
        if (!is_mm && (n.strides.size() != 2 || n.depth > 0))
            unsupported(id, "quantized convolutions are planned over one and two spatial dimensions (three: with f32 weights only)");
        const Value x = value(n.in[0]);
        // Subtract(zero point) in front of the convolution: an integer per tensor (what optimizeSubtract
        // leaves, network_helper.cpp:1479-1521) goes into the accumulators' initial value
        int zero_point = 0;
        std::vector<int32_t> zero_points;   // filled when the channels' zero points differ
        if (x.kind == VK_DEQ && x.mul.empty() && !x.sub.empty() && tensors[x.tensor].esize() == 1) {
            const float z = x.sub[0];
            bool uniform = true;
            for (float v : x.sub) {
                if (v != std::nearbyintf(v)) unsupported(id, "activation zero point that is not an integer level");
                uniform = uniform && v == z;
            }
            if (uniform) {
                zero_point = static_cast<int>(z);
            } else {
                if (static_cast<int>(x.sub.size()) != tensors[x.tensor].c) unsupported(id, "zero points for other than every input channel");
                for (float v : x.sub) zero_points.push_back(static_cast<int32_t>(v));
            }
        } else if (x.kind != VK_TENSOR || tensors[x.tensor].esize() != 1) {
            unsupported(id, x.kind == VK_DEQ ? "dequantized (f32) convolution inputs are not planned"
                                             : "input must be a quantized (u8/i8) tensor");
        }
        const GNode& W = N(n.in[1]);
        if (W.op != OP_CONSTANT || W.dtype != HIPIE_I8) unsupported(id, "weights must be an i8 constant");
        auto st = std::make_unique<ConvStep>();
        const TensorInfo& tin = tensors[x.tensor];
        hipie_conv_desc& d = st->desc;
        d.groups = 1;
        int64_t OC, IC, grouped_macs_div = 1;
        if (is_mm) {
            if (n.ta || W.shape.size() != 2 || N(n.in[0]).shape.size() != 2)
                unsupported(id, "MatMul is planned for [N,K] x constant [K,OC] / [OC,K]^T");
            IC = n.tb ? W.shape[1] : W.shape[0];
            OC = n.tb ? W.shape[0] : W.shape[1];
            d.kh = d.kw = d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1;
            st->weights.resize(OC * IC);
            const int8_t* w = reinterpret_cast<const int8_t*>(W.data.data());
            for (int64_t o = 0; o < OC; ++o)
                for (int64_t k = 0; k < IC; ++k) st->weights[o * IC + k] = n.tb ? w[o * IC + k] : w[k * OC + o];
            if (x.flat) {
                // rows of [C * H * W] weights are [C][H][W] filters: the layer is the convolution of the whole map
                if (IC != static_cast<int64_t>(tin.c) * tin.h * tin.w) unsupported(id, "MatMul whose reduction length is not the flattened map's");
                IC = tin.c;
                d.kh = tin.h;
                d.kw = tin.w;
            }
        } else {
            const bool grouped = n.op == OP_GROUP_CONVOLUTION;
            // [G, OC/G, IC/G, kh, kw].  One filter per channel (depthwise) has kernels of its own; any other grouping runs
            // as the dense convolution with block-diagonal weights it is equal to (reference::group_convolution,
            // group_convolution.hpp:78-144, convolves each slice on its own: the products outside the blocks are the
            // zeros added here, and integer sums do not change with them)
            const bool depthwise = grouped && W.shape[1] == 1 && W.shape[2] == 1;
            const int64_t G = grouped ? W.shape[0] : 1, ocg = grouped ? W.shape[1] : 0, icg = grouped ? W.shape[2] : 0;
            OC = grouped ? G * ocg : W.shape[0];
            IC = grouped ? G * icg : W.shape[1];
            // groups of 16-byte-aligned channel spans under tiles of 64 output channels run in the grouped form of the
            // tiled kernels (hipie_conv_create decides by the same rule); the weights go to it as they are
            const bool own_form = grouped && !depthwise && G > 1 && OC % 64 == 0 &&
                                  ((64 % ocg == 0 && ((64 / ocg) * icg) % 16 == 0 && (64 / ocg) * icg < IC) || (ocg % 64 == 0 && icg % 16 == 0));
            if (depthwise || own_form) d.groups = static_cast<int>(G);
            grouped_macs_div = grouped && !depthwise ? G : 1;
            d.kh = static_cast<int>(W.shape[grouped ? 3 : 2]); d.kw = static_cast<int>(W.shape[grouped ? 4 : 3]);
            d.stride_h = static_cast<int>(n.strides[0]); d.stride_w = static_cast<int>(n.strides[1]);
            d.dil_h = static_cast<int>(n.dilations[0]); d.dil_w = static_cast<int>(n.dilations[1]);
            d.pad_top = static_cast<int>(n.pads_begin[0]); d.pad_left = static_cast<int>(n.pads_begin[1]);
            d.pad_bottom = static_cast<int>(n.pads_end[0]); d.pad_right = static_cast<int>(n.pads_end[1]);
            const int8_t* wsrc = reinterpret_cast<const int8_t*>(W.data.data());
            if (grouped && !depthwise && !own_form) {
                const int64_t taps = static_cast<int64_t>(d.kh) * d.kw;
                st->weights.assign(static_cast<size_t>(OC * IC * taps), 0);
                for (int64_t gi = 0; gi < G; ++gi)
                    for (int64_t o = 0; o < ocg; ++o)
                        for (int64_t i = 0; i < icg; ++i)
                            for (int64_t t = 0; t < taps; ++t)
                                st->weights[static_cast<size_t>(((gi * ocg + o) * IC + gi * icg + i) * taps + t)] =
                                    wsrc[((gi * ocg + o) * icg + i) * taps + t];
            } else {
                st->weights.assign(wsrc, wsrc + W.data.size());
            }
        }
        d.ic = static_cast<int>(IC);
        d.oc = static_cast<int>(OC);
        HIPIE_REQUIRE(tin.c == IC, HIPIE_PARAMETER_MISMATCH, "node %d: input has %d channels, weights %lld", id,
                      tin.c, (long long)IC);
        const int halo = std::max(std::max(d.pad_top, d.pad_bottom), std::max(d.pad_left, d.pad_right));
        tensors[x.tensor].halo = std::max(tensors[x.tensor].halo, halo);
        st->in = x.tensor;
        d.in_zero_point = zero_point;
        st->zero_points = zero_points;
        if (halo > 0) {   // padding is applied behind the Subtract: the halo must read as the zero point
            TensorInfo& ti = tensors[x.tensor];
            const std::vector<int> levels(zero_points.begin(), zero_points.end());
            if (ti.fill_fixed && (ti.fill_level != zero_point || ti.fill_levels != levels))
                unsupported(id, "consumers of one tensor pad it with different levels");
            ti.fill_level = zero_point;
            ti.fill_levels = levels;
            ti.fill_fixed = true;
        }

        // ---- absorb the elementwise chain behind the accumulator --------------------------------
        EpilogueSpec& e = st->epi;
        int cur = id, stage = 0, shortcut_step = -1;
        const size_t rank = n.shape.size();
        while (single_user(cur)) {
            const int nx = N(cur).users[0];
            const GNode& u = N(nx);
            if (u.op == OP_ADD || u.op == OP_MULTIPLY) {
                const int other = u.in[0] == cur ? u.in[1] : u.in[0];
                std::vector<float> c;
                if (channel_constant(other, OC, rank, c)) {
                    if (u.op == OP_ADD && stage < 1) { e.bias = c; stage = 1; }
                    else if (u.op == OP_MULTIPLY && stage < 2) { e.scale = c; stage = 2; }
                    else if (u.op == OP_MULTIPLY && stage == 3) { e.post_scale = c; stage = 4; }
                    else break;
                } else if (u.op == OP_ADD && stage < 3 && N(other).op != OP_CONSTANT) {
                    // schedules the other branch first; if that branch is the one being planned
                    // right now (it reached this Add from the other side) leave the Add to it
                    if (!visit(other)) break;
                    const Value r = values[other];
                    if (r.kind == VK_DEQ) {
                        const TensorInfo& tr = tensors[r.tensor];
                        e.residual_dtype = tr.dtype;
                        e.res_sub = r.sub;
                        e.res_mul = r.mul;
                    } else if (r.kind == VK_TENSOR && tensors[r.tensor].dtype == HIPIE_F32) {
                        e.residual_dtype = HIPIE_F32;
                        shortcut_step = find_shortcut(r.tensor, other);
                    } else {
                        break;
                    }
                    if (N(other).shape != u.shape) break;
                    st->res = r.tensor;
                    stage = 3;
                } else {
                    break;
                }
            } else if (u.op == OP_RELU && stage < 5) {
                e.activation = 1;
                stage = 5;
            } else if (u.op == OP_CLAMP && stage < 5) {
                e.activation = 2;
                e.clamp_lo = u.lo;
                e.clamp_hi = u.hi;
                stage = 5;
            } else if (u.op == OP_FAKE_QUANTIZE && u.in[0] == cur && u.dtype != HIPIE_F32) {
                std::vector<float> ol, oh;
                if (!channel_constant(u.in[1], OC, rank, e.fq_il) || !channel_constant(u.in[2], OC, rank, e.fq_ih) ||
                    !channel_constant(u.in[3], OC, rank, ol) || !channel_constant(u.in[4], OC, rank, oh) ||
                    ol.size() != 1 || oh.size() != 1)
                    break;
                e.fq_ol = ol[0];
                e.fq_oh = oh[0];
                e.levels = u.levels;
                e.out_dtype = storage_type(u.dtype);
                cur = nx;
                stage = 6;
                break;
            } else {
                break;
            }
            cur = nx;
        }
        if (e.residual_dtype == 0) { e.res_sub.clear(); e.res_mul.clear(); }
        if (shortcut_step >= 0 && st->res >= 0 && !is_mm && d.groups == 1) {
            // take the projection shortcut out of the step list: it runs inside this step
            st->shortcut.reset(static_cast<ConvStep*>(steps[shortcut_step].release()));
            steps.erase(steps.begin() + shortcut_step);
        }
        // mark the absorbed nodes
        for (int k = id; k != cur;) {
            const int nx = N(k).users[0];
            if (nx != cur) values[nx].kind = VK_FUSED;  // never read: its only user is in the chain
            k = nx;
        }
        int nn, c, h, w;
        nhwc_dims(N(cur).shape, nn, c, h, w);
        st->out = new_tensor(cur, e.out_dtype, nn, h, w, c);
        st->name = N(cur).name;
        st->type = is_mm ? "MatMul" : (n.op == OP_GROUP_CONVOLUTION ? "GroupConvolution" : "Convolution");
        st->macs = N(id).numel() * (IC / std::max<int64_t>(d.groups, grouped_macs_div)) * d.kh * d.kw + (st->shortcut ? st->shortcut->macs : 0);
        st->results = N(id).numel();
        // algorithmic HBM bytes: every operand once (input, weights, output, residual); a fused
        // projection shortcut adds its input and weights and removes the f32 residual round trip
        auto elems = [&](int t) {
            const TensorInfo& ti = tensors[t];
            return static_cast<int64_t>(ti.n) * ti.h * ti.w * ti.c * ti.esize();
        };
        st->in_w_bytes = elems(st->in) + static_cast<int64_t>(OC) * (IC / std::max<int64_t>(d.groups, 1)) * d.kh * d.kw;
        st->bytes = st->in_w_bytes + elems(st->out);
        if (st->shortcut) st->bytes += st->shortcut->in_w_bytes;
        else if (st->res >= 0) st->bytes += elems(st->res);
        st->out_node = cur;
        values[cur].kind = VK_TENSOR;
        values[cur].tensor = st->out;
        if (cur != id) values[id].kind = VK_FUSED;
        steps.push_back(std::move(st));
    }

    // A dense convolution step that produces f32 tensor `t` with nothing but bias and scale, consumed
    // only by the residual Add: candidate for running inside the consumer's kernel.
    int find_shortcut(int t, int value_node) const {
        if (N(value_node).users.size() != 1) return -1;
        for (size_t i = 0; i < steps.size(); ++i) {
            auto* cs = dynamic_cast<ConvStep*>(steps[i].get());
            if (!cs || cs->out != t) continue;
            const EpilogueSpec& e = cs->epi;
            const bool plain = !e.bias.empty() && !e.scale.empty() && e.residual_dtype == 0 && e.post_scale.empty() &&
                               e.activation == 0 && e.out_dtype == HIPIE_F32 && cs->desc.groups == 1 && !cs->shortcut;
            return plain && cs->type == "Convolution" ? static_cast<int>(i) : -1;
        }
        return -1;
    }

    void plan_pool(int id) {
        const GNode& n = N(id);
        const Value x = value(n.in[0]);
        if (x.kind != VK_TENSOR || tensors[x.tensor].esize() != 1) {
            plan_pool_f32(id);
            return;
        }
        auto st = std::make_unique<PoolStep>();
        st->avg = n.op == OP_AVG_POOL;
        PoolArgs& a = st->a;
        a.kh = static_cast<int>(n.kernel[0]); a.kw = static_cast<int>(n.kernel[1]);
        a.sh = static_cast<int>(n.strides[0]); a.sw = static_cast<int>(n.strides[1]);
        a.pt = static_cast<int>(n.pads_begin[0]); a.pl = static_cast<int>(n.pads_begin[1]);
        a.pb = static_cast<int>(n.pads_end[0]); a.pr = static_cast<int>(n.pads_end[1]);
        a.include_pad = st->avg && !n.exclude_pad;
        // pooling reads no padding: both kernels keep their windows on the tensor's own cells (the reference
        // skips padding cells), so the border may hold whatever the tensor's other consumers need
        st->in = x.tensor;
        int cur = id;
        int out_dtype = tensors[x.tensor].dtype;
        if (st->avg && n.dtype != HIPIE_F32) {
            // precision preserved (LPT leaves the AvgPool on the quantized type when what reads it is quantized too,
            // low_precision_transformations/src/avg_pool.cpp:36-45): the reference's integer instantiation
            if (storage_type(n.dtype) != tensors[x.tensor].dtype) unsupported(id, "AvgPool whose result type is not its input's");
            a.preserve = tensors[x.tensor].dtype == HIPIE_U8B ? 1 : 2;
        } else if (st->avg) {
            out_dtype = HIPIE_F32;
            const int64_t C = n.shape[1];
            bool scaled = false;
            while (single_user(cur)) {
                const int nx = N(cur).users[0];
                const GNode& u = N(nx);
                std::vector<float> c;
                if (u.op == OP_MULTIPLY && !scaled &&
                    channel_constant(u.in[0] == cur ? u.in[1] : u.in[0], C, u.shape.size(), c)) {
                    st->mul = c;
                    scaled = true;
                } else if (u.op == OP_RESHAPE && N(cur).shape.size() == 4 && N(cur).shape[2] == 1 &&
                           N(cur).shape[3] == 1 && u.shape.size() == 2 && u.shape[1] == C) {
                    // metadata only
                } else if (u.op == OP_FAKE_QUANTIZE && u.in[0] == cur && u.dtype != HIPIE_F32) {
                    std::vector<float> ol, oh;
                    if (!channel_constant(u.in[1], C, u.shape.size(), st->fq_il) ||
                        !channel_constant(u.in[2], C, u.shape.size(), st->fq_ih) ||
                        !channel_constant(u.in[3], C, u.shape.size(), ol) ||
                        !channel_constant(u.in[4], C, u.shape.size(), oh) || ol.size() != 1 || oh.size() != 1)
                        break;
                    st->fq_ol = ol[0];
                    st->fq_oh = oh[0];
                    st->levels = u.levels;
                    out_dtype = storage_type(u.dtype);
                    cur = nx;
                    break;
                } else {
                    break;
                }
                cur = nx;
            }
            for (int k = id; k != cur;) {
                const int nx = N(k).users[0];
                if (nx != cur) values[nx].kind = VK_FUSED;
                k = nx;
            }
        }
        int nn, c, h, w;
        nhwc_dims(n.shape, nn, c, h, w);
        st->out = new_tensor(cur, out_dtype, nn, h, w, c, out_dtype == tensors[x.tensor].dtype ? tensors[x.tensor].cs : 0);
        st->name = N(cur).name;
        st->type = st->avg ? "AvgPool" : "MaxPool";
        st->bytes = N(n.in[0]).numel() + n.numel() * (out_dtype == HIPIE_F32 ? 4 : 1);
        st->out_node = cur;
        values[cur].kind = VK_TENSOR;
        values[cur].tensor = st->out;
        if (cur != id) values[id].kind = VK_FUSED;
        steps.push_back(std::move(st));
    }

    // pooling of an f32 value (a layer in front of the first FakeQuantize, or behind a layer left in f32)
    void plan_pool_f32(int id) {
        const GNode& n = N(id);
        auto st = std::make_unique<PoolF32Step>();
        if (n.shape.size() != 4 || n.dtype != HIPIE_F32 || !f32_input(n.in[0], st->src))
            unsupported(id, "pooling is planned on quantized (u8/i8) tensors and on 4-D f32 values");
        PoolF32Args& a = st->geo;
        a.avg = n.op == OP_AVG_POOL;
        a.kh = static_cast<int>(n.kernel[0]); a.kw = static_cast<int>(n.kernel[1]);
        a.sh = static_cast<int>(n.strides[0]); a.sw = static_cast<int>(n.strides[1]);
        a.pt = static_cast<int>(n.pads_begin[0]); a.pl = static_cast<int>(n.pads_begin[1]);
        a.pb = static_cast<int>(n.pads_end[0]); a.pr = static_cast<int>(n.pads_end[1]);
        a.include_pad = a.avg && !n.exclude_pad;
        int nn, c, h, w;
        nhwc_dims(n.shape, nn, c, h, w);
        a.N = nn; a.C = c; a.H = st->src.h; a.W = st->src.w; a.OH = h; a.OW = w;
        st->out = new_tensor(id, HIPIE_F32, nn, h, w, c);
        st->name = n.name;
        st->type = a.avg ? "AvgPool" : "MaxPool";
        st->f32_kernel = true;
        st->bytes = st->src.bytes(tensors) + n.numel() * 4;
        st->out_node = id;
        values[id].kind = VK_TENSOR;
        values[id].tensor = st->out;
        steps.push_back(std::move(st));
    }

    // Concat of quantized branches (after LPT they share one interval, concat.cpp:42-190, and the dequantization sits
    // behind the Concat): the levels are copied side by side
    void plan_concat(int id) {
        const GNode& n = N(id);
        if (n.shape.size() != 4 || n.axes[0] < 0) unsupported(id, "Concat is planned on 4-D tensors");
        auto st = std::make_unique<ConcatStep>();
        st->axis = static_cast<int>(n.axes[0]);
        const int ax = st->axis;
        int dtype = -1, off = 0;
        int64_t bytes = 0;
        for (int in : n.in) {
            const Value x = value(in);
            // quantized branches (their levels side by side), or f32 ones (branches no FakeQuantize follows)
            if (x.kind != VK_TENSOR)
                unsupported(id, "Concat inputs must be quantized (u8/i8) or f32 tensors: dequantized branches are concatenated by LPT before it");
            if (dtype >= 0 && tensors[x.tensor].dtype != dtype) unsupported(id, "Concat of values of different types");
            dtype = tensors[x.tensor].dtype;
            st->ins.push_back(x.tensor);
            st->c_off.push_back(off);
            off += static_cast<int>(N(in).shape[static_cast<size_t>(ax)]);
            bytes += N(in).numel() * tensors[x.tensor].esize();
        }
        int nn, c, h, w;
        nhwc_dims(n.shape, nn, c, h, w);
        st->out = new_tensor(id, dtype, nn, h, w, c);
        st->name = n.name;
        st->type = "Concat";
        st->bytes = 2 * bytes;
        st->out_node = id;
        values[id].kind = VK_TENSOR;
        values[id].tensor = st->out;
        steps.push_back(std::move(st));
    }

    // An elementwise node nothing absorbed: Add / Subtract / Multiply of two values (or a value and a per-channel
    // constant in an order a dequantization does not have), Relu, Clamp, or a FakeQuantize of a computed value; with the
    // Relu | Clamp and the FakeQuantize that follow it taken into the same kernel.
    void plan_eltwise(int id) {
        const GNode& n = N(id);
        // ([N, C, H, W], or [N, C] behind a flattening Reshape or an f32 MatMul: a tensor with one pixel per batch element)
        if (n.shape.size() != 4 && n.shape.size() != 2) unsupported(id, "stand-alone elementwise nodes are planned on [N, C, H, W] and [N, C] values");
        int nn, c, h, w;
        nhwc_dims(n.shape, nn, c, h, w);
        auto st = std::make_unique<EltwiseStep>();
        auto operand = [&](int in, EltwiseStep::Operand& o) {
            if (N(in).op == OP_CONSTANT) {
                // (a PRelu's one-dimensional slope with one element per channel names the channels, prelu.hpp:28-35)
                const GNode& k = N(in);
                if (n.op == OP_PRELU && k.dtype == HIPIE_F32 && k.shape.size() == 1 && k.shape[0] == c && n.shape.size() > 1)
                    o.konst.assign(k.f32(), k.f32() + c);
                else if (!channel_constant(in, c, n.shape.size(), o.konst)) unsupported(id, "elementwise constant must be scalar or per-channel");
                return;
            }
            const Value x = value(in);
            // numpy broadcasting between two tensors along the batch and the spatial axes (a per-image, per-channel
            // factor [N, C, 1, 1] on a feature map, a per-pixel map shared by the batch, ...); not along the channels
            const std::vector<int64_t>& xs = N(in).shape;
            if (xs.size() != n.shape.size() || (xs.size() > 1 && xs[1] != n.shape[1]))
                unsupported(id, "elementwise operands that differ in rank or in their channels (broadcast along the channel axis)");
            for (size_t k = 0; k < xs.size(); ++k) {
                if (xs[k] == n.shape[k]) continue;
                if (xs[k] != 1) unsupported(id, "elementwise operands whose shapes do not broadcast");
                (k == 0 ? o.bn : (k == 2 ? o.bh : o.bw)) = true;
            }
            if (x.kind == VK_DEQ) {
                o.tensor = x.tensor;
                o.sub = x.sub;
                o.mul = x.mul;
            } else if (x.kind == VK_TENSOR && tensors[x.tensor].dtype == HIPIE_F32) {
                o.tensor = x.tensor;
            } else if (x.kind == VK_PARAM && N(in).op == OP_PARAMETER && N(in).dtype == HIPIE_F32) {
                o.tensor = param_as_tensor(in);
            } else {
                unsupported(id, "elementwise operand must be an f32 graph input, an f32 tensor or a dequantized byte tensor");
            }
        };
        const bool binary = n.op == OP_ADD || n.op == OP_SUBTRACT || n.op == OP_MULTIPLY || n.op == OP_PRELU;
        operand(n.in[0], st->a);
        if (binary) {
            operand(n.in[1], st->b);
            st->op = n.op == OP_ADD ? 1 : (n.op == OP_SUBTRACT ? 2 : (n.op == OP_MULTIPLY ? 3 : 4));
            if (st->a.tensor < 0 && st->b.tensor < 0) unsupported(id, "elementwise node on two constants (constant folding is the front end's)");
        }
        int cur = id;
        auto is_activation = [](int op) {
            return op == OP_RELU || op == OP_CLAMP || op == OP_SIGMOID || op == OP_HSWISH || op == OP_HSIGMOID || op == OP_SWISH;
        };
        auto take_activation = [&](const GNode& u) {
            if (u.op == OP_RELU) st->act = 1;
            else if (u.op == OP_CLAMP) { st->act = 2; st->lo = u.lo; st->hi = u.hi; }
            else if (u.op == OP_SIGMOID) st->act = 3;
            else if (u.op == OP_HSWISH) st->act = 4;
            else if (u.op == OP_HSIGMOID) st->act = 5;
            else { st->act = 6; st->lo = u.lo; }      // Swish: beta
        };
        auto take_fq = [&](int node) {
            const GNode& u = N(node);
            std::vector<float> ol, oh;
            if (u.dtype == HIPIE_F32 || !channel_constant(u.in[1], c, u.shape.size(), st->il) ||
                !channel_constant(u.in[2], c, u.shape.size(), st->ih) || !channel_constant(u.in[3], c, u.shape.size(), ol) ||
                !channel_constant(u.in[4], c, u.shape.size(), oh) || ol.size() != 1 || oh.size() != 1)
                return false;
            st->quantize = true;
            st->levels = u.levels;
            st->ol = ol[0];
            st->oh = oh[0];
            return true;
        };
        if (is_activation(n.op)) take_activation(n);
        if (n.op == OP_FAKE_QUANTIZE) {
            if (!take_fq(id)) unsupported(id, "FakeQuantize with f32 output or bounds that are not per-channel constants");
        } else {
            while (single_user(cur) && !st->quantize) {
                const int nx = N(cur).users[0];
                const GNode& u = N(nx);
                if (is_activation(u.op) && st->act == 0) take_activation(u);
                else if (u.op == OP_FAKE_QUANTIZE && u.in[0] == cur && take_fq(nx)) {}
                else break;
                cur = nx;
            }
            mark_chain(id, cur);
        }
        const int out_dtype = st->quantize ? storage_type(N(cur).dtype) : HIPIE_F32;
        st->out = new_tensor(cur, out_dtype, nn, h, w, c);
        st->name = N(cur).name;
        st->type = std::string(n.op == OP_FAKE_QUANTIZE ? "FakeQuantize" : op_name(n.op)) + (st->quantize && n.op != OP_FAKE_QUANTIZE ? "+FakeQuantize" : "");
        st->bytes = n.numel() * ((st->a.tensor >= 0 ? tensors[st->a.tensor].esize() : 0) + (st->b.tensor >= 0 ? tensors[st->b.tensor].esize() : 0) +
                                 (out_dtype == HIPIE_F32 ? 4 : 1));
        st->out_node = cur;
        values[cur].kind = VK_TENSOR;
        values[cur].tensor = st->out;
        steps.push_back(std::move(st));
    }

    void plan_result(int id) {
        const GNode& n = N(id);
        const Value x = value(n.in[0]);
        if (x.kind != VK_TENSOR && x.kind != VK_DEQ) unsupported(id, "result of a constant or parameter");
        auto st = std::make_unique<ExitStep>();
        st->in = x.tensor;
        st->C = tensors[x.tensor].c;
        st->sub = x.sub;
        st->mul = x.mul;
        st->out_u8 = x.kind == VK_TENSOR && tensors[x.tensor].esize() == 1;
        for (size_t i = 0; i < g.results.size(); ++i)
            if (g.results[i] == id) st->result_index = static_cast<int>(i);
        st->name = n.name;
        st->type = "Result";
        st->bytes = n.numel() * 5;
        st->out_node = id;
        steps.push_back(std::move(st));
    }
};

}  // namespace
}  // namespace hipie

using namespace hipie;

struct hipie_plan {
    int device = 0;
    hipie_graph graph;                       // the description the plan was compiled from (what an export writes)
    std::vector<TensorInfo> tensors;
    std::vector<std::unique_ptr<Step>> steps;
    std::map<int, int> node_tensor;          // graph node -> tensor holding its value
    struct Slice { int tensor; int64_t offset, rows, cols, pitch; };
    std::map<int, Slice> node_slice;         // graph node -> rows x cols window of a tensor (row-major views)
    int64_t arena_bytes = 0;
    struct Io { std::string name; int dtype; std::vector<int64_t> shape; int64_t bytes; };
    std::vector<Io> inputs, outputs;
    PlanConfig config;
    std::map<int, DeviceBuffer> fill_patterns;   // tensor -> cs bytes: what a pixel of its halo holds, channel by channel
    // what building the steps computed on the host, kept for export: a plan loaded from a stream that holds them
    // uploads the packed operands and takes the checks' verdicts instead of packing and checking again
    FqVerdicts verdicts;
    PackTape tape;
};

struct hipie_request {
    const hipie_plan* plan = nullptr;
    DeviceBuffer arena;
    std::vector<DeviceBuffer> in_dev, out_dev;
    hipStream_t stream = nullptr;
    bool perf = false;
    std::vector<hipEvent_t> events;
    // written by the thread that starts and waits, and by whichever thread calls hipie_request_cancel meanwhile
    std::atomic<bool> started{false};
    std::atomic<bool> cancelled{false};      // hipie_request_cancel was called on the running inference
    std::vector<void*> pending_out;          // host destinations of the running async infer
    ~hipie_request() {
        for (auto e : events) (void)hipEventDestroy(e);
        if (stream) {
            (void)hipStreamSynchronize(stream);
            if (plan) release_split_workspace(plan->device, stream);
            (void)hipStreamDestroy(stream);
        }
    }
};

namespace {

// every pixel of a tensor (halo included) gets the byte pattern[c] in channel c
__global__ void fill_pixels(uint8_t* p, int64_t pixels, int cs, const uint8_t* pattern) {
    const int64_t n = pixels * cs;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        p[i] = pattern[i % cs];
}

__global__ void fill_bytes(uint8_t* p, int64_t n, uint8_t v) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) p[i] = v;
}

void enqueue(hipie_request* r, void* const* in, void* const* out) {
    const hipie_plan& p = *r->plan;
    uint8_t* arena = r->arena.as<uint8_t>();
    for (size_t i = 0; i < p.steps.size(); ++i) {
        if (r->perf) HIPIE_CHECK_HIP(hipEventRecord(r->events[i], r->stream));
        p.steps[i]->run(arena, p.tensors, in, out, r->stream);
    }
    if (r->perf) HIPIE_CHECK_HIP(hipEventRecord(r->events[p.steps.size()], r->stream));
}

// `preset`: kernel variants of an imported plan, one per step; used when they fit the steps planned
// here (same count, variants exactly where steps have them), else the plan is tuned like a new one
struct PlanPrepared {       // the host work an exported plan carries (hipie_plan_import)
    FqVerdicts verdicts;
    PackTape tape;
};

// The planner's values have two spatial dimensions.  Convolutions and pools over ONE ([N, C, W]) are planned over two
// with H = 1 - what reference::convolution does with its own shapes (extend_to_3D, convolution.hpp:148-167: unit
// dimensions in front of the spatial ones, stride and dilation 1 and no padding along them).  Convolutions over THREE
// ([N, C, D, H, W]) keep their attributes and filters, and their values are held as [N, C, D * H, W]: the same bytes
// with depth and rows named by one index (GNode::depth keeps D for the kernel).  Every value of the same rank connected
// to such a node through nodes that keep the layout (FakeQuantize, elementwise, Convert, Concat, pools, convolutions,
// inputs and results) changes with it; the constants they read get or lose the unit axis in the same place.
// Returns false when the graph has no such node (`out` is then untouched).
bool to_two_spatial_dimensions(const hipie_graph& g, hipie_graph& out) {
    auto spatial_op = [](int op) { return op == OP_CONVOLUTION || op == OP_GROUP_CONVOLUTION || op == OP_MAX_POOL || op == OP_AVG_POOL; };
    auto keeps_layout = [&](int op) {
        return spatial_op(op) || op == OP_FAKE_QUANTIZE || op == OP_ADD || op == OP_SUBTRACT || op == OP_MULTIPLY || op == OP_RELU || op == OP_PRELU || op == OP_SIGMOID ||
               op == OP_HSWISH || op == OP_HSIGMOID || op == OP_SWISH ||
               op == OP_CLAMP || op == OP_CONVERT || op == OP_CONCAT || op == OP_PARAMETER || op == OP_RESULT;
    };
    const int n_nodes = static_cast<int>(g.nodes.size());
    std::vector<char> change(g.nodes.size(), 0);
    std::vector<int> stack;
    for (int i = 0; i < n_nodes; ++i) {
        const GNode& n = g.nodes[static_cast<size_t>(i)];
        if (spatial_op(n.op) && (n.shape.size() == 3 || n.shape.size() == 5)) { change[static_cast<size_t>(i)] = 1; stack.push_back(i); }
    }
    if (stack.empty()) return false;
    while (!stack.empty()) {
        const int v = stack.back();
        stack.pop_back();
        const GNode& n = g.nodes[static_cast<size_t>(v)];
        auto take = [&](int u) {
            const GNode& m = g.nodes[static_cast<size_t>(u)];
            if (change[static_cast<size_t>(u)] || m.shape.size() != n.shape.size() || !keeps_layout(m.op)) return;
            change[static_cast<size_t>(u)] = 1;
            stack.push_back(u);
        };
        // (a convolution's filter and a FakeQuantize's bounds are constants: handled below, never part of the walk)
        for (int in : n.in)
            if (in >= 0 && g.nodes[static_cast<size_t>(in)].op != OP_CONSTANT) take(in);
        for (int u : n.users) take(u);
    }
    out = g;
    auto unit_axis = [](std::vector<int64_t>& shape, size_t at) { shape.insert(shape.begin() + static_cast<std::ptrdiff_t>(at), 1); };
    auto front = [](std::vector<int64_t>& v, int64_t unit) { v.insert(v.begin(), unit); };
    for (int i = 0; i < n_nodes; ++i) {
        if (!change[static_cast<size_t>(i)]) continue;
        GNode& n = out.nodes[static_cast<size_t>(i)];
        const bool filter_op = n.op == OP_CONVOLUTION || n.op == OP_GROUP_CONVOLUTION;
        if (n.shape.size() == 5) {
            // [N, C, D, H, W] -> [N, C, D * H, W]
            if (filter_op) n.depth = g.nodes[static_cast<size_t>(n.in[0])].shape[2];
            n.shape = {n.shape[0], n.shape[1], n.shape[2] * n.shape[3], n.shape[4]};
            if (n.op == OP_CONCAT && !n.axes.empty()) {
                // along the depth: whole blocks of rows side by side, the same bytes; along the rows: not these bytes
                if (n.axes[0] == 3) n.axes[0] = -1;             // refused by the planner (no such axis)
                else if (n.axes[0] == 4) n.axes[0] = 3;
            }
            for (size_t k = 0; k < n.in.size(); ++k) {
                if (n.in[k] < 0 || (filter_op && k == 1)) continue;
                GNode& c = out.nodes[static_cast<size_t>(n.in[k])];
                // [1, C, 1, 1, 1] and the like lose a unit axis; anything that names a depth or a row stays and is refused
                if (c.op == OP_CONSTANT && c.shape.size() == 5 && c.shape[2] == 1 && c.shape[3] == 1) c.shape.erase(c.shape.begin() + 2);
            }
            continue;
        }
        unit_axis(n.shape, 2);
        if (spatial_op(n.op)) {
            front(n.strides, 1);
            front(n.pads_begin, 0);
            front(n.pads_end, 0);
            if (n.op == OP_MAX_POOL || n.op == OP_AVG_POOL) front(n.kernel, 1);
            else front(n.dilations, 1);
        }
        if (n.op == OP_CONCAT && !n.axes.empty() && n.axes[0] == 2) n.axes[0] = 3;
        for (size_t k = 0; k < n.in.size(); ++k) {
            if (n.in[k] < 0) continue;
            GNode& c = out.nodes[static_cast<size_t>(n.in[k])];
            if (c.op != OP_CONSTANT) continue;
            const bool filter = filter_op && k == 1;
            const size_t full = filter ? (n.op == OP_GROUP_CONVOLUTION ? 4u : 3u) : 3u;
            // filters [OC, IC, KW] / [G, OC/G, IC/G, KW] and constants that name the width axis: the unit axis goes in
            // front of the last one; lower ranks align from the right as before, except [C, 1], which names the channels
            if (c.shape.size() == full || (!filter && c.shape.size() == 2)) unit_axis(c.shape, c.shape.size() - 1);
        }
    }
    return true;
}

std::unique_ptr<hipie_plan> compile_plan(const hipie_graph* g, int device, const std::vector<int>* preset,
                                         const PlanConfig& cfg = PlanConfig::from_environment(), PlanPrepared* prepared = nullptr) {
    HIPIE_REQUIRE(!g->results.empty(), HIPIE_PARAMETER_MISMATCH, "hipie_compile: graph has no Result");
    HIPIE_REQUIRE(cfg.device_id < 0 || device < 0 || cfg.device_id == device, HIPIE_PARAMETER_MISMATCH,
                  "hipie_compile: DEVICE_ID %d against device %d", cfg.device_id, device);
    auto plan = std::make_unique<hipie_plan>();
    plan->device = device;
    plan->graph = *g;                       // the description as it was given: what an exported plan carries
    const hipie_graph* const described = g;
    hipie_graph lifted;
    if (to_two_spatial_dimensions(*g, lifted)) g = &lifted;
    if (prepared) {
        plan->verdicts = std::move(prepared->verdicts);
        plan->tape = std::move(prepared->tape);
        plan->tape.playing = true;
        plan->tape.next = 0;
    }
    FqVerdicts::Scope verdict_scope(&plan->verdicts);
    PackTape::Scope tape_scope(&plan->tape);
    plan->config = cfg;
    plan->config.device_id = device;
    Planner pl(*g, cfg);
    for (int r : g->results) pl.visit(r);
    // arena layout: one region per tensor, 256-byte aligned, with slack on both sides so that
    // K-padding reads of a first-layer filter row stay inside the arena
    int64_t off = 256;
    for (auto& t : pl.tensors) {
        t.bytes = static_cast<int64_t>(t.n) * t.hp() * t.wp() * t.cs * t.esize();
        if (t.alias >= 0) {
            t.offset = pl.tensors[t.alias].offset;
            continue;
        }
        t.offset = off;
        off = round_up(off + t.bytes + 256, 256);
    }
    plan->arena_bytes = off;
    plan->tensors = pl.tensors;
    if (device >= 0)
        for (size_t i = 0; i < plan->tensors.size(); ++i) {
            const TensorInfo& t = plan->tensors[i];
            if (t.fill_levels.empty() || t.alias >= 0) continue;
            std::vector<uint8_t> pattern(t.cs, static_cast<uint8_t>(t.dtype == HIPIE_U8B ? 0x80 : 0));   // padding channels: level 0
            for (int c = 0; c < t.c; ++c) pattern[c] = static_cast<uint8_t>((t.fill_levels[c] - (t.dtype == HIPIE_U8B ? 128 : 0)) & 0xff);
            plan->fill_patterns[static_cast<int>(i)].upload(device, pattern.data(), pattern.size());
        }
    for (auto& s : pl.steps) s->create(device, plan->tensors);
    HIPIE_REQUIRE(!plan->tape.playing || plan->tape.next == plan->tape.blobs.size(), HIPIE_NETWORK_NOT_READ,
                  "hipie_plan_import: %zu packed operands in the stream, %zu used", plan->tape.blobs.size(), plan->tape.next);
    plan->steps = std::move(pl.steps);
    {
        auto type_name = [](int dt) {
            return dt == HIPIE_F32 ? "FP32" : (dt == HIPIE_I32 ? "I32" : (dt == HIPIE_I8 ? "I8" : "U8"));
        };
        std::vector<char> seen(g->nodes.size(), 0);
        for (auto& s : plan->steps) {
            if (s->out_node < 0) continue;
            // the step's own node and every node behind it that was fused away (chains, merged siblings, shortcuts)
            std::vector<int> stack(1, s->out_node), found;
            while (!stack.empty()) {
                const int v = stack.back();
                stack.pop_back();
                if (seen[v]) continue;
                seen[v] = 1;
                found.push_back(v);
                for (int in : g->nodes[v].in)
                    if (in >= 0 && pl.values[in].kind == VK_FUSED && g->nodes[in].op != OP_CONSTANT) stack.push_back(in);
            }
            std::sort(found.begin(), found.end());
            for (int v : found) s->original_names += (s->original_names.empty() ? "" : ",") + g->nodes[v].name;
            s->nodes = found;
            const GNode& on = g->nodes[s->out_node];
            for (size_t k = 0; k < on.shape.size(); ++k) s->output_dims += (k ? "," : "") + std::to_string(on.shape[k]);
            s->output_precision = type_name(on.dtype);
            s->output_layout = on.shape.size() == 4 ? "NHWC" : (on.shape.size() == 2 ? "NC" : (on.shape.size() == 3 ? "CHW" : "ANY"));
            // integer kernels compute in the type of the activations they read (through a symbolic dequantization
            // in front of them); everything else in f32
            int in_dt = HIPIE_F32;
            const bool integer_kernel = s->type.find("Convolution") != std::string::npos || s->type.find("MatMul") != std::string::npos ||
                                        s->type.find("Pool") != std::string::npos || s->type.find("Attention") != std::string::npos ||
                                        s->type == "Transpose";
            if (integer_kernel && !s->f32_kernel)
                for (int v : found)
                    for (int in : g->nodes[v].in) {
                        if (in < 0 || g->nodes[in].op == OP_CONSTANT || std::binary_search(found.begin(), found.end(), in)) continue;
                        const Value& iv = pl.values[in];
                        int dt = HIPIE_F32;
                        if ((iv.kind == VK_TENSOR || iv.kind == VK_DEQ) && iv.tensor >= 0) dt = pl.tensors[iv.tensor].dtype;
                        else if (iv.kind == VK_MAT) dt = iv.view.dtype;
                        if (dt == HIPIE_U8B || dt == HIPIE_U8) in_dt = HIPIE_U8;
                        else if (dt == HIPIE_I8 && in_dt != HIPIE_U8) in_dt = HIPIE_I8;
                    }
            s->runtime_precision = type_name(in_dt);
        }
    }
    // Bottleneck tails: a 3 x 3 convolution whose result only the next 1 x 1 convolution reads becomes one step with it
    // (the pair stands where the 1 x 1 layer stood: everything it reads is computed by then)
    if (cfg.fuse_convs != 0)
        for (size_t i = 0; i < plan->steps.size(); ++i) {
            auto* a = dynamic_cast<ConvStep*>(plan->steps[i].get());
            if (!a || !a->conv || a->shortcut || a->res >= 0 || a->res_param >= 0 || a->out_node < 0 || a->desc.kh != 3 || a->desc.kw != 3) continue;
            if (g->nodes[a->out_node].users.size() != 1) continue;
            size_t j = i + 1;
            ConvStep* b = nullptr;
            for (; j < plan->steps.size() && !b; ++j) {
                auto* c = dynamic_cast<ConvStep*>(plan->steps[j].get());
                if (c && c->in == a->out) b = c;
            }
            if (!b || !b->conv || b->shortcut || b->res < 0) continue;
            --j;
            int fits = 0;
            const TensorInfo& ti = plan->tensors[a->in];
            if (hipie_conv_pair_fits(a->conv, b->conv, ti.h, ti.w, &fits) != HIPIE_OK || !fits) continue;
            auto pair = std::make_unique<PairStep>();
            pair->mode = cfg.fuse_convs;
            pair->first.reset(static_cast<ConvStep*>(plan->steps[i].release()));
            pair->second.reset(static_cast<ConvStep*>(plan->steps[j].release()));
            pair->create(device, plan->tensors);
            plan->steps[j] = std::move(pair);
            plan->steps.erase(plan->steps.begin() + static_cast<std::ptrdiff_t>(i));
            --i;
        }
    {
        // the edges of the executed graph (what GetExecGraphInfo draws): an operand of a step is a node outside its set -
        // computed by another step, held by a tensor another step produced (a symbolic dequantization in between belongs
        // to nobody), or a graph input
        std::map<int, int> step_of_node, param_index;
        for (size_t i = 0; i < plan->steps.size(); ++i)
            for (int v : plan->steps[i]->nodes) step_of_node[v] = static_cast<int>(i);
        for (size_t k = 0; k < g->params.size(); ++k) param_index[g->params[k]] = static_cast<int>(k);
        for (size_t i = 0; i < plan->steps.size(); ++i) {
            Step& st = *plan->steps[i];
            std::vector<int> src;
            for (int v : st.nodes) {
                std::vector<int> pending(g->nodes[v].in.begin(), g->nodes[v].in.end());
                while (!pending.empty()) {
                    const int in = pending.back();
                    pending.pop_back();
                    if (in < 0 || g->nodes[in].op == OP_CONSTANT || std::binary_search(st.nodes.begin(), st.nodes.end(), in)) continue;
                    int from = 0;
                    bool known = true;
                    const auto own = step_of_node.find(in);
                    if (own != step_of_node.end() && own->second != static_cast<int>(i)) from = own->second;
                    else if (param_index.count(in)) from = -(1 + param_index[in]);
                    else if (own == step_of_node.end()) {   // a node no step owns (Convert / Subtract / Multiply over bytes, Reshape): look through it
                        for (int up : g->nodes[in].in) pending.push_back(up);
                        known = false;
                    } else known = false;
                    if (known && std::find(src.begin(), src.end(), from) == src.end()) src.push_back(from);
                }
            }
            st.sources = src;
        }
    }
    for (size_t i = 0; i < pl.values.size(); ++i)
        if (pl.values[i].kind == VK_TENSOR) {
            plan->node_tensor[static_cast<int>(i)] = pl.values[i].tensor;
        } else if (pl.values[i].kind == VK_MAT) {   // a view that is [rows, cols] with one row pitch
            const View& v = pl.values[i].view;
            const size_t r = v.rank();
            bool ok = v.tensor >= 0 && r >= 1 && v.stride[r - 1] == 1;
            for (size_t k = 0; ok && k + 2 < r; ++k) ok = v.stride[k] == v.stride[k + 1] * v.shape[k + 1];
            if (ok) {
                const int64_t cols = v.shape[r - 1], rows = v.numel() / cols;
                plan->node_slice[static_cast<int>(i)] = {v.tensor, v.offset, rows, cols, r >= 2 ? v.stride[r - 2] : cols};
            }
        }
    // (inputs and outputs in the shapes of the description: [N, C, W] and [N, C, 1, W] are the same bytes)
    for (int p : described->params) {
        const GNode& n = described->nodes[p];
        plan->inputs.push_back({n.name, n.dtype, n.shape, n.numel() * (n.dtype == HIPIE_F32 || n.dtype == HIPIE_I32 ? 4 : 1)});
    }
    for (int r : described->results) {
        const GNode& n = described->nodes[r];
        const int dt = n.dtype == HIPIE_F32 ? HIPIE_F32 : HIPIE_U8;
        plan->outputs.push_back({n.name, dt, n.shape, n.numel() * (dt == HIPIE_F32 ? 4 : 1)});
    }
    // Kernel selection by measurement on a scratch request (HIPIE_TUNE=0 keeps the shape-based
    // defaults).  HIPIE_TUNE_FILE names a cache of the choices, one "step variant" pair a line:
    // read when it matches this plan, written after tuning otherwise (the reference's GPU plugin
    // keeps its tuning results in a file the same way, inference-engine/include/cldnn/cldnn_config.hpp:125 KEY_TUNING_FILE).
    bool preset_used = false;
    if (device >= 0 && preset && preset->size() == plan->steps.size()) {
        bool match = true;
        for (size_t i = 0; match && i < preset->size(); ++i) match = ((*preset)[i] < 0) == (plan->steps[i]->variant() < 0);
        if (match) {
            for (size_t i = 0; i < preset->size(); ++i) plan->steps[i]->set_variant((*preset)[i]);
            preset_used = true;
        }
    }
    if (device >= 0 && !preset_used && cfg.tune) {
        const char* cache = cfg.tune_file.empty() ? nullptr : cfg.tune_file.c_str();
        bool loaded = false;
        if (cache) {
            if (FILE* f = std::fopen(cache, "r")) {
                std::vector<int> v(plan->steps.size(), -2);
                size_t n = 0;
                int idx = 0, var = 0;
                while (std::fscanf(f, "%d %d", &idx, &var) == 2)
                    if (idx >= 0 && static_cast<size_t>(idx) < v.size() && v[idx] == -2) {
                        v[idx] = var;
                        ++n;
                    }
                std::fclose(f);
                bool match = n == v.size();
                for (size_t i = 0; match && i < v.size(); ++i)
                    match = (v[i] < 0) == (plan->steps[i]->variant() < 0);
                if (match) {
                    for (size_t i = 0; i < v.size(); ++i) plan->steps[i]->set_variant(v[i]);
                    loaded = true;
                }
            }
        }
        if (!loaded) {
            // HIPIE_TUNE_STREAMS requests are assumed in flight together (default 3, the throughput
            // mode of a plugin with three streams; 1 tunes for the latency of a lone request)
            const int n_lanes = std::max(1, std::min(8, cfg.streams));
            struct Scratch {
                std::vector<hipie_request*> r;
                ~Scratch() { for (auto* q : r) hipie_request_destroy(q); }
            } scratch;
            std::vector<TuneLane> lanes;
            for (int l = 0; l < n_lanes; ++l) {
                hipie_request* q = nullptr;
                check_status(hipie_request_create(plan.get(), 0, &q), "hipie_compile: tuning request");
                scratch.r.push_back(q);
                TuneLane lane{q->arena.as<uint8_t>(), q->stream, {}};
                for (auto& b : q->in_dev) lane.inputs.push_back(b.ptr);
                lanes.push_back(std::move(lane));
            }
            DeviceGuard dg(device);
            for (auto& s : plan->steps) s->tune(lanes, plan->tensors);
            if (cache) {
                if (FILE* f = std::fopen(cache, "w")) {
                    for (size_t i = 0; i < plan->steps.size(); ++i)
                        std::fprintf(f, "%zu %d\n", i, plan->steps[i]->variant());
                    std::fclose(f);
                }
            }
        }
    }
    return plan;
}

constexpr char kPlanMagic[8] = {'H', 'I', 'P', 'I', 'E', 'P', 'L', 'N'};
constexpr uint32_t kPlanFormat = 2;

uint64_t fnv1a(const uint8_t* p, size_t n) {
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < n; ++i) h = (h ^ p[i]) * 1099511628211ull;
    return h;
}

}  // namespace

extern "C" {

int hipie_compile(const hipie_graph* g, int device, hipie_plan** out) {
    return guarded([&] {
        HIPIE_REQUIRE(g && out, HIPIE_PARAMETER_MISMATCH, "hipie_compile: null argument");
        *out = compile_plan(g, device, nullptr).release();
    });
}

int hipie_compile_opts(const hipie_graph* g, int device, const char* const* keys, const char* const* values, int n_opts,
                       hipie_plan** out) {
    return guarded([&] {
        HIPIE_REQUIRE(g && out && n_opts >= 0 && (n_opts == 0 || (keys && values)), HIPIE_PARAMETER_MISMATCH,
                      "hipie_compile_opts: null argument");
        PlanConfig cfg = PlanConfig::from_environment();
        for (int i = 0; i < n_opts; ++i) cfg.set(keys[i], values[i]);
        *out = compile_plan(g, device, nullptr, cfg).release();
    });
}

/* IInferencePlugin::QueryNetwork (template_plugin.cpp:117-195): which nodes of the graph this engine can take.
 * The planner is run without a device; a node it refuses is marked, turned into a boundary (its value becomes an
 * input of the rest, its own inputs become results so that what feeds it is still planned) and the planner runs
 * again, until a plan exists.  A node counts as supported when no run refused it. */
int hipie_query(const hipie_graph* g, int* supported, int n_nodes, int* n_unsupported) {
    return guarded([&] {
        HIPIE_REQUIRE(g && supported && n_nodes == static_cast<int>(g->nodes.size()), HIPIE_PARAMETER_MISMATCH,
                      "hipie_query: `supported` must hold one entry per node (%zu)", g ? g->nodes.size() : size_t(0));
        hipie_graph work = *g;
        {
            hipie_graph lifted;
            if (to_two_spatial_dimensions(work, lifted)) work = std::move(lifted);
        }
        for (int i = 0; i < n_nodes; ++i) supported[i] = 1;
        int bad = 0;
        const PlanConfig cfg = PlanConfig::from_environment();
        for (int round = 0; round <= n_nodes; ++round) {
            try {
                if (work.results.empty()) break;
                Planner pl(work, cfg);
                for (int r : work.results) pl.visit(r);
                break;
            } catch (const UnsupportedNode& u) {
                HIPIE_REQUIRE(u.node >= 0 && u.node < n_nodes && supported[u.node], HIPIE_UNEXPECTED,
                              "hipie_query: the planner refused node %d twice", u.node);
                supported[u.node] = 0;
                ++bad;
                GNode& x = work.nodes[u.node];
                const std::vector<int> feeds = x.in;
                if (x.op == OP_RESULT) {
                    work.results.erase(std::remove(work.results.begin(), work.results.end(), u.node), work.results.end());
                } else {
                    for (int f : feeds) {                       // this node no longer uses its inputs
                        auto& us = work.nodes[f].users;
                        us.erase(std::remove(us.begin(), us.end(), u.node), us.end());
                    }
                    x.op = OP_PARAMETER;
                    x.in.clear();
                    x.data.clear();
                    work.params.push_back(u.node);
                }
                for (int f : feeds) {                           // what fed it is still wanted: a result of the rest
                    const GNode& fn = work.nodes[f];
                    if (fn.op == OP_CONSTANT || fn.op == OP_PARAMETER) continue;
                    GNode res;
                    res.op = OP_RESULT;
                    res.in = {f};
                    res.dtype = fn.dtype;
                    res.shape = fn.shape;
                    res.name = "query_boundary_" + std::to_string(f);
                    work.nodes[f].users.push_back(static_cast<int>(work.nodes.size()));
                    work.results.push_back(static_cast<int>(work.nodes.size()));
                    work.nodes.push_back(std::move(res));
                }
            }
        }
        if (n_unsupported) *n_unsupported = bad;
    });
}

static int copy_text(const std::string& v, char* buf, size_t cap, const char* what) {
    HIPIE_REQUIRE(buf && cap > v.size(), HIPIE_OUT_OF_BOUNDS, "%s: %zu bytes needed", what, v.size() + 1);
    std::memcpy(buf, v.c_str(), v.size() + 1);
    return HIPIE_OK;
}

/* IInferencePlugin::GetMetric (template_plugin.cpp:218-259): device-level metrics as text */
int hipie_get_metric(int device, const char* name, char* buf, size_t cap) {
    return guarded([&] {
        HIPIE_REQUIRE(name, HIPIE_PARAMETER_MISMATCH, "hipie_get_metric: null name");
        const std::string k = name;
        std::string v;
        if (k == "SUPPORTED_METRICS")
            v = "AVAILABLE_DEVICES SUPPORTED_METRICS SUPPORTED_CONFIG_KEYS FULL_DEVICE_NAME IMPORT_EXPORT_SUPPORT DEVICE_ARCHITECTURE "
                "OPTIMIZATION_CAPABILITIES RANGE_FOR_ASYNC_INFER_REQUESTS RANGE_FOR_STREAMS";
        else if (k == "SUPPORTED_CONFIG_KEYS") v = kConfigKeys;
        else if (k == "AVAILABLE_DEVICES") {
            const int n = hipie_device_count();
            for (int i = 0; i < n; ++i) v += (i ? " " : "") + std::to_string(i);
        } else if (k == "FULL_DEVICE_NAME") {
            char nm[256] = "";
            check_status(hipie_device_name(device, nm, sizeof nm), "hipie_get_metric");
            v = nm;
        } else if (k == "IMPORT_EXPORT_SUPPORT") v = "YES";
        else if (k == "DEVICE_ARCHITECTURE") v = "gfx950";
        // INT8 only: convolutions and MatMuls are planned over quantized operands alone (an unquantized one is refused and
        // reported unsupported by hipie_query); f32 is what the elementwise, Softmax, MVN and Gelu steps between them compute in
        else if (k == "OPTIMIZATION_CAPABILITIES") v = "INT8";
        else if (k == "RANGE_FOR_ASYNC_INFER_REQUESTS") v = "1 8 1";
        else if (k == "RANGE_FOR_STREAMS") v = "1 8";
        else fail(HIPIE_NOT_FOUND, "metric '%s' is not supported", name);
        copy_text(v, buf, cap, "hipie_get_metric");
    });
}

/* IExecutableNetworkInternal::GetMetric / GetConfig (template_executable_network.cpp:154-176) */
int hipie_plan_get_metric(const hipie_plan* p, const char* name, char* buf, size_t cap) {
    return guarded([&] {
        HIPIE_REQUIRE(p && name, HIPIE_PARAMETER_MISMATCH, "hipie_plan_get_metric: null argument");
        const std::string k = name;
        std::string v;
        if (k == "SUPPORTED_METRICS") v = "NETWORK_NAME SUPPORTED_METRICS SUPPORTED_CONFIG_KEYS OPTIMAL_NUMBER_OF_INFER_REQUESTS";
        else if (k == "SUPPORTED_CONFIG_KEYS") v = kConfigKeys;
        else if (k == "NETWORK_NAME") v = p->config.network_name;
        else if (k == "OPTIMAL_NUMBER_OF_INFER_REQUESTS") v = std::to_string(p->config.streams);
        else fail(HIPIE_NOT_FOUND, "metric '%s' is not supported", name);
        copy_text(v, buf, cap, "hipie_plan_get_metric");
    });
}

int hipie_plan_get_config(const hipie_plan* p, const char* key, char* buf, size_t cap) {
    return guarded([&] {
        HIPIE_REQUIRE(p && key, HIPIE_PARAMETER_MISMATCH, "hipie_plan_get_config: null argument");
        std::string v;
        HIPIE_REQUIRE(p->config.get(key, v), HIPIE_NOT_FOUND, "config key '%s' is not supported", key);
        copy_text(v, buf, cap, "hipie_plan_get_config");
    });
}

/* stream layout: magic[8], format u32, step count u32, one i32 kernel variant per step, graph bytes u64 + the graph
 * description, the load-time checks' verdicts (count u64 + 6 u32 each: il, ih, d, r, levels - 1, exact; count u64 +
 * 4 u32 each: d, zh, zl, verified), the packed operands (count u64, then byte count u64 + bytes each), FNV-1a of
 * everything before it u64 */
int hipie_plan_export(const hipie_plan* p, void* buffer, size_t capacity, size_t* size) {
    return guarded([&] {
        HIPIE_REQUIRE(p && size, HIPIE_PARAMETER_MISMATCH, "hipie_plan_export: null argument");
        const size_t head = 16 + 4 * p->steps.size();
        const size_t graph_bytes = serialize_graph(p->graph, nullptr);
        size_t prepared = 8 + 24 * p->verdicts.rcp.size() + 8 + 16 * p->verdicts.div2.size() + 8;
        for (const auto& blob : p->tape.blobs) prepared += 8 + blob.size();
        *size = head + 8 + graph_bytes + prepared + 8;
        if (!buffer) return;                              // size query
        HIPIE_REQUIRE(capacity >= *size, HIPIE_OUT_OF_BOUNDS, "hipie_plan_export: %zu bytes needed, %zu given", *size, capacity);
        uint8_t* b = static_cast<uint8_t*>(buffer);
        std::memcpy(b, kPlanMagic, 8);
        const uint32_t fmt = kPlanFormat, ns = static_cast<uint32_t>(p->steps.size());
        std::memcpy(b + 8, &fmt, 4);
        std::memcpy(b + 12, &ns, 4);
        for (size_t i = 0; i < p->steps.size(); ++i) {
            const int32_t v = p->steps[i]->variant();
            std::memcpy(b + 16 + 4 * i, &v, 4);
        }
        const uint64_t gb = graph_bytes;
        std::memcpy(b + head, &gb, 8);
        serialize_graph(p->graph, b + head + 8);
        uint8_t* w = b + head + 8 + graph_bytes;
        auto put = [&](const void* src, size_t n) {
            std::memcpy(w, src, n);
            w += n;
        };
        auto put64 = [&](uint64_t v) { put(&v, 8); };
        put64(p->verdicts.rcp.size());
        for (const auto& kv : p->verdicts.rcp) {
            put(kv.first.data(), 20);
            put(&kv.second, 4);
        }
        put64(p->verdicts.div2.size());
        for (const auto& kv : p->verdicts.div2) {
            put(&kv.first, 4);
            put(&kv.second.zh, 4);
            put(&kv.second.zl, 4);
            put(&kv.second.ok, 4);
        }
        put64(p->tape.blobs.size());
        for (const auto& blob : p->tape.blobs) {
            put64(blob.size());
            put(blob.data(), blob.size());
        }
        const uint64_t h = fnv1a(b, *size - 8);
        std::memcpy(b + *size - 8, &h, 8);
    });
}

int hipie_plan_import(const void* blob, size_t size, int device, hipie_plan** out) {
    return guarded([&] {
        HIPIE_REQUIRE(blob && out, HIPIE_PARAMETER_MISMATCH, "hipie_plan_import: null argument");
        const uint8_t* b = static_cast<const uint8_t*>(blob);
        HIPIE_REQUIRE(size >= 8 + 4 + 4 + 8 + 24 + 8 && std::memcmp(b, kPlanMagic, 8) == 0, HIPIE_NETWORK_NOT_READ,
                      "hipie_plan_import: not an exported plan");
        uint32_t fmt, ns;
        std::memcpy(&fmt, b + 8, 4);
        std::memcpy(&ns, b + 12, 4);
        HIPIE_REQUIRE(fmt == kPlanFormat, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: stream format %u, this library reads %u", fmt, kPlanFormat);
        uint64_t stored;
        std::memcpy(&stored, b + size - 8, 8);
        HIPIE_REQUIRE(stored == fnv1a(b, size - 8), HIPIE_NETWORK_NOT_READ, "hipie_plan_import: checksum mismatch (damaged stream)");
        HIPIE_REQUIRE(ns <= (size - 56) / 4, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: %u steps in %zu bytes", ns, size);
        std::vector<int> variants(ns);
        for (uint32_t i = 0; i < ns; ++i) {
            int32_t v;
            std::memcpy(&v, b + 16 + 4 * size_t(i), 4);
            variants[i] = v;
        }
        const size_t at = 16 + 4 * size_t(ns);
        const uint8_t* const end = b + size - 8;            // the checksum follows
        uint64_t gb;
        std::memcpy(&gb, b + at, 8);
        HIPIE_REQUIRE(gb <= size - at - 8 - 24 - 8, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: graph description of %llu bytes in a stream of %zu",
                      (unsigned long long)gb, size);
        std::unique_ptr<hipie_graph> g(deserialize_graph(b + at + 8, static_cast<size_t>(gb)));
        const uint8_t* r = b + at + 8 + gb;
        auto need = [&](uint64_t n, const char* what) {
            HIPIE_REQUIRE(n <= static_cast<uint64_t>(end - r), HIPIE_NETWORK_NOT_READ, "hipie_plan_import: the stream ends inside its %s", what);
        };
        auto get64 = [&](const char* what) {
            need(8, what);
            uint64_t v;
            std::memcpy(&v, r, 8);
            r += 8;
            return v;
        };
        PlanPrepared prepared;
        const uint64_t n_rcp = get64("verdicts");
        HIPIE_REQUIRE(n_rcp <= static_cast<uint64_t>(end - r) / 24, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: %llu verdicts", (unsigned long long)n_rcp);
        for (uint64_t i = 0; i < n_rcp; ++i) {
            std::array<uint32_t, 5> key;
            uint32_t exact;
            std::memcpy(key.data(), r, 20);
            std::memcpy(&exact, r + 20, 4);
            r += 24;
            HIPIE_REQUIRE(exact <= 1, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: verdict %u", exact);
            prepared.verdicts.rcp[key] = exact;
        }
        const uint64_t n_div2 = get64("division constants");
        HIPIE_REQUIRE(n_div2 <= static_cast<uint64_t>(end - r) / 16, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: %llu divisors", (unsigned long long)n_div2);
        for (uint64_t i = 0; i < n_div2; ++i) {
            uint32_t key;
            FqVerdicts::Div2 v;
            std::memcpy(&key, r, 4);
            std::memcpy(&v.zh, r + 4, 4);
            std::memcpy(&v.zl, r + 8, 4);
            std::memcpy(&v.ok, r + 12, 4);
            r += 16;
            HIPIE_REQUIRE(v.ok <= 1, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: verdict %u", v.ok);
            prepared.verdicts.div2[key] = v;
        }
        const uint64_t n_blobs = get64("packed operands");
        HIPIE_REQUIRE(n_blobs <= static_cast<uint64_t>(end - r) / 8, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: %llu packed operands", (unsigned long long)n_blobs);
        prepared.tape.blobs.reserve(static_cast<size_t>(n_blobs));
        for (uint64_t i = 0; i < n_blobs; ++i) {
            const uint64_t n = get64("packed operands");
            need(n, "packed operands");
            prepared.tape.blobs.emplace_back(r, r + n);
            r += n;
        }
        HIPIE_REQUIRE(r == end, HIPIE_NETWORK_NOT_READ, "hipie_plan_import: %zu bytes behind the packed operands", static_cast<size_t>(end - r));
        *out = compile_plan(g.get(), device, &variants, PlanConfig::from_environment(), &prepared).release();
    });
}

void hipie_plan_destroy(hipie_plan* p) { delete p; }

int hipie_plan_num_inputs(const hipie_plan* p) { return p ? static_cast<int>(p->inputs.size()) : 0; }
int hipie_plan_num_outputs(const hipie_plan* p) { return p ? static_cast<int>(p->outputs.size()) : 0; }
int hipie_plan_num_steps(const hipie_plan* p) { return p ? static_cast<int>(p->steps.size()) : 0; }
int64_t hipie_plan_arena_bytes(const hipie_plan* p) { return p ? p->arena_bytes : 0; }

int hipie_plan_io_desc(const hipie_plan* p, int is_output, int index, char* name, size_t name_len, int* dtype,
                       int64_t* dims, int* rank) {
    return guarded([&] {
        HIPIE_REQUIRE(p && dtype && dims && rank, HIPIE_PARAMETER_MISMATCH, "hipie_plan_io_desc: null argument");
        const auto& v = is_output ? p->outputs : p->inputs;
        HIPIE_REQUIRE(index >= 0 && index < static_cast<int>(v.size()), HIPIE_OUT_OF_BOUNDS,
                      "hipie_plan_io_desc: index %d", index);
        if (name && name_len) snprintf(name, name_len, "%s", v[index].name.c_str());
        *dtype = v[index].dtype;
        *rank = static_cast<int>(v[index].shape.size());
        HIPIE_REQUIRE(*rank <= 8, HIPIE_UNEXPECTED, "hipie_plan_io_desc: rank %d", *rank);   // `dims` holds 8 entries
        for (int i = 0; i < *rank; ++i) dims[i] = v[index].shape[i];
    });
}

int hipie_plan_step_info(const hipie_plan* p, int index, char* name, size_t name_len, char* type,
                         size_t type_len, int64_t* macs, int64_t* bytes) {
    return guarded([&] {
        HIPIE_REQUIRE(p && index >= 0 && index < static_cast<int>(p->steps.size()), HIPIE_OUT_OF_BOUNDS,
                      "hipie_plan_step_info: index %d", index);
        const Step& s = *p->steps[index];
        if (name && name_len) snprintf(name, name_len, "%s", s.name.c_str());
        if (type && type_len) snprintf(type, type_len, "%s", s.type.c_str());
        if (macs) *macs = s.macs;
        if (bytes) *bytes = s.bytes;
    });
}

/* the attributes GetExecGraphInfo attaches to an executed node (exec_graph_info.hpp:34-76), by their key there */
int hipie_plan_step_rt_info(const hipie_plan* p, int index, const char* key, char* buf, size_t cap) {
    return guarded([&] {
        HIPIE_REQUIRE(p && key && index >= 0 && index < static_cast<int>(p->steps.size()), HIPIE_OUT_OF_BOUNDS,
                      "hipie_plan_step_rt_info: index %d", index);
        const Step& s = *p->steps[index];
        const std::string k = key;
        std::string v;
        if (k == "originalLayersNames") v = s.original_names;
        else if (k == "layerType") v = s.type;
        else if (k == "runtimePrecision") v = s.runtime_precision;
        else if (k == "outputPrecisions") v = s.output_precision;
        else if (k == "outputLayouts") v = s.output_layout;
        else if (k == "execOrder") v = std::to_string(index);
        else if (k == "primitiveType") v = s.variant() >= 0 ? "hip_int8_v" + std::to_string(s.variant()) : "hip";
        else if (k == "kernels") v = std::to_string(s.launches());
        else if (k == "valuOps") v = std::to_string(static_cast<long long>(s.valu_ops()));
        else if (k == "epilogueFlags") v = std::to_string(s.epilogue_flags());
        else if (k == "outputDims") v = s.output_dims;
        else fail(HIPIE_NOT_FOUND, "hipie_plan_step_rt_info: key '%s' (execTimeMcs is hipie_request_perf)", key);
        copy_text(v, buf, cap, "hipie_plan_step_rt_info");
    });
}

int hipie_plan_step_sources(const hipie_plan* p, int index, int* sources, int capacity, int* count) {
    return guarded([&] {
        HIPIE_REQUIRE(p && count && index >= 0 && index < static_cast<int>(p->steps.size()), HIPIE_OUT_OF_BOUNDS,
                      "hipie_plan_step_sources: index %d", index);
        const std::vector<int>& src = p->steps[index]->sources;
        *count = static_cast<int>(src.size());
        HIPIE_REQUIRE(sources || capacity == 0, HIPIE_PARAMETER_MISMATCH, "hipie_plan_step_sources: null array");
        for (int i = 0; i < capacity && i < *count; ++i) sources[i] = src[static_cast<size_t>(i)];
    });
}

int hipie_plan_step_variant(const hipie_plan* p, int index, int* variant) {
    return guarded([&] {
        HIPIE_REQUIRE(p && variant && index >= 0 && index < static_cast<int>(p->steps.size()), HIPIE_OUT_OF_BOUNDS,
                      "hipie_plan_step_variant: index %d", index);
        *variant = p->steps[index]->variant();
    });
}

int hipie_request_create(const hipie_plan* p, int perf_count, hipie_request** out) {
    return guarded([&] {
        HIPIE_REQUIRE(p && out, HIPIE_PARAMETER_MISMATCH, "hipie_request_create: null argument");
        HIPIE_REQUIRE(p->device >= 0, HIPIE_NOT_ALLOCATED,
                      "hipie_request_create: the plan was compiled without a device (dry run)");
        auto r = std::make_unique<hipie_request>();
        r->plan = p;
        r->perf = perf_count < 0 ? p->config.perf_count : perf_count != 0;   // < 0: the plan's PERF_COUNT
        DeviceGuard g(p->device);
        HIPIE_CHECK_HIP(hipStreamCreateWithFlags(&r->stream, hipStreamNonBlocking));
        r->arena.alloc(p->device, static_cast<size_t>(p->arena_bytes));
        // level 0 everywhere: halos and channel padding are never written again
        uint8_t* a = r->arena.as<uint8_t>();
        HIPIE_CHECK_HIP(hipMemsetAsync(a, 0, static_cast<size_t>(p->arena_bytes), r->stream));
        for (const auto& t : p->tensors) {
            if (t.alias >= 0) continue;
            const int byte = t.dtype == HIPIE_U8B ? t.fill_level - 128 : (t.dtype == HIPIE_I8 ? t.fill_level : 0);
            if (byte != 0)
                hipLaunchKernelGGL(fill_bytes, dim3(1024), dim3(256), 0, r->stream, a + t.offset, t.bytes,
                                   static_cast<uint8_t>(byte & 0xff));
        }
        for (const auto& kv : p->fill_patterns) {
            const TensorInfo& t = p->tensors[kv.first];
            hipLaunchKernelGGL(fill_pixels, dim3(1024), dim3(256), 0, r->stream, a + t.offset,
                               static_cast<int64_t>(t.n) * t.hp() * t.wp(), t.cs, kv.second.as<uint8_t>());
        }
        HIPIE_CHECK_HIP(hipGetLastError());
        for (const auto& io : p->inputs) {
            r->in_dev.emplace_back();
            r->in_dev.back().alloc(p->device, static_cast<size_t>(io.bytes));
        }
        for (const auto& io : p->outputs) {
            r->out_dev.emplace_back();
            r->out_dev.back().alloc(p->device, static_cast<size_t>(io.bytes));
        }
        if (r->perf) {
            r->events.resize(p->steps.size() + 1);
            for (auto& e : r->events) HIPIE_CHECK_HIP(hipEventCreate(&e));
        }
        HIPIE_CHECK_HIP(hipStreamSynchronize(r->stream));
        *out = r.release();
    });
}

void hipie_request_destroy(hipie_request* r) {
    if (r && r->stream) (void)hipStreamSynchronize(r->stream);
    delete r;
}

int hipie_request_stream(hipie_request* r, void** stream) {
    return guarded([&] {
        HIPIE_REQUIRE(r && stream, HIPIE_PARAMETER_MISMATCH, "hipie_request_stream: null argument");
        *stream = r->stream;
    });
}

int hipie_request_start(hipie_request* r, const void* const* inputs, void* const* outputs, int device_memory) {
    return guarded([&] {
        HIPIE_REQUIRE(r && inputs && outputs, HIPIE_PARAMETER_MISMATCH, "hipie_request_start: null argument");
        HIPIE_REQUIRE(!r->started, HIPIE_REQUEST_BUSY, "hipie_request_start: request is busy");
        const hipie_plan& p = *r->plan;
        DeviceGuard g(p.device);
        // a failure half-way leaves copies or kernels queued that read the caller's buffers: the stream is drained
        // before the error is reported, so that the caller may free or reuse them
        struct Drain {
            hipStream_t s;
            bool armed = true;
            ~Drain() { if (armed) (void)hipStreamSynchronize(s); }
        } drain{r->stream};
        std::vector<void*> in(p.inputs.size()), out(p.outputs.size());
        for (size_t i = 0; i < in.size(); ++i) {
            HIPIE_REQUIRE(inputs[i], HIPIE_PARAMETER_MISMATCH, "hipie_request_start: input %zu is null", i);
            if (device_memory) {
                in[i] = const_cast<void*>(inputs[i]);
            } else {
                in[i] = r->in_dev[i].ptr;
                HIPIE_CHECK_HIP(hipMemcpyAsync(in[i], inputs[i], static_cast<size_t>(p.inputs[i].bytes),
                                               hipMemcpyHostToDevice, r->stream));
            }
        }
        for (size_t i = 0; i < out.size(); ++i) {
            HIPIE_REQUIRE(outputs[i], HIPIE_PARAMETER_MISMATCH, "hipie_request_start: output %zu is null", i);
            out[i] = device_memory ? outputs[i] : r->out_dev[i].ptr;
        }
        enqueue(r, in.data(), out.data());
        if (!device_memory)
            for (size_t i = 0; i < out.size(); ++i)
                HIPIE_CHECK_HIP(hipMemcpyAsync(outputs[i], out[i], static_cast<size_t>(p.outputs[i].bytes),
                                               hipMemcpyDeviceToHost, r->stream));
        drain.armed = false;
        r->started = true;
        r->cancelled = false;
    });
}

/* Wait(millis_timeout) of AsyncInferRequestThreadSafeDefault (ie_infer_async_request_thread_safe_default.hpp:167-204):
 * -1 (RESULT_READY) blocks until the result is there, 0 (STATUS_ONLY) only asks, a positive value waits that many
 * milliseconds at most; HIPIE_RESULT_NOT_READY leaves the request busy.  A request that was cancelled while it
 * ran reports HIPIE_INFER_CANCELLED once its queued work has drained, and is idle afterwards. */
int hipie_request_wait_for(hipie_request* r, int64_t timeout_ms) {
    return guarded([&] {
        HIPIE_REQUIRE(r, HIPIE_PARAMETER_MISMATCH, "hipie_request_wait_for: null argument");
        HIPIE_REQUIRE(timeout_ms >= -1, HIPIE_PARAMETER_MISMATCH,
                      "hipie_request_wait_for: timeout %lld (RESULT_READY = -1, STATUS_ONLY = 0, or milliseconds)", (long long)timeout_ms);
        HIPIE_REQUIRE(r->started, HIPIE_INFER_NOT_STARTED, "hipie_request_wait: nothing was started");
        DeviceGuard g(r->plan->device);
        if (timeout_ms < 0) {
            // (the request stays busy while this blocks: a Cancel from another thread in the meantime is seen below)
            const hipError_t e = hipStreamSynchronize(r->stream);
            r->started = false;
            HIPIE_CHECK_HIP(e);
        } else {
            const auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(timeout_ms);
            for (;;) {
                const hipError_t q = hipStreamQuery(r->stream);
                if (q == hipSuccess) break;
                if (q != hipErrorNotReady) HIPIE_CHECK_HIP(q);
                if (std::chrono::steady_clock::now() >= deadline) fail(HIPIE_RESULT_NOT_READY, "the inference is still running");
                std::this_thread::sleep_for(std::chrono::microseconds(50));
            }
            r->started = false;
        }
        if (r->cancelled.exchange(false)) fail(HIPIE_INFER_CANCELLED, "the inference was cancelled");
    });
}

int hipie_request_wait(hipie_request* r) { return hipie_request_wait_for(r, -1); }

/* Cancel (ie_infer_async_request_thread_safe_default.hpp:255-267).  The kernels and copies of a started inference are
 * already queued on the request's stream and run to their end (nothing on the device can be revoked); the request is
 * marked, its outputs are to be taken as undefined, and the next wait reports HIPIE_INFER_CANCELLED.  On an idle
 * request it does nothing. */
int hipie_request_cancel(hipie_request* r) {
    return guarded([&] {
        HIPIE_REQUIRE(r, HIPIE_PARAMETER_MISMATCH, "hipie_request_cancel: null argument");
        if (r->started) r->cancelled = true;
    });
}

int hipie_request_infer(hipie_request* r, const void* const* inputs, void* const* outputs, int device_memory) {
    const int st = hipie_request_start(r, inputs, outputs, device_memory);
    return st != HIPIE_OK ? st : hipie_request_wait(r);
}

/* enqueue only (no copies, no synchronisation): inputs/outputs are device buffers and the caller
 * owns ordering on the request's stream; used for back-to-back throughput runs */
int hipie_request_enqueue(hipie_request* r, const void* const* inputs, void* const* outputs) {
    return guarded([&] {
        HIPIE_REQUIRE(r && inputs && outputs, HIPIE_PARAMETER_MISMATCH, "hipie_request_enqueue: null argument");
        DeviceGuard g(r->plan->device);
        std::vector<void*> in(r->plan->inputs.size());
        for (size_t i = 0; i < in.size(); ++i) in[i] = const_cast<void*>(inputs[i]);
        enqueue(r, in.data(), outputs);
    });
}

int hipie_request_perf(hipie_request* r, int step, float* ms) {
    return guarded([&] {
        HIPIE_REQUIRE(r && ms, HIPIE_PARAMETER_MISMATCH, "hipie_request_perf: null argument");
        HIPIE_REQUIRE(r->perf, HIPIE_NOT_FOUND, "hipie_request_perf: request was created without PERF_COUNT");
        HIPIE_REQUIRE(step >= 0 && step < static_cast<int>(r->plan->steps.size()), HIPIE_OUT_OF_BOUNDS,
                      "hipie_request_perf: step %d", step);
        HIPIE_CHECK_HIP(hipEventElapsedTime(ms, r->events[step], r->events[step + 1]));
    });
}

/* the arena tensor that holds the value of graph node `node_id` (for inspection and tests) */
int hipie_request_tensor(const hipie_request* r, int node_id, hipie_tensor* t) {
    return guarded([&] {
        HIPIE_REQUIRE(r && t, HIPIE_PARAMETER_MISMATCH, "hipie_request_tensor: null argument");
        auto sl = r->plan->node_slice.find(node_id);
        if (sl != r->plan->node_slice.end()) {   // row-major value: n = h = 1, w = rows, c = columns
            const hipie_plan::Slice& v = sl->second;
            const TensorInfo& ti = r->plan->tensors[v.tensor];
            t->dtype = ti.dtype;
            t->n = t->h = 1;
            t->w = static_cast<int32_t>(v.rows);
            t->c = static_cast<int32_t>(v.cols);
            t->stride_w = v.pitch;
            t->stride_h = t->stride_n = v.pitch * v.rows;
            t->halo = 0;
            t->data = r->arena.as<uint8_t>() + ti.offset + v.offset * ti.esize();
            return;
        }
        auto it = r->plan->node_tensor.find(node_id);
        HIPIE_REQUIRE(it != r->plan->node_tensor.end(), HIPIE_NOT_FOUND,
                      "hipie_request_tensor: node %d was fused away or is not a tensor", node_id);
        for (const auto& st : r->plan->steps)
            if (auto* pair = dynamic_cast<const PairStep*>(st.get()))
                HIPIE_REQUIRE(!(pair->fused && pair->first->out == it->second), HIPIE_NOT_FOUND,
                              "hipie_request_tensor: node %d lives in LDS only (two convolutions run as one kernel)", node_id);
        *t = r->plan->tensors[it->second].desc(r->arena.as<uint8_t>());
    });
}

}  // extern "C"
