"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares, and
its load-time (host) logic agrees with the oracle.  No kernel is launched here."""
import os
import re

import numpy as np
import pytest

import dldt_amd
from dldt_amd import FakeQuantize, HipieError

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for fn in os.listdir(os.path.join(ROOT, "include")):
        src = open(os.path.join(ROOT, "include", fn)).read()
        src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
        names |= set(re.findall(r"\b(hipie_\w+)\s*\(", src))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    lib = dldt_amd.lib()
    syms = declared_symbols()
    assert len(syms) >= 8
    missing = [s for s in syms if not hasattr(lib, s)]
    assert not missing, missing
    assert b"gfx950" in lib.hipie_version()


def test_fq_create_rejects_bad_arguments():
    with pytest.raises(HipieError) as e:
        FakeQuantize(4, 256, [0, 0, 0], 1.0, 0.0, 255.0, device=-1)   # 3 values for 4 channels
    assert e.value.status == -4
    with pytest.raises(HipieError):
        FakeQuantize(4, 1, 0.0, 1.0, 0.0, 255.0, device=-1)           # levels < 2


def test_fq_host_arithmetic_matches_oracle(orc):
    rng = np.random.default_rng(0)
    C = 48
    il = rng.uniform(-3, -1, C).astype(np.float32)
    ih = rng.uniform(1, 3, C).astype(np.float32)
    fq = FakeQuantize(C, 256, il, ih, 0.0, 255.0, device=-1)
    assert fq.uses_reciprocal
    x = rng.normal(0, 2, 4000).astype(np.float32)
    # (a channel with il <= -2 and ih >= 2 among them: the load-time check bisects between the bounds' ordered integer
    # images, which are 2^31 or more apart there)
    wide = int(np.argmax((il <= -2) & (ih >= 2)))
    assert il[wide] <= -2 and ih[wide] >= 2
    for c in (0, 17, 47, wide):
        # tie-dense probe: level midpoints of this channel and their float neighbours
        k = np.arange(255, dtype=np.float32) + np.float32(0.5)
        mid = (il[c] + (ih[c] - il[c]) * (k / np.float32(255))).astype(np.float32)
        xs = np.concatenate([x, mid, np.nextafter(mid, np.float32(9)), np.nextafter(mid, np.float32(-9))])
        want = orc.fake_quantize(xs.reshape(1, 1, -1), il[c], ih[c], np.float32(0), np.float32(255), 256)
        got = np.array([fq.host_eval(c, v) for v in xs], np.float32)
        np.testing.assert_array_equal(got, want.ravel())


def test_fq_host_only_object_cannot_run():
    import ctypes
    fq = FakeQuantize(4, 256, 0.0, 1.0, 0.0, 255.0, device=-1)
    st = dldt_amd.lib().hipie_fq_run_f32(fq._h, ctypes.c_void_p(16), ctypes.c_void_p(16),
                                         ctypes.c_int64(1), ctypes.c_int64(4), None)
    assert st == -10  # NOT_ALLOCATED


def _host_conv(c, oc, k, epilogue=None):
    """a convolution object without a device (weights packed on the host only)"""
    import types
    from dldt_amd import Convolution
    t = types.SimpleNamespace(dtype=41, cs=-(-c // 16) * 16, stride_w=-(-c // 16) * 16, stride_h=20 * (-(-c // 16) * 16))
    w = np.random.default_rng(1).integers(-127, 128, (oc, c, k, k)).astype(np.int8)
    return Convolution(w, t, pads_begin=(k // 2, k // 2), pads_end=(k // 2, k // 2), epilogue=epilogue, device=-1)


def test_conv_variant_numbers_are_checked_without_a_device():
    """hipie_conv_set_tile: unknown numbers, the K split over workgroups on a K loop too short for its parts,
    the first-layer and row-tile kernels on geometries they do not take"""
    from dldt_amd import HipieError
    long_k = _host_conv(256, 64, 3)            # 36 K steps of 64 bytes
    for tile in (0, 4, 12, 14, 15, 16, 17, 18, 19, 20, 21, 22):
        long_k.set_tile(tile)
    short_k = _host_conv(64, 64, 1)            # one K step of 64 bytes: no 128-byte K steps either
    short_k.set_tile(22)
    short_k.set_tile(23)                       # an unpadded 1 x 1 with raw sums: the few-pixel kernel takes it
    for tile in (24, -1, 12, 13, 14, 17, 18, 21):
        with pytest.raises(HipieError) as e:
            short_k.set_tile(tile)
        assert e.value.status == -4, tile      # PARAMETER_MISMATCH
    with pytest.raises(HipieError):
        long_k.set_tile(13)                    # not a 4-byte-pixel first layer
    with pytest.raises(HipieError):
        long_k.set_tile(23)                    # not a 1 x 1


def test_epilogue_rejects_an_inverted_clamp_range():
    from dldt_amd import HipieError, make_epilogue
    fq = (256, 0.0, 6.0, 0.0, 255.0)
    _host_conv(32, 32, 1, make_epilogue(activation="clamp", clamp=(0.0, 6.0), out_dtype=41, fq=fq))
    with pytest.raises(HipieError) as e:
        _host_conv(32, 32, 1, make_epilogue(activation="clamp", clamp=(6.0, 0.0), out_dtype=41, fq=fq))
    assert e.value.status == -4


# ---- plugin-level surface: config map, metrics, QueryNetwork, request status paths (no device needed) ----
def _tiny_graph(extra_relu=False):
    """FakeQuantize -> 1x1 convolution -> bias -> FakeQuantize -> dequantization; optionally two stray Gelu nodes"""
    from dldt_amd.graph import Graph
    from dldt_amd.tensor import F32, I8, U8
    g = Graph()
    x = g.parameter("x", (1, 16, 4, 4))
    q = g.fake_quantize(x, 0.0, 2.55, 0.0, 255.0, 256, out_dtype=U8)
    w = g.constant(np.ones((16, 16, 1, 1), np.int8), I8)
    y = g.add(g.convolution(q, w), g.constant(np.zeros((1, 16, 1, 1), np.float32)))
    q2 = g.fake_quantize(y, 0.0, 255.0, 0.0, 255.0, 256, out_dtype=U8)
    out = g.multiply(g.convert(q2, F32), g.constant(np.float32(0.01).reshape(1, 1, 1, 1)))
    ids = dict(x=x, q=q, conv=y, q2=q2, out=out)
    if extra_relu:
        ids["relu_a"] = g.gelu(x)                       # Gelu of a 4-D value: not planned (it runs on the row-major path)
        ids["relu_b"] = g.gelu(g.multiply(x, g.constant(np.float32(2).reshape(1, 1, 1, 1))))
        g.result(ids["relu_a"], "a")
        g.result(ids["relu_b"], "b")
    g.result(out, "y")
    return g, ids


def test_compile_options_and_their_status_codes():
    g, _ = _tiny_graph()
    plan = g.compile(-1, config={"PERF_COUNT": "YES", "HIP_THROUGHPUT_STREAMS": "5", "HIP_TUNE": "NO"})
    assert plan.config("PERF_COUNT") == "YES" and plan.config("HIP_THROUGHPUT_STREAMS") == "5" and plan.config("HIP_TUNE") == "NO"
    assert plan.metric("OPTIMAL_NUMBER_OF_INFER_REQUESTS") == "5"          # what benchmark_app asks the network for
    assert "OPTIMAL_NUMBER_OF_INFER_REQUESTS" in plan.metric("SUPPORTED_METRICS").split()
    assert "HIP_THROUGHPUT_STREAMS" in plan.metric("SUPPORTED_CONFIG_KEYS").split()
    assert g.compile(-1, config={"HIP_THROUGHPUT_STREAMS": "HIP_THROUGHPUT_AUTO"}).metric("OPTIMAL_NUMBER_OF_INFER_REQUESTS") == "3"
    assert g.compile(-1, config={}).config("PERF_COUNT") == "NO"
    with pytest.raises(HipieError) as e:                                       # unknown key: NOT_FOUND
        g.compile(-1, config={"CPU_THREADS_NUM": "4"})
    assert e.value.status == -5 and "CPU_THREADS_NUM" in str(e.value)
    for key, value in (("PERF_COUNT", "maybe"), ("HIP_THROUGHPUT_STREAMS", "0"), ("HIP_THROUGHPUT_STREAMS", "many"),
                       ("DEVICE_ID", "x")):
        with pytest.raises(HipieError) as e:                                   # a value the key does not take
            g.compile(-1, config={key: value})
        assert e.value.status == -4, (key, value)
    with pytest.raises(HipieError) as e:
        plan.metric("NO_SUCH_METRIC")
    assert e.value.status == -5
    with pytest.raises(HipieError) as e:
        plan.config("NO_SUCH_KEY")
    assert e.value.status == -5


def test_environment_variables_are_only_defaults(monkeypatch):
    g, _ = _tiny_graph()
    monkeypatch.setenv("HIPIE_TUNE_STREAMS", "2")
    monkeypatch.setenv("HIPIE_KEEP_F32", "1")
    plan = g.compile(-1, config={})
    assert plan.config("HIP_THROUGHPUT_STREAMS") == "2" and plan.config("HIP_KEEP_F32") == "YES"
    plan = g.compile(-1, config={"HIP_THROUGHPUT_STREAMS": "4", "HIP_KEEP_F32": "NO"})
    assert plan.config("HIP_THROUGHPUT_STREAMS") == "4" and plan.config("HIP_KEEP_F32") == "NO"


def test_device_metrics():
    import ctypes
    lib = dldt_amd.lib()

    def metric(name, cap=1024):
        buf = ctypes.create_string_buffer(cap)
        st = lib.hipie_get_metric(0, name.encode(), buf, ctypes.c_size_t(cap))
        return st, buf.value.decode()

    st, names = metric("SUPPORTED_METRICS")
    assert st == 0
    for name in ("AVAILABLE_DEVICES", "OPTIMIZATION_CAPABILITIES", "RANGE_FOR_ASYNC_INFER_REQUESTS", "IMPORT_EXPORT_SUPPORT",
                 "DEVICE_ARCHITECTURE", "SUPPORTED_CONFIG_KEYS"):
        assert name in names.split()
    # (the unquantized layers of an INT8 network run in f32 kernels that are correct, not fast: not an FP32 device)
    assert metric("OPTIMIZATION_CAPABILITIES") == (0, "INT8")
    assert metric("IMPORT_EXPORT_SUPPORT") == (0, "YES")
    assert metric("DEVICE_ARCHITECTURE") == (0, "gfx950")
    assert metric("RANGE_FOR_ASYNC_INFER_REQUESTS")[1].split() == ["1", "8", "1"]
    assert metric("NO_SUCH_METRIC")[0] == -5
    assert metric("SUPPORTED_METRICS", cap=8)[0] == -6                          # buffer too small: OUT_OF_BOUNDS


def test_query_reports_every_unsupported_node():
    g, ids = _tiny_graph(extra_relu=True)
    with pytest.raises(HipieError) as e:                                       # compiling stops at the first one ...
        g.compile(-1)
    assert e.value.status == -2
    ok = g.query()                                                             # ... the query names them all
    assert len(ok) == len(g.nodes)
    assert not ok[ids["relu_a"]] and not ok[ids["relu_b"]]
    for name in ("x", "q", "conv", "q2", "out"):
        assert ok[ids[name]], name
    g2, ids2 = _tiny_graph()
    assert all(g2.query())


def test_request_entry_points_reject_null_handles():
    import ctypes
    lib = dldt_amd.lib()
    assert lib.hipie_request_wait_for(None, ctypes.c_int64(0)) == -4
    assert lib.hipie_request_cancel(None) == -4
    assert lib.hipie_request_wait(None) == -4


def test_exec_graph_attributes_per_step():
    """what GetExecGraphInfo attaches to an executed node (exec_graph_info.hpp:34-76): the fused original layers, the
    type the kernel computes in (U8 for the integer convolutions, as the CPU plugin reports it), output type / layout"""
    from dldt_amd import HipieError, builders
    g, _ = builders.resnet50(batch=1, res=224)
    plan = g.compile(-1)
    info = [{k: plan.step_rt_info(i, k) for k in ("originalLayersNames", "layerType", "runtimePrecision", "outputPrecisions",
                                                   "outputLayouts", "execOrder", "primitiveType")}
            for i in range(len(plan.steps))]
    assert info[0]["layerType"] == "FakeQuantize" and info[0]["runtimePrecision"] == "FP32" and info[0]["outputPrecisions"] == "U8"
    convs = [r for r in info if r["layerType"].startswith("Convolution")]
    # ten bottleneck tails (3 x 3 -> 1 x 1 + residual, stages 1 to 3 without the blocks whose shortcut is a convolution) are
    # one step each: planned as a pair, run as one kernel or two ("kernels") as the load-time measurement decides
    pairs = [r for r in convs if r["layerType"] in ("Convolution,Convolution", "Convolution+Convolution")]
    assert len(pairs) == 10 and len(convs) == 49 - 10
    assert sum(int(plan.step_rt_info(i, "kernels")) for i in range(len(plan.steps))) == 54
    assert all(r["runtimePrecision"] == "U8" and r["outputLayouts"] == "NHWC" for r in convs)
    assert all(r["primitiveType"].startswith("hip_int8_v") for r in convs)
    # a convolution stands for itself, its bias Add and the FakeQuantize behind it at least
    assert all(len(r["originalLayersNames"].split(",")) >= 3 for r in convs)
    fc = [r for r in info if r["layerType"] == "MatMul"]
    assert len(fc) == 1 and fc[0]["outputPrecisions"] == "FP32" and fc[0]["runtimePrecision"] == "U8"
    assert [int(r["execOrder"]) for r in info] == list(range(len(info)))
    # every graph node that computes is named by exactly one step
    named = [n for r in info for n in r["originalLayersNames"].split(",") if n]
    assert len(named) == len(set(named))
    # the edges of the executed graph: the entry kernel reads graph input 0, everything else reads earlier steps; a
    # bottleneck tail reads its 3 x 3 layer's input and the block input (the residual); every step but the Result is read
    src = [plan.step_sources(i) for i in range(len(info))]
    assert src[0] == [-1] and all(s and all(-1 <= v < i for v in s) for i, s in enumerate(src))
    assert all(len(src[i]) == 2 for i, r in enumerate(info) if r["layerType"] == "Convolution,Convolution")
    assert info[-1]["layerType"] == "Result" and set(range(len(info) - 1)) == {v for s in src for v in s if v >= 0}
    assert plan.step_rt_info(1, "outputDims") == "1,64,112,112"
    # the vector work of a step's f32 chain (results x instructions of its epilogue) and the chain's flag word: the stem
    # is bias + FakeQuantize from 0 with the two-operation division, 6.25 instructions for each of 64 x 112 x 112 results
    assert int(plan.step_rt_info(1, "epilogueFlags")) & ~(1 << 14) == 338433
    assert int(plan.step_rt_info(1, "valuOps")) == int(6.25 * 64 * 112 * 112)
    assert int(plan.step_rt_info(0, "valuOps")) == 0 and int(plan.step_rt_info(0, "epilogueFlags")) == 0
    from dldt_amd.layers import attainable, floors
    steps = [dict(s, valu_ops=int(plan.step_rt_info(i, "valuOps")), ms=1e-3) for i, s in enumerate(plan.steps)]
    f = floors(steps[1])
    assert f["mfma_us"] == pytest.approx(2 * steps[1]["macs"] / 5e15 * 1e6) and f["valu_us"] == pytest.approx(5017600 / 39.3216e12 * 1e6)
    assert f["attainable_us"] == max(f["mfma_us"], f["valu_us"], f["hbm_us"]) and f["bound"] in ("mfma", "valu", "hbm")
    a = attainable(steps)
    assert a["measured_ms"] == pytest.approx(1e-3 * len(steps)) and 0 < a["frac"] and sum(a["bounds"].values()) == len(steps)
    with pytest.raises(HipieError) as e:
        plan.step_rt_info(0, "execTimeMcs")
    assert e.value.status == -5
    with pytest.raises(HipieError) as e:
        plan.step_rt_info(len(plan.steps), "layerType")
    assert e.value.status == -6


def test_concat_shape_inference_and_planner_limits():
    """Concat infers its shape like op::v0::Concat (negative axis included), refuses mismatched inputs when the graph
    is described, and the planner takes it on 4-D tensors (bytes or f32), along any axis"""
    from dldt_amd import HipieError, builders
    from dldt_amd.graph import Graph
    from dldt_amd.tensor import U8
    g = Graph()
    a = g.parameter("a", (2, 3, 5, 5))
    b = g.parameter("b", (2, 4, 5, 5))
    c = g.concat([a, b], axis=-3)                   # the channel axis, counted from the end
    with pytest.raises(HipieError) as e:
        g.concat([a, b], axis=2)                    # dimension 1 differs
    assert e.value.status == -4
    with pytest.raises(HipieError):
        g.concat([a, b], axis=4)
    g.result(c, "c")
    with pytest.raises(HipieError) as e:            # f32 branches: LPT would not have left the Concat there
        g.compile(-1)
    assert e.value.status == -2 and "Concat" in str(e.value)
    g2, _, meta = builders.concat_net()
    plan = g2.compile(-1)
    assert [s["type"] for s in plan.steps].count("Concat") == 1
    assert tuple(plan.outputs[0]["shape"]) == (2, 24 + 40 + 16, 18, 18)
    sup = g2.query()
    assert all(sup)
    # along the rows: the output takes the sum of the inputs' heights
    net = builders.QuantizedNet()
    q = net.input("data", (2, 8, 5, 6), 1.0)
    tall = net.g.concat([q["node"], q["node"], q["node"]], axis=2)
    net.g.result(net.dequantize(dict(node=tall, scale=q["scale"])), "tall")
    plan = net.g.compile(-1)
    assert [s["type"] for s in plan.steps].count("Concat") == 1 and tuple(plan.outputs[0]["shape"]) == (2, 8, 15, 6)


def test_one_spatial_dimension_is_described_and_planned():
    """[N, C, W] convolutions and pools: one attribute per spatial dimension, shapes inferred like the reference's
    (infer_forward_conv_output_shape), planned as [N, C, 1, W] with the plan's inputs and outputs in the described rank;
    three spatial dimensions: f32 convolutions only"""
    from dldt_amd import HipieError, builders
    from dldt_amd.graph import Graph, Plan
    net = builders.QuantizedNet()
    g = net.g
    rng = np.random.default_rng(3)
    a0 = net.input("data", (2, 8, 40), 1.0)
    w = rng.standard_normal((16, 8, 5), dtype=np.float32) * np.float32(0.1)
    a1 = net.conv(a0, w, np.zeros(16, np.float32), 2.0, strides=(2,), pads=(1,), dilations=(2,))
    assert g.nodes[a1["node"]]["op"] == "FakeQuantize"
    a2 = net.max_pool(a1, (3,), (2,), (1,))
    g.result(net.dequantize(a2), "out")
    plan = g.compile(-1)
    # (40 + 2 - (2 * 4 + 1)) / 2 + 1 = 17 columns, then (17 + 2 - 3) / 2 + 1 = 9
    assert tuple(plan.outputs[0]["shape"]) == (2, 16, 9) and tuple(plan.inputs[0]["shape"]) == (2, 8, 40)
    assert [s["type"] for s in plan.steps] == ["FakeQuantize", "Convolution", "MaxPool", "Result"]
    assert plan.step_rt_info(1, "runtimePrecision") == "U8" and all(g.query())
    blob = plan.export()
    back = Plan.load(blob, -1)
    assert tuple(back.outputs[0]["shape"]) == (2, 16, 9)
    # three spatial dimensions: convolutions with f32 weights are planned (values held as [N, C, D * H, W]), quantized
    # ones are reported unsupported, pools are refused where they are described
    g5 = Graph()
    x5 = g5.parameter("x", (1, 4, 6, 5, 7))
    y5 = g5.convolution(x5, g5.constant(np.ones((3, 4, 3, 1, 2), np.float32)), (2, 1, 1), (1, 1, 1), (1, 0, 0), (1, 0, 1))
    g5.result(y5, "y")
    plan = g5.compile(-1)
    assert tuple(plan.outputs[0]["shape"]) == (1, 3, 3, 5, 7) and plan.steps[0]["type"] == "Convolution"
    assert plan.steps[0]["macs"] == 3 * 3 * 5 * 7 * 4 * 3 * 1 * 2
    with pytest.raises(HipieError) as e:
        g5.max_pool(x5, (1, 1, 1), (1, 1, 1), (0, 0, 0), (0, 0, 0))
    assert e.value.status == -2
    from dldt_amd.tensor import I8, U8
    q5 = Graph()
    xq = q5.fake_quantize(q5.parameter("x", (1, 4, 6, 5, 7)), np.float32(0), np.float32(2.55), np.float32(0), np.float32(255), 256, U8)
    q5.result(q5.convolution(q5.convert(xq, 10), q5.constant(np.ones((3, 4, 1, 1, 1), np.int8), I8), (1, 1, 1), (1, 1, 1), (0, 0, 0), (0, 0, 0)), "y")
    with pytest.raises(HipieError) as e:
        q5.compile(-1)
    assert e.value.status == -2 and "three" in str(e.value)
    assert not all(q5.query())


def test_matmul_zero_point_correction_must_be_integers():
    """the Subtract behind a MatMul with u8 activations goes into the integer accumulators: a constant that is not
    integer-valued (it is zero point x column sums of i8 weights) is refused.  A MatMul between two u8 activations is
    planned (level 0 standing for 0.0 on both sides) when its reduction length is a multiple of 64"""
    from dldt_amd import HipieError, builders
    from dldt_amd.graph import Graph
    from dldt_amd.tensor import I8, U8
    plan = builders.matmul_zero_point_net()[0].compile(-1)
    assert [s["type"] for s in plan.steps].count("MatMul") == 2

    def net(corr, between_activations=False, hidden=32):
        g = Graph()
        x = g.parameter("x", (2, 16, hidden))
        q = g.fake_quantize(x, -1.0, 2.0, 0.0, 255.0, 256, U8)
        if between_activations:
            y = g.matmul(q, q, False, True)
        else:
            w = g.constant(np.ones((48, 32), np.int8), I8)
            y = g.subtract(g.matmul(q, w, False, True), g.constant(np.full(48, corr, np.float32)))
        g.result(g.multiply(y, g.constant(np.float32(0.01).reshape(()))), "y")
        return g
    net(32.0 * 85).compile(-1)
    with pytest.raises(HipieError) as e:
        net(2720.5).compile(-1)
    assert e.value.status == -2 and "integer" in str(e.value)
    with pytest.raises(HipieError) as e:
        net(0.0, between_activations=True).compile(-1)
    assert e.value.status == -2 and "multiple of 64" in str(e.value)
    plan = net(0.0, between_activations=True, hidden=64).compile(-1)
    assert [s["type"] for s in plan.steps].count("MatMul") == 1


def test_matmul_between_activations_descriptor_and_workspace():
    """hipie_matmul_create on the host (device -1): operand types, zero points as levels of a u8 operand only, and the
    workspace a u8 operand asks for - one i32 per padded output column (u8 left operand: sums over the right operand's
    rows) plus one per output row rounded up to four (u8 right operand: sums over the left operand's rows), per batch
    element"""
    import ctypes
    from dldt_amd import HipieError, lib
    from dldt_amd.ops import BatchedMatMul
    from dldt_amd.tensor import I8, U8B, F32

    def size(mm, m, batch, outer):
        need = ctypes.c_size_t(12345)
        st = lib().hipie_matmul_workspace_size(mm._h, ctypes.c_int32(m), ctypes.c_int32(batch), ctypes.c_int32(outer),
                                               ctypes.byref(need))
        assert st == 0
        return need.value

    assert size(BatchedMatMul(64, 200, device=-1), 100, 3, 2) == 0
    assert size(BatchedMatMul(64, 200, device=-1, a_dtype=U8B, a_zero_point=7), 100, 3, 2) == 6 * 256 * 4
    assert size(BatchedMatMul(64, 200, device=-1, b_dtype=U8B), 101, 3, 2) == 6 * 104 * 4
    assert size(BatchedMatMul(128, 64, device=-1, a_dtype=U8B, b_dtype=U8B, b_zero_point=255), 7, 5, 1) == 5 * (128 + 8) * 4
    for bad in (dict(a_dtype=F32), dict(b_dtype=F32), dict(a_zero_point=1), dict(b_zero_point=1),
                dict(a_dtype=U8B, a_zero_point=-1), dict(b_dtype=U8B, b_zero_point=256)):
        with pytest.raises(HipieError):
            BatchedMatMul(64, 64, device=-1, **bad)
    with pytest.raises(HipieError):
        BatchedMatMul(96, 64, device=-1)            # the reduction length is a multiple of 64


def test_unquantized_layers_are_planned_in_f32():
    """a convolution with f32 weights (no FakeQuantize in front of it) and a FakeQuantize that keeps its f32 result are
    planned as f32 steps, not refused: QueryNetwork takes every node, the exec graph reports FP32 for them and the
    integer type for the quantized layer behind them"""
    from dldt_amd.graph import Graph
    from dldt_amd.tensor import I8, U8
    g = Graph()
    x = g.parameter("x", (1, 3, 8, 8))
    y = g.relu(g.add(g.convolution(x, g.constant(np.ones((16, 3, 3, 3), np.float32)), pads_begin=(1, 1), pads_end=(1, 1)),
                     g.constant(np.zeros((1, 16, 1, 1), np.float32))))
    f = g.fake_quantize(y, -1.0, 1.0, -1.0, 1.0, 256)                        # f32 result
    q = g.fake_quantize(f, 0.0, 2.55, 0.0, 255.0, 256, out_dtype=U8)
    out = g.multiply(g.convolution(q, g.constant(np.ones((16, 16, 1, 1), np.int8), I8)), g.constant(np.float32(0.01).reshape(1, 1, 1, 1)))
    g.result(out, "y")
    assert all(g.query())
    plan = g.compile(-1, config={"HIP_TUNE": "NO"})
    rows = [(plan.steps[i]["type"], plan.step_rt_info(i, "runtimePrecision")) for i in range(len(plan.steps))]
    assert rows[0] == ("Convolution", "FP32") and ("FakeQuantize", "FP32") in rows and ("Convolution", "U8") in rows, rows
    assert plan.steps[0]["macs"] == 16 * 8 * 8 * 27
