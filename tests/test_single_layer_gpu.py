"""The single-layer lists a plugin instantiates for itself, with the shapes and attribute grids of the template plugin's
(docs/template_plugin/tests/functional/shared_tests_instances/single_layer_tests/{convolution,softmax}.cpp): one layer
between a graph input and a result, f32, compared with the reference kernels' restatement.  Convolutions bit for bit
(reference::convolution<float>'s order of summation); Softmax to rounding (exp is the device's).  The lists' FP16
network precision is the plugin's ConvertPrecision pass in front of the same f32 kernels and has no counterpart at this
boundary."""
import itertools

import numpy as np
import pytest

from interp import evaluate

pytestmark = pytest.mark.gpu


def _run(g, feeds):
    plan = g.compile()
    req = plan.create_request()
    outs = req.infer(*[feeds[i["name"]] for i in plan.inputs])
    return plan, dict(zip([o["name"] for o in plan.outputs], outs))


def _conv_case(orc, rng, shape, kernel, strides, pads_begin, pads_end, dilations, oc):
    from dldt_amd.graph import Graph
    g = Graph()
    x = rng.uniform(-2, 2, shape).astype(np.float32)
    w = rng.standard_normal((oc, shape[1]) + tuple(kernel)).astype(np.float32)
    p = g.parameter("data", shape)
    g.result(g.convolution(p, g.constant(w), strides, dilations, pads_begin, pads_end), "out")
    want, _ = evaluate(orc, g.nodes, {"data": x})
    plan, got = _run(g, {"data": x})
    what = "kernel %s strides %s pads %s %s dilations %s oc %d" % (kernel, strides, pads_begin, pads_end, dilations, oc)
    assert got["out"].shape == want["out"].shape and tuple(plan.outputs[0]["shape"]) == want["out"].shape, what
    np.testing.assert_array_equal(got["out"].view(np.uint32), want["out"].view(np.uint32), err_msg=what)
    assert [s["type"] for s in plan.steps] == ["Convolution", "Result"] and plan.step_rt_info(0, "runtimePrecision") == "FP32"
    return want["out"].size


@pytest.mark.parametrize("kernel", [(3, 3), (3, 5)])
def test_convolution_2d(orc, kernel):
    """Convolution2D_ExplicitPadding and Convolution2D_AutoPadValid: input [1, 3, 30, 30]"""
    rng = np.random.default_rng(sum(kernel))
    cases = 0
    for strides, pb, pe, dil, oc in itertools.product([(1, 1), (1, 3)], [(0, 0), (0, 3)], [(0, 0), (0, 3)], [(1, 1), (3, 1)], [1, 5]):
        cases += _conv_case(orc, rng, (1, 3, 30, 30), kernel, strides, pb, pe, dil, oc) > 0
    assert cases == 32          # (PadType::VALID is the subset with pads (0, 0), (0, 0))


@pytest.mark.parametrize("kernel", [(3, 3, 3), (3, 5, 3)])
def test_convolution_3d(orc, kernel):
    """smoke_Convolution3D_ExplicitPadding and nightly_Convolution3D_AutoPadValid: input [1, 3, 10, 10, 10], 5 filters"""
    rng = np.random.default_rng(sum(kernel))
    cases = 0
    for strides, pb, pe, dil in itertools.product([(1, 1, 1), (1, 2, 1)], [(0, 0, 0), (0, 2, 0)], [(0, 0, 0), (0, 2, 0)], [(1, 1, 1), (1, 2, 1)]):
        cases += _conv_case(orc, rng, (1, 3, 10, 10, 10), kernel, strides, pb, pe, dil, 5) > 0
    assert cases == 16


def test_convolution_3d_along_the_depth(orc):
    """beyond the list: stride, dilation and unequal padding along the depth axis itself, a batch, groups"""
    from dldt_amd.graph import Graph
    rng = np.random.default_rng(333)
    _conv_case(orc, rng, (2, 4, 9, 7, 6), (3, 2, 3), (2, 1, 2), (1, 0, 2), (2, 1, 0), (2, 1, 1), 6)
    _conv_case(orc, rng, (1, 2, 5, 5, 5), (5, 5, 5), (1, 1, 1), (2, 2, 2), (2, 2, 2), (1, 1, 1), 3)
    g = Graph()
    x = rng.uniform(-1, 1, (2, 6, 5, 6, 7)).astype(np.float32)
    w = rng.standard_normal((3, 4, 2, 2, 3, 3)).astype(np.float32)          # [G, OC / G, IC / G, KD, KH, KW]
    b = rng.standard_normal((1, 12, 1, 1, 1)).astype(np.float32)
    p = g.parameter("data", x.shape)
    y = g.relu(g.add(g.convolution(p, g.constant(w), (1, 1, 1), (1, 1, 1), (1, 1, 1), (0, 1, 1), grouped=True), g.constant(b)))
    g.result(y, "out")
    want, _ = evaluate(orc, g.nodes, {"data": x})
    plan, got = _run(g, {"data": x})
    assert got["out"].shape == (2, 12, 5, 6, 7) and [s["type"] for s in plan.steps][0] == "GroupConvolution"
    np.testing.assert_array_equal(got["out"].view(np.uint32), want["out"].view(np.uint32))


@pytest.mark.parametrize("shape", [(1, 100), (100, 1), (10, 10), (1, 100, 1, 1), (1, 3, 4, 3), (2, 3, 4, 5)])
def test_softmax(orc, shape):
    """smoke_SoftMax2D (axes 0, 1) and smoke_SoftMax4D (axes 0 .. 3)"""
    from dldt_amd.graph import Graph
    rng = np.random.default_rng(len(shape) + shape[0])
    for axis in range(len(shape)):
        g = Graph()
        x = (rng.standard_normal(shape) * 3).astype(np.float32)
        g.result(g.softmax(g.parameter("data", shape), axis), "out")
        want, _ = evaluate(orc, g.nodes, {"data": x})
        plan, got = _run(g, {"data": x})
        assert [s["type"] for s in plan.steps] == ["Softmax", "Result"]
        np.testing.assert_allclose(got["out"], want["out"], rtol=3e-6, atol=1e-9, err_msg="axis %d" % axis)
        np.testing.assert_allclose(got["out"].sum(axis), 1.0, rtol=1e-6)


@pytest.mark.parametrize("shape,target", [((30, 30, 30, 30), (30, 30, 30, 30)), ((10, 10, 10, 10), (10, 10, 100))])
def test_reshape(orc, shape, target):
    """smoke_ReshapeCheckDynBatch, smoke_ReshapeCheck and smoke_ReshapeCheckNegative ({10, 0, 100} and {10, -1, 100}
    both resolve to [10, 10, 100] before a plugin sees them): the same bytes under other dimensions"""
    from dldt_amd.graph import Graph
    g = Graph()
    x = np.random.default_rng(len(target)).standard_normal(shape).astype(np.float32)
    g.result(g.reshape(g.parameter("data", shape), target), "out")
    want, _ = evaluate(orc, g.nodes, {"data": x})
    plan, got = _run(g, {"data": x})
    assert got["out"].shape == tuple(target)
    np.testing.assert_array_equal(got["out"].view(np.uint32), want["out"].view(np.uint32))


@pytest.mark.parametrize("axis", [0, 1, 2, 3])
def test_split(orc, axis):
    """smoke_NumSplitsCheck: [30, 30, 30, 30] into 1, 2, 3, 5, 6, 10 and 30 equal parts along every axis, every part a
    result"""
    from dldt_amd.graph import Graph
    x = np.random.default_rng(axis).standard_normal((30, 30, 30, 30)).astype(np.float32)
    for parts in (1, 2, 3, 5, 6, 10, 30):
        g = Graph()
        p = g.parameter("data", x.shape)
        for k, piece in enumerate(g.split(p, axis, parts, 30)):
            g.result(piece, "out%d" % k)
        plan, got = _run(g, {"data": x})
        assert len(got) == parts
        for k, piece in enumerate(np.split(x, parts, axis)):
            np.testing.assert_array_equal(got["out%d" % k].view(np.uint32), piece.view(np.uint32), err_msg="%d parts, part %d" % (parts, k))
