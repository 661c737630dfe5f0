"""Evaluates a recorded post-LPT graph (dldt_amd.graph.Graph.nodes) with the oracle's reference
kernels, the way the reference's INTERPRETER backend walks a Function
(ngraph/test/runtime/interpreter/int_executable.cpp:33-154), except that TypeRelaxed integer ops
are evaluated in int32 on widened inputs (the interpreter has no mixed-type evaluator)."""
import numpy as np

F32, U8, I8, I32 = 10, 40, 50, 70
_NP = {F32: np.float32, U8: np.uint8, I8: np.int8, I32: np.int32}


def needed_nodes(nodes, targets, stop=()):
    """ids of the nodes that `targets` depend on, not looking behind the nodes in `stop` (whose values are given)"""
    need, todo = set(), list(targets)
    while todo:
        i = todo.pop()
        if i in need:
            continue
        need.add(i)
        if i not in stop:
            todo.extend(nodes[i]["inputs"])
    return need


def _pool(orc, n, x):
    oshape = orc.pool_out_shape(x.shape, n["kernel"], n["strides"], n["pads_begin"], n["pads_end"], n["ceil_mode"])
    if n["op"] == "MaxPool":
        return orc.max_pool(x, n["kernel"], n["strides"], n["pads_begin"], n["pads_end"], out_shape=oshape)
    # f32 result: TypeRelaxed<AvgPool> over widened levels; u8 / i8 result (precision preserved): the reference's
    # integer instantiation, whose accumulator has the element type (avg_pool.hpp:114-265)
    src = x.astype(np.float32) if n["dtype"] == 10 else x
    return orc.avg_pool(src, n["kernel"], n["strides"], n["pads_begin"], n["pads_end"], not n["exclude_pad"], out_shape=oshape)


def evaluate(orc, nodes, feeds, keep=None, override=None, targets=None):
    """feeds: {parameter name: array}.  Returns ({result name: array}, {node id: array} for `keep`).
    override: {node id: array} continues from these values behind the given nodes (a checker passes the
    device's own result of an op that only has tolerance parity); what the oracle computed for such a
    node from the same inputs is returned in the second dict under ("oracle", node id).
    targets: evaluate only what these nodes need, taking every overridden node as given (its own inputs are
    not evaluated and it gets no ("oracle", id) entry): a slice of a deep graph at full size."""
    val = {}
    results = {}
    override = override or {}
    shadow = {}
    need = needed_nodes(nodes, targets, stop=set(override)) if targets is not None else None
    for i, n in enumerate(nodes):
        if need is not None:
            if i not in need:
                continue
            if i in override:
                val[i] = np.asarray(override[i])
                continue
        op = n["op"]
        x = [val[j] for j in n["inputs"]]
        if op == "Parameter":
            v = np.ascontiguousarray(feeds[n["name"]], _NP[n["dtype"]])
        elif op == "Constant":
            v = n["value"]
        elif op == "FakeQuantize":
            v = orc.fake_quantize(x[0], x[1], x[2], x[3], x[4], n["levels"])
            if n["dtype"] != F32:
                v = v.astype(_NP[n["dtype"]])            # TypeRelaxed output: Convert of the f32 result
        elif op in ("Convolution", "GroupConvolution") and x[1].dtype == np.float32:
            # a layer the transformations left alone: f32 weights, the reference's float instantiation
            v = orc.convolution(x[0].astype(np.float32), x[1], n["strides"], n["dilations"], n["pads_begin"], n["pads_end"],
                                grouped=op == "GroupConvolution")
        elif op in ("Convolution", "GroupConvolution"):
            v = orc.convolution(x[0].astype(np.int32), x[1].astype(np.int32), n["strides"], n["dilations"],
                                n["pads_begin"], n["pads_end"], grouped=op == "GroupConvolution")
            v = v.astype(np.float32)                      # declared f32 holding the integer sum
        elif op == "MatMul" and x[1].dtype == np.float32 and x[0].dtype == np.float32 and nodes[n["inputs"][1]]["op"] == "Constant":
            v = orc.matmul(x[0], x[1], n["ta"], n["tb"])
        elif op == "MatMul":
            v = orc.matmul(x[0].astype(np.int32), x[1].astype(np.int32), n["ta"], n["tb"]).astype(np.float32)
        elif op == "Add":
            v = orc.add(x[0], x[1])
        elif op == "Multiply":
            v = orc.multiply(x[0], x[1])
        elif op == "Subtract":
            v = orc.subtract(x[0], x[1])
        elif op == "PRelu":
            v = orc.prelu(x[0], x[1])
        elif op in ("Sigmoid", "HSwish", "HSigmoid"):
            v = getattr(orc, op.lower())(x[0])
        elif op == "Swish":
            v = orc.swish(x[0], n["beta"])
        elif op == "Relu":
            v = orc.relu(x[0])
        elif op == "Clamp":
            v = orc.clamp(x[0], n["lo"], n["hi"])
        elif op == "Convert":
            v = x[0].astype(_NP[n["dtype"]])
        elif op in ("MaxPool", "AvgPool") and x[0].ndim == 3:
            # one spatial dimension: the same windows over [N, C, 1, W] (the reference's pools walk any number of
            # spatial axes; a unit axis adds no cell to any window)
            lifted = dict(n, kernel=(1, n["kernel"][0]), strides=(1, n["strides"][0]), pads_begin=(0, n["pads_begin"][0]),
                          pads_end=(0, n["pads_end"][0]))
            v = _pool(orc, lifted, x[0][:, :, None, :])[:, :, 0, :]
        elif op in ("MaxPool", "AvgPool"):
            v = _pool(orc, n, x[0])
        elif op == "Reshape":
            v = x[0].reshape(n["shape"])
        elif op == "Gather":
            idx = np.where(x[1] < 0, x[1] + x[0].shape[n["axis"]], x[1])      # gather.hpp:58-59
            v = np.ascontiguousarray(np.take(x[0], idx, axis=n["axis"]))
        elif op == "Transpose":
            v = np.ascontiguousarray(np.transpose(x[0], n["order"]))
        elif op == "Slice":
            # one output of reference::split: the box [begin, end) along the axis, every other axis whole
            box = [slice(None)] * x[0].ndim
            box[n["axis"]] = slice(n["begin"], n["end"])
            v = np.ascontiguousarray(x[0][tuple(box)])
        elif op == "Concat":
            v = np.concatenate(x, axis=n["axis"])             # concat.hpp:17-57: the inputs' elements side by side
        elif op == "Softmax":
            v = orc.softmax(x[0], n["axis"])
        elif op == "MVN":
            assert tuple(a % x[0].ndim for a in n["axes"]) == (x[0].ndim - 1,)
            v = orc.mvn_last_axis(x[0], n["normalize_variance"], n["eps"], n["eps_inside_sqrt"])
        elif op == "Gelu":
            v = orc.gelu_erf(x[0])
        elif op == "Result":
            v = x[0]
            results[n["name"]] = v
        else:
            raise NotImplementedError(op)
        if i in override:
            shadow[i] = v                                 # what the oracle makes of the same inputs
            v = np.asarray(override[i], v.dtype).reshape(v.shape)
        val[i] = v
        # free what is no longer needed (full-size ResNet keeps ~1 GB otherwise)
        if keep is not None:
            for j in n["inputs"]:
                if j not in keep and nodes[j]["op"] != "Constant" and all(j not in m["inputs"] for m in nodes[i + 1:]):
                    val.pop(j, None)
    kept = {k: val[k] for k in (keep or []) if k in val}
    for k, v in shadow.items():
        kept[("oracle", k)] = v
    return results, kept
