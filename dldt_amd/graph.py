"""Graph-level binding: describes a post-LPT function node by node through the C ABI
(include/hipie.h section 2), compiles it and runs infer requests.

Every node is also recorded in ``Graph.nodes`` (plain dicts with numpy constants) so that a
checker can evaluate the very same graph with reference kernels.
"""
import ctypes

import numpy as np

from ._lib import check, lib
from .tensor import F32, I8, I32, U8, U8B, hipie_tensor

OP_ADD, OP_MULTIPLY, OP_SUBTRACT, OP_PRELU = 6, 7, 8, 23
OP_SIGMOID, OP_HSWISH, OP_HSIGMOID, OP_SWISH = 24, 25, 26, 27
_NP = {F32: np.float32, U8: np.uint8, I8: np.int8, I32: np.int32}


def _i64(v):
    return (ctypes.c_int64 * max(len(v), 1))(*[int(x) for x in v])


class Graph:
    def __init__(self):
        self._h = ctypes.c_void_p()
        check(lib().hipie_graph_create(ctypes.byref(self._h)))
        self.nodes = []
        self.params, self.results = [], []

    def __del__(self):
        if getattr(self, "_h", None):
            lib().hipie_graph_destroy(self._h)
            self._h = None

    def _rec(self, id_, op, inputs, dtype, **attrs):
        assert id_ == len(self.nodes), (id_, len(self.nodes))
        self.nodes.append(dict(op=op, inputs=list(inputs), dtype=dtype, **attrs))
        return id_

    def parameter(self, name, shape, dtype=F32):
        i = ctypes.c_int()
        check(lib().hipie_graph_parameter(self._h, name.encode(), dtype, _i64(shape), len(shape), ctypes.byref(i)))
        self.params.append(i.value)
        return self._rec(i.value, "Parameter", [], dtype, name=name, shape=tuple(shape))

    def constant(self, value, dtype=F32):
        a = np.ascontiguousarray(value, _NP[dtype])
        i = ctypes.c_int()
        check(lib().hipie_graph_constant(self._h, dtype, _i64(a.shape), a.ndim, a.ctypes.data_as(ctypes.c_void_p),
                                         ctypes.byref(i)))
        return self._rec(i.value, "Constant", [], dtype, value=a)

    def _const_if_needed(self, v):
        return v if isinstance(v, int) and not isinstance(v, bool) else self.constant(np.asarray(v, np.float32))

    def fake_quantize(self, x, in_low, in_high, out_low, out_high, levels, out_dtype=F32):
        b = [self.constant(np.asarray(v, np.float32)) for v in (in_low, in_high, out_low, out_high)]
        i = ctypes.c_int()
        check(lib().hipie_graph_fake_quantize(self._h, x, *b, ctypes.c_int64(levels), out_dtype, ctypes.byref(i)))
        return self._rec(i.value, "FakeQuantize", [x] + b, out_dtype, levels=levels)

    def convolution(self, x, w, strides=(1, 1), dilations=(1, 1), pads_begin=(0, 0), pads_end=(0, 0), grouped=False):
        i = ctypes.c_int()
        fn = lib().hipie_graph_group_convolution if grouped else lib().hipie_graph_convolution
        check(fn(self._h, x, w, _i64(strides), _i64(dilations), _i64(pads_begin), _i64(pads_end), ctypes.byref(i)))
        return self._rec(i.value, "GroupConvolution" if grouped else "Convolution", [x, w], F32,
                         strides=tuple(strides), dilations=tuple(dilations), pads_begin=tuple(pads_begin),
                         pads_end=tuple(pads_end))

    def matmul(self, a, b, transpose_a=False, transpose_b=False):
        i = ctypes.c_int()
        check(lib().hipie_graph_matmul(self._h, a, b, int(transpose_a), int(transpose_b), ctypes.byref(i)))
        return self._rec(i.value, "MatMul", [a, b], F32, ta=transpose_a, tb=transpose_b)

    def _eltwise(self, kind, name, a, b):
        i = ctypes.c_int()
        check(lib().hipie_graph_eltwise(self._h, kind, a, b, ctypes.byref(i)))
        return self._rec(i.value, name, [a, b], F32)

    def add(self, a, b):
        return self._eltwise(OP_ADD, "Add", a, b)

    def multiply(self, a, b):
        return self._eltwise(OP_MULTIPLY, "Multiply", a, b)

    def subtract(self, a, b):
        return self._eltwise(OP_SUBTRACT, "Subtract", a, b)

    def prelu(self, x, slope):
        return self._eltwise(OP_PRELU, "PRelu", x, slope)

    def _activation(self, kind, name, x, beta=1.0):
        i = ctypes.c_int()
        check(lib().hipie_graph_activation(self._h, kind, x, ctypes.c_float(beta), ctypes.byref(i)))
        return self._rec(i.value, name, [x], F32, beta=float(np.float32(beta)))

    def sigmoid(self, x):
        return self._activation(OP_SIGMOID, "Sigmoid", x)

    def hswish(self, x):
        return self._activation(OP_HSWISH, "HSwish", x)

    def hsigmoid(self, x):
        return self._activation(OP_HSIGMOID, "HSigmoid", x)

    def swish(self, x, beta=1.0):
        return self._activation(OP_SWISH, "Swish", x, beta)

    def relu(self, x):
        i = ctypes.c_int()
        check(lib().hipie_graph_relu(self._h, x, ctypes.byref(i)))
        return self._rec(i.value, "Relu", [x], self.nodes[x]["dtype"])

    def clamp(self, x, lo, hi):
        i = ctypes.c_int()
        check(lib().hipie_graph_clamp(self._h, x, ctypes.c_float(lo), ctypes.c_float(hi), ctypes.byref(i)))
        return self._rec(i.value, "Clamp", [x], self.nodes[x]["dtype"], lo=float(lo), hi=float(hi))

    def convert(self, x, dtype):
        i = ctypes.c_int()
        check(lib().hipie_graph_convert(self._h, x, dtype, ctypes.byref(i)))
        return self._rec(i.value, "Convert", [x], dtype)

    def max_pool(self, x, kernel, strides, pads_begin=(0, 0), pads_end=(0, 0), ceil_mode=False):
        i = ctypes.c_int()
        check(lib().hipie_graph_max_pool(self._h, x, _i64(kernel), _i64(strides), _i64(pads_begin), _i64(pads_end),
                                         int(ceil_mode), ctypes.byref(i)))
        return self._rec(i.value, "MaxPool", [x], self.nodes[x]["dtype"], kernel=tuple(kernel),
                         strides=tuple(strides), pads_begin=tuple(pads_begin), pads_end=tuple(pads_end),
                         ceil_mode=ceil_mode)

    def avg_pool(self, x, kernel, strides, pads_begin=(0, 0), pads_end=(0, 0), exclude_pad=True, ceil_mode=False,
                 out_dtype=F32):
        i = ctypes.c_int()
        check(lib().hipie_graph_avg_pool(self._h, x, _i64(kernel), _i64(strides), _i64(pads_begin), _i64(pads_end),
                                         int(exclude_pad), int(ceil_mode), out_dtype, ctypes.byref(i)))
        return self._rec(i.value, "AvgPool", [x], out_dtype, kernel=tuple(kernel), strides=tuple(strides),
                         pads_begin=tuple(pads_begin), pads_end=tuple(pads_end), exclude_pad=exclude_pad,
                         ceil_mode=ceil_mode)

    def reshape(self, x, shape):
        i = ctypes.c_int()
        check(lib().hipie_graph_reshape(self._h, x, _i64(shape), len(shape), ctypes.byref(i)))
        return self._rec(i.value, "Reshape", [x], self.nodes[x]["dtype"], shape=tuple(shape))

    def softmax(self, x, axis=-1):
        i = ctypes.c_int()
        check(lib().hipie_graph_softmax(self._h, x, ctypes.c_int64(axis), ctypes.byref(i)))
        return self._rec(i.value, "Softmax", [x], F32, axis=axis)

    def mvn(self, x, axes=(-1,), normalize_variance=True, eps=1e-5, eps_inside_sqrt=True):
        i = ctypes.c_int()
        check(lib().hipie_graph_mvn(self._h, x, _i64(axes), len(axes), int(normalize_variance), ctypes.c_float(eps),
                                    int(eps_inside_sqrt), ctypes.byref(i)))
        return self._rec(i.value, "MVN", [x], F32, axes=tuple(axes), normalize_variance=normalize_variance,
                         eps=float(eps), eps_inside_sqrt=eps_inside_sqrt)

    def gelu(self, x):
        i = ctypes.c_int()
        check(lib().hipie_graph_gelu(self._h, x, ctypes.byref(i)))
        return self._rec(i.value, "Gelu", [x], F32)

    def transpose(self, x, order):
        i = ctypes.c_int()
        check(lib().hipie_graph_transpose(self._h, x, _i64(order), len(order), ctypes.byref(i)))
        return self._rec(i.value, "Transpose", [x], self.nodes[x]["dtype"], order=tuple(order))

    def gather(self, data, indices, axis=0):
        i = ctypes.c_int()
        check(lib().hipie_graph_gather(self._h, data, indices, ctypes.c_int64(axis), ctypes.byref(i)))
        return self._rec(i.value, "Gather", [data, indices], self.nodes[data]["dtype"], axis=axis)

    def concat(self, inputs, axis=1):
        i = ctypes.c_int()
        ids = (ctypes.c_int * len(inputs))(*inputs)
        check(lib().hipie_graph_concat(self._h, ids, len(inputs), ctypes.c_int64(axis), ctypes.byref(i)))
        return self._rec(i.value, "Concat", list(inputs), self.nodes[inputs[0]]["dtype"], axis=axis)

    def slice(self, x, axis, begin, end):
        i = ctypes.c_int()
        check(lib().hipie_graph_slice(self._h, x, ctypes.c_int64(axis), ctypes.c_int64(begin), ctypes.c_int64(end), ctypes.byref(i)))
        return self._rec(i.value, "Slice", [x], self.nodes[x]["dtype"], axis=axis, begin=begin, end=end)

    def split(self, x, axis, parts, length):
        """op::v1::Split of an axis of `length` elements into `parts` equal outputs, one Slice each"""
        assert length % parts == 0
        step = length // parts
        return [self.slice(x, axis, k * step, (k + 1) * step) for k in range(parts)]

    def result(self, x, name):
        check(lib().hipie_graph_result(self._h, x, name.encode()))
        self.results.append(len(self.nodes))
        return self._rec(len(self.nodes), "Result", [x], self.nodes[x]["dtype"], name=name)

    def set_name(self, id_, name):
        check(lib().hipie_graph_set_name(self._h, id_, name.encode()))
        self.nodes[id_]["name"] = name

    def compile(self, device=0, config=None):
        """config: {key: value} as for Core::LoadNetwork (hipie_compile_opts); None = the process defaults"""
        return Plan(self, device, config=config)

    def query(self):
        """QueryNetwork: list of booleans, one per node added so far (Result nodes included)"""
        n = len(self.nodes)
        flags = (ctypes.c_int * max(n, 1))()
        bad = ctypes.c_int()
        check(lib().hipie_query(self._h, flags, n, ctypes.byref(bad)))
        return [bool(flags[i]) for i in range(n)]


class Plan:
    """ExecutableNetwork analogue: fused steps + arena layout + uploaded constants."""

    def __init__(self, graph, device=0, _handle=None, config=None):
        self._h = ctypes.c_void_p()
        if _handle is not None:
            self._h = _handle
        elif config is None:
            check(lib().hipie_compile(graph._h, device, ctypes.byref(self._h)))
        else:
            items = [(str(k).encode(), str(v).encode()) for k, v in config.items()]
            keys = (ctypes.c_char_p * max(len(items), 1))(*[k for k, _ in items])
            vals = (ctypes.c_char_p * max(len(items), 1))(*[v for _, v in items])
            check(lib().hipie_compile_opts(graph._h, device, keys, vals, len(items), ctypes.byref(self._h)))
        self.device = device
        L = lib()
        L.hipie_plan_arena_bytes.restype = ctypes.c_int64
        self.inputs = [self._io(0, i) for i in range(L.hipie_plan_num_inputs(self._h))]
        self.outputs = [self._io(1, i) for i in range(L.hipie_plan_num_outputs(self._h))]
        self.arena_bytes = L.hipie_plan_arena_bytes(self._h)
        self.steps = []
        for i in range(L.hipie_plan_num_steps(self._h)):
            name, typ = ctypes.create_string_buffer(256), ctypes.create_string_buffer(64)
            macs, byts = ctypes.c_int64(), ctypes.c_int64()
            check(L.hipie_plan_step_info(self._h, i, name, 256, typ, 64, ctypes.byref(macs), ctypes.byref(byts)))
            var = ctypes.c_int()
            check(L.hipie_plan_step_variant(self._h, i, ctypes.byref(var)))
            self.steps.append(dict(name=name.value.decode(errors="replace"), type=typ.value.decode(errors="replace"), macs=macs.value,
                                   bytes=byts.value, variant=var.value))

    def step_sources(self, index):
        """hipie_plan_step_sources: where the step's operands come from (step indices; -(1 + k) = graph input k)"""
        n = ctypes.c_int()
        check(lib().hipie_plan_step_sources(self._h, index, None, 0, ctypes.byref(n)))
        buf = (ctypes.c_int * max(n.value, 1))()
        check(lib().hipie_plan_step_sources(self._h, index, buf, n.value, ctypes.byref(n)))
        return [buf[i] for i in range(n.value)]

    def step_rt_info(self, index, key):
        """an exec-graph attribute of one executed step (originalLayersNames, layerType, runtimePrecision,
        outputPrecisions, outputLayouts, execOrder, primitiveType)"""
        buf = ctypes.create_string_buffer(8192)
        check(lib().hipie_plan_step_rt_info(self._h, index, key.encode(), buf, ctypes.c_size_t(len(buf))))
        return buf.value.decode(errors="replace")

    def export(self):
        """ExecutableNetwork::Export: the plan as bytes (graph description, constants, kernel choices)."""
        size = ctypes.c_size_t()
        check(lib().hipie_plan_export(self._h, None, ctypes.c_size_t(0), ctypes.byref(size)))
        buf = ctypes.create_string_buffer(size.value)
        check(lib().hipie_plan_export(self._h, buf, ctypes.c_size_t(size.value), ctypes.byref(size)))
        return buf.raw[:size.value]

    @classmethod
    def load(cls, blob, device=0):
        """Plugin::ImportNetwork: a plan from exported bytes; runs the kernels the exported plan ran."""
        h = ctypes.c_void_p()
        check(lib().hipie_plan_import(blob, ctypes.c_size_t(len(blob)), device, ctypes.byref(h)))
        return cls(None, device, _handle=h)

    def metric(self, name):
        buf = ctypes.create_string_buffer(1024)
        check(lib().hipie_plan_get_metric(self._h, name.encode(), buf, ctypes.c_size_t(1024)))
        return buf.value.decode()

    def config(self, key):
        buf = ctypes.create_string_buffer(1024)
        check(lib().hipie_plan_get_config(self._h, key.encode(), buf, ctypes.c_size_t(1024)))
        return buf.value.decode()

    def _io(self, is_out, idx):
        name = ctypes.create_string_buffer(256)
        dt, rank = ctypes.c_int(), ctypes.c_int()
        dims = (ctypes.c_int64 * 8)()
        check(lib().hipie_plan_io_desc(self._h, is_out, idx, name, 256, ctypes.byref(dt), dims, ctypes.byref(rank)))
        return dict(name=name.value.decode(errors="replace"), dtype=dt.value, shape=tuple(dims[:rank.value]))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().hipie_plan_destroy(self._h)
            self._h = None

    def create_request(self, perf_count=False):
        """perf_count: True / False, or None for the plan's PERF_COUNT"""
        return Request(self, perf_count)


class PinnedArray:
    """numpy array over page-locked host memory from hipie_host_alloc (`.array`); freed with the object"""

    def __init__(self, shape, dtype):
        self._p = ctypes.c_void_p()
        n = int(np.prod(shape)) * np.dtype(dtype).itemsize
        check(lib().hipie_host_alloc(ctypes.c_size_t(n), ctypes.byref(self._p)))
        raw = (ctypes.c_uint8 * max(n, 1)).from_address(self._p.value)
        self.array = np.frombuffer(raw, dtype=dtype, count=int(np.prod(shape))).reshape(shape)

    def __del__(self):
        if getattr(self, "_p", None):
            self.array = None
            lib().hipie_host_free(self._p)
            self._p = None


class Request:
    """InferRequest analogue: own stream and activation arena."""

    def __init__(self, plan, perf_count=False):
        self.plan = plan
        self._h = ctypes.c_void_p()
        check(lib().hipie_request_create(plan._h, -1 if perf_count is None else int(perf_count), ctypes.byref(self._h)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().hipie_request_destroy(self._h)
            self._h = None

    def infer(self, *inputs):
        """Host path: numpy NCHW in, numpy out (H2D, kernels, D2H)."""
        ins = [np.ascontiguousarray(a, _NP[d["dtype"]]) for a, d in zip(inputs, self.plan.inputs)]
        for a, d in zip(ins, self.plan.inputs):
            assert a.shape == d["shape"], (a.shape, d["shape"])
        outs = [np.empty(d["shape"], _NP[d["dtype"]]) for d in self.plan.outputs]
        ip = (ctypes.c_void_p * len(ins))(*[a.ctypes.data for a in ins])
        op = (ctypes.c_void_p * len(outs))(*[a.ctypes.data for a in outs])
        check(lib().hipie_request_infer(self._h, ip, op, 0))
        return outs

    def host_buffers(self):
        """page-locked numpy arrays shaped like the plan's inputs and outputs (the request's blobs)"""
        return ([PinnedArray(d["shape"], _NP[d["dtype"]]) for d in self.plan.inputs],
                [PinnedArray(d["shape"], _NP[d["dtype"]]) for d in self.plan.outputs])

    def start(self, ins, outs):
        """StartAsync from host buffers (PinnedArray or numpy): copies and kernels are queued on the
        request's stream; wait() returns when the outputs are complete."""
        arr = lambda b: b.array if isinstance(b, PinnedArray) else b
        ip = (ctypes.c_void_p * len(ins))(*[arr(b).ctypes.data for b in ins])
        op = (ctypes.c_void_p * len(outs))(*[arr(b).ctypes.data for b in outs])
        check(lib().hipie_request_start(self._h, ip, op, 0))

    def wait(self):
        check(lib().hipie_request_wait(self._h))

    def wait_for(self, timeout_ms):
        """Wait(ms): -1 blocks, 0 asks only; raises HipieError with status -9 (RESULT_NOT_READY) while it runs"""
        check(lib().hipie_request_wait_for(self._h, ctypes.c_int64(timeout_ms)))

    def cancel(self):
        check(lib().hipie_request_cancel(self._h))

    def device_buffers(self):
        """torch tensors shaped like the plan's inputs and outputs (for resident-in-HBM runs)."""
        import torch
        tdt = {F32: torch.float32, U8: torch.uint8, I32: torch.int32}
        dev = "cuda:%d" % self.plan.device
        ins = [torch.empty(d["shape"], dtype=tdt[d["dtype"]], device=dev) for d in self.plan.inputs]
        outs = [torch.empty(d["shape"], dtype=tdt[d["dtype"]], device=dev) for d in self.plan.outputs]
        return ins, outs

    def _ptrs(self, ins, outs):
        ip = (ctypes.c_void_p * len(ins))(*[t.data_ptr() for t in ins])
        op = (ctypes.c_void_p * len(outs))(*[t.data_ptr() for t in outs])
        return ip, op

    def infer_device(self, ins, outs):
        ip, op = self._ptrs(ins, outs)
        check(lib().hipie_request_infer(self._h, ip, op, 1))

    def enqueue(self, ins, outs):
        ip, op = self._ptrs(ins, outs)
        check(lib().hipie_request_enqueue(self._h, ip, op))

    @property
    def stream(self):
        s = ctypes.c_void_p()
        check(lib().hipie_request_stream(self._h, ctypes.byref(s)))
        return s.value

    def perf(self):
        out = []
        for i, st in enumerate(self.plan.steps):
            ms = ctypes.c_float()
            check(lib().hipie_request_perf(self._h, i, ctypes.byref(ms)))
            out.append(dict(st, ms=ms.value))
        return out

    def matrix(self, node_id):
        """numpy [rows, last dimension] copy of a value of the row-major (transformer) path."""
        v = self.tensor(node_id)              # stored as n = h = 1, w = rows, c = columns
        return np.ascontiguousarray(v[0, :, 0, :].T)

    def tensor(self, node_id, fused_ok=False):
        """numpy NCHW copy of the arena tensor holding graph node `node_id` (u8 levels / f32).  fused_ok: None instead of
        an error for a node whose value never reaches memory (fused away, or kept in LDS between two convolutions
        that run as one kernel)."""
        import torch
        t = hipie_tensor()
        status = lib().hipie_request_tensor(self._h, node_id, ctypes.byref(t))
        if status == -5 and fused_ok:
            return None
        check(status)
        esz = 4 if t.dtype in (F32, I32) else 1
        tdt = {F32: torch.float32, I32: torch.int32}.get(t.dtype, torch.int8)
        # view [n, h, w, c] through the strides
        span = (t.n - 1) * t.stride_n + (t.h - 1) * t.stride_h + (t.w - 1) * t.stride_w + t.c
        flat = torch.empty(span, dtype=tdt)
        check(lib().hipie_memcpy(ctypes.c_void_p(flat.data_ptr()), ctypes.c_void_p(t.data),
                                 ctypes.c_size_t(span * esz), 0))
        v = torch.as_strided(flat, (t.n, t.h, t.w, t.c), (t.stride_n, t.stride_h, t.stride_w, 1)).numpy()
        if t.dtype == U8B:
            v = (v.astype(np.int16) + 128).astype(np.uint8)
        return np.ascontiguousarray(np.transpose(v, (0, 3, 1, 2)))
