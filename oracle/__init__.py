"""TEST INFRASTRUCTURE ONLY: numpy front-end to the CPU checker.

``ops`` is our C restatement of the nGraph reference kernels (``liboracle.so`` built from
``ngraph_ops.c``); ``ref`` is the reference's own header kernels compiled in place
(``_ref/libngraph_ref.so``) or ``None`` when that build is not present.  Both expose the same
methods, so a test can fuzz one against the other.  Only tests, the smoke check and the
benchmark's CPU-baseline leg may import this package; the shipped library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_i64p = ctypes.POINTER(ctypes.c_int64)


def build(with_ref=True):
    """Compile liboracle.so (always) and _ref (only where the reference checkout exists)."""
    subprocess.check_call(["make", "-C", _HERE, "liboracle.so"] + (["ref"] if with_ref else []))


def _shape(s):
    a = (ctypes.c_int64 * max(len(s), 1))(*[int(v) for v in s])
    return a, len(s)


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


_SUFFIX = {np.dtype(np.float32): "f32", np.dtype(np.int32): "i32", np.dtype(np.int64): "i64",
           np.dtype(np.uint8): "u8", np.dtype(np.int8): "i8"}


def conv_out_shape(in_shape, f_shape, strides, dilations, pads_begin, pads_end, grouped=False):
    sp = len(in_shape) - 2
    off = 1 if grouped else 0
    oc = f_shape[0] * f_shape[1] if grouped else f_shape[0]
    out = [in_shape[0], oc]
    for i in range(sp):
        k = f_shape[off + 2 + i]
        padded = in_shape[2 + i] + pads_begin[i] + pads_end[i]
        out.append((padded - (dilations[i] * (k - 1) + 1)) // strides[i] + 1)
    return tuple(out)


def matmul_out_shape(a_shape, b_shape, ta, tb):
    A, B = list(a_shape), list(b_shape)
    if ta and len(A) > 1:
        A[-1], A[-2] = A[-2], A[-1]
    if tb and len(B) > 1:
        B[-1], B[-2] = B[-2], B[-1]
    return tuple(np.matmul(np.empty(A, np.int8), np.empty(B, np.int8)).shape)


class _Ops:
    def __init__(self, path, prefix):
        self.lib = ctypes.CDLL(path)
        self.prefix = prefix
        self.path = path

    def _fn(self, name):
        f = getattr(self.lib, self.prefix + name)
        f.restype = None
        return f

    # ---- FakeQuantize (fake_quantize.hpp) ------------------------------------------------
    def fake_quantize(self, x, il, ih, ol, oh, levels, bcast_axis=-2):
        x = np.ascontiguousarray(x, np.float32)
        bs = [np.ascontiguousarray(b, np.float32) for b in (il, ih, ol, oh)]
        out = np.empty_like(x)
        args = [_ptr(x), *_shape(x.shape)]
        for b in bs:
            args += [_ptr(b), *_shape(b.shape)]
        args += [ctypes.c_int64(int(levels)), ctypes.c_int(bcast_axis), _ptr(out)]
        self._fn("fake_quantize_f32")(*args)
        return out

    # ---- Convolution / GroupConvolution (convolution.hpp, group_convolution.hpp) --------
    def convolution(self, x, f, strides, dilations, pads_begin, pads_end, grouped=False):
        x = np.ascontiguousarray(x)
        f = np.ascontiguousarray(f, x.dtype)
        oshape = conv_out_shape(x.shape, f.shape, strides, dilations, pads_begin, pads_end, grouped)
        out = np.empty(oshape, x.dtype)
        name = "convolution_" + _SUFFIX[x.dtype] + ("_group" if grouped else "")
        xs, rank = _shape(x.shape)
        fs, _ = _shape(f.shape)
        self._fn(name)(_ptr(x), _ptr(f), _ptr(out), xs, fs, ctypes.c_int(rank),
                       _shape(strides)[0], _shape(dilations)[0], _shape(pads_begin)[0],
                       _shape(pads_end)[0])
        return out

    # ---- MatMul (matmul.hpp) --------------------------------------------------------------
    def matmul(self, a, b, ta=False, tb=False):
        a = np.ascontiguousarray(a)
        b = np.ascontiguousarray(b, a.dtype)
        oshape = matmul_out_shape(a.shape, b.shape, ta, tb)
        out = np.empty(oshape, a.dtype)
        name = "matmul_" + _SUFFIX[a.dtype]
        a_s, ar = _shape(a.shape)
        b_s, br = _shape(b.shape)
        if self.prefix == "ref_":
            o_s, orank = _shape(oshape)
            self._fn(name)(_ptr(a), _ptr(b), _ptr(out), a_s, ctypes.c_int(ar), b_s,
                           ctypes.c_int(br), o_s, ctypes.c_int(orank), int(ta), int(tb))
        else:
            self._fn(name)(_ptr(a), _ptr(b), _ptr(out), a_s, ctypes.c_int(ar), b_s,
                           ctypes.c_int(br), int(ta), int(tb))
        return out

    # ---- elementwise (autobroadcast_binop.hpp, relu.hpp, clamp.hpp) ----------------------
    def _binop(self, name, a, b):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        oshape = np.broadcast_shapes(a.shape, b.shape)
        out = np.empty(oshape, np.float32)
        self._fn(name)(_ptr(a), *_shape(a.shape), _ptr(b), *_shape(b.shape), *_shape(oshape),
                       _ptr(out))
        return out

    def add(self, a, b):
        return self._binop("add_f32", a, b)

    def subtract(self, a, b):
        return self._binop("subtract_f32", a, b)

    def multiply(self, a, b):
        return self._binop("multiply_f32", a, b)

    def divide(self, a, b):
        return self._binop("divide_f32", a, b)

    def prelu(self, x, slope):
        x = np.ascontiguousarray(x, np.float32)
        slope = np.ascontiguousarray(slope, np.float32)
        out = np.empty_like(x)
        self._fn("prelu_f32")(_ptr(x), *_shape(x.shape), _ptr(slope), *_shape(slope.shape), _ptr(out))
        return out

    def _unary(self, name, x, *extra):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        self._fn(name)(_ptr(x), *extra, _ptr(out), ctypes.c_int64(x.size))
        return out

    def sigmoid(self, x):
        return self._unary("sigmoid_f32", x)

    def hswish(self, x):
        return self._unary("hswish_f32", x)

    def hsigmoid(self, x):
        return self._unary("hsigmoid_f32", x)

    def swish(self, x, beta=1.0):
        return self._unary("swish_f32", x, ctypes.c_float(beta))

    def relu(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        self._fn("relu_f32")(_ptr(x), _ptr(out), ctypes.c_int64(x.size))
        return out

    def clamp(self, x, mn, mx):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        self._fn("clamp_f32")(_ptr(x), _ptr(out), ctypes.c_float(mn), ctypes.c_float(mx),
                              ctypes.c_int64(x.size))
        return out

    # ---- pooling (max_pool.hpp, avg_pool.hpp) --------------------------------------------
    @staticmethod
    def pool_out_shape(shape, kernel, strides, pads_begin, pads_end, ceil_mode=False):
        out = list(shape[:2])
        for i in range(2):
            span = shape[2 + i] + pads_begin[i] + pads_end[i] - kernel[i]
            o = (-(-span // strides[i]) if ceil_mode else span // strides[i]) + 1
            out.append(o)
        return tuple(out)

    def _pool(self, name, x, kernel, strides, pads_begin, pads_end, extra=(), out_shape=None):
        x = np.ascontiguousarray(x)
        oshape = out_shape or self.pool_out_shape(x.shape, kernel, strides, pads_begin, pads_end)
        out = np.empty(oshape, x.dtype)
        i64 = ctypes.c_int64
        self._fn(name + _SUFFIX[x.dtype])(
            _ptr(x), _ptr(out), *[i64(int(v)) for v in x.shape],
            i64(kernel[0]), i64(kernel[1]), i64(strides[0]), i64(strides[1]),
            i64(pads_begin[0]), i64(pads_begin[1]), i64(pads_end[0]), i64(pads_end[1]),
            i64(oshape[2]), i64(oshape[3]), *extra)
        return out

    def max_pool(self, x, kernel, strides, pads_begin, pads_end, out_shape=None):
        return self._pool("max_pool_", x, kernel, strides, pads_begin, pads_end,
                          out_shape=out_shape)

    def avg_pool(self, x, kernel, strides, pads_begin, pads_end, include_pad, out_shape=None):
        return self._pool("avg_pool_", x, kernel, strides, pads_begin, pads_end,
                          extra=(ctypes.c_int(int(include_pad)),), out_shape=out_shape)

    # ---- fp32 glue (softmax.hpp, mvn.hpp, gelu.hpp) ---------------------------------------
    def softmax(self, x, axis):
        x = np.ascontiguousarray(x, np.float32)
        axis %= x.ndim
        outer = int(np.prod(x.shape[:axis], dtype=np.int64))
        inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
        out = np.empty_like(x)
        i64 = ctypes.c_int64
        self._fn("softmax_f32")(_ptr(x), _ptr(out), i64(outer), i64(x.shape[axis]), i64(inner))
        return out

    def mvn_last_axis(self, x, normalize_variance=True, eps=1e-5, eps_inside=True):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        i64 = ctypes.c_int64
        self._fn("mvn_last_axis_f32")(_ptr(x), _ptr(out), i64(x.size // x.shape[-1]),
                                      i64(x.shape[-1]), int(normalize_variance),
                                      ctypes.c_double(eps), int(eps_inside))
        return out

    def gelu_erf(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        self._fn("gelu_erf_f32")(_ptr(x), _ptr(out), ctypes.c_int64(x.size))
        return out


def _load(path, prefix):
    return _Ops(path, prefix) if os.path.exists(path) else None


ops = _load(os.path.join(_HERE, "liboracle.so"), "orc_")
ref = _load(os.path.join(_HERE, "_ref", "libngraph_ref.so"), "ref_")


def require_ops():
    global ops
    if ops is None:
        build(with_ref=False)
        ops = _load(os.path.join(_HERE, "liboracle.so"), "orc_")
    return ops
