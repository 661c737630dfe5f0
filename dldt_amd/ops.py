"""Operator-level bindings (one class per load-time object of include/hipie.h).

Device memory is passed as torch CUDA tensors (plumbing only): the classes hand their
``data_ptr()`` and the current HIP stream to the C ABI.
"""
import ctypes

import numpy as np

from ._lib import check, lib

F32, U8, I8, I32, U8B = 10, 40, 50, 70, 41
NCHW, NHWC = 1, 2
_DT = {"u8": U8, "u8b": U8B, "i8": I8}


def _fptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dptr(t):
    return ctypes.c_void_p(t.data_ptr())


class FakeQuantize:
    """Per-channel FakeQuantize (ngraph op FakeQuantize-1; reference fake_quantize.hpp:175-265).

    Bounds are scalars or per-channel arrays (any shape with C or 1 elements, e.g. [1,C,1,1]).
    ``device=-1`` builds a host-only object for load-time checks.
    """

    def __init__(self, channels, levels, in_low, in_high, out_low, out_high, device=0):
        self.C, self.levels, self.device = int(channels), int(levels), device
        bounds = [np.ascontiguousarray(np.asarray(b, np.float32).reshape(-1))
                  for b in (in_low, in_high, out_low, out_high)]
        self._h = ctypes.c_void_p()
        args = []
        for b in bounds:
            args += [_fptr(b), ctypes.c_int64(b.size)]
        check(lib().hipie_fq_create(ctypes.c_int(device), ctypes.c_int64(self.C),
                                    ctypes.c_int64(self.levels), *args, ctypes.byref(self._h)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().hipie_fq_destroy(self._h)
            self._h = None

    @property
    def uses_reciprocal(self):
        return bool(lib().hipie_fq_uses_reciprocal(self._h))

    def host_eval(self, channel, x):
        return float(lib().hipie_fq_host_eval(self._h, ctypes.c_int64(channel), ctypes.c_float(x)))

    def _nhw(self, x):
        assert x.is_contiguous() and x.shape[1] == self.C, (x.shape, self.C)
        hw = 1
        for d in x.shape[2:]:
            hw *= d
        return x.shape[0], hw

    def run_f32(self, x, out=None):
        import torch
        n, hw = self._nhw(x)
        y = torch.empty_like(x) if out is None else out
        check(lib().hipie_fq_run_f32(self._h, _dptr(x), _dptr(y), ctypes.c_int64(n),
                                     ctypes.c_int64(hw), _stream()))
        return y

    def run_q8(self, x, dtype="u8", layout="nchw", c_stride=None, out=None):
        import torch
        n, hw = self._nhw(x)
        tdt = torch.int8 if dtype in ("i8", "u8b") else torch.uint8
        if layout == "nchw":
            y = torch.empty(x.shape, dtype=tdt, device=x.device) if out is None else out
            cs = 0
        else:
            cs = c_stride or -(-self.C // 16) * 16
            y = torch.empty((n,) + tuple(x.shape[2:]) + (cs,), dtype=tdt, device=x.device) \
                if out is None else out
        check(lib().hipie_fq_run_q8(self._h, _dptr(x), _dptr(y), ctypes.c_int64(n),
                                    ctypes.c_int64(hw), ctypes.c_int(_DT[dtype]),
                                    ctypes.c_int(NCHW if layout == "nchw" else NHWC),
                                    ctypes.c_int64(cs), _stream()))
        return y
