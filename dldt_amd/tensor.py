"""Device tensors in the engine's activation layout (NHWC, padded channels, halo of level 0).

torch provides the device memory; everything handed to the C ABI is a raw pointer inside a
``hipie_tensor`` struct.
"""
import ctypes

import numpy as np

F32, U8, I8, I32, U8B = 10, 40, 50, 70, 41


class hipie_tensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32),
                ("n", ctypes.c_int32), ("h", ctypes.c_int32), ("w", ctypes.c_int32), ("c", ctypes.c_int32),
                ("stride_n", ctypes.c_int64), ("stride_h", ctypes.c_int64), ("stride_w", ctypes.c_int64),
                ("halo", ctypes.c_int32)]


_TORCH = {F32: "float32", I32: "int32", U8B: "int8", I8: "int8", U8: "uint8"}
_SLACK = 256  # bytes readable before and after the tensor (K-padding reads of the first layer)


class DeviceTensor:
    def __init__(self, n, h, w, c, dtype, halo=0, c_stride=None, device="cuda", fill_level=0):
        import torch
        self.n, self.h, self.w, self.c, self.dtype, self.halo = n, h, w, c, dtype, halo
        gran = 16 if dtype in (U8B, I8, U8) else 4
        self.cs = c_stride or -(-c // gran) * gran
        self.hp, self.wp = h + 2 * halo, w + 2 * halo
        tdt = getattr(torch, _TORCH[dtype])
        esz = torch.empty((), dtype=tdt).element_size()
        slack = _SLACK // esz
        self.numel = n * self.hp * self.wp * self.cs
        fill = fill_level - 128 if dtype == U8B else fill_level      # halo and channel padding: this level
        self.buf = torch.full((self.numel + 2 * slack,), fill, dtype=tdt, device=device)
        self.view = self.buf[slack:slack + self.numel].view(n, self.hp, self.wp, self.cs)
        self.stride_w = self.cs
        self.stride_h = self.wp * self.cs
        self.stride_n = self.hp * self.wp * self.cs
        origin = slack + (halo * self.wp + halo) * self.cs
        self.data_ptr = self.buf.data_ptr() + origin * esz

    def interior(self):
        hl = self.halo
        return self.view[:, hl:hl + self.h, hl:hl + self.w, :]

    def desc(self):
        return hipie_tensor(ctypes.c_void_p(self.data_ptr), self.dtype, self.n, self.h, self.w, self.c,
                            self.stride_n, self.stride_h, self.stride_w, self.halo)

    # ---- host <-> device in the reference's layout (NCHW, plain values) ----------------------
    @classmethod
    def from_nchw(cls, x, dtype, halo=0, c_stride=None, device="cuda", fill_level=0):
        import torch
        n, c, h, w = x.shape
        t = cls(n, h, w, c, dtype, halo, c_stride, device, fill_level)
        a = np.ascontiguousarray(np.transpose(x, (0, 2, 3, 1)))
        if dtype == U8B:
            a = (a.astype(np.int16) - 128).astype(np.int8)
        elif dtype == I8:
            a = a.astype(np.int8)
        elif dtype == F32:
            a = a.astype(np.float32)
        elif dtype == I32:
            a = a.astype(np.int32)
        t.interior()[..., :c] = torch.from_numpy(a).to(device)
        return t

    def to_nchw(self):
        a = self.interior()[..., :self.c].cpu().numpy()
        if self.dtype == U8B:
            a = (a.astype(np.int16) + 128).astype(np.uint8)
        return np.ascontiguousarray(np.transpose(a, (0, 3, 1, 2)))

    def padded_channels(self):
        """Values of the channel padding [c, c_stride) of the interior (plain levels for U8B)."""
        a = self.interior()[..., self.c:].cpu().numpy()
        if self.dtype == U8B:
            a = (a.astype(np.int16) + 128).astype(np.uint8)
        return a
