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


class hipie_epilogue(ctypes.Structure):
    _fp = ctypes.POINTER(ctypes.c_float)
    _fields_ = [("bias", _fp), ("n_bias", ctypes.c_int64), ("scale", _fp), ("n_scale", ctypes.c_int64),
                ("residual_dtype", ctypes.c_int32),
                ("res_sub", _fp), ("n_res_sub", ctypes.c_int64), ("res_mul", _fp), ("n_res_mul", ctypes.c_int64),
                ("post_scale", _fp), ("n_post_scale", ctypes.c_int64),
                ("activation", ctypes.c_int32), ("clamp_lo", ctypes.c_float), ("clamp_hi", ctypes.c_float),
                ("out_dtype", ctypes.c_int32), ("fq_levels", ctypes.c_int64),
                ("fq_in_low", _fp), ("n_fq_in_low", ctypes.c_int64),
                ("fq_in_high", _fp), ("n_fq_in_high", ctypes.c_int64),
                ("fq_out_low", ctypes.c_float), ("fq_out_high", ctypes.c_float)]


class hipie_conv_desc(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int32) for k in (
        "in_dtype", "ic", "oc", "kh", "kw", "stride_h", "stride_w", "dil_h", "dil_w",
        "pad_top", "pad_left", "pad_bottom", "pad_right", "groups", "in_c_stride",
        "in_stride_h", "in_stride_w", "in_zero_point")] + [("in_zero_points", ctypes.POINTER(ctypes.c_int32)),
                                                            ("acc_sub", ctypes.POINTER(ctypes.c_int32))]


def make_epilogue(bias=None, scale=None, residual_dtype=0, res_sub=None, res_mul=None,
                  post_scale=None, activation=None, clamp=(0.0, 0.0), out_dtype=F32,
                  fq=None):
    """fq = (levels, in_low, in_high, out_low, out_high) for 8-bit outputs."""
    e = hipie_epilogue()
    keep = []

    def put(name, v):
        if v is None:
            return
        a = np.ascontiguousarray(np.asarray(v, np.float32).reshape(-1))
        keep.append(a)
        setattr(e, name, _fptr(a))
        setattr(e, "n_" + name, a.size)

    put("bias", bias)
    put("scale", scale)
    e.residual_dtype = residual_dtype
    put("res_sub", res_sub)
    put("res_mul", res_mul)
    put("post_scale", post_scale)
    e.activation = {None: 0, "relu": 1, "clamp": 2}[activation]
    e.clamp_lo, e.clamp_hi = float(clamp[0]), float(clamp[1])
    e.out_dtype = out_dtype
    if fq is not None:
        e.fq_levels = int(fq[0])
        put("fq_in_low", fq[1])
        put("fq_in_high", fq[2])
        e.fq_out_low, e.fq_out_high = float(fq[3]), float(fq[4])
    e._keep = keep
    return e


class Convolution:
    """u8/i8 x i8 convolution with fused epilogue (ngraph Convolution-1 after LPT).

    ``weights`` is int8 OIHW; ``in_tensor`` fixes the input geometry the weights are packed for.
    """

    def __init__(self, weights, in_tensor, strides=(1, 1), dilations=(1, 1), pads_begin=(0, 0),
                 pads_end=(0, 0), epilogue=None, device=0, zero_point=0):
        w = np.ascontiguousarray(weights, np.int8)
        if w.ndim == 5:   # GroupConvolution filters [G, OC/G, IC/G, kh, kw] = [oc][ic / groups][kh][kw] in memory
            groups = w.shape[0]
            self.oc, self.ic = groups * w.shape[1], groups * w.shape[2]
            self.kh, self.kw = w.shape[3:]
        else:
            groups = 1
            self.oc, self.ic, self.kh, self.kw = w.shape
        # zero_point: one integer level, or one per input channel
        zps = None if np.ndim(zero_point) == 0 else np.ascontiguousarray(zero_point, np.int32)
        d = hipie_conv_desc(in_tensor.dtype, self.ic, self.oc, self.kh, self.kw, strides[0], strides[1],
                            dilations[0], dilations[1], pads_begin[0], pads_begin[1], pads_end[0],
                            pads_end[1], groups, in_tensor.cs, in_tensor.stride_h, in_tensor.stride_w,
                            0 if zps is not None else int(zero_point),
                            zps.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)) if zps is not None else None, None)
        assert zps is None or zps.shape == (self.ic,)
        self.epilogue = epilogue or make_epilogue(out_dtype=I32)
        self._h = ctypes.c_void_p()
        check(lib().hipie_conv_create(ctypes.c_int(device), ctypes.byref(d),
                                      w.ctypes.data_as(ctypes.c_void_p), ctypes.byref(self.epilogue),
                                      ctypes.byref(self._h)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().hipie_conv_destroy(self._h)
            self._h = None

    def out_dims(self, h, w):
        oh, ow = ctypes.c_int32(), ctypes.c_int32()
        check(lib().hipie_conv_out_dims(self._h, h, w, ctypes.byref(oh), ctypes.byref(ow)))
        return oh.value, ow.value

    def set_tile(self, tile, stages=0):
        check(lib().hipie_conv_set_tile(self._h, tile))
        check(lib().hipie_conv_set_stages(self._h, stages))

    def get_tile(self):
        t = ctypes.c_int()
        check(lib().hipie_conv_get_tile(self._h, ctypes.byref(t)))
        return t.value

    def run(self, x, out, residual=None):
        xd, od = x.desc(), out.desc()
        rd = residual.desc() if residual is not None else None
        check(lib().hipie_conv_run(self._h, ctypes.byref(xd), ctypes.byref(rd) if rd else None,
                                   ctypes.byref(od), _stream()))
        return out

    def pair_fits(self, second, h, w):
        """hipie_conv_pair_fits: does the fused kernel take this layer followed by ``second`` on h x w inputs"""
        return bool(self.pair_forms(second, h, w))

    def pair_forms(self, second, h, w):
        """the raw answer of hipie_conv_pair_fits: 0, or bit 0 (fits) and bit 1 (also with two wave groups: stages 7)"""
        fits = ctypes.c_int()
        check(lib().hipie_conv_pair_fits(self._h, second._h, h, w, ctypes.byref(fits)))
        return fits.value

    def set_stages(self, stages):
        check(lib().hipie_conv_set_stages(self._h, stages))

    def run_pair(self, second, x, out, residual=None):
        """hipie_conv_run_pair: this layer and ``second`` in one kernel, the intermediate tensor kept in LDS"""
        xd, od = x.desc(), out.desc()
        rd = residual.desc() if residual is not None else None
        check(lib().hipie_conv_run_pair(self._h, second._h, ctypes.byref(xd), ctypes.byref(rd) if rd else None,
                                        ctypes.byref(od), _stream()))
        return out

    def run_static(self, x, out, residual=None):
        """hipie_conv_run_static: the same launch with the K-split workspace in the library's fixed device array"""
        xd, od = x.desc(), out.desc()
        rd = residual.desc() if residual is not None else None
        check(lib().hipie_conv_run_static(self._h, ctypes.byref(xd), ctypes.byref(rd) if rd else None,
                                          ctypes.byref(od), _stream()))
        return out


class hipie_matmul_desc(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int32) for k in ("a_dtype", "b_dtype", "k", "n", "a_zero_point", "b_zero_point")]


class BatchedMatMul:
    """i8 / u8 x i8 / u8 MatMul between two activation tensors: out[b] = A[b] @ Bt[b]^T (+ fused epilogue).

    ``a`` is a torch int8 tensor [batch, M, K] (u8 levels stored as level - 128 with ``a_dtype=U8B``), ``bt`` is
    [batch, N, K] (the transpose_b = true form, ``b_dtype`` likewise); the result is [batch, M, ldo] with ldo = N
    padded to the store granularity.
    """

    def __init__(self, k, n, epilogue=None, device=0, a_dtype=I8, a_zero_point=0, b_dtype=I8, b_zero_point=0):
        self.k, self.n = k, n
        self.epilogue = epilogue or make_epilogue(out_dtype=I32)
        d = hipie_matmul_desc(a_dtype, b_dtype, k, n, a_zero_point, b_zero_point)
        self._h = ctypes.c_void_p()
        check(lib().hipie_matmul_create(ctypes.c_int(device), ctypes.byref(d), ctypes.byref(self.epilogue),
                                        ctypes.byref(self._h)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().hipie_matmul_destroy(self._h)
            self._h = None

    def run(self, a, bt, out=None):
        import torch
        batch, m, k = a.shape
        assert bt.shape[0] == batch and bt.shape[2] == k and bt.shape[1] == self.n and k == self.k
        assert a.is_contiguous() and bt.is_contiguous()
        od = self.epilogue.out_dtype
        tdt, gran = {I32: (torch.int32, 4), F32: (torch.float32, 4)}.get(od, (torch.int8, 16))
        ldo = -(-self.n // gran) * gran
        if out is None:
            out = torch.zeros((batch, m, ldo), dtype=tdt, device=a.device)
        assert out.shape == (batch, m, ldo) and out.dtype == tdt and out.is_contiguous()
        i64 = ctypes.c_int64
        need = ctypes.c_size_t()
        check(lib().hipie_matmul_workspace_size(self._h, ctypes.c_int32(m), ctypes.c_int32(batch), ctypes.c_int32(1),
                                                ctypes.byref(need)))
        ws = torch.empty(max(need.value, 16), dtype=torch.int8, device=a.device)
        check(lib().hipie_matmul_run_nested_ws(self._h, _dptr(a), i64(k), i64(m * k), i64(0), _dptr(bt), i64(k),
                                               i64(self.n * k), i64(0), _dptr(out), i64(ldo), i64(m * ldo), i64(0),
                                               ctypes.c_int32(m), ctypes.c_int32(batch), ctypes.c_int32(1),
                                               _dptr(ws) if need.value else None, ctypes.c_size_t(need.value), _stream()))
        return out[..., :self.n]


def matmul_strided(mm, a, lda, stride_a, bt, ldb, stride_b, out, ldo, stride_o, m, batch,
                   batch_outer=1, outer_a=0, outer_b=0, outer_o=0):
    """hipie_matmul_run_nested on raw device pointers (ints) with explicit leading dimensions and
    batch strides, for operands that are slices of larger tensors (attention heads inside [T, 3H]:
    batch = heads with stride 64, batch_outer = sequences)."""
    i64 = ctypes.c_int64
    check(lib().hipie_matmul_run_nested(mm._h, ctypes.c_void_p(a), i64(lda), i64(stride_a), i64(outer_a),
                                        ctypes.c_void_p(bt), i64(ldb), i64(stride_b), i64(outer_b), ctypes.c_void_p(out),
                                        i64(ldo), i64(stride_o), i64(outer_o), ctypes.c_int32(m), ctypes.c_int32(batch),
                                        ctypes.c_int32(batch_outer), _stream()))


def transpose_bytes(src, ld_src, bs_src, dst, ld_dst, bs_dst, rows, cols, batch, batch_outer=1, outer_src=0, outer_dst=0):
    """dst[o][b][c][r] = src[o][b][r][c] on raw device pointers (ints), sizes in bytes."""
    i64 = ctypes.c_int64
    check(lib().hipie_transpose_bytes_nested(ctypes.c_void_p(src), i64(ld_src), i64(bs_src), i64(outer_src),
                                             ctypes.c_void_p(dst), i64(ld_dst), i64(bs_dst), i64(outer_dst),
                                             ctypes.c_int32(rows), ctypes.c_int32(cols), ctypes.c_int32(batch),
                                             ctypes.c_int32(batch_outer), _stream()))


class hipie_requant(ctypes.Structure):
    _fields_ = [("in_low", ctypes.c_float), ("in_high", ctypes.c_float), ("out_low", ctypes.c_float),
                ("levels", ctypes.c_int64)]


def _glue_outputs(x, requant, keep_f32):
    """(y, q, requant struct pointer): f32 result and / or i8 levels of the fused per-tensor FakeQuantize
    requant = (in_low, in_high, out_low, levels)."""
    import torch
    assert x.is_contiguous() and x.dtype == torch.float32
    y = torch.empty_like(x) if (requant is None or keep_f32) else None
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device) if requant is not None else None
    r = hipie_requant(*[float(v) for v in requant[:3]], int(requant[3])) if requant is not None else None
    return y, q, r


def _ret(y, q):
    return y if q is None else (q if y is None else (y, q))


def softmax(x, requant=None, keep_f32=True):
    """Softmax over the last axis; with requant also (or only, keep_f32=False) the i8 levels of the
    FakeQuantize behind it."""
    y, q, r = _glue_outputs(x, requant, keep_f32)
    rows, axis = ctypes.c_int64(x.numel() // x.shape[-1]), ctypes.c_int64(x.shape[-1])
    if q is None:
        check(lib().hipie_softmax_f32(_dptr(x), _dptr(y), rows, axis, _stream()))
    else:
        check(lib().hipie_softmax_q8(_dptr(x), _dptr(y) if y is not None else None, _dptr(q), rows, axis,
                                     ctypes.byref(r), _stream()))
    return _ret(y, q)


def mvn(x, normalize_variance=True, eps=1e-5, eps_inside=True, gamma=None, beta=None, requant=None, keep_f32=True):
    y, q, r = _glue_outputs(x, requant, keep_f32)
    args = [ctypes.c_int64(x.numel() // x.shape[-1]), ctypes.c_int64(x.shape[-1]), int(normalize_variance),
            ctypes.c_float(eps), int(eps_inside), _dptr(gamma) if gamma is not None else None,
            _dptr(beta) if beta is not None else None]
    if q is None:
        check(lib().hipie_mvn_f32(_dptr(x), _dptr(y), *args, _stream()))
    else:
        check(lib().hipie_mvn_q8(_dptr(x), _dptr(y) if y is not None else None, _dptr(q), *args, ctypes.byref(r),
                                 _stream()))
    return _ret(y, q)


def gelu(x, requant=None, keep_f32=True):
    y, q, r = _glue_outputs(x, requant, keep_f32)
    if q is None:
        check(lib().hipie_gelu_f32(_dptr(x), _dptr(y), ctypes.c_int64(x.numel()), _stream()))
    else:
        check(lib().hipie_gelu_q8(_dptr(x), _dptr(y) if y is not None else None, _dptr(q), ctypes.c_int64(x.numel()),
                                  ctypes.byref(r), _stream()))
    return _ret(y, q)


def add_broadcast(x, addend, out=None):
    """x + addend for a contiguous f32 device tensor of up to four dimensions and an addend of the same rank whose
    dimensions are x's or 1 (hipie_add_broadcast_f32); out may be x itself."""
    import torch
    assert x.is_contiguous() and addend.is_contiguous() and x.dtype == addend.dtype == torch.float32 and x.dim() == addend.dim()
    y = torch.empty_like(x) if out is None else out
    dims = (ctypes.c_int64 * x.dim())(*x.shape)
    adims = (ctypes.c_int64 * x.dim())(*addend.shape)
    check(lib().hipie_add_broadcast_f32(_dptr(x), dims, _dptr(addend), adims, x.dim(), _dptr(y), _stream()))
    return y


class hipie_attention_desc(ctypes.Structure):
    _fields_ = [("seq", ctypes.c_int32), ("head_dim", ctypes.c_int32), ("score_scale", ctypes.c_float),
                ("context_scale", ctypes.c_float), ("prob_fq", hipie_requant), ("out_dtype", ctypes.c_int32),
                ("out_fq", hipie_requant), ("prob_dtype", ctypes.c_int32)]


class Attention:
    """Fused attention core (hipie_attention_*): MatMul'(q, k^T) * score_scale -> Softmax ->
    FakeQuantize(prob_fq) -> MatMul'(., v) * context_scale [-> FakeQuantize(out_fq)].
    prob_fq / out_fq = (in_low, in_high, out_low, levels)."""

    def __init__(self, seq, head_dim, score_scale, context_scale, prob_fq, out_fq=None, device=0, prob_dtype=I8):
        d = hipie_attention_desc()
        d.prob_dtype = prob_dtype
        d.seq, d.head_dim = seq, head_dim
        d.score_scale, d.context_scale = float(score_scale), float(context_scale)
        d.prob_fq = hipie_requant(*[float(x) for x in prob_fq[:3]], int(prob_fq[3]))
        d.out_dtype = I8 if out_fq is not None else F32
        if out_fq is not None:
            d.out_fq = hipie_requant(*[float(x) for x in out_fq[:3]], int(out_fq[3]))
        self.byte_out = out_fq is not None
        self._h = ctypes.c_void_p()
        check(lib().hipie_attention_create(ctypes.c_int(device), ctypes.byref(d), ctypes.byref(self._h)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().hipie_attention_destroy(self._h)
            self._h = None

    def run(self, q, k, v, dump=False, out=None, mask=None):
        """q, k, v: i8 [B, NH, S, 64] (any strides with contiguous rows); mask: f32 [B, S] added to the
        scaled scores of every head and query, or None.  Returns the context [B, NH, S, 64] and, with
        dump=True, also the f32 Softmax inputs and probabilities [B, NH, S, S]."""
        import torch
        B, NH, S, D = q.shape
        assert k.shape == q.shape and v.shape == q.shape and q.dtype == torch.int8
        for t in (q, k, v):
            assert t.stride(3) == 1
        if out is None:
            out = torch.empty((B, NH, S, D), dtype=torch.int8 if self.byte_out else torch.float32, device=q.device)
        scores = torch.empty((B, NH, S, S), dtype=torch.float32, device=q.device) if dump else None
        probs = torch.empty_like(scores) if dump else None
        i64 = ctypes.c_int64
        args = []
        for t in (q, k, v, out):
            args += [_dptr(t), i64(t.stride(2)), i64(t.stride(1)), i64(t.stride(0))]
        if mask is not None:
            assert mask.shape == (B, S) and mask.is_contiguous() and mask.dtype == torch.float32
        check(lib().hipie_attention_run(self._h, *args, ctypes.c_int32(NH), ctypes.c_int32(B),
                                        _dptr(mask) if mask is not None else None, i64(0), i64(S),
                                        _dptr(scores) if dump else None, _dptr(probs) if dump else None, _stream()))
        return (out, scores, probs) if dump else out


def attention(q, k, v, score_scale, context_scale, prob_fq, out_fq=None, dump=False, mask=None):
    """One-shot form of Attention (creates the load-time object for this call)."""
    att = Attention(q.shape[2], q.shape[3], score_scale, context_scale, prob_fq, out_fq, q.device.index or 0)
    return att.run(q, k, v, dump=dump, mask=mask)
