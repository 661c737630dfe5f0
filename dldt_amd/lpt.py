"""Bindings to the load-time LPT arithmetic (include/hipie.h section 3) and the few compositions
a model builder needs to write down the post-LPT constants of a quantized layer.

Every float operation is a single IEEE f32 step in the order the reference's constant folding
performs it (numpy float32 elementwise ops == reference::multiply / divide on constants).
"""
import ctypes

import numpy as np

from ._lib import check, lib

U8, I8 = 40, 50
_f32p = ctypes.POINTER(ctypes.c_float)


def _p(a):
    return a.ctypes.data_as(_f32p)


def precision_details(levels, out_low, out_high):
    """LayerTransformation::getPrecisionDetails -> (precision or None, has_negative, has_zero_point)."""
    ol = np.ascontiguousarray(np.asarray(out_low, np.float32).reshape(-1))
    oh = np.ascontiguousarray(np.asarray(out_high, np.float32).reshape(-1))
    prec, neg, zp = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    check(lib().hipie_lpt_precision_details(ctypes.c_int64(levels), _p(ol), _p(oh), ctypes.c_int64(ol.size),
                                            ctypes.byref(prec), ctypes.byref(neg), ctypes.byref(zp)))
    return (prec.value or None), bool(neg.value), bool(zp.value)


def data_precision_range(precision, levels):
    mn, mx = ctypes.c_float(), ctypes.c_float()
    check(lib().hipie_lpt_data_precision_range(precision, ctypes.c_int64(levels), ctypes.byref(mn),
                                               ctypes.byref(mx)))
    return mn.value, mx.value


def decompose_fake_quantize(levels, out_low, out_high, allow_zero_point=False, precision=None):
    """NetworkHelper::decomposeFakeQuantize for an FQ whose precision getPrecisionDetails resolves, or
    (allow_zero_point) for an asymmetric range: the first supported activation precision, u8, with a
    zero point (fake_quantize_decomposition.cpp:343-372).

    precision forces the data precision (a layer that only takes u8 activations: the intervals'
    own precision is then not among the supported ones and a zero point is used, :359-366).

    Returns dict(precision, new_low, new_high, scale, shift) with arrays shaped like out_low.
    """
    ol = np.ascontiguousarray(np.asarray(out_low, np.float32))
    oh = np.ascontiguousarray(np.asarray(out_high, np.float32))
    prec, _, zp = precision_details(levels, ol, oh)
    if precision is not None and prec != precision:
        prec, zp = precision, True
    if prec is None and allow_zero_point:
        prec, zp = U8, True
    if prec is None:
        raise NotImplementedError("FakeQuantize needs a zero point (asymmetric range): pass allow_zero_point")
    mn, mx = data_precision_range(prec, levels)
    sc, sh, nl, nh = (np.empty(ol.size, np.float32) for _ in range(4))
    check(lib().hipie_lpt_decompose_fake_quantize(_p(ol.reshape(-1)), _p(oh.reshape(-1)), ctypes.c_int64(ol.size),
                                                  ctypes.c_float(mn), ctypes.c_float(mx), _p(sc), _p(sh),
                                                  _p(nl), _p(nh)))
    return dict(precision=prec, new_low=np.float32(mn), new_high=np.float32(mx),
                scale=sc.reshape(ol.shape), shift=sh.reshape(ol.shape), has_zero_point=zp)


def fold_fake_quantize(values, in_low, in_high, out_low, out_high, levels, round_values=True):
    """NetworkHelper::foldFakeQuantize on a constant whose axis 0 is the output-channel axis."""
    v = np.ascontiguousarray(values, np.float32)
    oc = v.shape[0]
    inner = v.size // oc
    b = [np.ascontiguousarray(np.asarray(x, np.float32).reshape(-1)) for x in (in_low, in_high, out_low, out_high)]
    out = np.empty_like(v)
    args = []
    for x in b:
        args += [_p(x), ctypes.c_int64(x.size)]
    check(lib().hipie_lpt_fold_fake_quantize(_p(v), ctypes.c_int64(oc), ctypes.c_int64(inner), *args,
                                             ctypes.c_int64(levels), int(round_values), _p(out)))
    return out


def quantize_weights(w, levels=255):
    """Per-output-channel symmetric weight FakeQuantize (range +-max|w_c|) taken through
    decomposeFakeQuantize + foldFakeQuantize: returns (i8 weights, scale[OC])."""
    w = np.ascontiguousarray(w, np.float32)
    oc = w.shape[0]
    m = np.abs(w.reshape(oc, -1)).max(axis=1).astype(np.float32)
    m = np.where(m == 0, np.float32(1.0), m)
    d = decompose_fake_quantize(levels, -m, m)
    assert d["precision"] == I8 and not d["has_zero_point"]
    q = fold_fake_quantize(w, -m, m, d["new_low"], d["new_high"], levels, round_values=True)
    assert np.abs(q).max() <= 127
    return q.astype(np.int8), d["scale"].astype(np.float32)


def round_zero_point(shift):
    """NetworkHelper::round(shift, u8) of optimizeSubtract (network_helper.cpp:485-494, 1500-1501):
    Round-5 HALF_AWAY_FROM_ZERO, then Convert to the activation's integer type."""
    s = np.asarray(shift, np.float32)
    return (np.sign(s) * np.floor(np.abs(s) + np.float32(0.5))).astype(np.float32)


MULTIPLY, SUBTRACT, ADD = 1, 2, 3


def _vec(a):
    return np.ascontiguousarray(np.asarray(a, np.float32).reshape(-1))


def swap_multiply_and_add(b, a):
    """NetworkHelper::swapMultiplyAndAdd: the constant b / a of x * a + b ==> (x + b / a) * a (0 where both are 0)."""
    bv, av = _vec(b), _vec(a)
    n = max(bv.size, av.size)
    out = np.empty(n, np.float32)
    check(lib().hipie_lpt_swap_multiply_and_add(_p(bv), ctypes.c_int64(bv.size), _p(av), ctypes.c_int64(av.size), _p(out),
                                                ctypes.c_int64(n)))
    return out


def fuse_elementwise(kind, in_low, in_high, value):
    """FakeQuantizeTransformation::fuseElementwise: (new_low, new_high) of a FakeQuantize that absorbs the Multiply /
    Subtract / Add by a constant in front of it, or None when the reference does not fuse (a non-positive factor)."""
    lo, hi, v = _vec(in_low), _vec(in_high), _vec(value)
    assert lo.size == hi.size
    n = max(lo.size, v.size)
    nl, nh = np.empty(n, np.float32), np.empty(n, np.float32)
    fused = ctypes.c_int()
    check(lib().hipie_lpt_fuse_elementwise(kind, _p(lo), _p(hi), ctypes.c_int64(lo.size), _p(v), ctypes.c_int64(v.size),
                                           _p(nl), _p(nh), ctypes.c_int64(n), ctypes.byref(fused)))
    return (nl, nh) if fused.value else None


def add_both_branches(shift_full, scale_full, shift_empty, scale_empty):
    """AddTransformation with dequantizations on both branches: (new shift, new scale) of the full path and the
    scale of the Multiply behind the Add."""
    a = [_vec(x) for x in (shift_full, scale_full, shift_empty, scale_empty)]
    n = max(x.size for x in a)
    a = [np.ascontiguousarray(np.broadcast_to(x, (n,))) for x in a]
    out = [np.empty(n, np.float32) for _ in range(3)]
    check(lib().hipie_lpt_add_both_branches(*[_p(x) for x in a], ctypes.c_int64(n), *[_p(x) for x in out]))
    return tuple(out)


def clamp_bounds(lo, hi, scale, shift=0.0):
    """ClampTransformation: the bounds of a Clamp moved in front of the per-tensor dequantization (x - shift) * scale"""
    a, b = ctypes.c_double(), ctypes.c_double()
    check(lib().hipie_lpt_clamp_bounds(ctypes.c_double(lo), ctypes.c_double(hi), ctypes.c_double(scale), ctypes.c_double(shift),
                                       ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value
