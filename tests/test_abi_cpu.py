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
    for c in (0, 17, 47):
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
    for tile in (0, 4, 12, 14, 15, 16, 17):
        long_k.set_tile(tile)
    short_k = _host_conv(64, 64, 1)            # one K step
    for tile in (18, -1, 12, 13, 14, 17):
        with pytest.raises(HipieError) as e:
            short_k.set_tile(tile)
        assert e.value.status == -4, tile      # PARAMETER_MISMATCH
    with pytest.raises(HipieError):
        long_k.set_tile(13)                    # not a 4-byte-pixel first layer


def test_epilogue_rejects_an_inverted_clamp_range():
    from dldt_amd import HipieError, make_epilogue
    fq = (256, 0.0, 6.0, 0.0, 255.0)
    _host_conv(32, 32, 1, make_epilogue(activation="clamp", clamp=(0.0, 6.0), out_dtype=41, fq=fq))
    with pytest.raises(HipieError) as e:
        _host_conv(32, 32, 1, make_epilogue(activation="clamp", clamp=(6.0, 0.0), out_dtype=41, fq=fq))
    assert e.value.status == -4
