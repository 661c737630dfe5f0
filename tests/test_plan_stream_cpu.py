"""Export / Import of a plan (dry runs: no device needed): the stream round-trips, and a stream that is
not what an export wrote is refused with NETWORK_NOT_READ, whatever was done to it."""
import struct

import numpy as np
import pytest

from dldt_amd import HipieError, builders
from dldt_amd.graph import Plan


def _fnv1a(b):
    h = 1469598103934665603
    for x in b:
        h = ((h ^ x) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def _reseal(body):
    """a stream with `body` (everything but the checksum) and the checksum that fits it"""
    return body + struct.pack("<Q", _fnv1a(body))


def _summary(plan):
    return [(s["name"], s["type"], s["macs"], s["bytes"]) for s in plan.steps], plan.inputs, plan.outputs, plan.arena_bytes


@pytest.mark.parametrize("net", ["conv_block", "resnet", "mobilenet", "encoder", "zero_point"])
def test_round_trip(net):
    if net == "conv_block":
        g = builders.conv_block()[0]
    elif net == "resnet":
        g = builders.resnet50(batch=2, res=64, width=16, classes=10, seed=7)[0]
    elif net == "mobilenet":
        g = builders.mobilenet_v2(batch=2, res=64, width=0.5, classes=10, last=128, seed=3)[0]
    elif net == "encoder":
        g = builders.bert_encoder(layers=2, batch=2, seq=64, hidden=128, heads=2, ffn=256, seed=3, vocab=50, mask=True)[0]
    else:
        g = builders.zero_point_net()[0]
    plan = g.compile(-1)
    blob = plan.export()
    assert blob[:8] == b"HIPIEPLN" and struct.unpack("<Q", blob[-8:])[0] == _fnv1a(blob[:-8])
    back = Plan.load(blob, -1)
    assert _summary(back) == _summary(plan)
    assert back.export() == blob                       # the description survives unchanged, constants included


def test_refused_streams():
    blob = builders.conv_block()[0].compile(-1).export()
    cases = {
        "empty": b"",
        "short": blob[:20],
        "not a plan": b"RIFF" + blob[4:],
        "truncated": blob[:-9],
        "flipped bit": blob[:200] + bytes([blob[200] ^ 4]) + blob[201:],
        "other format": _reseal(blob[:8] + struct.pack("<I", 99) + blob[12:-8]),
        "bytes behind the graph": _reseal(blob[:-8] + b"\0\0\0\0"),
        "too many steps": _reseal(blob[:12] + struct.pack("<I", 1 << 30) + blob[16:-8]),
    }
    for what, bad in cases.items():
        with pytest.raises(HipieError) as e:
            Plan.load(bad, -1)
        assert e.value.status == -12, what


def test_damaged_streams_with_a_valid_checksum_never_get_past_validation():
    """the checksum only catches accidents; behind it every field is checked again: random damage inside
    the graph description either still describes a valid graph or is refused with a status, never worse"""
    blob = builders.conv_block(n=1, c=16, hw=8, oc=16)[0].compile(-1).export()
    body = bytearray(blob[:-8])
    n_steps = struct.unpack("<I", blob[12:16])[0]
    start = 16 + 4 * n_steps + 8
    rng = np.random.default_rng(1)
    # the structured part of the description (node headers) is where damage matters; constants are payload
    offsets = [int(o) for o in rng.integers(start, len(body), 150)] + list(range(start, start + 120))
    refused = loaded = 0
    for o in offsets:
        bad = bytearray(body)
        bad[o] = (bad[o] + int(rng.integers(1, 256))) & 0xFF
        try:
            Plan.load(_reseal(bytes(bad)), -1)
            loaded += 1
        except HipieError as e:
            assert e.status in (-12, -2, -4), (o, e.status, str(e))
            refused += 1
    assert refused > 20 and loaded > 0


def test_export_needs_room():
    import ctypes
    from dldt_amd._lib import lib
    plan = builders.conv_block()[0].compile(-1)
    size = ctypes.c_size_t()
    assert lib().hipie_plan_export(plan._h, None, ctypes.c_size_t(0), ctypes.byref(size)) == 0 and size.value > 0
    small = ctypes.create_string_buffer(16)
    assert lib().hipie_plan_export(plan._h, small, ctypes.c_size_t(16), ctypes.byref(size)) == -6
