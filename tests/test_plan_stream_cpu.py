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


def sections(blob):
    """offsets inside an exported stream: (graph start, graph bytes, [(key offset of every reciprocal verdict)],
    [(offset, size) of every packed operand])"""
    n_steps = struct.unpack("<I", blob[12:16])[0]
    at = 16 + 4 * n_steps
    gb = struct.unpack("<Q", blob[at:at + 8])[0]
    r = at + 8 + gb
    n_rcp = struct.unpack("<Q", blob[r:r + 8])[0]
    rcp = [r + 8 + 24 * i for i in range(n_rcp)]
    r += 8 + 24 * n_rcp
    n_div2 = struct.unpack("<Q", blob[r:r + 8])[0]
    r += 8 + 16 * n_div2
    n_blobs = struct.unpack("<Q", blob[r:r + 8])[0]
    r += 8
    blobs = []
    for _ in range(n_blobs):
        n = struct.unpack("<Q", blob[r:r + 8])[0]
        blobs.append((r + 8, n))
        r += 8 + n
    assert r == len(blob) - 8
    return at + 8, gb, rcp, blobs


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


def test_prepared_sections_are_validated():
    """behind the graph: the load-time checks' verdicts and the packed operands.  What is not a verdict, ends early or
    does not fit the layers of the graph is refused."""
    blob = builders.conv_block()[0].compile(-1).export()
    start, gb, rcp, blobs = sections(blob)
    assert rcp and len(blobs) >= 2                       # a convolution: the packed matrix and its correction vector
    off, n = blobs[0]
    cases = {
        "verdict that is no 0 / 1": blob[:rcp[0] + 20] + struct.pack("<I", 7) + blob[rcp[0] + 24:-8],
        "operand of another size": blob[:off - 8] + struct.pack("<Q", n - 64) + blob[off:off + n - 64] + blob[off + n:-8],
    }
    count_at = blobs[0][0] - 16
    cases["operand count beyond the stream"] = blob[:count_at] + struct.pack("<Q", 1 << 40) + blob[count_at + 8:-8]
    # one operand fewer than the layers ask for
    last_off, last_n = blobs[-1]
    cases["operand missing"] = blob[:count_at] + struct.pack("<Q", len(blobs) - 1) + blob[count_at + 8:last_off - 8]
    # one more than they use
    cases["operand too many"] = blob[:count_at] + struct.pack("<Q", len(blobs) + 1) + blob[count_at + 8:-8] + struct.pack("<Q", 4) + b"abcd"
    for what, body in cases.items():
        with pytest.raises(HipieError) as e:
            Plan.load(_reseal(body), -1)
        assert e.value.status == -12, what


def test_damaged_streams_with_a_valid_checksum_never_get_past_validation():
    """the checksum only catches accidents; behind it every field is checked again: random damage inside
    the graph description either still describes a valid graph or is refused with a status, never worse"""
    blob = builders.conv_block(n=1, c=16, hw=8, oc=16)[0].compile(-1).export()
    body = bytearray(blob[:-8])
    start, gb, _, _ = sections(blob)
    rng = np.random.default_rng(1)
    # the structured part of the description (node headers) is where damage matters; constants are payload
    offsets = ([int(o) for o in rng.integers(start, start + gb, 150)] + list(range(start, start + 120)) +
               [int(o) for o in rng.integers(start + gb, len(body), 80)])
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
