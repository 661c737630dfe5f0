"""Whole graphs through the planner (graph-level C ABI) vs the oracle interpreter."""
import numpy as np
import pytest

from interp import evaluate

pytestmark = pytest.mark.gpu


def test_conv_block_config1(orc):
    """benchmark configuration 1: [1,64,56,56] -> FQ u8 -> 3x3 conv (i8 per-channel W) -> bias -> ReLU."""
    from dldt_amd import builders
    g, feeds, _ = builders.conv_block()
    want, _ = evaluate(orc, g.nodes, feeds)
    plan = g.compile()
    assert [s["type"] for s in plan.steps] == ["FakeQuantize", "Convolution", "Result"]
    req = plan.create_request()
    (got,) = req.infer(feeds["data"])
    np.testing.assert_array_equal(got.view(np.uint32), want["out"].view(np.uint32))
    # the quantized input levels held in the arena are the reference's
    q_node = next(i for i, n in enumerate(g.nodes) if n["op"] == "FakeQuantize")
    _, kept = evaluate(orc, g.nodes, feeds, keep=[q_node])
    np.testing.assert_array_equal(req.tensor(q_node), kept[q_node])


@pytest.mark.parametrize("batch", [1, 3])
def test_small_resnet_bit_exact(orc, batch):
    """ResNet-50 v1.5 topology at reduced width/resolution: every quantized activation and the
    f32 logits must equal the oracle's."""
    from dldt_amd import builders
    g, meta = builders.resnet50(batch=batch, res=64, width=16, classes=10, seed=7)
    rng = np.random.default_rng(99)
    x = rng.uniform(0, 1, (batch, 3, 64, 64)).astype(np.float32)
    keep = [a["node"] for a in meta["acts"].values()]
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=keep)
    plan = g.compile()
    req = plan.create_request()
    (got,) = req.infer(x)
    for name, a in meta["acts"].items():
        w = kept[a["node"]]
        have = req.tensor(a["node"], fused_ok=True)
        if have is not None:        # (None: the tensor between two convolutions that the plan runs as one kernel)
            np.testing.assert_array_equal(have.reshape(w.shape), w, err_msg=name)
    np.testing.assert_array_equal(got.view(np.uint32), want["logits"].view(np.uint32))
    # device-resident path gives the same bytes
    import torch
    ins, outs = req.device_buffers()
    ins[0].copy_(torch.from_numpy(x))
    req.infer_device(ins, outs)
    np.testing.assert_array_equal(outs[0].cpu().numpy(), got)


def test_small_resnet_with_u8_image_input(orc):
    """the same topology with input precision U8 (the image bytes are the first FakeQuantize's levels): the plan the
    host-inclusive measurement with u8 blobs runs"""
    from dldt_amd import builders
    g, meta = builders.resnet50(batch=2, res=64, width=16, classes=10, seed=7, u8_input=True)
    x = np.random.default_rng(98).integers(0, 256, (2, 3, 64, 64)).astype(np.uint8)
    keep = [a["node"] for a in meta["acts"].values()]
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=keep)
    plan = g.compile()
    assert plan.inputs[0]["dtype"] == 40
    req = plan.create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(req.tensor(meta["acts"]["input"]["node"]), x)
    for name, a in meta["acts"].items():
        w = kept[a["node"]]
        have = req.tensor(a["node"], fused_ok=True)
        if have is not None:        # (None: the tensor between two convolutions that the plan runs as one kernel)
            np.testing.assert_array_equal(have.reshape(w.shape), w, err_msg=name)
        assert len(np.unique(w)) > 50, name                 # the calibrated ranges are used, not saturated
    np.testing.assert_array_equal(got.view(np.uint32), want["logits"].view(np.uint32))


def test_planner_reports_unsupported_nodes():
    from dldt_amd import HipieError
    from dldt_amd.graph import Graph
    g = Graph()
    x = g.parameter("x", (1, 8, 4, 4))
    y = g.gelu(x)                                   # Gelu of a 4-D value: it is planned on the row-major path only
    g.result(y, "y")
    with pytest.raises(HipieError) as e:
        g.compile()
    assert e.value.status == -2 and "Gelu" in str(e.value)


def test_small_mobilenet_v2_bit_exact(orc):
    """MobileNetV2 topology (config 4) at reduced width/resolution: pointwise MFMA convs, depthwise
    GroupConvolutions, ReLU6 (Clamp), signed i8 bottleneck outputs, residual adds."""
    from dldt_amd import builders
    g, meta = builders.mobilenet_v2(batch=2, res=64, width=0.5, classes=10, last=128, seed=3)
    x = np.random.default_rng(4).uniform(0, 1, (2, 3, 64, 64)).astype(np.float32)
    keep = [a["node"] for a in meta["acts"].values()]
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=keep)
    plan = g.compile()
    assert any(s["type"] == "GroupConvolution" for s in plan.steps)
    req = plan.create_request()
    (got,) = req.infer(x)
    for name, a in meta["acts"].items():
        w = kept[a["node"]]
        have = req.tensor(a["node"], fused_ok=True)
        if have is None:
            continue
        have = have.reshape(w.shape)
        if w.dtype == np.int8:      # signed levels are stored as they are
            have = have.view(np.int8)
        np.testing.assert_array_equal(have, w, err_msg=name)
    np.testing.assert_array_equal(got.view(np.uint32), want["logits"].view(np.uint32))


@pytest.mark.parametrize("net", ["resnet50", "mobilenet_v2"])
def test_full_size_batch_consistency(net):
    """Full-size networks (224x224, width 1.0) at a batch the oracle would take a while for: every image's
    logits in a batch-16 inference must equal, bit for bit, the logits of the same image inferred
    alone.  The two plans differ in tile counts, in the kernel variants the tuner picks and in which
    tiles are partial, so this pins the full-size indexing that the reduced networks cannot reach."""
    from dldt_amd import builders
    build = getattr(builders, net)
    rng = np.random.default_rng(2024)
    x = rng.uniform(0, 1, (16, 3, 224, 224)).astype(np.float32)
    g16, _ = build(batch=16, res=224)
    (y16,) = g16.compile().create_request().infer(x)
    assert np.isfinite(y16).all() and not np.array_equal(y16[0], y16[7])   # the images do differ
    g1, _ = build(batch=1, res=224)
    req1 = g1.compile().create_request()
    for i in (0, 7, 15):
        (y1,) = req1.infer(x[i:i + 1])
        np.testing.assert_array_equal(y1.view(np.uint32), y16[i:i + 1].view(np.uint32), err_msg="image %d" % i)


@pytest.mark.parametrize("net", ["resnet50", "mobilenet_v2"])
def test_full_size_logits_match_oracle(orc, net):
    """Full-size networks (224x224, width 1.0), two images: the dequantised f32 logits equal the oracle's bit
    for bit, hence zero deviation relative to the output range and the same top-1 class for every image."""
    from dldt_amd import builders
    g, _ = getattr(builders, net)(batch=2, res=224)
    x = np.random.default_rng(77).uniform(0, 1, (2, 3, 224, 224)).astype(np.float32)
    (got,) = g.compile().create_request().infer(x)
    want, _ = evaluate(orc, g.nodes, {"data": x}, keep=[])
    np.testing.assert_array_equal(got.view(np.uint32), want["logits"].view(np.uint32))
    assert (got.argmax(axis=1) == want["logits"].argmax(axis=1)).all()
    assert np.ptp(want["logits"]) > 0


def test_requests_in_flight_do_not_disturb_each_other(orc):
    """Three requests of one plan on their own streams and arenas, fed different images and kept in
    flight together (the throughput mode bench.py measures): every result equals the oracle's for the same
    image, and so does the result of a request that runs alone."""
    import torch
    from dldt_amd import builders
    g, _ = builders.resnet50(batch=4, res=96, width=32, classes=16, seed=5)
    plan = g.compile()
    rng = np.random.default_rng(6)
    xs = [rng.uniform(0, 1, (4, 3, 96, 96)).astype(np.float32) for _ in range(3)]
    want = [evaluate(orc, g.nodes, {"data": x})[0]["logits"] for x in xs]
    alone = plan.create_request()
    for x, w in zip(xs, want):
        np.testing.assert_array_equal(alone.infer(x)[0].view(np.uint32), w.view(np.uint32))
    reqs = [plan.create_request() for _ in xs]
    bufs = [r.device_buffers() for r in reqs]
    for (ins, _), x in zip(bufs, xs):
        ins[0].copy_(torch.from_numpy(x))
    torch.cuda.synchronize()
    for _ in range(5):                      # several rounds back to back, nothing waits in between
        for r, (ins, outs) in zip(reqs, bufs):
            r.enqueue(ins, outs)
    for r in reqs:
        torch.cuda.ExternalStream(r.stream).synchronize()
    for (_, outs), w in zip(bufs, want):
        np.testing.assert_array_equal(outs[0].cpu().numpy().view(np.uint32), w.view(np.uint32))


@pytest.mark.parametrize("c,hw", [(64, 56), (3, 32), (20, 9), (128, 28), (320, 6)])
def test_u8_graph_input(orc, c, hw):
    """input precision U8: Parameter(u8) -> Convert(f32) -> FakeQuantize runs as one entry kernel that
    reads the bytes (image-like 4-byte pixels, 64-channel tiles, whole-pixel tiles from 128 channels up, ragged
    channels and widths)"""
    from dldt_amd import builders
    g, feeds, _ = builders.conv_block(seed=5, n=2, c=c, hw=hw, oc=32, u8_input=True)
    want, _ = evaluate(orc, g.nodes, feeds)
    plan = g.compile()
    assert [s["type"] for s in plan.steps] == ["FakeQuantize", "Convolution", "Result"]
    assert plan.inputs[0]["dtype"] == 40
    req = plan.create_request()
    (got,) = req.infer(feeds["data"])
    np.testing.assert_array_equal(got.view(np.uint32), want["out"].view(np.uint32))
    q_node = next(i for i, n in enumerate(g.nodes) if n["op"] == "FakeQuantize")
    np.testing.assert_array_equal(req.tensor(q_node), feeds["data"])       # levels 0 .. 255 are the input bytes


def test_compile_and_infer_from_many_threads(orc):
    """LoadNetwork and Infer are called concurrently from many threads (behavior/core_threading_tests.hpp):
    four host threads each compile their own plan of the same graph and run host-path inferences on their
    own requests at the same time; a fifth provokes errors meanwhile (the error text is per thread).
    Every result equals the single-threaded one."""
    import threading
    from dldt_amd import HipieError, builders
    from dldt_amd.graph import Graph
    g, _ = builders.resnet50(batch=2, res=64, width=16, classes=10, seed=7)
    rng = np.random.default_rng(8)
    xs = [rng.uniform(0, 1, (2, 3, 64, 64)).astype(np.float32) for _ in range(4)]
    ref_req = g.compile().create_request()
    want = [ref_req.infer(x)[0].copy() for x in xs]
    got, errors = [None] * 4, []

    def worker(i):
        try:
            req = g.compile().create_request()
            for _ in range(6):
                (y,) = req.infer(xs[i])
            got[i] = y
        except Exception as e:                                 # noqa: BLE001 - reported below
            errors.append(repr(e))

    def troublemaker():
        for _ in range(20):
            bad = Graph()
            bad.result(bad.gelu(bad.parameter("x", (1, 8, 4, 4))), "y")     # Gelu of a 4-D value: not planned
            try:
                bad.compile()
                errors.append("unsupported graph compiled")
            except HipieError as e:
                if "Gelu" not in str(e):
                    errors.append("error text of another thread: %s" % e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)] + [threading.Thread(target=troublemaker)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for y, w in zip(got, want):
        np.testing.assert_array_equal(y.view(np.uint32), w.view(np.uint32))


def test_activation_zero_points(orc):
    """asymmetric activation ranges: u8 levels with an integer zero point subtracted in front of the
    convolution (padding applies behind the Subtract: the padded taps contribute nothing)"""
    from dldt_amd import builders
    g, feeds, meta = builders.zero_point_net()
    keep = [a["node"] for a in meta["acts"].values()]
    want, kept = evaluate(orc, g.nodes, feeds, keep=keep)
    plan = g.compile()
    req = plan.create_request()
    (got,) = req.infer(feeds["data"])
    for name, a in meta["acts"].items():
        np.testing.assert_array_equal(req.tensor(a["node"]), kept[a["node"]], err_msg=name)
        assert kept[a["node"]].min() == 0 and kept[a["node"]].max() == 255      # both ends saturate
    np.testing.assert_array_equal(got.view(np.uint32), want["out"].view(np.uint32))


def test_imported_plan_uploads_the_packed_operands_of_the_stream(orc):
    """Import does not pack weights again: it uploads what the stream holds.  Shown by a stream whose first packed
    matrix was replaced by zeros (and sealed again): the graph description still holds the weights, the imported plan
    computes with the zeros."""
    from dldt_amd import builders
    from dldt_amd.graph import Plan
    from test_plan_stream_cpu import _reseal, sections
    g = builders.conv_block(n=2, c=32, hw=12, oc=32)[0]
    x = np.random.default_rng(5).uniform(0, 2.55, (2, 32, 12, 12)).astype(np.float32)
    names = [n["name"] for n in g.nodes if n["op"] == "Parameter"]
    ref, _ = evaluate(orc, g.nodes, {names[0]: x})
    plan = g.compile()
    blob = plan.export()
    want = plan.create_request().infer(x)[0]
    np.testing.assert_array_equal(want.view(np.uint32), ref[plan.outputs[0]["name"]].view(np.uint32))
    np.testing.assert_array_equal(Plan.load(blob).create_request().infer(x)[0], want)
    _, _, _, blobs = sections(blob)
    off, n = max(blobs, key=lambda b: b[1])              # the packed weight matrix
    zeroed = _reseal(blob[:off] + bytes(n) + blob[off + n:-8])
    got = Plan.load(zeroed).create_request().infer(x)[0]
    assert not np.array_equal(got, want)


@pytest.mark.parametrize("net", ["resnet", "encoder"])
def test_exported_plan_runs_the_same_kernels(orc, net, monkeypatch):
    """ExecutableNetwork::Export -> Plugin::ImportNetwork: the imported plan takes its kernel variants from
    the stream (no timing runs) and gives the oracle's result like the exported plan (bit for bit for the
    convolutional network; the encoder's f32 output within the tolerance its Softmax / MVN / Gelu are held to, and the
    exported plan's own bytes)"""
    from dldt_amd import builders
    from dldt_amd.graph import Plan
    rng = np.random.default_rng(31)
    if net == "resnet":
        g, _ = builders.resnet50(batch=2, res=64, width=16, classes=10, seed=7)
        feeds = [rng.uniform(0, 1, (2, 3, 64, 64)).astype(np.float32)]
    else:
        g, _ = builders.bert_encoder(layers=2, batch=2, seq=64, hidden=128, heads=2, ffn=256, seed=3)
        feeds = [rng.normal(0, 1, (2, 64, 128)).astype(np.float32)]
    names = [n["name"] for n in g.nodes if n["op"] == "Parameter"]
    ref, _ = evaluate(orc, g.nodes, dict(zip(names, feeds)))
    monkeypatch.setenv("HIPIE_TUNE", "0")                # shape-based defaults in the exported plan ...
    plan = g.compile()
    want = plan.create_request().infer(*feeds)
    for o, w in zip(plan.outputs, want):
        if net == "resnet":
            np.testing.assert_array_equal(w.view(np.uint32), ref[o["name"]].view(np.uint32))
        else:
            np.testing.assert_allclose(w, ref[o["name"]].reshape(w.shape), rtol=1e-4, atol=2e-5)
    blob = plan.export()
    variants = [s["variant"] for s in plan.steps]
    assert any(v >= 0 for v in variants)
    monkeypatch.delenv("HIPIE_TUNE")                     # ... which a timing run at import would not keep everywhere
    back = Plan.load(blob)
    assert [s["variant"] for s in back.steps] == variants
    assert [(s["name"], s["type"]) for s in back.steps] == [(s["name"], s["type"]) for s in plan.steps]
    got = back.create_request().infer(*feeds)
    for o, a, b in zip(back.outputs, got, want):
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
        if net == "resnet":
            np.testing.assert_array_equal(a.view(np.uint32), ref[o["name"]].view(np.uint32))
    tuned = g.compile()                                  # and the other way round: tuned choices survive HIPIE_TUNE=0
    blob = tuned.export()
    monkeypatch.setenv("HIPIE_TUNE", "0")
    assert [s["variant"] for s in Plan.load(blob).steps] == [s["variant"] for s in tuned.steps]
    monkeypatch.delenv("HIPIE_TUNE")
    # a stream exported without a device (dry run) imports too: its steps carry no choices, the plan is tuned here
    dry = Plan.load(g.compile(-1).export())
    for a, b in zip(dry.create_request().infer(*feeds), want):
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))


def test_asynchronous_requests_from_page_locked_blobs(orc):
    """StartAsync / Wait over the request's own page-locked blobs, three requests in flight with different
    images (benchmark_app's loop): results equal the oracle's (and the synchronous host path's); a started request
    is busy, and waiting on an idle one is an error"""
    from dldt_amd import HipieError, builders
    g, _ = builders.resnet50(batch=4, res=96, width=32, classes=16, seed=5)
    plan = g.compile()
    rng = np.random.default_rng(12)
    xs = [rng.uniform(0, 1, (4, 3, 96, 96)).astype(np.float32) for _ in range(7)]
    want = [evaluate(orc, g.nodes, {"data": x})[0]["logits"] for x in xs]
    sync = plan.create_request()
    for x, w in zip(xs[:2], want):
        np.testing.assert_array_equal(sync.infer(x)[0].view(np.uint32), w.view(np.uint32))
    reqs = [plan.create_request() for _ in range(3)]
    blobs = [r.host_buffers() for r in reqs]
    got = [None] * len(xs)
    running = {}
    for i, x in enumerate(xs):
        k = i % 3
        if k in running:
            reqs[k].wait()
            got[running.pop(k)] = blobs[k][1][0].array.copy()
        blobs[k][0][0].array[...] = x
        reqs[k].start(*blobs[k])
        running[k] = i
    with pytest.raises(HipieError) as e:                 # REQUEST_BUSY: already started
        reqs[0].start(*blobs[0])
    assert e.value.status == -8
    for k, i in running.items():
        reqs[k].wait()
        got[i] = blobs[k][1][0].array.copy()
    with pytest.raises(HipieError) as e:                 # INFER_NOT_STARTED
        reqs[0].wait()
    assert e.value.status == -11
    for a, b in zip(got, want):
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("net", ["resnet50", "mobilenet_v2"])
def test_full_size_batch_64(orc, net):
    """The benchmarked configurations at their stated size (224x224, width 1.0, batch 64): the logits of four images
    of a batch-64 inference equal, bit for bit, those of the same images inferred alone, and for two of them the
    oracle's f32 logits (same top-1 class, zero deviation)."""
    from dldt_amd import builders
    build = getattr(builders, net)
    rng = np.random.default_rng(64)
    x = rng.uniform(0, 1, (64, 3, 224, 224)).astype(np.float32)
    g64, _ = build(batch=64, res=224)
    (y64,) = g64.compile().create_request().infer(x)
    assert np.isfinite(y64).all() and len({y64[i].tobytes() for i in range(64)}) == 64   # 64 different images, 64 different results
    g1, _ = build(batch=1, res=224)
    req1 = g1.compile().create_request()
    for i in (0, 21, 42, 63):
        (y1,) = req1.infer(x[i:i + 1])
        np.testing.assert_array_equal(y1.view(np.uint32), y64[i:i + 1].view(np.uint32), err_msg="image %d" % i)
    for i in (0, 63):
        want, _ = evaluate(orc, g1.nodes, {"data": x[i:i + 1]}, keep=[])
        np.testing.assert_array_equal(y64[i:i + 1].view(np.uint32), want["logits"].view(np.uint32), err_msg="image %d" % i)
        assert y64[i].argmax() == want["logits"][0].argmax()


def test_timed_wait_status_only_and_cancel():
    """Wait(ms) and Cancel of the asynchronous request (ie_infer_async_request_thread_safe_default.hpp:167-204, 255-267):
    STATUS_ONLY on a running inference says RESULT_NOT_READY and leaves it running, a timed wait returns the result, a
    cancelled inference reports INFER_CANCELLED once and leaves the request idle and usable."""
    from dldt_amd import HipieError, builders
    g, _ = builders.resnet50(batch=64, res=224)
    plan = g.compile(config={"HIP_TUNE": "NO", "PERF_COUNT": "YES"})
    assert plan.config("PERF_COUNT") == "YES"
    x = np.random.default_rng(21).uniform(0, 1, (64, 3, 224, 224)).astype(np.float32)
    (want,) = plan.create_request().infer(x)
    req = plan.create_request(perf_count=None)            # the plan's PERF_COUNT
    ins, outs = req.host_buffers()
    ins[0].array[...] = x
    with pytest.raises(HipieError) as e:                  # idle: INFER_NOT_STARTED
        req.wait_for(0)
    assert e.value.status == -11
    req.start(ins, outs)
    not_ready = 0
    while True:                                           # STATUS_ONLY until it is done
        try:
            req.wait_for(0)
            break
        except HipieError as err:
            assert err.status == -9
            not_ready += 1
    assert not_ready > 0                                  # 38 MB over the host link and 54 kernels were not done at once
    np.testing.assert_array_equal(outs[0].array.view(np.uint32), want.view(np.uint32))
    assert sum(s["ms"] for s in req.perf()) > 0           # the per-step counters of PERF_COUNT = YES
    outs[0].array[...] = 0
    req.start(ins, outs)
    req.wait_for(60000)
    np.testing.assert_array_equal(outs[0].array.view(np.uint32), want.view(np.uint32))
    req.start(ins, outs)
    req.cancel()
    with pytest.raises(HipieError) as e:
        req.wait()
    assert e.value.status == -13                          # INFER_CANCELLED, after the queued work has drained
    with pytest.raises(HipieError) as e:                  # idle again
        req.wait()
    assert e.value.status == -11
    req.cancel()                                          # nothing to cancel: no effect
    outs[0].array[...] = 0
    req.start(ins, outs)
    req.wait()
    np.testing.assert_array_equal(outs[0].array.view(np.uint32), want.view(np.uint32))
    # Cancel from another thread while this one is blocked inside Wait(RESULT_READY): the wait reports INFER_CANCELLED
    # (AsyncInferRequestThreadSafeDefault does the same in that window) and the request is idle afterwards
    import threading
    import time
    seen = []
    for _ in range(10):
        status = []

        def waiter():
            try:
                req.wait()
                status.append(0)
            except HipieError as err:
                status.append(err.status)

        req.start(ins, outs)
        t = threading.Thread(target=waiter)
        t.start()
        time.sleep(0.0002)                                # the copy of 38 MB alone takes longer
        req.cancel()
        t.join()
        assert status[0] in (0, -13)                      # (0: the inference had ended before the Cancel arrived)
        seen.append(status[0])
        with pytest.raises(HipieError) as e:
            req.wait()
        assert e.value.status == -11
        if status[0] == -13:
            break
    assert -13 in seen


@pytest.mark.parametrize("branches,signed", [((24, 40, 16), False), ((64, 64), False), ((7, 33, 5, 19), False), ((32, 16), True)])
def test_concat_of_quantized_branches(orc, branches, signed):
    """Concat of u8 / i8 branches with one shared interval (what ConcatTransformation leaves): the levels side by side,
    bit-exact, whatever the slices' alignment; a padded convolution reads the concatenated tensor"""
    from dldt_amd import builders
    g, feeds, meta = builders.concat_net(branches=branches, signed=signed)
    want, kept = evaluate(orc, g.nodes, feeds, keep=[meta["concat"]])
    plan = g.compile()
    assert [s["type"] for s in plan.steps].count("Concat") == 1
    req = plan.create_request()
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(feeds["data"])))
    np.testing.assert_array_equal(req.tensor(meta["concat"]), kept[meta["concat"]])
    for name in ("cat", "out"):
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    # a second inference into the same arena: the slices are rewritten, nothing is left from the first
    other = np.random.default_rng(5).uniform(0, 1, feeds["data"].shape).astype(np.float32)
    want2, _ = evaluate(orc, g.nodes, dict(data=other))
    got2 = dict(zip([o["name"] for o in plan.outputs], req.infer(other)))
    np.testing.assert_array_equal(got2["out"].view(np.uint32), want2["out"].view(np.uint32))


def _flattened_map_net(shape, oc, levels, seed=77):
    from dldt_amd import builders
    N, C, H, W = shape
    rng = np.random.default_rng(seed + oc)
    x = rng.uniform(0, 1, (N, 8, 2 * H - 1, 2 * W - 1)).astype(np.float32)
    rnd = lambda s, scale: (rng.standard_normal(s, dtype=np.float32) * np.float32(scale)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    w0, b0 = rnd((C, 8, 3, 3), 0.1), rnd(C, 0.2)
    if levels == "zero point":
        a1 = net.asymmetric(net.conv_f32(a0, w0, b0, strides=(2, 2), pads=(1, 1)), -0.7, 1.3)
    else:
        a1 = net.conv(a0, w0, b0, 2.0, strides=(2, 2), pads=(1, 1), signed=levels == "i8")
    flat = dict(a1, node=g.reshape(a1["node"], (N, C * H * W)))
    g.result(net.conv_f32(flat, rnd((oc, C * H * W), 0.05), rnd(oc, 0.2), matmul=True, relu=True), "fc")
    return g, x, a1["node"]


@pytest.mark.parametrize("shape,oc,levels", [((3, 32, 5, 6), 50, "u8"), ((2, 24, 7, 7), 130, "i8"), ((4, 16, 3, 4), 10, "zero point"),
                                             ((64, 128, 7, 7), 1000, "u8")])
def test_fully_connected_layer_behind_a_flattened_feature_map(orc, shape, oc, levels):
    """u8 / i8 feature map [N, C, H, W] -> Reshape [N, C * H * W] -> MatMul with i8 weights (a classifier without a global
    pool in front, VGG / AlexNet style): the bytes stay where they are and the MatMul runs as the convolution with an
    H x W filter that it is equal to; bit-exact, also where the activations carry a zero point"""
    g, x, a1 = _flattened_map_net(shape, oc, levels)
    N, C, H, W = shape
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=[a1])
    assert kept[a1].shape == shape
    plan = g.compile()
    types = [s["type"] for s in plan.steps]
    assert types[-2:] == ["MatMul", "Result"] and plan.steps[-2]["macs"] == N * oc * C * H * W
    req = plan.create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(req.tensor(a1), kept[a1])
    assert got.shape == (N, oc)
    np.testing.assert_array_equal(got.view(np.uint32), want["fc"].view(np.uint32))


@pytest.mark.parametrize("axis", [0, 2, 3, -1])
@pytest.mark.parametrize("quantized", [True, False])
def test_concat_along_the_batch_and_the_spatial_axes(orc, axis, quantized):
    """Concat along N, H or W: every input lands in its box of the output (boxes of unequal extent along H and W);
    u8 branches with one shared interval and f32 branches, and a padded convolution that reads across the seam"""
    from dldt_amd import builders
    rng = np.random.default_rng(300 + axis)
    x = rng.uniform(0, 1, (2, 12, 11, 13)).astype(np.float32)
    ax = axis % 4
    kernels = [(1, 1), (3, 1) if ax == 2 else ((1, 3) if ax == 3 else (1, 1)), (1, 1)]
    net = builders.QuantizedNet()
    g = net.g
    branches = []
    if quantized:
        a0 = net.input("data", x.shape, 1.0)
        for k in kernels:
            w = (rng.standard_normal((20, 12) + k, dtype=np.float32) * np.float32(0.15)).astype(np.float32)
            b = (rng.standard_normal(20, dtype=np.float32) * np.float32(0.3)).astype(np.float32)
            branches.append(net.conv(a0, w, b, 2.5))
        cat = dict(node=g.concat([a["node"] for a in branches], axis=axis), scale=branches[0]["scale"])
        node = cat["node"]
        g.result(net.dequantize(cat), "cat")
        w = (rng.standard_normal((24, 20, 3, 3), dtype=np.float32) * np.float32(0.05)).astype(np.float32)
        g.result(net.conv_f32(cat, w, np.zeros(24, np.float32), pads=(1, 1)), "out")
    else:
        p = g.parameter("data", x.shape)
        for k in kernels:
            w = (rng.standard_normal((20, 12) + k, dtype=np.float32) * np.float32(0.15)).astype(np.float32)
            branches.append(g.relu(g.convolution(p, g.constant(w))))
        node = g.concat(branches, axis=axis)
        g.result(node, "cat")
        g.result(g.max_pool(node, (3, 3), (1, 1), (1, 1), (1, 1)), "out")
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=[node])
    assert want["cat"].shape[ax] == {0: 6, 2: 31, 3: 37}[ax]
    plan = g.compile()
    assert [s["type"] for s in plan.steps].count("Concat") == 1
    req = plan.create_request()
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(x)))
    np.testing.assert_array_equal(req.tensor(node).view(np.uint8), kept[node].view(np.uint8))
    for name in ("cat", "out"):
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    assert all(g.query())


def test_elementwise_broadcast_between_tensors(orc):
    """Multiply / Add of a feature map with a value that has one element along the batch or the spatial axes: a
    per-image, per-channel gate [N, C, 1, 1] (a squeeze-and-excitation block's), a map [1, C, H, W] shared by the batch
    and a row [N, C, 1, W]; operands on either side, dequantized bytes and f32"""
    from dldt_amd import builders
    rng = np.random.default_rng(311)
    x = rng.uniform(0, 1, (3, 16, 9, 10)).astype(np.float32)
    shared = rng.uniform(-1, 1, (1, 16, 9, 10)).astype(np.float32)
    row = rng.uniform(-1, 1, (3, 16, 1, 10)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    w = (rng.standard_normal((16, 16, 3, 3), dtype=np.float32) * np.float32(0.08)).astype(np.float32)
    b = (rng.standard_normal(16, dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    fmap = net.conv(a0, w, b, 2.0, pads=(1, 1))                         # u8 feature map
    # squeeze: global average of the dequantized map, a 1 x 1 convolution on it, its result [N, C, 1, 1] in f32
    pooled = g.avg_pool(net.dequantize(fmap), (9, 10), (1, 1), (0, 0), (0, 0), exclude_pad=False)
    wg = (rng.standard_normal((16, 16, 1, 1), dtype=np.float32) * np.float32(0.4)).astype(np.float32)
    gate = g.relu(g.convolution(pooled, g.constant(wg)))
    gated = g.multiply(net.dequantize(fmap), gate)                      # [N, C, H, W] * [N, C, 1, 1]
    q = net.requantize(gated, 1.5)
    g.result(net.dequantize(q), "gated")
    ps = g.parameter("shared", shared.shape)
    pr = g.parameter("row", row.shape)
    g.result(g.add(ps, net.dequantize(fmap)), "plus_shared")            # the small operand first
    g.result(g.subtract(net.dequantize(fmap), pr), "minus_row")
    g.result(g.multiply(ps, pr), "outer")                               # both sides repeat: [1,C,H,W] * [N,C,1,W]
    feeds = {"data": x, "shared": shared, "row": row}
    want, kept = evaluate(orc, g.nodes, feeds, keep=[q["node"]])
    plan = g.compile()
    req = plan.create_request()
    order = [feeds[i["name"]] for i in plan.inputs]
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(*order)))
    assert len(np.unique(kept[q["node"]])) > 30
    np.testing.assert_array_equal(req.tensor(q["node"]), kept[q["node"]])
    for name in ("gated", "plus_shared", "minus_row", "outer"):
        assert got[name].shape == want[name].shape == (3, 16, 9, 10)
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    assert all(g.query())


def test_convolutions_over_one_spatial_dimension(orc):
    """[N, C, W] values: quantized Convolution (stride, dilation, padding), depthwise GroupConvolution, MaxPool and
    AvgPool with filters and windows over the one axis, and an f32 convolution of the graph input - planned as the
    same layers over [N, C, 1, W], bit-exact against the oracle's own one-dimensional loops; the plan's inputs and
    outputs keep their rank, and an exported plan brings the description back as it was"""
    from dldt_amd import builders
    from dldt_amd.graph import Plan
    rng = np.random.default_rng(71)
    x = rng.uniform(0, 1, (3, 16, 50)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    rnd = lambda shape, s: (rng.standard_normal(shape, dtype=np.float32) * np.float32(s)).astype(np.float32)
    a1 = net.conv(a0, rnd((32, 16, 5), 0.1), rnd(32, 0.2), 2.0, strides=(2,), pads=(2,), dilations=(1,))
    a2 = net.conv(a1, rnd((32, 1, 3), 0.3), rnd(32, 0.2), 2.0, strides=(1,), pads=(2,), dilations=(2,), grouped=True)
    a3 = net.max_pool(a2, (3,), (2,), (1,))
    y = net.conv_f32(a3, rnd((24, 32, 3), 0.06), rnd(24, 0.1), strides=(1,), pads=(1,), relu=True)
    g.result(y, "out")
    g.result(g.avg_pool(net.dequantize(a3), (13,), (1,), (0,), (0,)), "mean")
    p = g.nodes[g.nodes[a0["node"]]["inputs"][0]]
    assert p["op"] == "Parameter"
    f32 = g.relu(g.convolution(g.nodes[a0["node"]]["inputs"][0], g.constant(rnd((8, 16, 4), 0.2)), strides=(3,), dilations=(2,),
                               pads_begin=(1,), pads_end=(2,)))
    g.result(f32, "f32")
    keep = [a1["node"], a2["node"], a3["node"]]
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=keep)
    assert want["out"].shape == (3, 24, 13) and want["mean"].shape == (3, 32, 1) and want["f32"].ndim == 3
    plan = g.compile()
    assert [tuple(i["shape"]) for i in plan.inputs] == [x.shape]
    assert {o["name"]: tuple(o["shape"]) for o in plan.outputs} == {k: v.shape for k, v in want.items()}
    again = Plan.load(plan.export())
    for pl in (plan, again):
        req = pl.create_request()
        got = dict(zip([o["name"] for o in pl.outputs], req.infer(x)))
        for node in keep:
            assert len(np.unique(kept[node])) > 40
            np.testing.assert_array_equal(req.tensor(node)[:, :, 0, :], kept[node])
        for name in want:
            np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    assert all(g.query())


def test_split_of_quantized_and_f32_values(orc):
    """a channel-split unit: the u8 levels of a convolution split along the channels, one half through another
    quantized convolution, the halves concatenated again and convolved; an f32 feature map split along its rows; a
    split of dequantized levels with per-channel scales (every part keeps its own channels' scales)"""
    from dldt_amd import builders
    rng = np.random.default_rng(404)
    x = rng.uniform(0, 1, (2, 16, 12, 10)).astype(np.float32)
    rnd = lambda shape, s: (rng.standard_normal(shape, dtype=np.float32) * np.float32(s)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    a1 = net.conv(a0, rnd((48, 16, 3, 3), 0.08), rnd(48, 0.2), 2.5, pads=(1, 1))
    left, right = [dict(node=n, scale=a1["scale"]) for n in g.split(a1["node"], 1, 2, 48)]
    worked = net.conv(right, rnd((24, 24, 3, 3), 0.07), rnd(24, 0.2), 2.5, pads=(1, 1))
    assert worked["scale"] == a1["scale"]
    cat = dict(node=g.concat([left["node"], worked["node"]], axis=1), scale=a1["scale"])
    g.result(net.conv_f32(cat, rnd((20, 48, 1, 1), 0.1), rnd(20, 0.1)), "out")
    f = net.conv_f32(a0, rnd((6, 16, 1, 1), 0.3), rnd(6, 0.1))
    for k, piece in enumerate(g.split(f, 2, 3, 12)):
        g.result(piece, "rows%d" % k)
    deq = g.multiply(g.convert(a1["node"], 10), g.constant(rng.uniform(0.5, 2, (1, 48, 1, 1)).astype(np.float32)))
    for k, piece in enumerate(g.split(deq, 1, 3, 48)):
        g.result(piece, "scaled%d" % k)
    keep = [left["node"], right["node"], worked["node"], cat["node"]]
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=keep)
    plan = g.compile()
    assert [s["type"] for s in plan.steps].count("Split") == 2 + 3 + 3
    req = plan.create_request()
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(x)))
    for node in keep:
        np.testing.assert_array_equal(req.tensor(node), kept[node])
    for name in want:
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    assert all(g.query())


def test_prelu_between_a_quantized_convolution_and_its_fake_quantize(orc):
    """what PReluTransformation leaves (prelu.cpp:39-47: the dequantization Multiply moves behind the PRelu and the
    FakeQuantize that follows absorbs it): Conv' -> Add(b') -> PRelu(slope[C]) -> FakeQuantize with per-channel input
    ranges -> i8 levels; a leaky ReLU (scalar slope) on dequantized levels; a [1, C, 1, 1] slope on an f32 value"""
    from dldt_amd import builders, lpt
    rng = np.random.default_rng(909)
    x = rng.uniform(0, 1, (2, 16, 12, 10)).astype(np.float32)
    rnd = lambda shape, s: (rng.standard_normal(shape, dtype=np.float32) * np.float32(s)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    y, s, rank = net._accumulate(a0, rnd((24, 16, 3, 3), 0.08), rnd(24, 0.3),
                                 dict(strides=(1, 1), dilations=(1, 1), pads_begin=(1, 1), pads_end=(1, 1)))
    y = g.prelu(y, g.constant(rng.uniform(0.05, 0.3, 24).astype(np.float32)))          # [C]: one slope per channel
    lo, hi = net.signed_range(2.0)
    d = lpt.decompose_fake_quantize(256, lo, hi)
    il, ih = lpt.fuse_elementwise(lpt.MULTIPLY, lo, hi, s)
    q = g.fake_quantize(y, net._channel(il, rank), net._channel(ih, rank), d["new_low"], d["new_high"], 256, d["precision"])
    a1 = dict(node=q, scale=np.float32(d["scale"]))
    g.result(net.conv_f32(a1, rnd((8, 24, 1, 1), 0.1), rnd(8, 0.1)), "out")
    g.result(g.prelu(net.dequantize(a1), g.constant(np.float32(0.1))), "leaky")
    f = net.conv_f32(a0, rnd((6, 16, 1, 1), 0.3), rnd(6, 0.2))
    g.result(g.prelu(f, g.constant(rng.uniform(-0.5, 0.5, (1, 6, 1, 1)).astype(np.float32))), "per_channel")
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=[q])
    levels = kept[q].astype(np.int32)
    assert len(np.unique(levels)) > 80 and 0.2 < (levels < 0).mean() < 0.8
    plan = g.compile()
    assert "PRelu+FakeQuantize" in [s["type"] for s in plan.steps]
    req = plan.create_request()
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(x)))
    np.testing.assert_array_equal(req.tensor(q), kept[q])
    for name in want:
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    assert all(g.query())


def test_hswish_sigmoid_swish_blocks(orc):
    """the activations the low-precision transformations leave in f32 between a quantized convolution's dequantization
    and the next FakeQuantize: Conv' -> Add -> Multiply -> HSwish -> FakeQuantize (bit-exact: every operation of
    hswish.hpp is an IEEE f32 operation), an HSigmoid gate on a pooled value multiplied back onto the feature map (a
    MobileNetV3 squeeze-and-excitation block), and Sigmoid / Swish, which use the device's exp: their f32 results to
    rounding, and the quantized layers behind them bit-exact from the device's own values"""
    from dldt_amd import builders
    rng = np.random.default_rng(515)
    x = rng.uniform(0, 1, (2, 16, 10, 12)).astype(np.float32)
    rnd = lambda shape, s: (rng.standard_normal(shape, dtype=np.float32) * np.float32(s)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    hs = g.hswish(net.conv_f32(a0, rnd((24, 16, 3, 3), 0.12), rnd(24, 0.5), pads=(1, 1)))
    a1 = net.requantize(hs, 3.0, signed=True)                     # i8: HSwish goes down to -0.375
    g.result(net.dequantize(a1), "hswish_levels")
    # squeeze-and-excitation with an HSigmoid gate
    pooled = g.avg_pool(net.dequantize(a1), (10, 12), (1, 1), (0, 0), (0, 0))
    gate = g.hsigmoid(g.convolution(pooled, g.constant(rnd((24, 24, 1, 1), 0.8))))
    a2 = net.requantize(g.multiply(net.dequantize(a1), gate), 3.0, signed=True)
    g.result(net.conv_f32(a2, rnd((8, 24, 1, 1), 0.1), rnd(8, 0.1)), "out")
    f = net.conv_f32(a0, rnd((12, 16, 1, 1), 0.6), rnd(12, 0.5))
    sg, sw = g.sigmoid(f), g.swish(f, 0.6)
    g.result(sg, "sigmoid")
    g.result(sw, "swish")
    a3 = net.requantize(sw, 2.0, signed=True)
    g.result(net.conv_f32(a3, rnd((6, 12, 1, 1), 0.2), rnd(6, 0.1)), "behind_swish")
    keep = [hs, a1["node"], gate, a2["node"], a3["node"]]
    plan = g.compile()
    types = [s["type"] for s in plan.steps]
    assert "HSwish+FakeQuantize" in types and "HSigmoid" in types and "Sigmoid" in types
    req = plan.create_request()
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(x)))
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=keep)
    assert kept[hs].min() < -0.3 and len(np.unique(kept[a1["node"]])) > 80
    for node in (a1["node"], a2["node"]):
        np.testing.assert_array_equal(req.tensor(node), kept[node])
    np.testing.assert_array_equal(req.tensor(gate).view(np.uint32), kept[gate].view(np.uint32))
    for name in ("hswish_levels", "out"):
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    np.testing.assert_allclose(got["sigmoid"], want["sigmoid"], rtol=3e-7, atol=0)
    np.testing.assert_allclose(got["swish"], want["swish"], rtol=5e-7, atol=1e-9)
    # what follows the Swish, from the device's own Swish
    want2, kept2 = evaluate(orc, g.nodes, {"data": x}, keep=[a3["node"]], override={sw: got["swish"]})
    np.testing.assert_array_equal(req.tensor(a3["node"]), kept2[a3["node"]])
    np.testing.assert_array_equal(got["behind_swish"].view(np.uint32), want2["behind_swish"].view(np.uint32))
    assert all(g.query())


@pytest.mark.parametrize("stride", [1, 2])
def test_per_channel_activation_zero_points(orc, stride):
    """one integer zero point per channel in front of a padded depthwise convolution: the halo holds every channel's
    own level, the accumulators start from each channel's own correction"""
    from dldt_amd import builders
    g, feeds, meta = builders.per_channel_zero_point_net(stride=stride)
    keep = [a["node"] for a in meta["acts"].values()]
    want, kept = evaluate(orc, g.nodes, feeds, keep=keep)
    plan = g.compile()
    req = plan.create_request()
    (got,) = req.infer(feeds["data"])
    for name, a in meta["acts"].items():
        np.testing.assert_array_equal(req.tensor(a["node"]), kept[a["node"]], err_msg=name)
    np.testing.assert_array_equal(got.view(np.uint32), want["out"].view(np.uint32))


def test_stand_alone_elementwise_nodes(orc):
    """Add / Multiply / Subtract / Relu / Clamp / FakeQuantize that no convolution absorbs run as steps of their own,
    with the activation and the FakeQuantize behind them in the same kernel; bit-exact"""
    from dldt_amd import builders
    g, feeds, meta = builders.eltwise_net()
    keep = [a["node"] for a in meta["acts"].values()]
    want, kept = evaluate(orc, g.nodes, feeds, keep=keep)
    plan = g.compile()
    types = [s["type"] for s in plan.steps]
    assert "Add+FakeQuantize" in types and "Multiply" in types and "Subtract" in types and types.count("FakeQuantize") == 2
    req = plan.create_request()
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(feeds["data"])))
    for name, a in meta["acts"].items():
        w = kept[a["node"]]
        assert len(np.unique(w)) > 50
        np.testing.assert_array_equal(req.tensor(a["node"]).astype(np.int16), w.astype(np.int16), err_msg=name)
    for name in ("prod", "left"):
        np.testing.assert_array_equal(got[name].view(np.uint32), want[name].view(np.uint32), err_msg=name)
    assert all(g.query())


def test_grouped_convolution_in_a_graph(orc):
    """a GroupConvolution with four channels per group between two dense convolutions, through the planner"""
    from dldt_amd import builders
    from dldt_amd.builders import QuantizedNet
    rng = np.random.default_rng(61)
    n, c, hw, groups = 2, 32, 12, 8
    x = rng.uniform(0, 1, (n, c, hw, hw)).astype(np.float32)
    net = QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    wn = lambda *s, k=0.1: (rng.standard_normal(s, dtype=np.float32) * np.float32(k)).astype(np.float32)
    a1 = net.conv(a0, wn(64, c, 1, 1), wn(64, k=0.2), 2.0)
    a2 = net.conv(a1, wn(64, 64 // groups, 3, 3, k=0.15), wn(64, k=0.2), 2.5, pads=(1, 1), groups=groups)
    g.result(net.conv_f32(a2, wn(40, 64, 1, 1), wn(40, k=0.2)), "out")
    want, kept = evaluate(orc, g.nodes, dict(data=x), keep=[a2["node"]])
    plan = g.compile()
    assert [s["type"] for s in plan.steps].count("GroupConvolution") == 1
    req = plan.create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(req.tensor(a2["node"]), kept[a2["node"]])
    np.testing.assert_array_equal(got.view(np.uint32), want["out"].view(np.uint32))


@pytest.mark.parametrize("groups,width", [(32, 128), (8, 256)])
def test_resnext_block_through_the_planner(orc, groups, width):
    """a ResNeXt bottleneck (1 x 1 reduce, grouped 3 x 3 with cardinality 32 x 4 or 8 x 32, 1 x 1 expand with the residual
    Add): the grouped layer runs in its own form (its step counts a groups-th of the dense multiply-accumulates and is
    tuned over the two 64-channel-tile kernels), everything bit-exact"""
    from dldt_amd.builders import QuantizedNet
    rng = np.random.default_rng(groups)
    n, c, hw = 2, 64, 14
    x = rng.uniform(0, 1, (n, c, hw, hw)).astype(np.float32)
    net = QuantizedNet()
    g = net.g
    wn = lambda *s, k=0.1: (rng.standard_normal(s, dtype=np.float32) * np.float32(k)).astype(np.float32)
    a0 = net.input("data", x.shape, 1.0)
    a1 = net.conv(a0, wn(width, c, 1, 1), wn(width, k=0.2), 2.0)
    a2 = net.conv(a1, wn(width, width // groups, 3, 3, k=0.2), wn(width, k=0.2), 2.5, pads=(1, 1), groups=groups)
    g.result(net.conv_f32(a2, wn(48, width, 1, 1), wn(48, k=0.2)), "out")
    want, kept = evaluate(orc, g.nodes, dict(data=x), keep=[a2["node"]])
    plan = g.compile()
    steps = [s for s in plan.steps if s["type"] == "GroupConvolution"]
    assert len(steps) == 1 and steps[0]["macs"] == n * hw * hw * width * (width // groups) * 9 and steps[0]["variant"] in (1, 2)
    req = plan.create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(req.tensor(a2["node"]), kept[a2["node"]])
    np.testing.assert_array_equal(got.view(np.uint32), want["out"].view(np.uint32))
    blob = plan.export()                                 # the packed grouped operands travel in the stream too
    from dldt_amd.graph import Plan
    (again,) = Plan.load(blob).create_request().infer(x)
    np.testing.assert_array_equal(again.view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("mode", ["YES", "NO", "AUTO"])
def test_bottleneck_tails_as_one_kernel(orc, mode):
    """HIP_FUSE_CONVOLUTIONS: the 3 x 3 convolution of a bottleneck block and the 1 x 1 convolution with the residual add
    behind it as one kernel (YES: wherever the kernel takes the pair - 64 and 128 channels in this net), as two (NO), or
    as the load-time measurement decides (AUTO).  The same bytes in every tensor that reaches memory, and the tensor
    between the two layers is reported as living in LDS only exactly where they run fused."""
    from dldt_amd import builders
    batch = 3
    g, meta = builders.resnet50(batch=batch, res=64, width=32, classes=10, seed=11)
    x = np.random.default_rng(5).uniform(0, 1, (batch, 3, 64, 64)).astype(np.float32)
    keep = [a["node"] for a in meta["acts"].values()]
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=keep)
    plan = g.compile(config={"HIP_FUSE_CONVOLUTIONS": mode})
    types = [s["type"] for s in plan.steps]
    fused, apart = types.count("Convolution+Convolution"), types.count("Convolution,Convolution")
    # width 32: stages of 32, 64, 128 and 256 channels; the tails of the blocks without a convolution in the shortcut
    # of stages 2, 3 and 4 are pairs (3 + 5 + 2)
    assert fused + apart == (0 if mode == "NO" else 10)
    assert (fused, apart) == {"YES": (10, 0), "NO": (0, 0)}.get(mode, (fused, apart))
    assert sum(int(plan.step_rt_info(i, "kernels")) for i in range(len(types))) == 54 - fused
    req = plan.create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(got.view(np.uint32), want["logits"].view(np.uint32))
    missing = 0
    for name, a in meta["acts"].items():
        have = req.tensor(a["node"], fused_ok=True)
        if have is None:
            missing += 1
            assert name.endswith(".b"), name
        else:
            np.testing.assert_array_equal(have.reshape(kept[a["node"]].shape), kept[a["node"]], err_msg=name)
    assert missing == fused
