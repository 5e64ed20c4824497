"""Sessions of a data-graph pipeline (reference: graph/graph_layer.cpp:1297-1425, 1844-1980): the counterparts of the
reference's UpdateAfterDispatch, SequentialDispatch, MultiSessionsInOneCommandBuffer, MultiSessionsOneAtTheTime and
GetDataGraphPipelineSessionBindPointRequirementsARMTwoCallPattern tests (tests/vulkan.cpp:867-996, 2149-2308,
2836-2926), on the one- and two-layer MAX_POOL2D graphs of tests/shader/maxpool.spvasm / twolayer-maxpool.spvasm with
the expected bytes those tests hold."""
import importlib

import numpy as np
import pytest

from conftest import fixture_array as arr
from hip_util import gpu_available, hb

abi = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.abi")
gb = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graph_backend")


class _NoDevice:
    ctx = None
    stream = None


def maxpool_graph(dev, kats, layers):
    """MAX_POOL2D 2x2 stride 2, once or twice; input 1x16x16x3 int8; not bound to any memory yet"""
    k = kats["max_pool2d"] if layers == 1 else kats["two_layer_max_pool2d"]
    a = k["attr"]
    g = gb.Graph(dev)
    g.external("input", abi.I8, k["input"]["shape"])
    g.external("output", abi.I8, k["expected"]["shape"])
    g.mark_input("input")
    iattr = list(a["kernel"]) + list(a["stride"]) + list(a["pad"]) + [a["nan_mode"]]
    if layers == 2:
        g.tensor("mid", abi.I8, k["intermediate_shape"])
        g.op("MAX_POOL2D", ["input"], ["mid"], iattr)
        g.op("MAX_POOL2D", ["mid"], ["output"], iattr)
    else:
        g.op("MAX_POOL2D", ["input"], ["output"], iattr)
    g.mark_output("output")
    g._check(g.lib.mlel_graph_finalize(g.g, 1))
    return g, arr(k["input"]), arr(k["expected"])


# ------------------------------------------------------------------------------------------------ host only
def test_bind_point_requirements_two_call_pattern(kats):
    """tests/vulkan.cpp:2836-2926: the counting call, then the retrieving call with the indicated count; plus the
    short-array case of graph_layer.cpp:1379 (VK_INCOMPLETE)."""
    g1, _, _ = maxpool_graph(_NoDevice(), kats, 1)
    s1 = g1.new_session(allocate=False)
    rc, count, _ = s1.bind_point_requirements()
    assert (rc, count) == (0, 0)  # no intermediate tensor: no transient memory, no bind point
    rc, count, entries = s1.bind_point_requirements(capacity=count)
    assert (rc, count, entries) == (0, 0, [])
    assert s1.memory_requirements()[0] == 0
    s1.close()
    g1.close()

    g2, _, _ = maxpool_graph(_NoDevice(), kats, 2)
    s2 = g2.new_session(allocate=False)
    rc, count, _ = s2.bind_point_requirements()
    assert (rc, count) == (0, 1)
    rc, got, entries = s2.bind_point_requirements(capacity=count)
    assert (rc, got) == (0, count) and entries == [(gb.BIND_POINT_TRANSIENT, 0, 1)]
    rc, got, entries = s2.bind_point_requirements(capacity=0)
    assert rc == gb.INCOMPLETE and got == 1 and entries == []
    size, align = s2.memory_requirements()
    assert size >= 8 * 8 * 3 and align == 256
    with pytest.raises(hb.MlelError, match="Invalid bind point"):
        s2.bind_memory(256, bind_point=7)
    with pytest.raises(hb.MlelError, match="aligned"):
        s2.bind_memory(128)
    with pytest.raises(hb.MlelError, match="no CPU path"):
        s2.dispatch()
    s2.close()
    g2.close()


# ------------------------------------------------------------------------------------------------ GPU
@pytest.fixture(scope="module")
def dev():
    if not gpu_available():
        pytest.skip("no GPU visible")
    d = hb.Device(0)
    yield d
    d.close()


@pytest.mark.gpu
def test_update_after_dispatch_and_sequential_dispatch(dev, kats):
    """tests/vulkan.cpp:867-916: the external tensors are bound after the dispatch has been set up; :918-996: the same
    pipeline dispatched twice in a row with two output tensors.  Both outputs hold the MaxPool2D bytes."""
    g, x, exp = maxpool_graph(dev, kats, 1)
    s = g.new_session()
    s.set_input("input", x)
    s.dispatch()
    first = s.ext_tensors["output"]
    np.testing.assert_array_equal(first.download(), exp)
    second = dev.tensor(abi.I8, exp.shape)
    s.bind("output", second)  # re-bind, dispatch again: the new tensor is written, the old one keeps its bytes
    s.ext_tensors["keep"] = first
    s.dispatch()
    s.dispatch()
    np.testing.assert_array_equal(second.download(), exp)
    np.testing.assert_array_equal(first.download(), exp)
    s.set_input("input", np.zeros_like(x))
    s.dispatch()
    assert not second.download().any() and np.array_equal(first.download(), exp)
    s.close()
    g.close()


@pytest.mark.gpu
def test_multi_sessions_on_two_streams_and_one_at_a_time(dev, kats):
    """tests/vulkan.cpp:2149-2236: two pipelines of the two-layer graph, two sessions of the first and three of the
    second, all dispatched before anything is waited for -- here alternating between two streams, every session with
    transient memory of its own; :2238-2308: the sessions one at a time.  Every output holds the TwoLayerMaxPool2D
    bytes."""
    pipelines = [maxpool_graph(dev, kats, 2)[0] for _ in range(2)]
    _, x, exp = maxpool_graph(_NoDevice(), kats, 2)
    streams = [dev.new_stream(), dev.new_stream()]
    sessions = [pipelines[0].new_session() for _ in range(2)] + [pipelines[1].new_session() for _ in range(3)]
    assert len({s.session_mem for s in sessions}) == 5
    for s in sessions:
        s.set_input("input", x)
    for rounds in range(3):  # repeated: the bindings of a pipeline switch between its sessions every dispatch
        for i, s in enumerate(sessions):
            s.dispatch(streams[i % 2])
    for st in streams:
        dev._check(dev.lib.mlel_hip_sync(dev.ctx, st))
    for s in sessions:
        np.testing.assert_array_equal(s.get_output("output"), exp)
    # one at a time, a fresh session per dispatch
    for p in pipelines:
        for _ in range(2):
            s = p.new_session()
            s.set_input("input", x)
            s.dispatch()
            np.testing.assert_array_equal(s.get_output("output"), exp)
            s.close()
    # a session that has not bound an external tensor must not inherit another session's pointer
    bare = pipelines[0].new_session(allocate=False)
    with pytest.raises(hb.MlelError, match="transient memory is not bound"):  # graph_layer.cpp:1944-1947
        bare.dispatch()
    bare.session_mem = dev.alloc(4096)
    bare.bind_memory(bare.session_mem)
    with pytest.raises(hb.MlelError, match="no memory bound"):
        bare.dispatch()
    bare.close()
    for s in sessions:
        s.close()
    for p in pipelines:
        p.close()
    for st in streams:
        dev._check(dev.lib.mlel_hip_stream_destroy(dev.ctx, st))


@pytest.mark.gpu
def test_replayed_dispatch_equals_the_eager_one(dev, kats):
    """mlel_graph_session_dispatch_replayed: the launches of a dispatch recorded once and submitted many times (the
    command buffer of tests/vulkan.cpp:918-996, re-submitted).  Same bytes as the eager dispatch; a bind after the
    recording is honoured (the recording is made again); two sessions replay on two streams at once; a MobileNetV2-shaped
    graph of 38 launches replays to the bits of its eager dispatch."""
    g, x, exp = maxpool_graph(dev, kats, 2)
    streams = [dev.new_stream(), dev.new_stream()]
    s = g.new_session()
    s.set_input("input", x)
    for _ in range(3):
        s.dispatch_replayed(streams[0])
    dev._check(dev.lib.mlel_hip_sync(dev.ctx, streams[0]))
    np.testing.assert_array_equal(s.get_output("output"), exp)
    # new contents of the same input tensor: the recording reads the tensor, not a copy of its bytes
    s.set_input("input", np.zeros_like(x))
    s.dispatch_replayed(streams[0])
    dev._check(dev.lib.mlel_hip_sync(dev.ctx, streams[0]))
    assert not s.get_output("output").any()
    # another output tensor bound after the recording: it is written, the first one keeps its bytes
    first = s.ext_tensors["output"]
    second = dev.tensor(abi.I8, exp.shape)
    s.bind("output", second)
    s.ext_tensors["keep"] = first
    s.set_input("input", x)
    s.dispatch_replayed(streams[0])
    dev._check(dev.lib.mlel_hip_sync(dev.ctx, streams[0]))
    np.testing.assert_array_equal(second.download(), exp)
    assert not first.download().any()
    # the same session on another stream, and a second session beside it
    t = g.new_session()
    t.set_input("input", x)
    for _ in range(3):
        s.dispatch_replayed(streams[1])
        t.dispatch_replayed(streams[0])
    for st in streams:
        dev._check(dev.lib.mlel_hip_sync(dev.ctx, st))
    np.testing.assert_array_equal(second.download(), exp)
    np.testing.assert_array_equal(t.get_output("output"), exp)
    s.close()
    t.close()
    g.close()

    graphs = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graphs")
    spec = graphs.mobilenetv2_spec(batch=2, image=64, spread=True)
    net = graphs.build(dev, spec, fuse=True)
    rng = np.random.default_rng(3)
    image = rng.integers(-128, 127, spec.inputs[0][2], endpoint=True).astype(np.int8)
    net.set_input("input", image)
    net.dispatch()
    dev.sync()
    want = net.get_output("output")
    assert len(np.unique(want)) > 3
    r = net.new_session()
    r.set_input("input", image)
    for _ in range(3):
        r.dispatch_replayed(streams[0])
    dev._check(dev.lib.mlel_hip_sync(dev.ctx, streams[0]))
    np.testing.assert_array_equal(r.get_output("output"), want)
    r.close()
    net.close()
    for st in streams:
        dev._check(dev.lib.mlel_hip_stream_destroy(dev.ctx, st))
