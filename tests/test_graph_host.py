"""Host-side logic without a GPU: the interval planner against the reference's unit-test vectors, the format table,
the fusion pass and the session-memory plan of the benchmark graphs (built with no device context)."""
import importlib

import pytest

abi = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.abi")
gb = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graph_backend")
graphs = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graphs")
hb = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.hip_backend")


def test_interval_planner_reference_vectors(kats):
    for case in kats["interval_planner"]:
        offsets, size = gb.allocate_intervals(case["intervals"], case["unseen"], case["alignment"])
        assert size == case["memory_size"], case["name"]
        for k, v in case.get("offsets", {}).items():
            assert offsets[int(k)] == v, case["name"]
        for a, b in case.get("distinct", []):
            assert offsets[a] != offsets[b], case["name"]
        for k in case.get("present", []):
            assert k in offsets, case["name"]
        for k in case.get("absent", []):
            assert k not in offsets, case["name"]


def test_interval_planner_ordering_rules():
    # same first use: the larger tensor is placed first; ties on size by creation order
    offsets, size = gb.allocate_intervals([[0, 0, 1, 64, 0], [1, 0, 1, 256, 1], [2, 0, 1, 64, 2]], [], 64)
    assert offsets == {1: 0, 0: 256, 2: 320} and size == 384
    # best fit: the smallest released block that is large enough is taken, the remainder stays usable
    offsets, size = gb.allocate_intervals(
        [[0, 0, 0, 256, 0], [1, 0, 0, 128, 1], [2, 1, 2, 64, 2], [3, 1, 2, 64, 3], [4, 1, 2, 256, 4]], [], 64)
    assert offsets[4] == 0 and offsets[2] == 256 and offsets[3] == 320 and size == 384
    # alignment applies to the arena end and the total
    offsets, size = gb.allocate_intervals([[0, 0, 0, 10, 0], [1, 0, 0, 10, 1]], [[2, 5]], 16)
    assert offsets == {0: 0, 1: 16, 2: 32} and size == 48


def test_vk_format_table():
    lib = gb.load_graph_library()
    # VK_FORMAT_R8_SINT=14, R8_UINT=13, S8_UINT=127, R16_SINT=75, R16_SFLOAT=76, R32_SINT=99, R32_SFLOAT=100,
    # R64_SINT=111, R8_BOOL_ARM=1000460000
    expect = {14: abi.I8, 13: abi.U8, 127: abi.U8, 75: abi.I16, 74: abi.U16, 76: abi.F16, 99: abi.I32, 98: abi.U32,
              100: abi.F32, 111: abi.I64, 110: abi.U64, 112: abi.F64, 1000460000: abi.BOOL}
    for fmt, dt in expect.items():
        assert lib.mlel_graph_dtype_from_vk_format(fmt) == dt
    assert lib.mlel_graph_dtype_from_vk_format(37) < 0  # VK_FORMAT_R8G8B8A8_UNORM is not a tensor format
    assert b"Unsupported tensor buffer format: 37" in lib.mlel_graph_last_error()


class _NoDevice:
    """Stands in for hip_backend.Device when only the host-side logic is exercised."""
    ctx = None
    stream = None

    def alloc(self, n):
        raise AssertionError("no device")


def _build_host_only(spec, fuse):
    g = gb.Graph(_NoDevice())
    for name, dtype, shape in spec.inputs + spec.outputs:
        g.external(name, dtype, shape)
    for name, array in spec.consts.items():
        g.const(name, array)
    for name, (dtype, shape) in spec.tensors.items():
        g.tensor(name, dtype, shape)
    for name, _, _ in spec.inputs:
        g.mark_input(name)
    for op in spec.ops:
        g.op(op["op"], op["in"], op["out"], op["iattr"], op["fattr"], op["name"])
    for name, _, _ in spec.outputs:
        g.mark_output(name)
    g._check(g.lib.mlel_graph_finalize(g.g, 1 if fuse else 0))
    return g


def test_fusion_of_inverted_residual_block():
    spec = graphs.inverted_residual_spec(batch=2, hw=8)
    g = _build_host_only(spec, fuse=True)
    # the residual addition sits in the epilogue of the projection that feeds it
    assert g.op_names() == ["CONV2D+RESCALE+CLAMP", "DEPTHWISE_CONV2D+RESCALE+CLAMP",
                            "CONV2D+RESCALE+RESCALE+RESCALE+ADD+RESCALE"]
    u = _build_host_only(spec, fuse=False)
    assert u.op_names() == [o["op"] for o in spec.ops]
    # fused: the int32 accumulators are gone, nothing that is live at the same time overlaps
    live = [t for t in g.session_tensors() if t["offset"] is not None]
    assert len(live) == 2 and all(t["size"] == 2 * 8 * 8 * 144 for t in live)
    for a in live:
        for b in live:
            if a is not b and not (a["last"] < b["first"] or b["last"] < a["first"]):
                assert a["offset"] + a["size"] <= b["offset"] or b["offset"] + b["size"] <= a["offset"]
    g.close()
    u.close()


def test_mobilenetv2_graph_structure_and_plan():
    spec = graphs.mobilenetv2_spec(batch=1, image=32)
    assert sum(o["op"] == "CONV2D" for o in spec.ops) == 35
    assert sum(o["op"] == "DEPTHWISE_CONV2D" for o in spec.ops) == 17
    assert sum(o["op"] == "MATMUL" for o in spec.ops) == 1
    full = graphs.mobilenetv2_spec(batch=32)
    assert (full.macs["dense"] + full.macs["depthwise"]) // 32 == 300774272
    g = _build_host_only(spec, fuse=True)
    names = g.op_names()
    # contractions (10 of the projections carry their block's residual addition; from 28 x 28 positions down the 13
    # expansions run in one launch with the depthwise stage behind them; in front of that stage two projections share
    # a launch with the expansion that reads them, the second one still storing its result for the residual
    # connection of the next block; the last expansion pools its result in the same launch), fc; the RESHAPE between two
    # session tensors became a view of its input
    assert len(names) == 35 + 17 + 2 - 13 - 2 - 1 and "RESHAPE" not in names
    assert names[-2] == "CONV2D+RESCALE+CLAMP+AVG_POOL2D"
    assert names.count("CONV2D+RESCALE+CLAMP+DEPTHWISE_CONV2D+RESCALE+CLAMP") == 13
    assert names[2] == "CONV2D+RESCALE+CONV2D+RESCALE+CLAMP" and names[4] == "CONV2D+RESCALE+KEEP+CONV2D+RESCALE+CLAMP"
    assert names.count("CONV2D+RESCALE+RESCALE+RESCALE+ADD+RESCALE") == 10 and names[-1] == "MATMUL+RESCALE"
    planned = [t for t in g.session_tensors() if t["offset"] is not None]
    views = [t for t in planned if t["first"] == 0xFFFFFFFF]
    source = [t for t in planned if t["handle"] == views[0]["handle"] - 1]
    assert len(views) == 1 and source[0]["offset"] == views[0]["offset"] and source[0]["size"] == views[0]["size"]
    total = sum((t["size"] + 255) // 256 * 256 for t in planned)
    size = gb.C.c_uint64()
    g._check(g.lib.mlel_graph_session_memory_requirements(g.g, gb.C.byref(size), None))
    assert 0 < size.value < total / 2  # live ranges are short: the arena is much smaller than the sum of tensors
    for a in planned:
        for b in planned:
            if a is not b and not (a["last"] < b["first"] or b["last"] < a["first"]):
                assert a["offset"] + a["size"] <= b["offset"] or b["offset"] + b["size"] <= a["offset"]
    g.close()


def test_fusion_respects_observable_intermediates():
    """An accumulator that is also a graph output, or has a second consumer, must stay materialised."""
    spec = graphs.inverted_residual_spec(batch=1, hw=4)
    acc = spec.ops[0]["out"][0]
    spec.ops.append({"op": "CAST", "in": [acc], "out": ["extra"], "iattr": [], "fattr": [], "name": "tap"})
    spec.outputs.append(("extra", abi.I32, spec.tensors[acc][1]))
    g = _build_host_only(spec, fuse=True)
    assert g.op_names()[:3] == ["CONV2D", "RESCALE", "CLAMP"]
    g.close()


def test_error_conventions_of_the_operator_surface():
    g = gb.Graph(_NoDevice())
    g.external("x", abi.I8, (1, 4, 4, 4))
    g.tensor("y", abi.I32, (1, 4, 4, 4))
    with pytest.raises(hb.MlelError) as e:
        g.op("FROBNICATE", ["x"], ["y"])
    assert e.value.code == abi.ERR_UNSUPPORTED and "Unsupported TOSA operator" in str(e.value)
    with pytest.raises(hb.MlelError) as e:
        g.op("MIN_SAD", ["x"], ["y"])  # the motion-engine instruction set is not TOSA
    assert e.value.code == abi.ERR_UNSUPPORTED
    g.const("w", __import__("numpy").zeros((4, 1, 1, 4), "int8"))
    g.const("b", __import__("numpy").zeros((4,), "int32"))
    with pytest.raises(hb.MlelError) as e:
        g.op("CONV2D", ["x", "w", "b"], ["y"], [0, 0, 0, 0, 1, 1, 1, 1, 0, 0, 7])
    assert "Unsupported acc type 7" in str(e.value)
    with pytest.raises(hb.MlelError):
        g._check(g.lib.mlel_graph_get_tensor(g.g, 3, 0, 0))  # unknown descriptor set
    g._check(g.lib.mlel_graph_finalize(g.g, 1))
    with pytest.raises(hb.MlelError) as e:
        g.dispatch()
    assert "no CPU path" in str(e.value)
    g.close()


# ---------------------------------------------------------------------------------------- the three memory planners
def _build_no_device(spec, planner=None):
    g = gb.Graph(_NoDevice())
    if planner:
        g.set_planner(planner)
    for name, dtype, shape in spec.inputs + spec.outputs:
        g.external(name, dtype, shape)
    for name, array in spec.consts.items():
        g.const(name, array)
    for name, (dtype, shape) in spec.tensors.items():
        g.tensor(name, dtype, shape)
    g.mark_input("input")
    for op in spec.ops:
        g.op(op["op"], op["in"], op["out"], op["iattr"], op["fattr"], op["name"])
    g.mark_output("output")
    g._check(g.lib.mlel_graph_finalize(g.g, 1))
    size, align = __import__("ctypes").c_uint64(), __import__("ctypes").c_uint64()
    g._check(g.lib.mlel_graph_session_memory_requirements(g.g, size, align))
    return g, size.value, align.value


@pytest.mark.parametrize("which", ["mobilenetv2", "transformer", "inverted_residual"])
def test_memory_planners_give_valid_plans(which):
    """Interval, Linear and BestFit (VMEL_MEMORY_PLANNER in the reference): tensors whose live ranges overlap never
    share bytes, every offset is aligned, Linear is the sum of the aligned sizes, the reusing planners need no more
    than Linear.  The reference has no unit test for Linear / BestFit; the plan's validity is what can be pinned."""
    spec = {"mobilenetv2": lambda: graphs.mobilenetv2_spec(batch=2, image=64, classes=40),
            "transformer": lambda: graphs.transformer_block_spec(batch=1, seq=16, d_model=32, heads=2, ffn=64),
            "inverted_residual": lambda: graphs.inverted_residual_spec(batch=2, hw=14)}[which]()
    sizes = {}
    for planner in ("interval", "linear", "bestfit"):
        g, size, align = _build_no_device(spec, planner)
        assert g.planner() == planner
        placed = [t for t in g.session_tensors() if t["offset"] is not None]
        assert placed and all(t["offset"] % align == 0 for t in placed)
        assert max(t["offset"] + t["size"] for t in placed) <= size
        for i, a in enumerate(placed):
            for b in placed[i + 1:]:
                same_range = a["first"] == b["first"] and a["last"] == b["last"]
                if a["handle"] == b["handle"] or (a["offset"] == b["offset"] and a["size"] == b["size"] and same_range):
                    continue  # a RESHAPE view and the tensor it aliases
                lives_overlap = a["first"] <= b["last"] and b["first"] <= a["last"]
                bytes_overlap = a["offset"] < b["offset"] + b["size"] and b["offset"] < a["offset"] + a["size"]
                assert not (lives_overlap and bytes_overlap), (planner, a, b)
        sizes[planner] = size
        if planner == "linear":
            distinct = {(t["offset"], t["size"]) for t in placed}
            assert size == sum((s + align - 1) // align * align for _, s in distinct)
        g.close()
    assert sizes["interval"] <= sizes["linear"] and sizes["bestfit"] <= sizes["linear"]
    if which != "inverted_residual":  # (its two session tensors are live together once the addition is fused away)
        assert sizes["interval"] < sizes["linear"]  # the graphs do have tensors with disjoint lifetimes


def _build_split(spec, planner="interval"):
    g = gb.Graph(_NoDevice())
    g.set_planner(planner)
    g.set_batch_split(True)
    for name, dtype, shape in spec.inputs + spec.outputs:
        g.external(name, dtype, shape)
    for name, array in spec.consts.items():
        g.const(name, array)
    for name, (dtype, shape) in spec.tensors.items():
        g.tensor(name, dtype, shape)
    for name, _, _ in spec.inputs:
        g.mark_input(name)
    for op in spec.ops:
        g.op(op["op"], op["in"], op["out"], op["iattr"], op["fattr"], op["name"])
    for name, _, _ in spec.outputs:
        g.mark_output(name)
    g._check(g.lib.mlel_graph_finalize(g.g, 1))
    size = gb.C.c_uint64()
    g._check(g.lib.mlel_graph_session_memory_requirements(g.g, gb.C.byref(size), None))
    return g, size.value


def test_batch_split_plan():
    """The plan of a pipeline whose leading launches are issued per half batch on two streams: session tensors that
    only the split run touches are stored as two halves behind the whole tensors -- [whole | first halves | second
    halves] -- and inside the half region no two tensors whose live ranges overlap share a byte at half their size;
    whole tensors the run touches (here the pooled tensor the fully connected layer reads behind the join) share
    nothing with each other.  The library checks the same on its side at finalize and refuses a plan that fails."""
    spec = graphs.mobilenetv2_spec(batch=4, image=64, classes=40)
    plain = _build_host_only(spec, fuse=True)
    g, size = _build_split(spec)
    assert g.op_names() == plain.op_names()
    launches = g.batch_split_launches()
    assert launches == len(g.op_names()) - 1  # everything but the fully connected layer
    placed = [t for t in g.session_tensors() if t["offset"] is not None and t["first"] != 0xFFFFFFFF]
    halves = [t for t in placed if t["first"] >= 1 and t["last"] <= launches]
    whole = [t for t in placed if t not in halves]
    assert halves and whole
    whole_end = max(t["offset"] + t["size"] for t in whole)
    half_start = min(t["offset"] for t in halves)
    assert half_start >= whole_end and half_start % 256 == 0
    region = (size - half_start) // 2
    assert half_start + 2 * region == size
    for i, a in enumerate(halves):
        assert a["offset"] - half_start + a["size"] // 2 <= region
        for b in halves[i + 1:]:
            lives_overlap = a["first"] <= b["last"] and b["first"] <= a["last"]
            bytes_overlap = a["offset"] < b["offset"] + b["size"] // 2 and b["offset"] < a["offset"] + a["size"] // 2
            assert not (lives_overlap and bytes_overlap), (a, b)
    g.close()
    plain.close()
    # an odd batch, or the best-fit planner: left unsplit, the plan is the unsplit one
    odd, _ = _build_split(graphs.mobilenetv2_spec(batch=3, image=64, classes=40))
    assert odd.batch_split_launches() == 0
    odd.close()
    bf, bf_size = _build_split(spec, "bestfit")
    ref, ref_size, _ = _build_no_device(spec, "bestfit")
    assert bf.batch_split_launches() == 0 and bf_size == ref_size
    bf.close()
    ref.close()
    lin, _ = _build_split(spec, "linear")  # no reuse at all: every tensor stays whole
    assert lin.batch_split_launches() == launches
    lin.close()
    # the fp16 encoder block starts with a LayerNorm region: nothing to split
    enc, _ = _build_split(graphs.transformer_block_spec(batch=2, seq=16, d_model=32, heads=2, ffn=64))
    assert enc.batch_split_launches() == 0
    enc.close()


def test_memory_planner_from_environment(monkeypatch):
    spec = graphs.inverted_residual_spec(batch=1, hw=8)
    for value, expect in (("Linear", "linear"), ("BestFit", "bestfit"), ("Interval", "interval"), ("nonsense", "interval")):
        monkeypatch.setenv("VMEL_MEMORY_PLANNER", value)
        g, _, _ = _build_no_device(spec)
        assert g.planner() == expect
        g.close()
    monkeypatch.delenv("VMEL_MEMORY_PLANNER")
    g, _, _ = _build_no_device(spec)
    assert g.planner() == "interval"
    with pytest.raises(hb.MlelError, match="before finalize"):
        g.set_planner("linear")
    g.close()


def test_best_fit_allocation_rules():
    """BestFit on a chain a -> b -> c -> d (each read once): c may reuse a, d may reuse a or b; the largest tensor is
    placed first and a smaller one moves into the smallest block that is large enough."""
    g = gb.Graph(_NoDevice())
    g.set_planner("bestfit")
    g.external("input", abi.I8, (1, 1024))
    g.external("output", abi.I8, (1, 256))
    for name, n in (("a", 1024), ("b", 4096), ("c", 512), ("d", 256)):
        g.tensor(name, abi.I8, (1, n))
    g.mark_input("input")
    g.op("ABS", ["input"], ["a"])
    g.op("TILE", ["a"], ["b"])
    g.op("SLICE", ["b"], ["c"], [0, 0])
    g.op("SLICE", ["c"], ["d"], [0, 0])
    g.op("ABS", ["d"], ["output"])
    g.mark_output("output")
    g._check(g.lib.mlel_graph_finalize(g.g, 0))
    by_size = {t["size"]: t["offset"] for t in g.session_tensors()}
    assert by_size[4096] == 0 and by_size[1024] == 4096     # placed by size; a and b are alive together
    assert by_size[512] == by_size[1024]                     # c: only a is dead when c is produced
    assert by_size[256] == by_size[4096]                     # d: a's block holds c (alive), b's block is free
    g.close()


def test_profiling_switch_from_environment(monkeypatch):
    """VMEL_GRAPH_PROFILING as the reference reads it (graph/graph_profiler.cpp:29-38, 107): unset, empty, 0, false, off
    and no (any case) leave profiling off, anything else turns it on; the report of an idle graph is empty."""
    for value, expect in (("1", True), ("true", True), ("yes", True), ("anything", True), ("0", False), ("FALSE", False),
                          ("Off", False), ("no", False), ("", False)):
        monkeypatch.setenv("VMEL_GRAPH_PROFILING", value)
        g = gb.Graph(_NoDevice())
        assert g.profiling() is expect, value
        g.close()
    monkeypatch.delenv("VMEL_GRAPH_PROFILING")
    g = gb.Graph(_NoDevice())
    assert g.profiling() is False
    g.set_profiling(True)
    assert g.profiling() is True
    assert g.profiling_report() == {"timestamp_period_ns": None, "samples": [], "by_operator": []}
    g.close()


# ------------------------------------------------------------------------------------- fp16 fusion patterns, host only
def _f16_projection(spec, x, rows, k, n, seed):
    """MATMUL (fp32 result) + fp32 bias + CAST to fp16, as the transformer block spells a projection."""
    import numpy as np
    rng = np.random.default_rng(seed)
    w = spec.const("w", (0.02 * rng.standard_normal((1, k, n))).astype(np.float16))
    b = spec.const("b", (0.02 * rng.standard_normal((1, 1, n))).astype(np.float32))
    acc = spec.tensor("acc", abi.F32, (1, rows, n))
    spec.op("MATMUL", [x, w], [acc], [0, 0])
    summed = spec.tensor("t", abi.F32, (1, rows, n))
    spec.op("ADD", [acc, b], [summed])
    out = spec.tensor("t", abi.F16, (1, rows, n))
    spec.op("CAST", [summed], [out])
    return out


def test_transformer_block_fused_operator_list():
    """The encoder block after fusion, on the host: nine launches, no stand-alone reduction, transpose or reshape."""
    spec = graphs.transformer_block_spec(batch=2, seq=64, d_model=64, heads=4, ffn=128)
    g = _build_host_only(spec, fuse=True)
    three = " | ".join(["MATMUL+ADD+CAST+RESHAPE+TRANSPOSE"] * 3)
    assert g.op_names() == ["ELEMENTWISE+REDUCE x11", three, "MATMUL+CAST", "ELEMENTWISE+REDUCE x7",
                            "MATMUL+CAST+RESHAPE+TRANSPOSE", "MATMUL+ADD+CAST+ADD", "ELEMENTWISE+REDUCE x11",
                            "MATMUL+ADD+CAST+ELEMENTWISE x9", "MATMUL+ADD+CAST+ADD"]
    g.close()


def test_attention_fusion_on_heads_of_64():
    """Scores, softmax and the product with V become one launch when the heads are 64 wide and the key count is a
    multiple of 64 up to 512 (config 4: seven launches); other head sizes or key counts keep the three launches."""
    three = " | ".join(["MATMUL+ADD+CAST+RESHAPE+TRANSPOSE"] * 3)
    attention = "MATMUL+CAST+ELEMENTWISE+REDUCE x7+MATMUL+CAST+RESHAPE+TRANSPOSE"
    fused = ["ELEMENTWISE+REDUCE x11", three, attention, "MATMUL+ADD+CAST+ADD", "ELEMENTWISE+REDUCE x11",
             "MATMUL+ADD+CAST+ELEMENTWISE x9", "MATMUL+ADD+CAST+ADD"]
    g = _build_host_only(graphs.transformer_block_spec(), fuse=True)
    assert g.op_names() == fused
    g.close()
    g = _build_host_only(graphs.transformer_block_spec(batch=1, seq=128, d_model=128, heads=2, ffn=256), fuse=True)
    assert attention in g.op_names() and "ELEMENTWISE+REDUCE x7" not in g.op_names()
    g.close()
    for kwargs in (dict(batch=1, seq=576, d_model=128, heads=2, ffn=256),   # 576 keys
                   dict(batch=1, seq=96, d_model=128, heads=2, ffn=256),    # 96 keys and query rows
                   dict(batch=1, seq=128, d_model=128, heads=4, ffn=256)):  # heads of 32
        g = _build_host_only(graphs.transformer_block_spec(**kwargs), fuse=True)
        names = g.op_names()
        assert attention not in names and "ELEMENTWISE+REDUCE x7" in names, kwargs
        g.close()


def test_projection_patterns_leave_observable_or_mismatched_cases_alone():
    """Residual, grouping and view fusions behind fp16 products apply only when nothing else can observe the product's
    result and the shapes fit."""
    import numpy as np
    rows, d = 64, 32

    def base():
        spec = graphs.Spec()
        spec.inputs.append(("input", abi.F16, (1, rows, d)))
        return spec

    # 1. two projections of one tensor group; a third with other extents does not join; results that are graph
    #    outputs are still written by the grouped launch
    spec = base()
    p1 = _f16_projection(spec, "input", rows, d, d, 1)
    p2 = _f16_projection(spec, "input", rows, d, d, 2)
    p3 = _f16_projection(spec, "input", rows, d, 2 * d, 3)
    spec.op("MUL", [p1, p2], ["out_a"], [0])
    spec.outputs.append(("out_a", abi.F16, (1, rows, d)))
    spec.op("CAST", [p3], ["out_b"])
    spec.outputs.append(("out_b", abi.F32, (1, rows, 2 * d)))
    g = _build_host_only(spec, fuse=True)
    assert g.op_names() == ["MATMUL+ADD+CAST | MATMUL+ADD+CAST", "MATMUL+ADD+CAST", "MUL", "CAST"]
    g.close()

    # 1b. the sum of two projections: the first one's result is the second one's residual, and a product that carries
    #     a residual joins no group
    spec = base()
    p1 = _f16_projection(spec, "input", rows, d, d, 1)
    p2 = _f16_projection(spec, "input", rows, d, d, 2)
    spec.op("ADD", [p1, p2], ["out"])
    spec.outputs.append(("out", abi.F16, (1, rows, d)))
    g = _build_host_only(spec, fuse=True)
    assert g.op_names() == ["MATMUL+ADD+CAST", "MATMUL+ADD+CAST+ADD"]
    g.close()

    # 2. the residual operand is produced after the projection: the ADD stays
    spec = base()
    p = _f16_projection(spec, "input", rows, d, d, 4)
    late = spec.tensor("t", abi.F16, (1, rows, d))
    spec.op("ABS", ["input"], [late])
    spec.op("ADD", [p, late], ["out"])
    spec.outputs.append(("out", abi.F16, (1, rows, d)))
    g = _build_host_only(spec, fuse=True)
    assert g.op_names() == ["MATMUL+ADD+CAST", "ABS", "ADD"]
    g.close()

    # 2b. an elementwise region behind the product moves into its call only when the product's kernel applies it
    #     itself (the transformer block's GELU above); any other region stays a pass of its own
    spec = base()
    p = _f16_projection(spec, "input", rows, d, d, 4)
    late = spec.tensor("t", abi.F16, (1, rows, d))
    spec.op("MUL", ["input", "input"], [late], [0])
    spec.op("ADD", [p, late], ["out"])
    spec.outputs.append(("out", abi.F16, (1, rows, d)))
    g = _build_host_only(spec, fuse=True)
    assert g.op_names() == ["MATMUL+ADD+CAST", "ELEMENTWISE x2"]
    g.close()

    # 3. the residual exists before the projection: it rides on it; a second reader of the product prevents that
    for second_reader in (False, True):
        spec = base()
        p = _f16_projection(spec, "input", rows, d, d, 5)
        spec.op("ADD", ["input", p], ["out"])
        spec.outputs.append(("out", abi.F16, (1, rows, d)))
        if second_reader:
            spec.op("CAST", [p], ["tap"])
            spec.outputs.append(("tap", abi.F32, (1, rows, d)))
        g = _build_host_only(spec, fuse=True)
        assert g.op_names() == (["MATMUL+ADD+CAST", "ADD", "CAST"] if second_reader else ["MATMUL+ADD+CAST+ADD"])
        g.close()

    # 4. a head split whose innermost extent is no multiple of eight keeps its RESHAPE (an alias) and TRANSPOSE
    spec = base()
    p = _f16_projection(spec, "input", rows, d, 24, 6)
    split = spec.tensor("t", abi.F16, (1, rows, 2, 12))
    spec.op("RESHAPE", [p], [split])
    spec.op("TRANSPOSE", [split], ["out"], [0, 2, 1, 3])
    spec.outputs.append(("out", abi.F16, (1, 2, rows, 12)))
    g = _build_host_only(spec, fuse=True)
    assert g.op_names() == ["MATMUL+ADD+CAST", "TRANSPOSE"]
    g.close()


def test_elementwise_region_emits_an_absorbed_square_once():
    """An intermediate that one operator reads twice -- MUL(t, t) over t = EXP(x) -- is absorbed into the region as ONE
    step: EXP, MUL, ADD make a region of three steps, not four with EXP emitted twice."""
    spec = graphs.Spec()
    shape = (1, 16, 64)
    spec.inputs.append(("input", abi.F16, shape))
    t = spec.tensor("t", abi.F16, shape)
    spec.op("EXP", ["input"], [t])
    sq = spec.tensor("t", abi.F16, shape)
    spec.op("MUL", [t, t], [sq], [0])
    spec.op("ADD", [sq, "input"], ["output"])
    spec.outputs.append(("output", abi.F16, shape))
    g = _build_host_only(spec, fuse=True)
    assert g.op_names() == ["ELEMENTWISE x3"]
    g.close()


def test_graph_log_severity_from_environment(tmp_path):
    """VMEL_GRAPH_SEVERITY as the reference reads it (common/log.cpp:29-71, graph/graph_log.cpp:19): unset or unknown
    words mean Error, names compare without case; at Info the loader prints one line per decoded instruction
    (graph_tosa_1_0_ext_inst.cpp:453-457), the planner in use (graph_layer.cpp:286-295) and a line per pipeline; failures
    are Error lines.  Lines have the reference's shape: timestamp, logger name, severity."""
    import os
    import re
    import subprocess
    import sys

    script = tmp_path / "log_probe.py"
    script.write_text('''
import importlib, os, sys
sys.path.insert(0, os.environ["MLEL_REPO"])
sys.path.insert(0, os.path.join(os.environ["MLEL_REPO"], "tests"))
gb = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graph_backend")
graphs = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graphs")
import spvasm_writer
lib = gb.load_graph_library()
print("LEVEL", lib.mlel_graph_log_level(), flush=True)
class NoDevice:
    ctx = None
    stream = None
spec = graphs.inverted_residual_spec(batch=1, hw=8)
w = spvasm_writer.from_spec(spec)
g = gb.Graph(NoDevice())
g.load_spvasm(w.text(), w.bindings, w.constants, w.names)
g._check(g.lib.mlel_graph_finalize(g.g, 1))
try:
    gb.Graph(NoDevice()).load_spvasm("OpCapability Nonsense\\n%1 = OpBogus", [], [], [])
except Exception as e:
    print("RAISED", flush=True)
''')
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

    def run(value):
        env = dict(os.environ, MLEL_REPO=repo)
        env.pop("VMEL_GRAPH_SEVERITY", None)
        if value is not None:
            env["VMEL_GRAPH_SEVERITY"] = value
        out = subprocess.run([sys.executable, str(script)], env=env, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        return out.stdout.splitlines()

    line = re.compile(r"^\d{4}-\d\d-\d\d \d\d:\d\d:\d\d,\d{3} \[Graph\]\[(Error|Warning|Info|Debug)\] .+")
    for value, level in ((None, 0), ("nonsense", 0), ("warning", 1), ("INFO", 2), ("Debug", 3)):
        lines = run(value)
        assert lines[0] == f"LEVEL {level}", (value, lines[:2])
        logged = [l for l in lines if "[Graph][" in l]
        assert all(line.match(l) for l in logged), logged[:3]
        kinds = {line.match(l).group(1) for l in logged}
        assert "RAISED" in lines
        assert "Error" in kinds  # the refused module is reported at every level
        if level < 2:
            assert kinds == {"Error"}
        else:
            ops = [l for l in logged if "OpExtInst result=%" in l]
            assert len(ops) == 12 and any("CONV2D" in l for l in ops) and any("RESCALE" in l for l in ops), ops[:3]
            assert sum("Using interval memory planner" in l for l in logged) == 1
            assert sum("Graph pipeline created: 12 operators recorded, 3 launches" in l for l in logged) == 1
            assert ("Debug" in kinds) == (level == 3)
