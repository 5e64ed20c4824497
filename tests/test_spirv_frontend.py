"""The SPIR-V assembly front-end (csrc/graph/spirv_graph_loader.cpp).

CPU part: modules are decoded with no device context and the recorded graph is inspected -- the reference's own
test modules (tests/shader/*.spvasm, read from the reference checkout when it is present), the benchmark graphs
written by tests/spvasm_writer.py against the same graphs built call by call, and the error paths.

GPU part: the reference's known-answer vectors (tests/vulkan.cpp, committed under tests/golden/) run through modules
of the same structure as the reference's, and the benchmark graphs run from assembly text against the CPU oracle.
"""
import importlib
import os

import numpy as np
import pytest

import spvasm_writer as sw
from conftest import fixture_array as arr
from hip_util import gpu_available, hb
from oracle_graph import run_spec

abi = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.abi")
gb = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graph_backend")
graphs = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graphs")

REFERENCE_SHADERS = "/root/reference/tests/shader"


class _NoDevice:
    ctx = None
    stream = None

    def alloc(self, n):
        raise AssertionError("no device")


def decode(text, bindings=None, constants=None, names=None, fuse=False):
    """Loads a module with no device; returns (graph, inputs, outputs, TOSA instruction count)."""
    g = gb.Graph(_NoDevice())
    ins, outs, count = g.load_spvasm(text, bindings, constants, names)
    g._check(g.lib.mlel_graph_finalize(g.g, 1 if fuse else 0))
    return g, ins, outs, count


def described(g, names):
    return [(g.externals[n][3], g.externals[n][4]) for n in names]


# ------------------------------------------------------------------------------------------ reference test modules
I8_1883 = (abi.I8, (1, 8, 8, 3))
REFERENCE_MODULES = {
    # file: (bindings, constants, inputs, outputs, executed operators)
    "conv2d.spvasm": ({}, {}, [I8_1883, (abi.I8, (3, 2, 2, 3)), (abi.I32, (3,))], [(abi.I32, (1, 4, 4, 3))],
                      ["CONV2D"]),
    "conv2_acc_int64.spvasm": ({}, {}, [(abi.I16, (1, 2, 2, 4)), (abi.I8, (4, 1, 1, 4)), (abi.I64, (4,))],
                               [(abi.I64, (1, 2, 2, 4))], ["CONV2D"]),
    "maxpool.spvasm": ({(0, 0, 1): (1, 16, 16, 3), (0, 1, 0): (1, 8, 8, 3)}, {}, [(abi.I8, (1, 16, 16, 3))],
                       [I8_1883], ["MAX_POOL2D"]),
    "twolayer-maxpool.spvasm": ({(0, 0, 0): (1, 16, 16, 3), (0, 1, 0): (1, 4, 4, 3)}, {}, [(abi.I8, (1, 16, 16, 3))],
                                [(abi.I8, (1, 4, 4, 3))], ["MAX_POOL2D", "MAX_POOL2D"]),
    "concat.spvasm": ({(0, 0, 0): (1, 2, 2, 2), (0, 1, 0): (1, 2, 2, 2), (0, 2, 0): (1, 4, 2, 2)}, {},
                      [(abi.I8, (1, 2, 2, 2))] * 2, [(abi.I8, (1, 4, 2, 2))], ["CONCAT"] * 2),  # one copy per input
    "concat_interval.spvasm": ({}, {}, [(abi.F32, (3, 3)), (abi.F32, (3, 3)), (abi.F32, (3, 1))], [(abi.F32, (12,))],
                               ["ADD", "CONCAT", "CONCAT", "RESHAPE"]),
    "slice.spvasm": ({(0, 0, 0): (1, 8, 8, 3), (0, 1, 0): (1, 2, 2, 2)}, {}, [I8_1883], [(abi.I8, (1, 2, 2, 2))],
                     ["SLICE"]),
    "maximum.spvasm": ({(0, b, 0): (1, 2, 2, 2) for b in range(3)}, {}, [(abi.I32, (1, 2, 2, 2))] * 2,
                       [(abi.I32, (1, 2, 2, 2))], ["MAXIMUM"]),
    "sin.spvasm": ({}, {}, [(abi.F32, (54, 40, 39))], [(abi.F32, (54, 40, 39))], ["SIN"]),
    "inlined-higher-rank-constant.spvasm": ({}, {}, [(abi.I8, (1, 3, 3, 1))], [(abi.I8, (1, 3, 3, 1))],
                                            ["CONV2D", "CAST"]),
    "graph-constant-arm.spvasm": ({}, {0: np.array([2], np.int32), 1: np.array([0], np.int8),
                                       2: np.array([3], np.int32), 3: np.array([0], np.int8),
                                       4: np.array([4], np.int32), 5: np.array([0], np.int8)},
                                  [(abi.I8, (5,))] * 2, [(abi.I8, (5,))], ["RESCALE", "RESCALE", "ADD", "RESCALE"]),
    "fft2d.spvasm": ({}, {}, [(abi.F32, (1, 4, 4096))] * 2, [(abi.F32, (1, 4, 4096))] * 2, ["FFT2D"]),
    "arshift_specbool.spvasm": ({}, {}, [(abi.I16, (4,))] * 2, [(abi.I16, (4,))], ["ARITHMETIC_RIGHT_SHIFT"]),
    "conv3d_large_stride.spvasm": ({}, {0: np.zeros((3, 2, 2, 8192, 4), np.int8)}, [(abi.I8, (1, 3, 2, 2, 4))],
                                   [(abi.I32, (1, 3, 2, 2, 3))], ["CONV3D"]),
    "conv3d_inline_bf16_constant.spvasm": ({}, {}, [(abi.BF16, (1, 1, 1, 1, 1))], [(abi.BF16, (1, 1, 1, 1, 1))], ["CONV3D"]),
    "conv3d_inline_fp8e4m3_constant.spvasm": ({}, {}, [(abi.F8E4M3, (1, 1, 1, 1, 1))], [(abi.F8E4M3, (1, 1, 1, 1, 1))],
                                              ["CONV3D"]),
    "conv3d_inline_fp8e5m2_constant.spvasm": ({}, {}, [(abi.F8E5M2, (1, 1, 1, 1, 1))], [(abi.F8E5M2, (1, 1, 1, 1, 1))],
                                              ["CONV3D"]),
    "nop-outputs.spvasm": ({(0, 0, 0): (1, 8, 8, 3), (0, 1, 0): (1, 2, 2, 2), (0, 2, 0): (1, 8, 8, 3),
                            (0, 3, 0): (1, 8, 8, 3)}, {0: np.zeros((1, 8, 8, 3), np.int8)}, [I8_1883],
                           [(abi.I8, (1, 2, 2, 2)), I8_1883, I8_1883], ["SLICE", "CAST", "CAST"]),
}


@pytest.mark.skipif(not os.path.isdir(REFERENCE_SHADERS), reason="reference checkout not present")
@pytest.mark.parametrize("name", sorted(REFERENCE_MODULES))
def test_reference_modules_decode(name):
    bindings, constants, exp_in, exp_out, exp_ops = REFERENCE_MODULES[name]
    with open(os.path.join(REFERENCE_SHADERS, name)) as f:
        text = f.read()
    g, ins, outs, count = decode(text, bindings, constants)
    assert described(g, ins) == exp_in
    assert described(g, outs) == exp_out
    assert g.op_names() == exp_ops
    g.close()


@pytest.mark.skipif(not os.path.isdir(REFERENCE_SHADERS), reason="reference checkout not present")
def test_reference_modules_outside_the_operator_set_are_refused():
    def error_of(name, bindings=None, constants=None):
        with open(os.path.join(REFERENCE_SHADERS, name)) as f:
            text = f.read()
        with pytest.raises(hb.MlelError) as e:
            decode(text, bindings, constants)
        return str(e.value)

    assert "does not import" in error_of("me_raw_sad_sr0.spvasm")          # motion-engine instruction set
    assert "no data supplied for graph constant 1" in error_of("graph-constant-arm.spvasm",
                                                               constants={0: np.array([2], np.int32)})
    assert "no shape for set 0 binding 0 element 1" in error_of("maxpool.spvasm", {(0, 1, 0): (1, 8, 8, 3)})


# ------------------------------------------------------------------------------------------ writer -> loader, CPU
def small_specs():
    return {
        "inverted_residual": graphs.inverted_residual_spec(batch=2, hw=14, spread=True),
        "mobilenetv2": graphs.mobilenetv2_spec(batch=2, image=64, spread=True, classes=40),
        "transformer": graphs.transformer_block_spec(batch=1, seq=16, d_model=32, heads=2, ffn=64),
    }


@pytest.mark.parametrize("which", ["inverted_residual", "mobilenetv2", "transformer"])
@pytest.mark.parametrize("shaped_io", [True, False], ids=["shaped", "unshaped_io"])
def test_written_module_records_the_same_graph(which, shaped_io):
    """The graph decoded from assembly text is the graph built call by call: same operators after fusion, same
    session-memory plan."""
    spec = small_specs()[which]
    w = sw.from_spec(spec, inline_limit=64, shaped_io=shaped_io)
    assert shaped_io or w.bindings
    g, ins, outs, count = decode(w.text(), w.bindings, w.constants, w.names, fuse=True)
    assert count == len(spec.ops) and ins == ["input"] and outs == ["output"]
    d = gb.Graph(_NoDevice())
    for name, dtype, shape in spec.inputs + spec.outputs:
        d.external(name, dtype, shape)
    for name, array in spec.consts.items():
        d.const(name, array)
    for name, (dtype, shape) in spec.tensors.items():
        d.tensor(name, dtype, shape)
    d.mark_input("input")
    for op in spec.ops:
        d.op(op["op"], op["in"], op["out"], op["iattr"], op["fattr"], op["name"])
    d.mark_output("output")
    d._check(d.lib.mlel_graph_finalize(d.g, 1))
    assert g.op_names() == d.op_names()
    plan = lambda graph: sorted((t["offset"], t["size"], t["first"], t["last"]) for t in graph.session_tensors()
                                if t["offset"] is not None)
    assert plan(g) == plan(d)
    assert described(g, ins + outs) == described(d, ["input", "output"])
    g.close()
    d.close()


def tiny_module(op_line, extra=""):
    return f"""
        OpCapability GraphARM
        %tosa = OpExtInstImport "TOSA.001000.1"
        OpDecorate %a DescriptorSet 0
        OpDecorate %a Binding 0
        OpDecorate %b DescriptorSet 0
        OpDecorate %b Binding 1
        %uint = OpTypeInt 32 0
        %uchar = OpTypeInt 8 0
        %bool = OpTypeBool
        %true = OpConstantTrue %bool
        %false = OpConstantFalse %bool
        %uint_0 = OpConstant %uint 0
        %uint_1 = OpConstant %uint 1
        %uint_2 = OpConstant %uint 2
        %uint_4 = OpConstant %uint 4
        %arr1 = OpTypeArray %uint %uint_1
        %s4 = OpConstantComposite %arr1 %uint_4
        %s1 = OpConstantComposite %arr1 %uint_1
        %t = OpTypeTensorARM %uchar %uint_1 %s4
        %t32 = OpTypeTensorARM %uint %uint_1 %s4
        %one8 = OpTypeTensorARM %uchar %uint_1 %s1
        %one32 = OpTypeTensorARM %uint %uint_1 %s1
        %z8 = OpConstantNull %one8
        %z32 = OpConstantNull %one32
        %mult = OpConstantComposite %one32 %uint_1
        {extra}
        %ptr = OpTypePointer UniformConstant %t
        %gt = OpTypeGraphARM 1 %t %t
        %a = OpVariable %ptr UniformConstant
        %b = OpVariable %ptr UniformConstant
        OpGraphEntryPointARM %g "main" %a %b
        %g = OpGraphARM %gt
        %in = OpGraphInputARM %t %uint_0
        {op_line}
        OpGraphSetOutputARM %r %uint_0
        OpGraphEndARM
    """


def test_loader_error_paths():
    def error_of(op_line, extra=""):
        with pytest.raises(hb.MlelError) as e:
            decode(tiny_module(op_line, extra))
        return str(e.value)

    g, ins, outs, count = decode(tiny_module("%r = OpExtInst %t %tosa ABS %in"))
    assert count == 1 and g.op_names() == ["ABS"]
    g.close()
    assert "FROBNICATE is not decoded" in error_of("%r = OpExtInst %t %tosa FROBNICATE %in")
    assert "rounding mode 2" in error_of("%r = OpExtInst %t %tosa RESCALE %true %uint_2 %false %false %false %in "
                                         "%mult %z8 %z8 %z8")
    assert "expects 10 arguments" in error_of("%r = OpExtInst %t %tosa RESCALE %true %uint_1 %in")
    assert "%nowhere is not a constant" in error_of("%r = OpExtInst %t %tosa ADD %in %nowhere")
    assert "is not TOSA.001000.1" in error_of("%r = OpExtInst %t %other ABS %in",
                                              '%other = OpExtInstImport "GLSL.std.450"')
    assert "may appear in a graph body" in error_of("%r = OpIAdd %t %in %in")
    assert "line 35" in error_of("%r = OpExtInst %t %tosa FROBNICATE %in")
    with pytest.raises(hb.MlelError, match="no graph entry point"):
        decode("%uint = OpTypeInt 32 0\n")


def test_loader_reads_signed_values_from_unsigned_declarations():
    """`OpTypeInt 8 0` tensors hold signed data: 0xF6 as a zero point means -10 (CLAMP bounds likewise)."""
    w = sw.SpvAsm()
    x = w.input("input", abi.I8, (1, 4))
    out = w.output("output", abi.I8, (1, 4))
    r = w.op("CLAMP", abi.I8, (1, 4), [w.scalar(abi.I8, -10), w.scalar(abi.I8, 20), w.u32(1), x])
    w.set_output(r, out)
    text = w.text()
    assert "OpConstant %uint8 246" in text and "OpTypeInt 8 0" in text
    g, ins, outs, count = decode(text)
    assert g.op_names() == ["CLAMP"]
    g.close()


# ------------------------------------------------------------------------------------------------------- GPU part
@pytest.fixture(scope="module")
def dev():
    if not gpu_available():
        pytest.skip("no GPU visible")
    d = hb.Device(0)
    yield d
    d.close()


def run_module(dev, w, inputs, fuse=True):
    g = gb.Graph(dev)
    ins, outs, count = g.load_spvasm(w.text(), w.bindings, w.constants, w.names)
    g.finalize(fuse)
    for name, array in inputs.items():
        g.set_input(name, array)
    g.dispatch()
    result = {o: g.get_output(o) for o in outs}
    names = g.op_names()
    g.close()
    return result, names


def conv_operands(w, a, zp_dtype=abi.I8):
    return [w.attr(a["pad"]), w.attr(a["stride"]), w.attr(a["dilation"]), w.u32(a["acc_type"]),
            w.scalar(abi.BOOL, False)], [w.attr([a["input_zp"]], zp_dtype), w.attr([a["weight_zp"]], zp_dtype)]


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["conv2d", "conv2d_acc_int64"])
def test_kat_conv2d_modules(dev, kats, case):
    """tests/vulkan.cpp:998-1089 and :1158-1209: input, weights and bias are graph inputs."""
    k = kats[case]
    x, wt, b, exp = arr(k["input"]), arr(k["weights"]), arr(k["bias"]), arr(k["expected"])
    w = sw.SpvAsm()
    ids = [w.input(n, abi.dtype_of_numpy(t.dtype), t.shape) for n, t in (("input", x), ("weights", wt), ("bias", b))]
    out = w.output("output", abi.dtype_of_numpy(exp.dtype), exp.shape)
    head, tail = conv_operands(w, k["attr"])
    w.set_output(w.op("CONV2D", abi.dtype_of_numpy(exp.dtype), exp.shape, head + ids + tail), out)
    got, _ = run_module(dev, w, {"input": x, "weights": wt, "bias": b})
    np.testing.assert_array_equal(got["output"], exp)


@pytest.mark.gpu
def test_kat_inlined_higher_rank_constant_module(dev, kats):
    """tests/vulkan.cpp:1636-1678: rank-4 weights inlined as nested composites, replicated attribute tensors, null
    zero points, CONV2D then CAST to the int8 output."""
    k = kats["higher_rank_constant"]
    a, x, exp = k["attr"], arr(k["input"]), arr(k["expected"])
    w = sw.SpvAsm()
    xin = w.input("input", abi.I8, x.shape)
    out = w.output("output", abi.I8, exp.shape)
    weights = w.const(arr(k["weights"]))
    assert w.text().count("OpConstantComposite %tensor_uint8_") >= 1 + 3 + 9  # one composite per level and row
    zero = w.const(np.zeros(1, np.int8), replicate=True)
    operands = [w.const(np.array(a["pad"], np.int32), replicate=True),
                w.const(np.array(a["stride"], np.int32), replicate=True),
                w.const(np.array(a["dilation"], np.int32), replicate=True), w.u32(a["acc_type"]),
                w.scalar(abi.BOOL, False), xin, weights, w.const(arr(k["bias"])), zero, zero]
    assert "OpConstantCompositeReplicateEXT" in w.text()
    acc = w.op("CONV2D", abi.I32, exp.shape, operands)
    w.set_output(w.op("CAST", abi.I8, exp.shape, [acc]), out)
    got, names = run_module(dev, w, {"input": x}, fuse=False)
    assert names == ["CONV2D", "CAST"]
    np.testing.assert_array_equal(got["output"], exp)


@pytest.mark.gpu
def test_kat_max_pool_modules(dev, kats):
    """tests/vulkan.cpp:611-658 (input = element 1 of a tensor array, unshaped types) and :752-792 (two layers, the
    intermediate tensor typed with its shape)."""
    k, k2 = kats["max_pool2d"], kats["two_layer_max_pool2d"]
    a, x = k["attr"], arr(k["input"])
    for layers, exp in ((1, arr(k["expected"])), (2, arr(k2["expected"]))):
        w = sw.SpvAsm("maxpool")
        if layers == 1:
            value = w.tensor_array("inputs", abi.I8, [x.shape] * 4, as_input=True, used=[1])[1]
            feed = {"inputs1": x}
            del w.bindings[(0, 0, 0)], w.bindings[(0, 0, 2)], w.bindings[(0, 0, 3)]  # unused elements stay undescribed
        else:
            value = w.input("inputs1", abi.I8, x.shape, shaped=False)
            feed = {"inputs1": x}
        out = w.output("output", abi.I8, exp.shape, shaped=False)
        attrs = [w.attr(a["kernel"]), w.attr(a["stride"]), w.attr(a["pad"]), w.u32(a["nan_mode"])]
        if layers == 2:
            value = w.op("MAX_POOL2D", abi.I8, k2["intermediate_shape"], attrs + [value])
        w.set_output(w.op("MAX_POOL2D", abi.I8, exp.shape, attrs + [value], shaped=False), out)
        got, names = run_module(dev, w, feed)
        assert names == ["MAX_POOL2D"] * layers
        np.testing.assert_array_equal(got["output"], exp)


@pytest.mark.gpu
def test_kat_graph_constant_module(dev, kats):
    """tests/vulkan.cpp:1579-1634: RESCALE, RESCALE, ADD, RESCALE with every multiplier and shift an
    OpGraphConstantARM and every zero point an OpConstantNull."""
    k = kats["graph_constant_arm"]
    r = k["rescale"]
    a, b, exp = arr(k["input0"]), arr(k["input1"]), arr(k["expected"])
    for fuse in (False, True):
        w = sw.SpvAsm()
        ia, ib = w.input("input0", abi.I8, a.shape), w.input("input1", abi.I8, b.shape)
        out = w.output("output", abi.I8, exp.shape)
        flags = [w.scalar(abi.BOOL, r["scale32"]), w.u32(3 if r["double_round"] else 1),
                 w.scalar(abi.BOOL, r["per_channel"]), w.scalar(abi.BOOL, False), w.scalar(abi.BOOL, False)]
        z8, z32 = w.const(np.zeros(1, np.int8), replicate=True), w.const(np.zeros(1, np.int32), replicate=True)
        consts = []
        for i in range(3):
            consts.append((w.const(np.array([k["multipliers"][i]], np.int32), graph_constant=2 * i),
                           w.const(np.array([k["shifts"][i]], np.int8), graph_constant=2 * i + 1)))
        ra = w.op("RESCALE", abi.I32, a.shape, flags + [ia, consts[0][0], consts[0][1], z8, z32])
        rb = w.op("RESCALE", abi.I32, b.shape, flags + [ib, consts[1][0], consts[1][1], z8, z32])
        s = w.op("ADD", abi.I32, a.shape, [ra, rb])
        w.set_output(w.op("RESCALE", abi.I8, exp.shape, flags + [s, consts[2][0], consts[2][1], z32, z8]), out)
        assert len(w.constants) == 6
        got, names = run_module(dev, w, {"input0": a, "input1": b}, fuse=fuse)
        assert len(names) == (1 if fuse else 4)
        np.testing.assert_array_equal(got["output"], exp)


@pytest.mark.gpu
def test_kat_data_movement_modules(dev, kats):
    """tests/vulkan.cpp:1333-1404 (CONCAT), :1406-1439 (ADD, CONCAT, RESHAPE), :1441-1492 (SLICE), :1680-1744
    (MAXIMUM), :1796-1842 (SIN), each as a module of the structure of the reference's."""
    k = kats["concat"]
    w = sw.SpvAsm("concat")
    a, b, exp = arr(k["input0"]), arr(k["input1"]), arr(k["expected"])
    ia, ib = w.input("input0", abi.I8, a.shape, shaped=False), w.input("input1", abi.I8, b.shape, shaped=False)
    out = w.output("output", abi.I8, exp.shape, shaped=False)
    w.set_output(w.op("CONCAT", abi.I8, exp.shape, [w.u32(k["axis"]), ia, ib], shaped=False), out)
    np.testing.assert_array_equal(run_module(dev, w, {"input0": a, "input1": b})[0]["output"], exp)

    k = kats["concat_interval"]
    w = sw.SpvAsm()
    x, one, zero, exp = arr(k["input"]), arr(k["one"]), arr(k["zero"]), arr(k["expected"])
    ix, io, iz = (w.input(n, abi.F32, t.shape) for n, t in (("input", x), ("one", one), ("zero", zero)))
    out = w.output("output", abi.F32, exp.shape)
    s = w.op("ADD", abi.F32, (3, 3), [ix, io])
    c = w.op("CONCAT", abi.F32, (3, 4), [w.u32(1), s, iz])
    w.set_output(w.op("RESHAPE", abi.F32, (12,), [c, w.attr([12])]), out)
    got, names = run_module(dev, w, {"input": x, "one": one, "zero": zero})
    np.testing.assert_array_equal(got["output"], exp)

    k = kats["slice"]
    w = sw.SpvAsm()
    x, exp = arr(k["input"]), arr(k["expected"])
    ix = w.input("input", abi.I8, x.shape, shaped=False)
    out = w.output("output", abi.I8, exp.shape, shaped=False)
    w.set_output(w.op("SLICE", abi.I8, exp.shape, [ix, w.attr(k["start"]), w.attr(k["size"])], shaped=False), out)
    np.testing.assert_array_equal(run_module(dev, w, {"input": x})[0]["output"], exp)

    k = kats["maximum"]
    w = sw.SpvAsm()
    a, b, exp = arr(k["input0"]), arr(k["input1"]), arr(k["expected"])
    ia, ib = w.input("input0", abi.I32, a.shape, shaped=False), w.input("input1", abi.I32, b.shape, shaped=False)
    out = w.output("output", abi.I32, exp.shape, shaped=False)
    w.set_output(w.op("MAXIMUM", abi.I32, exp.shape, [w.u32(k["nan_mode"]), ia, ib], shaped=False), out)
    np.testing.assert_array_equal(run_module(dev, w, {"input0": a, "input1": b})[0]["output"], exp)

    k = kats["sin"]
    w = sw.SpvAsm()
    x = np.full((6, 5, 4), k["input"], np.float32)
    w.set_output(w.op("SIN", abi.F32, x.shape, [w.input("input", abi.F32, x.shape)]),
                 w.output("output", abi.F32, x.shape))
    got = run_module(dev, w, {"input": x})[0]["output"]
    assert np.all(np.abs(got.astype(np.float64) - k["reference"]) <= k["error_bound"])


@pytest.mark.gpu
def test_kat_nop_outputs_module(dev, kats):
    """tests/vulkan.cpp:1494-1577: one operator result, the graph input itself and a graph constant of unshaped type
    are each routed to an output."""
    k = kats["nop_outputs"]
    x, const = arr(k["input"]), arr(k["constant"])
    s = kats["slice"]
    w = sw.SpvAsm("no-op")
    ix = w.input("input", abi.I8, x.shape, shaped=False)
    outs = [w.output(f"output{i}", abi.I8, shape, shaped=False) for i, shape in
            enumerate((s["size"], x.shape, const.shape))]
    sliced = w.op("SLICE", abi.I8, s["size"], [ix, w.attr(s["start"]), w.attr(s["size"])], shaped=False)
    # a graph constant whose tensor type carries no shape: the shape travels with the data
    t = w.tensor_type(abi.I8, rank=const.ndim)
    w.declarations.append(f"%const_tensor = OpGraphConstantARM {t} 0")
    w.constants[0] = const
    w.set_output(sliced, outs[0])
    w.set_output(ix, outs[1])
    w.set_output("%const_tensor", outs[2])
    got, names = run_module(dev, w, {"input": x})
    assert names == ["SLICE", "CAST", "CAST"]
    x8 = x.astype(np.int8)
    st, sz = s["start"], s["size"]
    np.testing.assert_array_equal(got["output0"], x8[tuple(slice(a, a + n) for a, n in zip(st, sz))])
    np.testing.assert_array_equal(got["output1"], x8)
    np.testing.assert_array_equal(got["output2"], const)


def random_input(spec, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(-128, 127, spec.inputs[0][2], endpoint=True).astype(np.int8)


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["inverted_residual", "mobilenetv2"])
@pytest.mark.parametrize("fuse", [False, True], ids=["unfused", "fused"])
def test_int8_graphs_from_assembly_vs_oracle(dev, oracle, which, fuse):
    spec = small_specs()[which]
    x = random_input(spec, 77)
    exp, _ = run_spec(oracle, spec, {"input": x})
    w = sw.from_spec(spec, inline_limit=64, shaped_io=not fuse)
    got, names = run_module(dev, w, {"input": x}, fuse=fuse)
    np.testing.assert_array_equal(got["output"], exp["output"])
    assert fuse or len(names) <= len(spec.ops)


@pytest.mark.gpu
def test_transformer_block_from_assembly_vs_oracle(dev, oracle):
    """fp16 graph: f16 literals, float zero points on MATMUL, REDUCE / TRANSPOSE / RESHAPE attribute decoding."""
    spec = graphs.transformer_block_spec(batch=2, seq=64, d_model=64, heads=4, ffn=128)
    rng = np.random.default_rng(5)
    x = rng.standard_normal(spec.inputs[0][2]).astype(np.float16)
    exp, _ = run_spec(oracle, spec, {"input": x})
    w = sw.from_spec(spec, inline_limit=16)
    got, _ = run_module(dev, w, {"input": x})
    assert np.max(np.abs(got["output"].astype(np.float32) - exp["output"].astype(np.float32))) <= 1e-2


@pytest.mark.gpu
def test_config3_mobilenetv2_b32_from_assembly_equals_direct_build(dev):
    """BASELINE config 3 through the front-end: same fused operator list and bit-identical logits as the graph
    built call by call."""
    spec = graphs.mobilenetv2_spec(batch=32, spread=True)
    x = random_input(spec, 1003)
    w = sw.from_spec(spec)
    got, names = run_module(dev, w, {"input": x})
    g = graphs.build(dev, spec, fuse=True)
    g.set_input("input", x)
    g.dispatch()
    direct = g.get_output("output")
    assert names == g.op_names() and len(names) == 38
    g.close()
    np.testing.assert_array_equal(got["output"], direct)


@pytest.mark.gpu
def test_kat_conv3d_module(dev, kats):
    """tests/vulkan.cpp:1211-1290 as a module: weights in an OpGraphConstantARM, null bias of length 1, attribute
    tensors of six and three values."""
    from test_oracle_kats import conv3d_kat
    x, wt, exp, a = conv3d_kat(kats["conv3d_large_stride"])
    w = sw.SpvAsm("conv3d_large_stride")
    xin = w.input("input", abi.I8, x.shape)
    out = w.output("output", abi.I32, exp.shape)
    operands = [w.attr(a[0]), w.attr(a[1]), w.attr(a[2]), w.u32(a[5]), w.scalar(abi.BOOL, False), xin,
                w.const(wt, graph_constant=0), w.attr([0]), w.attr([a[3]], abi.I8), w.attr([a[4]], abi.I8)]
    w.set_output(w.op("CONV3D", abi.I32, exp.shape, operands), out)
    got, names = run_module(dev, w, {"input": x})
    assert names == ["CONV3D"]
    np.testing.assert_array_equal(got["output"], exp)


@pytest.mark.gpu
def test_multi_result_and_specialised_modules(dev, oracle):
    """FFT2D / RFFT2D (two results picked apart with OpCompositeExtract), ARITHMETIC_RIGHT_SHIFT whose rounding flag is a
    specialization constant, RESIZE and SCATTER operand decoding."""
    rng = np.random.default_rng(8)
    re, im = rng.standard_normal((1, 4, 16)).astype(np.float32), rng.standard_normal((1, 4, 16)).astype(np.float32)
    w = sw.SpvAsm()
    a, b = w.input("real", abi.F32, re.shape), w.input("imag", abi.F32, im.shape)
    o0, o1 = w.output("out_real", abi.F32, re.shape), w.output("out_imag", abi.F32, re.shape)
    t = w.tensor_type(abi.F32, re.shape)
    w.declarations.append(f"%pair = OpTypeStruct {t} {t}")
    w.body.append(f"%fft = OpExtInst %pair %tosa FFT2D {w.scalar(abi.BOOL, False)} {w.scalar(abi.BOOL, False)} {a} {b}")
    w.body.append(f"%fft_re = OpCompositeExtract {t} %fft 0")
    w.body.append(f"%fft_im = OpCompositeExtract {t} %fft 1")
    w.set_output("%fft_re", o0)
    w.set_output("%fft_im", o1)
    got, names = run_module(dev, w, {"real": re, "imag": im})
    er, ei = oracle.fft2d(re, im)
    assert names == ["FFT2D"]
    assert np.abs(got["out_real"] - er).max() <= 1e-3 and np.abs(got["out_imag"] - ei).max() <= 1e-3

    # RFFT2D feeding a second operator: the extracted members are ordinary values
    w = sw.SpvAsm()
    x = w.input("input", abi.F32, re.shape)
    out = w.output("output", abi.F32, (1, 4, 9))
    t = w.tensor_type(abi.F32, (1, 4, 9))
    w.declarations.append(f"%pair = OpTypeStruct {t} {t}")
    w.body.append(f"%rfft = OpExtInst %pair %tosa RFFT2D {w.scalar(abi.BOOL, False)} {x}")
    w.body.append(f"%r_re = OpCompositeExtract {t} %rfft 0")
    w.body.append(f"%r_im = OpCompositeExtract {t} %rfft 1")
    w.set_output(w.op("ADD", abi.F32, (1, 4, 9), ["%r_re", "%r_im"]), out)
    got, names = run_module(dev, w, {"input": re})
    rr, rimag = oracle.rfft2d(re)
    assert names == ["RFFT2D", "ADD"] and np.abs(got["output"] - (rr + rimag)).max() <= 1e-3

    # ARITHMETIC_RIGHT_SHIFT: `round` is OpSpecConstantFalse with SpecId 0; specialising it to true changes the result
    v = np.array([-7, 7, 100, -100, 3, -3, 1, 0], np.int16)
    s = np.array([1, 1, 3, 3, 2, 2, 1, 5], np.int16)
    for spec, round_ in (({}, False), ({0: 1}, True)):
        w = sw.SpvAsm("spec_arshift")
        i0, i1 = w.input("in0", abi.I16, v.shape), w.input("in1", abi.I16, s.shape)
        out = w.output("out0", abi.I16, v.shape)
        w.decorations.append("OpDecorate %roundc SpecId 0")
        w.declarations.append(f"%roundc = OpSpecConstantFalse {w.scalar_type(abi.BOOL)}")
        w.set_output(w.op("ARITHMETIC_RIGHT_SHIFT", abi.I16, v.shape, ["%roundc", i0, i1]), out)
        g = gb.Graph(dev)
        ins, outs, _ = g.load_spvasm(w.text(), w.bindings, w.constants, w.names, specializations=spec)
        g.finalize()
        g.set_input("in0", v)
        g.set_input("in1", s)
        g.dispatch()
        np.testing.assert_array_equal(g.get_output("out0"), oracle.arithmetic_right_shift(v, s, v.shape, round_))
        g.close()

    # RESIZE (mode input scale offset border) and SCATTER (valuesIn indices input)
    x8 = rng.integers(-128, 127, (1, 5, 6, 3), endpoint=True).astype(np.int8)
    w = sw.SpvAsm()
    xin = w.input("input", abi.I8, x8.shape)
    out = w.output("output", abi.I32, (1, 9, 11, 3))
    w.set_output(w.op("RESIZE", abi.I32, (1, 9, 11, 3), [w.u32(2), xin, w.attr([4, 2, 4, 2]), w.attr([0, 0]), w.attr([0, 0])]),
                 out)
    got, _ = run_module(dev, w, {"input": x8})
    np.testing.assert_array_equal(got["output"], oracle.resize(x8, (1, 9, 11, 3), abi.I32,
                                                             abi.resize_attr((4, 2, 4, 2), (0, 0), (0, 0), 2)))
    vals = rng.integers(-99, 99, (2, 7, 3)).astype(np.int32)
    idx = np.array([[1, 3, 5, 0], [6, 2, 4, 1]], np.int32)
    inp = rng.integers(-99, 99, (2, 4, 3)).astype(np.int32)
    w = sw.SpvAsm()
    iv, ii, ix = w.input("values", abi.I32, vals.shape), w.input("indices", abi.I32, idx.shape), w.input("input", abi.I32, inp.shape)
    out = w.output("output", abi.I32, vals.shape)
    w.set_output(w.op("SCATTER", abi.I32, vals.shape, [iv, ii, ix]), out)
    got, _ = run_module(dev, w, {"values": vals, "indices": idx, "input": inp})
    np.testing.assert_array_equal(got["output"], oracle.scatter(vals, idx, inp))


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [abi.BF16, abi.F8E4M3, abi.F8E5M2], ids=["bf16", "f8e4m3", "f8e5m2"])
def test_inline_constants_of_reduced_precision_types(dev, oracle, dt):
    """The structure of tests/shader/conv3d_inline_{bf16,fp8e4m3,fp8e5m2}_constant.spvasm (the reference only checks
    that these pipelines are created and dispatched, tests/vulkan.cpp:1319-1329): a 1x1x1 CONV3D over a tensor of a
    reduced-precision type whose weights and bias are replicated inline constants, once with the modules' integer
    accumulator (operands truncated toward zero) and once with the floating-point accumulator of the type."""
    enc = lambda values: oracle.cast(np.asarray(values, np.float32), dt)
    shape = (1, 2, 1, 2, 1)
    x = enc(np.float32([2.0, -3.5, 1.5, 0.75]).reshape(shape))
    for acc, wv, bv in ((abi.ACC_I32, 1.0, 1.0), (abi.ACC_F32 if dt == abi.BF16 else abi.ACC_F16, 2.5, 0.25)):
        w = sw.SpvAsm("inline_encoded_constant")
        xin = w.input("input", dt, shape)
        out = w.output("output", dt, shape)
        weights = w.const(np.full((1, 1, 1, 1, 1), wv, np.float32), dt, replicate=True)
        bias = w.const(np.full((1,), bv, np.float32), dt, replicate=True)
        operands = [w.attr([0] * 6), w.attr([1] * 3), w.attr([1] * 3), w.u32(acc), w.scalar(abi.BOOL, False), xin,
                    weights, bias, w.attr([0], abi.I8), w.attr([0], abi.I8)]
        w.set_output(w.op("CONV3D", dt, shape, operands), out)
        got, names = run_module(dev, w, {"input": np.asarray(x)})
        assert names == ["CONV3D"]
        want = oracle.conv3d(x, enc(np.full((1, 1, 1, 1, 1), wv)), enc(np.full((1,), bv)), shape, dt,
                             abi.conv3d_attr(acc_type=acc))
        np.testing.assert_array_equal(got["output"], want)
        values = oracle.cast(want, abi.F32).ravel()
        if acc == abi.ACC_I32:
            np.testing.assert_array_equal(values, [3.0, -2.0, 2.0, 1.0])  # trunc(x) * 1 + 1
        else:
            np.testing.assert_array_equal(values, oracle.cast(enc(np.float32([5.25, -8.5, 4.0, 2.125])), abi.F32).ravel())
