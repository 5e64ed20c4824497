"""The binary SPIR-V front-end (mlel_graph_load_spirv, csrc/graph/spirv_graph_loader.cpp: decodeWords).

The words are produced by tests/spv_assembler.py from the same assembly text the text front-end reads: the
reference's own test modules (tests/shader/*.spvasm, when the reference checkout is present) and the modules
tests/spvasm_writer.py writes for the benchmark graphs.  Both loaders must record the same graph, and on the GPU
compute the same bytes.

Parity unpinned for the numbers themselves: the opcode, enumerant and "TOSA.001000.1" instruction numbers in the
decoder and in the assembler are two independent restatements of the published grammar; the SPIRV-Headers package
the reference takes them from is not available here, so neither is checked against it.
"""
import os

import numpy as np
import pytest

import spv_assembler as sa
import spvasm_writer as sw
from hip_util import gpu_available, hb
from test_spirv_frontend import REFERENCE_MODULES, REFERENCE_SHADERS, _NoDevice, abi, described, gb, small_specs


def decode_words(words, bindings=None, constants=None, names=None, fuse=False):
    g = gb.Graph(_NoDevice())
    ins, outs, count = g.load_spirv(words, bindings, constants, names)
    g._check(g.lib.mlel_graph_finalize(g.g, 1 if fuse else 0))
    return g, ins, outs, count


# ------------------------------------------------------------------------------------------------- the word stream
def test_assembled_words_follow_the_published_layout():
    """Spot checks of the assembler against encodings that can be written down by hand from the SPIR-V
    specification: header, word count in the upper half of the first word, result id before operands, strings
    nul-terminated and padded, 64-bit literals low word first, narrow signed literals sign-extended."""
    words = sa.assemble('%i = OpTypeInt 32 0\n%l = OpTypeInt 64 1\n%b = OpTypeInt 8 1\n%t = OpExtInstImport "TOSA.001000.1"\n'
                        "%c = OpConstant %i 7\n%d = OpConstant %l -2\n%e = OpConstant %b -3\n").tolist()
    assert words[:5] == [0x07230203, 0x00010600, 0, 8, 0]
    assert words[5:9] == [(4 << 16) | 21, 1, 32, 0]
    assert words[9:13] == [(4 << 16) | 21, 2, 64, 1]
    assert words[13:17] == [(4 << 16) | 21, 3, 8, 1]
    text = b"TOSA.001000.1\0\0\0"
    assert words[17:23] == [(6 << 16) | 11, 4] + [int.from_bytes(text[i:i + 4], "little") for i in range(0, 16, 4)]
    assert words[23:27] == [(4 << 16) | 43, 1, 5, 7]
    assert words[27:32] == [(5 << 16) | 43, 2, 6, 0xFFFFFFFE, 0xFFFFFFFF]
    assert words[32:36] == [(4 << 16) | 43, 3, 7, 0xFFFFFFFD]


@pytest.mark.skipif(not os.path.isdir(REFERENCE_SHADERS), reason="reference checkout not present")
@pytest.mark.parametrize("name", sorted(REFERENCE_MODULES))
def test_reference_modules_decode_from_words(name):
    """Every reference module the text front-end decodes gives the same interface and operators from words."""
    bindings, constants, exp_in, exp_out, exp_ops = REFERENCE_MODULES[name]
    with open(os.path.join(REFERENCE_SHADERS, name)) as f:
        words = sa.assemble(f.read())
    g, ins, outs, count = decode_words(words, bindings, constants)
    assert described(g, ins) == exp_in
    assert described(g, outs) == exp_out
    assert g.op_names() == exp_ops
    g.close()


@pytest.mark.parametrize("which", ["inverted_residual", "mobilenetv2", "transformer"])
@pytest.mark.parametrize("swapped", [False, True], ids=["native", "byte_swapped"])
def test_words_record_the_same_graph_as_text(which, swapped):
    w = sw.from_spec(small_specs()[which], inline_limit=64, shaped_io=False)
    gt = gb.Graph(_NoDevice())
    t_in, t_out, t_count = gt.load_spvasm(w.text(), w.bindings, w.constants, w.names)
    gt._check(gt.lib.mlel_graph_finalize(gt.g, 1))
    g, ins, outs, count = decode_words(sa.assemble(w.text(), byte_swapped=swapped), w.bindings, w.constants, w.names, fuse=True)
    assert (ins, outs, count) == (t_in, t_out, t_count)
    assert described(g, ins + outs) == described(gt, t_in + t_out)
    assert g.op_names() == gt.op_names()
    assert g.session_tensors() == gt.session_tensors()
    g.close()
    gt.close()


def test_malformed_modules_are_refused():
    good = sa.assemble(sw.from_spec(small_specs()["inverted_residual"]).text())

    def error_of(words):
        with pytest.raises(hb.MlelError) as e:
            decode_words(np.asarray(words, np.uint32))
        return str(e.value)

    assert "five-word header" in error_of(good[:4])
    assert "magic" in error_of(np.concatenate([[0x12345678], good[1:]]))
    assert "past the end" in error_of(good[:-1].tolist() + [(9 << 16) | 4186])
    assert "zero words" in error_of(good.tolist() + [4186])
    assert "more words than" in error_of(good.tolist() + [(2 << 16) | 4186, 0])
    # a module with no graph at all: only the header
    assert "no graph entry point" in error_of(good[:5])


def test_unknown_numbers_are_named_in_the_error():
    text = sw.from_spec(small_specs()["inverted_residual"]).text()
    words = sa.assemble(text).tolist()
    # the first OpExtInst: replace its instruction number by one past the table
    at = 5
    while (words[at] & 0xFFFF) != 12:
        at += words[at] >> 16
    bad = list(words)
    bad[at + 4] = len(sa.TOSA)
    with pytest.raises(hb.MlelError) as e:
        decode_words(np.asarray(bad, np.uint32))
    assert "instruction#%d" % len(sa.TOSA) in str(e.value)
    # an opcode the decoder has no layout for inside the graph body (OpNop)
    body = list(words)
    body.insert(at, (1 << 16) | 0)
    with pytest.raises(hb.MlelError) as e:
        decode_words(np.asarray(body, np.uint32))
    assert "Op#0" in str(e.value) and "word %d" % at in str(e.value)


# ------------------------------------------------------------------------------------------------------------ GPU
@pytest.fixture(scope="module")
def dev():
    if not gpu_available():
        pytest.skip("no GPU visible")
    d = hb.Device(0)
    yield d
    d.close()


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["inverted_residual", "mobilenetv2", "transformer"])
def test_binary_module_computes_the_same_bytes_as_text(dev, which):
    """Inline composites, replicated composites, graph constants and scalar attributes of every width arrive intact:
    the graph loaded from words produces the bytes of the graph loaded from text."""
    spec = small_specs()[which]
    w = sw.from_spec(spec, inline_limit=64)
    rng = np.random.default_rng(5)
    inputs = {}
    for name, dtype, shape in spec.inputs:
        if dtype == abi.I8:
            inputs[name] = rng.integers(-128, 127, shape, endpoint=True).astype(np.int8)
        else:
            inputs[name] = rng.standard_normal(shape).astype(abi.NP_OF[dtype])
    results = []
    for module in (w.text(), sa.assemble(w.text())):
        g = gb.Graph(dev)
        load = g.load_spvasm if isinstance(module, str) else g.load_spirv
        ins, outs, _ = load(module, w.bindings, w.constants, w.names)
        g.finalize(True)
        for name, array in inputs.items():
            g.set_input(name, array)
        g.dispatch()
        results.append({o: g.get_output(o) for o in outs})
        g.close()
    assert results[0].keys() == results[1].keys()
    for name in results[0]:
        a, b = results[0][name], results[1][name]
        np.testing.assert_array_equal(a.view(np.uint8), b.view(np.uint8))
