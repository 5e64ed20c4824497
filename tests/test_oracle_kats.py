"""The CPU oracle against every known-answer vector the reference's own tests hold for the TOSA path
(fixtures: tests/golden/reference_kats.json, transcribed from the reference's tests/vulkan.cpp)."""
import numpy as np
import pytest

from conftest import fixture_array as arr


def _conv_attr(abi, a):
    return abi.conv2d_attr(a["pad"], a["stride"], a["dilation"], a["input_zp"], a["weight_zp"], a["acc_type"])


def test_conv2d_kat(kats, abi, oracle):
    k = kats["conv2d"]
    exp = arr(k["expected"])
    out = oracle.conv2d(arr(k["input"]), arr(k["weights"]), arr(k["bias"]), exp.shape, abi.I32,
                        _conv_attr(abi, k["attr"]))
    np.testing.assert_array_equal(out, exp)


def test_conv2d_kat_generic_path_matches_fast_path(kats, abi, oracle):
    """Non-contiguous views force the generic accessor path of the oracle; it must agree with the packed path."""
    k = kats["conv2d"]
    x = arr(k["input"])
    xs = np.zeros((1, 8, 8, 5), np.int8)[..., :3]
    xs[...] = x
    exp = arr(k["expected"])
    out = oracle.conv2d(xs, arr(k["weights"]), arr(k["bias"]), exp.shape, abi.I32, _conv_attr(abi, k["attr"]))
    np.testing.assert_array_equal(out, exp)


def test_higher_rank_constant_kat(kats, abi, oracle):
    k = kats["higher_rank_constant"]
    exp = arr(k["expected"])
    acc = oracle.conv2d(arr(k["input"]), arr(k["weights"]), arr(k["bias"]), exp.shape, abi.I32,
                        _conv_attr(abi, k["attr"]))
    out = oracle.cast(acc, abi.I8)
    np.testing.assert_array_equal(out, exp)


def test_conv2d_acc_int64_kat(kats, abi, oracle):
    k = kats["conv2d_acc_int64"]
    exp = arr(k["expected"])
    out = oracle.conv2d(arr(k["input"]), arr(k["weights"]), arr(k["bias"]), exp.shape, abi.I64,
                        _conv_attr(abi, k["attr"]))
    np.testing.assert_array_equal(out, exp)


@pytest.mark.parametrize("shape", [(1, 1, 1), (1, 1, 2053), (1, 2053, 1)])
def test_conv2d_all_ones_closed_form(kats, abi, oracle, shape):
    """Reference: all-ones 1x1 conv, every output equals IC (run there at OC=262144 and H/W=524281; the
    closed form is size independent, so the oracle is checked at reduced sizes and once at the full OC)."""
    c = kats["conv2d_all_ones"]["channels"]
    n, h, w = shape
    x = np.ones((n, h, w, c), np.int8)
    wt = np.ones((c, 1, 1, c), np.int8)
    b = np.zeros(c, np.int32)
    out = oracle.conv2d(x, wt, b, (n, h, w, c), abi.I32, abi.conv2d_attr())
    assert (out == c).all()


def test_conv2d_large_output_channels(kats, abi, oracle):
    oc = kats["conv2d_all_ones"]["large_oc"]
    x = np.ones((1, 1, 1, 4), np.int8)
    wt = np.ones((oc, 1, 1, 4), np.int8)
    out = oracle.conv2d(x, wt, np.zeros(oc, np.int32), (1, 1, 1, oc), abi.I32, abi.conv2d_attr())
    assert (out == 4).all()


def test_max_pool2d_kat(kats, abi, oracle):
    k = kats["max_pool2d"]
    a = k["attr"]
    exp = arr(k["expected"])
    out = oracle.max_pool2d(arr(k["input"]), exp.shape,
                            abi.pool2d_attr(a["kernel"], a["stride"], a["pad"], nan_mode=a["nan_mode"]))
    np.testing.assert_array_equal(out, exp)


def test_two_layer_max_pool2d_kat(kats, abi, oracle):
    k = kats["two_layer_max_pool2d"]
    a = k["attr"]
    attr = abi.pool2d_attr(a["kernel"], a["stride"], a["pad"], nan_mode=a["nan_mode"])
    exp = arr(k["expected"])
    mid = oracle.max_pool2d(arr(k["input"]), k["intermediate_shape"], attr)
    out = oracle.max_pool2d(mid, exp.shape, attr)
    np.testing.assert_array_equal(out, exp)


def test_graph_constant_arm_kat(kats, abi, oracle):
    """RESCALE x2 + RESCALE x3 -> ADD(i32) -> RESCALE x4 with shift 0: the residual-add pattern."""
    k = kats["graph_constant_arm"]
    r = k["rescale"]
    attr = abi.rescale_attr(r["input_zp"], r["output_zp"], r["scale32"], r["double_round"], r["per_channel"],
                            r["input_unsigned"], r["output_unsigned"])
    m = [np.array([v], np.int32) for v in k["multipliers"]]
    s = [np.array([v], np.int8) for v in k["shifts"]]
    a = oracle.rescale(arr(k["input0"]), m[0], s[0], abi.I32, attr)
    b = oracle.rescale(arr(k["input1"]), m[1], s[1], abi.I32, attr)
    c = oracle.elementwise_binary("ADD", a, b, a.shape, abi.I32)
    out = oracle.rescale(c, m[2], s[2], abi.I8, attr)
    np.testing.assert_array_equal(out, arr(k["expected"]))


def test_concat_kat(kats, abi, oracle):
    k = kats["concat"]
    out = oracle.concat([arr(k["input0"]), arr(k["input1"])], k["axis"])
    np.testing.assert_array_equal(out, arr(k["expected"]))


def test_concat_interval_kat(kats, abi, oracle):
    k = kats["concat_interval"]
    s = oracle.elementwise_binary("ADD", arr(k["input"]), arr(k["one"]), (3, 3), abi.F32)
    c = oracle.concat([s, arr(k["zero"])], 1)
    out = oracle.reshape(c, (12,))
    np.testing.assert_array_equal(out, arr(k["expected"]))


def test_slice_kat(kats, abi, oracle):
    k = kats["slice"]
    out = oracle.slice_(arr(k["input"]), k["start"], k["size"])
    np.testing.assert_array_equal(out, arr(k["expected"]))


def test_nop_outputs_kat(kats, abi, oracle):
    """Pass-through graph outputs are implemented as CAST to the same type: identity."""
    k = kats["nop_outputs"]
    for name in ("input", "constant"):
        x = arr(k[name])
        np.testing.assert_array_equal(oracle.cast(x, abi.I8), x)


def test_maximum_kat(kats, abi, oracle):
    k = kats["maximum"]
    out = oracle.elementwise_binary("MAXIMUM", arr(k["input0"]), arr(k["input1"]), k["expected"]["shape"], abi.I32,
                                    k["nan_mode"])
    np.testing.assert_array_equal(out, arr(k["expected"]))


def test_sin_kat(kats, abi, oracle):
    k = kats["sin"]
    out = oracle.elementwise_unary("SIN", np.array([k["input"]], np.float32))
    assert abs(float(out[0]) - k["reference"]) <= k["error_bound"]


def conv3d_kat(k):
    w = np.zeros(k["weights_shape"], np.int8)
    w[:, :, :, 8190:8192, :] = np.array(k["relevant_weights"], np.int8).reshape(3, 2, 2, 2, 4)
    a = k["attr"]
    return arr(k["input"]), w, arr(k["expected"]), (a["pad"], a["stride"], a["dilation"], a["input_zp"], a["weight_zp"],
                                                   a["acc_type"])


def test_kat_conv3d_large_stride(oracle, kats, abi):
    """tests/vulkan.cpp:1211-1290: CONV3D with a kernel 8192 wide, pad (1,0,1,0,8190,8192), stride (1,1,8192), input
    zero point 9; a null bias of length 1 is broadcast."""
    x, w, exp, a = conv3d_kat(kats["conv3d_large_stride"])
    out = oracle.conv3d(x, w, np.zeros(1, np.int32), exp.shape, abi.I32, abi.conv3d_attr(*a))
    np.testing.assert_array_equal(out, exp)
