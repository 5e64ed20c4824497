"""GPU parity: every operator of the C ABI against the CPU oracle on the same seeded inputs (bit-exact for
integers, stated tolerance for floats), the reference's known-answer vectors run on the GPU, and the
BASELINE configs 0 and 1 at full size."""
import os
import zlib

import numpy as np
import pytest

from conftest import fixture_array as arr
from hip_util import Runner, abi, gpu_available, hb

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def run():
    if not gpu_available():
        pytest.skip("no GPU visible")
    dev = hb.Device(0)
    yield Runner(dev)
    dev.close()


def ri(rng, lo, hi, shape, dt):
    return rng.integers(lo, hi, size=shape, endpoint=True).astype(dt)


def rescale_params(rng, channels, per_channel=True):
    n = channels if per_channel else 1
    mult = ri(rng, 2 ** 30, 2 ** 31 - 1, (n,), np.int32)
    shift = ri(rng, 30, 38, (n,), np.int8)
    return mult, shift


# ------------------------------------------------------------------------------------------------ reference KATs
def test_kat_conv2d(run, kats):
    k = kats["conv2d"]
    a = k["attr"]
    exp = arr(k["expected"])
    attr = abi.conv2d_attr(a["pad"], a["stride"], a["dilation"], a["input_zp"], a["weight_zp"], a["acc_type"])
    out = run.conv2d(arr(k["input"]), arr(k["weights"]), arr(k["bias"]), exp.shape, abi.I32, attr)
    np.testing.assert_array_equal(out, exp)


def test_kat_higher_rank_constant(run, kats):
    k = kats["higher_rank_constant"]
    a = k["attr"]
    attr = abi.conv2d_attr(a["pad"], a["stride"], a["dilation"], a["input_zp"], a["weight_zp"], a["acc_type"])
    acc = run.conv2d(arr(k["input"]), arr(k["weights"]), arr(k["bias"]), k["expected"]["shape"], abi.I32, attr)
    np.testing.assert_array_equal(run.cast(acc, abi.I8), arr(k["expected"]))


def test_kat_conv2d_acc_int64(run, kats):
    k = kats["conv2d_acc_int64"]
    a = k["attr"]
    exp = arr(k["expected"])
    attr = abi.conv2d_attr(a["pad"], a["stride"], a["dilation"], a["input_zp"], a["weight_zp"], a["acc_type"])
    out = run.conv2d(arr(k["input"]), arr(k["weights"]), arr(k["bias"]), exp.shape, abi.I64, attr)
    np.testing.assert_array_equal(out, exp)


@pytest.mark.parametrize("which", ["oc", "w", "h"])
def test_kat_conv2d_large_dims(run, kats, which):
    """Reference sizes: OC = 262144, W or H = 524281 (beyond a Vulkan work-group-count limit there)."""
    k = kats["conv2d_all_ones"]
    c = k["channels"]
    if which == "oc":
        oc, h, w = k["large_oc"], 1, 1
    elif which == "w":
        oc, h, w = c, 1, k["large_spatial"]
    else:
        oc, h, w = c, k["large_spatial"], 1
    x = np.ones((1, h, w, c), np.int8)
    wt = np.ones((oc, 1, 1, c), np.int8)
    out = run.conv2d(x, wt, np.zeros(oc, np.int32), (1, h, w, oc), abi.I32, abi.conv2d_attr())
    assert out.shape == (1, h, w, oc) and (out == c).all()


def test_kat_max_pool2d_and_two_layers(run, kats):
    k = kats["max_pool2d"]
    a = k["attr"]
    attr = abi.pool2d_attr(a["kernel"], a["stride"], a["pad"], nan_mode=a["nan_mode"])
    out = run.pool("max_pool2d", arr(k["input"]), k["expected"]["shape"], attr)
    np.testing.assert_array_equal(out, arr(k["expected"]))
    k2 = kats["two_layer_max_pool2d"]
    out2 = run.pool("max_pool2d", out, k2["expected"]["shape"], attr)
    np.testing.assert_array_equal(out2, arr(k2["expected"]))


def test_kat_graph_constant_arm(run, kats):
    k = kats["graph_constant_arm"]
    r = k["rescale"]
    attr = abi.rescale_attr(r["input_zp"], r["output_zp"], r["scale32"], r["double_round"], r["per_channel"])
    m = [np.array([v], np.int32) for v in k["multipliers"]]
    s = [np.array([v], np.int8) for v in k["shifts"]]
    a = run.rescale(arr(k["input0"]), m[0], s[0], abi.I32, attr)
    b = run.rescale(arr(k["input1"]), m[1], s[1], abi.I32, attr)
    c = run.binary("ADD", a, b, a.shape, abi.I32)
    np.testing.assert_array_equal(run.rescale(c, m[2], s[2], abi.I8, attr), arr(k["expected"]))
    fused = run.rescale_add_rescale(arr(k["input0"]), (m[0], s[0], attr, None), arr(k["input1"]),
                                    (m[1], s[1], attr, None), (m[2], s[2], attr, None), abi.I8)
    np.testing.assert_array_equal(fused, arr(k["expected"]))


def test_kat_data_movement_and_maximum(run, kats):
    k = kats["concat"]
    np.testing.assert_array_equal(run.concat([arr(k["input0"]), arr(k["input1"])], k["axis"]), arr(k["expected"]))
    k = kats["slice"]
    np.testing.assert_array_equal(run.slice_(arr(k["input"]), k["start"], k["size"]), arr(k["expected"]))
    k = kats["concat_interval"]
    s = run.binary("ADD", arr(k["input"]), arr(k["one"]), (3, 3), abi.F32)
    np.testing.assert_array_equal(run.reshape(run.concat([s, arr(k["zero"])], 1), (12,)), arr(k["expected"]))
    k = kats["maximum"]
    out = run.binary("MAXIMUM", arr(k["input0"]), arr(k["input1"]), k["expected"]["shape"], abi.I32, k["nan_mode"])
    np.testing.assert_array_equal(out, arr(k["expected"]))
    k = kats["nop_outputs"]
    np.testing.assert_array_equal(run.cast(arr(k["input"]), abi.I8), arr(k["input"]))
    k = kats["sin"]
    out = run.unary("SIN", np.array([k["input"]], np.float32))
    assert abs(float(out[0]) - k["reference"]) <= k["error_bound"]


# ------------------------------------------------------------------------------------------------ CONV2D int8
CONV_CASES = [
    # name, x shape, OC, (KH,KW), pad, stride, dil, zi, zw
    ("c0_like_small", (1, 12, 12, 64), 64, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), -5, 0),
    ("stem_ic3_s2", (2, 17, 17, 3), 32, (3, 3), (0, 1, 0, 1), (2, 2), (1, 1), 7, 0),
    ("pw_24_144", (2, 9, 9, 24), 144, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), -3, 0),
    ("pw_144_24", (2, 9, 9, 144), 24, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 4, 0),
    ("pw_16_96_big_m", (3, 20, 21, 16), 96, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), -128, 0),
    ("both_zp", (1, 10, 7, 32), 40, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), 11, -7),
    ("dilated_rect", (1, 13, 11, 8), 10, (2, 3), (2, 0, 1, 2), (1, 2), (2, 1), -128, 127),
    ("odd_everything", (2, 7, 5, 5), 7, (3, 2), (1, 0, 0, 1), (2, 1), (1, 1), 3, 2),
    ("ic20_oc130", (1, 6, 6, 20), 130, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 1, 0),
    ("k_tail_ic48", (1, 5, 5, 48), 64, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 0, 0),
    ("pw_960_320", (1, 7, 7, 960), 320, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), -1, 0),
    ("pw_24_both_zp", (2, 9, 9, 24), 40, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 5, -3),
    ("pw_36_k_tail_dwords", (1, 5, 7, 36), 20, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), -2, 0),
    ("pw_72_two_k_steps", (3, 8, 8, 72), 24, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 9, 1),
    ("stem_ic3_s1_pad1_zw", (2, 11, 13, 3), 16, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), -128, 5),
    ("stem_ic3_s2_big", (3, 33, 31, 3), 32, (3, 3), (1, 0, 1, 0), (2, 2), (1, 1), 127, 0),
    ("stem_ic1", (2, 9, 10, 1), 16, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), 3, -3),
    ("stem_ic3_s1_pad1_16ch", (2, 12, 14, 3), 16, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), -9, 0),
    ("stem_ic3_s3_pad2", (1, 20, 23, 3), 32, (3, 3), (2, 1, 2, 0), (3, 3), (1, 1), 5, 0),
    ("stem_ic3_tall_s1x2", (3, 70, 9, 3), 32, (3, 3), (1, 1, 1, 1), (1, 2), (1, 1), -128, 0),
    ("stem_ic3_images_of_40", (5, 10, 12, 3), 32, (3, 3), (0, 0, 1, 1), (2, 1), (1, 1), 1, 0),
    ("stem_ic4_s3", (1, 14, 15, 4), 48, (3, 3), (2, 1, 0, 2), (3, 2), (1, 1), -7, 1),
    ("pw_32_16_zw", (2, 12, 12, 32), 16, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 6, -6),
    ("pw_32_192", (1, 28, 28, 32), 192, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), -100, 0),
    # enough positions for the direct kernel to take two per thread, ragged last block; a long run of 24-byte pixels
    ("pw_16_96_two_positions", (2, 223, 225, 16), 96, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 17, 0),
    ("pw_24_144_many_positions", (1, 251, 243, 24), 144, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), -9, 4),
    # short contractions on the matrix cores: half-used channel columns, 8-byte pixels, fewer positions than a group
    ("pw_8_16_tiny", (1, 5, 5, 8), 16, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 33, 0),
    ("pw_16_48", (2, 9, 11, 16), 48, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), -77, 0),
    ("pw_32_80", (3, 13, 7, 32), 80, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 127, 0),
    ("pw_24_176", (1, 31, 33, 24), 176, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), -128, 0),
    ("pw_32_16_many", (4, 56, 57, 32), 16, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 5, 0),
]


def out_hw(h, w, k, pad, stride, dil):
    oh = (h + pad[0] + pad[1] - (k[0] - 1) * dil[0] - 1) // stride[0] + 1
    ow = (w + pad[2] + pad[3] - (k[1] - 1) * dil[1] - 1) // stride[1] + 1
    return oh, ow


@pytest.mark.parametrize("case", CONV_CASES, ids=[c[0] for c in CONV_CASES])
def test_conv2d_i8_vs_oracle(run, oracle, case):
    name, xs, oc, k, pad, stride, dil, zi, zw = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    x = ri(rng, -128, 127, xs, np.int8)
    w = ri(rng, -128, 127, (oc,) + k + (xs[3],), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
    oh, ow = out_hw(xs[1], xs[2], k, pad, stride, dil)
    attr = abi.conv2d_attr(pad, stride, dil, zi, zw)
    shape = (xs[0], oh, ow, oc)
    exp = oracle.conv2d(x, w, b, shape, abi.I32, attr)
    out = run.conv2d(x, w, b, shape, abi.I32, attr)
    np.testing.assert_array_equal(out, exp)
    # fused RESCALE + CLAMP epilogue == the three operators one after another
    mult, shift = rescale_params(rng, oc)
    rattr = abi.rescale_attr(0, 3, True, True, True)
    exp8 = oracle.clamp(oracle.rescale(exp, mult, shift, abi.I8, rattr), -20, 90)
    out8 = run.conv2d(x, w, b, shape, abi.I8, attr, epilogue=(mult, shift, rattr, (-20, 90)))
    np.testing.assert_array_equal(out8, exp8)


def test_conv2d_bias_broadcast_and_strided_input(run, oracle):
    rng = np.random.default_rng(5)
    x = ri(rng, -128, 127, (1, 6, 6, 16), np.int8)
    w = ri(rng, -128, 127, (8, 3, 3, 16), np.int8)
    b = np.array([1234], np.int32)
    attr = abi.conv2d_attr((1, 1, 1, 1), input_zp=9)
    exp = oracle.conv2d(x, w, b, (1, 6, 6, 8), abi.I32, attr)
    np.testing.assert_array_equal(run.conv2d(x, w, b, (1, 6, 6, 8), abi.I32, attr), exp)
    # input rows padded to 32 bytes per pixel (explicit strides are honoured)
    strides = (6 * 6 * 32, 6 * 32, 32, 1)
    np.testing.assert_array_equal(run.conv2d(x, w, b, (1, 6, 6, 8), abi.I32, attr, x_strides=strides), exp)


def test_conv2d_i16_and_f32_generic(run, oracle):
    rng = np.random.default_rng(6)
    x = ri(rng, -3000, 3000, (1, 5, 5, 3), np.int16)
    w = ri(rng, -128, 127, (4, 3, 3, 3), np.int8)
    b = ri(rng, -10 ** 9, 10 ** 9, (4,), np.int64)
    attr = abi.conv2d_attr((1, 1, 1, 1), acc_type=abi.ACC_I64)
    np.testing.assert_array_equal(run.conv2d(x, w, b, (1, 5, 5, 4), abi.I64, attr),
                                  oracle.conv2d(x, w, b, (1, 5, 5, 4), abi.I64, attr))
    xf = rng.standard_normal((1, 5, 5, 3)).astype(np.float32)
    wf = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    bf = rng.standard_normal(4).astype(np.float32)
    attrf = abi.conv2d_attr((1, 1, 1, 1), acc_type=abi.ACC_F32)
    np.testing.assert_allclose(run.conv2d(xf, wf, bf, (1, 5, 5, 4), abi.F32, attrf),
                               oracle.conv2d(xf, wf, bf, (1, 5, 5, 4), abi.F32, attrf), rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------------------------ MATMUL int8
MM_CASES = [
    ("aligned", 2, 128, 128, 128, 2, -1),
    ("c1_like_small", 3, 96, 256, 192, 2, -1),
    ("ragged", 2, 37, 53, 29, -4, 6),
    ("n_mod4", 1, 64, 70, 36, 0, 0),
    ("fc_like", 1, 32, 1280, 1000, 0, 0),
    ("zp_a_only", 2, 33, 64, 64, 9, 0),
    ("zp_b_only", 2, 33, 64, 64, 0, -9),
    ("k_small", 4, 300, 8, 16, 1, 1),
]


@pytest.mark.parametrize("case", MM_CASES, ids=[c[0] for c in MM_CASES])
def test_matmul_i8_vs_oracle(run, oracle, case):
    name, nb, m, k, n, za, zb = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    a = ri(rng, -128, 127, (nb, m, k), np.int8)
    b = ri(rng, -128, 127, (nb, k, n), np.int8)
    exp = oracle.matmul(a, b, abi.I32, za, zb)
    np.testing.assert_array_equal(run.matmul(a, b, abi.I32, za, zb), exp)
    mult, shift = np.array([1518500250], np.int32), np.array([39], np.int8)
    rattr = abi.rescale_attr(0, 0, True, True, False)
    exp8 = oracle.rescale(exp, mult, shift, abi.I8, rattr)
    np.testing.assert_array_equal(run.matmul(a, b, abi.I8, za, zb, epilogue=(mult, shift, rattr, None)), exp8)
    # B handed over as a view of a matrix stored row-wise (what a graph does once with a constant weight matrix)
    np.testing.assert_array_equal(run.matmul(a, b, abi.I32, za, zb, b_rows=True), exp)
    np.testing.assert_array_equal(run.matmul(a, b, abi.I8, za, zb, epilogue=(mult, shift, rattr, None), b_rows=True), exp8)


DL_CASES = [
    # name, batches, M, K, N, a_zp, b_zp: sizes at which the direct-to-LDS tiles are chosen on a 256-CU device
    ("tile256_kmajor", 1, 4096, 128, 4096, 2, -1),        # 256 tiles of 256 x 256
    ("tile256_ragged", 1, 4000, 192, 4224, -3, 5),        # partial last tile row and column
    ("tile256_no_zp", 2, 2048, 64, 4096, 0, 0),           # a single K step, no zero-point sums
    ("tile128_band_walk", 1, 2944, 192, 2944, 7, 0),      # 529 tiles of 128 x 128, three K steps
    ("tile128_batched", 16, 640, 320, 1024, 0, -6),       # 5 x 8 tiles per batch, five K steps
    ("tile128_ring_once", 8, 512, 576, 1024, -1, 3),      # nine K steps: the eight-stage ring is filled and refilled
    ("tile128_ring_wraps", 4, 1024, 1600, 1024, 4, -2),   # 25 K steps: the ring wraps three times and drains
    # exactly one 128 x 128 tile per compute unit of a 256-CU device (config 1's geometry), even numbers of K steps
    ("tile128_one_per_cu_4_steps", 8, 512, 256, 1024, -2, 5),
    ("tile128_one_per_cu_no_zp", 8, 512, 384, 1024, 0, 0),
    ("tile128_one_per_cu_18_steps", 4, 1024, 1152, 1024, -7, -1),
    ("tile128_one_per_cu_ragged", 1, 2000, 512, 2032, 1, 2),      # partial last tile row and column
]


@pytest.mark.parametrize("case", DL_CASES, ids=[c[0] for c in DL_CASES])
def test_matmul_i8_direct_to_lds_tiles(run, oracle, case):
    """Large int8 MATMULs (K a multiple of 64) run on the direct-to-LDS pipeline with 256 x 256 or 128 x 128 tiles
    and the banded tile walk: int32 result and fused per-tensor RESCALE, bit for bit against the oracle."""
    name, nb, m, k, n, za, zb = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    a = ri(rng, -128, 127, (nb, m, k), np.int8)
    b = ri(rng, -128, 127, (nb, k, n), np.int8)
    exp = oracle.matmul(a, b, abi.I32, za, zb)
    np.testing.assert_array_equal(run.matmul(a, b, abi.I32, za, zb), exp)
    mult, shift = np.array([1518500250], np.int32), np.array([37], np.int8)
    rattr = abi.rescale_attr(0, -4, True, True, False)
    exp8 = oracle.rescale(exp, mult, shift, abi.I8, rattr)
    np.testing.assert_array_equal(run.matmul(a, b, abi.I8, za, zb, epilogue=(mult, shift, rattr, None)), exp8)
    assert len(np.unique(exp8)) > 100


def test_conv2d_i8_direct_to_lds_row_weights(run, oracle):
    """1x1 CONV2D with OHWI weights (row-major W) on the direct-to-LDS pipeline: 4096 positions x 4096 channels,
    IC = 128, per-channel RESCALE + CLAMP fused, and the int32 accumulator."""
    rng = np.random.default_rng(4242)
    x = ri(rng, -128, 127, (4, 32, 32, 128), np.int8)
    w = ri(rng, -127, 127, (4096, 1, 1, 128), np.int8)
    bias = ri(rng, -2 ** 15, 2 ** 15, (4096,), np.int32)
    attr = abi.conv2d_attr(input_zp=-5, weight_zp=3)
    acc = oracle.conv2d(x, w, bias, (4, 32, 32, 4096), abi.I32, attr)
    np.testing.assert_array_equal(run.conv2d(x, w, bias, (4, 32, 32, 4096), abi.I32, attr), acc)
    mult, shift = rescale_params(rng, 4096)
    rattr = abi.rescale_attr(0, 3, True, True, True)
    exp = np.clip(oracle.rescale(acc, mult, shift, abi.I8, rattr), -100, 90).astype(np.int8)
    out = run.conv2d(x, w, bias, (4, 32, 32, 4096), abi.I8, attr, epilogue=(mult, shift, rattr, (-100, 90)))
    np.testing.assert_array_equal(out, exp)


def test_conv2d_i8_direct_to_lds_ragged_channels(run, oracle):
    """The 128 x 128 tile of the direct-to-LDS pipeline where the channel extent is not a multiple of 16 and the positions
    are not a multiple of 128: the staged 8-bit tile leaves through the general stores (whole pieces, then the dwords of
    the last channels of a row), nothing is written beyond a row's end, and the int32 accumulator agrees as well."""
    rng = np.random.default_rng(777)
    oc = 2036  # 15 whole tiles of channels and one of 116: 7 whole pieces and a dword
    x = ri(rng, -128, 127, (4, 32, 31, 128), np.int8)
    w = ri(rng, -127, 127, (oc, 1, 1, 128), np.int8)
    bias = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
    attr = abi.conv2d_attr(input_zp=7, weight_zp=-2)
    acc = oracle.conv2d(x, w, bias, (4, 32, 31, oc), abi.I32, attr)
    np.testing.assert_array_equal(run.conv2d(x, w, bias, (4, 32, 31, oc), abi.I32, attr), acc)
    mult, shift = rescale_params(rng, oc)
    rattr = abi.rescale_attr(0, -3, True, True, True)
    exp = np.clip(oracle.rescale(acc, mult, shift, abi.I8, rattr), -128, 100).astype(np.int8)
    out = run.conv2d(x, w, bias, (4, 32, 31, oc), abi.I8, attr, epilogue=(mult, shift, rattr, (-128, 100)))
    np.testing.assert_array_equal(out, exp)


def test_matmul_float_generic(run, oracle):
    rng = np.random.default_rng(8)
    a = rng.standard_normal((2, 9, 33)).astype(np.float32)
    b = rng.standard_normal((2, 33, 12)).astype(np.float32)
    np.testing.assert_allclose(run.matmul(a, b, abi.F32), oracle.matmul(a, b, abi.F32), rtol=1e-5, atol=1e-5)
    a16, b16 = a.astype(np.float16), b.astype(np.float16)
    # fp16 inputs with fp32 accumulate: max abs error <= 1e-2
    out = run.matmul(a16, b16, abi.F32)
    assert np.max(np.abs(out - oracle.matmul(a16, b16, abi.F32))) <= 1e-2


HMM_CASES = [
    # name, batches, M, K, N
    ("proj_like", 1, 200, 768, 256),
    ("scores_like", 6, 128, 64, 128),
    ("av_like", 6, 128, 128, 64),
    ("ragged_m_n", 2, 77, 40, 72),
    ("k_tail", 1, 130, 104, 136),
    ("tiny", 1, 3, 8, 8),
    ("wide", 1, 64, 256, 1000),
]


@pytest.mark.parametrize("case", HMM_CASES, ids=[c[0] for c in HMM_CASES])
def test_matmul_f16_mfma_vs_oracle(run, oracle, case):
    """fp16 operands, fp32 result (the matrix-core kernel): max abs error <= 1e-2 against the oracle's sequential
    fp32 accumulation, on activations ~N(0,1) and weights ~N(0,0.02) as in config 4, and on unit-normal operands."""
    name, nb, m, k, n = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    a = rng.standard_normal((nb, m, k)).astype(np.float16)
    for scale in (0.02, 1.0):
        b = (scale * rng.standard_normal((nb, k, n))).astype(np.float16)
        exp = oracle.matmul(a, b, abi.F32)
        out = run.matmul(a, b, abi.F32)
        assert out.shape == exp.shape
        err = np.abs(out - exp).max()
        assert err <= 1e-2 and err <= 1e-5 * max(1.0, np.abs(exp).max()) * k, (scale, err)
    # exact cases: small integers are exact in fp16 and their sums in fp32, whatever the summation order
    ai = rng.integers(-8, 8, (nb, m, k)).astype(np.float16)
    bi = rng.integers(-8, 8, (nb, k, n)).astype(np.float16)
    np.testing.assert_array_equal(run.matmul(ai, bi, abi.F32), np.einsum("bmk,bkn->bmn", ai.astype(np.float32), bi.astype(np.float32)))


@pytest.mark.parametrize("case", HMM_CASES, ids=[c[0] for c in HMM_CASES])
def test_matmul_bias_cast_equals_the_three_operators(run, oracle, case):
    """The fused fp16 projection (MATMUL -> ADD fp32 bias -> CAST fp16) is bit-identical to the three operators run one
    after another on the GPU, and within 1e-2 of the oracle's sequential fp32 accumulation."""
    name, nb, m, k, n = case
    rng = np.random.default_rng(zlib.crc32(name.encode()) + 1)
    a = rng.standard_normal((nb, m, k)).astype(np.float16)
    b = (0.05 * rng.standard_normal((nb, k, n))).astype(np.float16)
    for bias in (rng.standard_normal((1, 1, n)).astype(np.float32), np.array([[[0.25]]], np.float32), None):
        acc = run.matmul(a, b, abi.F32)
        unfused = run.cast(run.binary("ADD", acc, bias, acc.shape, abi.F32) if bias is not None else acc, abi.F16)
        fused = run.matmul_bias_cast(a, b, bias)
        np.testing.assert_array_equal(fused, unfused)
        exp = oracle.matmul(a, b, abi.F32) + (bias if bias is not None else 0)
        assert np.abs(fused.astype(np.float32) - exp).max() <= 1e-2
        # ... followed by the ADD of a residual connection (an fp16 tensor of the output's shape) in the same launch
        res = rng.standard_normal((nb, m, n)).astype(np.float16)
        res[0, 0, :2] = [np.float16(-0.0), np.float16(6e-8)]
        with_res = run.matmul_bias_cast_add(a, b, bias, res)
        np.testing.assert_array_equal(with_res.view(np.uint16), run.binary("ADD", unfused, res, res.shape, abi.F16).view(np.uint16))


@pytest.mark.parametrize("shape", [(1, 200, 96, 64), (2, 130, 264, 136), (1, 33, 40, 8), (1, 64, 36, 64)], ids=str)
def test_matmul_bias_cast_group_equals_the_products_one_by_one(run, shape):
    """Two and three products of one A in one launch (the query, key and value projections) are the products computed
    one after another, bit for bit; K = 36 is no multiple of eight, which the grouped kernel declines (one call each
    inside the entry point)."""
    nb, m, k, n = shape
    rng = np.random.default_rng(m * 7 + n)
    a = rng.standard_normal((nb, m, k)).astype(np.float16)
    bs = [(0.1 * rng.standard_normal((nb, k, n))).astype(np.float16) for _ in range(3)]
    biases = [rng.standard_normal((1, 1, n)).astype(np.float32) for _ in range(3)]
    for count in (2, 3):
        got = run.matmul_bias_cast_group(a, bs[:count], biases[:count])
        for i in range(count):
            np.testing.assert_array_equal(got[i].view(np.uint16), run.matmul_bias_cast(a, bs[i], biases[i]).view(np.uint16))
    got = run.matmul_bias_cast_group(a, bs[:2], [None, None])
    for i in range(2):
        np.testing.assert_array_equal(got[i].view(np.uint16), run.matmul_bias_cast(a, bs[i], None).view(np.uint16))


def test_matmul_bias_cast_chain_equals_product_then_chain(run):
    """The activation of a feed-forward layer inside the product's call: the tanh form of GELU (applied by the matrix
    kernel to the tile on its way out) and a chain the kernel does not know (product into a temporary, then the chain)
    both equal the product followed by mlel_hip_elementwise_chain, bit for bit."""
    rng = np.random.default_rng(23)
    B, M, U = 0, 1, 2
    ADD = abi.BIN["ADD"]
    f16 = abi.F16

    def scalar(v):
        return np.array(v, np.float16).reshape(1, 1, 1)

    gelu_inputs = [scalar(0.5), scalar(0.044715), scalar(np.sqrt(2 / np.pi)), scalar(1.0)]
    gelu = [(M, 0, 0, 1, f16), (M, 0, 0, 0, f16), (M, 0, 6, 0, f16), (M, 0, 7, 2, f16), (B, ADD, 0, 8, f16),
            (M, 0, 9, 3, f16), (U, abi.UN["TANH"], 10, 0, f16), (B, ADD, 11, 4, f16), (M, 0, 5, 12, f16)]
    other_inputs = [scalar(0.25)]
    other = [(M, 0, 0, 1, f16), (U, abi.UN["EXP"], 2, 0, f16)]
    for nb, m, k, n in ((1, 200, 96, 256), (2, 70, 40, 72), (1, 64, 36, 64)):
        a = rng.standard_normal((nb, m, k)).astype(np.float16)
        b = (0.3 * rng.standard_normal((nb, k, n))).astype(np.float16)
        bias = rng.standard_normal((1, 1, n)).astype(np.float32)
        product = run.matmul_bias_cast(a, b, bias)
        for inputs, steps in ((gelu_inputs, gelu), (other_inputs, other)):
            want = run.chain([product] + inputs, steps, product.shape, f16)
            got = run.matmul_bias_cast_chain(a, b, bias, inputs, steps)
            np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16), err_msg=f"{(nb, m, k, n)} {len(steps)}")


BROWS_SHAPES = [(1, 256, 768, 768), (2, 130, 96, 136), (1, 33, 32, 8), (1, 512, 3072, 768), (1, 300, 64, 392), (3, 64, 160, 128),
                (1, 1024, 768, 1024), (1, 200, 2080, 136), (1, 4096, 256, 3072)]  # the last one: 192 tiles of 256 x 256


@pytest.mark.parametrize("shape", BROWS_SHAPES, ids=str)
def test_fp16_products_with_row_wise_b_equal_the_k_major_form(run, shape):
    """B handed over as a [K][N] view of a matrix stored row-wise ([N][K], what a graph does once with a constant
    weight matrix) takes the direct-to-LDS loop; the result is the K-major kernel's bit for bit (same matrix
    instruction, same order of K), for the plain fused form, with a residual, with the GELU chain, for grouped products
    and through a head-splitting view; rows beyond M and N are padding."""
    nb, m, k, n = shape
    rng = np.random.default_rng(m * 13 + n)
    a = rng.standard_normal((nb, m, k)).astype(np.float16)
    bs = [(0.1 * rng.standard_normal((nb, k, n))).astype(np.float16) for _ in range(3)]
    biases = [rng.standard_normal((1, 1, n)).astype(np.float32) for _ in range(3)]
    b, bias = bs[0], biases[0]
    want = run.matmul_bias_cast(a, b, bias)
    assert len(np.unique(want)) > 100
    np.testing.assert_array_equal(run.matmul_bias_cast(a, b, bias, b_rows=True).view(np.uint16), want.view(np.uint16))
    np.testing.assert_array_equal(run.matmul_bias_cast(a, b, None, b_rows=True).view(np.uint16),
                                  run.matmul_bias_cast(a, b, None).view(np.uint16))
    res = rng.standard_normal((nb, m, n)).astype(np.float16)
    np.testing.assert_array_equal(run.matmul_bias_cast_add(a, b, bias, res, b_rows=True).view(np.uint16),
                                  run.matmul_bias_cast_add(a, b, bias, res).view(np.uint16))
    got = run.matmul_bias_cast_group(a, bs, biases, b_rows=True)
    for i in range(3):
        np.testing.assert_array_equal(got[i].view(np.uint16), run.matmul_bias_cast(a, bs[i], biases[i]).view(np.uint16))

    def scalar(v):
        return np.array(v, np.float16).reshape(1, 1, 1)

    B, M, U, ADD, f16 = 0, 1, 2, abi.BIN["ADD"], abi.F16
    gelu_inputs = [scalar(0.5), scalar(0.044715), scalar(np.sqrt(2 / np.pi)), scalar(1.0)]
    gelu = [(M, 0, 0, 1, f16), (M, 0, 0, 0, f16), (M, 0, 6, 0, f16), (M, 0, 7, 2, f16), (B, ADD, 0, 8, f16),
            (M, 0, 9, 3, f16), (U, abi.UN["TANH"], 10, 0, f16), (B, ADD, 11, 4, f16), (M, 0, 5, 12, f16)]
    np.testing.assert_array_equal(run.matmul_bias_cast_chain(a, b, bias, gelu_inputs, gelu, b_rows=True).view(np.uint16),
                                  run.matmul_bias_cast_chain(a, b, bias, gelu_inputs, gelu).view(np.uint16))


def test_matmul_bias_cast_through_a_view(run):
    """A six-dimensional output view = the RESHAPE -> TRANSPOSE that splits or merges attention heads behind the
    product: same bytes as the product followed by numpy's reshape and transpose.  The last case has an inner extent
    that is no multiple of eight, which the fused kernel declines (dense temporary + strided copy inside the call)."""
    rng = np.random.default_rng(11)
    cases = [  # (NB, M, K, N), split [NB1, NB2, M1, M2, N1, N2], perms
        ((1, 6 * 40, 64, 3 * 16), (1, 1, 6, 40, 3, 16), (0, 1, 2, 4, 3, 5)),   # [B, S, H, d] -> [B, H, S, d]
        ((2 * 3, 72, 48, 32), (2, 3, 72, 1, 1, 32), (0, 2, 3, 1, 4, 5)),       # [B, H, S, d] -> [B, S, H, d]
        ((1, 300, 128, 256), (1, 1, 300, 1, 2, 128), (0, 1, 4, 2, 3, 5)),      # columns split, rows not
        ((1, 6 * 40, 64, 3 * 16), (1, 1, 6, 40, 3, 16), (0, 1, 2, 4, 5, 3)),   # [B, S, H, d] -> [B, H, d, S]: transposing
        ((1, 2 * 136, 72, 5 * 24), (1, 1, 2, 136, 5, 24), (0, 1, 2, 4, 5, 3)), # the same over partial tiles
        ((1, 4 * 10, 32, 2 * 12), (1, 1, 4, 10, 2, 12), (0, 1, 2, 4, 3, 5)),   # inner extent 12: declined
    ]
    for (nb, m, k, n), split, perms in cases:
        a = rng.standard_normal((nb, m, k)).astype(np.float16)
        b = (0.1 * rng.standard_normal((nb, k, n))).astype(np.float16)
        bias = rng.standard_normal((1, 1, n)).astype(np.float32)
        want = run.matmul_bias_cast(a, b, bias).reshape(split).transpose(perms)
        got = run.matmul_bias_cast_view(a, b, bias, split, perms)
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16), err_msg=str(split))


ATTENTION_CASES = [  # heads, queries, keys, scaled, head-merge view
    (3, 64, 64, True, False),
    (2, 128, 512, True, False),
    (5, 192, 320, False, False),
    (2 * 3, 64, 128, True, True),
    (4, 64, 256, True, False),   # the keys of exactly one pass through shared memory
    (2 * 3, 128, 448, False, True),  # a full pass and three chunks of a second one
]


@pytest.mark.parametrize("case", ATTENTION_CASES, ids=[f"h{c[0]}_m{c[1]}_s{c[2]}_{'scaled' if c[3] else 'plain'}{'_view' if c[4] else ''}"
                                                       for c in ATTENTION_CASES])
def test_attention_equals_the_three_launches(run, case):
    """mlel_hip_attention_f16 against the launches it replaces: the fp16 product QK^T, the softmax chain over its rows,
    the fp16 product with V (optionally written through a head-merge view) -- the same bits."""
    nb, m, s, scaled, view = case
    rng = np.random.default_rng(zlib.crc32(repr(case).encode()))
    q = rng.standard_normal((nb, m, 64)).astype(np.float16)
    kt = rng.standard_normal((nb, 64, s)).astype(np.float16)
    v = rng.standard_normal((nb, s, 64)).astype(np.float16)
    Bk, Mk, Uk, Rk = 0, 1, 2, 4  # step kinds: binary, mul, unary, reduce
    f16 = abi.F16
    o = 2 if scaled else 0  # with a scale every value index moves up by two
    steps = [(Rk, abi.RED["MAX"], o, 0, f16), (Bk, abi.BIN["SUB"], o, o + 1, f16), (Uk, abi.UN["EXP"], o + 2, 0, f16),
             (Rk, abi.RED["SUM"], o + 3, 0, f16), (Uk, abi.UN["RECIPROCAL"], o + 4, 0, f16), (Mk, 0, o + 3, o + 5, f16)]
    extra = []
    if scaled:
        steps = [(Mk, 0, 0, 1, f16)] + steps
        extra = [np.array(0.125, np.float16).reshape(1, 1, 1)]
    scores = run.matmul_bias_cast(q, kt, None)
    prob = run.chain([scores] + extra, steps, scores.shape, f16)
    assert np.isfinite(prob.astype(np.float32)).all() and len(np.unique(prob)) > 100
    want = run.matmul_bias_cast(prob, v, None)
    if view:
        split, perms = (2, 3, m, 1, 1, 64), (0, 2, 3, 1, 4, 5)  # [B, H, S, d] -> [B, S, H, d]
        want = want.reshape(split).transpose(perms)
        got = run.attention(q, kt, v, extra, steps, split, perms)
    else:
        got = run.attention(q, kt, v, extra, steps)
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))


def test_attention_with_special_values_equals_the_three_launches(run):
    """Rows whose scores overflow to +-infinity or hold a NaN: a row with a NaN or +infinity comes out all NaN from both
    paths, a row with -infinity scores (a masked key) stays finite and keeps the launches' bits; 320 keys, so the rows
    cross the boundary between two passes through shared memory."""
    nb, m, s = 2, 64, 320
    rng = np.random.default_rng(77)
    q = rng.standard_normal((nb, m, 64)).astype(np.float16)
    kt = rng.standard_normal((nb, 64, s)).astype(np.float16)
    v = rng.standard_normal((nb, s, 64)).astype(np.float16)
    q[0, 3, :] = 200.0
    q[0, 5, :] = -200.0
    kt[0, :, 300] = 200.0       # row 3: +inf at key 300, row 5: -inf there
    q[1, 7, 10] = np.nan        # row 7 of the second head: NaN scores everywhere
    kt[1, :, 17] = -65504.0     # a key that is very negative for positive queries
    Bk, Mk, Uk, Rk = 0, 1, 2, 4
    f16 = abi.F16
    steps = [(Rk, abi.RED["MAX"], 0, 0, f16), (Bk, abi.BIN["SUB"], 0, 1, f16), (Uk, abi.UN["EXP"], 2, 0, f16),
             (Rk, abi.RED["SUM"], 3, 0, f16), (Uk, abi.UN["RECIPROCAL"], 4, 0, f16), (Mk, 0, 3, 5, f16)]
    scores = run.matmul_bias_cast(q, kt, None)
    assert np.isposinf(scores[0, 3, 300]) and np.isneginf(scores[0, 5, 300]) and np.isnan(scores[1, 7]).all()
    prob = run.chain([scores], steps, scores.shape, f16)
    want = run.matmul_bias_cast(prob, v, None)
    got = run.attention(q, kt, v, [], steps)
    assert np.isnan(want[0, 3]).all() and np.isnan(want[1, 7]).all() and np.isfinite(want[0, 5].astype(np.float32)).all()
    _same_bits_or_both_nan(got, want)


def test_random_sweep_of_attention_and_row_wise_products(run):
    """Random extents: the attention kernel against the three launches it replaces (1 - 4 heads, 64 - 256 queries, 64 -
    512 keys, with and without the scale, queries of different spread), and fp16 products with a row-wise B against the
    K-major form (M 1 - 599, K 32 - 1248, N 8 - 472, with and without bias): the same bits."""
    rng0 = np.random.default_rng(4242)
    Bk, Mk, Uk, Rk = 0, 1, 2, 4
    f16 = abi.F16
    for i in range(60):
        nb, m, s = int(rng0.integers(1, 5)), 64 * int(rng0.integers(1, 5)), 64 * int(rng0.integers(1, 9))
        scaled, spread = bool(rng0.integers(0, 2)), float(rng0.uniform(0.3, 3))
        rng = np.random.default_rng(i)
        q = (rng.standard_normal((nb, m, 64)) * spread).astype(np.float16)
        kt = rng.standard_normal((nb, 64, s)).astype(np.float16)
        v = rng.standard_normal((nb, s, 64)).astype(np.float16)
        o = 2 if scaled else 0
        steps = [(Rk, abi.RED["MAX"], o, 0, f16), (Bk, abi.BIN["SUB"], o, o + 1, f16), (Uk, abi.UN["EXP"], o + 2, 0, f16),
                 (Rk, abi.RED["SUM"], o + 3, 0, f16), (Uk, abi.UN["RECIPROCAL"], o + 4, 0, f16), (Mk, 0, o + 3, o + 5, f16)]
        extra = []
        if scaled:
            steps = [(Mk, 0, 0, 1, f16)] + steps
            extra = [np.array(0.125, np.float16).reshape(1, 1, 1)]
        scores = run.matmul_bias_cast(q, kt, None)
        prob = run.chain([scores] + extra, steps, scores.shape, f16)
        want = run.matmul_bias_cast(prob, v, None)
        got = run.attention(q, kt, v, extra, steps)
        _same_bits_or_both_nan(got, want)
    for i in range(60):
        rng = np.random.default_rng(1000 + i)
        nb, m = int(rng.integers(1, 3)), int(rng.integers(1, 600))
        k, n = 32 * int(rng.integers(1, 40)), 8 * int(rng.integers(1, 60))
        a = rng.standard_normal((nb, m, k)).astype(np.float16)
        b = (0.1 * rng.standard_normal((nb, k, n))).astype(np.float16)
        bias = rng.standard_normal((1, 1, n)).astype(np.float32) if i % 2 else None
        want = run.matmul_bias_cast(a, b, bias)
        got = run.matmul_bias_cast(a, b, bias, b_rows=True)
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16), err_msg=str((nb, m, k, n)))


def test_attention_declines_what_the_kernel_was_not_written_for(run):
    """Other head sizes, row counts or chains are MLEL_ERR_UNSUPPORTED: nothing is allocated, nothing falls back."""
    rng = np.random.default_rng(5)
    f16 = abi.F16
    steps = [(4, abi.RED["MAX"], 0, 0, f16), (0, abi.BIN["SUB"], 0, 1, f16), (2, abi.UN["EXP"], 2, 0, f16),
             (4, abi.RED["SUM"], 3, 0, f16), (2, abi.UN["RECIPROCAL"], 4, 0, f16), (1, 0, 3, 5, f16)]
    mk = lambda *shape: rng.standard_normal(shape).astype(np.float16)
    for q, kt, v, st in ((mk(1, 64, 32), mk(1, 32, 64), mk(1, 64, 32), steps),      # heads of 32
                         (mk(1, 40, 64), mk(1, 64, 64), mk(1, 64, 64), steps),      # 40 query rows
                         (mk(1, 64, 64), mk(1, 64, 576), mk(1, 576, 64), steps),    # 576 keys
                         (mk(1, 64, 64), mk(1, 64, 64), mk(1, 64, 64), steps[:5] + [(1, 0, 3, 3, f16)])):  # another chain
        with pytest.raises(hb.MlelError) as err:
            run.attention(q, kt, v, [], st)
        assert err.value.code == abi.ERR_UNSUPPORTED


def test_elementwise_chain_equals_the_operators_one_by_one(run):
    """mlel_hip_elementwise_chain against the same operators launched one after another (bit for bit): a GELU-shaped
    chain over fp16 with scalar constants, a chain with row- and column-broadcast inputs and a cast, short rows, and a
    chain the one-pass kernel declines (unaligned rows), which takes the operator-by-operator path inside the call."""
    rng = np.random.default_rng(77)
    B, U, M, C_ = 0, 2, 1, 3  # step kinds: binary, unary, mul, cast
    ADD, SUB = abi.BIN["ADD"], abi.BIN["SUB"]
    f16, f32 = abi.F16, abi.F32

    def scalar(v):
        return np.array(v, np.float16).reshape(1, 1, 1)

    h = rng.standard_normal((1, 96, 256)).astype(np.float16)
    consts = [scalar(0.044715), scalar(np.sqrt(2 / np.pi)), scalar(0.5), scalar(1.0)]
    # values: 0 h, 1..4 constants, then steps
    steps = [(M, 0, 0, 0, f16), (M, 0, 5, 0, f16), (M, 0, 6, 1, f16), (B, ADD, 0, 7, f16), (M, 0, 8, 2, f16),
             (U, abi.UN["TANH"], 9, 0, f16), (B, ADD, 10, 4, f16), (M, 0, 0, 3, f16), (M, 0, 12, 11, f16)]
    got = run.chain([h] + consts, steps, h.shape, f16)
    t = run.mul(run.mul(run.mul(h, h, h.shape, f16), h, h.shape, f16), consts[0], h.shape, f16)
    inner = run.mul(run.binary("ADD", h, t, h.shape, f16), consts[1], h.shape, f16)
    exp = run.mul(run.mul(h, consts[2], h.shape, f16),
                  run.binary("ADD", run.unary("TANH", inner), consts[3], h.shape, f16), h.shape, f16)
    np.testing.assert_array_equal(got, exp)

    # the same expression in the order the graph's region builder emits it, which has a kernel compiled ahead of time
    # (values 0 h, 1 half, 2 cubic coefficient, 3 sqrt(2 / pi), 4 one)
    g_consts = [consts[2], consts[0], consts[1], consts[3]]
    g_steps = [(M, 0, 0, 1, f16), (M, 0, 0, 0, f16), (M, 0, 6, 0, f16), (M, 0, 7, 2, f16), (B, ADD, 0, 8, f16),
               (M, 0, 9, 3, f16), (U, abi.UN["TANH"], 10, 0, f16), (B, ADD, 11, 4, f16), (M, 0, 5, 12, f16)]
    for hh in (h, (8 * rng.standard_normal((3, 5, 24))).astype(np.float16)):
        np.testing.assert_array_equal(run.chain([hh] + g_consts, g_steps, hh.shape, f16).view(np.uint16),
                                      run.chain([hh] + consts, steps, hh.shape, f16).view(np.uint16))

    x32 = rng.standard_normal((4, 24, 64)).astype(np.float32)
    col = rng.standard_normal((4, 24, 1)).astype(np.float16)
    row = rng.standard_normal((1, 1, 64)).astype(np.float16)
    steps = [(C_, 0, 0, 0, f16), (B, SUB, 3, 1, f16), (U, abi.UN["EXP"], 4, 0, f16), (M, 0, 5, 2, f16),
             (C_, 0, 6, 0, f32)]
    got = run.chain([x32, col, row], steps, x32.shape, f32)
    x16 = run.cast(x32, f16)
    e = run.unary("EXP", run.binary("SUB", x16, col, x32.shape, f16))
    np.testing.assert_array_equal(got, run.cast(run.mul(e, row, x32.shape, f16), f32))

    v = np.abs(rng.standard_normal((8, 64, 1))).astype(np.float16)
    steps = [(M, 0, 0, 1, f16), (B, ADD, 3, 2, f16), (U, abi.UN["RSQRT"], 4, 0, f16)]
    got = run.chain([v, scalar(1 / 64), scalar(1e-3)], steps, v.shape, f16)
    exp = run.unary("RSQRT", run.binary("ADD", run.mul(v, scalar(1 / 64), v.shape, f16), scalar(1e-3), v.shape, f16))
    np.testing.assert_array_equal(got, exp)

    odd = rng.standard_normal((3, 5, 12)).astype(np.float16)  # rows of 12: neither a vector multiple nor flat-able
    steps = [(M, 0, 0, 0, f16), (B, ADD, 2, 1, f16)]
    rowb = rng.standard_normal((1, 1, 12)).astype(np.float16)
    got = run.chain([odd, rowb], steps, odd.shape, f16)
    np.testing.assert_array_equal(got, run.binary("ADD", run.mul(odd, odd, odd.shape, f16), rowb, odd.shape, f16))


def _same_bits_or_both_nan(got, want):
    nan = np.isnan(want)
    np.testing.assert_array_equal(np.isnan(got), nan)
    np.testing.assert_array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])


@pytest.mark.parametrize("shape", [(2, 48, 768), (5, 1, 64), (300, 8), (3, 2048), (1, 1, 4096), (16384, 768), (777, 1016),
                                   (8192, 768), (2100, 1000)], ids=str)
def test_chain_with_reductions_layernorm(run, shape):
    """LayerNorm as the operators a TOSA graph spells it with (REDUCE_SUM, MUL 1/N, SUB, MUL, REDUCE_SUM, MUL 1/N,
    ADD eps, RSQRT, MUL, MUL gamma, ADD beta), in one mlel_hip_elementwise_chain call against the eleven stand-alone
    kernels: the same bits wherever the result is a number (sequential fp16 sums, a rounding after every step)."""
    rng = np.random.default_rng(shape[-1] + len(shape))
    B, M, U, R = 0, 1, 2, 4
    ADD, SUB = abi.BIN["ADD"], abi.BIN["SUB"]
    f16 = abi.F16
    n = shape[-1]
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float16)
    if x.reshape(-1, n).shape[0] > 2:
        x.reshape(-1, n)[1, 3] = np.nan
        x.reshape(-1, n)[2, :] = 1.25
    one = (1,) * len(shape)
    inv_n, eps = np.full(one, 1.0 / n, np.float16), np.full(one, 1e-3, np.float16)
    gamma = rng.standard_normal(one[:-1] + (n,)).astype(np.float16)
    beta = rng.standard_normal(one[:-1] + (n,)).astype(np.float16)
    # values: 0 x, 1 1/N, 2 eps, 3 gamma, 4 beta; steps start at 5
    steps = [(R, abi.RED["SUM"], 0, 0, f16), (M, 0, 5, 1, f16), (B, SUB, 0, 6, f16), (M, 0, 7, 7, f16),
             (R, abi.RED["SUM"], 8, 0, f16), (M, 0, 9, 1, f16), (B, ADD, 10, 2, f16), (U, abi.UN["RSQRT"], 11, 0, f16),
             (M, 0, 7, 12, f16), (M, 0, 13, 3, f16), (B, ADD, 14, 4, f16)]
    got = run.chain([x, inv_n, eps, gamma, beta], steps, shape, f16)
    last = len(shape) - 1
    rowshape = shape[:-1] + (1,)
    mean = run.mul(run.reduce("SUM", x, last), inv_n, rowshape, f16)
    d = run.binary("SUB", x, mean, shape, f16)
    var = run.mul(run.reduce("SUM", run.mul(d, d, shape, f16), last), inv_n, rowshape, f16)
    rstd = run.unary("RSQRT", run.binary("ADD", var, eps, rowshape, f16))
    want = run.binary("ADD", run.mul(run.mul(d, rstd, shape, f16), gamma, shape, f16), beta, shape, f16)
    _same_bits_or_both_nan(got, want)


def test_chain_with_reductions_other_forms(run):
    """Softmax with its scale in front (seven steps, REDUCE_MAX over rows with infinities and a NaN); a chain that ends
    in a reduction (one value per row); a per-row input; and chains the one-pass kernel declines (fp32 values, rows
    that are no multiple of eight), which take the operator-by-operator path inside the call."""
    rng = np.random.default_rng(4)
    B, M, U, R = 0, 1, 2, 4
    ADD, SUB = abi.BIN["ADD"], abi.BIN["SUB"]
    f16, f32 = abi.F16, abi.F32
    shape = (3, 40, 256)
    x = (rng.standard_normal(shape) * 4).astype(np.float16)
    flat = x.reshape(-1, 256)
    flat[0, 5] = np.inf
    flat[1, 7] = -np.inf
    flat[2, 9] = np.nan
    flat[3, :] = -0.0
    k = np.full((1, 1, 1), 0.125, np.float16)
    steps = [(M, 0, 0, 1, f16), (R, abi.RED["MAX"], 2, 0, f16), (B, SUB, 2, 3, f16), (U, abi.UN["EXP"], 4, 0, f16),
             (R, abi.RED["SUM"], 5, 0, f16), (U, abi.UN["RECIPROCAL"], 6, 0, f16), (M, 0, 5, 7, f16)]
    got = run.chain([x, k], steps, shape, f16)
    s = run.mul(x, k, shape, f16)
    e = run.unary("EXP", run.binary("SUB", s, run.reduce("MAX", s, 2), shape, f16))
    want = run.mul(e, run.unary("RECIPROCAL", run.reduce("SUM", e, 2)), shape, f16)
    _same_bits_or_both_nan(got, want)

    # sum of squares per row, scaled by a per-row input: the result has one value per row
    w = rng.standard_normal((3, 40, 1)).astype(np.float16)
    steps = [(M, 0, 0, 0, f16), (R, abi.RED["SUM"], 2, 0, f16), (M, 0, 3, 1, f16)]
    y = (rng.standard_normal(shape)).astype(np.float16)
    got = run.chain([y, w], steps, (3, 40, 1), f16)
    want = run.mul(run.reduce("SUM", run.mul(y, y, shape, f16), 2), w, (3, 40, 1), f16)
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))

    # declined by the one-pass kernel: fp32 values; rows of 12
    y32 = rng.standard_normal((6, 64)).astype(np.float32)
    steps = [(R, abi.RED["MAX"], 0, 0, f32), (B, SUB, 0, 1, f32)]
    got = run.chain([y32], steps, y32.shape, f32)
    np.testing.assert_array_equal(got, run.binary("SUB", y32, run.reduce("MAX", y32, 1), y32.shape, f32))
    odd = rng.standard_normal((5, 12)).astype(np.float16)
    steps = [(R, abi.RED["SUM"], 0, 0, f16), (B, SUB, 0, 1, f16)]
    got = run.chain([odd], steps, odd.shape, f16)
    np.testing.assert_array_equal(got, run.binary("SUB", odd, run.reduce("SUM", odd, 1), odd.shape, f16))


# ------------------------------------------------------------------------------------------------ DEPTHWISE
DW_CASES = [
    ("c2_like_small", (2, 14, 14, 144), 1, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), -4, 0),
    ("stride2", (1, 16, 16, 96), 1, (3, 3), (0, 1, 0, 1), (2, 2), (1, 1), 6, 0),
    ("c32", (1, 9, 9, 32), 1, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), -128, 0),
    ("mult2_zw", (1, 7, 8, 5), 2, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), 3, -2),
    ("k5_dil", (1, 11, 11, 8), 1, (5, 5), (2, 2, 2, 2), (1, 1), (1, 1), 0, 0),
    ("c960", (1, 7, 7, 960), 1, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), -1, 0),
    ("odd_rows_zw", (2, 9, 10, 12), 1, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), 8, 3),
    ("single_row_out", (1, 3, 13, 8), 1, (3, 3), (0, 0, 1, 1), (1, 1), (1, 1), -9, 0),
    ("stride2_odd", (2, 15, 13, 20), 1, (3, 3), (1, 1, 1, 1), (2, 2), (1, 1), 2, -1),
    ("stride_2x1", (1, 9, 9, 8), 1, (3, 3), (1, 1, 1, 1), (2, 1), (1, 1), 1, 0),
    ("c2052", (1, 4, 5, 2052), 1, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), -3, 0),
    ("one_strip_many_rows", (2, 9, 4, 384), 1, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), 5, 0),
    ("one_quad", (1, 10, 9, 4), 1, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), -6, 2),
    ("many_spatial_blocks", (2, 32, 32, 32), 1, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), 7, 0),
]


@pytest.mark.parametrize("case", DW_CASES, ids=[c[0] for c in DW_CASES])
def test_depthwise_vs_oracle(run, oracle, case):
    name, xs, mch, k, pad, stride, dil, zi, zw = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    c = xs[3]
    x = ri(rng, -128, 127, xs, np.int8)
    w = ri(rng, -128, 127, k + (c, mch), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (c * mch,), np.int32)
    oh, ow = out_hw(xs[1], xs[2], k, pad, stride, dil)
    shape = (xs[0], oh, ow, c * mch)
    attr = abi.conv2d_attr(pad, stride, dil, zi, zw)
    exp = oracle.depthwise_conv2d(x, w, b, shape, abi.I32, attr)
    np.testing.assert_array_equal(run.conv2d(x, w, b, shape, abi.I32, attr, depthwise=True), exp)
    mult, shift = rescale_params(rng, c * mch)
    rattr = abi.rescale_attr(0, -7, True, True, True)
    exp8 = oracle.clamp(oracle.rescale(exp, mult, shift, abi.I8, rattr), -7, 100)
    out8 = run.conv2d(x, w, b, shape, abi.I8, attr, depthwise=True, epilogue=(mult, shift, rattr, (-7, 100)))
    np.testing.assert_array_equal(out8, exp8)


# ------------------------------------------------------------------------------- 1x1 CONV2D + 3x3 DEPTHWISE, one launch
#   name, input [N, H, W, IC], expanded channels, depthwise padding, stride, conv input zp, depthwise input zp
CONV_DW_CASES = [
    ("b14_64_to_64", (2, 14, 14, 64), 64, (1, 1, 1, 1), 1, -3, 5),
    ("b7_160_to_64", (3, 7, 7, 160), 64, (1, 1, 1, 1), 1, 7, -128),
    ("b28_32_to_32", (1, 28, 28, 32), 32, (1, 1, 1, 1), 1, -128, -9),
    ("stride2_even", (2, 16, 16, 32), 96, (0, 1, 0, 1), 2, 4, 2),
    ("stride2_odd", (1, 15, 13, 96), 32, (1, 1, 1, 1), 2, 0, -1),
    ("ragged_9x10", (2, 9, 10, 128), 32, (1, 1, 1, 1), 1, -20, 11),
    ("no_padding", (1, 12, 6, 32), 32, (0, 0, 0, 0), 1, 1, 3),
    ("pad_2_one_side", (1, 5, 7, 64), 32, (2, 0, 0, 2), 1, -1, -4),
    ("one_position", (4, 1, 1, 32), 32, (1, 1, 1, 1), 1, 9, 9),
    ("widest_32x32", (1, 32, 32, 32), 32, (1, 1, 1, 1), 1, 2, -2),
]


@pytest.mark.parametrize("case", CONV_DW_CASES, ids=[c[0] for c in CONV_DW_CASES])
def test_conv2d_dwconv_one_launch_vs_oracle(run, oracle, case):
    name, xs, c, pad, stride, zx, zi = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    n, h, w_, ic = xs
    x = ri(rng, -128, 127, xs, np.int8)
    w1 = ri(rng, -128, 127, (c, 1, 1, ic), np.int8)
    b1 = ri(rng, -2 ** 12, 2 ** 12, (c,), np.int32)
    w2 = ri(rng, -128, 127, (3, 3, c, 1), np.int8)
    b2 = ri(rng, -2 ** 10, 2 ** 10, (c,), np.int32)
    m1, s1 = ri(rng, 2 ** 30, 2 ** 31 - 1, (c,), np.int32), ri(rng, 40, 43, (c,), np.int8)
    m2, s2 = ri(rng, 2 ** 30, 2 ** 31 - 1, (c,), np.int32), ri(rng, 36, 39, (c,), np.int8)
    a1 = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), zx, 0)
    a2 = abi.conv2d_attr(pad, (stride, stride), (1, 1), zi, 0)
    r1 = abi.rescale_attr(0, zi, True, True, True)
    r2 = abi.rescale_attr(0, -11, True, True, True)
    clamp1, clamp2 = (-100, 127), None
    oh, ow = out_hw(h, w_, (3, 3), pad, (stride, stride), (1, 1))
    mid_shape, out_shape = (n, h, w_, c), (n, oh, ow, c)
    mid = oracle.clamp(oracle.rescale(oracle.conv2d(x, w1, b1, mid_shape, abi.I32, a1), m1, s1, abi.I8, r1), *clamp1)
    assert len(np.unique(mid)) > 50, "the intermediate values must not all sit on the clamp"
    exp = oracle.rescale(oracle.depthwise_conv2d(mid, w2, b2, out_shape, abi.I32, a2), m2, s2, abi.I8, r2)
    covered, got = run.conv2d_dwconv(x, w1, b1, a1, (m1, s1, r1, clamp1), w2, b2, a2, (m2, s2, r2, clamp2), out_shape)
    assert covered == 1
    np.testing.assert_array_equal(got, exp)


@pytest.mark.parametrize("seed", range(16))
def test_conv2d_dwconv_one_launch_random_shapes(run, oracle, seed):
    """Extents, strides, paddings and zero points drawn at random inside what the kernel takes (bands, partial
    strips, odd widths, one to five 32-byte pieces per pixel)."""
    rng = np.random.default_rng(9000 + seed)
    stride = int(rng.integers(1, 3))
    h, w_ = int(rng.integers(3, 33)), int(rng.integers(3, 33))
    ic, c = 32 * int(rng.integers(1, 6)), 32 * int(rng.integers(1, 4))
    n = int(rng.integers(1, 4))
    pad = tuple(int(v) for v in rng.integers(0, 3, size=4))
    zx, zi = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    oh, ow = out_hw(h, w_, (3, 3), pad, (stride, stride), (1, 1))
    if oh < 1 or ow < 1:
        pytest.skip("no output position")
    x = ri(rng, -128, 127, (n, h, w_, ic), np.int8)
    w1 = ri(rng, -128, 127, (c, 1, 1, ic), np.int8)
    b1 = ri(rng, -2 ** 12, 2 ** 12, (c,), np.int32)
    w2 = ri(rng, -128, 127, (3, 3, c, 1), np.int8)
    b2 = ri(rng, -2 ** 10, 2 ** 10, (c,), np.int32)
    per_channel = bool(rng.integers(0, 2))
    k = c if per_channel else 1
    m1, s1 = ri(rng, 2 ** 30, 2 ** 31 - 1, (k,), np.int32), ri(rng, 40, 44, (k,), np.int8)
    m2, s2 = ri(rng, 2 ** 30, 2 ** 31 - 1, (k,), np.int32), ri(rng, 36, 39, (k,), np.int8)
    a1 = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), zx, 0)
    a2 = abi.conv2d_attr(pad, (stride, stride), (1, 1), zi, 0)
    double_round = bool(rng.integers(0, 2))
    r1 = abi.rescale_attr(0, zi, True, double_round, per_channel)
    r2 = abi.rescale_attr(0, int(rng.integers(-20, 20)), True, double_round, per_channel)
    clamp1 = (-90, 110) if rng.integers(0, 2) else None
    mid_shape, out_shape = (n, h, w_, c), (n, oh, ow, c)
    mid = oracle.rescale(oracle.conv2d(x, w1, b1, mid_shape, abi.I32, a1), m1, s1, abi.I8, r1)
    if clamp1:
        mid = oracle.clamp(mid, *clamp1)
    exp = oracle.rescale(oracle.depthwise_conv2d(mid, w2, b2, out_shape, abi.I32, a2), m2, s2, abi.I8, r2)
    covered, got = run.conv2d_dwconv(x, w1, b1, a1, (m1, s1, r1, clamp1), w2, b2, a2, (m2, s2, r2, None), out_shape)
    assert covered == 1
    np.testing.assert_array_equal(got, exp)


@pytest.mark.parametrize("seed", range(12))
def test_rgb_stem_random_shapes(run, oracle, seed):
    """The 3x3 convolution over 3-byte pixels on the matrix cores: extents, strides and paddings drawn at random."""
    rng = np.random.default_rng(9100 + seed)
    n, h, w_ = int(rng.integers(1, 4)), int(rng.integers(8, 40)), int(rng.integers(8, 40))
    oc = 16 * int(rng.integers(1, 3))
    stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    pad = tuple(int(v) for v in rng.integers(0, 3, size=4))
    zx = int(rng.integers(-128, 128))
    oh, ow = out_hw(h, w_, (3, 3), pad, stride, (1, 1))
    x = ri(rng, -128, 127, (n, h, w_, 3), np.int8)
    w = ri(rng, -128, 127, (oc, 3, 3, 3), np.int8)
    b = ri(rng, -2 ** 12, 2 ** 12, (oc,), np.int32)
    mult, shift = ri(rng, 2 ** 30, 2 ** 31 - 1, (oc,), np.int32), ri(rng, 38, 42, (oc,), np.int8)
    attr = abi.conv2d_attr(pad, stride, (1, 1), zx, 0)
    rattr = abi.rescale_attr(0, int(rng.integers(-20, 20)), True, bool(rng.integers(0, 2)), True)
    shape = (n, oh, ow, oc)
    exp = oracle.clamp(oracle.rescale(oracle.conv2d(x, w, b, shape, abi.I32, attr), mult, shift, abi.I8, rattr), -100, 120)
    got = run.conv2d(x, w, b, shape, abi.I8, attr, epilogue=(mult, shift, rattr, (-100, 120)))
    np.testing.assert_array_equal(got, exp)
    assert len(np.unique(got)) > 20


def test_conv2d_dwconv_declines_what_the_kernel_was_not_written_for(run):
    rng = np.random.default_rng(5)

    def attempt(xs, c, zw1=0, zw2=0, stride=1, kernel=(3, 3)):
        n, h, w_, ic = xs
        x = ri(rng, -128, 127, xs, np.int8)
        w1 = ri(rng, -128, 127, (c, 1, 1, ic), np.int8)
        w2 = ri(rng, -128, 127, kernel + (c, 1), np.int8)
        b = ri(rng, -100, 100, (c,), np.int32)
        m, s = rescale_params(rng, c)
        a1 = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), 0, zw1)
        pad = (kernel[0] // 2,) * 4
        a2 = abi.conv2d_attr(pad, (stride, stride), (1, 1), 0, zw2)
        r = abi.rescale_attr(0, 0, True, True, True)
        oh, ow = out_hw(h, w_, kernel, pad, (stride, stride), (1, 1))
        return run.conv2d_dwconv(x, w1, b, a1, (m, s, r, None), w2, b, a2, (m, s, r, None), (n, oh, ow, c), expect=-1)

    assert attempt((1, 8, 8, 32), 32) == (1, abi.OK)
    for kwargs in (dict(xs=(1, 8, 8, 48), c=32), dict(xs=(1, 8, 8, 192), c=32), dict(xs=(1, 8, 8, 32), c=48),
                   dict(xs=(1, 40, 8, 32), c=32), dict(xs=(1, 8, 8, 32), c=32, zw1=1),
                   dict(xs=(1, 8, 8, 32), c=32, zw2=-1), dict(xs=(1, 8, 8, 32), c=32, kernel=(5, 5))):
        assert attempt(**kwargs) == (0, abi.ERR_UNSUPPORTED), kwargs


def test_fused_epilogue_with_nonzero_input_zero_point_vs_oracle(run, oracle):
    """TOSA fixes the input zero point of a RESCALE of int32 values at 0 and the fused kernels rely on it; an
    operator that names another must still give the reference's result (it runs as the operator sequence)."""
    rng = np.random.default_rng(77)
    x = ri(rng, -128, 127, (1, 9, 9, 32), np.int8)
    w = ri(rng, -128, 127, (32, 1, 1, 32), np.int8)
    b = ri(rng, -2 ** 10, 2 ** 10, (32,), np.int32)
    mult, shift = ri(rng, 2 ** 30, 2 ** 31 - 1, (32,), np.int32), ri(rng, 38, 41, (32,), np.int8)
    attr = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), 3, 0)
    for zp in (0, 1500, -1500):
        rattr = abi.rescale_attr(zp, -4, True, True, True)
        acc = oracle.conv2d(x, w, b, (1, 9, 9, 32), abi.I32, attr)
        exp = oracle.rescale(acc, mult, shift, abi.I8, rattr)
        got = run.conv2d(x, w, b, (1, 9, 9, 32), abi.I8, attr, epilogue=(mult, shift, rattr, None))
        np.testing.assert_array_equal(got, exp)
        wd = ri(rng, -128, 127, (3, 3, 32, 1), np.int8)
        dattr = abi.conv2d_attr((1, 1, 1, 1), (1, 1), (1, 1), -2, 0)
        dacc = oracle.depthwise_conv2d(x, wd, b, (1, 9, 9, 32), abi.I32, dattr)
        mult2, shift2 = mult, (shift - 3).astype(np.int8)
        dexp = oracle.rescale(dacc, mult2, shift2, abi.I8, rattr)
        dgot = run.conv2d(x, wd, b, (1, 9, 9, 32), abi.I8, dattr, depthwise=True, epilogue=(mult2, shift2, rattr, None))
        np.testing.assert_array_equal(dgot, dexp)
        assert len(np.unique(got)) > 20 and len(np.unique(dgot)) > 20
        a = ri(rng, -128, 127, (2, 40, 64), np.int8)
        bm = ri(rng, -128, 127, (2, 64, 32), np.int8)
        macc = oracle.matmul(a, bm, abi.I32, 1, -1)
        mexp = oracle.rescale(macc, mult, shift, abi.I8, rattr)
        mgot = run.matmul(a, bm, abi.I8, 1, -1, epilogue=(mult, shift, rattr, None))
        np.testing.assert_array_equal(mgot, mexp)


def test_fp16_product_on_the_256_tile_equals_its_halves(run):
    """4096 x 768 x 3072 runs on the 256 x 256 tile of eight wavefronts; each half of its columns alone runs on the
    128 x 128 tile.  The order of the additions along K is the same in both, so the bits are."""
    rng = np.random.default_rng(31)
    a = (rng.standard_normal((1, 4096, 768)) * 0.5).astype(np.float16)
    b = (rng.standard_normal((1, 768, 3072)) * 0.05).astype(np.float16)
    bias = rng.standard_normal((1, 1, 3072)).astype(np.float32)
    whole = run.matmul_bias_cast(a, b, bias)
    left = run.matmul_bias_cast(a, np.ascontiguousarray(b[:, :, :1536]), np.ascontiguousarray(bias[:, :, :1536]))
    right = run.matmul_bias_cast(a, np.ascontiguousarray(b[:, :, 1536:]), np.ascontiguousarray(bias[:, :, 1536:]))
    np.testing.assert_array_equal(whole.view(np.uint16), np.concatenate([left, right], axis=2).view(np.uint16))
    ref = (a[0, :64].astype(np.float64) @ b[0].astype(np.float64) + bias[0, 0]).astype(np.float32)
    assert np.max(np.abs(whole[0, :64].astype(np.float32) - ref)) <= 1e-2


# ------------------------------------------------------------------------------------------------ RESCALE & co
@pytest.mark.parametrize("double_round", [False, True])
@pytest.mark.parametrize("per_channel", [False, True])
def test_rescale_vs_oracle(run, oracle, double_round, per_channel):
    rng = np.random.default_rng(11)
    c = 24
    x = ri(rng, -2 ** 26, 2 ** 26, (3, 7, 5, c), np.int32)
    mult, shift = rescale_params(rng, c, per_channel)
    if per_channel:
        shift[:4] = [2, 31, 32, 62]
    attr = abi.rescale_attr(0, -3, True, double_round, per_channel)
    for odt in (abi.I8, abi.I16, abi.I32):
        np.testing.assert_array_equal(run.rescale(x, mult, shift, odt, attr), oracle.rescale(x, mult, shift, odt, attr))
    x8 = ri(rng, -128, 127, (3, 7, 5, c), np.int8)
    attr8 = abi.rescale_attr(-5, 0, True, double_round, per_channel)
    np.testing.assert_array_equal(run.rescale(x8, mult, shift, abi.I32, attr8),
                                  oracle.rescale(x8, mult, shift, abi.I32, attr8))
    attru = abi.rescale_attr(128, 0, True, double_round, per_channel, input_unsigned=True, output_unsigned=True)
    np.testing.assert_array_equal(run.rescale(x8, mult, shift, abi.I8, attru),
                                  oracle.rescale(x8, mult, shift, abi.I8, attru))
    m16 = ri(rng, 1, 32767, mult.shape, np.int16)
    s16 = ri(rng, 8, 20, shift.shape, np.int8)
    attr16 = abi.rescale_attr(0, 1, False, True, per_channel)
    np.testing.assert_array_equal(run.rescale(x, m16, s16, abi.I16, attr16),
                                  oracle.rescale(x, m16, s16, abi.I16, attr16))


def test_rescale_add_rescale_vs_oracle(run, oracle):
    rng = np.random.default_rng(12)
    c = 24
    a = ri(rng, -128, 127, (2, 9, 9, c), np.int8)
    b = ri(rng, -128, 127, (2, 9, 9, c), np.int8)
    m1, s1 = np.array([1 << 30], np.int32), np.array([11], np.int8)
    m2, s2 = np.array([1431655765], np.int32), np.array([12], np.int8)
    mo, so = np.array([1717986918], np.int32), np.array([50], np.int8)
    a1 = abi.rescale_attr(-3, 0, True, True, False)
    a2 = abi.rescale_attr(5, 0, True, True, False)
    ao = abi.rescale_attr(0, -1, True, True, False)
    ra = oracle.rescale(a, m1, s1, abi.I32, a1)
    rb = oracle.rescale(b, m2, s2, abi.I32, a2)
    exp = oracle.rescale(oracle.elementwise_binary("ADD", ra, rb, ra.shape, abi.I32), mo, so, abi.I8, ao)
    out = run.rescale_add_rescale(a, (m1, s1, a1, None), b, (m2, s2, a2, None), (mo, so, ao, None), abi.I8)
    np.testing.assert_array_equal(out, exp)


def test_clamp_binary_mul_table_vs_oracle(run, oracle):
    rng = np.random.default_rng(13)
    x8 = ri(rng, -128, 127, (4, 33, 7), np.int8)
    np.testing.assert_array_equal(run.clamp(x8, -3, 100), oracle.clamp(x8, -3, 100))
    f = rng.standard_normal((5, 40)).astype(np.float32)
    f[1, 3] = np.nan
    for mode in (abi.NAN_PROPAGATE, abi.NAN_IGNORE):
        np.testing.assert_array_equal(run.clamp(f, -0.5, 0.25, mode), oracle.clamp(f, -0.5, 0.25, mode))
    a = ri(rng, -2 ** 31, 2 ** 31 - 1, (2, 3, 40), np.int32)
    b = ri(rng, -2 ** 31, 2 ** 31 - 1, (2, 1, 40), np.int32)
    for op in ("ADD", "SUB", "MAXIMUM", "MINIMUM", "BITWISE_AND", "BITWISE_OR", "BITWISE_XOR"):
        np.testing.assert_array_equal(run.binary(op, a, b, a.shape, abi.I32),
                                      oracle.elementwise_binary(op, a, b, a.shape, abi.I32), err_msg=op)
    for op in ("EQUAL", "GREATER", "GREATER_EQUAL"):
        np.testing.assert_array_equal(run.binary(op, a, b, a.shape, abi.BOOL),
                                      oracle.elementwise_binary(op, a, b, a.shape, abi.BOOL), err_msg=op)
    sh = ri(rng, 0, 31, (2, 3, 40), np.int32)
    for op in ("LOGICAL_LEFT_SHIFT", "LOGICAL_RIGHT_SHIFT"):
        np.testing.assert_array_equal(run.binary(op, a, sh, a.shape, abi.I32),
                                      oracle.elementwise_binary(op, a, sh, a.shape, abi.I32), err_msg=op)
    for shift in (0, 7, 31):
        np.testing.assert_array_equal(run.mul(a, b, a.shape, abi.I32, shift), oracle.mul(a, b, a.shape, abi.I32, shift))
    tab = ri(rng, -128, 127, (256,), np.int8)
    np.testing.assert_array_equal(run.table(x8, tab, abi.I8), oracle.table(x8, tab, abi.I8))
    x16 = ri(rng, -32768, 32767, (500,), np.int16)
    t16 = ri(rng, -32768, 32767, (513,), np.int16)
    np.testing.assert_array_equal(run.table(x16, t16, abi.I32), oracle.table(x16, t16, abi.I32))


def test_packed_integer_operators_vs_oracle(run, oracle):
    """The 128-bit kernels behind stand-alone RESCALE, CLAMP, TABLE, MAX_POOL2D and same-shape int32 elementwise
    operators: packed tensors large enough for several blocks, element counts with a tail behind the last 16 bytes,
    every input / output width, extreme values, bit for bit against the oracle."""
    rng = np.random.default_rng(1313)
    # RESCALE: int32 accumulators -> int8 / int16 / int32 per channel (24 channels: not a multiple of 16), extremes
    acc = ri(rng, -2 ** 27, 2 ** 27, (2, 29, 31, 24), np.int32)
    acc[0, 0, 0, :6] = [2 ** 31 - 1, -2 ** 31, 0, -1, 1, 2 ** 30]
    mult, shift = rescale_params(rng, 24)
    shift[:5] = [2, 31, 32, 48, 62]
    for dr in (False, True):
        for zi, zo in ((0, 3), (-77, -128)):
            attr = abi.rescale_attr(zi, zo, True, dr, True)
            for odt in (abi.I8, abi.I16, abi.I32):
                np.testing.assert_array_equal(run.rescale(acc, mult, shift, odt, attr),
                                              oracle.rescale(acc, mult, shift, odt, attr), err_msg=f"{dr} {zi} {odt}")
    # int8 / int16 inputs, signed and unsigned, per tensor, into int32 and int8 (the operands of the residual ADD)
    x8 = ri(rng, -128, 127, (3, 17, 13, 20), np.int8)
    x16 = ri(rng, -32768, 32767, (3, 17, 13, 20), np.int16)
    m1, s1 = np.array([1 << 30], np.int32), np.array([11], np.int8)
    for x in (x8, x16):
        for unsigned in (False, True):
            attr = abi.rescale_attr(5, 0, True, True, False, input_unsigned=unsigned)
            np.testing.assert_array_equal(run.rescale(x, m1, s1, abi.I32, attr), oracle.rescale(x, m1, s1, abi.I32, attr))
    attru = abi.rescale_attr(128, 128, True, False, False, input_unsigned=True, output_unsigned=True)
    m2, s2 = np.array([1234567890], np.int32), np.array([30], np.int8)
    np.testing.assert_array_equal(run.rescale(x8, m2, s2, abi.I8, attru), oracle.rescale(x8, m2, s2, abi.I8, attru))
    m16, s16 = ri(rng, 1, 32767, (20,), np.int16), ri(rng, 8, 20, (20,), np.int8)
    attr16 = abi.rescale_attr(0, -1, False, False, True)
    np.testing.assert_array_equal(run.rescale(x16, m16, s16, abi.I8, attr16), oracle.rescale(x16, m16, s16, abi.I8, attr16))
    # CLAMP: every signed width, odd element counts (a tail behind the last 16 bytes)
    for dt, lo, hi in ((np.int8, -128, 127), (np.int16, -32768, 32767), (np.int32, -2 ** 31, 2 ** 31 - 1)):
        x = ri(rng, lo, hi, (7, 1009), dt)
        for mn, mx in ((-3, 100), (lo, hi), (5, 5)):
            np.testing.assert_array_equal(run.clamp(x, mn, mx), oracle.clamp(x, mn, mx), err_msg=f"{dt} {mn} {mx}")
    # int32 elementwise, same shape, with a tail
    a = ri(rng, -2 ** 31, 2 ** 31 - 1, (5, 1001), np.int32)
    b = ri(rng, -2 ** 31, 2 ** 31 - 1, (5, 1001), np.int32)
    for op in ("ADD", "SUB", "MAXIMUM", "MINIMUM", "BITWISE_AND", "BITWISE_OR", "BITWISE_XOR"):
        np.testing.assert_array_equal(run.binary(op, a, b, a.shape, abi.I32),
                                      oracle.elementwise_binary(op, a, b, a.shape, abi.I32), err_msg=op)
    # TABLE
    t8 = ri(rng, -128, 127, (256,), np.int8)
    xt = ri(rng, -128, 127, (3, 4099), np.int8)
    xt[0, :256] = np.arange(-128, 128)
    np.testing.assert_array_equal(run.table(xt, t8, abi.I8), oracle.table(xt, t8, abi.I8))
    t16 = ri(rng, -32768, 32767, (513,), np.int16)
    xt16 = ri(rng, -32768, 32767, (4101,), np.int16)
    xt16[:4] = [-32768, 32767, 0, -1]
    np.testing.assert_array_equal(run.table(xt16, t16, abi.I32), oracle.table(xt16, t16, abi.I32))
    # MAX_POOL2D int8: stride 2 with padding, a window larger than the image, all-lowest input
    xp = ri(rng, -128, 127, (2, 19, 23, 36), np.int8)
    xp[1, :3] = -128
    ap = abi.pool2d_attr((3, 3), (2, 2), (1, 1, 1, 1))
    np.testing.assert_array_equal(run.pool("max_pool2d", xp, (2, 10, 12, 36), ap), oracle.max_pool2d(xp, (2, 10, 12, 36), ap))
    ap2 = abi.pool2d_attr((2, 5), (1, 3), (0, 1, 2, 1))
    np.testing.assert_array_equal(run.pool("max_pool2d", xp, (2, 19, 8, 36), ap2), oracle.max_pool2d(xp, (2, 19, 8, 36), ap2))
    # 16 channels per thread (pixels of whole 16-byte pieces): the same windows, the extreme values in every byte lane
    xw = ri(rng, -128, 127, (3, 19, 23, 48), np.int8)
    xw[0, :2, :, :16] = -128
    xw[1, 5, 7] = np.tile(np.array([127, -128, -1, 0], np.int8), 12)
    np.testing.assert_array_equal(run.pool("max_pool2d", xw, (3, 10, 12, 48), ap), oracle.max_pool2d(xw, (3, 10, 12, 48), ap))
    np.testing.assert_array_equal(run.pool("max_pool2d", xw, (3, 19, 8, 48), ap2), oracle.max_pool2d(xw, (3, 19, 8, 48), ap2))
    ap3 = abi.pool2d_attr((30, 30), (7, 9), (4, 4, 4, 4))  # the window holds the whole image
    np.testing.assert_array_equal(run.pool("max_pool2d", xw, (3, 1, 1, 48), ap3), oracle.max_pool2d(xw, (3, 1, 1, 48), ap3))


def test_pool_reduce_cast_negate_vs_oracle(run, oracle):
    rng = np.random.default_rng(14)
    x = ri(rng, -128, 127, (2, 7, 7, 40), np.int8)
    a = abi.pool2d_attr((7, 7), (1, 1), (0, 0, 0, 0), input_zp=-3, output_zp=2)
    np.testing.assert_array_equal(run.pool("avg_pool2d", x, (2, 1, 1, 40), a), oracle.avg_pool2d(x, (2, 1, 1, 40), a))
    a2 = abi.pool2d_attr((3, 3), (2, 2), (1, 1, 1, 1), input_zp=4, output_zp=-1)
    np.testing.assert_array_equal(run.pool("avg_pool2d", x, (2, 4, 4, 40), a2), oracle.avg_pool2d(x, (2, 4, 4, 40), a2))
    np.testing.assert_array_equal(run.pool("max_pool2d", x, (2, 4, 4, 40), a2), oracle.max_pool2d(x, (2, 4, 4, 40), a2))
    # channel counts off the dword fast path, rectangular windows, extreme values against the zero point
    x5 = ri(rng, -128, 127, (1, 6, 5, 5), np.int8)
    a3 = abi.pool2d_attr((2, 3), (1, 2), (1, 0, 0, 2), input_zp=100, output_zp=-100)
    np.testing.assert_array_equal(run.pool("avg_pool2d", x5, (1, 6, 3, 5), a3), oracle.avg_pool2d(x5, (1, 6, 3, 5), a3))
    lo = np.full((3, 9, 11, 64), -128, np.int8)
    lo[:, ::2] = 127
    a4 = abi.pool2d_attr((3, 2), (2, 1), (1, 0, 1, 0), input_zp=127, output_zp=127)
    np.testing.assert_array_equal(run.pool("avg_pool2d", lo, (3, 4, 11, 64), a4), oracle.avg_pool2d(lo, (3, 4, 11, 64), a4))
    g = ri(rng, -128, 127, (4, 7, 7, 1280), np.int8)
    a5 = abi.pool2d_attr((7, 7), (1, 1), (0, 0, 0, 0), input_zp=-100, output_zp=-100)
    np.testing.assert_array_equal(run.pool("avg_pool2d", g, (4, 1, 1, 1280), a5), oracle.avg_pool2d(g, (4, 1, 1, 1280), a5))
    r = ri(rng, -1000, 1000, (3, 4, 50), np.int32)
    for op in ("SUM", "MAX", "MIN", "PRODUCT"):
        for axis in range(3):
            np.testing.assert_array_equal(run.reduce(op, r, axis), oracle.reduce(op, r, axis), err_msg=f"{op}{axis}")
    big = ri(rng, -2 ** 31, 2 ** 31 - 1, (1000,), np.int32)
    for odt in (abi.I8, abi.I16, abi.BOOL):
        np.testing.assert_array_equal(run.cast(big, odt), oracle.cast(big, odt))
    f = (rng.standard_normal(1000) * 100).astype(np.float32)
    f[:6] = [0.5, 1.5, 2.5, -0.5, 1e9, -1e9]
    np.testing.assert_array_equal(run.cast(f, abi.I8), oracle.cast(f, abi.I8))
    np.testing.assert_array_equal(run.cast(big, abi.F16).view(np.uint16), oracle.cast(big, abi.F16).view(np.uint16))
    x1 = ri(rng, -128, 127, (300,), np.int8)
    np.testing.assert_array_equal(run.negate(x1, 3, -2), oracle.negate(x1, 3, -2))


def test_data_movement_vs_oracle(run, oracle):
    rng = np.random.default_rng(15)
    x = ri(rng, -128, 127, (2, 3, 4, 5), np.int8)
    np.testing.assert_array_equal(run.reshape(x, (6, 20)), x.reshape(6, 20))
    for perms in [(0, 2, 1, 3), (3, 2, 1, 0), (1, 0, 3, 2)]:
        np.testing.assert_array_equal(run.transpose(x, perms), x.transpose(perms))
    np.testing.assert_array_equal(run.slice_(x, (1, 0, 2, 1), (1, 3, 2, 3)), x[1:2, 0:3, 2:4, 1:4])
    pads = [(0, 0), (1, 2), (0, 1), (2, 0)]
    shape = tuple(d + a + b for d, (a, b) in zip(x.shape, pads))
    x32 = x.astype(np.int32)
    np.testing.assert_array_equal(run.pad(x32, np.array(pads).reshape(-1), shape, pad_const_int=-7),
                                  np.pad(x32, pads, constant_values=-7))
    h = rng.standard_normal((8, 16, 4, 6)).astype(np.float16)
    np.testing.assert_array_equal(run.transpose(h, (0, 2, 1, 3)).view(np.uint16),
                                  h.transpose(0, 2, 1, 3).view(np.uint16))


def test_out_of_bounds_reads_are_zero_and_writes_are_dropped(run, oracle):
    """The reference's tensor accessors (tensor/shaders/tensor.glsl:26-86, graph_op/common.comp:64-182): an element read
    outside a tensor's extents is 0, an element written outside is dropped.  Operands whose extents disagree with the
    output reach that rule: an addend shorter than the output along two axes, a MATMUL whose B has fewer K rows than A
    has columns, and a CONCAT part that sticks out of the output."""
    rng = np.random.default_rng(99)
    a = ri(rng, -1000, 1000, (2, 5, 12), np.int32)
    b = ri(rng, -1000, 1000, (2, 3, 7), np.int32)
    exp = a.copy()
    exp[:, :3, :7] += b
    np.testing.assert_array_equal(oracle.elementwise_binary("ADD", a, b, a.shape, abi.I32), exp)
    np.testing.assert_array_equal(run.binary("ADD", a, b, a.shape, abi.I32), exp)
    x = ri(rng, -128, 127, (1, 8, 16), np.int8)
    w = ri(rng, -128, 127, (1, 12, 8), np.int8)   # K rows 12 .. 15 do not exist: they read as 0, not as the zero point
    got = run.matmul(x, w, abi.I32, 3, -2)
    ref = np.einsum("bmk,bkn->bmn", x.astype(np.int64)[:, :, :12] - 3, w.astype(np.int64) + 2) + \
        ((x.astype(np.int64)[:, :, 12:] - 3).sum(axis=2, keepdims=True) * (0 + 2))
    np.testing.assert_array_equal(oracle.matmul(x, w, abi.I32, 3, -2), ref.astype(np.int32))
    np.testing.assert_array_equal(got, ref.astype(np.int32))
    # CONCAT writes its part at an offset along the axis: what lands beyond the output's extent is dropped
    part = ri(rng, -128, 127, (2, 4), np.int8)
    out = run.concat_at(np.zeros((2, 5), np.int8), part, axis=1, offset=3)
    want = np.zeros((2, 5), np.int8)
    want[:, 3:] = part[:, :2]
    np.testing.assert_array_equal(out, want)


def test_external_memory_import_by_file_descriptor(run):
    """mlel_hip_arena_import_fd (what vkBindDataGraphPipelineSessionMemoryARM would call with the fd of an exported
    VkDeviceMemory, graph_layer.cpp:1391-1420): a device allocation exported as a dma-buf fd through HIP stands in for
    the Vulkan export; the imported mapping shows the same bytes, operators run on it, and the import is released."""
    import ctypes as C
    dev = run.dev
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemGetHandleForAddressRange.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_ulonglong]
    n = 1 << 20
    src = dev.alloc(n)
    data = np.random.default_rng(3).integers(-128, 127, n, endpoint=True).astype(np.int8)
    dev._check(dev.lib.mlel_hip_memcpy_h2d(dev.ctx, C.c_void_p(src), data.ctypes.data_as(C.c_void_p), n, None))
    fd = C.c_int(-1)
    if hip.hipMemGetHandleForAddressRange(C.byref(fd), C.c_void_p(src), n, 1, 0) != 0:  # hipMemRangeHandleTypeDmaBufFd
        dev.free(src)
        pytest.skip("this driver does not export device memory as a dma-buf fd")
    mapped, handle = C.c_void_p(), C.c_void_p()
    dev._check(dev.lib.mlel_hip_arena_import_fd(dev.ctx, fd.value, n, C.byref(mapped), C.byref(handle)))
    back = np.zeros(n, np.int8)
    dev._check(dev.lib.mlel_hip_memcpy_d2h(dev.ctx, back.ctypes.data_as(C.c_void_p), mapped, n, None))
    np.testing.assert_array_equal(back, data)
    # an operator reading the imported mapping and writing an ordinary allocation
    tin = abi.make_tensor(mapped.value, abi.I8, (n,), (1,))
    tout = dev.tensor(abi.I8, (n,))
    dev.op("clamp", tout.ref, C.byref(tin), C.byref(abi.ClampAttr(-5.0, 9.0, int(abi.NAN_PROPAGATE))))
    np.testing.assert_array_equal(tout.download(), np.clip(data, -5, 9))
    dev._check(dev.lib.mlel_hip_arena_release_import(dev.ctx, handle))
    os.close(fd.value)
    dev.free(src)
    tout.free()


def test_float_unary_and_reduce_tolerance(run, oracle):
    """fp16/fp32 elementwise: the reference's results depend on its driver's builtins (parity unpinned); the
    bar is max abs error <= 1e-2 against the oracle's fp32 evaluation rounded once to the storage type."""
    rng = np.random.default_rng(16)
    x = rng.standard_normal((4, 300)).astype(np.float16)
    for op in ("EXP", "TANH", "SIGMOID", "ABS", "FLOOR", "CEIL", "ERF", "SIN", "COS"):
        d = np.abs(run.unary(op, x).astype(np.float32) - oracle.elementwise_unary(op, x).astype(np.float32))
        assert np.nanmax(d) <= 1e-2, op
    xp = np.abs(x) + np.float16(0.5)
    for op in ("RECIPROCAL", "RSQRT", "LOG"):
        d = np.abs(run.unary(op, xp).astype(np.float32) - oracle.elementwise_unary(op, xp).astype(np.float32))
        assert np.nanmax(d) <= 1e-2, op
    f = rng.standard_normal((6, 512)).astype(np.float32)
    np.testing.assert_allclose(run.reduce("SUM", f, 1), oracle.reduce("SUM", f, 1), rtol=1e-5, atol=1e-4)
    np.testing.assert_array_equal(run.reduce("MAX", f, 1), oracle.reduce("MAX", f, 1))
    a = rng.standard_normal((4, 1, 64)).astype(np.float16)
    b = rng.standard_normal((4, 8, 64)).astype(np.float16)
    for op in ("ADD", "SUB"):
        np.testing.assert_array_equal(run.binary(op, a, b, b.shape, abi.F16).view(np.uint16),
                                      oracle.elementwise_binary(op, a, b, b.shape, abi.F16).view(np.uint16))
    np.testing.assert_array_equal(run.mul(a, b, b.shape, abi.F16).view(np.uint16),
                                  oracle.mul(a, b, b.shape, abi.F16).view(np.uint16))


def test_float_vectorised_paths_vs_oracle(run, oracle):
    """Dense fp16/fp32 tensors whose last extent is a multiple of 8 take the 128-bit elementwise kernels and the
    row-slab reduction: ADD/SUB/MUL/CAST and the sequential fp16 REDUCE_SUM/REDUCE_MAX are bit-exact against the
    oracle (same fp32-then-round arithmetic, same left-to-right fold); transcendental unaries within 1e-2."""
    rng = np.random.default_rng(18)
    bits = lambda t: t.view(np.uint16) if t.dtype == np.float16 else t.view(np.uint32)
    for dt, odt in ((np.float16, abi.F16), (np.float32, abi.F32)):
        full = rng.standard_normal((3, 50, 200)).astype(dt)
        other = rng.standard_normal((3, 50, 200)).astype(dt)
        per_row = rng.standard_normal((3, 50, 1)).astype(dt)
        per_col = rng.standard_normal((1, 1, 200)).astype(dt)
        scalar = rng.standard_normal((1, 1, 1)).astype(dt)
        for b in (other, per_row, per_col, scalar):
            for op in ("ADD", "SUB"):
                np.testing.assert_array_equal(bits(run.binary(op, full, b, full.shape, odt)),
                                              bits(oracle.elementwise_binary(op, full, b, full.shape, odt)))
                np.testing.assert_array_equal(bits(run.binary(op, b, full, full.shape, odt)),
                                              bits(oracle.elementwise_binary(op, b, full, full.shape, odt)))
            np.testing.assert_array_equal(bits(run.mul(full, b, full.shape, odt)), bits(oracle.mul(full, b, full.shape, odt)))
        for op in ("EXP", "TANH"):
            d = np.abs(run.unary(op, full).astype(np.float32) - oracle.elementwise_unary(op, full).astype(np.float32))
            assert d.max() <= 1e-2, op
        pos = np.abs(full) + dt(0.25)
        for op in ("RECIPROCAL", "RSQRT"):
            d = np.abs(run.unary(op, pos).astype(np.float32) - oracle.elementwise_unary(op, pos).astype(np.float32))
            assert d.max() <= 1e-2, op
    f32 = (rng.standard_normal((7, 33, 72)) * 300).astype(np.float32)
    f32[0, 0, :4] = [1e6, -1e6, 65519.9, 6e-8]
    np.testing.assert_array_equal(run.cast(f32, abi.F16).view(np.uint16), oracle.cast(f32, abi.F16).view(np.uint16))
    f16 = rng.standard_normal((5, 40, 64)).astype(np.float16)
    np.testing.assert_array_equal(run.cast(f16, abi.F32), oracle.cast(f16, abi.F32))
    # sequential fp16 fold: rows that are not a multiple of 64, columns across several 64-column slabs
    for shape in ((3, 50, 200), (2, 130, 768), (1, 64, 8), (4, 7, 512)):
        x = rng.standard_normal(shape).astype(np.float16)
        for op in ("SUM", "MAX"):
            np.testing.assert_array_equal(run.reduce(op, x, 2).view(np.uint16), oracle.reduce(op, x, 2).view(np.uint16),
                                          err_msg=f"{op} {shape}")
    wide = rng.standard_normal((2, 3, 2056)).astype(np.float16)  # more than one 1024-column slab per row
    for op in ("SUM", "MAX"):
        np.testing.assert_array_equal(run.reduce(op, wide, 2).view(np.uint16), oracle.reduce(op, wide, 2).view(np.uint16))
    xn = rng.standard_normal((2, 9, 128)).astype(np.float16)
    xn[0, 3, 77] = np.nan
    xn[1, 0, 0] = np.nan
    for op in ("SUM", "MAX"):
        for mode in (abi.NAN_PROPAGATE, abi.NAN_IGNORE):
            got, exp = run.reduce(op, xn, 2, mode), oracle.reduce(op, xn, 2, mode)
            np.testing.assert_array_equal(np.isnan(got), np.isnan(exp), err_msg=f"{op} {mode}")
            np.testing.assert_array_equal(got[~np.isnan(exp)].view(np.uint16), exp[~np.isnan(exp)].view(np.uint16))


def test_transpose_fast_paths_vs_numpy(run, oracle):
    """Dense transposes: whole-row moves when the last axis stays, 64x64 shared-memory tiles when it moves."""
    rng = np.random.default_rng(19)
    cases = [((2, 5, 12, 64), (0, 2, 1, 3), np.float16), ((2, 7, 3, 40), (0, 2, 3, 1), np.float16),
             ((3, 70, 130), (0, 2, 1), np.int8), ((65, 67), (1, 0), np.int32), ((4, 33, 9), (2, 0, 1), np.float32),
             ((2, 3, 4, 5, 16), (3, 1, 0, 2, 4), np.int16), ((6, 128, 64), (0, 2, 1), np.float16),
             ((2, 16, 4, 8), (0, 2, 1, 3), np.int8), ((1, 1, 200), (2, 1, 0), np.int8),
             # 2-byte elements, both moving extents in multiples of eight: the 16-byte-piece tile kernel, partial tiles
             ((2, 72, 3, 40), (0, 2, 3, 1), np.float16), ((3, 136, 200), (0, 2, 1), np.int16), ((8, 8), (1, 0), np.float16),
             ((2, 512, 12, 64), (0, 2, 3, 1), np.float16)]
    for shape, perms, dt in cases:
        x = (rng.standard_normal(shape) * 50).astype(dt)
        got = run.transpose(x, perms)
        np.testing.assert_array_equal(got, np.transpose(x, perms), err_msg=f"{shape} {perms}")
        np.testing.assert_array_equal(got, oracle.transpose(x, perms))


# ------------------------------------------------------------------------------------------------ split K
SPLIT_CONV_CASES = [
    # name, x shape, OC, kernel, pad, stride, zi, zw: few output tiles and a K of at least 32 steps of 64 bytes, so
    # that K is split over blocks
    ("tap_ic256_3x3", (1, 9, 9, 256), 64, (3, 3), (1, 1, 1, 1), (1, 1), -5, 0),         # one tap per K step
    ("tap_ic320_3x3_s2_zw", (2, 11, 9, 320), 40, (3, 3), (1, 0, 1, 0), (2, 2), 7, -3),
    ("generic_ic232_3x3", (1, 8, 8, 232), 24, (3, 3), (1, 1, 1, 1), (1, 1), 9, 1),       # byte gathers
    ("plain_2560_160", (2, 7, 7, 2560), 160, (1, 1), (0, 0, 0, 0), (1, 1), -1, 0),       # 16-byte rows
    ("plain4_ic2200", (1, 6, 6, 2200), 36, (1, 1), (0, 0, 0, 0), (1, 1), 3, 2),          # dword rows, K tail
    ("plain_k_tail_2096", (1, 5, 5, 2096), 130, (1, 1), (0, 0, 0, 0), (1, 1), 0, 0),     # last split shorter
]


@pytest.mark.parametrize("case", SPLIT_CONV_CASES, ids=[c[0] for c in SPLIT_CONV_CASES])
def test_conv2d_i8_split_k_vs_oracle(run, oracle, case):
    """Contractions with few tiles and a very long K split K over several blocks that exchange int32 partial tiles
    through the context's workspace: int32 result and fused epilogue, bit for bit, and
    again on a second launch (the arrival counters are back at zero)."""
    name, xs, oc, k, pad, stride, zi, zw = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    x = ri(rng, -128, 127, xs, np.int8)
    w = ri(rng, -128, 127, (oc,) + k + (xs[3],), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
    oh, ow = out_hw(xs[1], xs[2], k, pad, stride, (1, 1))
    attr = abi.conv2d_attr(pad, stride, (1, 1), zi, zw)
    shape = (xs[0], oh, ow, oc)
    exp = oracle.conv2d(x, w, b, shape, abi.I32, attr)
    mult, shift = rescale_params(rng, oc)
    rattr = abi.rescale_attr(0, -2, True, True, True)
    exp8 = oracle.clamp(oracle.rescale(exp, mult, shift, abi.I8, rattr), -100, 110)
    for _ in range(2):
        np.testing.assert_array_equal(run.conv2d(x, w, b, shape, abi.I32, attr), exp)
        np.testing.assert_array_equal(run.conv2d(x, w, b, shape, abi.I8, attr, epilogue=(mult, shift, rattr, (-100, 110))),
                                      exp8)


SPLIT_MM_CASES = [
    ("kmajor_zp", 1, 64, 4096, 256, 2, -1),
    ("kmajor4_n100", 2, 40, 2112, 100, -4, 6),
    ("generic_n29_k2100", 1, 37, 2100, 29, 5, -5),
    ("fc_like_long_k", 1, 32, 5120, 1000, 3, 0),
]


@pytest.mark.parametrize("case", SPLIT_MM_CASES, ids=[c[0] for c in SPLIT_MM_CASES])
def test_matmul_i8_split_k_vs_oracle(run, oracle, case):
    name, nb, m, k, n, za, zb = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    a = ri(rng, -128, 127, (nb, m, k), np.int8)
    b = ri(rng, -128, 127, (nb, k, n), np.int8)
    exp = oracle.matmul(a, b, abi.I32, za, zb)
    mult, shift = np.array([1518500250], np.int32), np.array([39], np.int8)
    rattr = abi.rescale_attr(0, 1, True, True, False)
    exp8 = oracle.rescale(exp, mult, shift, abi.I8, rattr)
    for _ in range(2):
        np.testing.assert_array_equal(run.matmul(a, b, abi.I32, za, zb), exp)
        np.testing.assert_array_equal(run.matmul(a, b, abi.I8, za, zb, epilogue=(mult, shift, rattr, None)), exp8)


PAIR_CASES = [
    # name, (N, H, W), IC, OC1, OC2, one pass expected
    ("mnv2_32_16_96", (2, 12, 16), 32, 16, 96, True),
    ("mnv2_96_24_144", (1, 10, 16), 96, 24, 144, True),
    ("wide_32_32_192", (3, 4, 8), 32, 32, 192, True),
    ("wide_96_32_192", (1, 6, 16), 96, 32, 192, True),
    ("ragged_rows_32_16_96", (1, 5, 7), 32, 16, 96, True),       # 35 positions: a partial last group
    ("ragged_rows_96_24_144", (1, 5, 6), 96, 24, 144, True),
    ("odd_extent_96_24_144", (1, 5, 7), 96, 24, 144, True),       # 35 x 24 bytes: not whole 16-byte pieces, two launches
    ("not_instantiated_64_16_96", (1, 4, 8), 64, 16, 96, False),  # runs as the two fused operators
    ("odd_channels_32_12_96", (1, 4, 8), 32, 12, 96, False),
]


@pytest.mark.parametrize("case", PAIR_CASES, ids=[c[0] for c in PAIR_CASES])
def test_conv2d_conv2d_pair_vs_oracle(run, oracle, case):
    """mlel_hip_conv2d_conv2d_rescale_clamp: a 1x1 projection and the 1x1 expansion behind it in one launch, with and
    without the intermediate tensor stored, against the oracle running CONV2D, RESCALE, CLAMP twice; shapes outside
    the one-pass kernel give the same bytes through the two fused operators."""
    name, nhw, ic, oc1, oc2, one_pass = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    n, h, w = nhw
    x = ri(rng, -128, 127, (n, h, w, ic), np.int8)
    w1 = ri(rng, -127, 127, (oc1, 1, 1, ic), np.int8)
    b1 = ri(rng, -2 ** 15, 2 ** 15, (oc1,), np.int32)
    w2 = ri(rng, -127, 127, (oc2, 1, 1, oc1), np.int8)
    b2 = ri(rng, -2 ** 15, 2 ** 15, (oc2,), np.int32)
    m1, s1 = rescale_params(rng, oc1)
    m2, s2 = rescale_params(rng, oc2)
    a1 = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), -5, 0)
    a2 = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), 7, 0)
    r1, r2 = abi.rescale_attr(0, 7, True, True, True), abi.rescale_attr(0, -128, True, True, True)
    mid = oracle.rescale(oracle.conv2d(x, w1, b1, (n, h, w, oc1), abi.I32, a1), m1, s1, abi.I8, r1)
    exp = oracle.clamp(oracle.rescale(oracle.conv2d(mid, w2, b2, (n, h, w, oc2), abi.I32, a2), m2, s2, abi.I8, r2), -128, 60)
    for keep in (False, True):
        covered, got, got_mid = run.conv2d_conv2d(x, w1, b1, a1, (m1, s1, r1, None), w2, b2, a2, (m2, s2, r2, (-128, 60)),
                                                  (n, h, w, oc2), keep_mid=keep)
        ragged = (n * h * w * oc1) % 16 != 0
        assert bool(covered) == (one_pass and not ragged), name
        np.testing.assert_array_equal(got, exp, err_msg=f"{name}, intermediate stored: {keep}")
        if keep:
            np.testing.assert_array_equal(got_mid, mid, err_msg=name)


POOL_CASES = [
    # name, (N, H, W), IC, OC, conv input zp, pool zps (in, out), one launch expected
    ("mnv2_head_320_1280", (3, 7, 7), 320, 1280, -3, (-128, -128), True),
    ("whole_64_positions", (2, 8, 8), 64, 96, 0, (5, -7), True),
    ("one_group_of_channels", (1, 5, 6), 48, 24, 9, (0, 0), True),        # 30 positions, 24 channels: ragged both ways
    ("odd_group_count", (2, 3, 3), 32, 72, -128, (-4, 3), True),          # three groups of 32 channels: an idle wavefront pair
    ("single_position", (4, 1, 1), 16, 40, 1, (2, 2), True),
    ("too_many_positions", (1, 9, 9), 32, 32, 0, (0, 0), False),          # 81 positions: convolution, then pooling
    ("odd_channels_in", (1, 4, 4), 24, 32, 0, (0, 0), False),             # 24 bytes of K: not whole 16-byte pieces
]


@pytest.mark.parametrize("case", POOL_CASES, ids=[c[0] for c in POOL_CASES])
def test_conv2d_avgpool_vs_oracle(run, oracle, case):
    """mlel_hip_conv2d_rescale_clamp_avgpool: a 1x1 CONV2D + RESCALE + CLAMP and the AVG_POOL2D over all positions of an
    image in one launch, against the oracle running the four operators; shapes outside the kernel give the same bytes
    through the fused convolution and the pooling operator."""
    name, nhw, ic, oc, zi, (pzi, pzo), one_launch = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    n, h, w_ = nhw
    x = ri(rng, -128, 127, (n, h, w_, ic), np.int8)
    w = ri(rng, -127, 127, (oc, 1, 1, ic), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
    m, s = rescale_params(rng, oc)
    a = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), zi, 0)
    r = abi.rescale_attr(0, pzi, True, True, True)
    pool = abi.pool2d_attr((h, w_), (1, 1), (0, 0, 0, 0), pzi, pzo)
    mid = oracle.clamp(oracle.rescale(oracle.conv2d(x, w, b, (n, h, w_, oc), abi.I32, a), m, s, abi.I8, r), -100, 127)
    exp = oracle.avg_pool2d(mid, (n, 1, 1, oc), pool)
    covered, got = run.conv2d_avgpool(x, w, b, a, (m, s, r, (-100, 127)), pool)
    assert bool(covered) == one_launch, name
    np.testing.assert_array_equal(got, exp, err_msg=name)


def test_copy_kernels_move_exactly_the_requested_bytes(run):
    """mlel_hip_copy_kernel (ragged length: whole pieces by the one-pass kernel, the tail bytewise) and every mode of
    mlel_hip_copy_kernel_variant leave the destination equal to the source over the requested bytes and untouched
    behind them; the read-only mode writes nothing."""
    import ctypes as C
    dev, lib = run.dev, run.dev.lib
    rng = np.random.default_rng(8)
    n = 3 * 4096 * 16 + 7
    src = ri(rng, 0, 255, (n + 64,), np.uint8)
    ts = run.put(src)
    td = run.put(np.full(n + 64, 0xEE, np.uint8))
    dev._check(lib.mlel_hip_copy_kernel(dev.ctx, dev.stream, C.c_void_p(td.ptr), C.c_void_p(ts.ptr), n))
    got = td.download()
    np.testing.assert_array_equal(got[:n], src[:n])
    assert (got[n:] == 0xEE).all()
    whole = (n // 16) * 16
    for blocks in (0, 7, 64):
        for pieces in (1, 2, 4, 8):
            for nt in (0, 1):
                td.upload(np.full(n + 64, 0xEE, np.uint8))
                dev._check(lib.mlel_hip_copy_kernel_variant(dev.ctx, dev.stream, C.c_void_p(td.ptr), C.c_void_p(ts.ptr),
                                                            whole, blocks, pieces, nt, 0))
                got = td.download()
                np.testing.assert_array_equal(got[:whole], src[:whole], err_msg=str((blocks, pieces, nt)))
                assert (got[whole:] == 0xEE).all()
    td.upload(np.full(n + 64, 0xEE, np.uint8))
    dev._check(lib.mlel_hip_copy_kernel_variant(dev.ctx, dev.stream, C.c_void_p(td.ptr), C.c_void_p(ts.ptr), whole, 0, 4, 1, 1))
    assert (td.download() == 0xEE).all()
    dev._check(lib.mlel_hip_copy_kernel_variant(dev.ctx, dev.stream, C.c_void_p(td.ptr), C.c_void_p(ts.ptr), whole, 0, 4, 0, 2))
    got = td.download()
    assert (got[:whole].view(np.uint32).reshape(-1, 4) == np.array([1, 2, 3, 4], np.uint32)).all() and (got[whole:] == 0xEE).all()
    run.done()
    with pytest.raises(hb.MlelError):
        dev._check(lib.mlel_hip_copy_kernel_variant(dev.ctx, dev.stream, C.c_void_p(ts.ptr), C.c_void_p(ts.ptr), 24, 0, 1, 0, 0))


def test_issue_probe_runs_every_mix_and_rejects_bad_arguments(run):
    """mlel_hip_issue_probe: every instruction mix finishes and reports a clock count that grows with the rounds; the
    matrix instructions alone are never slower than the same four with other instructions behind them; a mode outside
    the list, no rounds and a misaligned operand pointer are refused before any launch."""
    import ctypes as C
    dev, lib = run.dev, run.dev.lib
    ops = run.put(ri(np.random.default_rng(3), 0, 255, (65536,), np.uint8))
    cus = int(dev.info()["compute_units"])
    out = run.put(np.zeros(2 + 256 * cus, np.int32))

    def clocks(mode, iters):
        dev._check(lib.mlel_hip_issue_probe(dev.ctx, dev.stream, C.c_void_p(ops.ptr), C.c_void_p(out.ptr), mode, iters))
        w = out.download().view(np.uint32)
        return int(w[0]) | (int(w[1]) << 32)

    alone = None
    for mode in range(15):
        clocks(mode, 64)
        short, long_ = clocks(mode, 64), clocks(mode, 256)
        assert 0 < short < long_ < 256 * 4000, (mode, short, long_)
        if mode == 0:
            alone = long_
    assert alone * 0.9 <= clocks(2, 256)
    for mode, iters, ptr in ((15, 8, ops.ptr), (-1, 8, ops.ptr), (0, 0, ops.ptr), (0, 8, ops.ptr + 4)):
        with pytest.raises(hb.MlelError):
            dev._check(lib.mlel_hip_issue_probe(dev.ctx, dev.stream, C.c_void_p(ptr), C.c_void_p(out.ptr), mode, iters))
    run.done()


def test_split_k_workspaces_are_released_with_their_streams(run, oracle):
    """More streams than the context has workspace slots, one after the other: each splits K (its workspace appears),
    matches the oracle, and gives the workspace back when it is destroyed -- the twentieth stream still splits."""
    dev, lib = run.dev, run.dev.lib
    name, xs, oc, k, pad, stride, zi, zw = SPLIT_CONV_CASES[3]
    rng = np.random.default_rng(5)
    x = ri(rng, -128, 127, xs, np.int8)
    w = ri(rng, -128, 127, (oc,) + k + (xs[3],), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
    attr = abi.conv2d_attr(pad, stride, (1, 1), zi, zw)
    shape = (xs[0], xs[1], xs[2], oc)
    exp = oracle.conv2d(x, w, b, shape, abi.I32, attr)
    base = lib.mlel_hip_split_workspaces(dev.ctx)
    keep = dev.stream
    try:
        for i in range(20):
            dev.stream = dev.new_stream()
            got = run.conv2d(x, w, b, shape, abi.I32, attr)
            assert lib.mlel_hip_split_workspaces(dev.ctx) == base + 1, i
            stream, dev.stream = dev.stream, keep
            dev.free_stream(stream)
            assert lib.mlel_hip_split_workspaces(dev.ctx) == base, i
            np.testing.assert_array_equal(got, exp, err_msg=f"stream {i}")
    finally:
        dev.stream = keep


# ------------------------------------------------------------------------------------------------ error paths
def test_error_conventions(run):
    x = np.zeros((1, 4, 4, 4), np.int8)
    w = np.zeros((4, 1, 1, 4), np.int8)
    b = np.zeros(4, np.int32)
    with pytest.raises(hb.MlelError) as e:
        run.conv2d(x, w, b, (1, 4, 4, 4), abi.I32, abi.conv2d_attr(acc_type=9))
    run.done()
    assert e.value.code == abi.ERR_INVALID and "Unsupported acc type 9" in str(e.value)
    with pytest.raises(hb.MlelError):
        run.rescale(np.zeros(4, np.int32), np.zeros(1, np.int16), np.zeros(1, np.int8), abi.I8,
                    abi.rescale_attr(scale32=True))
    run.done()


def test_fused_fp16_entry_points_reject_null_data_before_any_launch(run):
    """A tensor with extents but no data pointer is MLEL_ERR_INVALID in the fused fp16 products, as in every other
    entry point: the check runs on the host, nothing is launched."""
    import ctypes as C

    dev = run.dev
    a = run.put(np.zeros((1, 64, 64), np.float16))
    b = run.put(np.zeros((1, 64, 64), np.float16))
    out = run.new(abi.F16, (1, 64, 64))
    res = run.put(np.zeros((1, 64, 64), np.float16))
    null16 = abi.make_tensor(None, abi.F16, (1, 64, 64))
    attr = abi.MatmulAttr(0, 0)
    for args in ((out.ref, C.byref(null16), b.ref, None, C.byref(attr), res.ref),
                 (out.ref, a.ref, C.byref(null16), None, C.byref(attr), res.ref)):
        with pytest.raises(hb.MlelError) as e:
            dev.op("matmul_bias_cast_add", *args)
        assert e.value.code == abi.ERR_INVALID and "null data pointer" in str(e.value)
    prod = (abi.MatmulProduct * 2)()
    for i in range(2):
        prod[i].out, prod[i].b, prod[i].bias = C.pointer(out.view), C.pointer(b.view), None
    prod[1].b = C.pointer(null16)
    with pytest.raises(hb.MlelError) as e:
        dev.op("matmul_bias_cast_group", prod, 2, a.ref, C.byref(attr))
    assert e.value.code == abi.ERR_INVALID and "null data pointer" in str(e.value)
    run.done()


# ------------------------------------------------------------------------------------------------ BASELINE configs
def test_config0_conv_rescale_full_size(run, oracle):
    """BASELINE config 0: CONV2D 1x56x56x64 -> 64, 3x3 s1 p1, zi=-5, then per-channel RESCALE (double round) to
    int8 with output zero point 3; unfused and fused must both equal the oracle."""
    rng = np.random.default_rng(1000)
    x = ri(rng, -128, 127, (1, 56, 56, 64), np.int8)
    w = ri(rng, -127, 127, (64, 3, 3, 64), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (64,), np.int32)
    mult = ri(rng, 2 ** 30, 2 ** 31 - 1, (64,), np.int32)
    shift = ri(rng, 30, 38, (64,), np.int8)
    attr = abi.conv2d_attr((1, 1, 1, 1), (1, 1), (1, 1), -5, 0)
    rattr = abi.rescale_attr(0, 3, True, True, True)
    acc = oracle.conv2d(x, w, b, (1, 56, 56, 64), abi.I32, attr)
    exp = oracle.rescale(acc, mult, shift, abi.I8, rattr)
    np.testing.assert_array_equal(run.conv2d(x, w, b, (1, 56, 56, 64), abi.I32, attr), acc)
    np.testing.assert_array_equal(run.rescale(acc, mult, shift, abi.I8, rattr), exp)
    np.testing.assert_array_equal(run.conv2d(x, w, b, (1, 56, 56, 64), abi.I8, attr,
                                             epilogue=(mult, shift, rattr, None)), exp)


def test_config1_matmul_rescale_full_size(run, oracle):
    """BASELINE config 1: MATMUL 8x512x1024 . 8x1024x1024 int8, a_zp=2, b_zp=-1, then per-tensor RESCALE
    (multiplier 1518500250, shift 39, double round) to int8."""
    rng = np.random.default_rng(1001)
    a = ri(rng, -128, 127, (8, 512, 1024), np.int8)
    b = ri(rng, -128, 127, (8, 1024, 1024), np.int8)
    mult, shift = np.array([1518500250], np.int32), np.array([39], np.int8)
    rattr = abi.rescale_attr(0, 0, True, True, False)
    acc = oracle.matmul(a, b, abi.I32, 2, -1)
    exp = oracle.rescale(acc, mult, shift, abi.I8, rattr)
    np.testing.assert_array_equal(run.matmul(a, b, abi.I32, 2, -1), acc)
    np.testing.assert_array_equal(run.matmul(a, b, abi.I8, 2, -1, epilogue=(mult, shift, rattr, None)), exp)
    # the requantised result uses the whole int8 range (a degenerate all-zero output would prove nothing)
    assert exp.min() < -20 and exp.max() > 20


POINTWISE_CASES = [
    # name, x shape, OC, input zp, per channel: 1x1 convolutions of few 32 x 32 tiles (one tile per wavefront, or
    # four wavefronts per tile when the contraction is long and the tiles are very few)
    ("p_96_24_56x56", (1, 56, 56, 96), 24, -3, True),
    ("p_144_32_28x28", (2, 28, 28, 144), 32, 7, True),
    ("p_192_64_14x14", (3, 14, 14, 192), 64, 0, False),
    ("p_384_96_14x14", (2, 14, 14, 384), 96, -128, True),
    ("p_960_320_7x7", (2, 7, 7, 960), 320, 5, True),
    ("p_320_1280_7x7", (1, 7, 7, 320), 1280, -9, False),
    ("p_208_44_ragged", (1, 5, 13, 208), 44, 11, True),
    ("p_1040_36_one_position", (3, 1, 1, 1040), 36, -1, True),
]


@pytest.mark.parametrize("case", POINTWISE_CASES, ids=[c[0] for c in POINTWISE_CASES])
def test_pointwise_conv_of_few_tiles_vs_oracle(run, oracle, case):
    name, xs, oc, zx, per_channel = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    x = ri(rng, -128, 127, xs, np.int8)
    w = ri(rng, -128, 127, (oc, 1, 1, xs[3]), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
    attr = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), zx, 0)
    shape = xs[:3] + (oc,)
    n = oc if per_channel else 1
    mult, shift = ri(rng, 2 ** 30, 2 ** 31 - 1, (n,), np.int32), ri(rng, 39, 43, (n,), np.int8)
    rattr = abi.rescale_attr(0, -6, True, True, per_channel)
    acc = oracle.conv2d(x, w, b, shape, abi.I32, attr)
    exp = oracle.clamp(oracle.rescale(acc, mult, shift, abi.I8, rattr), -100, 110)
    got = run.conv2d(x, w, b, shape, abi.I8, attr, epilogue=(mult, shift, rattr, (-100, 110)))
    np.testing.assert_array_equal(got, exp)
    assert len(np.unique(exp)) > 50


@pytest.mark.parametrize("seed", range(16))
def test_pointwise_conv_random_shapes_with_and_without_residual(run, oracle, seed):
    """1x1 convolutions whose extents, channel counts (16-byte pieces of K, dwords of output channels), zero points and
    scale forms are drawn at random over the range the one-tile-per-wavefront kernel serves: whole and partial tiles
    in both directions, one or four wavefronts per tile, grids that do not fill their last group of eight blocks;
    with the residual addition behind it on every second draw."""
    rng = np.random.default_rng(9500 + seed)
    n, h, w_ = int(rng.integers(1, 4)), int(rng.integers(1, 30)), int(rng.integers(1, 30))
    ic, oc = 16 * int(rng.integers(1, 61)), 4 * int(rng.integers(1, 81))
    zx = int(rng.integers(-128, 128))
    per_channel = bool(rng.integers(0, 2))
    x = ri(rng, -128, 127, (n, h, w_, ic), np.int8)
    w = ri(rng, -128, 127, (oc, 1, 1, ic), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
    attr = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), zx, 0)
    shape = (n, h, w_, oc)
    k = oc if per_channel else 1
    mult, shift = ri(rng, 2 ** 30, 2 ** 31 - 1, (k,), np.int32), ri(rng, 38, 44, (k,), np.int8)
    rattr = abi.rescale_attr(0, int(rng.integers(-20, 20)), True, bool(rng.integers(0, 2)), per_channel)
    conv8 = oracle.clamp(oracle.rescale(oracle.conv2d(x, w, b, shape, abi.I32, attr), mult, shift, abi.I8, rattr), -100, 110)
    if seed % 2 == 0:
        got = run.conv2d(x, w, b, shape, abi.I8, attr, epilogue=(mult, shift, rattr, (-100, 110)))
        np.testing.assert_array_equal(got, conv8)
        return
    res = ri(rng, -128, 127, shape, np.int8)
    m1, s1 = np.array([int(rng.integers(2 ** 29, 2 ** 31 - 1))], np.int32), np.array([int(rng.integers(8, 14))], np.int8)
    m2, s2 = np.array([int(rng.integers(2 ** 29, 2 ** 31 - 1))], np.int32), np.array([int(rng.integers(8, 14))], np.int8)
    mo, so = np.array([int(rng.integers(2 ** 30, 2 ** 31 - 1))], np.int32), np.array([int(rng.integers(48, 52))], np.int8)
    a_conv = abi.rescale_attr(int(rattr.output_zp), 0, True, True, False)
    a_res = abi.rescale_attr(int(rng.integers(-20, 20)), 0, True, True, False)
    a_out = abi.rescale_attr(0, int(rng.integers(-20, 20)), True, True, False)
    r_conv = oracle.rescale(conv8, m1, s1, abi.I32, a_conv)
    r_res = oracle.rescale(res, m2, s2, abi.I32, a_res)
    exp = oracle.rescale(oracle.elementwise_binary("ADD", r_res, r_conv, shape, abi.I32), mo, so, abi.I8, a_out)
    got = run.conv2d_rescale_add_rescale(x, w, b, attr, (mult, shift, rattr, (-100, 110)), (m1, s1, a_conv, None), res,
                                         (m2, s2, a_res, None), (mo, so, a_out, None), residual_first=bool(rng.integers(0, 2)))
    np.testing.assert_array_equal(got, exp)


def test_random_sweep_of_fused_contractions(run, oracle):
    """A few hundred random draws each of the fused CONV2D (any kernel up to 3x3, stride, padding, dilation, channel
    counts that are and are not multiples of four), DEPTHWISE_CONV2D (kernels up to 5x5, channel multiplier 1 or 2) and
    int8 MATMUL + RESCALE (K-major and row-wise B) against the oracle, bit for bit: whichever kernel the dispatcher
    picks for a draw has to agree."""
    ran = [0, 0, 0]
    for i in range(400):
        rng = np.random.default_rng(20000 + i)
        n, h, w_ = int(rng.integers(1, 4)), int(rng.integers(3, 40)), int(rng.integers(3, 40))
        kh, kw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        sy, sx = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        dy, dx = (int(rng.integers(1, 3)), int(rng.integers(1, 3))) if i % 5 == 0 else (1, 1)
        ic = int(rng.choice([3, 4, 8, 16, 24, 32, 48, 64, 96, 100, 144]))
        oc = int(rng.choice([1, 4, 8, 16, 24, 32, 40, 64, 96, 130]))
        pt, pb, pl, pr = [int(v) for v in rng.integers(0, 2, 4)]
        eh, ew = (kh - 1) * dy + 1, (kw - 1) * dx + 1
        if h + pt + pb < eh or w_ + pl + pr < ew or (h + pt + pb - eh) % sy or (w_ + pl + pr - ew) % sx:
            continue
        shape = (n, (h + pt + pb - eh) // sy + 1, (w_ + pl + pr - ew) // sx + 1, oc)
        x = ri(rng, -128, 127, (n, h, w_, ic), np.int8)
        w = ri(rng, -127, 127, (oc, kh, kw, ic), np.int8)
        b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
        attr = abi.conv2d_attr((pt, pb, pl, pr), (sy, sx), (dy, dx), int(rng.integers(-128, 128)), 0)
        per_channel = bool(rng.integers(0, 2))
        k = oc if per_channel else 1
        mult, shift = ri(rng, 2 ** 30, 2 ** 31 - 1, (k,), np.int32), ri(rng, 36, 46, (k,), np.int8)
        rattr = abi.rescale_attr(0, int(rng.integers(-20, 20)), True, bool(rng.integers(0, 2)), per_channel)
        exp = oracle.clamp(oracle.rescale(oracle.conv2d(x, w, b, shape, abi.I32, attr), mult, shift, abi.I8, rattr), -110, 100)
        got = run.conv2d(x, w, b, shape, abi.I8, attr, epilogue=(mult, shift, rattr, (-110, 100)))
        np.testing.assert_array_equal(got, exp, err_msg=f"conv draw {i}")
        ran[0] += 1
    for i in range(400):
        rng = np.random.default_rng(30000 + i)
        n, h, w_ = int(rng.integers(1, 4)), int(rng.integers(3, 40)), int(rng.integers(3, 40))
        kh, kw = (3, 3) if i % 3 else (int(rng.integers(1, 6)), int(rng.integers(1, 6)))
        st = int(rng.integers(1, 3))
        c, mch = int(rng.choice([4, 8, 16, 32, 48, 96, 144, 20, 36])), 1 if i % 7 else 2
        pt, pb, pl, pr = [int(v) for v in rng.integers(0, 2, 4)]
        if h + pt + pb < kh or w_ + pl + pr < kw or (h + pt + pb - kh) % st or (w_ + pl + pr - kw) % st:
            continue
        oc = c * mch
        shape = (n, (h + pt + pb - kh) // st + 1, (w_ + pl + pr - kw) // st + 1, oc)
        x = ri(rng, -128, 127, (n, h, w_, c), np.int8)
        w = ri(rng, -127, 127, (kh, kw, c, mch), np.int8)
        b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
        attr = abi.conv2d_attr((pt, pb, pl, pr), (st, st), (1, 1), int(rng.integers(-128, 128)), 0)
        mult, shift = ri(rng, 2 ** 30, 2 ** 31 - 1, (oc,), np.int32), ri(rng, 32, 40, (oc,), np.int8)
        rattr = abi.rescale_attr(0, int(rng.integers(-20, 20)), True, True, True)
        exp = oracle.clamp(oracle.rescale(oracle.depthwise_conv2d(x, w, b, shape, abi.I32, attr), mult, shift, abi.I8, rattr), -128, 127)
        got = run.conv2d(x, w, b, shape, abi.I8, attr, depthwise=True, epilogue=(mult, shift, rattr, (-128, 127)))
        np.testing.assert_array_equal(got, exp, err_msg=f"depthwise draw {i}")
        ran[1] += 1
    for i in range(200):
        rng = np.random.default_rng(40000 + i)
        nb, m = int(rng.integers(1, 4)), int(rng.integers(1, 300))
        k, n = int(rng.choice([16, 32, 48, 64, 100, 256, 500, 1024])), int(rng.choice([1, 4, 16, 20, 64, 128, 200, 512]))
        a, b = ri(rng, -128, 127, (nb, m, k), np.int8), ri(rng, -128, 127, (nb, k, n), np.int8)
        za, zb = int(rng.integers(-128, 128)), (int(rng.integers(-128, 128)) if i % 2 else 0)
        mult = np.array([int(rng.integers(2 ** 30, 2 ** 31 - 1))], np.int32)
        shift = np.array([int(rng.integers(36, 46))], np.int8)
        rattr = abi.rescale_attr(0, int(rng.integers(-20, 20)), True, True, False)
        exp = oracle.rescale(oracle.matmul(a, b, abi.I32, za, zb), mult, shift, abi.I8, rattr)
        for rows in (False, True):
            got = run.matmul(a, b, abi.I8, za, zb, epilogue=(mult, shift, rattr, None), b_rows=rows)
            np.testing.assert_array_equal(got, exp, err_msg=f"matmul draw {i} b_rows={rows}")
        ran[2] += 1
    assert ran[0] > 150 and ran[1] > 150 and ran[2] == 200, ran


RESIDUAL_CASES = [
    # name, x shape, OC, kernel, pad: 1x1 projections take the one-pass kernel, the 3x3 case the two-kernel sequence
    ("project_96_24", (2, 14, 14, 96), 24, (1, 1), (0, 0, 0, 0)),
    ("project_192_32_ragged", (3, 7, 9, 192), 32, (1, 1), (0, 0, 0, 0)),
    ("project_960_160", (1, 7, 7, 960), 160, (1, 1), (0, 0, 0, 0)),
    ("project_384_64_b4", (4, 14, 14, 384), 64, (1, 1), (0, 0, 0, 0)),
    ("project_576_96", (2, 14, 14, 576), 96, (1, 1), (0, 0, 0, 0)),
    ("project_144_24_many_tiles", (2, 56, 56, 144), 24, (1, 1), (0, 0, 0, 0)),
    ("project_208_44_ragged", (1, 9, 11, 208), 44, (1, 1), (0, 0, 0, 0)),
    ("k3_32_16", (1, 8, 8, 32), 16, (3, 3), (1, 1, 1, 1)),
]


@pytest.mark.parametrize("case", RESIDUAL_CASES, ids=[c[0] for c in RESIDUAL_CASES])
def test_conv2d_rescale_add_rescale_equals_the_operator_sequence(run, oracle, case):
    name, xs, oc, k, pad = case
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    x = ri(rng, -128, 127, xs, np.int8)
    w = ri(rng, -128, 127, (oc,) + k + (xs[3],), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (oc,), np.int32)
    attr = abi.conv2d_attr(pad, (1, 1), (1, 1), -4, 0)
    shape = (xs[0], xs[1], xs[2], oc)
    res = ri(rng, -128, 127, shape, np.int8)
    mult, shift = rescale_params(rng, oc)
    rattr = abi.rescale_attr(0, 3, True, True, True)
    m1, s1 = np.array([1 << 30], np.int32), np.array([11], np.int8)
    m2, s2 = np.array([1431655765], np.int32), np.array([12], np.int8)
    mo, so = np.array([1717986918], np.int32), np.array([50], np.int8)
    a_conv = abi.rescale_attr(3, 0, True, True, False)
    a_res = abi.rescale_attr(-7, 0, True, True, False)
    a_out = abi.rescale_attr(0, -2, True, True, False)
    conv8 = oracle.clamp(oracle.rescale(oracle.conv2d(x, w, b, shape, abi.I32, attr), mult, shift, abi.I8, rattr), -90, 90)
    r_conv = oracle.rescale(conv8, m1, s1, abi.I32, a_conv)
    r_res = oracle.rescale(res, m2, s2, abi.I32, a_res)
    exp = oracle.rescale(oracle.elementwise_binary("ADD", r_res, r_conv, shape, abi.I32), mo, so, abi.I8, a_out)
    for first in (False, True):
        out = run.conv2d_rescale_add_rescale(x, w, b, attr, (mult, shift, rattr, (-90, 90)), (m1, s1, a_conv, None), res,
                                             (m2, s2, a_res, None), (mo, so, a_out, None), residual_first=first)
        np.testing.assert_array_equal(out, exp)


def test_fp16_products_keep_the_sign_of_zero(run, oracle):
    """(-0) * x is -0, also where the product underflows: a multiplication folded into a fused multiply-add with a +0
    addend would give +0."""
    a = np.array([[-0.0, 1.0, -6e-8, -1.0, 0.0, 3.0]], np.float16)
    b = np.array([[1.0, -0.0, 6e-8, 0.0, -2.0, -0.0]], np.float16)
    got, want = run.mul(a, b, a.shape, abi.F16), oracle.mul(a, b, a.shape, abi.F16)
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    assert np.all(np.signbit(got))
    big_a, big_b = np.tile(a, (64, 16)), np.tile(b, (64, 16))  # the vectorised elementwise kernel
    np.testing.assert_array_equal(run.mul(big_a, big_b, big_a.shape, abi.F16).view(np.uint16),
                                  oracle.mul(big_a, big_b, big_a.shape, abi.F16).view(np.uint16))
    rows = np.array([[-0.0, 1.0, 2.0], [-6e-8, 6e-8, 1.0], [1.0, -1.0, 0.0]], np.float16)
    np.testing.assert_array_equal(run.reduce("PRODUCT", rows, 1).view(np.uint16),
                                  oracle.reduce("PRODUCT", rows, 1).view(np.uint16))


@pytest.mark.parametrize("shape", [(3, 70, 512), (2, 5, 7, 64), (130, 1024), (4, 8), (12000, 512), (9000, 776),
                                   (20000, 768)], ids=str)
def test_softmax_rows_equals_the_six_operators(run, shape):
    """REDUCE_MAX, SUB, EXP, REDUCE_SUM, RECIPROCAL, MUL in one pass == the six stand-alone kernels, bit for bit, on
    ordinary rows and on rows with NaN, infinities, signed zeros and a constant row.  Where the result is NaN only
    NaN-ness is compared: a product of two NaNs takes the sign of whichever operand the compiler put first, and the
    reference's shading language leaves the sign and payload of a NaN unspecified."""
    rng = np.random.default_rng(len(shape) * 1000 + shape[-1])
    x = (rng.standard_normal(shape) * 3).astype(np.float16)
    flat = x.reshape(-1, shape[-1])
    flat[0, 3] = np.nan
    flat[1, 0] = np.inf
    flat[2, 1] = -np.inf
    flat[3, :] = -0.0
    flat[4 % len(flat), :] = 7.5
    flat[5 % len(flat), 2:4] = [np.nan, -np.nan]
    last = len(shape) - 1
    m = run.reduce("MAX", x, last)
    e = run.unary("EXP", run.binary("SUB", x, m, x.shape, abi.F16))
    r = run.unary("RECIPROCAL", run.reduce("SUM", e, last))
    want = run.mul(e, r, x.shape, abi.F16)
    got = run.softmax_rows(x)
    nan = np.isnan(want)
    np.testing.assert_array_equal(np.isnan(got), nan)
    np.testing.assert_array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
    ok = ~nan.any(axis=-1)
    assert np.all(np.abs(got.astype(np.float32)[ok].sum(axis=-1) - 1.0) < 5e-2)  # fp16 sum of up to 1024 rounded terms


def test_softmax_rows_falls_back_for_other_layouts(run):
    """fp32 rows take the operator sequence behind the entry point (no one-pass kernel): same result as the operators"""
    rng = np.random.default_rng(77)
    x = rng.standard_normal((5, 33)).astype(np.float32)
    m = run.reduce("MAX", x, 1)
    e = run.unary("EXP", run.binary("SUB", x, m, x.shape, abi.F32))
    want = run.mul(e, run.unary("RECIPROCAL", run.reduce("SUM", e, 1)), x.shape, abi.F32)
    np.testing.assert_array_equal(run.softmax_rows(x).view(np.uint32), want.view(np.uint32))
