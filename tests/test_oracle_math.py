"""Pins the oracle functions that no reference test covers, against what the mathematics fixes: exact rational
arithmetic, numpy library routines, special cases that reduce to an already pinned operator, brute force."""
from fractions import Fraction

import numpy as np
import pytest

RNG = np.random.default_rng(7)


def ri(lo, hi, shape, dt):
    return RNG.integers(lo, hi, size=shape, endpoint=True).astype(dt)


# ---------------------------------------------------------------- CONV2D with zero points, padding, stride, dilation
def conv_numpy(x, w, b, pad, stride, dil, zi, zw):
    """im2col on an input whose padding holds zi (so padded taps contribute (zi-zi)*.. = 0), int64 einsum."""
    n, h, wd, ic = x.shape
    oc, kh, kw, _ = w.shape
    xp = np.full((n, h + pad[0] + pad[1], wd + pad[2] + pad[3], ic), zi, np.int64)
    xp[:, pad[0]:pad[0] + h, pad[2]:pad[2] + wd] = x
    oh = (h + pad[0] + pad[1] - (kh - 1) * dil[0] - 1) // stride[0] + 1
    ow = (wd + pad[2] + pad[3] - (kw - 1) * dil[1] - 1) // stride[1] + 1
    out = np.zeros((n, oh, ow, oc), np.int64)
    for ky in range(kh):
        for kx in range(kw):
            patch = xp[:, ky * dil[0]: ky * dil[0] + (oh - 1) * stride[0] + 1: stride[0],
                       kx * dil[1]: kx * dil[1] + (ow - 1) * stride[1] + 1: stride[1]]
            out += np.einsum("nhwc,oc->nhwo", patch - zi, w[:, ky, kx].astype(np.int64) - zw)
    return (out + b.astype(np.int64)).astype(np.int32)  # wraps mod 2^32


@pytest.mark.parametrize("cfg", [
    dict(x=(2, 7, 9, 5), oc=6, k=(3, 3), pad=(1, 1, 1, 1), stride=(1, 1), dil=(1, 1), zi=-5, zw=0),
    dict(x=(1, 8, 8, 3), oc=4, k=(3, 3), pad=(0, 1, 0, 1), stride=(2, 2), dil=(1, 1), zi=7, zw=-3),
    dict(x=(1, 9, 6, 4), oc=3, k=(2, 3), pad=(2, 0, 1, 2), stride=(1, 2), dil=(2, 1), zi=-128, zw=127),
    dict(x=(3, 5, 5, 16), oc=8, k=(1, 1), pad=(0, 0, 0, 0), stride=(1, 1), dil=(1, 1), zi=3, zw=0),
])
def test_conv2d_vs_numpy(abi, oracle, cfg):
    x = ri(-128, 127, cfg["x"], np.int8)
    w = ri(-128, 127, (cfg["oc"],) + cfg["k"] + (cfg["x"][3],), np.int8)
    b = ri(-2 ** 31, 2 ** 31 - 1, (cfg["oc"],), np.int32)
    exp = conv_numpy(x, w, b, cfg["pad"], cfg["stride"], cfg["dil"], cfg["zi"], cfg["zw"])
    attr = abi.conv2d_attr(cfg["pad"], cfg["stride"], cfg["dil"], cfg["zi"], cfg["zw"])
    out = oracle.conv2d(x, w, b, exp.shape, abi.I32, attr)
    np.testing.assert_array_equal(out, exp)


def test_conv2d_bias_broadcast_and_padding_contributes_nothing(abi, oracle):
    """A single-element bias is broadcast; a fully padded tap adds nothing even when zi != 0."""
    x = np.full((1, 1, 1, 1), 10, np.int8)
    w = np.ones((2, 3, 3, 1), np.int8)
    out = oracle.conv2d(x, w, np.array([100], np.int32), (1, 1, 1, 2), abi.I32,
                        abi.conv2d_attr((1, 1, 1, 1), input_zp=4))
    assert out.tolist() == [[[[106, 106]]]]


# ---------------------------------------------------------------- DEPTHWISE as a special case of CONV2D
@pytest.mark.parametrize("m", [1, 2])
def test_depthwise_equals_block_diagonal_conv2d(abi, oracle, m):
    c = 5
    x = ri(-128, 127, (2, 6, 7, c), np.int8)
    w = ri(-128, 127, (3, 3, c, m), np.int8)
    b = ri(-1000, 1000, (c * m,), np.int32)
    zi, zw = -9, 4
    attr = abi.conv2d_attr((1, 1, 1, 1), (1, 2), (1, 1), zi, zw)
    out = oracle.depthwise_conv2d(x, w, b, (2, 6, 4, c * m), abi.I32, attr)
    # dense weights [OC,KH,KW,IC]: channel c*m+mm only sees input channel c; other entries hold zw (=> factor 0)
    dense = np.full((c * m, 3, 3, c), zw, np.int8)
    for ch in range(c):
        for mm in range(m):
            dense[ch * m + mm, :, :, ch] = w[:, :, ch, mm]
    exp = oracle.conv2d(x, dense, b, (2, 6, 4, c * m), abi.I32, attr)
    np.testing.assert_array_equal(out, exp)


# ---------------------------------------------------------------- MATMUL
def test_matmul_vs_numpy_einsum(abi, oracle):
    a = ri(-128, 127, (3, 17, 70), np.int8)
    b = ri(-128, 127, (3, 70, 23), np.int8)
    za, zb = 2, -1
    exp = np.einsum("nhc,ncw->nhw", a.astype(np.int64) - za, b.astype(np.int64) - zb).astype(np.int32)
    np.testing.assert_array_equal(oracle.matmul(a, b, abi.I32, za, zb), exp)
    # B is [N,C,W] (not transposed): a transposed operand must fail
    bt = np.ascontiguousarray(b.transpose(0, 2, 1))
    if bt.shape == b.shape:
        assert not np.array_equal(oracle.matmul(a, bt, abi.I32, za, zb), exp)


def test_matmul_generic_path_equals_fast_path(abi, oracle):
    a = ri(-128, 127, (2, 9, 33), np.int8)
    b = ri(-128, 127, (2, 33, 12), np.int8)
    fast = oracle.matmul(a, b, abi.I32, 5, -7)
    a_s = np.zeros((2, 9, 40), np.int8)[..., :33]
    a_s[...] = a
    slow = oracle.matmul(a_s, b, abi.I32, 5, -7)
    np.testing.assert_array_equal(fast, slow)


def test_matmul_f32_vs_numpy(abi, oracle):
    a = RNG.standard_normal((2, 5, 16)).astype(np.float32)
    b = RNG.standard_normal((2, 16, 7)).astype(np.float32)
    np.testing.assert_allclose(oracle.matmul(a, b, abi.F32), np.einsum("nhc,ncw->nhw", a, b), rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- RESCALE against exact rational arithmetic
def rescale_exact(v, zi, mult, shift, double_round, zo, lo, hi):
    """TOSA apply_scale with exact rationals: single rounding = floor(x*m/2^s + 1/2); double rounding first
    nudges the product by +-2^30 when shift > 31."""
    v = int(v) - zi
    prod = v * int(mult)
    if double_round and shift > 31:
        prod += (1 << 30) if v >= 0 else -(1 << 30)
    q = Fraction(prod, 1 << shift) + Fraction(1, 2) if shift > 0 else Fraction(prod)
    r = q.numerator // q.denominator  # floor
    r = (r + (1 << 31)) % (1 << 32) - (1 << 31)  # int32 truncation before the zero point is added
    r = (r + zo + (1 << 31)) % (1 << 32) - (1 << 31)
    return min(max(r, lo), hi)


@pytest.mark.parametrize("double_round", [False, True])
@pytest.mark.parametrize("per_channel", [False, True])
def test_rescale_i32_to_i8_vs_exact(abi, oracle, double_round, per_channel):
    c = 8
    x = ri(-2 ** 24, 2 ** 24, (4, 5, c), np.int32)
    x[0, 0, :4] = [0, -1, 1, -(2 ** 24)]
    nch = c if per_channel else 1
    mult = ri(2 ** 30, 2 ** 31 - 1, (nch,), np.int32)
    shift = ri(30, 38, (nch,), np.int8)
    if per_channel:
        shift[:3] = [31, 32, 62]
    attr = abi.rescale_attr(0, 3, True, double_round, per_channel)
    out = oracle.rescale(x, mult, shift, abi.I8, attr)
    exp = np.zeros_like(out)
    for idx in np.ndindex(x.shape):
        ch = idx[-1] if per_channel else 0
        exp[idx] = rescale_exact(x[idx], 0, mult[ch], int(shift[ch]), double_round, 3, -128, 127)
    np.testing.assert_array_equal(out, exp)


def test_rescale_double_round_only_matters_above_shift_31(abi, oracle):
    x = ri(-2 ** 20, 2 ** 20, (1000,), np.int32)
    mult = np.array([1518500250], np.int32)
    for sh in (1, 16, 31):
        s = np.array([sh], np.int8)
        a = oracle.rescale(x, mult, s, abi.I32, abi.rescale_attr(double_round=True))
        b = oracle.rescale(x, mult, s, abi.I32, abi.rescale_attr(double_round=False))
        np.testing.assert_array_equal(a, b)
    s = np.array([33], np.int8)
    xs = np.array([1, -1, 2, -2, 3, -3], np.int32)  # x*m/2^33 ~ +-0.177k: the nudge flips nothing here ...
    m2 = np.array([2 ** 30 + 2 ** 29], np.int32)     # ... but 3*1.5*2^30 / 2^33 = 0.5625 vs 0.5 boundary does
    a = oracle.rescale(xs, m2, np.array([33], np.int8), abi.I32, abi.rescale_attr(double_round=True))
    exp = [rescale_exact(v, 0, int(m2[0]), 33, True, 0, -2 ** 31, 2 ** 31 - 1) for v in xs]
    assert a.tolist() == exp
    assert s[0] == 33


def test_rescale_truncates_to_int32_before_zero_point_and_clamps(abi, oracle):
    # value * mult >> shift = 2^32 + 5 -> int32 truncation gives 5 (no saturation), then +zp, then clamp
    x = np.array([2 ** 31 - 1, -(2 ** 31), 100], np.int32)
    mult = np.array([2 ** 30], np.int32)
    shift = np.array([2], np.int8)  # x * 2^28: overflows int32
    out = oracle.rescale(x, mult, shift, abi.I32, abi.rescale_attr(0, 0))
    exp = [rescale_exact(v, 0, 2 ** 30, 2, False, 0, -2 ** 31, 2 ** 31 - 1) for v in x]
    assert out.tolist() == exp
    out8 = oracle.rescale(np.array([1000, -1000, 5], np.int32), np.array([1 << 30], np.int32),
                          np.array([30], np.int8), abi.I8, abi.rescale_attr(0, 10))
    assert out8.tolist() == [127, -128, 15]


def test_rescale_i8_to_i32_input_zero_point_and_unsigned(abi, oracle):
    x = np.array([-128, -1, 0, 1, 127], np.int8)
    m = np.array([1 << 30], np.int32)
    s = np.array([30], np.int8)
    assert oracle.rescale(x, m, s, abi.I32, abi.rescale_attr(-5, 0)).tolist() == [-123, 4, 5, 6, 132]
    # input_unsigned: the same bytes read as uint8, zero point cast to uint8 as well
    assert oracle.rescale(x, m, s, abi.I32, abi.rescale_attr(128, 0, input_unsigned=True)).tolist() == \
        [0, 127, -128, -127, -1]
    # output_unsigned: clamp to [0,255], bytes stored as uint8
    out = oracle.rescale(np.array([-7, 100, 300], np.int32), m, s, abi.I8, abi.rescale_attr(0, 0, output_unsigned=True))
    assert out.view(np.uint8).tolist() == [0, 100, 255]


def test_rescale_scale16(abi, oracle):
    x = ri(-2 ** 20, 2 ** 20, (64,), np.int32)
    m = np.array([23170], np.int16)
    s = np.array([20], np.int8)
    out = oracle.rescale(x, m, s, abi.I16, abi.rescale_attr(0, -1, scale32=False, double_round=True))
    exp = [rescale_exact(v, 0, 23170, 20, False, -1, -32768, 32767) for v in x]
    assert out.tolist() == exp


# ---------------------------------------------------------------- CLAMP, ADD/SUB, MUL, TABLE
def test_clamp_vs_numpy(abi, oracle):
    x = ri(-128, 127, (3, 50), np.int8)
    np.testing.assert_array_equal(oracle.clamp(x, -3, 100), np.clip(x, -3, 100))
    f = RNG.standard_normal(100).astype(np.float32)
    f[5] = np.nan
    out = oracle.clamp(f, -0.5, 0.25, abi.NAN_PROPAGATE)
    assert np.isnan(out[5])
    np.testing.assert_array_equal(np.delete(out, 5), np.clip(np.delete(f, 5), -0.5, 0.25))
    assert oracle.clamp(f, -0.5, 0.25, abi.NAN_IGNORE)[5] == np.float32(-0.5)


def test_add_sub_i32_wrap_and_broadcast(abi, oracle):
    a = ri(-2 ** 31, 2 ** 31 - 1, (2, 3, 4), np.int32)
    b = ri(-2 ** 31, 2 ** 31 - 1, (2, 1, 4), np.int32)
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(oracle.elementwise_binary("ADD", a, b, a.shape, abi.I32), a + b)
        np.testing.assert_array_equal(oracle.elementwise_binary("SUB", a, b, a.shape, abi.I32), a - b)


def test_mul_shift_vs_python_ints(abi, oracle):
    a = ri(-2 ** 31, 2 ** 31 - 1, (200,), np.int32)
    b = ri(-2 ** 15, 2 ** 15, (200,), np.int32)
    for shift in (0, 1, 15, 31):
        out = oracle.mul(a, b, a.shape, abi.I32, shift)
        exp = []
        for x, y in zip(a.tolist(), b.tolist()):
            r = x * y
            if shift > 0:
                r = (r + (1 << (shift - 1))) >> shift
            exp.append((r + 2 ** 31) % 2 ** 32 - 2 ** 31)
        assert out.tolist() == exp


def test_table_i8_and_i16(abi, oracle):
    x = np.arange(-128, 128, dtype=np.int8)
    tab = ri(-128, 127, (256,), np.int8)
    np.testing.assert_array_equal(oracle.table(x, tab, abi.I8), tab[x.astype(np.int32) + 128])
    x16 = np.array([-32768, -32767, -1, 0, 1, 127, 128, 32767], np.int16)
    t16 = ri(-32768, 32767, (513,), np.int16)
    out = oracle.table(x16, t16, abi.I32)
    exp = []
    for v in x16.tolist():
        i, f = (v + 32768) >> 7, v & 0x7F
        exp.append((int(t16[i]) << 7) + (int(t16[i + 1]) - int(t16[i])) * f)
    assert out.tolist() == exp
    # a linear table interpolates exactly: table[i] = i - 256 -> out = 128*(i-256) + frac = v
    lin = (np.arange(513) - 256).astype(np.int16)
    np.testing.assert_array_equal(oracle.table(x16, lin, abi.I32), x16.astype(np.int32))


# ---------------------------------------------------------------- pooling
def round_half_away_div(acc, count):
    q = Fraction(acc, count)
    return int(q + Fraction(1, 2)) if q >= 0 else -int(-q + Fraction(1, 2))


def test_avg_pool2d_global_and_padded(abi, oracle):
    x = ri(-128, 127, (2, 7, 7, 6), np.int8)
    out = oracle.avg_pool2d(x, (2, 1, 1, 6), abi.pool2d_attr((7, 7), (1, 1), (0, 0, 0, 0), input_zp=-3, output_zp=2))
    for n in range(2):
        for c in range(6):
            acc = int(x[n, :, :, c].astype(np.int64).sum()) + 3 * 49
            assert out[n, 0, 0, c] == min(max(round_half_away_div(acc, 49) + 2, -128), 127)
    # padding: the divisor counts only in-bounds taps
    y = np.full((1, 2, 2, 1), 10, np.int8)
    o2 = oracle.avg_pool2d(y, (1, 2, 2, 1), abi.pool2d_attr((2, 2), (1, 1), (1, 0, 1, 0)))
    assert (o2 == 10).all()
    # round half away from zero on negatives: (-3)/2 -> -2 (not -1)
    z = np.array([-1, -2], np.int8).reshape(1, 1, 2, 1)
    assert oracle.avg_pool2d(z, (1, 1, 1, 1), abi.pool2d_attr((1, 2), (1, 1), (0, 0, 0, 0))).item() == -2


def test_max_pool2d_padding(abi, oracle):
    x = ri(-128, 127, (1, 5, 5, 3), np.int8)
    out = oracle.max_pool2d(x, (1, 3, 3, 3), abi.pool2d_attr((3, 3), (2, 2), (1, 1, 1, 1)))
    xp = np.full((1, 7, 7, 3), -128, np.int8)
    xp[:, 1:6, 1:6] = x
    for oy in range(3):
        for ox in range(3):
            np.testing.assert_array_equal(out[0, oy, ox], xp[0, 2 * oy:2 * oy + 3, 2 * ox:2 * ox + 3].max(axis=(0, 1)))


# ---------------------------------------------------------------- reduce, cast, data movement
def test_reduce_vs_numpy(abi, oracle):
    x = ri(-1000, 1000, (3, 4, 5), np.int32)
    for axis in range(3):
        np.testing.assert_array_equal(oracle.reduce("SUM", x, axis), x.sum(axis=axis, keepdims=True))
        np.testing.assert_array_equal(oracle.reduce("MAX", x, axis), x.max(axis=axis, keepdims=True))
        np.testing.assert_array_equal(oracle.reduce("MIN", x, axis), x.min(axis=axis, keepdims=True))
    f = RNG.standard_normal((4, 33)).astype(np.float32)
    np.testing.assert_allclose(oracle.reduce("SUM", f, 1), f.sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-5)
    b = RNG.integers(0, 2, (4, 6)).astype(np.bool_)
    np.testing.assert_array_equal(oracle.reduce("ALL", b, 1), b.all(axis=1, keepdims=True))
    np.testing.assert_array_equal(oracle.reduce("ANY", b, 1), b.any(axis=1, keepdims=True))


def test_reduce_sum_f16_is_sequential_in_f16(abi, oracle):
    # 2048 + 1 + 1 ... in binary16 never advances past 2048 (each +1 rounds back): sequential-f16 semantics
    x = np.array([[2048.0] + [1.0] * 10], np.float16)
    assert oracle.reduce("SUM", x, 1).item() == 2048.0


def test_cast_rules(abi, oracle):
    x = np.array([300, -300, 127, -128, 65536 + 7], np.int32)
    np.testing.assert_array_equal(oracle.cast(x, abi.I8), x.astype(np.int8))  # wraps
    f = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 1e9, -1e9, 126.5], np.float32)
    assert oracle.cast(f, abi.I8).tolist() == [0, 2, 2, 0, -2, 127, -128, 126]  # clamp + round half even
    big = np.array([70000, -70000, 1000], np.int32)
    out = oracle.cast(big, abi.F16)
    assert np.isposinf(out[0]) and np.isneginf(out[1]) and out[2] == 1000
    assert oracle.cast(np.array([0, 3, -1], np.int32), abi.BOOL).tolist() == [False, True, True]


def test_data_movement_vs_numpy(abi, oracle):
    x = ri(-128, 127, (2, 3, 4, 5), np.int8)
    np.testing.assert_array_equal(oracle.reshape(x, (6, 20)), x.reshape(6, 20))
    for perms in [(0, 2, 1, 3), (3, 2, 1, 0), (1, 0, 3, 2)]:
        np.testing.assert_array_equal(oracle.transpose(x, perms), x.transpose(perms))
    np.testing.assert_array_equal(oracle.slice_(x, (1, 0, 2, 1), (1, 3, 2, 3)), x[1:2, 0:3, 2:4, 1:4])
    np.testing.assert_array_equal(oracle.concat([x, x[:, :2]], 1), np.concatenate([x, x[:, :2]], axis=1))
    pads = [(0, 0), (1, 2), (0, 1), (2, 0)]
    x32 = x.astype(np.int32)
    out_shape = tuple(d + a + b for d, (a, b) in zip(x.shape, pads))
    np.testing.assert_array_equal(oracle.pad(x32, np.array(pads).reshape(-1), out_shape, pad_const_int=-7),
                                  np.pad(x32, pads, constant_values=-7))
    np.testing.assert_array_equal(oracle.pad(x, np.array(pads).reshape(-1), out_shape, pad_const=9),
                                  np.pad(x, pads, constant_values=9))


def test_negate(abi, oracle):
    x = np.array([-128, -1, 0, 5, 127], np.int8)
    assert oracle.negate(x, 0, 0).tolist() == [127, 1, 0, -5, -127]
    assert oracle.negate(x, 3, -2).tolist() == [127, 2, 1, -4, -126]


# ---------------------------------------------------------------- binary16 codec
def test_f16_codec_matches_numpy_for_all_bit_patterns(oracle):
    lib = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 7):
        got = lib.mlel_cpu_f16_to_f32(int(b))
        if np.isnan(ref[b]):
            assert np.isnan(got)
        else:
            assert got == ref[b]
    vals = np.concatenate([RNG.standard_normal(2000) * 10.0 ** RNG.integers(-8, 5, 2000), [65504, 65520, 65519.9, 1e-8,
                           6e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 0.0, -0.0]]).astype(np.float32)
    for v in vals:
        assert lib.mlel_cpu_f32_to_f16(float(v)) == int(np.float32(v).astype(np.float16).view(np.uint16))


def test_transformer_block_oracle_vs_fp32_numpy(oracle):
    """The fp16 encoder-block description executed by the oracle agrees with an independent fp32 numpy
    computation of the same mathematics (tests/transformer_ref.py) to fp16 rounding of the intermediates."""
    import importlib
    from oracle_graph import run_spec
    from transformer_ref import encoder_block_fp32
    graphs = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.graphs")
    spec = graphs.transformer_block_spec(batch=2, seq=48, d_model=128, heads=4, ffn=256)
    assert len(spec.ops) == 78
    x = np.random.default_rng(7).standard_normal((2, 48, 128)).astype(np.float16)
    out, env = run_spec(oracle, spec, {"input": x})
    ref = encoder_block_fp32(spec, x, 4)
    assert np.abs(out["output"].astype(np.float32) - ref).max() <= 5e-3
    # softmax rows (the MUL that follows RECIPROCAL) sum to 1 within fp16 rounding
    probs = [v for k, v in env.items() if isinstance(v, np.ndarray) and v.shape == (8, 48, 48) and v.dtype == np.float16
             and v.min() >= 0 and abs(float(v[0, 0].astype(np.float32).sum()) - 1.0) < 2e-2]
    assert probs, "no tensor with unit row sums found"
