"""bf16 and fp8 (e4m3, e5m2) tensors in the floating-point operators.

The reference decodes these storage formats into a wider type for the arithmetic (bf16 -> fp32, fp8 -> fp16) and
encodes results by rules of its own (graph/shaders/graph_op/common.comp:184-232, 300-418, 611-633): bf16 truncates
except in the ADD-like operators, MUL and CAST, which round to nearest even; fp8 goes through fp16 and then drops
mantissa bits (e5m2) or rounds them to nearest even (e4m3), saturating to infinity / the NaN code.  The reference's
tests create such pipelines but hold no values (tests/vulkan.cpp:1319-1329), so the CPU part pins the oracle's codecs
against torch's bfloat16 / float8 types where the rules coincide and against bit-level numpy statements where they
do not, and the operators against numpy statements built from those codecs.  The GPU part compares the HIP kernels
with the oracle bit for bit.
"""
import numpy as np
import pytest
import torch

from hip_util import Runner, abi, gpu_available, hb

BF16, E4M3, E5M2 = abi.BF16, abi.F8E4M3, abi.F8E5M2
LOWP = [BF16, E4M3, E5M2]
NAMES = {BF16: "bf16", E4M3: "f8e4m3", E5M2: "f8e5m2"}


# ------------------------------------------------------------------------------------------------ numpy codecs
def np_decode(bits, dt):
    bits = np.asarray(bits)
    if dt == BF16:
        return (bits.astype(np.uint32) << 16).view(np.float32)
    if dt == E5M2:
        return (bits.astype(np.uint16) << 8).view(np.float16).astype(np.float32)
    sign = np.where(bits & 0x80, -1.0, 1.0)
    e, m = (bits >> 3) & 0xF, bits & 7
    v = np.where(e == 0, m / 512.0, np.ldexp(1.0 + m / 8.0, e.astype(np.int32) - 7))
    v = np.where((e == 15) & (m == 7), np.nan, v)
    return (sign * v).astype(np.float32)


def np_bf16_trunc(x):
    return (np.asarray(x, np.float32).view(np.uint32) >> 16).astype(np.uint16)


def torch_bf16_rne(x):
    return torch.from_numpy(np.asarray(x, np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def np_e5m2_from_f32(x):
    """round to fp16 (nearest even), keep the upper byte; NaN -> 0x7d, beyond +-57344 -> infinity"""
    x = np.asarray(x, np.float32)
    sign = ((x.view(np.uint32) >> 24) & 0x80).astype(np.uint8)
    with np.errstate(over="ignore"):
        body = (x.astype(np.float16).view(np.uint16) >> 8).astype(np.uint8)
    body = np.where(np.isinf(x) | (np.abs(x) > 57344.0), sign | 0x7C, body)
    return np.where(np.isnan(x), sign | 0x7D, body).astype(np.uint8)


def torch_e4m3(x):
    return torch.from_numpy(np.asarray(x, np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def oracle_encode(oracle, x, dt, rne=False):
    lib = oracle.lib()
    x = np.asarray(x, np.float32).ravel()
    if dt == BF16:
        return np.array([lib.mlel_cpu_f32_to_bf16(float(v), 1 if rne else 0) for v in x], np.uint16)
    return np.array([lib.mlel_cpu_f32_to_f8(float(v), dt) for v in x], np.uint8)


def sample_floats(rng, n, lo_exp, hi_exp):
    """floats spread over binades lo_exp..hi_exp, both signs, plus values exactly between representable neighbours"""
    mant = rng.random(n).astype(np.float32) + 1.0
    exps = rng.integers(lo_exp, hi_exp, n, endpoint=True)
    sign = rng.choice([-1.0, 1.0], n).astype(np.float32)
    return (sign * np.ldexp(mant, exps)).astype(np.float32)


# ------------------------------------------------------------------------------------------------ CPU: codecs pinned
def test_decoders_agree_with_torch_on_every_code(oracle):
    lib = oracle.lib()
    codes = np.arange(256, dtype=np.uint8)
    for dt, tdt in ((E4M3, torch.float8_e4m3fn), (E5M2, torch.float8_e5m2)):
        want = torch.from_numpy(codes).view(tdt).to(torch.float32).numpy()
        got = np.array([lib.mlel_cpu_f8_to_f32(int(c), dt) for c in codes], np.float32)
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
        np.testing.assert_array_equal(got[~np.isnan(want)], want[~np.isnan(want)])
        np.testing.assert_array_equal(np_decode(codes, dt)[~np.isnan(want)], want[~np.isnan(want)])
    words = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = torch.from_numpy(words.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    got = oracle.cast(abi.typed(words, BF16), abi.F32)
    ok = ~np.isnan(want)
    np.testing.assert_array_equal(np.isnan(got), ~ok)
    np.testing.assert_array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok])  # signed zeros, infinities included


def test_bf16_encoders(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([sample_floats(rng, 4000, -130, 127), np.float32([0, -0.0, np.inf, -np.inf, 1, 1.00390625,
                                                                         1.01171875, 3.3895314e38, 3.4e38, 1e-40])])
    # exact ties between two bf16 neighbours, even and odd below
    ties = ((rng.integers(0, 2 ** 15, 500).astype(np.uint32) << 16) | 0x8000).view(np.float32)
    x = np.concatenate([x, ties[np.isfinite(ties)]])  # (NaN keeps its payload here, torch canonicalises it)
    np.testing.assert_array_equal(oracle_encode(oracle, x, BF16, rne=True), torch_bf16_rne(x))
    np.testing.assert_array_equal(oracle_encode(oracle, x, BF16, rne=False), np_bf16_trunc(x))
    nan = oracle_encode(oracle, np.float32([np.nan]), BF16, rne=True)
    assert np.isnan(np_decode(nan, BF16))[0]
    # the nearest-even encoder is the CAST to bf16, the truncating one the store of e.g. ABS
    xs = x[np.isfinite(x)]
    np.testing.assert_array_equal(oracle.cast(xs, BF16), torch_bf16_rne(xs))
    t = abi.typed(torch_bf16_rne(xs), BF16)
    np.testing.assert_array_equal(oracle.elementwise_unary("ABS", t), np.asarray(t) & 0x7FFF)


def test_e5m2_encoder(oracle):
    rng = np.random.default_rng(2)
    x = np.concatenate([sample_floats(rng, 4000, -20, 17),
                        np.float32([0, -0.0, np.inf, -np.inf, np.nan, 57344, 57345, 61440, 65504, 65520, 1e9, -1e9,
                                    2 ** -16, 2 ** -17, 1.5 * 2 ** -16, 6e-8])])
    np.testing.assert_array_equal(oracle_encode(oracle, x, E5M2), np_e5m2_from_f32(x))
    # values that are e5m2 values come back as themselves
    codes = np.array([c for c in range(256) if (c & 0x7C) != 0x7C], np.uint8)
    np.testing.assert_array_equal(oracle_encode(oracle, np_decode(codes, E5M2), E5M2), codes)
    assert oracle_encode(oracle, np.float32([np.nan]), E5M2)[0] & 0x7F == 0x7D


def test_e4m3_encoder_is_round_to_nearest_even_up_to_448(oracle):
    rng = np.random.default_rng(3)
    x = np.concatenate([sample_floats(rng, 6000, -12, 8), np.float32([0, -0.0, 448, -448, 2 ** -9, 2 ** -10,
                                                                      1.5 * 2 ** -9, 2 ** -6, 0.9999 * 2 ** -6])])
    # every midpoint between two neighbouring e4m3 values (ties go to the even code)
    codes = np.arange(0, 0x7E, dtype=np.uint8)
    vals = np_decode(codes, E4M3).astype(np.float64)
    mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)
    x = np.concatenate([x, mids, -mids])
    x = x[np.abs(x) <= 448]
    np.testing.assert_array_equal(oracle_encode(oracle, x, E4M3), torch_e4m3(x))
    np.testing.assert_array_equal(oracle_encode(oracle, np_decode(codes, E4M3), E4M3), codes)
    # beyond the largest value, infinities and NaN: the NaN code with the sign (common.comp:334-336)
    bad = np.float32([448.5, 500, 1e9, np.inf, np.nan, -449, -np.inf])
    np.testing.assert_array_equal(oracle_encode(oracle, bad, E4M3) & 0x7F, np.full(7, 0x7F))
    np.testing.assert_array_equal(oracle_encode(oracle, bad, E4M3)[[0, 5, 6]] >> 7, [0, 1, 1])


# ------------------------------------------------------------------------------------------------ CPU: operators pinned
def random_codes(rng, dt, shape, finite=True, small=False):
    """random storage words whose values are finite (and moderate when `small`)"""
    if dt == BF16:
        lo, hi = (-6, 6) if small else (-60, 60)
        x = sample_floats(rng, int(np.prod(shape)), lo, hi)
        return abi.typed(np_bf16_trunc(x).reshape(shape), dt)
    codes = rng.integers(0, 255, shape, endpoint=True).astype(np.uint8)
    if dt == E4M3:
        codes = np.where((codes & 0x7F) == 0x7F, codes & 0xF0, codes)
        if small:
            codes = np.where((codes & 0x7F) > 0x58, codes & 0xBF, codes)  # |v| <= 16
    else:
        codes = np.where((codes & 0x7C) == 0x7C, codes & 0xE3, codes)
        if small:
            codes = np.where((codes & 0x7F) > 0x4C, codes & 0xBF, codes)  # |v| <= 16
    return abi.typed(codes.astype(np.uint8), dt)


def np_store(v32, dt, mode):
    """numpy statement of the three store rules; v32 is the fp32 result"""
    v32 = np.asarray(v32, np.float32)
    if dt == BF16:
        return torch_bf16_rne(v32) if mode == "rne" else np_bf16_trunc(v32)
    f = v32 if mode == "acc" else v32.astype(np.float16).astype(np.float32)
    if dt == E5M2:
        return np_e5m2_from_f32(f)
    out = torch_e4m3(np.clip(f, -448, 448))
    return np.where(np.isnan(f) | (np.abs(f) > 448), ((f.view(np.uint32) >> 24) & 0x80).astype(np.uint8) | 0x7F, out)


@pytest.mark.parametrize("dt", LOWP, ids=[NAMES[d] for d in LOWP])
def test_oracle_add_mul_cast_against_numpy(oracle, dt):
    rng = np.random.default_rng(10 + dt)
    a, b = random_codes(rng, dt, (7, 33), small=True), random_codes(rng, dt, (7, 33), small=True)
    fa, fb = np_decode(np.asarray(a), dt), np_decode(np.asarray(b), dt)
    comp = (lambda v: v.astype(np.float16).astype(np.float32)) if dt != BF16 else (lambda v: v)
    np.testing.assert_array_equal(oracle.elementwise_binary("ADD", a, b, a.shape, dt), np_store(comp(fa + fb), dt, "rne"))
    np.testing.assert_array_equal(oracle.elementwise_binary("SUB", a, b, a.shape, dt), np_store(comp(fa - fb), dt, "rne"))
    np.testing.assert_array_equal(oracle.mul(a, b, a.shape, dt), np_store(fa * fb, dt, "rne"))
    np.testing.assert_array_equal(oracle.elementwise_binary("MAXIMUM", a, b, a.shape, dt),
                                  np_store(np.maximum(fa, fb), dt, "rne"))
    # widening casts are exact, narrowing ones follow the encoders
    np.testing.assert_array_equal(oracle.cast(a, abi.F32), fa)
    x = sample_floats(rng, 500, -8, 7)
    np.testing.assert_array_equal(oracle.cast(x, dt), np_store(x, dt, "rne" if dt == BF16 else "acc"))
    h = x.astype(np.float16)
    np.testing.assert_array_equal(oracle.cast(h, dt), np_store(h.astype(np.float32), dt, "rne" if dt == BF16 else "acc"))
    i = rng.integers(-300, 300, 200).astype(np.int32)
    np.testing.assert_array_equal(oracle.cast(i, dt), np_store(i.astype(np.float32), dt, "rne" if dt == BF16 else "acc"))
    np.testing.assert_array_equal(oracle.cast(a, abi.I32), np.clip(np.rint(fa), -2.0 ** 31, 2.0 ** 31 - 1).astype(np.int64))
    np.testing.assert_array_equal(oracle.cast(a, abi.BOOL), fa != 0)


@pytest.mark.parametrize("dt", LOWP, ids=[NAMES[d] for d in LOWP])
def test_oracle_reduce_clamp_conv_against_numpy(oracle, dt):
    rng = np.random.default_rng(20 + dt)
    a = random_codes(rng, dt, (5, 19), small=True)
    fa = np_decode(np.asarray(a), dt)
    # sequential fold in the compute type, truncating store
    acc = np.zeros(5, np.float32)
    for j in range(19):
        acc = acc + fa[:, j]
        if dt != BF16:
            acc = acc.astype(np.float16).astype(np.float32)
    np.testing.assert_array_equal(oracle.reduce("SUM", a, 1)[:, 0], np_store(acc, dt, "trunc"))
    np.testing.assert_array_equal(oracle.reduce("MAX", a, 1)[:, 0], np_store(fa.max(axis=1), dt, "trunc"))
    np.testing.assert_array_equal(oracle.clamp(a, -1.5, 2.0), np_store(np.clip(fa, -1.5, 2.0), dt, "trunc"))
    # CONV2D: the accumulator type is fp32 for bf16 and fp16 for fp8; the store encodes the accumulator directly
    x, w = random_codes(rng, dt, (1, 4, 4, 3), small=True), random_codes(rng, dt, (2, 2, 2, 3), small=True)
    bias = random_codes(rng, dt, (2,), small=True)
    fx, fw, fb = (np_decode(np.asarray(t), dt) for t in (x, w, bias))
    f16 = lambda v: np.float32(np.float16(v))
    out = np.zeros((1, 3, 3, 2), np.float32)
    for oy in range(3):
        for ox in range(3):
            for oc in range(2):
                s = np.float32(0)
                for ky in range(2):
                    for kx in range(2):
                        for ic in range(3):
                            p = np.float32(fx[0, oy + ky, ox + kx, ic] * fw[oc, ky, kx, ic])
                            s = f16(s + f16(p)) if dt != BF16 else np.float32(s + p)
                out[0, oy, ox, oc] = f16(s + fb[oc]) if dt != BF16 else np.float32(s + fb[oc])
    attr = abi.conv2d_attr(acc_type=abi.ACC_F32 if dt == BF16 else abi.ACC_F16)
    np.testing.assert_array_equal(oracle.conv2d(x, w, bias, (1, 3, 3, 2), dt, attr), np_store(out, dt, "acc"))


# ------------------------------------------------------------------------------------------------ GPU vs oracle
pytestmark_gpu = pytest.mark.skipif(not gpu_available(), reason="needs an AMD GPU (no CPU path exists)")


@pytest.fixture(scope="module")
def run():
    dev = hb.Device(0)
    yield Runner(dev)
    dev.close()


@pytest.mark.gpu
@pytestmark_gpu
@pytest.mark.parametrize("dt", LOWP, ids=[NAMES[d] for d in LOWP])
def test_hip_elementwise_cast_reduce_in_low_precision_formats(run, oracle, dt):
    rng = np.random.default_rng(30 + dt)
    a, b = random_codes(rng, dt, (6, 5, 40)), random_codes(rng, dt, (6, 1, 40))
    for op in ("ADD", "SUB", "MAXIMUM", "MINIMUM"):
        np.testing.assert_array_equal(run.binary(op, a, b, a.shape, dt), oracle.elementwise_binary(op, a, b, a.shape, dt),
                                      err_msg=op)
    for op in ("EQUAL", "GREATER", "GREATER_EQUAL"):
        np.testing.assert_array_equal(run.binary(op, a, b, a.shape, abi.BOOL),
                                      oracle.elementwise_binary(op, a, b, a.shape, abi.BOOL), err_msg=op)
    np.testing.assert_array_equal(run.mul(a, b, a.shape, dt), oracle.mul(a, b, a.shape, dt))
    for op in ("ABS", "CEIL", "FLOOR"):
        np.testing.assert_array_equal(run.unary(op, a), oracle.elementwise_unary(op, a), err_msg=op)
    np.testing.assert_array_equal(run.negate(a), oracle.negate(a))
    np.testing.assert_array_equal(run.clamp(a, -3.25, 17.5), oracle.clamp(a, -3.25, 17.5))
    for out_dt in (abi.F32, abi.F16, abi.I32, abi.I8, abi.BOOL, BF16, E4M3, E5M2):
        np.testing.assert_array_equal(run.cast(a, out_dt), oracle.cast(a, out_dt), err_msg=f"cast to {out_dt}")
    x = np.concatenate([sample_floats(rng, 3000, -20, 18), np.float32([0, -0.0, np.inf, -np.inf, 448, 449, 57344, 6e4])])
    with np.errstate(over="ignore"):
        halves = x.astype(np.float16)  # (values beyond 65504 become infinities on purpose)
    for src in (x, halves, rng.integers(-70000, 70000, 500).astype(np.int32),
                rng.integers(-128, 127, 300).astype(np.int8), rng.integers(0, 1, 50, endpoint=True).astype(np.bool_)):
        np.testing.assert_array_equal(run.cast(src, dt), oracle.cast(src, dt), err_msg=str(src.dtype))
    s = random_codes(rng, dt, (4, 37, 9), small=True)
    for op in ("SUM", "MAX", "MIN", "PRODUCT"):
        for axis in (1, 2):
            np.testing.assert_array_equal(run.reduce(op, s, axis), oracle.reduce(op, s, axis), err_msg=f"{op} {axis}")
    # transcendental results may differ in the last place of the compute type: at most one storage step apart
    e = random_codes(rng, dt, (500,), small=True)
    got, want = run.unary("EXP", e), oracle.elementwise_unary("EXP", e)
    assert np.max(np.abs(got.astype(np.int32) - np.asarray(want).astype(np.int32))) <= 1


@pytest.mark.gpu
@pytestmark_gpu
@pytest.mark.parametrize("dt", LOWP, ids=[NAMES[d] for d in LOWP])
def test_hip_packed_elementwise_and_cast_in_low_precision_formats(run, oracle, dt):
    """Dense tensors whose rows are a multiple of eight elements take the kernels with 64- / 128-bit accesses:
    ADD, SUB, MUL (same shape, a row broadcast, a column broadcast, a single element) and CAST in both directions."""
    rng = np.random.default_rng(50 + dt)
    shape = (5, 7, 48)
    a = random_codes(rng, dt, shape)
    for b in (random_codes(rng, dt, shape), random_codes(rng, dt, (1, 1, 48)), random_codes(rng, dt, (5, 7, 1)),
              random_codes(rng, dt, (1, 1, 1))):
        for op in ("ADD", "SUB"):
            np.testing.assert_array_equal(run.binary(op, a, b, shape, dt), oracle.elementwise_binary(op, a, b, shape, dt),
                                          err_msg=f"{op} {b.shape}")
        np.testing.assert_array_equal(run.mul(a, b, shape, dt), oracle.mul(a, b, shape, dt), err_msg=f"MUL {b.shape}")
    for out_dt in (abi.F32, abi.F16, BF16, E4M3, E5M2):
        if out_dt != dt:
            np.testing.assert_array_equal(run.cast(a, out_dt), oracle.cast(a, out_dt), err_msg=f"cast to {out_dt}")
    x = np.concatenate([sample_floats(rng, 4088, -20, 18), np.float32([0, -0.0, np.inf, -np.inf, 448, 449, 57344, 6e4])])
    with np.errstate(over="ignore"):
        halves = x.astype(np.float16)
    for src in (x.reshape(8, 512), halves.reshape(64, 64)):
        np.testing.assert_array_equal(run.cast(src, dt), oracle.cast(src, dt), err_msg=str(src.dtype))


@pytest.mark.gpu
@pytestmark_gpu
@pytest.mark.parametrize("dt", LOWP, ids=[NAMES[d] for d in LOWP])
def test_hip_contractions_pools_and_movement_in_low_precision_formats(run, oracle, dt):
    rng = np.random.default_rng(40 + dt)
    acc = abi.ACC_F32 if dt == BF16 else abi.ACC_F16
    x, w = random_codes(rng, dt, (2, 9, 8, 5), small=True), random_codes(rng, dt, (6, 3, 3, 5), small=True)
    bias = random_codes(rng, dt, (6,), small=True)
    attr = abi.conv2d_attr((1, 1, 1, 1), (2, 1), (1, 1), 0, 0, acc)
    np.testing.assert_array_equal(run.conv2d(x, w, bias, (2, 5, 8, 6), dt, attr),
                                  oracle.conv2d(x, w, bias, (2, 5, 8, 6), dt, attr))
    dw, dbias = random_codes(rng, dt, (3, 3, 5, 2), small=True), random_codes(rng, dt, (10,), small=True)
    dattr = abi.conv2d_attr((1, 1, 1, 1), (1, 1), (1, 1), 0, 0, acc)
    np.testing.assert_array_equal(run.conv2d(x, dw, dbias, (2, 9, 8, 10), dt, dattr, depthwise=True),
                                  oracle.depthwise_conv2d(x, dw, dbias, (2, 9, 8, 10), dt, dattr))
    a, b = random_codes(rng, dt, (2, 7, 12), small=True), random_codes(rng, dt, (2, 12, 5), small=True)
    for out_dt in ((abi.F32, BF16) if dt == BF16 else (abi.F16,)):
        np.testing.assert_array_equal(run.matmul(a, b, out_dt), oracle.matmul(a, b, out_dt), err_msg=f"matmul {out_dt}")
    pattr = abi.pool2d_attr((2, 2), (2, 2), (0, 0, 0, 0), acc)
    np.testing.assert_array_equal(run.pool("avg_pool2d", x[:, :8], (2, 4, 4, 5), pattr),
                                  oracle.avg_pool2d(x[:, :8], (2, 4, 4, 5), pattr))
    mattr = abi.pool2d_attr((3, 2), (1, 2), (1, 1, 0, 0), acc)
    np.testing.assert_array_equal(run.pool("max_pool2d", x, (2, 9, 4, 5), mattr), oracle.max_pool2d(x, (2, 9, 4, 5), mattr))
    np.testing.assert_array_equal(run.transpose(x, (0, 3, 1, 2)), oracle.transpose(x, (0, 3, 1, 2)))
    np.testing.assert_array_equal(run.concat([x, x[:, :2]], 1), oracle.concat([x, x[:, :2]], 1))
    padding = np.array([0, 0, 1, 2, 0, 1, 0, 0], np.int32).reshape(4, 2)
    np.testing.assert_array_equal(run.pad(x, padding, (2, 12, 9, 5), 1.3), oracle.pad(x, padding, (2, 12, 9, 5), 1.3))
    np.testing.assert_array_equal(run.argmax(x, 2), oracle.argmax(x, 2))
