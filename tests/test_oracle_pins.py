"""Pins the remaining oracle functions -- the floating-point unary operators, the elementwise binary operators beyond
ADD / SUB / MAXIMUM, and REDUCE PRODUCT / MIN / MAX -- against what the mathematics fixes: the C library in double
precision rounded once, Python's exact integers, the shader's own polynomial coefficients evaluated independently.
Reference arithmetic: graph/shaders/graph_op/tosa/elementwise_unary.comp:16-205, elementwise_binary.comp:33-173
(operation strings graph/compute_graph_op.cpp:2527-2946), reduce.comp:24-70.  CPU only."""
import math

import numpy as np
import pytest

RNG = np.random.default_rng(11)


def wrap(v, bits):
    """two's-complement truncation of a Python integer to `bits` bits"""
    m = 1 << bits
    return (v + (m >> 1)) % m - (m >> 1)


def f32(v):
    return float(np.float32(v))


# ---------------------------------------------------------------- floating-point unary operators
def unary_cases():
    lin = np.linspace(-12.0, 12.0, 481)
    small = np.array([0.0, -0.0, 1e-8, -1e-8, 1e-3, 0.1999, 0.2, 0.2001, -0.1999, -0.2, 0.5, 0.5999, 0.6, 0.6001,
                      3.9999, 4.0, 4.0001, 9.9999, 10.0, 10.0001, -10.0001, 80.0, -80.0])
    return np.concatenate([lin, small, RNG.standard_normal(200) * 3.0])


@pytest.mark.parametrize("dt", [np.float32, np.float16])
@pytest.mark.parametrize("op,fn", [
    ("EXP", np.exp), ("COS", np.cos), ("CEIL", np.ceil), ("FLOOR", np.floor), ("ABS", np.abs),
    ("RECIPROCAL", lambda v: 1.0 / v), ("SIGMOID", lambda v: 1.0 / (1.0 + np.exp(-v))),
])
def test_unary_equals_double_precision_library_rounded_once(oracle, op, fn, dt):
    """EXP, COS, CEIL, FLOOR, ABS, RECIPROCAL, SIGMOID: the operator's definition evaluated in double precision and
    rounded once to the storage type -- the correctly rounded result, whatever constant or rounding the restatement
    got wrong would differ from it."""
    x = unary_cases().astype(dt)
    with np.errstate(all="ignore"):
        exp = fn(x.astype(np.float64)).astype(dt)
    got = oracle.elementwise_unary(op, x)
    np.testing.assert_array_equal(got.view(np.uint16 if dt == np.float16 else np.uint32),
                                  exp.view(np.uint16 if dt == np.float16 else np.uint32))


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_log_and_rsqrt_domains(oracle, dt):
    """LOG of a negative number is NaN (log_guarded, elementwise_unary.comp:157-159), LOG(0) = -inf, RSQRT(0) = +inf;
    positive arguments equal the double-precision library rounded once."""
    x = np.abs(unary_cases()).astype(dt)
    x = x[x > 0]
    with np.errstate(all="ignore"):
        np.testing.assert_array_equal(oracle.elementwise_unary("LOG", x), np.log(x.astype(np.float64)).astype(dt))
        np.testing.assert_array_equal(oracle.elementwise_unary("RSQRT", x),
                                      (1.0 / np.sqrt(x.astype(np.float64))).astype(dt))
    edge = np.array([-1.0, -1e-3, 0.0, 1.0], dt)
    lg = oracle.elementwise_unary("LOG", edge)
    assert np.isnan(lg[0]) and np.isnan(lg[1]) and lg[2] == -np.inf and lg[3] == 0.0
    rs = oracle.elementwise_unary("RSQRT", edge)
    assert np.isnan(rs[0]) and rs[2] == np.inf and rs[3] == 1.0


@pytest.mark.parametrize("op", ["EXP", "LOG", "COS", "SIGMOID", "RECIPROCAL", "RSQRT", "CEIL", "FLOOR", "ERF", "TANH",
                                "SIN", "ABS"])
def test_unary_nan_passes_through(oracle, op):
    """a NaN input is returned as it is, before the operation is applied (elementwise_unary.comp:196-201)"""
    for dt in (np.float32, np.float16):
        out = oracle.elementwise_unary(op, np.array([np.nan, 1.0], dt))
        assert np.isnan(out[0]) and not np.isnan(out[1])


def test_tanh_three_branches(oracle):
    """tanh_clamped (elementwise_unary.comp:136-155): +-1 beyond |x| > 10, the odd polynomial
    x(1 - x^2(1/3 - x^2(2/15 - 17/315 x^2))) below 0.2, the library function between.  The polynomial is checked
    twice: against its own coefficients evaluated in exact rational arithmetic (a wrong coefficient or sign shows at
    1e-7), and against math.tanh, which it approximates to 3e-7 on its interval."""
    from fractions import Fraction as F

    x = np.array([0.0, 1e-4, 0.01, 0.05, 0.1, 0.15, 0.19, 0.1999, -0.1999, -0.1, -0.01], np.float32)
    got = oracle.elementwise_unary("TANH", x)
    for xv, g in zip(x.tolist(), got.tolist()):
        fx = F(xv)
        x2 = fx * fx
        exact_poly = fx * (1 - x2 * (F(1, 3) - x2 * (F(2, 15) - F(17, 315) * x2)))
        assert abs(g - float(exact_poly)) <= 1.5e-7 * max(abs(xv), 1e-30) + 1e-45, (xv, g, float(exact_poly))
        assert abs(g - math.tanh(xv)) <= 3e-7, (xv, g)
    # exactly at the cut-offs the other branch applies: |x| < 0.2 is strict, |x| > 10 is strict
    mid = np.array([0.2, 0.2001, -0.2, 0.5, 1.0, 3.0, 9.9999, 10.0, -10.0, -5.0], np.float32)
    gm = oracle.elementwise_unary("TANH", mid)
    for xv, g in zip(mid.tolist(), gm.tolist()):
        assert abs(g - math.tanh(xv)) <= 1.2e-7, (xv, g)  # fp32 library tanh: within one ulp of the exact value
    big = np.array([10.0001, 11.0, 1e30, np.inf, -10.0001, -1e30, -np.inf], np.float32)
    assert oracle.elementwise_unary("TANH", big).tolist() == [1.0, 1.0, 1.0, 1.0, -1.0, -1.0, -1.0]
    # fp16 storage: the fp32 result rounded once
    h = np.array([0.1, 0.5, -0.15, 11.0, -3.0], np.float16)
    exp = oracle.elementwise_unary("TANH", h.astype(np.float32)).astype(np.float16)
    np.testing.assert_array_equal(oracle.elementwise_unary("TANH", h), exp)


def test_erf_both_approximations(oracle):
    """erf (elementwise_unary.comp:54-134): series below 0.6, Pade product up to 4, +-1 beyond, odd symmetry, erf(0)
    = 0.  Both approximations stay within 5e-7 of math.erf in fp32 (measured 1.5e-7); a wrong coefficient in either
    table moves the result by far more."""
    x = np.concatenate([np.linspace(-4.5, 4.5, 721), [0.0, 0.5999, 0.6, 0.6001, 3.9999, 4.0, 4.0001]]).astype(np.float32)
    got = oracle.elementwise_unary("ERF", x)
    for xv, g in zip(x.tolist(), got.tolist()):
        assert abs(g - math.erf(xv)) <= 5e-7, (xv, g, math.erf(xv))
    np.testing.assert_array_equal(got[:721], -got[:721][::-1])  # erf(-x) = -erf(x) exactly (sign applied last)
    assert oracle.elementwise_unary("ERF", np.array([0.0, 5.0, -5.0, np.inf], np.float32)).tolist() == [0.0, 1.0, -1.0, 1.0]


def test_sin_small_angle_polynomial_and_library(oracle):
    """sin_hybrid (elementwise_unary.comp:161-186): the degree-11 polynomial below 1e-3, sin() above"""
    x = np.array([0.0, 1e-6, 5e-4, 9.99e-4, -5e-4, 1e-3, 0.5, 1.0, -2.0, 3.14159, 100.0], np.float32)
    got = oracle.elementwise_unary("SIN", x)
    for xv, g in zip(x.tolist(), got.tolist()):
        assert abs(g - math.sin(xv)) <= 1.2e-7 * max(1.0, abs(g)), (xv, g)


# ---------------------------------------------------------------- integer unary operators
def test_integer_unary_vs_python(abi, oracle):
    x = np.array([0, 1, -1, 2, 255, 256, -256, 2 ** 31 - 1, -2 ** 31, 0x00F00000, 12345], np.int32)
    np.testing.assert_array_equal(oracle.elementwise_unary("BITWISE_NOT", x), ~x)
    with np.errstate(over="ignore"):
        assert oracle.elementwise_unary("ABS", x).tolist() == [wrap(abs(v), 32) for v in x.tolist()]
    clz = [32 - (v & 0xFFFFFFFF).bit_length() for v in x.tolist()]  # negatives have bit 31 set: 0
    assert oracle.elementwise_unary("CLZ", x).tolist() == clz
    x8 = np.array([-128, -1, 0, 1, 127], np.int8)
    np.testing.assert_array_equal(oracle.elementwise_unary("BITWISE_NOT", x8), ~x8)
    b = np.array([True, False, True], np.bool_)
    np.testing.assert_array_equal(oracle.elementwise_unary("LOGICAL_NOT", b), ~b)


# ---------------------------------------------------------------- elementwise binary operators
@pytest.mark.parametrize("dt,bits", [(np.int8, 8), (np.int16, 16), (np.int32, 32)])
def test_bitwise_and_shifts_vs_python_ints(abi, oracle, dt, bits):
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    a = RNG.integers(lo, hi, 300, endpoint=True).astype(dt)
    b = RNG.integers(lo, hi, 300, endpoint=True).astype(dt)
    od = abi.dtype_of_numpy(dt)
    np.testing.assert_array_equal(oracle.elementwise_binary("BITWISE_AND", a, b, a.shape, od), a & b)
    np.testing.assert_array_equal(oracle.elementwise_binary("BITWISE_OR", a, b, a.shape, od), a | b)
    np.testing.assert_array_equal(oracle.elementwise_binary("BITWISE_XOR", a, b, a.shape, od), a ^ b)
    s = RNG.integers(0, bits - 1, 300, endpoint=True).astype(dt)
    # LOGICAL_LEFT_SHIFT: value1 << value2, truncated to the storage type
    got = oracle.elementwise_binary("LOGICAL_LEFT_SHIFT", a, s, a.shape, od)
    assert got.tolist() == [wrap(int(x) << int(k), bits) for x, k in zip(a, s)]
    # LOGICAL_RIGHT_SHIFT: the value zero-extended from ITS OWN width, then shifted (elementwise_binary.comp:33-37)
    got = oracle.elementwise_binary("LOGICAL_RIGHT_SHIFT", a, s, a.shape, od)
    assert got.tolist() == [wrap((int(x) & ((1 << bits) - 1)) >> int(k), bits) for x, k in zip(a, s)]
    # a shift of a negative 8-bit value by 0 gives the value back, by 1 a positive number below 128
    if bits == 8:
        neg = oracle.elementwise_binary("LOGICAL_RIGHT_SHIFT", np.array([-2, -2], dt), np.array([0, 1], dt), (2,), od)
        assert neg.tolist() == [-2, 127]


def test_comparisons_min_max_intdiv_vs_python_ints(abi, oracle):
    a = RNG.integers(-50, 50, (4, 60), endpoint=True).astype(np.int32)
    b = RNG.integers(-50, 50, (1, 60), endpoint=True).astype(np.int32)  # broadcast along axis 0
    for name, fn in (("EQUAL", np.equal), ("GREATER", np.greater), ("GREATER_EQUAL", np.greater_equal)):
        out = oracle.elementwise_binary(name, a, b, a.shape, abi.BOOL)
        assert out.dtype == np.bool_
        np.testing.assert_array_equal(out, fn(a, b))
    np.testing.assert_array_equal(oracle.elementwise_binary("MINIMUM", a, b, a.shape, abi.I32), np.minimum(a, b))
    np.testing.assert_array_equal(oracle.elementwise_binary("MAXIMUM", a, b, a.shape, abi.I32), np.maximum(a, b))
    # INTDIV truncates toward zero ("value1 / value2" on signed integers): -7 / 2 = -3, 7 / -2 = -3
    n = np.array([7, -7, 7, -7, 0, 1, -1, 2 ** 31 - 1, -2 ** 31 + 1, 100], np.int32)
    d = np.array([2, 2, -2, -2, 5, 3, 3, 7, 7, -7], np.int32)
    exp = [abs(int(x)) // abs(int(y)) * (1 if (int(x) < 0) == (int(y) < 0) else -1) for x, y in zip(n, d)]
    assert oracle.elementwise_binary("INTDIV", n, d, n.shape, abi.I32).tolist() == exp
    bb = RNG.integers(0, 2, (2, 40)).astype(np.bool_)
    cc = RNG.integers(0, 2, (2, 40)).astype(np.bool_)
    np.testing.assert_array_equal(oracle.elementwise_binary("LOGICAL_AND", bb, cc, bb.shape, abi.BOOL), bb & cc)
    np.testing.assert_array_equal(oracle.elementwise_binary("LOGICAL_OR", bb, cc, bb.shape, abi.BOOL), bb | cc)
    np.testing.assert_array_equal(oracle.elementwise_binary("LOGICAL_XOR", bb, cc, bb.shape, abi.BOOL), bb ^ cc)


@pytest.mark.parametrize("dt", [np.float32, np.float16])
def test_float_binary_vs_double_precision(abi, oracle, dt):
    od = abi.dtype_of_numpy(dt)
    a = (RNG.standard_normal(400) * 4).astype(dt)
    b = (RNG.standard_normal(400) * 4).astype(dt)
    b[:20] = a[:20]  # equal pairs for EQUAL / GREATER_EQUAL
    for name, fn in (("EQUAL", np.equal), ("GREATER", np.greater), ("GREATER_EQUAL", np.greater_equal)):
        np.testing.assert_array_equal(oracle.elementwise_binary(name, a, b, a.shape, abi.BOOL), fn(a, b))
    np.testing.assert_array_equal(oracle.elementwise_binary("MINIMUM", a, b, a.shape, od), np.minimum(a, b))
    np.testing.assert_array_equal(oracle.elementwise_binary("MAXIMUM", a, b, a.shape, od), np.maximum(a, b))
    # ADD / SUB: the exact sum rounded once to the storage type
    np.testing.assert_array_equal(oracle.elementwise_binary("ADD", a, b, a.shape, od),
                                  (a.astype(np.float64) + b.astype(np.float64)).astype(dt))
    np.testing.assert_array_equal(oracle.elementwise_binary("SUB", a, b, a.shape, od),
                                  (a.astype(np.float64) - b.astype(np.float64)).astype(dt))


def test_min_max_nan_modes(abi, oracle):
    """applyMin / applyMax (elementwise_binary.comp:105-144): propagate returns the NaN, ignore the other operand"""
    a = np.array([np.nan, 1.0, np.nan, 2.0], np.float32)
    b = np.array([3.0, np.nan, np.nan, 5.0], np.float32)
    for name, pick in (("MINIMUM", min), ("MAXIMUM", max)):
        p = oracle.elementwise_binary(name, a, b, a.shape, abi.F32, abi.NAN_PROPAGATE)
        assert np.isnan(p[0]) and np.isnan(p[1]) and np.isnan(p[2]) and p[3] == pick(2.0, 5.0)
        i = oracle.elementwise_binary(name, a, b, a.shape, abi.F32, abi.NAN_IGNORE)
        assert i[0] == 3.0 and i[1] == 1.0 and np.isnan(i[2]) and i[3] == pick(2.0, 5.0)


def test_pow_sign_rules(abi, oracle):
    """power() (elementwise_binary.comp:69-89): a negative base with an even exponent gives pow(-base, e), with an odd
    integer exponent -pow(-base, e), with any other exponent NaN; a non-negative base goes to pow() directly"""
    base = np.array([2.0, 2.0, -2.0, -2.0, -2.0, -8.0, 0.0, 9.0, -3.0, 1.5], np.float32)
    expo = np.array([3.0, -1.0, 2.0, 3.0, 0.5, 1.0 / 3.0, 0.0, 0.5, 4.0, 2.5], np.float32)
    got = oracle.elementwise_binary("POW", base, expo, base.shape, abi.F32)
    exp = [8.0, 0.5, 4.0, -8.0, None, None, 1.0, 3.0, 81.0, f32(1.5 ** 2.5)]
    for g, e in zip(got.tolist(), exp):
        assert (math.isnan(g) if e is None else g == e), (got.tolist(), exp)
    b = np.abs(RNG.standard_normal(200).astype(np.float32)) + 0.1
    e = RNG.standard_normal(200).astype(np.float32) * 3
    np.testing.assert_array_equal(oracle.elementwise_binary("POW", b, e, b.shape, abi.F32),
                                  np.power(b.astype(np.float64), e.astype(np.float64)).astype(np.float32))


# ---------------------------------------------------------------- REDUCE
def test_reduce_product_int_wraps_like_python_ints(abi, oracle):
    x = RNG.integers(-9, 9, (3, 12, 2), endpoint=True).astype(np.int32)
    x[x == 0] = 3
    out = oracle.reduce("PRODUCT", x, 1)
    for n in range(3):
        for c in range(2):
            p = 1
            for v in x[n, :, c].tolist():
                p = wrap(p * v, 32)  # the running product is held in the storage type (reduce.comp:24-70)
            assert out[n, 0, c] == p
    big = np.array([[65536, 65536, 3]], np.int32)  # 2^32 wraps to 0 and stays 0
    assert oracle.reduce("PRODUCT", big, 1).item() == 0


def test_reduce_product_float_is_sequential_in_the_storage_type(abi, oracle):
    x = (1.0 + RNG.standard_normal((5, 40)) * 0.05).astype(np.float16)
    out = oracle.reduce("PRODUCT", x, 1)
    for r in range(5):
        p = np.float16(1.0)
        for v in x[r]:
            p = np.float16(np.float64(p) * np.float64(v))  # exact product of two binary16 values, rounded once
        assert out[r, 0] == p
    f = (1.0 + RNG.standard_normal((4, 30)) * 0.1).astype(np.float32)
    o32 = oracle.reduce("PRODUCT", f, 1)
    for r in range(4):
        p = np.float32(1.0)
        for v in f[r]:
            p = np.float32(np.float64(p) * np.float64(v))
        assert o32[r, 0] == p


def test_reduce_min_max_float_and_nan_modes(abi, oracle):
    f = RNG.standard_normal((6, 37)).astype(np.float16)
    np.testing.assert_array_equal(oracle.reduce("MAX", f, 1), f.max(axis=1, keepdims=True))
    np.testing.assert_array_equal(oracle.reduce("MIN", f, 1), f.min(axis=1, keepdims=True))
    g = np.array([[1.0, np.nan, 3.0], [np.nan, np.nan, np.nan]], np.float32)
    p = oracle.reduce("MAX", g, 1, abi.NAN_PROPAGATE)
    assert np.isnan(p[0, 0]) and np.isnan(p[1, 0])
    i = oracle.reduce("MAX", g, 1, abi.NAN_IGNORE)
    assert i[0, 0] == 3.0 and np.isnan(i[1, 0])
    assert oracle.reduce("MIN", g, 1, abi.NAN_IGNORE)[0, 0] == 1.0
    # an empty fold returns the initial value: the lowest finite value of the type (compute_graph_op.cpp:2819-2859)
    e = np.zeros((2, 0), np.float16)
    assert oracle.reduce("MAX", e, 1).tolist() == [[-65504.0], [-65504.0]]
    assert oracle.reduce("SUM", e, 1).tolist() == [[0.0], [0.0]]
