"""The TOSA operators outside the benchmark graphs (ARGMAX, ARITHMETIC_RIGHT_SHIFT, CONV3D, TRANSPOSE_CONV2D, FFT2D,
RFFT2D, GATHER, SCATTER, RESIZE, REVERSE, TILE, SELECT).

CPU part: the oracle's restatement of each shader is pinned against independent numpy / brute-force statements of
the operator (the reference's tests hold no values for these operators: FFT2D runs without an assertion, CONV3D and
ARITHMETIC_RIGHT_SHIFT are only created).  FFT2D / RFFT2D depend on the driver's sine and cosine in the reference and
are compared with numpy's FFT to a tolerance: parity unpinned beyond the mathematics of the transform.
GPU part: every operator through the C ABI against the oracle on the same seeded inputs, bit for bit for integers.
"""
import ctypes as C

import numpy as np
import pytest

from hip_util import Runner, abi, gpu_available, hb


def ri(rng, lo, hi, shape, dt):
    return rng.integers(lo, hi, size=shape, endpoint=True).astype(dt)


# ------------------------------------------------------------------------------------------------ numpy statements
def np_conv3d(x, w, b, pad, stride, dil, zi, zw):
    n, d, h, wd, ic = x.shape
    oc, kd, kh, kw, _ = w.shape
    od = (d + pad[0] + pad[1] - (kd - 1) * dil[0] - 1) // stride[0] + 1
    oh = (h + pad[2] + pad[3] - (kh - 1) * dil[1] - 1) // stride[1] + 1
    ow = (wd + pad[4] + pad[5] - (kw - 1) * dil[2] - 1) // stride[2] + 1
    xp = np.zeros((n, d + pad[0] + pad[1], h + pad[2] + pad[3], wd + pad[4] + pad[5], ic), np.int64)
    xp[:, pad[0]:pad[0] + d, pad[2]:pad[2] + h, pad[4]:pad[4] + wd] = x.astype(np.int64) - zi  # padding adds nothing
    out = np.zeros((n, od, oh, ow, oc), np.int64)
    for a in range(kd):
        for e in range(kh):
            for f in range(kw):
                patch = xp[:, a * dil[0]:a * dil[0] + (od - 1) * stride[0] + 1:stride[0],
                           e * dil[1]:e * dil[1] + (oh - 1) * stride[1] + 1:stride[1],
                           f * dil[2]:f * dil[2] + (ow - 1) * stride[2] + 1:stride[2]]
                out += np.einsum("ndhwi,oi->ndhwo", patch, w[:, a, e, f].astype(np.int64) - zw)
    return out + b.astype(np.int64)


def np_transpose_conv2d(x, w, b, out_pad, stride, out_hw, zi, zw):
    """Scatter form of the TOSA definition: input (iy, ix) adds x * w[ky, kx] at oy = iy * sy + out_pad_top + ky."""
    n, h, wd, ic = x.shape
    oc, kh, kw, _ = w.shape
    out = np.zeros((n,) + tuple(out_hw) + (oc,), np.int64) + b.astype(np.int64)
    xs, ws = x.astype(np.int64) - zi, w.astype(np.int64) - zw
    for iy in range(h):
        for ix in range(wd):
            for ky in range(kh):
                for kx in range(kw):
                    oy, ox = iy * stride[0] + out_pad[0] + ky, ix * stride[1] + out_pad[2] + kx
                    if 0 <= oy < out_hw[0] and 0 <= ox < out_hw[1]:
                        out[:, oy, ox, :] += xs[:, iy, ix, :] @ ws[:, ky, kx, :].T
    return out


def np_resize_int(x, out_hw, scale, offset, mode, acc_dtype):
    """TOSA RESIZE for integer data, one output element at a time."""
    n, h, w, c = x.shape
    yn, yd, xn, xd = scale
    out = np.zeros((n, out_hw[0], out_hw[1], c), acc_dtype)
    for oy in range(out_hw[0]):
        for ox in range(out_hw[1]):
            y, xx = oy * yd + offset[0], ox * xd + offset[1]
            iy, ix = y // yn, xx // xn  # floor division
            ry, rx = y - iy * yn, xx - ix * xn
            iy0, iy1 = max(iy, 0), min(iy + 1, h - 1)
            ix0, ix1 = max(ix, 0), min(ix + 1, w - 1)
            if mode == 2:  # bilinear
                v = x.astype(np.int64)
                out[:, oy, ox, :] = (v[:, iy0, ix0] * (yn - ry) * (xn - rx) + v[:, iy0, ix1] * (yn - ry) * rx +
                                     v[:, iy1, ix0] * ry * (xn - rx) + v[:, iy1, ix1] * ry * rx)
            else:
                out[:, oy, ox, :] = x[:, iy1 if 2 * ry >= yn else iy0, ix1 if 2 * rx >= xn else ix0]
    return out


# ------------------------------------------------------------------------------------------------------- CPU: oracle
def test_oracle_data_movement_vs_numpy(oracle):
    rng = np.random.default_rng(0)
    x = ri(rng, -128, 127, (3, 5, 4, 6), np.int8)
    for axis in range(4):
        np.testing.assert_array_equal(oracle.argmax(x, axis), np.argmax(x, axis=axis))
        np.testing.assert_array_equal(oracle.reverse(x, axis), np.flip(x, axis))
    np.testing.assert_array_equal(oracle.tile(x, (6, 5, 8, 6)), np.tile(x, (2, 1, 2, 1)))
    cond = rng.integers(0, 2, (3, 1, 4, 1)).astype(np.bool_)
    y = ri(rng, -128, 127, (1, 5, 4, 6), np.int8)
    np.testing.assert_array_equal(oracle.select(cond, x, y, x.shape), np.where(cond, x, y))
    v = ri(rng, -1000, 1000, (2, 7, 3), np.int32)
    idx = ri(rng, 0, 6, (2, 4), np.int32)
    np.testing.assert_array_equal(oracle.gather(v, idx), np.take_along_axis(v, idx[:, :, None].astype(np.int64), 1))
    inp = ri(rng, -1000, 1000, (2, 4, 3), np.int32)
    idx2 = np.array([[1, 3, 5, 0], [6, 2, 4, 1]], np.int32)
    exp = v.copy()
    for n in range(2):
        for w in range(4):
            exp[n, idx2[n, w]] = inp[n, w]
    np.testing.assert_array_equal(oracle.scatter(v, idx2, inp), exp)
    # ties: the first maximum wins; a row of the lowest value gives index 0
    t = np.array([[5, 9, 9, 1], [-128, -128, -128, -128]], np.int8)
    np.testing.assert_array_equal(oracle.argmax(t, 1), [1, 0])
    f = np.array([[1.0, np.nan, 7.0], [np.nan, 2.0, 3.0], [-np.inf, -np.inf, -np.inf]], np.float32)
    np.testing.assert_array_equal(oracle.argmax(f, 1, abi.NAN_PROPAGATE), [1, 0, 0])
    np.testing.assert_array_equal(oracle.argmax(f, 1, abi.NAN_IGNORE), [2, 2, 0])


def test_oracle_arithmetic_right_shift_vs_integers(oracle):
    rng = np.random.default_rng(1)
    for dt, bits in ((np.int8, 8), (np.int16, 16), (np.int32, 32)):
        a = ri(rng, -2 ** (bits - 1), 2 ** (bits - 1) - 1, (4, 33), dt)
        s = ri(rng, 0, bits - 1, (1, 33), dt)
        np.testing.assert_array_equal(oracle.arithmetic_right_shift(a, s, a.shape), a >> s)
        # rounding: add half of the last dropped bit, in exact integers
        big = a.astype(object)
        exp = np.array([[(int(v) + (1 << (int(k) - 1)) >> int(k)) if k > 0 else int(v) for v, k in zip(row, s[0])]
                        for row in big], dtype=np.int64)
        np.testing.assert_array_equal(oracle.arithmetic_right_shift(a, s, a.shape, True), exp.astype(dt))


def test_oracle_conv3d_and_transpose_conv2d_vs_numpy(oracle):
    rng = np.random.default_rng(2)
    x = ri(rng, -128, 127, (2, 5, 6, 7, 3), np.int8)
    w = ri(rng, -128, 127, (4, 2, 3, 2, 3), np.int8)
    b = ri(rng, -1000, 1000, (4,), np.int32)
    pad, stride, dil = (1, 0, 1, 1, 0, 2), (2, 1, 2), (1, 2, 1)
    exp = np_conv3d(x, w, b, pad, stride, dil, -3, 2)
    attr = abi.conv3d_attr(pad, stride, dil, -3, 2)
    np.testing.assert_array_equal(oracle.conv3d(x, w, b, exp.shape, abi.I32, attr), exp.astype(np.int32))
    x2 = ri(rng, -128, 127, (2, 4, 5, 3), np.int8)
    w2 = ri(rng, -128, 127, (6, 3, 2, 3), np.int8)
    b2 = ri(rng, -1000, 1000, (6,), np.int32)
    for out_pad, stride2 in (((0, 0, 0, 0), (2, 3)), ((1, 0, 2, 1), (1, 2)), ((-1, 0, -1, 0), (2, 2))):
        oh = (4 - 1) * stride2[0] + out_pad[0] + out_pad[1] + 3
        ow = (5 - 1) * stride2[1] + out_pad[2] + out_pad[3] + 2
        exp2 = np_transpose_conv2d(x2, w2, b2, out_pad, stride2, (oh, ow), 5, -1)
        attr2 = abi.tconv2d_attr(out_pad, stride2, 5, -1)
        got = oracle.transpose_conv2d(x2, w2, b2, exp2.shape, abi.I32, attr2)
        np.testing.assert_array_equal(got, exp2.astype(np.int32))


def test_oracle_resize_vs_numpy(oracle):
    rng = np.random.default_rng(3)
    x = ri(rng, -128, 127, (2, 5, 7, 3), np.int8)
    for scale, offset, out_hw in (((4, 2, 4, 2), (0, 0), (9, 13)), ((3, 1, 5, 2), (-1, 2), (13, 16)),
                                  ((2, 3, 1, 1), (1, 0), (3, 7))):
        attr = abi.resize_attr(scale, offset, (0, 0), 2)
        exp = np_resize_int(x, out_hw, scale, offset, 2, np.int64)
        np.testing.assert_array_equal(oracle.resize(x, exp.shape, abi.I32, attr), exp.astype(np.int32))
        attr = abi.resize_attr(scale, offset, (0, 0), 1)
        exp = np_resize_int(x, out_hw, scale, offset, 1, np.int8)
        np.testing.assert_array_equal(oracle.resize(x, exp.shape, abi.I8, attr), exp)
    # float bilinear at scale 2: the midpoints are means of the neighbours, the grid points are copies
    f = rng.standard_normal((1, 4, 4, 2)).astype(np.float32)
    out = oracle.resize(f, (1, 7, 7, 2), abi.F32, abi.resize_attr((2, 1, 2, 1), (0, 0), (0, 0), 2))
    np.testing.assert_array_equal(out[:, ::2, ::2], f)
    np.testing.assert_allclose(out[:, 1::2, ::2], (f[:, :-1] + f[:, 1:]) / 2, rtol=1e-6, atol=1e-6)


def test_oracle_fft_vs_numpy(oracle):
    rng = np.random.default_rng(4)
    re, im = rng.standard_normal((2, 8, 16)).astype(np.float32), rng.standard_normal((2, 8, 16)).astype(np.float32)
    fr, fi = oracle.fft2d(re, im)
    ref = np.fft.fft2(re.astype(np.float64) + 1j * im)
    assert np.abs(fr - ref.real).max() <= 5e-4 and np.abs(fi - ref.imag).max() <= 5e-4  # float angles, as the shader
    fr, fi = oracle.fft2d(re, im, True)
    ref = np.fft.ifft2(re.astype(np.float64) + 1j * im) * (8 * 16)  # the inverse is not scaled
    assert np.abs(fr - ref.real).max() <= 5e-4 and np.abs(fi - ref.imag).max() <= 5e-4
    rr, rimag = oracle.rfft2d(re)
    ref = np.fft.rfft2(re.astype(np.float64))
    assert np.abs(rr - ref.real).max() <= 1e-5 and np.abs(rimag - ref.imag).max() <= 1e-5
    assert rimag[0, 0, 0] == 0 and rimag[0, 4, 8] == 0 and rimag[1, 0, 8] == 0  # purely real bins are exactly zero


# ------------------------------------------------------------------------------------------------------------- GPU
@pytest.fixture(scope="module")
def run():
    if not gpu_available():
        pytest.skip("no GPU visible")
    dev = hb.Device(0)
    yield Runner(dev)
    dev.close()


@pytest.mark.gpu
def test_data_movement_ops_vs_oracle(run, oracle):
    rng = np.random.default_rng(10)
    for dt in (np.int8, np.int16, np.int32, np.float16, np.float32):
        x = (rng.standard_normal((3, 5, 9, 6)) * 50).astype(dt)
        for axis in range(4):
            np.testing.assert_array_equal(run.reverse(x, axis), oracle.reverse(x, axis))
        np.testing.assert_array_equal(run.tile(x, (6, 5, 27, 6)), oracle.tile(x, (6, 5, 27, 6)))
        cond = rng.integers(0, 2, (3, 1, 9, 1)).astype(np.bool_)
        y = (rng.standard_normal((1, 5, 9, 6)) * 50).astype(dt)
        np.testing.assert_array_equal(run.select(cond, x, y, x.shape), oracle.select(cond, x, y, x.shape))
        v = (rng.standard_normal((4, 37, 11)) * 50).astype(dt)
        idx = ri(rng, 0, 36, (4, 20), np.int32)
        np.testing.assert_array_equal(run.gather(v, idx), oracle.gather(v, idx))
        inp = (rng.standard_normal((4, 20, 11)) * 50).astype(dt)
        idx_unique = np.stack([rng.permutation(37)[:20] for _ in range(4)]).astype(np.int32)
        np.testing.assert_array_equal(run.scatter(v, idx_unique, inp), oracle.scatter(v, idx_unique, inp))
        np.testing.assert_array_equal(run.scatter(v, idx, inp), oracle.scatter(v, idx, inp))  # repeated rows


@pytest.mark.gpu
def test_data_movement_in_pieces_vs_oracle(run, oracle):
    """SLICE, CONCAT, PAD, TILE, REVERSE and GATHER on packed tensors go through the kernel that moves whole pieces:
    shapes whose runs are multiples of 16, 8, 4, 2 and 1 bytes, operators acting on the innermost dimension, padding
    constants of every kind of type, indices outside the source, ranks from 1 to 6 (six non-trivial outer dimensions
    fall back to the element-wise kernel), and -- for SLICE and CONCAT -- ranges that leave a tensor (the
    out-of-bounds rules, also element-wise).  Bit for bit the oracle's (= the shaders') results."""
    rng = np.random.default_rng(21)

    def values(shape, dt):
        if np.issubdtype(dt, np.floating):
            return (rng.standard_normal(shape) * 40).astype(dt)
        info = np.iinfo(dt)
        return rng.integers(max(info.min, -2 ** 31), min(info.max, 2 ** 31 - 1), shape, endpoint=True).astype(dt)

    for dt, c in ((np.int8, 144), (np.int8, 24), (np.int8, 6), (np.int8, 5), (np.int16, 24), (np.int32, 5),
                  (np.float16, 7), (np.float32, 64), (np.int64, 3)):
        x = values((3, 10, 12, c), dt)
        # SLICE: spatial crop (runs of whole pixels), crop of the channels (unaligned start), nothing cropped
        for start, size in (((0, 2, 3, 0), (3, 7, 8, c)), ((1, 0, 0, 1), (2, 10, 12, c - 1)), ((0, 0, 0, 0), x.shape),
                            ((2, 9, 11, c - 1), (1, 1, 1, 1))):
            np.testing.assert_array_equal(run.slice_(x, start, size), oracle.slice_(x, start, size), err_msg=str((dt, c, start)))
        # a range that leaves the input: zeros, by the out-of-bounds rule
        np.testing.assert_array_equal(run.slice_(x, (1, 5, 0, 0), (3, 7, 12, c)), oracle.slice_(x, (1, 5, 0, 0), (3, 7, 12, c)))
        # CONCAT along every axis
        for axis in range(4):
            parts = [values(tuple(d if i != axis else k for i, d in enumerate(x.shape)), dt) for k in (3, 1, 5)]
            np.testing.assert_array_equal(run.concat(parts, axis), oracle.concat(parts, axis), err_msg=str((dt, c, axis)))
        # PAD: spatial, channels, everything, nothing
        const = dict(pad_const=-7.5, pad_const_int=-123456)
        for pads in (((0, 0), (1, 2), (3, 0), (0, 0)), ((0, 0), (0, 0), (0, 0), (2, 1)), ((1, 1), (1, 1), (1, 1), (1, 1)),
                     ((0, 0), (0, 0), (0, 0), (0, 0))):
            shape = tuple(d + a + b for d, (a, b) in zip(x.shape, pads))
            np.testing.assert_array_equal(run.pad(x, pads, shape, **const), oracle.pad(x, pads, shape, **const),
                                          err_msg=str((dt, c, pads)))
        # TILE: outer dimensions, the innermost one, a broadcast from extent 1
        small = values((2, 1, 4, c), dt)
        for shape in ((4, 3, 4, c), (2, 1, 12, 2 * c), (2, 5, 4, c)):
            np.testing.assert_array_equal(run.tile(small, shape), oracle.tile(small, shape), err_msg=str((dt, c, shape)))
        for axis in range(4):
            np.testing.assert_array_equal(run.reverse(x, axis), oracle.reverse(x, axis), err_msg=str((dt, c, axis)))
        # GATHER: some rows outside the source read as zeros; one batch, and several
        for n in (1, 3):
            v = values((n, 29, c), dt)
            idx = rng.integers(0, 28, (n, 17), endpoint=True).astype(np.int32)
            idx[0, 3], idx[-1, 5] = 29, -1
            np.testing.assert_array_equal(run.gather(v, idx), oracle.gather(v, idx), err_msg=str((dt, c, n)))
    # ranks 1, 2 and 6; six outer dimensions that all change stay with the element-wise kernel
    v1 = values((77,), np.int8)
    np.testing.assert_array_equal(run.slice_(v1, (5,), (60,)), oracle.slice_(v1, (5,), (60,)))
    np.testing.assert_array_equal(run.reverse(v1, 0), oracle.reverse(v1, 0))
    v2 = values((9, 32), np.int16)
    np.testing.assert_array_equal(run.tile(v2, (27, 32)), oracle.tile(v2, (27, 32)))
    np.testing.assert_array_equal(run.pad(v2, ((2, 1), (0, 0)), (12, 32)), oracle.pad(v2, ((2, 1), (0, 0)), (12, 32)))
    v6 = values((2, 3, 2, 3, 4, 16), np.int8)
    np.testing.assert_array_equal(run.slice_(v6, (1, 1, 0, 1, 2, 0), (1, 2, 2, 2, 2, 16)),
                                  oracle.slice_(v6, (1, 1, 0, 1, 2, 0), (1, 2, 2, 2, 2, 16)))
    np.testing.assert_array_equal(run.tile(v6, (4, 6, 4, 6, 8, 32)), oracle.tile(v6, (4, 6, 4, 6, 8, 32)))
    for axis in range(6):
        np.testing.assert_array_equal(run.reverse(v6, axis), oracle.reverse(v6, axis))
    # CONCAT into an output with other data around the part, and a part that does not fit (its overhang is dropped)
    base = values((2, 6, 8, 16), np.int8)
    part = values((2, 3, 8, 16), np.int8)
    want = base.copy()
    want[:, 2:5] = part
    np.testing.assert_array_equal(run.concat_at(base, part, 1, 2), want)
    want = base.copy()
    want[:, 4:6] = part[:, :2]
    np.testing.assert_array_equal(run.concat_at(base, part, 1, 4), want)


@pytest.mark.gpu
def test_argmax_and_arithmetic_right_shift_vs_oracle(run, oracle):
    rng = np.random.default_rng(11)
    for dt in (np.int8, np.int16, np.int32):
        x = ri(rng, -100, 100, (4, 33, 5, 7), dt)
        for axis in range(4):
            np.testing.assert_array_equal(run.argmax(x, axis), oracle.argmax(x, axis))
        bits = 8 * np.dtype(dt).itemsize
        a = ri(rng, -2 ** (bits - 1), 2 ** (bits - 1) - 1, (6, 65), dt)
        s = ri(rng, 0, bits - 1, (1, 65), dt)
        for round_ in (False, True):
            np.testing.assert_array_equal(run.arithmetic_right_shift(a, s, a.shape, round_),
                                          oracle.arithmetic_right_shift(a, s, a.shape, round_))
    for dt in (np.float16, np.float32):
        f = rng.standard_normal((5, 40)).astype(dt)
        f[1, 7] = np.nan
        f[3, :] = -np.inf
        for mode in (abi.NAN_PROPAGATE, abi.NAN_IGNORE):
            np.testing.assert_array_equal(run.argmax(f, 1, mode), oracle.argmax(f, 1, mode))


@pytest.mark.gpu
def test_conv3d_and_transpose_conv2d_vs_oracle(run, oracle):
    rng = np.random.default_rng(12)
    x = ri(rng, -128, 127, (2, 6, 9, 8, 5), np.int8)
    w = ri(rng, -128, 127, (7, 3, 3, 2, 5), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (7,), np.int32)
    for pad, stride, dil in (((1, 1, 1, 1, 0, 1), (1, 1, 1), (1, 1, 1)), ((2, 0, 0, 2, 1, 1), (2, 3, 1), (2, 1, 2))):
        od = (6 + pad[0] + pad[1] - 2 * dil[0] - 1) // stride[0] + 1
        oh = (9 + pad[2] + pad[3] - 2 * dil[1] - 1) // stride[1] + 1
        ow = (8 + pad[4] + pad[5] - 1 * dil[2] - 1) // stride[2] + 1
        attr = abi.conv3d_attr(pad, stride, dil, -7, 4)
        shape = (2, od, oh, ow, 7)
        np.testing.assert_array_equal(run.conv3d(x, w, b, shape, abi.I32, attr), oracle.conv3d(x, w, b, shape, abi.I32, attr))
    x16 = ri(rng, -3000, 3000, (1, 3, 4, 4, 2), np.int16)
    b64 = ri(rng, -2 ** 40, 2 ** 40, (7,), np.int64)
    w8 = ri(rng, -128, 127, (7, 2, 2, 2, 2), np.int8)
    attr = abi.conv3d_attr(acc_type=abi.ACC_I64)
    np.testing.assert_array_equal(run.conv3d(x16, w8, b64, (1, 2, 3, 3, 7), abi.I64, attr),
                                  oracle.conv3d(x16, w8, b64, (1, 2, 3, 3, 7), abi.I64, attr))
    x2 = ri(rng, -128, 127, (2, 7, 6, 9), np.int8)
    w2 = ri(rng, -128, 127, (5, 3, 4, 9), np.int8)
    b2 = ri(rng, -2 ** 15, 2 ** 15, (5,), np.int32)
    for out_pad, stride2 in (((0, 0, 0, 0), (2, 2)), ((1, 2, 0, 1), (3, 1)), ((-1, -1, -2, 0), (2, 3))):
        oh = (7 - 1) * stride2[0] + out_pad[0] + out_pad[1] + 3
        ow = (6 - 1) * stride2[1] + out_pad[2] + out_pad[3] + 4
        attr2 = abi.tconv2d_attr(out_pad, stride2, 9, -2)
        shape = (2, oh, ow, 5)
        np.testing.assert_array_equal(run.transpose_conv2d(x2, w2, b2, shape, abi.I32, attr2),
                                      oracle.transpose_conv2d(x2, w2, b2, shape, abi.I32, attr2))
    # fp16 data with fp32 accumulation: max abs error <= 1e-2
    xf = rng.standard_normal((1, 5, 5, 8)).astype(np.float16)
    wf = (0.1 * rng.standard_normal((4, 3, 3, 8))).astype(np.float16)
    bf = rng.standard_normal((4,)).astype(np.float16)
    attrf = abi.tconv2d_attr((0, 0, 0, 0), (2, 2), acc_type=abi.ACC_F32)
    got = run.transpose_conv2d(xf, wf, bf, (1, 11, 11, 4), abi.F16, attrf).astype(np.float32)
    exp = oracle.transpose_conv2d(xf, wf, bf, (1, 11, 11, 4), abi.F16, attrf).astype(np.float32)
    assert np.abs(got - exp).max() <= 1e-2


@pytest.mark.gpu
def test_resize_vs_oracle(run, oracle):
    rng = np.random.default_rng(13)
    x8 = ri(rng, -128, 127, (2, 9, 11, 5), np.int8)
    x16 = ri(rng, -32768, 32767, (1, 6, 5, 3), np.int16)
    for scale, offset, out_hw in (((4, 2, 4, 2), (0, 0), (17, 21)), ((3, 1, 5, 2), (-1, 2), (25, 26)),
                                  ((2, 3, 1, 1), (1, 0), (6, 11)), ((16, 2, 16, 2), (-7, -7), (72, 88))):
        for mode, out8, out16 in ((1, abi.I8, abi.I16), (2, abi.I32, abi.I64)):
            attr = abi.resize_attr(scale, offset, (0, 0), mode)
            shape = (2,) + out_hw + (5,)
            np.testing.assert_array_equal(run.resize(x8, shape, out8, attr), oracle.resize(x8, shape, out8, attr))
            shape16 = (1, 7, 9, 3)
            np.testing.assert_array_equal(run.resize(x16, shape16, out16, attr), oracle.resize(x16, shape16, out16, attr))
    for dt, code, tol in ((np.float32, abi.F32, 1e-6), (np.float16, abi.F16, 1e-2)):
        f = rng.standard_normal((1, 8, 8, 4)).astype(dt)
        for mode in (1, 2):
            attr = abi.resize_attr((3, 1, 3, 1), (1, -1), (0, 0), mode)
            got = run.resize(f, (1, 20, 20, 4), code, attr).astype(np.float32)
            exp = oracle.resize(f, (1, 20, 20, 4), code, attr).astype(np.float32)
            assert np.abs(got - exp).max() <= tol


@pytest.mark.gpu
def test_fft_vs_oracle_and_numpy(run, oracle):
    """Tolerances: the device's sinf / cosf differ from the C library's in the last bits (as the Vulkan driver's do in
    the reference); sums of H * W terms of magnitude ~1."""
    rng = np.random.default_rng(14)
    re, im = rng.standard_normal((2, 16, 32)).astype(np.float32), rng.standard_normal((2, 16, 32)).astype(np.float32)
    for inverse in (False, True):
        gr, gi = run.fft2d(re, im, inverse)
        er, ei = oracle.fft2d(re, im, inverse)
        assert np.abs(gr - er).max() <= 1e-3 and np.abs(gi - ei).max() <= 1e-3
        ref = (np.fft.ifft2(re + 1j * im) * 512) if inverse else np.fft.fft2(re + 1j * im)
        assert np.abs(gr - ref.real).max() <= 2e-3 and np.abs(gi - ref.imag).max() <= 2e-3
    gr, gi = run.rfft2d(re)
    er, ei = oracle.rfft2d(re)
    assert np.abs(gr - er).max() <= 1e-4 and np.abs(gi - ei).max() <= 1e-4
    assert gi[0, 0, 0] == 0 and gi[0, 8, 16] == 0


@pytest.mark.gpu
def test_conv3d_through_conv2d_vs_oracle(run, oracle):
    """int8 CONV3D with an int32 result and a few million multiply-adds runs as one CONV2D on the matrix cores (the depth
    taps laid side by side along the channels of a temporary; a kernel one slice deep needs no temporary): 16-, 4- and
    1-byte pieces, depth padding / stride / dilation, both zero points, bias of one value."""
    rng = np.random.default_rng(77)
    cases = [  # x shape, w shape, pad (front, back, top, bottom, left, right), stride, dilation, zi, zw, bias length
        ((2, 6, 12, 12, 16), (32, 3, 3, 3, 16), (1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1), -7, 4, 32),
        ((2, 7, 20, 20, 5), (40, 2, 3, 3, 5), (0, 1, 1, 0, 2, 1), (2, 1, 2), (2, 1, 1), 3, 0, 40),
        ((1, 9, 16, 16, 4), (48, 3, 3, 3, 4), (3, 3, 0, 0, 1, 1), (1, 1, 1), (2, 2, 1), 0, -5, 1),
        ((3, 5, 14, 14, 32), (16, 2, 1, 1, 32), (0, 0, 0, 0, 0, 0), (1, 1, 1), (1, 1, 1), -128, 0, 16),
        ((2, 4, 9, 9, 8), (16, 1, 3, 3, 8), (0, 0, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1), 5, 2, 16),   # one slice deep
        ((1, 3, 6, 6, 8), (8, 3, 3, 3, 8), (1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1), 1, 1, 8),     # small: generic kernel
    ]
    for xs, ws, pad, stride, dil, zi, zw, bl in cases:
        x = ri(rng, -128, 127, xs, np.int8)
        w = ri(rng, -128, 127, ws, np.int8)
        b = ri(rng, -2 ** 20, 2 ** 20, (bl,), np.int32)
        od = (xs[1] + pad[0] + pad[1] - (ws[1] - 1) * dil[0] - 1) // stride[0] + 1
        oh = (xs[2] + pad[2] + pad[3] - (ws[2] - 1) * dil[1] - 1) // stride[1] + 1
        ow = (xs[3] + pad[4] + pad[5] - (ws[3] - 1) * dil[2] - 1) // stride[2] + 1
        shape = (xs[0], od, oh, ow, ws[0])
        attr = abi.conv3d_attr(pad, stride, dil, zi, zw)
        np.testing.assert_array_equal(run.conv3d(x, w, b, shape, abi.I32, attr), oracle.conv3d(x, w, b, shape, abi.I32, attr),
                                      err_msg=str((xs, ws, pad, stride, dil)))


@pytest.mark.gpu
def test_conv3d_on_a_capturing_stream(run, oracle):
    """CONV3D recorded into a HIP graph on a fresh stream (no staging memory yet and none can be allocated: the
    one-thread-per-output kernel is recorded) and again after an eager call has given the stream its staging memory
    (the CONV2D route is recorded); every replay over new inputs gives the oracle's bits."""
    dev, lib = run.dev, run.dev.lib
    rng = np.random.default_rng(79)
    xs, ws = (1, 5, 12, 12, 16), (32, 3, 3, 3, 16)
    w = ri(rng, -128, 127, ws, np.int8)
    b = ri(rng, -2 ** 20, 2 ** 20, (32,), np.int32)
    attr = abi.conv3d_attr((1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1), -4, 3)
    shape = (1, 5, 12, 12, 32)
    stream = dev.new_stream()
    null_stream, dev.stream = dev.stream, stream
    try:
        tx, tw, tb = run.put(np.zeros(xs, np.int8)), run.put(w), run.put(b)
        to = run.new(abi.I32, shape)
        for phase in ("no staging memory", "staging memory from an eager call"):
            if phase.startswith("staging"):
                dev.op("conv3d", to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr))
                dev.sync()
            dev._check(lib.mlel_hip_capture_begin(dev.ctx, stream))
            try:
                dev.op("conv3d", to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr))
            finally:
                exe = C.c_void_p()
                dev._check(lib.mlel_hip_capture_end(dev.ctx, stream, C.byref(exe)))
            for rep in range(2):
                x = ri(rng, -128, 127, xs, np.int8)
                tx.upload(x)
                dev._check(lib.mlel_hip_graph_launch(dev.ctx, exe, stream))
                np.testing.assert_array_equal(to.download(), oracle.conv3d(x, w, b, shape, abi.I32, attr),
                                              err_msg=f"{phase}, replay {rep}")
            dev._check(lib.mlel_hip_graph_destroy(dev.ctx, exe))
    finally:
        dev.stream = null_stream
        run.done()
        dev._check(lib.mlel_hip_stream_destroy(dev.ctx, stream))


@pytest.mark.gpu
def test_kat_conv3d_large_stride(run, kats):
    """The reference's CONV3D known-answer test (tests/vulkan.cpp:1211-1290) on the GPU."""
    from test_oracle_kats import conv3d_kat
    x, w, exp, a = conv3d_kat(kats["conv3d_large_stride"])
    out = run.conv3d(x, w, np.zeros(1, np.int32), exp.shape, abi.I32, abi.conv3d_attr(*a))
    np.testing.assert_array_equal(out, exp)
