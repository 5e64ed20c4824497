"""mlel_hip_conv2d_rescale_clamp_static, the entry point that allocates nothing: its output against
mlel_hip_conv2d_rescale_clamp's (and the oracle's), bit for bit, on calls in a row that use the static device array
in both ways -- the partial tiles and counters of a split-K contraction, then, with a smaller input, the int32
accumulator of the operator sequence -- and the refusal of a size beyond the array."""
import ctypes as C

import numpy as np
import pytest

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


def both(run, x, w, b, shape, attr, mult, shift, rattr, clamp, x_strides=None):
    """the same operands through the allocating and the static entry point"""
    outs = []
    for name in ("conv2d_rescale_clamp", "conv2d_rescale_clamp_static"):
        tx, tw, tb = run.put(x, strides=x_strides), run.put(w), run.put(b)
        to = run.new(abi.I8, shape)
        e = run._epi(mult, shift, rattr, clamp)
        run.dev.op(name, to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr), C.byref(e))
        outs.append(to.download())
        run.done()
    return outs


def test_static_entry_point_equals_the_allocating_one(run, oracle):
    rng = np.random.default_rng(77)
    rattr = abi.rescale_attr(0, 3, True, True, True)
    # call 1: 1x1 convolution, 98 positions x 160 channels over K = 2560: a handful of tiles, forty K steps -> K is
    # split and the partial tiles and counters live in the static array
    x = ri(rng, -128, 127, (2, 7, 7, 2560), np.int8)
    w = ri(rng, -128, 127, (160, 1, 1, 2560), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (160,), np.int32)
    mult, shift = ri(rng, 2 ** 30, 2 ** 31 - 1, (160,), np.int32), ri(rng, 30, 38, (160,), np.int8)
    attr = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), -1, 2)
    shape = (2, 7, 7, 160)
    ref, got = both(run, x, w, b, shape, attr, mult, shift, rattr, (-90, 100))
    exp = oracle.clamp(oracle.rescale(oracle.conv2d(x, w, b, shape, abi.I32, attr), mult, shift, abi.I8, rattr), -90, 100)
    np.testing.assert_array_equal(ref, exp)
    np.testing.assert_array_equal(got, ref)
    assert run.dev.lib.mlel_hip_static_scratch_last_use(run.dev.ctx) == 1  # K was split through the static array
    # call 2, smaller: a 3x3 convolution whose input pixels are 32 bytes apart while holding 24 channels, which no
    # one-pass kernel takes -> the operator sequence with its int32 accumulator staged in the same array
    x2 = ri(rng, -128, 127, (1, 6, 5, 24), np.int8)
    w2 = ri(rng, -128, 127, (20, 3, 3, 24), np.int8)
    b2 = ri(rng, -2 ** 15, 2 ** 15, (20,), np.int32)
    m2, s2 = ri(rng, 2 ** 30, 2 ** 31 - 1, (20,), np.int32), ri(rng, 30, 38, (20,), np.int8)
    attr2 = abi.conv2d_attr((1, 1, 1, 1), (1, 1), (1, 1), 4, 0)
    shape2 = (1, 6, 5, 20)
    strides2 = (6 * 5 * 64, 5 * 64, 64, 2)  # element stride 2: a strided view
    ref2, got2 = both(run, x2, w2, b2, shape2, attr2, m2, s2, rattr, None, x_strides=strides2)
    exp2 = oracle.rescale(oracle.conv2d(x2, w2, b2, shape2, abi.I32, attr2), m2, s2, abi.I8, rattr)
    np.testing.assert_array_equal(ref2, exp2)
    np.testing.assert_array_equal(got2, ref2)
    assert run.dev.lib.mlel_hip_static_scratch_last_use(run.dev.ctx) == 2  # the accumulator was staged there
    # call 3: the split-K shape again after the array held an accumulator, on a smaller batch
    ref3, got3 = both(run, x[:1], w, b, (1, 7, 7, 160), attr, mult, shift, rattr, (-90, 100))
    np.testing.assert_array_equal(ref3, exp[:1])
    np.testing.assert_array_equal(got3, ref3)


def test_static_entry_point_runs_under_capture_and_replays(run, oracle):
    """Both uses of the static array recorded into one HIP graph (thread-local capture mode refuses hipMalloc and
    hipFree on the capturing thread, so an allocation would fail the call) and replayed three times over changing
    inputs, with uploads, downloads and synchronisations between the replays: every replay gives the oracle's bits."""
    dev, lib = run.dev, run.dev.lib
    rng = np.random.default_rng(78)
    rattr = abi.rescale_attr(0, 3, True, True, True)
    w = ri(rng, -128, 127, (160, 1, 1, 2560), np.int8)
    b = ri(rng, -2 ** 15, 2 ** 15, (160,), np.int32)
    mult, shift = ri(rng, 2 ** 30, 2 ** 31 - 1, (160,), np.int32), ri(rng, 30, 38, (160,), np.int8)
    attr = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), -1, 2)
    w2 = ri(rng, -128, 127, (20, 3, 3, 24), np.int8)
    b2 = ri(rng, -2 ** 15, 2 ** 15, (20,), np.int32)
    m2, s2 = ri(rng, 2 ** 30, 2 ** 31 - 1, (20,), np.int32), ri(rng, 30, 38, (20,), np.int8)
    attr2 = abi.conv2d_attr((1, 1, 1, 1), (1, 1), (1, 1), 4, 0)
    stream = dev.new_stream()
    null_stream, dev.stream = dev.stream, stream
    try:
        tx = run.put(np.zeros((2, 7, 7, 2560), np.int8))
        tw, tb = run.put(w), run.put(b)
        to = run.new(abi.I8, (2, 7, 7, 160))
        e = run._epi(mult, shift, rattr, (-90, 100))
        tx2 = run.put(np.zeros((1, 6, 5, 24), np.int8), strides=(6 * 5 * 64, 5 * 64, 64, 2))
        tw2, tb2 = run.put(w2), run.put(b2)
        to2 = run.new(abi.I8, (1, 6, 5, 20))
        e2 = run._epi(m2, s2, rattr, None)
        dev._check(lib.mlel_hip_capture_begin(dev.ctx, stream))
        try:
            dev.op("conv2d_rescale_clamp_static", to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr), C.byref(e))
            first_use = lib.mlel_hip_static_scratch_last_use(dev.ctx)
            dev.op("conv2d_rescale_clamp_static", to2.ref, tx2.ref, tw2.ref, tb2.ref, C.byref(attr2), C.byref(e2))
            second_use = lib.mlel_hip_static_scratch_last_use(dev.ctx)
        finally:
            exe = C.c_void_p()
            dev._check(lib.mlel_hip_capture_end(dev.ctx, stream, C.byref(exe)))
        assert (first_use, second_use) == (1, 2)
        for rep in range(3):
            x = ri(rng, -128, 127, (2, 7, 7, 2560), np.int8)
            x2 = ri(rng, -128, 127, (1, 6, 5, 24), np.int8)
            tx.upload(x)
            tx2.upload(x2)
            dev._check(lib.mlel_hip_graph_launch(dev.ctx, exe, stream))
            got, got2 = to.download(), to2.download()
            exp = oracle.clamp(oracle.rescale(oracle.conv2d(x, w, b, (2, 7, 7, 160), abi.I32, attr), mult, shift, abi.I8,
                                              rattr), -90, 100)
            exp2 = oracle.rescale(oracle.conv2d(x2, w2, b2, (1, 6, 5, 20), abi.I32, attr2), m2, s2, abi.I8, rattr)
            np.testing.assert_array_equal(got, exp, err_msg=f"replay {rep}, split-K call")
            np.testing.assert_array_equal(got2, exp2, err_msg=f"replay {rep}, operator-sequence call")
        dev._check(lib.mlel_hip_graph_destroy(dev.ctx, exe))
    finally:
        dev.stream = null_stream
        run.done()
        dev._check(lib.mlel_hip_stream_destroy(dev.ctx, stream))


def test_static_entry_point_refuses_an_accumulator_beyond_the_array(run):
    """operator-sequence route with more than 2 097 152 outputs: MLEL_ERR_LIMIT, nothing launched"""
    x = np.zeros((1, 1100, 1000, 1), np.int8)
    w = np.zeros((2, 1, 1, 1), np.int8)
    b = np.zeros(2, np.int32)
    mult, shift = np.full(2, 2 ** 30, np.int32), np.full(2, 30, np.int8)
    attr = abi.conv2d_attr((0, 0, 0, 0), (1, 1), (1, 1), 0, 0)
    tx = run.put(x, strides=(1100 * 1000 * 2, 1000 * 2, 2, 2))  # element stride 2: no one-pass kernel
    tw, tb = run.put(w), run.put(b)
    to = run.new(abi.I8, (1, 1100, 1000, 2))
    e = run._epi(mult, shift, abi.rescale_attr(0, 0, True, True, True), None)
    with pytest.raises(hb.MlelError) as err:
        run.dev.op("conv2d_rescale_clamp_static", to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr), C.byref(e))
    run.done()
    assert err.value.code == abi.ERR_LIMIT and "exceeds the static scratch" in str(err.value)
