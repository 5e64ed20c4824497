"""Neutral descriptions of the benchmark data graphs (BASELINE configs 2 and 3) and their construction on the
GraphPipeline.  A description is plain data: named tensors, numpy constants and a list of TOSA operators with the
operand order of the TOSA.001000.1 instruction set as the reference decodes it
(graph/graph_tosa_1_0_ext_inst.cpp:37-1032), so the same description can be executed operator by operator by
any backend (the tests run it through the CPU oracle, unfused, the way the reference executes it).
"""
import time

import numpy as np

from . import abi
from .graph_backend import Graph

# MobileNetV2 1.0: (expansion t, output channels c, repeats n, stride s)
MOBILENETV2_BLOCKS = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2),
                      (6, 320, 1, 1)]


class Spec:
    def __init__(self):
        self.tensors = {}   # name -> (dtype, shape): intermediates in session memory
        self.consts = {}    # name -> ndarray
        self.inputs = []    # (name, dtype, shape)
        self.outputs = []   # (name, dtype, shape)
        self.ops = []       # dicts: op, in, out, iattr, fattr, name
        self.macs = {"dense": 0, "depthwise": 0}
        # one entry per launch of the fused int8 graph, in execution order: kind ("conv" | "dw" | "avgpool" | "fc"),
        # shapes, MACs and the algorithmic bytes of the fused unit (every operand once + the output once)
        self.layers = []
        self._n = 0

    def fresh(self, prefix):
        self._n += 1
        return f"{prefix}{self._n}"

    def const(self, prefix, array):
        name = self.fresh(prefix)
        self.consts[name] = np.ascontiguousarray(array)
        return name

    def tensor(self, prefix, dtype, shape):
        name = self.fresh(prefix)
        self.tensors[name] = (dtype, tuple(int(d) for d in shape))
        return name

    def op(self, op, ins, outs, iattr=(), fattr=(), name=""):
        self.ops.append({"op": op, "in": list(ins), "out": list(outs), "iattr": [int(v) for v in iattr],
                         "fattr": [float(v) for v in fattr], "name": name or f"{op.lower()}_{len(self.ops)}"})

    def shape_of(self, name):
        if name in self.tensors:
            return self.tensors[name][1]
        if name in self.consts:
            return self.consts[name].shape
        for n, _, s in self.inputs + self.outputs:
            if n == name:
                return s
        raise KeyError(name)


class _Quant:
    """Draws RESCALE parameters: multiplier U[2^30, 2^31), shift U[30, 38] (BASELINE config 0).  With
    `spread=True` the shift grows with log2 of the contraction length so activations keep using the int8 range
    instead of saturating (used by the parity tests next to the literal draw)."""

    def __init__(self, rng, spread):
        self.rng = rng
        self.spread = spread

    def scale(self, channels, k):
        mult = self.rng.integers(2 ** 30, 2 ** 31 - 1, (channels,), endpoint=True).astype(np.int32)
        shift = self.rng.integers(30, 38, (channels,), endpoint=True).astype(np.int8)
        if self.spread:
            shift = (shift + int(np.ceil(np.log2(max(k, 1)))) // 2 + 2).astype(np.int8)
        return mult, shift


RELU6_ZP, RELU6_LO, RELU6_HI = -100, -100, 110   # output zero point and CLAMP bounds of the ReLU6 layers
LINEAR_ZP = 3                                    # output zero point of the linear (project) layers


def _conv_block(spec, q, rng, x, x_zp, cin, cout, k, stride, depthwise, relu6, out_name=None, out_kind="tensor"):
    """CONV2D | DEPTHWISE_CONV2D (int32) -> RESCALE (int8, per channel, double round) [-> CLAMP]."""
    n, h, w, _ = spec.shape_of(x)
    if k == 1:
        pad = (0, 0, 0, 0)
    elif stride == 1:
        pad = (1, 1, 1, 1)
    else:
        pad = (0, 1, 0, 1)  # even extents at stride 2: the only padding for which the TOSA output size divides
    oh = (h + pad[0] + pad[1] - k) // stride + 1
    ow = (w + pad[2] + pad[3] - k) // stride + 1
    if depthwise:
        wt = spec.const("dw_w", rng.integers(-127, 127, (k, k, cin, 1), endpoint=True).astype(np.int8))
        contraction = k * k
        spec.macs["depthwise"] += n * oh * ow * cout * k * k
    else:
        wt = spec.const("w", rng.integers(-127, 127, (cout, k, k, cin), endpoint=True).astype(np.int8))
        contraction = k * k * cin
        spec.macs["dense"] += n * oh * ow * cout * k * k * cin
    bias = spec.const("b", rng.integers(-2 ** 15, 2 ** 15, (cout,), endpoint=True).astype(np.int32))
    spec.layers.append({"kind": "dw" if depthwise else "conv", "in": (n, h, w, cin), "out": (n, oh, ow, cout),
                        "kernel": k, "stride": stride, "macs": n * oh * ow * cout * contraction,
                        "bytes": n * h * w * cin + spec.consts[wt].size + 9 * cout + n * oh * ow * cout})
    acc = spec.tensor("acc", abi.I32, (n, oh, ow, cout))
    spec.op("DEPTHWISE_CONV2D" if depthwise else "CONV2D", [x, wt, bias], [acc],
            list(pad) + [stride, stride, 1, 1, x_zp, 0, abi.ACC_I32])
    mult, shift = q.scale(cout, contraction)
    m, s = spec.const("m", mult), spec.const("s", shift)
    out_zp = RELU6_ZP if relu6 else LINEAR_ZP
    final_shape = (n, oh, ow, cout)

    def make_out(prefix):
        if out_name is not None:
            return out_name
        return spec.tensor(prefix, abi.I8, final_shape)

    if relu6:
        r = spec.tensor("r", abi.I8, final_shape)
        spec.op("RESCALE", [acc, m, s], [r], [0, out_zp, 1, 1, 1, 0, 0])
        y = make_out("y")
        spec.op("CLAMP", [r], [y], [abi.NAN_PROPAGATE], [RELU6_LO, RELU6_HI])
    else:
        y = make_out("y")
        spec.op("RESCALE", [acc, m, s], [y], [0, out_zp, 1, 1, 1, 0, 0])
    return y, out_zp


def _residual(spec, q, rng, x, x_zp, y, y_zp):
    """RESCALE(x -> i32) + RESCALE(y -> i32) -> ADD -> RESCALE(-> i8): the reference's residual-add pattern
    (tests/shader/graph-constant-arm.spvasm)."""
    shape = spec.shape_of(x)
    if spec.layers:  # the addition runs in the epilogue of the projection before it, which also reads x
        spec.layers[-1]["bytes"] += int(np.prod(shape))
        spec.layers[-1]["residual"] = True
    one = lambda v, dt: np.array([v], dt)
    ma = spec.const("m", one(rng.integers(2 ** 30, 2 ** 31 - 1), np.int32))
    mb = spec.const("m", one(rng.integers(2 ** 30, 2 ** 31 - 1), np.int32))
    mo = spec.const("m", one(rng.integers(2 ** 30, 2 ** 31 - 1), np.int32))
    sa, sb, so = spec.const("s", one(20, np.int8)), spec.const("s", one(20, np.int8)), spec.const("s", one(42, np.int8))
    xa, yb = spec.tensor("ra", abi.I32, shape), spec.tensor("rb", abi.I32, shape)
    spec.op("RESCALE", [x, ma, sa], [xa], [x_zp, 0, 1, 1, 0, 0, 0])
    spec.op("RESCALE", [y, mb, sb], [yb], [y_zp, 0, 1, 1, 0, 0, 0])
    total = spec.tensor("sum", abi.I32, shape)
    spec.op("ADD", [xa, yb], [total])
    out = spec.tensor("res", abi.I8, shape)
    spec.op("RESCALE", [total, mo, so], [out], [0, LINEAR_ZP, 1, 1, 0, 0, 0])
    return out, LINEAR_ZP


def _inverted_residual(spec, q, rng, x, x_zp, cin, cout, t, stride):
    h = x
    h_zp = x_zp
    hidden = cin * t
    if t != 1:
        h, h_zp = _conv_block(spec, q, rng, h, h_zp, cin, hidden, 1, 1, False, True)
    h, h_zp = _conv_block(spec, q, rng, h, h_zp, hidden, hidden, 3, stride, True, True)
    h, h_zp = _conv_block(spec, q, rng, h, h_zp, hidden, cout, 1, 1, False, False)
    if stride == 1 and cin == cout:
        h, h_zp = _residual(spec, q, rng, x, x_zp, h, h_zp)
    return h, h_zp


def inverted_residual_spec(batch=16, hw=56, channels=24, expansion=6, seed=1002, spread=False):
    """BASELINE config 2: one MobileNetV2 inverted-residual block with the residual add."""
    rng = np.random.default_rng(seed)
    spec, q = Spec(), None
    q = _Quant(rng, spread)
    spec.inputs.append(("input", abi.I8, (batch, hw, hw, channels)))
    y, _ = _inverted_residual(spec, q, rng, "input", -5, channels, channels, expansion, 1)
    # the last operator writes the graph output tensor
    _retarget_output(spec, y, "output")
    return spec


def mobilenetv2_spec(batch=32, image=224, seed=1003, spread=False, classes=1000):
    """BASELINE config 3: MobileNetV2-shaped int8 graph; 35 CONV2D, 17 DEPTHWISE_CONV2D, AVG_POOL2D and one
    MATMUL (the fully connected layer), RESCALE after every contraction, CLAMP for ReLU6."""
    rng = np.random.default_rng(seed)
    spec = Spec()
    q = _Quant(rng, spread)
    spec.inputs.append(("input", abi.I8, (batch, image, image, 3)))
    x, zp = _conv_block(spec, q, rng, "input", -5, 3, 32, 3, 2, False, True)
    cin = 32
    for t, c, n, s in MOBILENETV2_BLOCKS:
        for i in range(n):
            x, zp = _inverted_residual(spec, q, rng, x, zp, cin, c, t, s if i == 0 else 1)
            cin = c
    x, zp = _conv_block(spec, q, rng, x, zp, cin, 1280, 1, 1, False, True)
    n, h, w, c = spec.shape_of(x)
    pooled = spec.tensor("pool", abi.I8, (n, 1, 1, c))
    spec.op("AVG_POOL2D", [x], [pooled], [h, w, 1, 1, 0, 0, 0, 0, abi.ACC_I32, zp, zp])
    spec.layers.append({"kind": "avgpool", "in": (n, h, w, c), "out": (n, 1, 1, c), "kernel": h, "stride": 1,
                        "macs": 0, "bytes": n * h * w * c + n * c})
    flat = spec.tensor("flat", abi.I8, (1, n, c))
    spec.op("RESHAPE", [pooled], [flat])
    fc_w = spec.const("fc_w", rng.integers(-127, 127, (1, c, classes), endpoint=True).astype(np.int8))
    logits = spec.tensor("fc_acc", abi.I32, (1, n, classes))
    spec.op("MATMUL", [flat, fc_w], [logits], [zp, 0])
    spec.macs["dense"] += n * c * classes
    spec.layers.append({"kind": "fc", "in": (1, n, c), "out": (1, n, classes), "kernel": 1, "stride": 1,
                        "macs": n * c * classes, "bytes": n * c + c * classes + 5 + n * classes})
    mult, shift = q.scale(1, c)
    m, s = spec.const("m", mult), spec.const("s", shift)
    spec.op("RESCALE", [logits, m, s], ["output"], [0, 0, 1, 1, 0, 0, 0])
    spec.outputs.append(("output", abi.I8, (1, n, classes)))
    return spec


def transformer_block_spec(batch=8, seq=512, d_model=768, heads=12, ffn=3072, seed=1004):
    """BASELINE config 4: one fp16 transformer encoder block (pre-LayerNorm).  Projections are MATMUL with fp16
    operands and an fp32 result (bias added in fp32, then CAST to fp16); attention is MATMUL for QK^T, softmax as
    REDUCE_MAX / SUB / EXP / REDUCE_SUM / RECIPROCAL / MUL, then MATMUL with V; LayerNorm uses REDUCE_SUM and RSQRT;
    GELU uses TANH.  Activations ~N(0,1), weights ~N(0,0.02)."""
    rng = np.random.default_rng(seed)
    spec = Spec()
    spec.flops = 0
    B, S, D, H, F = batch, seq, d_model, heads, ffn
    dh = D // H
    f16, f32 = abi.F16, abi.F32
    spec.inputs.append(("input", f16, (B, S, D)))

    def c16(v):
        return spec.const("c", np.array(v, np.float16).reshape(1, 1, 1))

    def un(op, x, shape, dt=f16):
        y = spec.tensor("t", dt, shape)
        spec.op(op, [x], [y])
        return y

    def bi(op, a, b, shape, dt=f16):
        y = spec.tensor("t", dt, shape)
        spec.op(op, [a, b], [y], [0] if op == "MUL" else [])
        return y

    def red(op, x, shape):
        out = tuple(shape[:2]) + (1,)
        y = spec.tensor("t", f16, out)
        spec.op(op, [x], [y], [2, abi.NAN_PROPAGATE] if op in ("REDUCE_MAX", "REDUCE_MIN") else [2])
        return y

    def layer_norm(x, shape):
        inv = c16(1.0 / shape[2])
        mean = bi("MUL", red("REDUCE_SUM", x, shape), inv, shape[:2] + (1,))
        xc = bi("SUB", x, mean, shape)
        var = bi("MUL", red("REDUCE_SUM", bi("MUL", xc, xc, shape), shape), inv, shape[:2] + (1,))
        rstd = un("RSQRT", bi("ADD", var, c16(1e-3), shape[:2] + (1,)), shape[:2] + (1,))
        xn = bi("MUL", xc, rstd, shape)
        gamma = spec.const("gamma", (1.0 + 0.02 * rng.standard_normal((1, 1, shape[2]))).astype(np.float16))
        beta = spec.const("beta", (0.02 * rng.standard_normal((1, 1, shape[2]))).astype(np.float16))
        return bi("ADD", bi("MUL", xn, gamma, shape), beta, shape)

    def reshape(x, shape, dt=f16):
        y = spec.tensor("t", dt, shape)
        spec.op("RESHAPE", [x], [y])
        return y

    def transpose(x, perms):
        src = spec.shape_of(x)
        shape = tuple(src[p] for p in perms)
        y = spec.tensor("t", f16, shape)
        spec.op("TRANSPOSE", [x], [y], list(perms))
        return y

    def linear(x2, k, n, rows):
        """x2 [1, rows, k] fp16 -> [1, rows, n] fp16: MATMUL (fp32 result) + bias (fp32) -> CAST."""
        w = spec.const("w", (0.02 * rng.standard_normal((1, k, n))).astype(np.float16))
        b = spec.const("b", (0.02 * rng.standard_normal((1, 1, n))).astype(np.float32))
        acc = spec.tensor("acc", f32, (1, rows, n))
        spec.op("MATMUL", [x2, w], [acc], [0, 0])
        spec.flops += 2 * rows * k * n
        return un("CAST", bi("ADD", acc, b, (1, rows, n), f32), (1, rows, n))

    rows = B * S
    x = "input"
    y = reshape(layer_norm(x, (B, S, D)), (1, rows, D))
    q = reshape(transpose(reshape(linear(y, D, D, rows), (B, S, H, dh)), (0, 2, 1, 3)), (B * H, S, dh))
    kt = reshape(transpose(reshape(linear(y, D, D, rows), (B, S, H, dh)), (0, 2, 3, 1)), (B * H, dh, S))
    v = reshape(transpose(reshape(linear(y, D, D, rows), (B, S, H, dh)), (0, 2, 1, 3)), (B * H, S, dh))
    sc32 = spec.tensor("acc", f32, (B * H, S, S))
    spec.op("MATMUL", [q, kt], [sc32], [0, 0])
    spec.flops += 2 * B * H * S * S * dh
    pshape = (B * H, S, S)
    sc = bi("MUL", un("CAST", sc32, pshape), c16(1.0 / np.sqrt(dh)), pshape)
    e = un("EXP", bi("SUB", sc, red("REDUCE_MAX", sc, pshape), pshape), pshape)
    prob = bi("MUL", e, un("RECIPROCAL", red("REDUCE_SUM", e, pshape), (B * H, S, 1)), pshape)
    ctx32 = spec.tensor("acc", f32, (B * H, S, dh))
    spec.op("MATMUL", [prob, v], [ctx32], [0, 0])
    spec.flops += 2 * B * H * S * S * dh
    ctx = reshape(transpose(reshape(un("CAST", ctx32, (B * H, S, dh)), (B, H, S, dh)), (0, 2, 1, 3)), (1, rows, D))
    x1 = bi("ADD", x, reshape(linear(ctx, D, D, rows), (B, S, D)), (B, S, D))
    y2 = reshape(layer_norm(x1, (B, S, D)), (1, rows, D))
    h = linear(y2, D, F, rows)
    hs = (1, rows, F)
    inner = bi("MUL", bi("ADD", h, bi("MUL", bi("MUL", bi("MUL", h, h, hs), h, hs), c16(0.044715), hs), hs),
               c16(np.sqrt(2.0 / np.pi)), hs)
    gelu = bi("MUL", bi("MUL", h, c16(0.5), hs), bi("ADD", un("TANH", inner, hs), c16(1.0), hs), hs)
    f = reshape(linear(gelu, F, D, rows), (B, S, D))
    spec.op("ADD", [x1, f], ["output"])
    spec.outputs.append(("output", f16, (B, S, D)))
    return spec


def _retarget_output(spec, produced, name):
    """Makes the operator that produces `produced` write the external output tensor `name` instead."""
    dtype, shape = spec.tensors.pop(produced)
    for op in spec.ops:
        op["out"] = [name if o == produced else o for o in op["out"]]
        op["in"] = [name if i == produced else i for i in op["in"]]
    spec.outputs.append((name, dtype, shape))


def build(dev, spec, fuse=True, split=False):
    """Creates the GraphPipeline for `spec` on `dev`: constants are uploaded, inputs/outputs become external
    tensors, everything else lives in planned session memory.  `split`: the batch split over two streams."""
    g = Graph(dev)
    if split:
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
    g.finalize(fuse)
    return g


def _time_graph(dev, g, steps, warmup, rounds=5):
    """(wall seconds, event milliseconds) per graph: the median over `rounds` rounds of `steps` dispatches each, every
    round between two events and two host time stamps."""
    for _ in range(warmup):
        g.dispatch()
    dev.sync()
    ev0, ev1 = dev.event(), dev.event()
    walls, gpus = [], []
    for _ in range(rounds):
        t0 = time.perf_counter()
        dev.record(ev0)
        for _ in range(steps):
            g.dispatch()
        dev.record(ev1)
        dev.sync()
        walls.append((time.perf_counter() - t0) / steps)
        gpus.append(dev.elapsed_ms(ev0, ev1) / steps)
    return float(np.median(walls)), float(np.median(gpus))


_STREAMS = {}


def in_flight_streams(dev, count):
    """`count` streams of `dev`, created once and kept for every leg.  The runtime deals its hardware queues to streams
    as they are created, and which streams the hardware then runs side by side is not in this program's hands: on one
    box the first four streams of a process finish four MobileNetV2 sessions in 0.22 ms per graph and the next four in
    0.17 ms, with eight hardware queues instead of four it is the other way round, and three sessions reach 0.17 ms
    either way.  The legs report what the streams they were given deliver."""
    have = _STREAMS.setdefault(id(dev), [])
    while len(have) < count:
        have.append(dev.new_stream())
    return have[:count]


def _time_sessions(dev, g, input_name, output_name, steps, batch, count, replayed=False):
    """Throughput with `count` batches in flight: that many sessions of the one pipeline (session memory and external
    tensors of their own, the same input data) dispatched in turn on a stream each, as a serving loop that keeps the
    next batches queued behind the current one.  A dependent launch costs about 5 us whatever the batch, and the other
    streams' launches fill the gaps.  Every graph is a whole batch; every output is checked against the
    single-session result.  With four sessions the host's launch rate, about 4 us per launch, is the limit of eager
    dispatches; `replayed` dispatches through mlel_graph_session_dispatch_replayed (each session's launches recorded
    into a HIP graph on first use, one submission per dispatch afterwards)."""
    want = g.get_output(output_name)
    x = g.ext_tensors[input_name].download()
    sessions = [g.new_session() for _ in range(count)]
    streams = in_flight_streams(dev, count)
    for s in sessions:
        s.set_input(input_name, x)
    sync_all = lambda: dev._check(dev.lib.mlel_hip_sync(dev.ctx, None))
    go = (lambda k: sessions[k % count].dispatch_replayed(streams[k % count])) if replayed else \
        (lambda k: sessions[k % count].dispatch(streams[k % count]))
    for k in range(2 * count):
        go(k)
    sync_all()
    same = all(np.array_equal(s.get_output(output_name), want) for s in sessions)
    n = count * max(steps, 10)
    t0 = time.perf_counter()
    for k in range(n):
        go(k)
    sync_all()
    wall = (time.perf_counter() - t0) / n
    for s in sessions:
        s.close()
    return {"img_per_s": batch / wall, "ms_per_graph": wall * 1e3, "graphs_timed": n, "streams": count,
            "dispatch": "replayed" if replayed else "eager",
            "outputs_equal_single_session": bool(same)}


def _time_replayed(dev, g, input_name, output_name, want, steps, rounds=5):
    """Milliseconds per graph of one session's replayed dispatch (mlel_graph_session_dispatch_replayed: the launches
    recorded into a HIP graph once, one submission per dispatch), one batch in flight: the median over `rounds`
    rounds of `steps` dispatches on one stream; and whether the output equals `want`."""
    stream = in_flight_streams(dev, 1)[0]
    s = g.new_session()
    s.set_input(input_name, g.ext_tensors[input_name].download())
    for _ in range(3):
        s.dispatch_replayed(stream)
    dev._check(dev.lib.mlel_hip_sync(dev.ctx, stream))
    same = bool(np.array_equal(s.get_output(output_name), want))
    walls = []
    for _ in range(rounds):
        t0 = time.perf_counter()
        for _ in range(steps):
            s.dispatch_replayed(stream)
        dev._check(dev.lib.mlel_hip_sync(dev.ctx, stream))
        walls.append((time.perf_counter() - t0) / steps)
    s.close()
    return float(np.median(walls)) * 1e3, same


def bench_batch_split(dev, spec, g, input_name, output_name, steps, warmup):
    """One batch in flight, four ways: the pipeline `g` dispatched eagerly (timed by the caller) and replayed, and the
    same graph with the batch split over two streams (mlel_graph_set_batch_split) dispatched eagerly and replayed.
    Every output is compared with the eager unsplit one."""
    want = g.get_output(output_name)
    x = g.ext_tensors[input_name].download()
    rounds = max(5, -(-50 // steps))
    replayed_ms, same_r = _time_replayed(dev, g, input_name, output_name, want, steps, rounds)
    sp = build(dev, spec, fuse=True, split=True)
    sp.set_input(input_name, x)
    wall, _ = _time_graph(dev, sp, steps, warmup, rounds)
    same_e = bool(np.array_equal(sp.get_output(output_name), want))
    split_replayed_ms, same_s = _time_replayed(dev, sp, input_name, output_name, want, steps, rounds)
    res = {"launches_split": sp.batch_split_launches(), "session_memory_bytes": sp.session_size,
           "ms_per_graph": {"one_stream_eager": None, "one_stream_replayed": replayed_ms,
                            "split_eager": wall * 1e3, "split_replayed": split_replayed_ms},
           "outputs_equal_unsplit_eager": bool(same_r and same_e and same_s)}
    sp.close()
    return res


def time_operators(dev, g, reps=50, only=None):
    """Milliseconds per launch of every executed operator of `g` on its own: the operator is launched `reps` times
    back to back on the stream (its inputs are whatever the last whole dispatch left in session memory) between two
    events.  `only`: a list of operator positions."""
    s = g.new_session(allocate=False)
    s.bind_memory(g.session_mem)
    for name, t in g.ext_tensors.items():
        s.bind(name, t)
    out = {}
    ev0, ev1 = dev.event(), dev.event()
    for i in (range(g.op_count()) if only is None else only):
        for _ in range(3):
            s.dispatch_range(i, 1)
        dev.record(ev0)
        for _ in range(reps):
            s.dispatch_range(i, 1)
        dev.record(ev1)
        dev.sync()
        out[i] = dev.elapsed_ms(ev0, ev1) / reps
    s.close(free_tensors=False)
    return out


def launch_layers(g, spec):
    """The layers of `spec` (one per CONV2D / DEPTHWISE_CONV2D / AVG_POOL2D / MATMUL of the graph) grouped by the
    launches of the fused graph `g`: a launch whose name holds both CONV2D and DEPTHWISE_CONV2D covers the 1x1
    convolution and the depthwise layer behind it, whose intermediate tensor never reaches memory (its bytes leave
    the launch's algorithmic bytes).  None when the names do not account for every layer."""
    out, at = [], 0
    for i in range(g.op_count()):
        name = g.op_name(i)
        if at >= len(spec.layers):
            return None
        if name.startswith("CONV2D") and "DEPTHWISE_CONV2D" in name:
            if at + 1 >= len(spec.layers):
                return None
            conv, dw = spec.layers[at], spec.layers[at + 1]
            if conv["kind"] != "conv" or dw["kind"] != "dw":
                return None
            mid = int(np.prod(conv["out"]))
            out.append({"kind": "conv+dw", "in": conv["in"], "out": dw["out"], "kernel": dw["kernel"],
                        "stride": dw["stride"], "macs": conv["macs"] + dw["macs"],
                        "bytes": conv["bytes"] + dw["bytes"] - 2 * mid, "layers": [at, at + 1]})
            at += 2
        elif name.startswith("CONV2D") and name.count("CONV2D") == 2:
            # a projection and the expansion behind it: the intermediate tensor is neither written nor read, or, with
            # "+KEEP", written once for a later reader
            if at + 1 >= len(spec.layers):
                return None
            c1, c2 = spec.layers[at], spec.layers[at + 1]
            if c1["kind"] != "conv" or c2["kind"] != "conv":
                return None
            mid = int(np.prod(c1["out"]))
            kept = "+KEEP" in name
            out.append({"kind": "conv+conv", "in": c1["in"], "out": c2["out"], "kernel": 1, "stride": 1,
                        "macs": c1["macs"] + c2["macs"], "bytes": c1["bytes"] + c2["bytes"] - (mid if kept else 2 * mid),
                        "layers": [at, at + 1]})
            at += 2
        elif name.startswith("CONV2D") and name.endswith("AVG_POOL2D"):
            # the head: the convolution's result is pooled in registers and never reaches memory
            if at + 1 >= len(spec.layers):
                return None
            conv, pool = spec.layers[at], spec.layers[at + 1]
            if conv["kind"] != "conv" or pool["kind"] != "avgpool":
                return None
            mid = int(np.prod(conv["out"]))
            out.append({"kind": "conv+avgpool", "in": conv["in"], "out": pool["out"], "kernel": 1, "stride": 1,
                        "macs": conv["macs"] + pool["macs"], "bytes": conv["bytes"] + pool["bytes"] - 2 * mid,
                        "layers": [at, at + 1]})
            at += 2
        else:
            out.append(dict(spec.layers[at], layers=[at]))
            at += 1
    return out if at == len(spec.layers) else None


def bench_mobilenetv2(dev, steps=20, warmup=3, batch=32, per_layer=True, in_flight=(2, 3, 4)):
    """Times whole-graph dispatches of BASELINE config 3 (inputs resident in HBM) and every launch on its own; returns
    the extra fields bench.py adds to its JSON line, with the MFMA position of the dense (CONV2D / MATMUL) launches
    and the HBM position of the bandwidth-bound (DEPTHWISE_CONV2D, AVG_POOL2D) ones."""
    spec = mobilenetv2_spec(batch=batch)
    g = build(dev, spec, fuse=True)
    rng = np.random.default_rng(1003)
    g.set_input("input", rng.integers(-128, 127, spec.inputs[0][2], endpoint=True).astype(np.int8))
    rounds = max(5, -(-50 // steps))
    wall, gpu_ms = _time_graph(dev, g, steps, warmup, rounds)
    per_op = g.dispatch_profiled()
    dev.sync()
    by_kind = {}
    for name, ms in per_op:
        by_kind[name] = by_kind.get(name, 0.0) + ms
    macs = spec.macs["dense"] + spec.macs["depthwise"]
    res = {"img_per_s": batch / wall, "ms_per_graph": wall * 1e3, "gpu_ms_per_graph": gpu_ms,
           "graphs_timed": steps * rounds, "timing": f"median of {rounds} rounds of {steps} dispatches", "tops": 2.0 * macs / wall / 1e12, "gmac": macs / 1e9,
           "operators_executed": g.op_count(), "operators_in_graph": len(spec.ops),
           "session_memory_bytes": g.session_size,
           "ms_by_operator": {k: round(v, 4) for k, v in sorted(by_kind.items())}}
    # one batch in flight, the other ways to issue it: replayed, and with the batch split over two streams
    split = bench_batch_split(dev, spec, g, "input", "output", steps, warmup)
    split["ms_per_graph"]["one_stream_eager"] = wall * 1e3
    best = min(split["ms_per_graph"], key=lambda k: split["ms_per_graph"][k])
    split["best"] = best
    split["img_per_s_best"] = batch / (split["ms_per_graph"][best] * 1e-3)
    res["one_batch_dispatch_modes"] = split
    # The headline figures are those of the best way to issue ONE batch (the reference's counterpart is a command
    # buffer recorded once and submitted per batch); the eager single-stream dispatch stays beside them.
    res["ms_per_graph_eager_one_stream"], res["img_per_s_eager_one_stream"] = res["ms_per_graph"], res["img_per_s"]
    res["ms_per_graph"], res["img_per_s"] = split["ms_per_graph"][best], split["img_per_s_best"]
    res["tops"] = 2.0 * macs / (res["ms_per_graph"] * 1e-3) / 1e12
    res["dispatch"] = {"one_stream_eager": "eager, one stream", "one_stream_replayed": "replayed HIP graph, one stream",
                       "split_eager": "eager, batch split over two streams",
                       "split_replayed": "replayed HIP graph, batch split over two streams"}[best]
    res["sessions_in_flight"] = [_time_sessions(dev, g, "input", "output", steps, batch, c) for c in in_flight]
    if in_flight:
        res["sessions_in_flight"].append(_time_sessions(dev, g, "input", "output", steps, batch, max(in_flight), replayed=True))
    launches = launch_layers(g, spec) if per_layer else None
    if launches is not None:
        alone = time_operators(dev, g)
        layers = []
        for i, layer in enumerate(launches):
            ms = alone[i]
            layers.append({"index": i, "kind": layer["kind"], "in": list(layer["in"]), "out": list(layer["out"]),
                           "kernel": layer["kernel"], "stride": layer["stride"], "us": round(ms * 1e3, 2),
                           "tops": round(2.0 * layer["macs"] / (ms * 1e-3) / 1e12, 2),
                           "gbs": round(layer["bytes"] / (ms * 1e-3) / 1e9, 1)})
        # a launch that holds a CONV2D or MATMUL (also the expansion + depthwise pairs) is priced against the matrix
        # cores, a stand-alone DEPTHWISE_CONV2D or AVG_POOL2D against HBM
        dense = [(l, launches[l["index"]]) for l in layers if l["kind"] in ("conv", "fc", "conv+dw", "conv+conv", "conv+avgpool")]
        band = [(l, launches[l["index"]]) for l in layers if l["kind"] in ("dw", "avgpool")]

        def total(group, key):
            return float(sum(meta[key] for _, meta in group))

        d_ms = sum(l["us"] for l, _ in dense) * 1e-3
        b_ms = sum(l["us"] for l, _ in band) * 1e-3
        top_d = max(dense, key=lambda p: p[0]["us"])
        top_b = max(band, key=lambda p: p[0]["us"])
        res["layers"] = layers
        res["roofline_dense"] = {
            "bound": "mfma", "unit": "TFLOP/s", "peak": 5000.0, "launches": len(dense),
            "achieved": 2.0 * total(dense, "macs") / (d_ms * 1e-3) / 1e12,
            "frac": 2.0 * total(dense, "macs") / (d_ms * 1e-3) / 1e12 / 5000.0,
            "algorithmic_bytes": total(dense, "bytes"), "us_sum_of_launches": d_ms * 1e3,
            "hbm_frac_of_the_same_launches": total(dense, "bytes") / (d_ms * 1e-3) / 1e9 / 8000.0,
            "dominant_launch": dict(top_d[0], frac=top_d[0]["tops"] / 5000.0,
                                    hbm_frac=top_d[0]["gbs"] / 8000.0)}
        res["roofline_bandwidth"] = {
            "bound": "hbm", "unit": "GB/s", "peak": 8000.0, "launches": len(band),
            "achieved": total(band, "bytes") / (b_ms * 1e-3) / 1e9,
            "frac": total(band, "bytes") / (b_ms * 1e-3) / 1e9 / 8000.0,
            "algorithmic_bytes": total(band, "bytes"), "us_sum_of_launches": b_ms * 1e3,
            "dominant_launch": dict(top_b[0], frac=top_b[0]["gbs"] / 8000.0)}
    g.close()
    return {"mobilenetv2_b32": res}


def bench_inverted_residual(dev, steps=20, warmup=3):
    """BASELINE config 2 (one int8 inverted-residual block with its residual addition, 16 x 56 x 56 x 24) through the
    GraphPipeline: microseconds per graph, TOP/s, every launch of the fused graph on its own, and the position of the
    block against both rooflines (its launches are few and short: neither is close)."""
    spec = inverted_residual_spec()
    g = build(dev, spec, fuse=True)
    rng = np.random.default_rng(1002)
    g.set_input("input", rng.integers(-128, 127, spec.inputs[0][2], endpoint=True).astype(np.int8))
    rounds = max(5, -(-50 // steps))
    wall, gpu_ms = _time_graph(dev, g, steps, warmup, rounds)
    macs = spec.macs["dense"] + spec.macs["depthwise"]
    names = g.op_names()
    alone = time_operators(dev, g)
    launches = launch_layers(g, spec)
    # algorithmic bytes of the fused block: the input twice (expansion and residual), weights and constants, the two
    # intermediate activations written and read once each, the output once
    nbytes = sum(l["bytes"] for l in launches) + int(np.prod(spec.inputs[0][2])) if launches else None
    res = {"us_per_graph": wall * 1e6, "gpu_us_per_graph": gpu_ms * 1e3, "graphs_timed": steps * rounds,
           "timing": f"median of {rounds} rounds of {steps} dispatches", "img_per_s": spec.inputs[0][2][0] / wall,
           "tops": 2.0 * macs / wall / 1e12, "gmac": macs / 1e9, "operators_in_graph": len(spec.ops),
           "operators_executed": g.op_count(),
           "us_by_launch_alone": [{"index": i, "name": names[i], "us": round(ms * 1e3, 2)} for i, ms in alone.items()],
           "roofline": {"mfma_frac": 2.0 * macs / (gpu_ms * 1e-3) / 1e12 / 5000.0, "mfma_peak_tops": 5000.0,
                        "algorithmic_bytes": nbytes, "hbm_peak_gbs": 8000.0,
                        "hbm_frac": None if nbytes is None else nbytes / (gpu_ms * 1e-3) / 1e9 / 8000.0}}
    g.close()
    return {"config2_inverted_residual_b16": res}


def bench_transformer(dev, steps=20, warmup=3, in_flight=(2, 3, 4)):
    """Times whole-graph dispatches of BASELINE config 4 (fp16 encoder block, batch 8, seq 512, d_model 768) and every
    launch on its own; returns the extra fields bench.py adds to its JSON line, with the fp16 MFMA position of the
    launches that hold a MATMUL."""
    spec = transformer_block_spec()
    g = build(dev, spec, fuse=True)
    rng = np.random.default_rng(1004)
    g.set_input("input", rng.standard_normal(spec.inputs[0][2]).astype(np.float16))
    rounds = max(5, -(-50 // steps))
    wall, gpu_ms = _time_graph(dev, g, steps, warmup, rounds)
    per_op = g.dispatch_profiled()
    dev.sync()
    by_kind = {}
    for name, ms in per_op:
        by_kind[name] = by_kind.get(name, 0.0) + ms
    counts = in_flight
    in_flight = [_time_sessions(dev, g, "input", "output", steps, spec.inputs[0][2][0], c) for c in counts]
    if counts:
        in_flight.append(_time_sessions(dev, g, "input", "output", steps, spec.inputs[0][2][0], max(counts), replayed=True))
    for r in in_flight:  # a "graph" is one encoder block over the whole batch
        r["tflops"] = spec.flops / (r["ms_per_graph"] * 1e-3) / 1e12
        r["blocks_per_s"] = r.pop("img_per_s") / spec.inputs[0][2][0]
    alone = time_operators(dev, g)
    names = g.op_names()
    gemm_ms = sum(ms for i, ms in alone.items() if "MATMUL" in names[i])
    other_ms = sum(ms for i, ms in alone.items() if "MATMUL" not in names[i])
    res = {"transformer_b8_s512_d768": {
        "ms_per_graph": wall * 1e3, "gpu_ms_per_graph": gpu_ms, "graphs_timed": steps * rounds,
        "timing": f"median of {rounds} rounds of {steps} dispatches", "tflops": spec.flops / wall / 1e12,
        "gflop": spec.flops / 1e9, "operators_executed": g.op_count(), "operators_in_graph": len(spec.ops),
        "session_memory_bytes": g.session_size, "sessions_in_flight": in_flight,
        "ms_by_operator": {k: round(v, 4) for k, v in sorted(by_kind.items())},
        "us_by_launch_alone": [{"index": i, "name": names[i], "us": round(ms * 1e3, 2)} for i, ms in alone.items()],
        "roofline_gemm": {"bound": "mfma", "unit": "TFLOP/s", "peak": 2500.0,
                          "launches": sum(1 for n in names if "MATMUL" in n),
                          "achieved": spec.flops / (gemm_ms * 1e-3) / 1e12,
                          "frac": spec.flops / (gemm_ms * 1e-3) / 1e12 / 2500.0,
                          "us_sum_of_launches": gemm_ms * 1e3, "us_other_launches": other_ms * 1e3}}}
    g.close()
    return res
