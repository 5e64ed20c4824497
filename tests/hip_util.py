"""Helpers for the GPU parity tests: run one operator through the C ABI on numpy inputs."""
import ctypes as C
import importlib

import numpy as np

abi = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.abi")
hb = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.hip_backend")


def gpu_available():
    try:
        return hb.device_count() > 0
    except Exception:
        return False


class Runner:
    """Uploads numpy inputs, runs one C-ABI entry point, downloads the output; frees everything after."""

    def __init__(self, dev):
        self.dev = dev
        self.live = []

    def put(self, arr, dtype=None, strides=None):
        t = self.dev.from_numpy(np.asanyarray(arr), dtype, strides)
        self.live.append(t)
        return t

    def new(self, dtype, shape, strides=None):
        t = self.dev.tensor(dtype, shape, strides)
        self.live.append(t)
        return t

    def done(self):
        for t in self.live:
            t.free()
        self.live = []

    # ---- operators -------------------------------------------------------------------------------------------
    def conv2d(self, x, w, b, out_shape, out_dtype, attr, depthwise=False, epilogue=None, x_strides=None):
        tx, tw, tb = self.put(x, strides=x_strides), self.put(w), self.put(b)
        to = self.new(out_dtype, out_shape)
        name = "depthwise_conv2d" if depthwise else "conv2d"
        if epilogue is None:
            self.dev.op(name, to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr))
        else:
            e = self._epi(*epilogue)
            self.dev.op("dwconv_rescale_clamp" if depthwise else "conv2d_rescale_clamp", to.ref, tx.ref, tw.ref,
                        tb.ref, C.byref(attr), C.byref(e))
        r = to.download()
        self.done()
        return r

    def _epi(self, mult, shift, rattr, clamp):
        return self.dev.epilogue(self.put(mult), self.put(shift), rattr, clamp)

    def matmul(self, a, b, out_dtype, a_zp=0, b_zp=0, epilogue=None, b_rows=False):
        """b_rows: B described as the operator's [NB, K, N] tensor over a matrix stored row-wise, [NB, N, K]."""
        ta = self.put(a)
        if b_rows:
            nb, k, n = b.shape
            es = b.dtype.itemsize
            stored = self.put(np.ascontiguousarray(np.transpose(b, (0, 2, 1))))
            tb = abi.make_tensor(stored.view.ptr, stored.view.dtype, b.shape, [n * k * es, es, k * es])
        else:
            tb = self.put(b).view
        to = self.new(out_dtype, (a.shape[0], a.shape[1], b.shape[2]))
        attr = abi.MatmulAttr(int(a_zp), int(b_zp))
        if epilogue is None:
            self.dev.op("matmul", to.ref, ta.ref, C.byref(tb), C.byref(attr))
        else:
            e = self._epi(*epilogue)
            self.dev.op("matmul_rescale", to.ref, ta.ref, C.byref(tb), C.byref(attr), C.byref(e))
        r = to.download()
        self.done()
        return r

    def rescale(self, x, mult, shift, out_dtype, attr, in_dtype=None):
        tx, tm, ts = self.put(x, in_dtype), self.put(mult), self.put(shift)
        to = self.new(out_dtype, x.shape)
        self.dev.op("rescale", to.ref, tx.ref, tm.ref, ts.ref, C.byref(attr))
        r = to.download()
        self.done()
        return r

    def clamp(self, x, mn, mx, nan_mode=abi.NAN_PROPAGATE):
        tx = self.put(x)
        to = self.new(tx.dtype, x.shape)
        self.dev.op("clamp", to.ref, tx.ref, C.byref(abi.ClampAttr(float(mn), float(mx), int(nan_mode))))
        r = to.download()
        self.done()
        return r

    def binary(self, op, a, b, out_shape, out_dtype, nan_mode=abi.NAN_PROPAGATE):
        ta, tb = self.put(a), self.put(b)
        to = self.new(out_dtype, out_shape)
        self.dev.op("elementwise_binary", abi.BIN[op], to.ref, ta.ref, tb.ref, int(nan_mode))
        r = to.download()
        self.done()
        return r

    def mul(self, a, b, out_shape, out_dtype, shift=0):
        ta, tb = self.put(a), self.put(b)
        to = self.new(out_dtype, out_shape)
        self.dev.op("mul", to.ref, ta.ref, tb.ref, int(shift))
        r = to.download()
        self.done()
        return r

    def unary(self, op, x):
        tx = self.put(x)
        to = self.new(tx.dtype, x.shape)
        self.dev.op("elementwise_unary", abi.UN[op], to.ref, tx.ref)
        r = to.download()
        self.done()
        return r

    def reduce(self, op, x, axis, nan_mode=abi.NAN_PROPAGATE):
        tx = self.put(x)
        shape = list(x.shape)
        shape[axis] = 1
        to = self.new(tx.dtype, shape)
        self.dev.op("reduce", abi.RED[op], to.ref, tx.ref, int(axis), int(nan_mode))
        r = to.download()
        self.done()
        return r

    def pool(self, kind, x, out_shape, attr):
        tx = self.put(x)
        to = self.new(tx.dtype, out_shape)
        self.dev.op(kind, to.ref, tx.ref, C.byref(attr))
        r = to.download()
        self.done()
        return r

    def table(self, x, tab, out_dtype):
        tx, tt = self.put(x), self.put(tab)
        to = self.new(out_dtype, x.shape)
        self.dev.op("table", to.ref, tx.ref, tt.ref)
        r = to.download()
        self.done()
        return r

    def cast(self, x, out_dtype):
        tx = self.put(x)
        to = self.new(out_dtype, x.shape)
        self.dev.op("cast", to.ref, tx.ref)
        r = to.download()
        self.done()
        return r

    def negate(self, x, zi=0, zo=0):
        tx = self.put(x)
        to = self.new(tx.dtype, x.shape)
        self.dev.op("negate", to.ref, tx.ref, int(zi), int(zo))
        r = to.download()
        self.done()
        return r

    def reshape(self, x, out_shape):
        tx = self.put(x)
        to = self.new(tx.dtype, out_shape)
        self.dev.op("reshape", to.ref, tx.ref)
        r = to.download()
        self.done()
        return r

    def transpose(self, x, perms):
        tx = self.put(x)
        to = self.new(tx.dtype, [x.shape[p] for p in perms])
        arr = (C.c_uint32 * abi.MAX_RANK)(*[int(p) for p in perms])
        self.dev.op("transpose", to.ref, tx.ref, arr)
        r = to.download()
        self.done()
        return r

    def concat_at(self, base, part, axis, offset):
        """One CONCAT part written into an output that starts as `base`, at `offset` along `axis`."""
        to, ti = self.put(base), self.put(part)
        self.dev.op("concat", to.ref, ti.ref, int(axis), int(offset))
        r = to.download()
        self.done()
        return r

    def concat(self, inputs, axis):
        shape = list(inputs[0].shape)
        shape[axis] = sum(i.shape[axis] for i in inputs)
        to = self.new(abi.dtype_of_array(inputs[0]), shape)
        off = 0
        for i in inputs:
            ti = self.put(i)
            self.dev.op("concat", to.ref, ti.ref, int(axis), int(off))
            off += i.shape[axis]
        r = to.download()
        self.done()
        return r

    def slice_(self, x, start, size):
        tx = self.put(x)
        to = self.new(tx.dtype, size)
        arr = (C.c_uint32 * abi.MAX_RANK)(*[int(p) for p in start])
        self.dev.op("slice", to.ref, tx.ref, arr)
        r = to.download()
        self.done()
        return r

    def pad(self, x, padding, out_shape, pad_const=0.0, pad_const_int=0):
        tx = self.put(x)
        tp = self.put(np.ascontiguousarray(padding, dtype=np.int32).reshape(-1))
        to = self.new(tx.dtype, out_shape)
        self.dev.op("pad", to.ref, tx.ref, tp.ref, float(pad_const), int(pad_const_int))
        r = to.download()
        self.done()
        return r

    def rescale_add_rescale(self, a, ea, b, eb, eo, out_dtype):
        ta, tb = self.put(a), self.put(b)
        to = self.new(out_dtype, a.shape)
        e1, e2, e3 = self._epi(*ea), self._epi(*eb), self._epi(*eo)
        self.dev.op("rescale_add_rescale", to.ref, ta.ref, C.byref(e1), tb.ref, C.byref(e2), C.byref(e3))
        r = to.download()
        self.done()
        return r

    def conv2d_rescale_add_rescale(self, x, w, b, attr, epi, e_conv, res, e_res, e_out, residual_first=False,
                                   res_strides=None):
        tx, tw, tb, tr = self.put(x), self.put(w), self.put(b), self.put(res, strides=res_strides)
        to = self.new(abi.I8, res.shape)
        e0, e1, e2, e3 = self._epi(*epi), self._epi(*e_conv), self._epi(*e_res), self._epi(*e_out)
        self.dev.op("conv2d_rescale_add_rescale", to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr), C.byref(e0),
                    C.byref(e1), tr.ref, C.byref(e2), C.byref(e3), int(residual_first))
        r = to.download()
        self.done()
        return r

    def conv2d_dwconv(self, x, w1, b1, attr1, epi1, w2, b2, attr2, epi2, out_shape, expect=0):
        tx, tw1, tb1, tw2, tb2 = self.put(x), self.put(w1), self.put(b1), self.put(w2), self.put(b2)
        to = self.new(abi.I8, out_shape)
        e1, e2 = self._epi(*epi1), self._epi(*epi2)
        args = (tx.ref, tw1.ref, tb1.ref, C.byref(attr1), C.byref(e1), tw2.ref, tb2.ref, C.byref(attr2), C.byref(e2))
        covered = self.dev.lib.mlel_hip_conv2d_dwconv_in_kernel(to.ref, tx.ref, tw1.ref, tb1.ref, C.byref(attr1),
                                                                tw2.ref, tb2.ref, C.byref(attr2))
        if expect != 0:
            rc = self.dev.lib.mlel_hip_conv2d_dwconv_rescale_clamp(self.dev.ctx, self.dev.stream, to.ref, *args)
            self.done()
            return covered, rc
        self.dev.op("conv2d_dwconv_rescale_clamp", to.ref, *args)
        r = to.download()
        self.done()
        return covered, r

    def conv2d_conv2d(self, x, w1, b1, attr1, epi1, w2, b2, attr2, epi2, out_shape, keep_mid=False):
        """(covered by the one-pass kernel?, output, intermediate tensor or None)"""
        tx, tw1, tb1, tw2, tb2 = self.put(x), self.put(w1), self.put(b1), self.put(w2), self.put(b2)
        to = self.new(abi.I8, out_shape)
        tm = self.new(abi.I8, tuple(x.shape[:3]) + (w1.shape[0],)) if keep_mid else None
        e1, e2 = self._epi(*epi1), self._epi(*epi2)
        covered = self.dev.lib.mlel_hip_conv2d_conv2d_in_kernel(to.ref, tx.ref, tw1.ref, tb1.ref, C.byref(attr1),
                                                                tw2.ref, tb2.ref, C.byref(attr2))
        self.dev.op("conv2d_conv2d_rescale_clamp", to.ref, tm.ref if keep_mid else None, tx.ref, tw1.ref, tb1.ref,
                    C.byref(attr1), C.byref(e1), tw2.ref, tb2.ref, C.byref(attr2), C.byref(e2))
        r = to.download()
        m = tm.download() if keep_mid else None
        self.done()
        return covered, r, m

    def conv2d_avgpool(self, x, w, b, attr, epi, pool):
        """(covered by the one-launch kernel?, pooled output [N, 1, 1, OC])"""
        tx, tw, tb = self.put(x), self.put(w), self.put(b)
        to = self.new(abi.I8, (x.shape[0], 1, 1, w.shape[0]))
        e = self._epi(*epi)
        covered = self.dev.lib.mlel_hip_conv2d_avgpool_in_kernel(to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr), abi.I8,
                                                                 C.byref(pool))
        self.dev.op("conv2d_rescale_clamp_avgpool", to.ref, tx.ref, tw.ref, tb.ref, C.byref(attr), C.byref(e), abi.I8,
                    C.byref(pool))
        r = to.download()
        self.done()
        return covered, r

    def softmax_rows(self, x):
        tx = self.put(x)
        to = self.new(tx.dtype, x.shape)
        self.dev.op("softmax_rows", to.ref, tx.ref)
        r = to.download()
        self.done()
        return r

    def _b_operand(self, b, b_rows):
        """B [NB, K, N] as the operators define it, or (b_rows) the same tensor described over a matrix stored
        row-wise, [NB, N, K]: element (k, n) at n * 2K + 2k bytes.  Returns what a call takes as its B argument."""
        if not b_rows:
            return self.put(b).view
        nb, k, n = b.shape
        stored = self.put(np.ascontiguousarray(np.transpose(b, (0, 2, 1))))
        return abi.make_tensor(stored.view.ptr, abi.F16, b.shape, [n * k * 2, 2, k * 2])

    def matmul_bias_cast(self, a, b, bias, b_rows=False):
        ta, tb = self.put(a), self._b_operand(b, b_rows)
        tbias = self.put(bias) if bias is not None else None
        to = self.new(abi.F16, (a.shape[0], a.shape[1], b.shape[2]))
        self.dev.op("matmul_bias_cast", to.ref, ta.ref, C.byref(tb), tbias.ref if tbias else None, C.byref(abi.MatmulAttr(0, 0)))
        r = to.download()
        self.done()
        return r

    def matmul_bias_cast_view(self, a, b, bias, split_shape, perms):
        """The product written through the view that RESHAPE(split_shape) -> TRANSPOSE(perms) behind it amounts to;
        split_shape has six extents [NB1, NB2, M1, M2, N1, N2].  Returns the transposed tensor."""
        ta, tb = self.put(a), self.put(b)
        tbias = self.put(bias) if bias is not None else None
        moved_shape = tuple(split_shape[p] for p in perms)
        to = self.new(abi.F16, moved_shape)
        moved_strides = abi.packed_strides(moved_shape, 2)
        strides = [0] * 6
        for k, p in enumerate(perms):
            strides[p] = moved_strides[k]
        view = abi.make_tensor(to.view.ptr, abi.F16, split_shape, strides)
        self.dev.op("matmul_bias_cast", C.byref(view), ta.ref, tb.ref, tbias.ref if tbias else None,
                    C.byref(abi.MatmulAttr(0, 0)))
        r = to.download()
        self.done()
        return r

    def matmul_bias_cast_chain(self, a, b, bias, inputs, steps, b_rows=False):
        """The fused product followed by an elementwise chain whose value 0 is the product; `inputs`: the chain's
        other inputs."""
        ta, tb = self.put(a), self._b_operand(b, b_rows)
        tbias = self.put(bias) if bias is not None else None
        tin = [self.put(x) for x in inputs]
        to = self.new(abi.F16, (a.shape[0], a.shape[1], b.shape[2]))
        c = abi.Chain()
        c.n_inputs, c.n_steps = len(tin) + 1, len(steps)
        for i, t in enumerate(tin):
            c.inputs[i + 1] = C.pointer(t.view)
        for i, st in enumerate(steps):
            c.steps[i] = abi.ChainStep(*[int(v) for v in st])
        self.dev.op("matmul_bias_cast_chain", to.ref, ta.ref, C.byref(tb), tbias.ref if tbias else None,
                    C.byref(abi.MatmulAttr(0, 0)), C.byref(c))
        r = to.download()
        self.done()
        return r

    def matmul_bias_cast_group(self, a, bs, biases, b_rows=False):
        """Several fused products of one `a` in one call; returns the list of results."""
        ta = self.put(a)
        tbs = [self._b_operand(b, b_rows) for b in bs]
        tbias = [self.put(x) if x is not None else None for x in biases]
        touts = [self.new(abi.F16, (a.shape[0], a.shape[1], b.shape[2])) for b in bs]
        products = (abi.MatmulProduct * len(bs))()
        for i in range(len(bs)):
            products[i] = abi.MatmulProduct(C.pointer(touts[i].view), C.pointer(tbs[i]),
                                            C.pointer(tbias[i].view) if tbias[i] else None)
        self.dev.op("matmul_bias_cast_group", products, len(bs), ta.ref, C.byref(abi.MatmulAttr(0, 0)))
        r = [t.download() for t in touts]
        self.done()
        return r

    def matmul_bias_cast_add(self, a, b, bias, residual, b_rows=False):
        ta, tb, tr = self.put(a), self._b_operand(b, b_rows), self.put(residual)
        tbias = self.put(bias) if bias is not None else None
        to = self.new(abi.F16, (a.shape[0], a.shape[1], b.shape[2]))
        self.dev.op("matmul_bias_cast_add", to.ref, ta.ref, C.byref(tb), tbias.ref if tbias else None,
                    C.byref(abi.MatmulAttr(0, 0)), tr.ref)
        r = to.download()
        self.done()
        return r

    def attention(self, q, kt, v, chain_inputs, steps, split_shape=None, perms=None):
        """mlel_hip_attention_f16: `chain_inputs` are the softmax chain's inputs from 1 on (the scale, if any);
        with split_shape / perms the result goes through the view of a RESHAPE -> TRANSPOSE behind it."""
        tq, tk, tv = self.put(q), self.put(kt), self.put(v)
        tin = [self.put(x) for x in chain_inputs]
        c = abi.Chain()
        c.n_inputs, c.n_steps = len(tin) + 1, len(steps)
        for i, t in enumerate(tin):
            c.inputs[i + 1] = C.pointer(t.view)
        for i, st in enumerate(steps):
            c.steps[i] = abi.ChainStep(*[int(x) for x in st])
        shape = (q.shape[0], q.shape[1], v.shape[2])
        if split_shape is None:
            to = self.new(abi.F16, shape)
            self.dev.op("attention_f16", to.ref, tq.ref, tk.ref, tv.ref, C.byref(c))
        else:
            moved_shape = tuple(split_shape[p] for p in perms)
            to = self.new(abi.F16, moved_shape)
            moved_strides = abi.packed_strides(moved_shape, 2)
            strides = [0] * 6
            for k, p in enumerate(perms):
                strides[p] = moved_strides[k]
            view = abi.make_tensor(to.view.ptr, abi.F16, split_shape, strides)
            self.dev.op("attention_f16", C.byref(view), tq.ref, tk.ref, tv.ref, C.byref(c))
        r = to.download()
        self.done()
        return r

    def chain(self, inputs, steps, out_shape, out_dtype):
        """steps: (kind, selector, a, b, dtype) tuples as in mlel_chain_step."""
        tin = [self.put(x) for x in inputs]
        to = self.new(out_dtype, out_shape)
        c = abi.Chain()
        c.n_inputs, c.n_steps = len(tin), len(steps)
        for i, t in enumerate(tin):
            c.inputs[i] = C.pointer(t.view)
        for i, st in enumerate(steps):
            c.steps[i] = abi.ChainStep(*[int(v) for v in st])
        self.dev.op("elementwise_chain", to.ref, C.byref(c))
        r = to.download()
        self.done()
        return r

    # ---- the operators outside the benchmark graphs ------------------------------------------------------------
    def call(self, name, out_specs, inputs, *attrs):
        """Generic form: uploads `inputs`, allocates one output per (dtype, shape) in `out_specs`, calls
        mlel_hip_<name>(outputs..., inputs..., attrs...) and returns the downloaded outputs."""
        outs = [self.new(dt, shape) for dt, shape in out_specs]
        ins = [self.put(x) for x in inputs]
        self.dev.op(name, *[t.ref for t in outs], *[t.ref for t in ins], *attrs)
        result = [t.download() for t in outs]
        self.done()
        return result if len(result) > 1 else result[0]

    def argmax(self, x, axis, nan_mode=abi.NAN_PROPAGATE):
        shape = [d for i, d in enumerate(x.shape) if i != axis]
        return self.call("argmax", [(abi.I32, shape)], [x], int(axis), int(nan_mode))

    def arithmetic_right_shift(self, a, b, out_shape, round_=False):
        return self.call("arithmetic_right_shift", [(abi.dtype_of_array(a), out_shape)], [a, b], 1 if round_ else 0)

    def conv3d(self, x, w, b, out_shape, out_dtype, attr):
        return self.call("conv3d", [(out_dtype, out_shape)], [x, w, b], C.byref(attr))

    def transpose_conv2d(self, x, w, b, out_shape, out_dtype, attr):
        return self.call("transpose_conv2d", [(out_dtype, out_shape)], [x, w, b], C.byref(attr))

    def fft2d(self, real, imag, inverse=False):
        return self.call("fft2d", [(abi.F32, real.shape), (abi.F32, real.shape)], [real, imag], 1 if inverse else 0)

    def rfft2d(self, x):
        shape = (x.shape[0], x.shape[1], x.shape[2] // 2 + 1)
        return self.call("rfft2d", [(abi.F32, shape), (abi.F32, shape)], [x])

    def gather(self, values, indices):
        shape = (values.shape[0], indices.shape[1], values.shape[2])
        return self.call("gather", [(abi.dtype_of_array(values), shape)], [values, indices])

    def scatter(self, values_in, indices, input_):
        return self.call("scatter", [(abi.dtype_of_array(values_in), values_in.shape)], [values_in, indices, input_])

    def resize(self, x, out_shape, out_dtype, attr):
        return self.call("resize", [(out_dtype, out_shape)], [x], C.byref(attr))

    def reverse(self, x, axis):
        return self.call("reverse", [(abi.dtype_of_array(x), x.shape)], [x], int(axis))

    def tile(self, x, out_shape):
        return self.call("tile", [(abi.dtype_of_array(x), out_shape)], [x])

    def select(self, cond, a, b, out_shape):
        return self.call("select", [(abi.dtype_of_array(a), out_shape)], [cond, a, b])
