"""numpy front-end of the CPU oracle (oracle/libmlel_oracle.so).  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module; the product
path (the HIP backend) never does.  Each function allocates a zero-filled output, wraps host numpy buffers
in mlel_tensor views and calls the C restatement of one reference shader (see oracle/mlel_oracle.h).
"""
import ctypes as C
import importlib
import os
import subprocess

import numpy as np

_here = os.path.dirname(os.path.abspath(__file__))
abi = importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.abi")

_lib = None


def _bind(lib):
    """ctypes signatures of the oracle's mlel_cpu_* table: the operator argument lists are those of the C ABI."""
    for name, args in abi.OP_SIGNATURES.items():
        fn = getattr(lib, "mlel_cpu_" + name)
        fn.restype = C.c_int
        fn.argtypes = args
    lib.mlel_cpu_last_error.restype = C.c_char_p
    lib.mlel_cpu_num_threads.restype = C.c_int
    lib.mlel_cpu_f32_to_f16.restype = C.c_uint16
    lib.mlel_cpu_f32_to_f16.argtypes = [C.c_float]
    lib.mlel_cpu_f16_to_f32.restype = C.c_float
    lib.mlel_cpu_f16_to_f32.argtypes = [C.c_uint16]
    lib.mlel_cpu_f32_to_bf16.restype = C.c_uint16
    lib.mlel_cpu_f32_to_bf16.argtypes = [C.c_float, C.c_int]
    lib.mlel_cpu_f32_to_f8.restype = C.c_uint8
    lib.mlel_cpu_f32_to_f8.argtypes = [C.c_float, C.c_int]
    lib.mlel_cpu_f8_to_f32.restype = C.c_float
    lib.mlel_cpu_f8_to_f32.argtypes = [C.c_uint8, C.c_int]
    return lib


def build():
    subprocess.run(["make", "-C", _here, "-s", "-B"], check=True)


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_here, "libmlel_oracle.so")
        if not os.path.exists(path):
            build()
        _lib = _bind(C.CDLL(path))
    return _lib


class OracleError(RuntimeError):
    pass


def _view(arr, dtype=None):
    """mlel_tensor over a numpy array's own memory (honours its strides)."""
    if dtype is None:
        dtype = abi.dtype_of_array(arr)
    if arr.ndim == 0:
        arr = arr.reshape(1)
    return abi.make_tensor(arr.ctypes.data, dtype, arr.shape, arr.strides)


def _call(name, *args):
    rc = getattr(lib(), "mlel_cpu_" + name)(*args)
    if rc != 0:
        raise OracleError(f"mlel_cpu_{name}: {rc}: {lib().mlel_cpu_last_error().decode()}")


def _out(shape, dtype):
    out = np.zeros(shape, dtype=abi.NP_OF[dtype])
    return abi.typed(out, dtype) if dtype in abi.TAGGED else out


def _like(x, shape):
    """zero-filled array of `shape` with the element type of `x` (keeps a bf16 / fp8 tag)"""
    return _out(shape, abi.dtype_of_array(x))


def conv2d(x, w, bias, out_shape, out_dtype, attr, x_dtype=None, w_dtype=None):
    out = _out(out_shape, out_dtype)
    _call("conv2d", _view(out, out_dtype), _view(x, x_dtype), _view(w, w_dtype), _view(bias, out_dtype), attr)
    return out


def depthwise_conv2d(x, w, bias, out_shape, out_dtype, attr):
    out = _out(out_shape, out_dtype)
    _call("depthwise_conv2d", _view(out, out_dtype), _view(x), _view(w), _view(bias, out_dtype), attr)
    return out


def matmul(a, b, out_dtype, a_zp=0, b_zp=0):
    out = _out((a.shape[0], a.shape[1], b.shape[2]), out_dtype)
    _call("matmul", _view(out, out_dtype), _view(a), _view(b), abi.MatmulAttr(int(a_zp), int(b_zp)))
    return out


def rescale(x, multiplier, shift, out_dtype, attr, in_dtype=None):
    out = _out(x.shape, out_dtype)
    _call("rescale", _view(out, out_dtype), _view(x, in_dtype), _view(multiplier), _view(shift), attr)
    return out


def clamp(x, min_val, max_val, nan_mode=abi.NAN_PROPAGATE):
    out = np.zeros_like(x)
    _call("clamp", _view(out), _view(x), abi.ClampAttr(float(min_val), float(max_val), int(nan_mode)))
    return out


def elementwise_binary(op, a, b, out_shape, out_dtype, nan_mode=abi.NAN_PROPAGATE):
    out = _out(out_shape, out_dtype)
    _call("elementwise_binary", abi.BIN[op], _view(out, out_dtype), _view(a), _view(b), int(nan_mode))
    return out


def mul(a, b, out_shape, out_dtype, shift=0):
    out = _out(out_shape, out_dtype)
    _call("mul", _view(out, out_dtype), _view(a), _view(b), int(shift))
    return out


def elementwise_unary(op, x):
    out = np.zeros_like(x)
    _call("elementwise_unary", abi.UN[op], _view(out), _view(x))
    return out


def reduce(op, x, axis, nan_mode=abi.NAN_PROPAGATE):
    shape = list(x.shape)
    shape[axis] = 1
    out = _like(x, shape)
    _call("reduce", abi.RED[op], _view(out), _view(x), int(axis), int(nan_mode))
    return out


def avg_pool2d(x, out_shape, attr):
    out = _like(x, out_shape)
    _call("avg_pool2d", _view(out), _view(x), attr)
    return out


def max_pool2d(x, out_shape, attr):
    out = _like(x, out_shape)
    _call("max_pool2d", _view(out), _view(x), attr)
    return out


def table(x, tab, out_dtype):
    out = _out(x.shape, out_dtype)
    _call("table", _view(out, out_dtype), _view(x), _view(tab))
    return out


def cast(x, out_dtype, in_dtype=None):
    out = _out(x.shape, out_dtype)
    _call("cast", _view(out, out_dtype), _view(x, in_dtype))
    return out


def negate(x, input_zp=0, output_zp=0):
    out = np.zeros_like(x)
    _call("negate", _view(out), _view(x), int(input_zp), int(output_zp))
    return out


def reshape(x, out_shape):
    out = _like(x, out_shape)
    _call("reshape", _view(out), _view(x))
    return out


def transpose(x, perms):
    out_shape = [0] * x.ndim
    # output dim i has the extent of input dim perms[i] (reference: transpose.comp:23-26)
    for i, p in enumerate(perms):
        out_shape[i] = x.shape[p]
    out = _like(x, out_shape)
    arr = (C.c_uint32 * abi.MAX_RANK)(*[int(p) for p in perms])
    _call("transpose", _view(out), _view(x), arr)
    return out


def concat(inputs, axis):
    shape = list(inputs[0].shape)
    shape[axis] = sum(i.shape[axis] for i in inputs)
    out = _like(inputs[0], shape)
    offset = 0
    for i in inputs:
        _call("concat", _view(out), _view(i), int(axis), int(offset))
        offset += i.shape[axis]
    return out


def slice_(x, start, size):
    out = _like(x, size)
    arr = (C.c_uint32 * abi.MAX_RANK)(*[int(p) for p in start])
    _call("slice", _view(out), _view(x), arr)
    return out


def pad(x, padding, out_shape, pad_const=0.0, pad_const_int=0):
    out = _like(x, out_shape)
    padding = np.ascontiguousarray(padding, dtype=np.int32).reshape(-1)
    _call("pad", _view(out), _view(x), _view(padding), float(pad_const), int(pad_const_int))
    return out


def argmax(x, axis, nan_mode=abi.NAN_PROPAGATE):
    shape = [d for i, d in enumerate(x.shape) if i != axis]
    out = np.zeros(shape, dtype=np.int32)
    _call("argmax", _view(out), _view(x), int(axis), int(nan_mode))
    return out


def arithmetic_right_shift(a, b, out_shape, round_=False):
    out = _like(a, out_shape)
    _call("arithmetic_right_shift", _view(out), _view(a), _view(b), 1 if round_ else 0)
    return out


def conv3d(x, w, bias, out_shape, out_dtype, attr):
    out = _out(out_shape, out_dtype)
    _call("conv3d", _view(out, out_dtype), _view(x), _view(w), _view(bias, out_dtype), attr)
    return out


def transpose_conv2d(x, w, bias, out_shape, out_dtype, attr):
    out = _out(out_shape, out_dtype)
    _call("transpose_conv2d", _view(out, out_dtype), _view(x), _view(w), _view(bias, out_dtype), attr)
    return out


def fft2d(real, imag, inverse=False):
    out_r, out_i = np.zeros_like(real), np.zeros_like(imag)
    _call("fft2d", _view(out_r), _view(out_i), _view(real), _view(imag), 1 if inverse else 0)
    return out_r, out_i


def rfft2d(x):
    shape = (x.shape[0], x.shape[1], x.shape[2] // 2 + 1)
    out_r, out_i = np.zeros(shape, np.float32), np.zeros(shape, np.float32)
    _call("rfft2d", _view(out_r), _view(out_i), _view(x))
    return out_r, out_i


def gather(values, indices):
    out = _like(values, (values.shape[0], indices.shape[1], values.shape[2]))
    _call("gather", _view(out), _view(values), _view(indices))
    return out


def scatter(values_in, indices, input_):
    out = np.zeros_like(values_in)
    _call("scatter", _view(out), _view(values_in), _view(indices), _view(input_))
    return out


def resize(x, out_shape, out_dtype, attr):
    out = _out(out_shape, out_dtype)
    _call("resize", _view(out, out_dtype), _view(x), attr)
    return out


def reverse(x, axis):
    out = np.zeros_like(x)
    _call("reverse", _view(out), _view(x), int(axis))
    return out


def tile(x, out_shape):
    out = _like(x, out_shape)
    _call("tile", _view(out), _view(x))
    return out


def select(cond, a, b, out_shape):
    out = _like(a, out_shape)
    _call("select", _view(out), _view(cond, abi.BOOL), _view(a), _view(b))
    return out


def num_threads():
    return lib().mlel_cpu_num_threads()
