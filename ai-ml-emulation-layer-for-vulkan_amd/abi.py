"""ctypes mirror of include/mlel_hip.h (and of oracle/mlel_oracle.h, which shares its structs).

This module only describes the C ABI; it contains no arithmetic.  The HIP library is the product, the
oracle library is test infrastructure and is loaded only on request (tests, smoke check, CPU baseline).
"""
import ctypes as C
import os

import numpy as np

MAX_RANK = 6

# mlel_dtype
BOOL, I8, U8, I16, U16, I32, U32, I64, U64, F16, BF16, F32, F64, F8E4M3, F8E5M2 = range(15)

DTYPE_SIZE = {BOOL: 1, I8: 1, U8: 1, I16: 2, U16: 2, I32: 4, U32: 4, I64: 8, U64: 8, F16: 2, BF16: 2, F32: 4,
              F64: 8, F8E4M3: 1, F8E5M2: 1}
DTYPE_NAME = {BOOL: "bool", I8: "i8", U8: "u8", I16: "i16", U16: "u16", I32: "i32", U32: "u32", I64: "i64",
              U64: "u64", F16: "f16", BF16: "bf16", F32: "f32", F64: "f64", F8E4M3: "f8e4m3", F8E5M2: "f8e5m2"}
NP_OF = {BOOL: np.bool_, I8: np.int8, U8: np.uint8, I16: np.int16, U16: np.uint16, I32: np.int32, U32: np.uint32,
         I64: np.int64, U64: np.uint64, F16: np.float16, BF16: np.uint16, F32: np.float32, F64: np.float64,
         F8E4M3: np.uint8, F8E5M2: np.uint8}
_OF_NP = {np.dtype(np.bool_): BOOL, np.dtype(np.int8): I8, np.dtype(np.uint8): U8, np.dtype(np.int16): I16,
          np.dtype(np.uint16): U16, np.dtype(np.int32): I32, np.dtype(np.uint32): U32, np.dtype(np.int64): I64,
          np.dtype(np.uint64): U64, np.dtype(np.float16): F16, np.dtype(np.float32): F32,
          np.dtype(np.float64): F64}

ACC_I32, ACC_F16, ACC_F32, ACC_I64 = 1, 2, 3, 4
NAN_PROPAGATE, NAN_IGNORE = 1, 2
ROUND_SINGLE, ROUND_INEXACT, ROUND_DOUBLE = 1, 2, 3

OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_DEVICE, ERR_LIMIT = 0, -1, -2, -3, -4

BIN_OPS = ["ADD", "SUB", "BITWISE_AND", "BITWISE_OR", "BITWISE_XOR", "INTDIV", "LOGICAL_AND", "LOGICAL_OR",
           "LOGICAL_XOR", "LOGICAL_LEFT_SHIFT", "LOGICAL_RIGHT_SHIFT", "MAXIMUM", "MINIMUM", "POW", "EQUAL",
           "GREATER", "GREATER_EQUAL"]
UN_OPS = ["ABS", "BITWISE_NOT", "CEIL", "CLZ", "COS", "ERF", "EXP", "FLOOR", "LOG", "LOGICAL_NOT", "RECIPROCAL",
          "RSQRT", "SIGMOID", "SIN", "TANH"]
RED_OPS = ["ALL", "ANY", "MAX", "MIN", "PRODUCT", "SUM"]
BIN = {n: i for i, n in enumerate(BIN_OPS)}
UN = {n: i for i, n in enumerate(UN_OPS)}
RED = {n: i for i, n in enumerate(RED_OPS)}


def dtype_of_numpy(dt):
    return _OF_NP[np.dtype(dt)]


TAGGED = (BF16, F8E4M3, F8E5M2)  # element types carried in an unsigned integer array with a tag


class Typed(np.ndarray):
    """A numpy array that carries the element type of a format numpy has no dtype for: bf16 lives in uint16 words, the
    fp8 encodings in uint8 bytes.  Views, slices and `zeros_like` keep the tag."""

    def __array_finalize__(self, obj):
        self.mlel_dtype = getattr(obj, "mlel_dtype", None)


def typed(arr, dtype):
    """Tag `arr` (uint16 words for BF16, uint8 bytes for F8E4M3 / F8E5M2) with its element type."""
    arr = np.asarray(arr)
    assert arr.dtype == NP_OF[dtype], (arr.dtype, dtype)
    v = arr.view(Typed)
    v.mlel_dtype = dtype
    return v


def dtype_of_array(arr):
    tag = getattr(arr, "mlel_dtype", None)
    return tag if tag is not None else dtype_of_numpy(arr.dtype)


class Tensor(C.Structure):
    """struct mlel_tensor"""
    _fields_ = [("ptr", C.c_void_p), ("dtype", C.c_int32), ("rank", C.c_int32), ("dims", C.c_int64 * MAX_RANK),
                ("strides", C.c_int64 * MAX_RANK)]


class Conv2dAttr(C.Structure):
    _fields_ = [("input_zp", C.c_int32), ("weight_zp", C.c_int32), ("pad", C.c_int32 * 4),
                ("stride", C.c_int32 * 2), ("dilation", C.c_int32 * 2), ("acc_type", C.c_uint32)]


class Conv3dAttr(C.Structure):
    _fields_ = [("input_zp", C.c_int32), ("weight_zp", C.c_int32), ("pad", C.c_int32 * 6),
                ("stride", C.c_int32 * 3), ("dilation", C.c_int32 * 3), ("acc_type", C.c_uint32)]


class Tconv2dAttr(C.Structure):
    _fields_ = [("input_zp", C.c_int32), ("weight_zp", C.c_int32), ("out_pad", C.c_int32 * 4),
                ("stride", C.c_int32 * 2), ("acc_type", C.c_uint32)]


class ResizeAttr(C.Structure):
    _fields_ = [("scale", C.c_int32 * 4), ("offset", C.c_int32 * 2), ("border", C.c_int32 * 2), ("mode", C.c_uint32)]


class MatmulProduct(C.Structure):
    _fields_ = [("out", C.POINTER(Tensor)), ("b", C.POINTER(Tensor)), ("bias", C.POINTER(Tensor))]


class ChainStep(C.Structure):
    _fields_ = [("kind", C.c_int32), ("selector", C.c_int32), ("a", C.c_int32), ("b", C.c_int32), ("dtype", C.c_int32)]


class Chain(C.Structure):
    _fields_ = [("n_inputs", C.c_int32), ("n_steps", C.c_int32), ("inputs", C.POINTER(Tensor) * 8),
                ("steps", ChainStep * 24)]


class MatmulAttr(C.Structure):
    _fields_ = [("a_zp", C.c_int32), ("b_zp", C.c_int32)]


class RescaleAttr(C.Structure):
    _fields_ = [("input_zp", C.c_int32), ("output_zp", C.c_int32), ("scale32", C.c_uint32),
                ("double_round", C.c_uint32), ("per_channel", C.c_uint32), ("input_unsigned", C.c_uint32),
                ("output_unsigned", C.c_uint32)]


class ClampAttr(C.Structure):
    _fields_ = [("min_val", C.c_double), ("max_val", C.c_double), ("nan_mode", C.c_uint32)]


class Pool2dAttr(C.Structure):
    _fields_ = [("kernel", C.c_int32 * 2), ("stride", C.c_int32 * 2), ("pad", C.c_int32 * 4),
                ("input_zp", C.c_int32), ("output_zp", C.c_int32), ("acc_type", C.c_uint32),
                ("nan_mode", C.c_uint32)]


class Epilogue(C.Structure):
    _fields_ = [("multiplier", C.POINTER(Tensor)), ("shift", C.POINTER(Tensor)), ("rescale", RescaleAttr),
                ("has_clamp", C.c_int32), ("clamp", ClampAttr)]


def conv2d_attr(pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), input_zp=0, weight_zp=0, acc_type=ACC_I32):
    a = Conv2dAttr()
    a.input_zp, a.weight_zp, a.acc_type = int(input_zp), int(weight_zp), int(acc_type)
    a.pad[:] = [int(v) for v in pad]
    a.stride[:] = [int(v) for v in stride]
    a.dilation[:] = [int(v) for v in dilation]
    return a


def conv3d_attr(pad=(0,) * 6, stride=(1, 1, 1), dilation=(1, 1, 1), input_zp=0, weight_zp=0, acc_type=ACC_I32):
    a = Conv3dAttr()
    a.input_zp, a.weight_zp, a.acc_type = input_zp, weight_zp, acc_type
    a.pad[:] = list(pad)
    a.stride[:] = list(stride)
    a.dilation[:] = list(dilation)
    return a


def tconv2d_attr(out_pad=(0, 0, 0, 0), stride=(1, 1), input_zp=0, weight_zp=0, acc_type=ACC_I32):
    a = Tconv2dAttr()
    a.input_zp, a.weight_zp, a.acc_type = input_zp, weight_zp, acc_type
    a.out_pad[:] = list(out_pad)
    a.stride[:] = list(stride)
    return a


def resize_attr(scale, offset=(0, 0), border=(0, 0), mode=1):
    a = ResizeAttr()
    a.scale[:] = list(scale)
    a.offset[:] = list(offset)
    a.border[:] = list(border)
    a.mode = mode
    return a


def rescale_attr(input_zp=0, output_zp=0, scale32=True, double_round=False, per_channel=False,
                 input_unsigned=False, output_unsigned=False):
    return RescaleAttr(int(input_zp), int(output_zp), int(scale32), int(double_round), int(per_channel),
                       int(input_unsigned), int(output_unsigned))


def pool2d_attr(kernel, stride, pad, input_zp=0, output_zp=0, acc_type=ACC_I32, nan_mode=NAN_PROPAGATE):
    a = Pool2dAttr()
    a.kernel[:] = [int(v) for v in kernel]
    a.stride[:] = [int(v) for v in stride]
    a.pad[:] = [int(v) for v in pad]
    a.input_zp, a.output_zp, a.acc_type, a.nan_mode = int(input_zp), int(output_zp), int(acc_type), int(nan_mode)
    return a


def packed_strides(dims, elem_size):
    """Row-major byte strides (reference: tensor/tensor_arm.cpp:82-92)."""
    strides = [0] * len(dims)
    s = elem_size
    for i in range(len(dims) - 1, -1, -1):
        strides[i] = s
        s *= int(dims[i])
    return strides


def make_tensor(ptr, dtype, dims, strides=None):
    t = Tensor()
    t.ptr = ptr
    t.dtype = int(dtype)
    t.rank = len(dims)
    if strides is None:
        strides = packed_strides(dims, DTYPE_SIZE[int(dtype)])
    for i, (d, s) in enumerate(zip(dims, strides)):
        t.dims[i] = int(d)
        t.strides[i] = int(s)
    return t


_T = C.POINTER(Tensor)
_V = C.c_void_p

# name -> (argtypes after the (ctx, stream) prefix of the HIP ABI); the oracle has the same list w/o prefix
OP_SIGNATURES = {
    "conv2d": [_T, _T, _T, _T, C.POINTER(Conv2dAttr)],
    "depthwise_conv2d": [_T, _T, _T, _T, C.POINTER(Conv2dAttr)],
    "matmul": [_T, _T, _T, C.POINTER(MatmulAttr)],
    "rescale": [_T, _T, _T, _T, C.POINTER(RescaleAttr)],
    "clamp": [_T, _T, C.POINTER(ClampAttr)],
    "elementwise_binary": [C.c_int32, _T, _T, _T, C.c_uint32],
    "mul": [_T, _T, _T, C.c_uint32],
    "elementwise_unary": [C.c_int32, _T, _T],
    "reduce": [C.c_int32, _T, _T, C.c_uint32, C.c_uint32],
    "avg_pool2d": [_T, _T, C.POINTER(Pool2dAttr)],
    "max_pool2d": [_T, _T, C.POINTER(Pool2dAttr)],
    "table": [_T, _T, _T],
    "cast": [_T, _T],
    "negate": [_T, _T, C.c_int32, C.c_int32],
    "reshape": [_T, _T],
    "transpose": [_T, _T, C.POINTER(C.c_uint32)],
    "concat": [_T, _T, C.c_uint32, C.c_uint32],
    "slice": [_T, _T, C.POINTER(C.c_uint32)],
    "pad": [_T, _T, _T, C.c_double, C.c_int32],
    "argmax": [_T, _T, C.c_uint32, C.c_uint32],
    "arithmetic_right_shift": [_T, _T, _T, C.c_uint32],
    "conv3d": [_T, _T, _T, _T, C.POINTER(Conv3dAttr)],
    "transpose_conv2d": [_T, _T, _T, _T, C.POINTER(Tconv2dAttr)],
    "fft2d": [_T, _T, _T, _T, C.c_int32],
    "rfft2d": [_T, _T, _T],
    "gather": [_T, _T, _T],
    "scatter": [_T, _T, _T, _T],
    "resize": [_T, _T, C.POINTER(ResizeAttr)],
    "reverse": [_T, _T, C.c_uint32],
    "tile": [_T, _T],
    "select": [_T, _T, _T, _T],
}

FUSED_SIGNATURES = {
    "conv2d_rescale_clamp": [_T, _T, _T, _T, C.POINTER(Conv2dAttr), C.POINTER(Epilogue)],
    "conv2d_rescale_clamp_static": [_T, _T, _T, _T, C.POINTER(Conv2dAttr), C.POINTER(Epilogue)],
    "conv2d_rescale_add_rescale": [_T, _T, _T, _T, C.POINTER(Conv2dAttr), C.POINTER(Epilogue), C.POINTER(Epilogue), _T,
                                   C.POINTER(Epilogue), C.POINTER(Epilogue), C.c_int],
    "matmul_rescale": [_T, _T, _T, C.POINTER(MatmulAttr), C.POINTER(Epilogue)],
    "dwconv_rescale_clamp": [_T, _T, _T, _T, C.POINTER(Conv2dAttr), C.POINTER(Epilogue)],
    "conv2d_dwconv_rescale_clamp": [_T, _T, _T, _T, C.POINTER(Conv2dAttr), C.POINTER(Epilogue), _T, _T,
                                    C.POINTER(Conv2dAttr), C.POINTER(Epilogue)],
    "conv2d_conv2d_rescale_clamp": [_T, _T, _T, _T, _T, C.POINTER(Conv2dAttr), C.POINTER(Epilogue), _T, _T,
                                    C.POINTER(Conv2dAttr), C.POINTER(Epilogue)],
    "conv2d_rescale_clamp_avgpool": [_T, _T, _T, _T, C.POINTER(Conv2dAttr), C.POINTER(Epilogue), C.c_int32,
                                     C.POINTER(Pool2dAttr)],
    "matmul_bias_cast": [_T, _T, _T, _T, C.POINTER(MatmulAttr)],
    "matmul_bias_cast_add": [_T, _T, _T, _T, C.POINTER(MatmulAttr), _T],
    "matmul_bias_cast_group": [C.POINTER(MatmulProduct), C.c_int, _T, C.POINTER(MatmulAttr)],
    "softmax_rows": [_T, _T],
    "elementwise_chain": [_T, C.POINTER(Chain)],
    "matmul_bias_cast_chain": [_T, _T, _T, _T, C.POINTER(MatmulAttr), C.POINTER(Chain)],
    "attention_f16": [_T, _T, _T, _T, C.POINTER(Chain)],
    "rescale_add_rescale": [_T, _T, C.POINTER(Epilogue), _T, C.POINTER(Epilogue), C.POINTER(Epilogue)],
}

# every other symbol include/mlel_hip.h declares: name -> (restype, argtypes)
RUNTIME_SIGNATURES = {
    "mlel_hip_last_error": (C.c_char_p, []),
    "mlel_hip_device_count": (C.c_int, []),
    "mlel_hip_init": (C.c_int, [C.c_int, C.POINTER(_V)]),
    "mlel_hip_destroy": (None, [_V]),
    "mlel_hip_device_info": (C.c_int, [_V, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                       C.POINTER(C.c_int32), C.c_char_p, C.c_size_t]),
    "mlel_hip_static_scratch_last_use": (C.c_int, [_V]),
    "mlel_hip_split_workspaces": (C.c_int, [_V]),
    "mlel_hip_arena_alloc": (C.c_int, [_V, C.c_size_t, C.POINTER(_V)]),
    "mlel_hip_arena_free": (C.c_int, [_V, _V]),
    "mlel_hip_arena_import_fd": (C.c_int, [_V, C.c_int, C.c_size_t, C.POINTER(_V), C.POINTER(_V)]),
    "mlel_hip_arena_release_import": (C.c_int, [_V, _V]),
    "mlel_hip_memcpy_h2d": (C.c_int, [_V, _V, _V, C.c_size_t, _V]),
    "mlel_hip_memcpy_d2h": (C.c_int, [_V, _V, _V, C.c_size_t, _V]),
    "mlel_hip_memcpy_d2d": (C.c_int, [_V, _V, _V, C.c_size_t, _V]),
    "mlel_hip_memset": (C.c_int, [_V, _V, C.c_int, C.c_size_t, _V]),
    "mlel_hip_stream_create": (C.c_int, [_V, C.POINTER(_V)]),
    "mlel_hip_stream_destroy": (C.c_int, [_V, _V]),
    "mlel_hip_sync": (C.c_int, [_V, _V]),
    "mlel_hip_event_create": (C.c_int, [_V, C.POINTER(_V)]),
    "mlel_hip_event_destroy": (C.c_int, [_V, _V]),
    "mlel_hip_event_record": (C.c_int, [_V, _V, _V]),
    "mlel_hip_stream_wait_event": (C.c_int, [_V, _V, _V]),
    "mlel_hip_event_elapsed_ms": (C.c_int, [_V, _V, _V, C.POINTER(C.c_float)]),
    "mlel_hip_capture_begin": (C.c_int, [_V, _V]),
    "mlel_hip_capture_end": (C.c_int, [_V, _V, C.POINTER(_V)]),
    "mlel_hip_graph_launch": (C.c_int, [_V, _V, _V]),
    "mlel_hip_graph_destroy": (C.c_int, [_V, _V]),
    "mlel_hip_copy_kernel": (C.c_int, [_V, _V, _V, _V, C.c_size_t]),
    "mlel_hip_mfma_rate_probe": (C.c_int, [_V, _V, _V, _V, C.c_int, C.c_int]),
    "mlel_hip_issue_probe": (C.c_int, [_V, _V, _V, _V, C.c_int, C.c_int]),
    "mlel_hip_copy_kernel_variant": (C.c_int, [_V, _V, _V, _V, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int]),
    "mlel_hip_matmul_chain_in_kernel": (C.c_int, [C.POINTER(Chain)]),
    "mlel_hip_attention_f16_in_kernel": (C.c_int, [_T, _T, _T, _T, C.POINTER(Chain)]),
    "mlel_hip_conv2d_dwconv_in_kernel": (C.c_int, [_T, _T, _T, _T, C.POINTER(Conv2dAttr), _T, _T,
                                                   C.POINTER(Conv2dAttr)]),
    "mlel_hip_conv2d_conv2d_in_kernel": (C.c_int, [_T, _T, _T, _T, C.POINTER(Conv2dAttr), _T, _T,
                                                   C.POINTER(Conv2dAttr)]),
    "mlel_hip_conv2d_avgpool_in_kernel": (C.c_int, [_T, _T, _T, _T, C.POINTER(Conv2dAttr), C.c_int32,
                                                    C.POINTER(Pool2dAttr)]),
}


def hip_symbol_names():
    """All symbols include/mlel_hip.h declares."""
    names = list(RUNTIME_SIGNATURES)
    names += ["mlel_hip_" + n for n in OP_SIGNATURES]
    names += ["mlel_hip_" + n for n in FUSED_SIGNATURES]
    return names


def bind_hip(lib):
    for name, (res, args) in RUNTIME_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    for table in (OP_SIGNATURES, FUSED_SIGNATURES):
        for name, args in table.items():
            fn = getattr(lib, "mlel_hip_" + name)
            fn.restype = C.c_int
            fn.argtypes = [_V, _V] + args
    return lib


REPO_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIP_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libmlel_hip.so")
GRAPH_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libmlel_graph.so")
