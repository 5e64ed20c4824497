"""Thin ctypes harness over libmlel_hip.so (the C ABI of include/mlel_hip.h).

It mirrors the reference's test-side helpers (utilities/tensor.cpp: zero-filled tensors with packed row-major
strides; utilities/pipeline.cpp: dispatch then wait) and nothing more: every operator call goes to a HIP kernel
through the C ABI, errors surface as MlelError, and there is no CPU fallback.
"""
import ctypes as C
import os

import numpy as np

from . import abi


class MlelError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"mlel_hip error {code}: {message}")
        self.code = code


_lib = None


def load_library():
    """Loads the prebuilt in-tree library; fails loudly when it is missing (build with __graft_entry__.build())."""
    global _lib
    if _lib is None:
        if not os.path.exists(abi.HIP_LIB_PATH):
            raise MlelError(abi.ERR_DEVICE, f"{abi.HIP_LIB_PATH} is not built; run `python -c 'import "
                            "__graft_entry__ as g; g.build()'` (needs hipcc)")
        _lib = abi.bind_hip(C.CDLL(abi.HIP_LIB_PATH))
    return _lib


def device_count():
    return load_library().mlel_hip_device_count()


class DeviceTensor:
    """Device allocation + tensor view; zero-filled at creation, packed strides unless given."""

    def __init__(self, dev, dtype, shape, strides=None, data=None):
        self.dev = dev
        self.dtype = int(dtype)
        self.shape = tuple(int(d) for d in shape)
        esize = abi.DTYPE_SIZE[self.dtype]
        self.strides = tuple(strides) if strides is not None else tuple(abi.packed_strides(self.shape, esize))
        if len(self.shape) == 0:
            raise ValueError("rank 0 tensors are not supported")
        self.nbytes = max(int(self.shape[0] * self.strides[0]), esize) if all(self.shape) else esize
        self.ptr = dev.alloc(self.nbytes)
        self.view = abi.make_tensor(self.ptr, self.dtype, self.shape, self.strides)
        if data is not None:
            self.upload(data)

    @property
    def ref(self):
        return C.byref(self.view)

    def _is_packed(self):
        return list(self.strides) == abi.packed_strides(self.shape, abi.DTYPE_SIZE[self.dtype])

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        if arr.dtype != np.dtype(abi.NP_OF[self.dtype]) and arr.dtype.itemsize == abi.DTYPE_SIZE[self.dtype]:
            arr = arr.view(abi.NP_OF[self.dtype])
        assert arr.dtype == np.dtype(abi.NP_OF[self.dtype]), (arr.dtype, self.dtype)
        assert tuple(arr.shape) == self.shape, (arr.shape, self.shape)
        if self._is_packed():
            self.dev.h2d(self.ptr, arr.ctypes.data, arr.nbytes)
        else:
            raw = np.zeros(self.nbytes, np.uint8)
            v = np.lib.stride_tricks.as_strided(np.frombuffer(raw.data, dtype=arr.dtype,
                                                              count=self.nbytes // arr.dtype.itemsize),
                                                shape=self.shape, strides=self.strides, writeable=True)
            v[...] = arr
            self.dev.h2d(self.ptr, raw.ctypes.data, self.nbytes)

    def download(self):
        npdt = np.dtype(abi.NP_OF[self.dtype])
        if self._is_packed():
            out = np.empty(self.shape, npdt)
            if out.nbytes:
                self.dev.d2h(out.ctypes.data, self.ptr, out.nbytes)
            return out
        raw = np.zeros(self.nbytes, np.uint8)
        self.dev.d2h(raw.ctypes.data, self.ptr, self.nbytes)
        v = np.lib.stride_tricks.as_strided(np.frombuffer(raw.data, dtype=npdt, count=self.nbytes // npdt.itemsize),
                                            shape=self.shape, strides=self.strides)
        return np.array(v)

    def free(self):
        if self.ptr:
            self.dev.free(self.ptr)
            self.ptr = None


class Device:
    """One mlel_ctx on one GPU."""

    def __init__(self, index=0):
        self.lib = load_library()
        ctx = C.c_void_p()
        self._check(self.lib.mlel_hip_init(index, C.byref(ctx)))
        self.ctx = ctx
        self.stream = None  # NULL stream

    def _check(self, rc):
        if rc != 0:
            raise MlelError(rc, self.lib.mlel_hip_last_error().decode(errors="replace"))

    def close(self):
        if self.ctx:
            self.lib.mlel_hip_destroy(self.ctx)
            self.ctx = None

    # ---- memory
    def alloc(self, nbytes):
        p = C.c_void_p()
        self._check(self.lib.mlel_hip_arena_alloc(self.ctx, int(nbytes), C.byref(p)))
        return p.value

    def free(self, ptr):
        self._check(self.lib.mlel_hip_arena_free(self.ctx, C.c_void_p(ptr)))

    def h2d(self, dptr, hptr, nbytes):
        self._check(self.lib.mlel_hip_memcpy_h2d(self.ctx, C.c_void_p(dptr), C.c_void_p(hptr), int(nbytes),
                                                 self.stream))

    def d2h(self, hptr, dptr, nbytes):
        self._check(self.lib.mlel_hip_memcpy_d2h(self.ctx, C.c_void_p(hptr), C.c_void_p(dptr), int(nbytes),
                                                 self.stream))

    def sync(self):
        self._check(self.lib.mlel_hip_sync(self.ctx, self.stream))

    def info(self):
        cu, clk, mclk, bus = C.c_int32(), C.c_int32(), C.c_int32(), C.c_int32()
        name = C.create_string_buffer(256)
        self._check(self.lib.mlel_hip_device_info(self.ctx, C.byref(cu), C.byref(clk), C.byref(mclk), C.byref(bus),
                                                  name, 256))
        return {"compute_units": cu.value, "clock_khz": clk.value, "mem_clock_khz": mclk.value,
                "bus_width_bits": bus.value, "name": name.value.decode()}

    # ---- tensors
    def tensor(self, dtype, shape, strides=None, data=None):
        return DeviceTensor(self, dtype, shape, strides, data)

    def from_numpy(self, arr, dtype=None, strides=None):
        arr = np.asanyarray(arr)  # (a tagged bf16 / fp8 array keeps its tag)
        if dtype is None:
            dtype = abi.dtype_of_array(arr)
        return DeviceTensor(self, dtype, arr.shape, strides, arr)

    # ---- operators (asynchronous on self.stream; download() synchronises)
    def op(self, name, *args):
        self._check(getattr(self.lib, "mlel_hip_" + name)(self.ctx, self.stream, *args))

    def epilogue(self, mult, shift, rescale, clamp=None):
        e = abi.Epilogue()
        e.multiplier = C.pointer(mult.view)
        e.shift = C.pointer(shift.view)
        e.rescale = rescale
        if clamp is not None:
            e.has_clamp = 1
            e.clamp = abi.ClampAttr(float(clamp[0]), float(clamp[1]), abi.NAN_PROPAGATE)
        return e

    # events / timing
    def event(self):
        e = C.c_void_p()
        self._check(self.lib.mlel_hip_event_create(self.ctx, C.byref(e)))
        return e

    def record(self, ev):
        self._check(self.lib.mlel_hip_event_record(self.ctx, ev, self.stream))

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        self._check(self.lib.mlel_hip_event_elapsed_ms(self.ctx, start, stop, C.byref(ms)))
        return ms.value

    def new_stream(self):
        s = C.c_void_p()
        self._check(self.lib.mlel_hip_stream_create(self.ctx, C.byref(s)))
        return s

    def free_stream(self, stream):
        self._check(self.lib.mlel_hip_stream_destroy(self.ctx, stream))
