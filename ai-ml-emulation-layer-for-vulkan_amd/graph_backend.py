"""ctypes harness over libmlel_graph.so, the C view (include/mlel_graph.h) of the host-side GraphPipeline.

Builds a data graph from a neutral description (see graphs.py), binds device memory and dispatches it.  As in the
reference's test client (utilities/pipeline.cpp:297-330) external tensors are allocated by the caller, session
memory is queried, allocated and bound once, and a dispatch is followed by a wait.
"""
import ctypes as C
import os

import numpy as np

from . import abi
from .hip_backend import MlelError, load_library

_glib = None

_I64P = C.POINTER(C.c_int64)
_V = C.c_void_p


class SpvBinding(C.Structure):
    _fields_ = [("set", C.c_uint32), ("binding", C.c_uint32), ("array_index", C.c_uint32), ("rank", C.c_int32),
                ("dims", C.POINTER(C.c_int64))]


class SpvSpecialization(C.Structure):
    _fields_ = [("spec_id", C.c_uint32), ("bits", C.c_uint64)]


class SpvConstant(C.Structure):
    _fields_ = [("id", C.c_uint32), ("rank", C.c_int32), ("dims", C.POINTER(C.c_int64)), ("data", C.c_void_p)]


class BindPointRequirement(C.Structure):
    _fields_ = [("bind_point", C.c_uint32), ("bind_point_type", C.c_uint32), ("num_objects", C.c_uint32)]


INCOMPLETE = 5            # MLEL_GRAPH_INCOMPLETE
BIND_POINT_TRANSIENT = 0  # MLEL_GRAPH_BIND_POINT_TRANSIENT


def load_graph_library():
    global _glib
    if _glib is None:
        load_library()  # libmlel_hip.so first: the graph library is linked against it
        if not os.path.exists(abi.GRAPH_LIB_PATH):
            raise MlelError(abi.ERR_DEVICE, f"{abi.GRAPH_LIB_PATH} is not built; run __graft_entry__.build()")
        lib = C.CDLL(abi.GRAPH_LIB_PATH)
        lib.mlel_graph_last_error.restype = C.c_char_p
        lib.mlel_graph_create.argtypes = [_V, C.POINTER(_V)]
        lib.mlel_graph_destroy.argtypes = [_V]
        lib.mlel_graph_destroy.restype = None
        lib.mlel_graph_make_const_tensor.argtypes = [_V, C.c_uint32, C.c_int32, C.c_int32, _I64P, _I64P, _V]
        lib.mlel_graph_get_const_tensor.argtypes = [_V, C.c_uint32]
        lib.mlel_graph_make_const_composite_tensor.argtypes = [_V, C.c_int32, C.c_int32, _I64P, _V]
        lib.mlel_graph_make_descriptor_set_binding.argtypes = [_V, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int32,
                                                               C.c_int32, _I64P, _I64P]
        lib.mlel_graph_get_tensor.argtypes = [_V, C.c_uint32, C.c_uint32, C.c_uint32]
        lib.mlel_graph_make_tensor.argtypes = [_V, C.c_int32, C.c_int32, _I64P, _I64P]
        lib.mlel_graph_make_input.argtypes = [_V, C.c_int]
        lib.mlel_graph_make_output.argtypes = [_V, C.c_int]
        lib.mlel_graph_make_op.argtypes = [_V, C.c_char_p, C.POINTER(C.c_int), C.c_int, C.POINTER(C.c_int), C.c_int,
                                           _I64P, C.c_int, C.POINTER(C.c_double), C.c_int, C.c_char_p]
        lib.mlel_graph_load_spvasm.argtypes = [_V, C.c_char_p, C.c_size_t, C.POINTER(SpvBinding), C.c_int,
                                               C.POINTER(SpvConstant), C.c_int, C.POINTER(SpvSpecialization), C.c_int,
                                               C.POINTER(C.c_uint32), C.c_int,
                                               C.POINTER(C.c_int), C.POINTER(C.c_int)]
        lib.mlel_graph_load_spirv.argtypes = [_V, C.POINTER(C.c_uint32), C.c_size_t, C.POINTER(SpvBinding), C.c_int,
                                              C.POINTER(SpvConstant), C.c_int, C.POINTER(SpvSpecialization), C.c_int,
                                              C.POINTER(C.c_uint32), C.c_int,
                                              C.POINTER(C.c_int), C.POINTER(C.c_int)]
        lib.mlel_graph_tensor_info.argtypes = [_V, C.c_int, C.POINTER(C.c_int32), _I64P]
        lib.mlel_graph_finalize.argtypes = [_V, C.c_int]
        lib.mlel_graph_set_batch_split.argtypes = [_V, C.c_int]
        lib.mlel_graph_get_batch_split.argtypes = [_V]
        lib.mlel_graph_set_memory_planner.argtypes = [_V, C.c_int]
        lib.mlel_graph_get_memory_planner.argtypes = [_V]
        lib.mlel_graph_session_memory_requirements.argtypes = [_V, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        lib.mlel_graph_bind_session_memory.argtypes = [_V, _V]
        lib.mlel_graph_bind_external.argtypes = [_V, C.c_uint32, C.c_uint32, C.c_uint32, _V]
        lib.mlel_graph_dispatch.argtypes = [_V, _V]
        lib.mlel_graph_session_create.argtypes = [_V, C.POINTER(_V)]
        lib.mlel_graph_session_destroy.argtypes = [_V]
        lib.mlel_graph_session_destroy.restype = None
        lib.mlel_graph_session_bind_point_requirements.argtypes = [_V, C.POINTER(C.c_uint32),
                                                                  C.POINTER(BindPointRequirement)]
        lib.mlel_graph_session_get_memory_requirements.argtypes = [_V, C.c_uint32, C.POINTER(C.c_uint64),
                                                                  C.POINTER(C.c_uint64)]
        lib.mlel_graph_session_bind_memory.argtypes = [_V, C.c_uint32, _V]
        lib.mlel_graph_session_bind_external.argtypes = [_V, C.c_uint32, C.c_uint32, C.c_uint32, _V]
        lib.mlel_graph_session_dispatch.argtypes = [_V, _V]
        lib.mlel_graph_session_dispatch_replayed.argtypes = [_V, _V]
        lib.mlel_graph_session_dispatch_range.argtypes = [_V, _V, C.c_int, C.c_int]
        lib.mlel_graph_dispatch_profiled.argtypes = [_V, _V, C.POINTER(C.c_float), C.c_int]
        lib.mlel_graph_set_profiling.argtypes = [_V, C.c_int]
        lib.mlel_graph_get_profiling.argtypes = [_V]
        lib.mlel_graph_profiling_json.argtypes = [_V, C.c_char_p, C.c_size_t]
        lib.mlel_graph_profiling_json.restype = C.c_int64
        lib.mlel_graph_op_count.argtypes = [_V]
        lib.mlel_graph_op_name.argtypes = [_V, C.c_int, C.c_char_p, C.c_size_t]
        lib.mlel_graph_session_tensor_count.argtypes = [_V]
        lib.mlel_graph_session_tensor_info.argtypes = [_V, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_uint64),
                                                       C.POINTER(C.c_uint64), C.POINTER(C.c_uint32),
                                                       C.POINTER(C.c_uint32)]
        lib.mlel_graph_allocate_intervals.argtypes = [C.POINTER(C.c_uint64), C.c_int, C.POINTER(C.c_uint64), C.c_int,
                                                      C.c_uint64, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        lib.mlel_graph_dtype_from_vk_format.argtypes = [C.c_int32]
        _glib = lib
    return _glib


def _i64(values):
    values = [int(v) for v in values]
    return (C.c_int64 * max(1, len(values)))(*values)


def allocate_intervals(intervals, unseen, alignment):
    """details::allocateIntervals on its own: ({id: offset}, memory_size)."""
    lib = load_graph_library()
    flat_i = [v for iv in intervals for v in iv]
    flat_u = [v for u in unseen for v in u]
    n, m = len(intervals), len(unseen)
    ai = (C.c_uint64 * max(1, len(flat_i)))(*flat_i)
    au = (C.c_uint64 * max(1, len(flat_u)))(*flat_u)
    out = (C.c_uint64 * max(2, 2 * (n + m)))()
    size = C.c_uint64()
    k = lib.mlel_graph_allocate_intervals(ai, n, au, m, alignment, out, C.byref(size))
    if k < 0:
        raise MlelError(k, lib.mlel_graph_last_error().decode())
    return {int(out[2 * i]): int(out[2 * i + 1]) for i in range(k)}, int(size.value)


class Graph:
    """One GraphPipeline.  Tensors are named; names map to the integer handles of the C API."""

    def __init__(self, dev):
        self.dev = dev
        self.lib = load_graph_library()
        g = _V()
        self._check(self.lib.mlel_graph_create(dev.ctx, C.byref(g)))
        self.g = g
        self.handles = {}
        self.externals = {}      # name -> (set, binding, array index, dtype, shape)
        self.session_mem = None
        self.ext_tensors = {}    # name -> DeviceTensor
        self.next_binding = 0
        self.next_const = 0

    def _check(self, rc):
        if rc < 0:
            raise MlelError(rc, self.lib.mlel_graph_last_error().decode(errors="replace"))
        return rc

    def close(self):
        if self.g:
            self.lib.mlel_graph_destroy(self.g)
            self.g = None
        if self.session_mem:
            self.dev.free(self.session_mem)
            self.session_mem = None
        for t in self.ext_tensors.values():
            t.free()
        self.ext_tensors = {}

    # ---- tensors
    def const(self, name, array, dtype=None):
        array = np.ascontiguousarray(array)
        if dtype is None:
            dtype = abi.dtype_of_array(array)
        dims = array.shape if array.ndim else (1,)
        h = self._check(self.lib.mlel_graph_make_const_tensor(self.g, self.next_const, int(dtype), len(dims),
                                                              _i64(dims), None, array.ctypes.data))
        self.next_const += 1
        self.handles[name] = h
        return h

    def external(self, name, dtype, shape, set_=0, binding=None, array_index=0, strides=None):
        if binding is None:
            binding = self.next_binding
            self.next_binding += 1
        h = self._check(self.lib.mlel_graph_make_descriptor_set_binding(
            self.g, set_, binding, array_index, int(dtype), len(shape), _i64(shape),
            _i64(strides) if strides is not None else None))
        self.handles[name] = h
        self.externals[name] = (set_, binding, array_index, int(dtype), tuple(shape), strides)
        return h

    def tensor(self, name, dtype, shape):
        h = self._check(self.lib.mlel_graph_make_tensor(self.g, int(dtype), len(shape), _i64(shape), None))
        self.handles[name] = h
        return h

    def mark_input(self, name):
        self._check(self.lib.mlel_graph_make_input(self.g, self.handles[name]))

    def mark_output(self, name):
        self._check(self.lib.mlel_graph_make_output(self.g, self.handles[name]))

    # ---- operators
    def op(self, tosa_name, inputs, outputs, iattr=(), fattr=(), debug_name=""):
        ins = (C.c_int * max(1, len(inputs)))(*[self.handles[n] for n in inputs])
        outs = (C.c_int * max(1, len(outputs)))(*[self.handles[n] for n in outputs])
        fa = (C.c_double * max(1, len(fattr)))(*[float(v) for v in fattr])
        self._check(self.lib.mlel_graph_make_op(self.g, tosa_name.encode(), ins, len(inputs), outs, len(outputs),
                                                _i64(iattr), len(iattr), fa, len(fattr), debug_name.encode()))

    # ---- SPIR-V assembly front-end
    def load_spirv(self, words, bindings=None, constants=None, names=None, specializations=None):
        """Decodes a binary SPIR-V module (a sequence of 32-bit words, or bytes) into this graph; arguments and
        result as load_spvasm."""
        if isinstance(words, (bytes, bytearray, memoryview)):
            words = np.frombuffer(bytes(words), dtype=np.uint32)
        words = np.ascontiguousarray(np.asarray(words, dtype=np.uint32))
        return self._load_module(words, bindings, constants, names, specializations)

    def load_spvasm(self, text, bindings=None, constants=None, names=None, specializations=None):
        """Decodes a SPIR-V assembly module into this graph.  `bindings`: {(set, binding, element): shape} for
        interface tensors of unshaped type; `constants`: {graph constant id: ndarray}; `names`: {(set, binding,
        element): name} for the externals (default "s<set>b<binding>e<element>"); `specializations`: {SpecId: value
        bits}.  Returns (input names, output names, number of TOSA instructions)."""
        return self._load_module(text, bindings, constants, names, specializations)

    def _load_module(self, module, bindings=None, constants=None, names=None, specializations=None):
        bindings, constants, names = bindings or {}, constants or {}, names or {}
        keep = []
        barr = (SpvBinding * max(1, len(bindings)))()
        for i, ((s, b, e), shape) in enumerate(bindings.items()):
            dims = _i64(shape)
            keep.append(dims)
            barr[i] = SpvBinding(s, b, e, len(shape), dims)
        carr = (SpvConstant * max(1, len(constants)))()
        for i, (cid, array) in enumerate(constants.items()):
            array = np.ascontiguousarray(array)
            dims = _i64(array.shape)
            keep += [dims, array]
            carr[i] = SpvConstant(cid, array.ndim, dims, array.ctypes.data)
        specializations = specializations or {}
        sarr = (SpvSpecialization * max(1, len(specializations)))()
        for i, (sid, bits) in enumerate(specializations.items()):
            sarr[i] = SpvSpecialization(int(sid), int(bits) & (2 ** 64 - 1))
        io = (C.c_uint32 * 3072)()
        n_in, n_out = C.c_int(), C.c_int()
        if isinstance(module, str):
            raw = module.encode()
            count = self._check(self.lib.mlel_graph_load_spvasm(self.g, raw, len(raw), barr, len(bindings), carr,
                                                                len(constants), sarr, len(specializations), io, 3072,
                                                                C.byref(n_in), C.byref(n_out)))
        else:
            count = self._check(self.lib.mlel_graph_load_spirv(self.g, module.ctypes.data_as(C.POINTER(C.c_uint32)),
                                                               module.size, barr, len(bindings), carr, len(constants),
                                                               sarr, len(specializations), io, 3072, C.byref(n_in),
                                                               C.byref(n_out)))
        result = []
        for k in range(n_in.value + n_out.value):
            key = (int(io[3 * k]), int(io[3 * k + 1]), int(io[3 * k + 2]))
            name = names.get(key, "s%db%de%d" % key)
            h = self._check(self.lib.mlel_graph_get_tensor(self.g, *key))
            dtype, dims = C.c_int32(), (C.c_int64 * 8)()
            rank = self._check(self.lib.mlel_graph_tensor_info(self.g, h, C.byref(dtype), dims))
            self.handles[name] = h
            self.externals[name] = (key[0], key[1], key[2], int(dtype.value), tuple(int(dims[i]) for i in range(rank)), None)
            result.append(name)
        return result[:n_in.value], result[n_in.value:], count

    PLANNERS = {"interval": 0, "linear": 1, "bestfit": 2}

    def set_planner(self, name):
        self._check(self.lib.mlel_graph_set_memory_planner(self.g, self.PLANNERS[name]))

    def planner(self):
        code = self._check(self.lib.mlel_graph_get_memory_planner(self.g))
        return [k for k, v in self.PLANNERS.items() if v == code][0]

    def set_batch_split(self, enabled=True):
        """Before finalize(): the leading batch-separable operators are issued per half batch on two streams."""
        self._check(self.lib.mlel_graph_set_batch_split(self.g, 1 if enabled else 0))

    def batch_split_launches(self):
        return self._check(self.lib.mlel_graph_get_batch_split(self.g))

    # ---- finalize / memory / run
    def finalize(self, fuse=True):
        self._check(self.lib.mlel_graph_finalize(self.g, 1 if fuse else 0))
        size, align = C.c_uint64(), C.c_uint64()
        self._check(self.lib.mlel_graph_session_memory_requirements(self.g, C.byref(size), C.byref(align)))
        self.session_size = int(size.value)
        self.session_mem = self.dev.alloc(max(self.session_size, 256))
        self._check(self.lib.mlel_graph_bind_session_memory(self.g, C.c_void_p(self.session_mem)))
        for name, (s, b, a, dtype, shape, strides) in self.externals.items():
            t = self.dev.tensor(dtype, shape, strides)
            self.ext_tensors[name] = t
            self._check(self.lib.mlel_graph_bind_external(self.g, s, b, a, C.c_void_p(t.ptr)))
        return self.session_size

    def set_input(self, name, array):
        self.ext_tensors[name].upload(array)

    def get_output(self, name):
        return self.ext_tensors[name].download()

    def dispatch(self):
        self._check(self.lib.mlel_graph_dispatch(self.g, self.dev.stream))

    def new_session(self, allocate=True):
        """A further session of this (finalized) pipeline; with `allocate` it gets session memory and external tensors
        of its own, as the reference's test client gives every dispatch (utilities/pipeline.cpp:297-330)."""
        return Session(self, allocate)

    def dispatch_profiled(self):
        n = self.op_count()
        ms = (C.c_float * max(1, n))()
        self._check(self.lib.mlel_graph_dispatch_profiled(self.g, self.dev.stream, ms, n))
        return [(self.op_name(i), float(ms[i])) for i in range(n)]

    def set_profiling(self, enabled):
        """Every dispatch() records per-operator times (a new graph starts from VMEL_GRAPH_PROFILING)."""
        self._check(self.lib.mlel_graph_set_profiling(self.g, 1 if enabled else 0))

    def profiling(self):
        return bool(self._check(self.lib.mlel_graph_get_profiling(self.g)))

    def profiling_report(self):
        """The profiler's report ("samples", "by_operator") as a dict."""
        import json
        need = self._check(self.lib.mlel_graph_profiling_json(self.g, None, 0))
        buf = C.create_string_buffer(int(need))
        self._check(self.lib.mlel_graph_profiling_json(self.g, buf, need))
        return json.loads(buf.value.decode())

    def op_count(self):
        return self._check(self.lib.mlel_graph_op_count(self.g))

    def op_name(self, i):
        buf = C.create_string_buffer(128)
        self._check(self.lib.mlel_graph_op_name(self.g, i, buf, 128))
        return buf.value.decode()

    def op_names(self):
        return [self.op_name(i) for i in range(self.op_count())]

    def session_tensors(self):
        n = self._check(self.lib.mlel_graph_session_tensor_count(self.g))
        out = []
        for i in range(n):
            h, off, size, first, last = C.c_int(), C.c_uint64(), C.c_uint64(), C.c_uint32(), C.c_uint32()
            self._check(self.lib.mlel_graph_session_tensor_info(self.g, i, C.byref(h), C.byref(off), C.byref(size),
                                                                C.byref(first), C.byref(last)))
            out.append({"handle": h.value, "offset": None if off.value == 2 ** 64 - 1 else off.value,
                        "size": size.value, "first": first.value, "last": last.value})
        return out


class Session:
    """One mlel_graph_session: its own transient memory and external tensors."""

    def __init__(self, graph, allocate=True):
        self.graph, self.dev, self.lib = graph, graph.dev, graph.lib
        s = _V()
        graph._check(self.lib.mlel_graph_session_create(graph.g, C.byref(s)))
        self.s = s
        self.session_mem = None
        self.ext_tensors = {}
        if allocate:
            count = C.c_uint32()
            graph._check(self.lib.mlel_graph_session_bind_point_requirements(self.s, C.byref(count), None))
            if count.value:
                size, align = self.memory_requirements()
                self.session_mem = self.dev.alloc(max(size, 256))
                self.bind_memory(self.session_mem)
            for name, (st, b, a, dtype, shape, strides) in graph.externals.items():
                self.bind(name, self.dev.tensor(dtype, shape, strides))

    def bind_point_requirements(self, capacity=None):
        """(status, count, entries): capacity None is the counting call of the two-call pattern"""
        count = C.c_uint32(0 if capacity is None else capacity)
        arr = None if capacity is None else (BindPointRequirement * max(1, capacity))()
        rc = self.graph._check(self.lib.mlel_graph_session_bind_point_requirements(self.s, C.byref(count), arr))
        entries = [] if arr is None else [(arr[i].bind_point, arr[i].bind_point_type, arr[i].num_objects)
                                          for i in range(min(capacity, count.value))]
        return rc, count.value, entries

    def memory_requirements(self, bind_point=BIND_POINT_TRANSIENT):
        size, align = C.c_uint64(), C.c_uint64()
        self.graph._check(self.lib.mlel_graph_session_get_memory_requirements(self.s, bind_point, C.byref(size),
                                                                              C.byref(align)))
        return int(size.value), int(align.value)

    def bind_memory(self, device_base, bind_point=BIND_POINT_TRANSIENT):
        self.graph._check(self.lib.mlel_graph_session_bind_memory(self.s, bind_point, C.c_void_p(device_base)))

    def bind(self, name, tensor):
        """binds (or re-binds) the external tensor `name` to a DeviceTensor"""
        st, b, a = self.graph.externals[name][:3]
        self.ext_tensors[name] = tensor
        self.graph._check(self.lib.mlel_graph_session_bind_external(self.s, st, b, a, C.c_void_p(tensor.ptr)))

    def set_input(self, name, array):
        self.ext_tensors[name].upload(array)

    def get_output(self, name):
        return self.ext_tensors[name].download()

    def dispatch(self, stream=None):
        self.graph._check(self.lib.mlel_graph_session_dispatch(self.s, self.dev.stream if stream is None else stream))

    def dispatch_replayed(self, stream=None):
        """dispatch() through a HIP graph recorded on first use (one submission per dispatch afterwards)"""
        self.graph._check(self.lib.mlel_graph_session_dispatch_replayed(self.s, self.dev.stream if stream is None else stream))

    def dispatch_range(self, first, count, stream=None):
        self.graph._check(self.lib.mlel_graph_session_dispatch_range(
            self.s, self.dev.stream if stream is None else stream, int(first), int(count)))

    def close(self, free_tensors=True):
        if self.s:
            self.lib.mlel_graph_session_destroy(self.s)
            self.s = None
        if self.session_mem:
            self.dev.free(self.session_mem)
            self.session_mem = None
        if free_tensors:
            for t in self.ext_tensors.values():
                t.free()
        self.ext_tensors = {}
