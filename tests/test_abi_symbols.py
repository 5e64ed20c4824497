"""The C-ABI library loads and exports every symbol include/mlel_hip.h declares (no compute without a GPU)."""
import ctypes as C
import os
import re

import pytest


def test_library_exports_every_declared_symbol(abi):
    if not os.path.exists(abi.HIP_LIB_PATH):
        pytest.skip("libmlel_hip.so not built (run __graft_entry__.build())")
    lib = C.CDLL(abi.HIP_LIB_PATH)
    header = open(os.path.join(abi.REPO_ROOT, "include", "mlel_hip.h")).read()
    declared = set(re.findall(r"\b(mlel_hip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 45
    assert declared == set(abi.hip_symbol_names()), declared ^ set(abi.hip_symbol_names())
    for name in sorted(declared):
        assert hasattr(lib, name), name


def test_graph_library_exports_every_declared_symbol(abi):
    if not os.path.exists(abi.GRAPH_LIB_PATH):
        pytest.skip("libmlel_graph.so not built (run __graft_entry__.build())")
    C.CDLL(abi.HIP_LIB_PATH, mode=C.RTLD_GLOBAL)
    lib = C.CDLL(abi.GRAPH_LIB_PATH)
    header = open(os.path.join(abi.REPO_ROOT, "include", "mlel_graph.h")).read()
    declared = set(re.findall(r"\b(mlel_graph_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 35
    for name in sorted(declared):
        assert hasattr(lib, name), name


def test_no_gpu_fails_loudly(abi):
    """Without a device every entry point that needs one reports MLEL_ERR_DEVICE; there is no CPU fallback."""
    if not os.path.exists(abi.HIP_LIB_PATH):
        pytest.skip("libmlel_hip.so not built")
    lib = abi.bind_hip(C.CDLL(abi.HIP_LIB_PATH))
    if lib.mlel_hip_device_count() > 0:
        pytest.skip("a GPU is visible")
    ctx = C.c_void_p()
    assert lib.mlel_hip_init(0, C.byref(ctx)) == abi.ERR_DEVICE
    assert b"no CPU fallback" in lib.mlel_hip_last_error()
    t = abi.make_tensor(None, abi.I8, (1,))
    assert lib.mlel_hip_cast(None, None, C.byref(t), C.byref(t)) == abi.ERR_INVALID
