import importlib
import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


_NP = {"i8": np.int8, "u8": np.uint8, "i16": np.int16, "i32": np.int32, "i64": np.int64, "f32": np.float32,
       "f16": np.float16, "bool": np.bool_}


def fixture_array(d):
    """{"dtype","shape","data"} -> numpy array"""
    return np.array(d["data"], dtype=_NP[d["dtype"]]).reshape(d["shape"])


@pytest.fixture(scope="session")
def kats():
    with open(os.path.join(ROOT, "tests", "golden", "reference_kats.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def abi():
    return importlib.import_module("ai-ml-emulation-layer-for-vulkan_amd.abi")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure): numpy front-end over oracle/libmlel_oracle.so."""
    mod = importlib.import_module("oracle.mlel_oracle")
    mod.lib()
    return mod
