import importlib
import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box only)")


@pytest.fixture(scope="session")
def pkg():
    return importlib.import_module("hands-on-mlir_amd")


@pytest.fixture(scope="session")
def rt():
    return importlib.import_module("hands-on-mlir_amd.hom_runtime")


@pytest.fixture(scope="session")
def synth():
    return importlib.import_module("hands-on-mlir_amd.synth")


@pytest.fixture(scope="session")
def oracle():
    import oracle as o  # oracle/oracle.py
    o.lib()
    return o


@pytest.fixture(scope="session")
def literals():
    with open(os.path.join(ROOT, "tests", "golden", "reference_literals.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def gpu(rt):
    """The runtime library on a real GPU; fails loudly if the .so is missing."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    lib = rt.load_runtime()
    lib.homSetErrorMode(0)
    return lib
