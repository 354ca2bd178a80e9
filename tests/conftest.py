import os
import sys

import pytest
import torch  # noqa: F401  (first, so the process holds one HIP runtime: torch's)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "ascend-moe-engine_amd", "python"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session")
def lib():
    import mlakv_ffi
    return mlakv_ffi.load()


@pytest.fixture(scope="session")
def oracle():
    import oracle_ffi
    return oracle_ffi.load()


@pytest.fixture(scope="session")
def goldens():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "reference_goldens.json")) as handle:
        return json.load(handle)
