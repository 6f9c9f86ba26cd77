import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def oracle():
    from oracle import dot_oracle
    dot_oracle.build()
    return dot_oracle


@pytest.fixture(scope="session")
def gpu_wrapper():
    """The device context; loading fails loudly when libsharpnet_hip.so is absent."""
    from sharpnet_amd import GPUWrapper
    w = GPUWrapper.FromDeviceId(0)
    yield w
