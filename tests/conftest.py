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
def kat():
    with open(os.path.join(ROOT, "tests", "golden", "kat.json")) as f:
        return json.load(f)


def hx(s):
    return int(s, 16)


@pytest.fixture(autouse=True)
def builtin_launch_shapes():
    """Overrides a test sets through the tuning hook never outlive it, also when it fails half way."""
    yield
    from nerva_amd import abi
    if os.path.exists(abi.LIBRARY):
        abi.load().nerva_hip_test_set_tuning(None, 0)
