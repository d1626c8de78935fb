import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def kats():
    with open(os.path.join(ROOT, "tests", "golden", "reference_kats.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def pf():
    """The loaded C-ABI library; building it is the job of __graft_entry__.build()."""
    from pegaflow_amd import _lib
    return _lib.load()


@pytest.fixture(scope="session")
def gpu():
    """Select device 0; fails (not skips) when the HIP runtime has none."""
    from pegaflow_amd import runtime
    assert runtime.device_count() >= 1
    runtime.set_device(0)
    return 0
