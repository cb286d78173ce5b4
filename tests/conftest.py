import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _output_guards(request):
    """After every GPU test: the guard bytes around each output buffer the test allocated through
    gpu_util are still intact (an out-of-bounds store of a kernel fails the test that launched it)."""
    yield
    if request.node.get_closest_marker("gpu") is not None and "gpu_util" in sys.modules:
        sys.modules["gpu_util"].check_guards(clear=True)
