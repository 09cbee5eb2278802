import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before it touches the GPU, so a fault still identifies it
    if request.node.get_closest_marker("gpu"):
        print(f"\n[gpu-case] {request.node.nodeid}", flush=True)
    yield
