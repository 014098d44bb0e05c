import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs an MI355X (runs the HIP path)")


@pytest.fixture(autouse=True)
def _announce(request):
    # Name the case before it runs so that a GPU fault still leaves the test id in the output.
    print(f"\n[case] {request.node.nodeid}", flush=True)
    yield
