import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line(
        "markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line(
        "markers", "fused_math: runs with the SparseLengths kernels' fused "
                   "arithmetic (the library default); other tests switch it off "
                   "and compare bit for bit")


@pytest.fixture(autouse=True)
def _slws_arithmetic(request):
    """Tests compare SparseLengths results with the CPU loop bit for bit, which
    needs the kernels' separately rounded arithmetic; tests marked fused_math
    run the default (fused) arithmetic and compare to the stated tolerance."""
    from glow_amd import capi
    try:
        capi.lib()
    except capi.MI355XError:
        yield
        return
    capi.slws_set_fused_math(request.node.get_closest_marker("fused_math") is not None)
    yield
    capi.slws_set_fused_math(True)
