import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 device (run on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.load()
    return o


@pytest.fixture(scope="session")
def gpu():
    """One device handle for the whole session. GPU tests fail loudly when the library or the device is missing."""
    import qwental_amd as q
    g = q.Gpu()
    print("\n[gpu] %s, %d CUs" % (g.name(), g.cu_count()), flush=True)
    yield g
    g.close()


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before it touches the GPU, so that a lost box still shows which test was running
    if request.node.get_closest_marker("gpu"):
        print("\n[case] %s" % request.node.nodeid, flush=True)
    yield
