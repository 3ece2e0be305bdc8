import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ctx():
    """A library handle on GPU 0.  No skipping and no fallback: on a machine
    with a GPU a missing or unloadable libinfiniop.so is a failure."""
    from operators_amd.ops import Context

    c = Context(0)
    yield c
    c.close()
