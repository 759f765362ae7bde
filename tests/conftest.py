import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def hip():
    """The HIP engine.  On a GPU box its absence is a failure, never a skip."""
    from mongoose_amd import engine
    eng = engine.NewHIP()
    assert eng is not None, "NewHIP() returned None: no HIP device visible to a gpu-marked test"
    return eng
