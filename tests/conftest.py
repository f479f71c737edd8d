import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (checker). Built on demand here; on the GPU box the prebuilt .so is loaded."""
    from oracle import oracle as orc
    if not os.path.exists(orc.LIB):
        orc.build()
    orc.load()
    return orc
