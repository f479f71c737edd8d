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


@pytest.fixture
def tuned():
    """tuned(name=value, ...) sets kernel-choice switches of the library (tllm_debug_set_tuning) for the rest of
    the test; they are put back when it ends."""
    import ternary_llm_amd as tl
    entered = []

    def apply(**kw):
        ctx = tl.tuning(**kw)
        ctx.__enter__()
        entered.append(ctx)

    yield apply
    for ctx in reversed(entered):
        ctx.__exit__(None, None, None)
