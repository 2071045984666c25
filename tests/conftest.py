import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def kqo():
    """The CPU oracle binding (test infrastructure)."""
    from oracle import kqo as mod
    mod.lib()
    return mod


@pytest.fixture(scope="session")
def kqref(kqo):
    """The compiled reference; tests that need it skip where it was not built."""
    if kqo.ref() is None:
        pytest.skip("oracle/_ref/libbp_ref.so not built (reference sources absent)")
    return kqo
