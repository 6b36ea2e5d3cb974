import os
import sys

import numpy as np
import pytest

# the library's debug switches (kernel choice per test) work only with this set before its first use
os.environ.setdefault("PA_ENABLE_DEBUG", "1")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture
def rng():
    return np.random.default_rng(42)
