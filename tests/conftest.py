import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
# The package directory carries a hyphen, so its python binding is put on the path directly.
PKG_PY = os.path.join(ROOT, "ml-drift_amd", "python")
if PKG_PY not in sys.path:
    sys.path.insert(0, PKG_PY)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.build()
    return o
