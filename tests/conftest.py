import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def dev():
    """One device handle for the whole session (GPU tests only)."""
    from kalosm_amd.fusor import Device

    d = Device.gpu(0)
    yield d
    d.sync()


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o

    o.build()
    return o
