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


@pytest.fixture(scope="session")
def golden():
    """The committed input / expected-output vectors (tests/golden/make_golden.py writes them)."""
    import numpy as np

    path = os.path.join(ROOT, "tests", "golden", "fusor_golden.npz")
    with np.load(path, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}
