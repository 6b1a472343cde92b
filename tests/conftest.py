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
    from oracle import oracle as o
    o.build()
    return o


@pytest.fixture(scope="session")
def t12():
    """The product package (ctypes face of the C-ABI library)."""
    import __graft_entry__ as ge
    return ge.load_package()


@pytest.fixture(scope="session")
def golden():
    import numpy as np
    path = os.path.join(ROOT, "tests", "golden", "pack_cases.npz")
    z = np.load(path, allow_pickle=False)
    names = sorted({k.split(".")[0] for k in z.files})
    return {n: {k.split(".", 1)[1]: z[k] for k in z.files if k.startswith(n + ".")} for n in names}
