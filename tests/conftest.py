import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.binding import Oracle

    return Oracle()


@pytest.fixture(scope="session")
def reflib():
    from oracle.binding import RefLib

    if not RefLib.available():
        pytest.skip("oracle/_ref/libptoref.so not built (reference tree absent)")
    return RefLib()


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "pto_golden.npz")
    return np.load(path, allow_pickle=False)
