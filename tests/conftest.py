import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle_bind import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden.npz")
    return np.load(path, allow_pickle=False)


@pytest.fixture(scope="session")
def reflib():
    """The compiled reference library, when oracle/_ref/libaxref.so exists."""
    from oracle_bind import RefLib, ref_available
    if not ref_available():
        pytest.skip("oracle/_ref/libaxref.so not built (reference tree absent)")
    return RefLib()


@pytest.fixture(scope="session")
def hip():
    """libaxhip.so on a real GPU.  No fallback: a missing library or GPU is an error."""
    from axiom_amd import AxHip
    h = AxHip()
    h.init()
    return h
