"""Shared fixtures. Tests marked ``gpu`` need an MI355X and a built libbship.so;
everything else runs on the CPU."""
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
def hip():
    """The handler under test. No fallback: raises if the library or the GPU is missing."""
    from brainstorm_amd import HipHandler
    return HipHandler(seed=1234)


@pytest.fixture(scope="session")
def ref():
    """The CPU oracle (NumpyHandler semantics, float32)."""
    from oracle.numpy_ref_handler import NumpyRefHandler
    return NumpyRefHandler(np.float32, seed=1234)
