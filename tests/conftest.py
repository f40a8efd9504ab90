"""Shared fixtures. Tests marked ``gpu`` need an MI355X and a built libbship.so;
everything else runs on the CPU."""
import ctypes
import os
import subprocess
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


@pytest.fixture(scope="module")
def trace(tmp_path_factory):
    """A host-only library that logs launches instead of making them (window_trace/trace_lib.cpp), put in
    the place of libbship.so for the tests of one module: the real HipHandler then runs without a GPU."""
    from brainstorm_amd import _lib
    out = str(tmp_path_factory.mktemp("trace") / "libtrace.so")
    src = os.path.join(ROOT, "tests", "window_trace", "trace_lib.cpp")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-shared", "-fPIC", "-o", out, src], check=True)
    lib = ctypes.CDLL(out)
    for name, argtypes in _lib.SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            continue                       # the trace library has only what these tests call
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    lib.bship_last_error.restype = ctypes.c_char_p
    lib.trace_log.restype = ctypes.c_char_p
    saved = _lib._LIB
    _lib._LIB = lib
    try:
        yield lib
    finally:
        _lib._LIB = saved
