"""CPU-only checks of the boundary: the C ABI library loads and exports what
include/bship.h declares, fails cleanly without a device, and HipHandler keeps
the reference's handler interface (names, argument order, keyword names)."""
import ast
import ctypes
import inspect
import os
import re
import subprocess
import sys

import pytest

from brainstorm_amd import _lib, handler_api

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bship.h")
REFERENCE_BASE = "/root/reference/brainstorm/handlers/base_handler.py"
REFERENCE_NUMPY = "/root/reference/brainstorm/handlers/numpy_handler.py"


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bship_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_binds():
    assert declared_functions() == sorted(_lib.EXPORTED_SYMBOLS)


def test_library_loads_and_exports_every_declared_symbol():
    assert os.path.exists(_lib.lib_path()), "build libbship.so first (python -m brainstorm_amd.build)"
    lib = ctypes.CDLL(_lib.lib_path())
    for name in declared_functions():
        assert hasattr(lib, name), "libbship.so does not export %s" % name


def test_calls_fail_cleanly_before_init():
    # No compute without bship_init(): a negative status and a message, never a crash.
    # run in a child so that an initialised library in this process cannot hide the check
    code = (
        "import ctypes, sys; sys.path.insert(0, %r)\n"
        "from brainstorm_amd import _lib\n"
        "lib = _lib.load()\n"
        "st = lib.bship_fill_f32(None, 1.0, 16)\n"
        "msg = lib.bship_last_error().decode()\n"
        "assert st == -1 and 'bship_init' in msg, (st, msg)\n"
        "st = lib.bship_sync(); assert st == -1\n"
        "st = lib.bship_gemm_f32(0, 0, 2, 2, 2, 1.0, None, 2, None, 2, 0.0, None, 2); assert st == -1\n"
        "print('ok')\n" % ROOT)
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert res.returncode == 0 and "ok" in res.stdout, res.stdout + res.stderr


def test_missing_library_is_an_import_error(monkeypatch):
    monkeypatch.setenv("BSHIP_LIB", "/nonexistent/libbship.so")
    monkeypatch.setattr(_lib, "_LIB", None)
    with pytest.raises(ImportError):
        _lib.load()


def _methods_of(path):
    """name -> list of argument names (without self) for every method in the first class."""
    tree = ast.parse(open(path).read())
    cls = next(n for n in tree.body if isinstance(n, ast.ClassDef))
    out = {}
    for node in cls.body:
        if isinstance(node, ast.FunctionDef) and not node.name.startswith("_"):
            out[node.name] = [a.arg for a in node.args.args[1:]]
    return out


def test_hip_handler_has_every_interface_method():
    from brainstorm_amd.hip_handler import HipHandler
    assert not getattr(HipHandler, "__abstractmethods__", None)
    for name in handler_api.HANDLER_METHODS:
        assert callable(getattr(HipHandler, name)), name


def test_mirror_and_hip_handler_signatures_agree():
    from brainstorm_amd.hip_handler import HipHandler
    mirror = handler_api._MirrorHandler
    for name in sorted(mirror.__abstractmethods__):
        want = list(inspect.signature(getattr(mirror, name)).parameters)
        got = list(inspect.signature(getattr(HipHandler, name)).parameters)
        assert got == want, "%s: %r != %r" % (name, got, want)


@pytest.mark.skipif(not os.path.exists(REFERENCE_BASE), reason="reference sources not present")
def test_interface_matches_the_reference_sources():
    # The reference is only READ as text here: method names and argument names of its abstract
    # Handler (base_handler.py) and of NumpyHandler must be the ones our handler accepts.
    from brainstorm_amd.hip_handler import HipHandler
    ref = _methods_of(REFERENCE_BASE)
    mirror = handler_api._MirrorHandler
    assert set(ref) == set(mirror.__abstractmethods__), set(ref) ^ set(mirror.__abstractmethods__)
    for name, args in ref.items():
        got = list(inspect.signature(getattr(HipHandler, name)).parameters)[1:]
        assert got == args, "%s: ours %r, reference %r" % (name, got, args)
    # NumpyHandler adds mult_add_mv (numpy_handler.py:239), which the layers call
    numpy_methods = _methods_of(REFERENCE_NUMPY)
    assert "mult_add_mv" in numpy_methods
    assert list(inspect.signature(HipHandler.mult_add_mv).parameters)[1:] == numpy_methods["mult_add_mv"]
    for name in numpy_methods:
        assert hasattr(HipHandler, name), name


def test_description_round_trips_the_constructor_settings():
    # the reference handler describes its constructor argument and is rebuilt from it
    # (numpy_handler.py:25-33, describable.py); ours does the same for its settings. No GPU needed:
    # the constructor is replaced by a recorder.
    from brainstorm_amd.hip_handler import HipHandler
    h = object.__new__(HipHandler)
    h.device, h.pitched_views, h.fast_masks, h.fusing = 2, True, True, False
    desc = h.__describe__()
    assert desc == {"@type": "HipHandler", "device": 2, "pitched_views": True, "fast_masks": True, "fusing": False}
    seen = {}

    class Recorder(HipHandler):
        def __init__(self, seed=None, device=0, pitched_views=False, fast_masks=False, fusing=True):
            seen.update(seed=seed, device=device, pitched_views=pitched_views, fast_masks=fast_masks, fusing=fusing)

    r = object.__new__(Recorder)
    r.__init_from_description__(desc)
    assert seen == {"seed": None, "device": 2, "pitched_views": True, "fast_masks": True, "fusing": False}
    r.__init_from_description__({"@type": "HipHandler"})                  # descriptions written before
    assert seen == {"seed": None, "device": 0, "pitched_views": False, "fast_masks": False, "fusing": True}
