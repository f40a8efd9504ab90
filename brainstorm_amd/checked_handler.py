"""CheckedHandler: a handler that validates every call before passing it on.

A handler does not check shapes (base_handler.py:14-28); a layer that hands
mismatched arrays to a GPU handler corrupts memory silently. brainstorm guards
against that in its tests with a wrapper handler (debug_handler.py:61-548) that
asserts the shape contract of each operation. ``CheckedHandler`` plays that
role for any handler of this package -- ``CheckedHandler(HipHandler())`` or
``CheckedHandler(oracle)`` -- with the same contracts, stated as one table
(``CONTRACTS``) from which the methods are generated.

It works on the wrapped handler's own arrays (no proxy array type), so it can be
slipped under existing code. With ``check_finite=True`` every array argument is
also tested with ``is_fully_finite`` after the call, which is how brainstorm's
wrapper locates the operation that produced the first NaN.
"""
from __future__ import annotations

import inspect
import numbers

import numpy as np

from .handler_api import HANDLER_METHODS, Handler, _MirrorHandler


class ContractError(AssertionError):
    """An operation was called with arguments that violate its contract."""


def _fail(op, msg):
    raise ContractError("%s: %s" % (op, msg))


# ----------------------------------------------------------------- check builders
# A check is a function (op_name, arguments_by_name) -> None that raises ContractError.

def same_shape(*names):
    def check(op, a):
        shapes = [tuple(a[n].shape) for n in names if a[n] is not None]
        if any(s != shapes[0] for s in shapes[1:]):
            _fail(op, "shapes of %s differ: %s" % (", ".join(names), shapes))
    return check


def ndim(name, n):
    def check(op, a):
        if len(a[name].shape) != n:
            _fail(op, "%s must be %d-dimensional, has shape %r" % (name, n, tuple(a[name].shape)))
    return check


def vector_of(v, m, allow_full=False):
    """v is a column (rows, 1) or a row (1, cols) of the matrix m (or, for mult_mv, m's shape)."""
    def check(op, a):
        ms, vs = tuple(a[m].shape), tuple(a[v].shape)
        ok = vs in ((ms[0], 1), (1, ms[1])) or (allow_full and vs == ms)
        if not ok:
            _fail(op, "%s of shape %r does not broadcast against %s of shape %r" % (v, vs, m, ms))
    return check


def scalar(*names):
    def check(op, a):
        for n in names:
            if not isinstance(a[n], (numbers.Real, np.floating, np.integer)) or isinstance(a[n], bool):
                _fail(op, "%s must be a number, got %r" % (n, type(a[n]).__name__))
    return check


def shape_tuple(name, length=None):
    def check(op, a):
        s = a[name]
        if not isinstance(s, tuple) or any((not isinstance(i, (int, np.integer))) or i < 0 for i in s):
            _fail(op, "%s must be a tuple of non-negative integers, got %r" % (name, s))
        if length is not None and len(s) != length:
            _fail(op, "%s must have %d entries, got %r" % (name, length, s))
    return check


def padding_ok(op, a):
    p = a["padding"]
    if not isinstance(p, (int, np.integer)) or isinstance(p, bool) or p < 0:
        _fail(op, "padding must be a non-negative integer, got %r" % (p,))


def where(predicate, message):
    def check(op, a):
        if not predicate(a):
            _fail(op, message(a) if callable(message) else message)
    return check


def _matmul_shapes(op, a):
    (a1, a2), (b1, b2) = a["a"].shape, a["b"].shape
    if a["transa"] not in (True, False) or a["transb"] not in (True, False):
        _fail(op, "transa/transb must be booleans")
    if a["transa"]:
        a1, a2 = a2, a1
    if a["transb"]:
        b1, b2 = b2, b1
    if a2 != b1:
        _fail(op, "inner dimensions differ: %d != %d (transa=%s, transb=%s)" % (a2, b1, a["transa"], a["transb"]))
    if tuple(a["out"].shape) != (a1, b2):
        _fail(op, "out has shape %r, expected %r" % (tuple(a["out"].shape), (a1, b2)))


def _broadcastable(src, dest):
    """NumPy's rule for np.copyto(dest, src): trailing axes agree or are 1 in src."""
    return len(src) <= len(dest) and all(s in (1, d) for s, d in zip(reversed(src), reversed(dest)))


def _label_count(a):
    """Number of classes the labels of binarize_v / index_m_by_v select from."""
    return a["m"].shape[1] if "m" in a else a["out"].shape[1]


def _labels_in_range(handler, a):
    """Labels select a column like NumPy's indexing does (numpy_handler.py:101, 203): values in [-K, K),
    negative ones counted from the last column; NaN and infinities select nothing."""
    labels = handler.get_numpy_copy(a["v"])
    k = _label_count(a)
    return labels.size == 0 or bool(np.isfinite(labels).all() and -k <= int(labels.min()) and int(labels.max()) < k)


_POOL = [shape_tuple("window", 2), shape_tuple("stride", 2), padding_ok]
_MV = [same_shape("m", "out"), ndim("m", 2), vector_of("v", "m")]
_DERIV = [same_shape("x", "y", "dy", "dx")]          # x may be None (the handlers never read it)

# operation -> checks. Array-typed parameters are found from the interface's signature:
# every parameter that is not named in NON_ARRAY must be an array of the handler's array type.
CONTRACTS = {
    "allocate": [shape_tuple("shape")], "ones": [shape_tuple("shape")], "zeros": [shape_tuple("shape")],
    "copy_to": [where(lambda a: _broadcastable(a["src"].shape, a["dest"].shape), "src does not broadcast into dest")],
    "copy_to_if": [same_shape("src", "dest", "cond")],
    "create_from_numpy": [where(lambda a: isinstance(a["arr"], np.ndarray), "arr must be a numpy array")],
    "fill": [scalar("val")],
    "fill_if": [scalar("val"), same_shape("mem", "cond")],
    "get_numpy_copy": [],
    "set_from_numpy": [where(lambda a: isinstance(a["arr"], np.ndarray), "arr must be a numpy array"),
                       where(lambda a: tuple(a["mem"].shape) == a["arr"].shape,
                             lambda a: "shapes differ: %r != %r" % (tuple(a["mem"].shape), a["arr"].shape))],
    "is_fully_finite": [],
    "abs_t": [same_shape("a", "out")], "sign_t": [same_shape("a", "out")],
    "sqrt_t": [same_shape("a", "out")], "log_t": [same_shape("a", "out")],
    "add_into_if": [same_shape("a", "out", "cond")],
    "add_st": [scalar("s"), same_shape("t", "out")],
    "mult_st": [scalar("s"), same_shape("t", "out")],
    "mult_add_st": [scalar("s"), same_shape("t", "out")],
    "add_tt": [same_shape("a", "b", "out")], "subtract_tt": [same_shape("a", "b", "out")],
    "mult_tt": [same_shape("a", "b", "out")], "divide_tt": [same_shape("a", "b", "out")],
    "modulo_tt": [same_shape("a", "b", "out")], "mult_add_tt": [same_shape("a", "b", "out")],
    "add_mv": _MV, "subtract_mv": _MV, "divide_mv": _MV, "mult_add_mv": _MV,
    "mult_mv": [same_shape("m", "out"), ndim("m", 2), vector_of("v", "m", allow_full=True)],
    "clip_t": [scalar("a_min", "a_max"), same_shape("a", "out"),
               where(lambda a: a["a_min"] <= a["a_max"], "a_min must not exceed a_max")],
    "broadcast_t": [where(lambda a: isinstance(a["axis"], (int, np.integer)) and 0 <= a["axis"] < len(a["out"].shape),
                          "axis out of range"),
                    where(lambda a: tuple(a["a"].shape) == tuple(a["out"].shape[:a["axis"]]) + (1,)
                          + tuple(a["out"].shape[a["axis"] + 1:]),
                          lambda a: "a has shape %r, expected out's shape %r with a 1 at axis %d"
                          % (tuple(a["a"].shape), tuple(a["out"].shape), a["axis"]))],
    "merge_tt": [where(lambda a: a["a"].shape[-1] + a["b"].shape[-1] == a["out"].shape[-1],
                       "last dimensions of a and b must add up to out's")],
    "split_add_tt": [where(lambda a: a["out_a"].shape[-1] + a["out_b"].shape[-1] == a["x"].shape[-1],
                           "last dimensions of out_a and out_b must add up to x's")],
    "sum_t": [where(lambda a: a["axis"] is None or (isinstance(a["axis"], (int, np.integer))
                                                    and 0 <= a["axis"] < len(a["a"].shape)), "axis out of range")],
    "softmax_m": [same_shape("m", "out"), ndim("m", 2)],
    "binarize_v": [ndim("v", 2), ndim("out", 2),
                   where(lambda a: tuple(a["v"].shape) == (a["out"].shape[0], 1), "v must be (rows of out, 1)"),
                   "labels"],
    "index_m_by_v": [same_shape("v", "out"), ndim("m", 2), ndim("v", 2),
                     where(lambda a: tuple(a["v"].shape) == (a["m"].shape[0], 1), "v must be (rows of m, 1)"),
                     "labels"],
    "fill_gaussian": [where(lambda a: a["std"] >= 0.0, "std must not be negative")],
    "generate_probability_mask": [scalar("probability"),
                                  where(lambda a: 0.0 <= a["probability"] <= 1.0, "probability outside [0, 1]")],
    "dot_mm": [ndim("a", 2), ndim("b", 2), ndim("out", 2), _matmul_shapes],
    "dot_add_mm": [ndim("a", 2), ndim("b", 2), ndim("out", 2), _matmul_shapes],
    "conv2d_forward_batch": [padding_ok, shape_tuple("stride", 2)],
    "conv2d_backward_batch": [padding_ok, shape_tuple("stride", 2)],
    "maxpool2d_forward_batch": _POOL,
    "maxpool2d_backward_batch": _POOL + [same_shape("inputs", "in_deltas"), same_shape("outputs", "out_deltas")],
    "avgpool2d_forward_batch": _POOL,
    "avgpool2d_backward_batch": _POOL + [same_shape("inputs", "in_deltas"), same_shape("outputs", "out_deltas")],
    "sigmoid": [same_shape("x", "y")], "tanh": [same_shape("x", "y")],
    "rel": [same_shape("x", "y")], "el": [same_shape("x", "y")],
    "sigmoid_deriv": _DERIV, "tanh_deriv": _DERIV, "rel_deriv": _DERIV, "el_deriv": _DERIV,
}

# parameters that are not arrays
NON_ARRAY = {"shape", "val", "arr", "s", "a_min", "a_max", "axis", "mean", "std", "probability", "transa",
             "transb", "padding", "stride", "window"}
# array parameters that may be None
OPTIONAL_ARRAYS = {"x"}
# operations whose result is returned to the caller
RETURNING = {"allocate", "ones", "zeros", "create_from_numpy", "get_numpy_copy", "is_fully_finite"}


def _make_method(name):
    checks = CONTRACTS[name]

    def method(self, *args, **kwargs):
        inner = getattr(self.handler, name)
        try:
            bound = self._signatures[name].bind(*args, **kwargs)
        except TypeError as e:
            _fail(name, str(e))
        bound.apply_defaults()
        a = bound.arguments
        arrays = []
        for pname, value in a.items():
            if pname in NON_ARRAY:
                continue
            if value is None and pname in OPTIONAL_ARRAYS and name.endswith("_deriv"):
                continue
            if not isinstance(value, self.array_type):
                _fail(name, "%s must be a %s, got %s" % (pname, self.array_type.__name__, type(value).__name__))
            arrays.append((pname, value))
        for check in checks:
            if check == "labels":
                if not _labels_in_range(self.handler, a):
                    _fail(name, "labels outside [-%d, %d)" % (_label_count(a), _label_count(a)))
            else:
                check(name, a)
        result = inner(*a.values())           # positionally: handlers differ in some parameter names
        if self.check_finite and name != "is_fully_finite":
            for pname, value in a.items():
                if pname in NON_ARRAY and isinstance(value, (numbers.Real, np.floating)) and not np.isfinite(value):
                    raise ValueError('%s: NaN or Inf in argument "%s"' % (name, pname))
            for pname, value in arrays:
                if value.size and not self.handler.is_fully_finite(value):
                    raise ValueError('%s: NaN or Inf in "%s" after the call' % (name, pname))
        return result if name in RETURNING else None

    method.__name__ = name
    method.__doc__ = "Checked %s: contract of debug_handler.py, then the wrapped handler's %s." % (name, name)
    return method


def _interface_signature(name):
    """Parameters of an operation as the handler interface names them, without self."""
    if name == "mult_add_mv":             # called by the LSTM layers, not declared by the interface
        name = "add_mv"                   # same parameters (m, v, out)
    sig = inspect.signature(getattr(_MirrorHandler, name))
    return sig.replace(parameters=list(sig.parameters.values())[1:])


_SIGNATURES = {name: _interface_signature(name) for name in CONTRACTS}


class _CheckedBase(Handler):
    __undescribed__ = {"EMPTY", "array_type", "inplace_act_func", "inplace_act_func_deriv", "act_func",
                       "act_func_deriv"}

    def __init__(self, handler, check_finite=False):
        super().__init__()
        self.handler = handler
        self.check_finite = bool(check_finite)
        self.dtype = handler.dtype
        self.context = getattr(handler, "context", None)
        self.EMPTY = handler.EMPTY
        self.rnd = handler.rnd
        self.array_type = handler.array_type
        self._signatures = _SIGNATURES

    def __init_from_description__(self, description):
        self.__init__(self.handler)

    def __getattr__(self, name):
        # extensions of the wrapped handler (fused layer steps, synchronize, ...) pass through unchecked
        if name.startswith("__") or name == "handler":
            raise AttributeError(name)
        return getattr(self.handler, name)


CheckedHandler = type("CheckedHandler", (_CheckedBase,),
                      dict({name: _make_method(name) for name in CONTRACTS},
                           __doc__=__doc__, __module__=__name__))

assert set(HANDLER_METHODS) <= set(CONTRACTS), sorted(set(HANDLER_METHODS) - set(CONTRACTS))
