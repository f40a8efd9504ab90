"""Handler-call sequences that stand for brainstorm's value and gradient modifiers in the tests.

Each function returns a callable that issues handler operations only, the way a modifier of the
reference drives a handler after an update (trainer.py:101 -> network.py:490-495) or at the end
of the backward pass (network.py:445). Weight hooks are called with (handler, view), gradient
hooks with (handler, parameters, gradients). They exist to exercise the handler (among others
the ``*`` and ``**`` operators of the handler's arrays, the one place value_modifiers.py:79-80
needs them); they are not part of the library.
"""
import numpy as np


def cap_row_norms(limit, with_operators=True):
    """Rows of the view (flattened to two axes) longer than `limit` in the 2-norm are scaled back to it."""
    def hook(h, view):
        if len(view.shape) < 2:
            return
        rows = view.shape[0]
        m = view.reshape((rows, view.size // rows))
        scale = h.allocate((rows, 1))
        if with_operators:
            h.sum_t(m * m, axis=1, out=scale)
            h.mult_st(1.0 / limit, scale ** 0.5, out=scale)
        else:
            squares = h.allocate(m.shape)
            h.mult_tt(m, m, squares)
            h.sum_t(squares, axis=1, out=scale)
            h.sqrt_t(scale, scale)
            h.mult_st(1.0 / limit, scale, out=scale)
        h.clip_t(scale, 1.0, float(np.finfo(h.dtype).max), scale)
        h.divide_mv(m, scale, m)
    return hook


def clamp(low, high):
    return lambda h, view: h.clip_t(view, low, high, view)


def keep_where(mask):
    """Multiplies the view with a fixed 0/1 array, uploaded on first use."""
    held = {}

    def hook(h, view):
        if id(h) not in held:
            held[id(h)] = h.create_from_numpy(mask)
        h.mult_tt(view, held[id(h)], view)
    return hook


def hold_values(values=None):
    """Puts the view back to `values` (or to what it held at the first call) every time."""
    held = {}

    def hook(h, view):
        if "host" not in held:
            held["host"] = h.get_numpy_copy(view) if values is None else np.asarray(values)
        if id(h) not in held:
            held[id(h)] = h.create_from_numpy(held["host"])
        h.copy_to(held[id(h)], view)
    return hook


def shrink_l1(factor):
    """gradients += factor * sign(parameters)"""
    def hook(h, parameters, gradients):
        signs = h.allocate(parameters.shape)
        h.sign_t(parameters, signs)
        h.mult_add_st(factor, signs, gradients)
    return hook


def shrink_l2(factor):
    """gradients += factor * parameters"""
    return lambda h, parameters, gradients: h.mult_add_st(factor, parameters, gradients)


def on_gradients(weight_hook):
    """A weight hook applied to the gradients (the parameters are ignored)."""
    return lambda h, parameters, gradients: weight_hook(h, gradients)
