"""HipHandler: brainstorm's Handler interface on one MI355X.

Every method forwards to one (sometimes two) C calls of libbship.so, which
enqueue hand-written gfx950 kernels on the library's stream and return at
once. Only ``get_numpy_copy``, ``set_from_numpy``/``create_from_numpy``,
``is_fully_finite`` and ``fill_gaussian`` wait for the device.

Semantics follow brainstorm's NumpyHandler (brainstorm/handlers/numpy_handler.py)
operation by operation; the line of the reference each method mirrors is given
next to it. The handler computes in float32 only, like the reference's GPU
handler (pycuda_handler.py:31).
"""
from __future__ import annotations

import ctypes

import numpy as np

from . import _lib
try:
    from . import _fastcall
except ImportError as exc:          # no fallback: the extension is part of the build
    raise ImportError("brainstorm_amd._fastcall is not built; run `python -m brainstorm_amd.build` (%s)" % exc)
from ._lib import (ABS, ADD, ADD_IF, ADD_ST, COPY_IF, DIV, EL, EL_DERIV, FILL_IF, FMOD, LOG, MUL,
                   MULT_ADD_ST, MULT_ST, PITCHED_BINARY, PITCHED_CLIP, PITCHED_COND, PITCHED_DERIV,
                   PITCHED_FILL, PITCHED_MULT_ADD, PITCHED_SCALAR, PITCHED_UNARY, REL, REL_DERIV, SIGMOID,
                   SIGMOID_DERIV, SIGN, SQRT, SUB, TANH, TANH_DERIV)
from .device_array import DeviceArray, PitchedDeviceArray, _Block, _prod
from .handler_api import Handler

SEED_RANGE = (0, 1000000000)   # brainstorm/randomness.py:16


class HipRandomState:
    """The handler's random state: an MT19937 stream kept in device memory.

    Mirrors the seed bookkeeping of brainstorm.randomness.RandomState
    (randomness.py:10-64): it remembers its seed, can be re-seeded and reset.
    The stream equals numpy.random.RandomState(seed)'s, so masks drawn here
    equal the ones NumpyHandler draws from the same seed.

    Every instance is a generator of its own in the library (bship_rng_create), as every
    reference handler has its own ``self.rnd`` (numpy_handler.py:21): handlers that are alive
    together do not disturb each other's streams. Every random call names its generator, so the
    library selects and draws under one lock (handlers may be driven from different threads).
    """

    def __init__(self, handler, seed=None):
        self._handler = handler
        self._lib = handler._lib
        gid = ctypes.c_int()
        handler._call(self._lib.bship_rng_create(ctypes.byref(gid)))
        self._id = gid.value
        if seed is None:
            seed = int(np.random.randint(*SEED_RANGE))
        self.seed(seed)

    def select(self):
        """Makes this generator the one that the library's unnamed random calls and recordings use."""
        st = self._lib.bship_rng_select(self._id)
        if st:
            self._handler._call(st)

    def __del__(self):
        try:
            if self._id is not None and self._lib is not None:
                self._lib.bship_rng_destroy(self._id)
                self._id = None
        except Exception:
            pass

    def seed(self, seed=None):
        if seed is None:
            seed = int(np.random.randint(*SEED_RANGE))
        seed = int(seed)
        if not 0 <= seed < 2 ** 32:
            raise ValueError("seed must be between 0 and 2**32 - 1")
        self._handler._call(self._lib.bship_rng_seed_on(self._id, seed))
        if self._handler.fast_masks:               # the optional mask stream restarts with it
            self._handler._call(self._lib.bship_fast_rng_seed_on(self._id, seed))
        self._seed = seed

    def get_seed(self):
        return self._seed

    def set_seed(self, seed):
        self.seed(seed)

    def reset(self):
        self.seed(self._seed)

    def get_state(self):
        """('MT19937', key, pos, has_gauss, cached_gaussian) like RandomState.get_state()."""
        key = (ctypes.c_uint32 * 624)()
        pos, has_gauss, gauss = ctypes.c_int(), ctypes.c_int(), ctypes.c_double()
        h = self._handler
        h._call(h._lib.bship_rng_get_state_on(self._id, key, ctypes.byref(pos), ctypes.byref(has_gauss),
                                              ctypes.byref(gauss)))
        return ('MT19937', np.frombuffer(key, dtype=np.uint32).copy(), pos.value,
                has_gauss.value, gauss.value)


class RecordedStep(object):
    """A recorded sequence of handler calls (see :meth:`HipHandler.record`)."""

    def __init__(self, handler, graph_id):
        self._handler = handler
        self._id = graph_id

    def replay(self):
        if self._id is None:
            raise RuntimeError("this recorded step has been released")
        self._handler._call(self._handler._lib.bship_graph_launch(self._id))

    def release(self):
        if self._id is not None:
            gid, self._id = self._id, None
            self._handler._call(self._handler._lib.bship_graph_destroy(gid))

    def __del__(self):
        try:
            if self._id is not None and self._handler._lib is not None:
                self._handler._lib.bship_graph_destroy(self._id)
                self._id = None
        except Exception:
            pass


def _mismatch(op, *arrays):
    """NumPy raises ValueError when the operands of `out[:] = a + b` cannot be combined
    (numpy_handler.py:86-87); the kernels take one element count and raw addresses, so operands
    of different sizes are refused here, before anything reaches the device."""
    return ValueError("%s: operands with shapes %s do not match"
                      % (op, ", ".join(repr(tuple(a.shape)) for a in arrays)))


class _NoNativePath(Exception):
    """The operands of a call on row-pitched views do not fit the row-pitched kernels."""


def _without_self(arguments):
    return {k: v for k, v in arguments.items() if k != "self"}


def _native_pitched_table():
    """Handler operation -> function(handler, arguments) that runs it on row-pitched operands as they
    are (bship_elementwise_pitched_f32, bship_sum_pitched_f32, bship_copy2d_f32)."""
    def ew(family, op, out, a=None, b=None, s0=None, s1=None):
        def run(h, A):
            h._pitched_elementwise(family, op, A[out], A[a] if a else None, A[b] if b else None,
                                   A[s0] if s0 else 0.0, A[s1] if s1 else 0.0)
        return run

    def mv(family, op):
        def run(h, A):
            h._pitched_elementwise(family, op, A["out"], A["m"], A["v"], 0.0, 0.0, b_is_vector=True)
        return run

    table = {"mult_add_tt": ew(PITCHED_MULT_ADD, 0, "out", "a", "b"),
             "clip_t": ew(PITCHED_CLIP, 0, "out", "a", None, "a_min", "a_max"),
             "fill": ew(PITCHED_FILL, 0, "mem", None, None, "val"),
             "copy_to_if": ew(PITCHED_COND, COPY_IF, "dest", "src", "cond"),
             "fill_if": ew(PITCHED_COND, FILL_IF, "mem", None, "cond", "val"),
             "add_into_if": ew(PITCHED_COND, ADD_IF, "out", "a", "cond"),
             "mult_add_mv": mv(PITCHED_MULT_ADD, 0),
             "copy_to": lambda h, A: h._pitched_copy(A["src"], A["dest"]),
             "softmax_m": lambda h, A: h._pitched_softmax(A["m"], A["out"]),
             "binarize_v": lambda h, A: h._pitched_binarize(A["v"], A["out"]),
             "index_m_by_v": lambda h, A: h._pitched_index(A["m"], A["v"], A["out"]),
             "sum_t": lambda h, A: h._pitched_sum(A["a"], A["axis"], A["out"]),
             "generate_probability_mask": lambda h, A: h._pitched_mask(A["mask"], A["probability"]),
             "broadcast_t": lambda h, A: h._pitched_broadcast(A["a"], A["axis"], A["out"]),
             "merge_tt": lambda h, A: h._pitched_merge(A["a"], A["b"], A["out"]),
             "split_add_tt": lambda h, A: h._pitched_split_add(A["x"], A["out_a"], A["out_b"]),
             "maxpool2d_forward_batch": lambda h, A: h._pitched_maxpool_fwd(**_without_self(A)),
             "maxpool2d_backward_batch": lambda h, A: h._pitched_maxpool_bwd(**_without_self(A)),
             "avgpool2d_forward_batch": lambda h, A: h._pitched_avgpool_fwd(**_without_self(A)),
             "avgpool2d_backward_batch": lambda h, A: h._pitched_avgpool_bwd(**_without_self(A)),
             "conv2d_forward_batch": lambda h, A: h._pitched_conv_fwd(**_without_self(A)),
             "conv2d_backward_batch": lambda h, A: h._pitched_conv_bwd(**_without_self(A))}
    for name, op in (("add", ADD), ("subtract", SUB), ("mult", MUL), ("divide", DIV)):
        table[name + "_tt"] = ew(PITCHED_BINARY, op, "out", "a", "b")
        table[name + "_mv"] = mv(PITCHED_BINARY, op)
    table["modulo_tt"] = ew(PITCHED_BINARY, FMOD, "out", "a", "b")
    for name, op in (("add_st", ADD_ST), ("mult_st", MULT_ST), ("mult_add_st", MULT_ADD_ST)):
        table[name] = ew(PITCHED_SCALAR, op, "out", "t", None, "s")
    for name, op in (("abs_t", ABS), ("sign_t", SIGN), ("sqrt_t", SQRT), ("log_t", LOG)):
        table[name] = ew(PITCHED_UNARY, op, "out", "a")
    for name, op, dop in (("sigmoid", SIGMOID, SIGMOID_DERIV), ("tanh", TANH, TANH_DERIV),
                          ("rel", REL, REL_DERIV), ("el", EL, EL_DERIV)):
        table[name] = ew(PITCHED_UNARY, op, "y", "x")
        table[name + "_deriv"] = ew(PITCHED_DERIV, dop, "dx", "y", "dy")
    return table


class HipHandler(Handler):
    __undescribed__ = {'context', 'dtype', 'EMPTY', 'rnd'}

    array_type = DeviceArray
    ERR_TIMEOUT = _lib.ERR_TIMEOUT      # status of the BshipError that lstm_forward_sequence raises when a barrier ran out

    def __init__(self, seed=None, device=0, pitched_views=False, fast_masks=False, fusing=True):
        # fusing: the library's fusing window. brainstorm's layers issue primitive operations only; with
        # the window on, the library recognises the layers' call sequences (an LSTM time step, a batch
        # normalisation pass, bias + activation, dropout, softmax cross entropy, Highway, the momentum
        # update) and runs each as one fused kernel with the same float32 operations in the same order,
        # so results are the same bits as with fusing=False. fusing="stacked" additionally runs the four
        # recurrent matrix products of an LSTM time step as one product over the stacked weight matrices
        # (adjacent in brainstorm's parameter vector): faster, and equal to the other modes up to the order in
        # which a matrix product sums (about 1e-6 relative), not bit for bit. The switch is the library's: it
        # holds for every handler of the process (the last handler created, or set_fusing, decides).
        # fast_masks: dropout masks from a counter-based generator (Philox4x32-10) instead of
        # NumPy's MT19937 stream. One parallel launch per mask instead of a sequential walk, but
        # NOT the masks NumpyHandler draws for the same seed (the reference's own GPU handler does
        # not match NumPy either, pycuda_handler.py:37-39). fill_gaussian keeps NumPy's stream.
        # pitched_views: let slices that need a row pitch (feature slices of a hub with several
        # sources, buffer_structure.py:232-245) exist as PitchedDeviceArray and serve operations
        # on them through dense temporaries. Off by default: it puts a Python-level argument
        # check in front of every operation.
        self.pitched_views = bool(pitched_views)
        self.native_pitched = True      # False: every call on a pitched view goes through dense temporaries
        self.thin_convolutions = True   # False: convolutions with thin filters take the im2col path like all others
        if self.pitched_views:
            self._install_pitched_wrappers()        # before the activation tables bind the methods
        super(HipHandler, self).__init__()
        self._lib = _lib.load()
        self._call(self._lib.bship_init(int(device)))
        # the operations a network step issues by the thousand are called without ctypes' per-argument
        # conversions (csrc/fastcall.c); everything else goes through ctypes
        fast = _fastcall.Calls(_lib.entry_point_addresses(self._lib))
        self._fast = fast
        (self._binary, self._mult_add, self._scalar, self._unary, self._deriv, self._clip, self._mv_call,
         self._fill_call, self._gemm_call, self._d2d, self._sum_call) = (
            fast.binary, fast.mult_add_tt, fast.scalar, fast.unary, fast.deriv, fast.clip, fast.mv, fast.fill,
            fast.gemm, fast.d2d, fast.sum)
        self.dtype = np.float32
        self.device = int(device)
        self.context = self._lib
        self._free = self._lib.bship_free
        self.EMPTY = DeviceArray(0, (0,), None, self)
        self.fast_masks = bool(fast_masks)
        self.set_fusing(fusing)
        self.rnd = HipRandomState(self, seed)

    def __describe__(self):
        # the constructor's settings travel with a saved network description, as NumpyHandler's
        # dtype does (numpy_handler.py:25-33); the seed does not (the reference's does not either)
        return {'@type': self.__class__.__name__, 'device': self.device,
                'pitched_views': self.pitched_views, 'fast_masks': self.fast_masks, 'fusing': self.fusing}

    def __init_from_description__(self, description):
        self.__init__(device=int(description.get('device', 0)),
                      pitched_views=bool(description.get('pitched_views', False)),
                      fast_masks=bool(description.get('fast_masks', False)),
                      fusing=description.get('fusing', True))

    # ------------------------------------------------------------- plumbing
    # parameters an operation writes (everything else is only read); operations that are not
    # listed (the fused extensions) are assumed to write every array they get
    _WRITTEN = {
        "copy_to": ("dest",), "copy_to_if": ("dest",), "fill": ("mem",), "fill_if": ("mem",),
        "set_from_numpy": ("mem",), "get_numpy_copy": (), "is_fully_finite": (),
        "split_add_tt": ("out_a", "out_b"), "generate_probability_mask": ("mask",),
        "conv2d_forward_batch": ("outputs",),
        "conv2d_backward_batch": ("in_deltas", "weight_deltas", "bias_deltas"),
        "maxpool2d_forward_batch": ("outputs", "argmax"), "maxpool2d_backward_batch": ("in_deltas",),
        "avgpool2d_forward_batch": ("outputs",), "avgpool2d_backward_batch": ("in_deltas",),
        "sigmoid": ("y",), "tanh": ("y",), "rel": ("y",), "el": ("y",),
        "sigmoid_deriv": ("dx",), "tanh_deriv": ("dx",), "rel_deriv": ("dx",), "el_deriv": ("dx",),
        "dropout_forward": ("mask", "out"),
        "softmax_ce_forward": ("probs", "loss"), "softmax_ce_backward": ("t_bin", "dinputs"),
        "momentum_update": ("velocity", "parameters"),
        "batchnorm_forward": ("mu", "sigma", "sigma_b", "centered", "x_hat", "out"),
        "batchnorm_backward": ("dgamma", "dbeta", "in_deltas"),
    }

    def _install_pitched_wrappers(self):
        import functools
        import inspect
        cls = type(self)
        for name in dir(cls):
            if name.startswith("_") or name in ("allocate", "zeros", "ones", "create_from_numpy",
                                                "synchronize", "device_info", "stack_adjacent",
                                                "record", "dot_mm", "dot_add_mm"):
                continue                          # matrix products take row pitches natively (_gemm)
            fn = getattr(cls, name)
            if not inspect.isfunction(fn):
                continue
            sig = inspect.signature(fn)
            written = self._WRITTEN.get(name, ("out",) if "out" in sig.parameters else None)
            setattr(self, name, functools.partial(self._dense_call, fn, sig, written))

    def _copy2d(self, pitched, dense, to_dense):
        cols = pitched.run
        args = ((dense.ptr, cols, pitched._base, pitched.pitch) if to_dense
                else (pitched._base, pitched.pitch, dense.ptr, cols))
        self._call(self._lib.bship_copy2d_f32(*args, pitched.rows, cols))

    _NATIVE_PITCHED = _native_pitched_table()

    def _as_matrix(self, a, rows, cols):
        """(address, elements from row to row) of `a` read as a (rows, cols) matrix."""
        if type(a) is PitchedDeviceArray:
            if a.run != cols or a.rows != rows:
                raise _NoNativePath()
            return a._base, a.pitch
        if a.size != rows * cols:
            raise _NoNativePath()
        return a.ptr, cols

    @staticmethod
    def _common_run(*arrays):
        """The row length operands are read with: the run of the pitched ones (the same for all
        of them), else the last axis of the first."""
        runs = {x.run for x in arrays if type(x) is PitchedDeviceArray}
        if len(runs) > 1:
            raise _NoNativePath()
        if runs:
            return runs.pop()
        first = arrays[0]
        return first.shape[-1] if first.shape else 1

    def _pitched_elementwise(self, family, op, out, a, b, s0, s1, b_is_vector=False):
        if b_is_vector:
            cols = out.shape[-1] if out.shape else 1        # the matrix of a matrix-vector operation
        else:
            cols = self._common_run(*[x for x in (out, a, b) if x is not None])
        rows = out.size // cols if cols else 0
        po, ldo = self._as_matrix(out, rows, cols)
        pa, lda = self._as_matrix(a, rows, cols) if a is not None else (None, 0)
        pb, rsb, csb = None, 0, 1
        if b is not None and b_is_vector and b.shape != a.shape:
            vs = b.shape
            pitched = type(b) is PitchedDeviceArray
            if b.size == cols and (len(vs) == 1 or vs[0] == 1 or rows == 1) and not (pitched and b.rows != 1):
                pb, rsb, csb = b._address(), 0, 1                      # row vector
            elif b.size == rows and vs[-1] == 1:
                pb, rsb, csb = b._address(), (b.pitch if pitched else 1), 0     # column vector
            else:
                raise _NoNativePath()
        elif b is not None:
            pb, rsb = self._as_matrix(b, rows, cols)
        self._call(self._lib.bship_elementwise_pitched_f32(family, op, s0, s1, pa, lda, 1, pb, rsb, csb,
                                                           po, ldo, rows, cols))

    def _pitched_copy(self, src, dest):
        cols = self._common_run(dest, src)
        rows = dest.size // cols if cols else 0
        pd, ldd = self._as_matrix(dest, rows, cols)
        ps, lds = self._as_matrix(src, rows, cols)
        self._call(self._lib.bship_copy2d_f32(pd, ldd, ps, lds, rows, cols))

    def _as_column(self, v, rows):
        """(address, elements from entry to entry) of `v` read as a column of `rows` entries."""
        if v.size != rows:
            raise _NoNativePath()
        if type(v) is PitchedDeviceArray:
            if v.run != 1:
                raise _NoNativePath()
            return v._base, v.pitch
        return v.ptr, 1

    def _pitched_softmax(self, m, out):
        if m.ndim != 2 or out.shape != m.shape:
            raise _NoNativePath()
        rows, cols = m.shape
        pm, ldm = self._as_matrix(m, rows, cols)
        po, ldo = self._as_matrix(out, rows, cols)
        self._call(self._lib.bship_softmax_rows_pitched_f32(pm, ldm, po, ldo, rows, cols))

    def _pitched_binarize(self, v, out):
        if out.ndim != 2:
            raise _NoNativePath()
        rows, k = out.shape
        pv, ldv = self._as_column(v, rows)
        po, ldo = self._as_matrix(out, rows, k)
        self._call(self._lib.bship_binarize_pitched_f32(pv, ldv, po, ldo, rows, k))

    def _pitched_index(self, m, v, out):
        if m.ndim != 2:
            raise _NoNativePath()
        rows, k = m.shape
        pm, ldm = self._as_matrix(m, rows, k)
        pv, ldv = self._as_column(v, rows)
        po, ldo = self._as_column(out, rows)
        self._call(self._lib.bship_index_m_by_v_pitched_f32(pm, ldm, pv, ldv, po, ldo, rows, k))

    def _pitched_sum(self, a, axis, out):
        if (type(a) is not PitchedDeviceArray or type(out) is PitchedDeviceArray
                or (axis is not None and (a.ndim != 2 or axis not in (0, 1)))):
            raise _NoNativePath()
        cols = a.run
        if axis is not None and cols != a.shape[-1]:
            raise _NoNativePath()
        self._call(self._lib.bship_sum_pitched_f32(a._base, a.pitch, out.ptr, a.rows, cols,
                                                   -1 if axis is None else axis))

    # ---- operations on image-pitched and run-pitched views, no dense temporaries ----
    def _pitched_mask(self, mask, probability):
        if self.fast_masks or type(mask) is not PitchedDeviceArray:
            raise _NoNativePath()
        self._call(self._lib.bship_prob_mask_pitched_on_f32(self.rnd._id, mask._base, mask.pitch, mask.rows, mask.run,
                                                            probability))

    @staticmethod
    def _runs(a):
        """(address, run, elements from run to run) of any array."""
        if type(a) is PitchedDeviceArray:
            return a._base, a.run, a.pitch
        return a.ptr, max(a.size, 1), max(a.size, 1)

    def _pitched_broadcast(self, a, axis, out):
        assert (out.shape[:axis] + (1,) + out.shape[axis + 1:]) == a.shape
        if out.size >= 2 ** 32:
            raise _NoNativePath()
        outer = _prod(out.shape[:axis])
        inner = _prod(out.shape[axis + 1:])
        pa, ra, lda = self._runs(a)
        po, ro, ldo = self._runs(out)
        self._call(self._lib.bship_broadcast_pitched_f32(pa, ra, lda, po, ro, ldo, outer, out.shape[axis], inner))

    def _as_rows(self, a, cols):
        """`a` as a (rows, cols) matrix view that can be sliced by columns."""
        if type(a) is PitchedDeviceArray and a.run != cols:
            raise _NoNativePath()
        return a.reshape((a.size // cols, cols))

    def _pitched_merge(self, a, b, out):
        # out[..., :na] = a; out[..., na:] = b   (numpy 221-225): two strided copies
        na, nb = a.shape[-1], b.shape[-1]
        assert na + nb == out.shape[-1]
        if 0 in (na, nb, out.size):
            raise _NoNativePath()
        o2 = self._as_rows(out, na + nb)
        self._pitched_copy(self._as_rows(a, na), o2[:, :na])
        self._pitched_copy(self._as_rows(b, nb), o2[:, na:])

    def _pitched_split_add(self, x, out_a, out_b):
        # out_a += x[..., :na]; out_b += x[..., na:]   (numpy 251-256): two strided additions
        na, nb = out_a.shape[-1], out_b.shape[-1]
        assert na + nb == x.shape[-1]
        if 0 in (na, nb, x.size):
            raise _NoNativePath()
        x2 = self._as_rows(x, na + nb)
        oa, ob = self._as_rows(out_a, na), self._as_rows(out_b, nb)
        self._pitched_elementwise(PITCHED_BINARY, ADD, oa, x2[:, :na], oa, 0.0, 0.0)
        self._pitched_elementwise(PITCHED_BINARY, ADD, ob, x2[:, na:], ob, 0.0, 0.0)

    @staticmethod
    def _images(a):
        """(address, elements from image to image) of an (n, h, w, c) array."""
        image = _prod(a.shape[1:])
        if type(a) is PitchedDeviceArray:
            if a.run != image:
                raise _NoNativePath()
            return a._base, a.pitch
        return a.ptr, image

    def _pitched_maxpool_fwd(self, inputs, window, outputs, padding, stride, argmax, **_):
        n, h, w, c = inputs.shape
        self._window_geometry("maxpool2d_forward_batch", inputs, window, outputs, padding, stride, c)
        (pi, li), (po, lo), (pa, la) = self._images(inputs), self._images(outputs), self._images(argmax)
        self._call(self._lib.bship_maxpool_fwd_nhwc_pitched_f32(
            pi, li, po, lo, pa, la, n, h, w, c, outputs.shape[1], outputs.shape[2], window[0], window[1],
            padding, stride[0], stride[1]))

    def _pitched_maxpool_bwd(self, inputs, window, outputs, padding, stride, argmax, in_deltas, out_deltas, **_):
        n, h, w, c = inputs.shape
        self._window_geometry("maxpool2d_backward_batch", inputs, window, outputs, padding, stride, c)
        (pa, la), (pd, ld), (pi, li) = self._images(argmax), self._images(out_deltas), self._images(in_deltas)
        self._call(self._lib.bship_maxpool_bwd_nhwc_pitched_f32(
            pa, la, pd, ld, pi, li, n, h, w, c, outputs.shape[1], outputs.shape[2], window[0], window[1],
            padding, stride[0], stride[1]))

    def _pitched_avgpool_fwd(self, inputs, window, outputs, padding, stride, **_):
        n, h, w, c = inputs.shape
        self._window_geometry("avgpool2d_forward_batch", inputs, window, outputs, padding, stride, c)
        (pi, li), (po, lo) = self._images(inputs), self._images(outputs)
        self._call(self._lib.bship_avgpool_fwd_nhwc_pitched_f32(
            pi, li, po, lo, n, h, w, c, outputs.shape[1], outputs.shape[2], window[0], window[1],
            padding, stride[0], stride[1]))

    def _pitched_avgpool_bwd(self, inputs, window, outputs, padding, stride, in_deltas, out_deltas, **_):
        n, h, w, c = inputs.shape
        self._window_geometry("avgpool2d_backward_batch", inputs, window, outputs, padding, stride, c)
        (pd, ld), (pi, li) = self._images(out_deltas), self._images(in_deltas)
        self._call(self._lib.bship_avgpool_bwd_nhwc_pitched_f32(
            pd, ld, pi, li, n, h, w, c, outputs.shape[1], outputs.shape[2], window[0], window[1],
            padding, stride[0], stride[1]))

    def _densified(self, a):
        """A dense copy of a pitched array (for operands of the convolutions' matrix products)."""
        if type(a) is not PitchedDeviceArray:
            return a
        t = self._scratch(a.shape)
        self._copy2d(a, t, True)
        return t

    def _pitched_conv_fwd(self, inputs, weights, bias, outputs, padding, stride, **_):
        # im2col reads the image-pitched inputs as they are; the product's result is a matrix over
        # all images, so pitched outputs receive it through one dense block and one strided copy
        weights, bias = self._densified(weights), self._densified(bias)
        out = self._scratch(outputs.shape) if type(outputs) is PitchedDeviceArray else outputs
        self._conv_forward(inputs, weights, bias, out, padding, stride)
        if out is not outputs:
            self._copy2d(outputs, out, False)

    def _pitched_conv_bwd(self, inputs, weights, padding, stride, in_deltas, out_deltas, weight_deltas,
                          bias_deltas, **_):
        if type(weight_deltas) is PitchedDeviceArray or type(bias_deltas) is PitchedDeviceArray:
            raise _NoNativePath()
        self._conv_backward(inputs, self._densified(weights), padding, stride, in_deltas,
                            self._densified(out_deltas), weight_deltas, bias_deltas)

    def _dense_call(self, fn, sig, written, *args, **kwargs):
        """Runs fn on row-pitched operands: with the row-pitched kernels where they cover the call,
        else with every such operand replaced by a dense temporary."""
        for a in args:
            if type(a) is PitchedDeviceArray:
                break
        else:
            for a in kwargs.values():
                if type(a) is PitchedDeviceArray:
                    break
            else:
                return fn(self, *args, **kwargs)         # the usual case: nothing to do
        bound = sig.bind(self, *args, **kwargs)
        native = self._NATIVE_PITCHED.get(fn.__name__) if self.native_pitched else None
        if native is not None:
            try:
                return native(self, bound.arguments)
            except _NoNativePath:
                pass                                 # e.g. operands of different row lengths
        pitched = [(k, a) for k, a in bound.arguments.items() if type(a) is PitchedDeviceArray]
        temps = {}
        for name, a in pitched:
            key = (a._base, a.shape, a.pitch)
            if key not in temps:                 # the same view twice (out is an input): one temporary
                t = self._scratch(a.shape)
                self._copy2d(a, t, True)
                temps[key] = t
            bound.arguments[name] = temps[key]
        result = fn(*bound.args, **bound.kwargs)
        done = set()
        for name, a in pitched:
            key = (a._base, a.shape, a.pitch)
            if (written is None or name in written) and key not in done:
                self._copy2d(a, temps[key], False)
                done.add(key)
        return result

    def _call(self, status):
        if status:
            _lib.raise_for_status(self._lib, status)

    def synchronize(self):
        """Waits until every operation issued so far has finished."""
        self._call(self._lib.bship_sync())

    def set_fusing(self, mode):
        """Switches the library's fusing window: False, True (same bits as False) or "stacked" (see the
        constructor). What the window holds is enqueued first."""
        if mode not in (True, False, "stacked"):
            raise ValueError('fusing must be True, False or "stacked", not %r' % (mode,))
        self._call(self._lib.bship_fusing_set(2 if mode == "stacked" else int(mode)))
        self.fusing = mode

    def fusing_stats(self, reset=False):
        """Counters of the fusing window since the last reset: operations that entered it, operations
        enqueued as they were, operations replaced by fused launches, fused launches, matrix products
        that overtook held operations."""
        vals = [ctypes.c_ulonglong() for _ in range(5)]
        self._call(self._lib.bship_fusing_stats(*[ctypes.byref(v) for v in vals], int(bool(reset))))
        return dict(zip(("calls", "unfused", "fused_calls", "fused_launches", "overtaken"), (v.value for v in vals)))

    # --------------------------------------------------- recorded steps
    def record(self, fn):
        """Runs ``fn()`` once in recording mode and returns a :class:`RecordedStep`.

        While recording, the handler calls made by ``fn`` are captured, not executed; the
        returned object's ``replay()`` then issues all of them with one launch. ``fn`` must not
        read results back or upload data (``get_numpy_copy``, ``set_from_numpy``,
        ``is_fully_finite``, ``fill_gaussian``, ``synchronize`` raise while recording): place
        those around the replay. Arrays that ``fn`` allocates keep their memory for as long
        as the recording exists. Shapes and addresses are fixed at recording time.
        """
        self.rnd.select()        # the recording's masks come from this handler's generator, on every replay
        self._call(self._lib.bship_graph_begin())
        try:
            fn()
        except BaseException:
            gid = ctypes.c_int()
            if self._lib.bship_graph_end(ctypes.byref(gid)) == 0:
                self._lib.bship_graph_destroy(gid.value)
            raise
        gid = ctypes.c_int()
        self._call(self._lib.bship_graph_end(ctypes.byref(gid)))
        return RecordedStep(self, gid.value)

    def device_info(self):
        name = ctypes.create_string_buffer(256)
        cus = ctypes.c_int()
        self._call(self._lib.bship_device_info(name, 256, ctypes.byref(cus)))
        return name.value.decode(), cus.value

    # ------------------------------------------------- allocate new memory
    def allocate(self, shape):
        # numpy 36-37 / pycuda 70-71: "allocate" hands out zeros
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        shape = tuple(int(s) for s in shape)
        n = _prod(shape)
        if n == 0:
            return DeviceArray(0, shape, None, self)
        p = ctypes.c_void_p()
        self._call(self._lib.bship_malloc(n * 4, ctypes.byref(p)))
        return DeviceArray(p.value, shape, _Block(p.value, self._free), self)

    def _scratch(self, shape):
        """An array with arbitrary content, for buffers that are overwritten completely before use."""
        n = _prod(shape)
        if n == 0:
            return DeviceArray(0, tuple(shape), None, self)
        p = ctypes.c_void_p()
        self._call(self._lib.bship_malloc_scratch(n * 4, ctypes.byref(p)))
        return DeviceArray(p.value, tuple(shape), _Block(p.value, self._free), self)

    def empty(self, shape):
        """Like :meth:`allocate`, but with arbitrary content: for buffers that are overwritten completely
        before they are read (allocate's zero fill of a large buffer is a pass over memory)."""
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        return self._scratch(tuple(int(s) for s in shape))

    def zeros(self, shape):
        return self.allocate(shape)

    def ones(self, shape):
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        a = self._scratch(tuple(int(s) for s in shape))
        self.fill(a, 1.0)
        return a

    # --------------------------------------------------------- copy and fill
    def copy_to(self, src, dest):
        # numpy 47-52 / pycuda 83-85: np.copyto broadcasts src to dest's shape (a scalar, a row for every
        # row, a column for every column, ...). Every run of neighbouring axes that repeat is one broadcast_t.
        if src.shape == dest.shape:
            st = self._d2d(dest.ptr, src.ptr, dest.size * 4)
            if st:
                self._call(st)
            return
        if src.ndim > dest.ndim:
            raise ValueError("copy_to: could not broadcast %r into %r" % (src.shape, dest.shape))
        shape = (1,) * (dest.ndim - src.ndim) + tuple(src.shape)
        repeat = [k for k, (s, d) in enumerate(zip(shape, dest.shape)) if s != d]
        if any(shape[k] != 1 for k in repeat):
            raise ValueError("copy_to: could not broadcast %r into %r" % (src.shape, dest.shape))
        if dest.size == 0:
            return
        if not repeat:                       # only leading axes of length 1 differ
            self._call(self._lib.bship_d2d(dest.ptr, src.ptr, dest.size * 4))
            return
        runs = [[repeat[0], repeat[0]]]
        for k in repeat[1:]:
            if k == runs[-1][1] + 1:
                runs[-1][1] = k
            else:
                runs.append([k, k])
        current, shape = src, list(shape)
        for first, last in reversed(runs):   # innermost run first: the intermediate arrays stay small
            outer, inner = _prod(shape[:first]), _prod(shape[last + 1:])
            times = _prod(dest.shape[first:last + 1])
            shape[first:last + 1] = dest.shape[first:last + 1]
            out = dest if [first, last] == runs[0] else self._scratch(tuple(shape))
            self._call(self._lib.bship_broadcast_f32(current.ptr, out.ptr, outer, times, inner))
            current = out

    def copy_to_if(self, src, dest, cond):
        if src.size != dest.size or cond.size != dest.size:
            raise _mismatch("copy_to_if", src, dest, cond)
        self._call(self._lib.bship_cond_f32(COPY_IF, src.ptr, 0.0, dest.ptr, cond.ptr, dest.size))

    def create_from_numpy(self, arr):
        arr = np.asarray(arr, dtype=np.float32, order='C')    # keeps 0-d arrays 0-d
        out = self._scratch(arr.shape)
        if out.size:
            self._call(self._lib.bship_h2d(out.ptr, arr.ctypes.data, arr.nbytes))
        return out

    def fill(self, mem, val):
        st = self._fill_call(mem.ptr, val, mem.size)
        if st:
            self._call(st)

    def fill_if(self, mem, val, cond):
        if cond.size != mem.size:
            raise _mismatch("fill_if", mem, cond)
        self._call(self._lib.bship_cond_f32(FILL_IF, None, val, mem.ptr, cond.ptr, mem.size))

    def get_numpy_copy(self, mem):
        assert type(mem) == self.array_type
        out = np.empty(mem.shape, dtype=np.float32)
        if mem.size:
            self._call(self._lib.bship_d2h(out.ctypes.data, mem.ptr, mem.size * 4))
        return out

    def set_from_numpy(self, mem, arr):
        # numpy 64-65: mem[:] = arr.astype(dtype), which broadcasts
        arr = np.asarray(arr)
        if arr.shape != mem.shape:
            arr = np.broadcast_to(arr, mem.shape)
        arr = np.asarray(arr, dtype=np.float32, order='C')
        if mem.size:
            self._call(self._lib.bship_h2d(mem.ptr, arr.ctypes.data, arr.nbytes))

    # --------------------------------------------------------- debug helper
    def is_fully_finite(self, a):
        res = ctypes.c_int(1)
        self._call(self._lib.bship_isfinite_f32(a.ptr, a.size, ctypes.byref(res)))
        return bool(res.value)

    # ------------------------------------------------ elementwise operations
    def abs_t(self, a, out):
        if a.size != out.size:
            raise _mismatch("abs_t", a, out)
        st = self._unary(ABS, a.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def add_into_if(self, a, out, cond):
        if a.size != out.size or cond.size != out.size:
            raise _mismatch("add_into_if", a, out, cond)
        self._call(self._lib.bship_cond_f32(ADD_IF, a.ptr, 0.0, out.ptr, cond.ptr, out.size))

    def add_st(self, s, t, out):
        if t.size != out.size:
            raise _mismatch("add_st", t, out)
        st = self._scalar(ADD_ST, s, t.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def add_tt(self, a, b, out):
        if a.size != out.size or b.size != out.size:
            raise _mismatch("add_tt", a, b, out)
        st = self._binary(ADD, a.ptr, b.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def clip_t(self, a, a_min, a_max, out):
        if a.size != out.size:
            raise _mismatch("clip_t", a, out)
        st = self._clip(a.ptr, a_min, a_max, out.ptr, out.size)
        if st:
            self._call(st)

    def divide_tt(self, a, b, out):
        if a.size != out.size or b.size != out.size:
            raise _mismatch("divide_tt", a, b, out)
        st = self._binary(DIV, a.ptr, b.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def log_t(self, a, out):
        if a.size != out.size:
            raise _mismatch("log_t", a, out)
        st = self._unary(LOG, a.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def modulo_tt(self, a, b, out):
        if a.size != out.size or b.size != out.size:
            raise _mismatch("modulo_tt", a, b, out)
        st = self._binary(FMOD, a.ptr, b.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def mult_add_st(self, s, t, out):
        if t.size != out.size:
            raise _mismatch("mult_add_st", t, out)
        st = self._scalar(MULT_ADD_ST, s, t.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def mult_add_tt(self, a, b, out):
        if a.size != out.size or b.size != out.size:
            raise _mismatch("mult_add_tt", a, b, out)
        st = self._mult_add(a.ptr, b.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def mult_st(self, s, t, out):
        if t.size != out.size:
            raise _mismatch("mult_st", t, out)
        st = self._scalar(MULT_ST, s, t.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def mult_tt(self, a, b, out):
        if a.size != out.size or b.size != out.size:
            raise _mismatch("mult_tt", a, b, out)
        st = self._binary(MUL, a.ptr, b.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def sign_t(self, a, out):
        if a.size != out.size:
            raise _mismatch("sign_t", a, out)
        st = self._unary(SIGN, a.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def sqrt_t(self, a, out):
        if a.size != out.size:
            raise _mismatch("sqrt_t", a, out)
        st = self._unary(SQRT, a.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    def subtract_tt(self, a, b, out):
        assert a.shape == b.shape == out.shape     # numpy 265
        if a.size != out.size or b.size != out.size:     # also when assertions are switched off
            raise _mismatch("subtract_tt", a, b, out)
        st = self._binary(SUB, a.ptr, b.ptr, out.ptr, out.size)
        if st:
            self._call(st)

    # -------------------------------------------------- broadcast operations
    def _mv(self, op, m, v, out, accumulate):
        """out (+)= m (op) v with v a row vector (1,N)/(N,) or a column vector (M,1)."""
        if out.size != m.size:
            raise _mismatch("matrix-vector operation", m, v, out)
        if v.shape == m.shape:
            if accumulate:
                assert op == MUL
                return self._call(self._mult_add(m.ptr, v.ptr, out.ptr, out.size))
            return self._call(self._binary(op, m.ptr, v.ptr, out.ptr, out.size))
        n_cols = m.shape[-1] if m.shape else 1
        n_rows = m.size // n_cols if n_cols else 0
        vs = v.shape
        if v.size == n_cols and (len(vs) == 1 or vs[0] == 1 or n_rows == 1):
            is_col = 0
        elif v.size == n_rows and vs[-1] == 1:
            is_col = 1
        else:
            raise ValueError("cannot broadcast vector of shape %r against matrix of shape %r"
                             % (vs, m.shape))
        st = self._mv_call(op, m.ptr, v.ptr, out.ptr, n_rows, n_cols, is_col, accumulate)
        if st:
            self._call(st)

    def add_mv(self, m, v, out):
        self._mv(ADD, m, v, out, 0)

    def subtract_mv(self, m, v, out):
        self._mv(SUB, m, v, out, 0)

    def mult_mv(self, m, v, out):
        self._mv(MUL, m, v, out, 0)

    def divide_mv(self, m, v, out):
        self._mv(DIV, m, v, out, 0)

    def mult_add_mv(self, m, v, out):
        # numpy 239-240; not declared by the abstract class but called by the LSTM layers
        self._mv(MUL, m, v, out, 1)

    def broadcast_t(self, a, axis, out):
        # numpy 103-105
        assert (out.shape[:axis] + (1,) + out.shape[axis + 1:]) == a.shape
        if a.size * out.shape[axis] != out.size:
            raise _mismatch("broadcast_t", a, out)
        outer = _prod(out.shape[:axis])
        inner = _prod(out.shape[axis + 1:])
        self._call(self._lib.bship_broadcast_f32(a.ptr, out.ptr, outer, out.shape[axis], inner))

    def merge_tt(self, a, b, out):
        # numpy 221-225
        na, nb = a.shape[-1], b.shape[-1]
        assert na + nb == out.shape[-1]
        rows = out.size // out.shape[-1] if out.shape[-1] else 0
        if na + nb != out.shape[-1] or a.size != rows * na or b.size != rows * nb:
            raise _mismatch("merge_tt", a, b, out)
        self._call(self._lib.bship_merge_f32(a.ptr, b.ptr, out.ptr, rows, na, nb))

    def split_add_tt(self, x, out_a, out_b):
        # numpy 251-256
        na, nb = out_a.shape[-1], out_b.shape[-1]
        assert na + nb == x.shape[-1]
        rows = x.size // x.shape[-1] if x.shape[-1] else 0
        if na + nb != x.shape[-1] or out_a.size != rows * na or out_b.size != rows * nb:
            raise _mismatch("split_add_tt", x, out_a, out_b)
        self._call(self._lib.bship_split_add_f32(x.ptr, out_a.ptr, out_b.ptr, rows, na, nb))

    # ------------------------------------------------------------ reductions
    def sum_t(self, a, axis, out):
        # numpy 268-273; the shape of `out` decides keepdims, which does not change the layout
        if axis is None or a.ndim <= 1:
            if out.size != 1:
                raise _mismatch("sum_t", a, out)
            st = self._sum_call(a.ptr, out.ptr, 1, a.size, -1)
            if st:
                self._call(st)
            return
        if not isinstance(axis, (int, np.integer)):
            raise NotImplementedError("sum_t over axes %r" % (axis,))
        axis = int(axis) + (a.ndim if axis < 0 else 0)
        if not 0 <= axis < a.ndim:
            raise ValueError("sum_t: axis %d out of range for a %d-d array" % (axis, a.ndim))
        # any array is (outer, length of the axis, inner)
        outer, length, inner = _prod(a.shape[:axis]), a.shape[axis], _prod(a.shape[axis + 1:])
        lib = self._lib
        if out.size != outer * inner:
            raise _mismatch("sum_t over axis %d" % axis, a, out)
        if outer * inner == 0:
            return
        if inner == 1:
            self._call(self._sum_call(a.ptr, out.ptr, outer, length, 1))
        elif outer == 1:
            self._call(self._sum_call(a.ptr, out.ptr, length, inner, 0))
        elif outer <= length:
            # a column sum per outer index: slab o is a contiguous (length, inner) matrix
            for o in range(outer):
                self._call(lib.bship_sum_f32(a.ptr + o * length * inner * 4, out.ptr + o * inner * 4, length, inner, 0))
        else:
            # entry k of the axis is an (outer, inner) matrix with row pitch length * inner: add them up in order
            pitch = length * inner
            self._call(lib.bship_copy2d_f32(out.ptr, inner, a.ptr, pitch, outer, inner))
            for k in range(1, length):
                self._call(lib.bship_elementwise_pitched_f32(PITCHED_BINARY, ADD, 0.0, 0.0, out.ptr, inner, 1,
                                                             a.ptr + k * inner * 4, pitch, 1, out.ptr, inner, outer, inner))

    def softmax_m(self, m, out):
        if out.size != m.size or (out.shape and out.shape[-1] != m.shape[-1]):
            raise _mismatch("softmax_m", m, out)
        n_cols = m.shape[-1]
        self._call(self._lib.bship_softmax_rows_f32(m.ptr, out.ptr, m.size // n_cols if n_cols else 0,
                                                    n_cols))

    # -------------------------------------------------------------- indexing
    def binarize_v(self, v, out):
        if out.ndim != 2 or v.size != out.shape[0]:
            raise _mismatch("binarize_v", v, out)
        self._call(self._lib.bship_binarize_f32(v.ptr, out.ptr, out.shape[0], out.shape[1]))

    def index_m_by_v(self, m, v, out):
        if m.ndim != 2 or v.size != m.shape[0] or out.size != m.shape[0]:
            raise _mismatch("index_m_by_v", m, v, out)
        self._call(self._lib.bship_index_m_by_v_f32(m.ptr, v.ptr, out.ptr, m.shape[0], m.shape[1]))

    # ------------------------------------------------------------------- RNG
    def fill_gaussian(self, mean, std, out):
        self._call(self._lib.bship_fill_gaussian_on_f32(self.rnd._id, out.ptr, out.size, mean, std))

    def generate_probability_mask(self, mask, probability):
        if self.fast_masks:
            self._call(self._lib.bship_prob_mask_fast_on_f32(self.rnd._id, mask.ptr, mask.size, probability))
        else:
            self._call(self._lib.bship_prob_mask_on_f32(self.rnd._id, mask.ptr, mask.size, probability))

    def fast_mask_state(self):
        """(seed, next block) of the fast mask generator (fast_masks=True)."""
        seed, block = ctypes.c_ulonglong(), ctypes.c_ulonglong()
        self._call(self._lib.bship_fast_rng_get_state_on(self.rnd._id, ctypes.byref(seed), ctypes.byref(block)))
        return seed.value, block.value

    # ------------------------------------------------------- dense products
    def _gemm(self, a, b, out, transa, transb, beta):
        m, k = (a.shape[1], a.shape[0]) if transa else a.shape
        kb, n = (b.shape[1], b.shape[0]) if transb else b.shape
        if k != kb or out.shape != (m, n):
            raise ValueError("shapes %r%s . %r%s -> %r do not match"
                             % (a.shape, "^T" if transa else "", b.shape, "^T" if transb else "",
                                out.shape))
        # a row-pitched matrix (a feature slice of a hub) goes in as it is: its pitch is the
        # leading dimension of the product
        pa, lda = (a._base, a.pitch) if type(a) is PitchedDeviceArray else (a.ptr, a.shape[1])
        pb, ldb = (b._base, b.pitch) if type(b) is PitchedDeviceArray else (b.ptr, b.shape[1])
        pc, ldc = (out._base, out.pitch) if type(out) is PitchedDeviceArray else (out.ptr, n)
        st = self._gemm_call(1 if transa else 0, 1 if transb else 0, m, n, k, 1.0, pa, lda, pb, ldb, beta, pc, ldc)
        if st:
            self._call(st)

    def dot_mm(self, a, b, out, transa=False, transb=False):
        self._gemm(a, b, out, transa, transb, 0.0)

    def dot_add_mm(self, a, b, out, transa=False, transb=False):
        self._gemm(a, b, out, transa, transb, 1.0)

    def transpose(self, a, out):
        """out[:a.shape[1], :a.shape[0]] = a.T for 2-D dense arrays; out may have more columns than a
        has rows (they are left alone): the layout dot_small_tn wants is out of shape (k, 128)."""
        rows, cols = a.shape
        if len(out.shape) != 2 or out.shape[0] < cols or out.shape[1] < rows:
            raise ValueError("transpose: %r does not hold the transpose of %r" % (out.shape, a.shape))
        self._call(self._lib.bship_transpose_f32(a.ptr, rows, cols, cols, out.ptr, out.shape[1]))

    def dot_small_tn(self, a_t, rows, b, out, splits=1):
        """out = A . b for a thin A (rows <= 128) given transposed: a_t is (k, 128) with A[i][kk] at
        [kk, i] and zero columns from `rows` on. splits > 1: out is (splits, rows, n) and receives the
        partial products of `splits` ranges of k, to be added by the consumer in a fixed order."""
        k, n = b.shape
        if a_t.shape != (k, 128) or rows > 128:
            raise ValueError("dot_small_tn: the transposed operand must be (%d, 128), rows <= 128" % k)
        want = (rows, n) if splits == 1 else (splits, rows, n)
        if out.shape != want:
            raise ValueError("dot_small_tn: out must be %r, got %r" % (want, out.shape))
        self._call(self._lib.bship_dot_small_tn_f32(a_t.ptr, b.ptr, out.ptr, rows, n, k, n, n, splits, rows * n))

    def conv2d_forward_batch(self, inputs, weights, bias, outputs, padding, stride):
        self._conv_forward(inputs, weights, bias, outputs, padding, stride)

    def _conv_forward(self, inputs, weights, bias, outputs, padding, stride):
        # numpy 149-171, with the per-image loop folded into one im2col and one product:
        # col (N*oh*ow, kh*kw*C) . W(F, kh*kw*C)^T -> outputs (N*oh*ow, F), then + bias.
        # inputs may be image-pitched (images a hub's full feature count apart); outputs is dense.
        n, h, w, c = inputs.shape
        f, kh, kw = weights.shape[0], weights.shape[1], weights.shape[2]
        oh, ow = self._window_geometry("conv2d_forward_batch", inputs, (kh, kw), outputs, padding, stride, f)
        if weights.size != f * kh * kw * c or bias.size != f:
            raise _mismatch("conv2d_forward_batch", inputs, weights, bias)
        kc = kh * kw * c
        rows = n * oh * ow
        p_in, ld_in = self._images(inputs)
        if self.thin_convolutions and kc <= 128 and f % 16 == 0 and f <= 64 and tuple(stride) == (1, 1) and rows:
            # thin filters (an image network's first layer): the matrix cores read the windows out of a copy
            # of the image rows in LDS, no col matrix
            status = self._lib.bship_conv2d_fwd_thin_f32(p_in, ld_in, weights.ptr, bias.ptr, outputs.ptr, n, h, w, c,
                                                         f, kh, kw, padding, 1, 1)
            if status == 0:
                return
            if status != _lib.ERR_UNSUPPORTED:
                self._call(status)
        col = self._scratch((rows, kc))       # im2col writes every element
        self._call(self._lib.bship_im2col_nhwc_pitched_f32(p_in, ld_in, col.ptr, n, h, w, c, kh, kw,
                                                           padding, stride[0], stride[1]))
        # product and bias in one call (the bias goes into the product's epilogue)
        self._call(self._lib.bship_gemm_bias_f32(0, 1, rows, f, kc, col.ptr, kc, weights.ptr, kc,
                                                 bias.ptr, outputs.ptr, f))

    def conv2d_backward_batch(self, inputs, weights, padding, stride, in_deltas, out_deltas,
                              weight_deltas, bias_deltas):
        self._conv_backward(inputs, weights, padding, stride, in_deltas, out_deltas, weight_deltas, bias_deltas)

    def _conv_backward(self, inputs, weights, padding, stride, in_deltas, out_deltas, weight_deltas, bias_deltas):
        # numpy 110-147: weight_deltas and bias_deltas are overwritten, in_deltas accumulated.
        # inputs and in_deltas may be image-pitched; everything else is dense.
        n, h, w, c = inputs.shape
        f, kh, kw = weights.shape[0], weights.shape[1], weights.shape[2]
        oh, ow = self._window_geometry("conv2d_backward_batch", inputs, (kh, kw), out_deltas, padding, stride, f)
        if (weights.size != f * kh * kw * c or weight_deltas.size != weights.size or bias_deltas.size != f
                or in_deltas.size != inputs.size):
            raise _mismatch("conv2d_backward_batch", inputs, weights, in_deltas, weight_deltas, bias_deltas)
        kc = kh * kw * c
        rows = n * oh * ow
        p_in, ld_in = self._images(inputs)
        p_din, ld_din = self._images(in_deltas)
        if self.thin_convolutions and kc <= 127 and f % 16 == 0 and f <= 64 and tuple(stride) == (1, 1) and rows:
            status = self._lib.bship_conv2d_bwd_thin_f32(p_in, ld_in, weights.ptr, out_deltas.ptr, p_din, ld_din,
                                                         weight_deltas.ptr, bias_deltas.ptr, n, h, w, c, f, kh, kw,
                                                         padding, 1, 1)
            if status == 0:
                return
            if status != _lib.ERR_UNSUPPORTED:
                self._call(status)
        col = self._scratch((rows, kc))       # im2col writes every element
        self._call(self._lib.bship_im2col_nhwc_pitched_f32(p_in, ld_in, col.ptr, n, h, w, c, kh, kw,
                                                           padding, stride[0], stride[1]))
        dy = out_deltas.reshape((rows, f))
        self._gemm(dy, col, weight_deltas.reshape((f, kc)), True, False, 0.0)
        self._call(self._lib.bship_sum_f32(dy.ptr, bias_deltas.ptr, rows, f, 0))
        self._gemm(dy, weights.reshape((f, kc)), col, False, False, 0.0)
        self._call(self._lib.bship_col2im_nhwc_pitched_f32(col.ptr, p_din, ld_din, n, h, w, c, kh, kw,
                                                           padding, stride[0], stride[1]))

    @staticmethod
    def _window_geometry(op, inputs, window, outputs, padding, stride, channels_out):
        """(out_h, out_w) that a window over `inputs` gives, checked against `outputs`: the kernels size
        their loops from the inputs' geometry, the caller sized `outputs`."""
        if len(inputs.shape) != 4 or len(outputs.shape) != 4:
            raise _mismatch(op, inputs, outputs)
        n, h, w, _ = inputs.shape
        oh = (h + 2 * padding - window[0]) // stride[0] + 1
        ow = (w + 2 * padding - window[1]) // stride[1] + 1
        if tuple(outputs.shape) != (n, oh, ow, channels_out):
            raise ValueError("%s: inputs %r under a %r window (padding %r, stride %r) give outputs (%d, %d, %d, %d), "
                             "not %r" % (op, tuple(inputs.shape), tuple(window), padding, tuple(stride), n, oh, ow,
                                         channels_out, tuple(outputs.shape)))
        return oh, ow

    # --------------------------------------------------------------- pooling
    def maxpool2d_forward_batch(self, inputs, window, outputs, padding, stride, argmax):
        n, h, w, c = inputs.shape
        self._window_geometry("maxpool2d_forward_batch", inputs, window, outputs, padding, stride, c)
        if argmax.size != outputs.size:
            raise _mismatch("maxpool2d_forward_batch", outputs, argmax)
        self._call(self._lib.bship_maxpool_fwd_nhwc_f32(
            inputs.ptr, outputs.ptr, argmax.ptr, n, h, w, c, outputs.shape[1], outputs.shape[2],
            window[0], window[1], padding, stride[0], stride[1]))

    def maxpool2d_backward_batch(self, inputs, window, outputs, padding, stride, argmax,
                                 in_deltas, out_deltas):
        n, h, w, c = inputs.shape
        self._window_geometry("maxpool2d_backward_batch", inputs, window, outputs, padding, stride, c)
        if argmax.size != outputs.size or out_deltas.size != outputs.size or in_deltas.size != inputs.size:
            raise _mismatch("maxpool2d_backward_batch", inputs, outputs, argmax, in_deltas, out_deltas)
        self._call(self._lib.bship_maxpool_bwd_nhwc_f32(
            argmax.ptr, out_deltas.ptr, in_deltas.ptr, n, h, w, c, outputs.shape[1],
            outputs.shape[2], window[0], window[1], padding, stride[0], stride[1]))

    def avgpool2d_forward_batch(self, inputs, window, outputs, padding, stride):
        n, h, w, c = inputs.shape
        self._window_geometry("avgpool2d_forward_batch", inputs, window, outputs, padding, stride, c)
        self._call(self._lib.bship_avgpool_fwd_nhwc_f32(
            inputs.ptr, outputs.ptr, n, h, w, c, outputs.shape[1], outputs.shape[2],
            window[0], window[1], padding, stride[0], stride[1]))

    def avgpool2d_backward_batch(self, inputs, window, outputs, padding, stride, in_deltas,
                                 out_deltas):
        n, h, w, c = inputs.shape
        self._window_geometry("avgpool2d_backward_batch", inputs, window, outputs, padding, stride, c)
        if out_deltas.size != outputs.size or in_deltas.size != inputs.size:
            raise _mismatch("avgpool2d_backward_batch", inputs, outputs, in_deltas, out_deltas)
        self._call(self._lib.bship_avgpool_bwd_nhwc_f32(
            out_deltas.ptr, in_deltas.ptr, n, h, w, c, outputs.shape[1], outputs.shape[2],
            window[0], window[1], padding, stride[0], stride[1]))

    # -------------------------------------------------- activation functions
    def rel(self, x, y):
        if x.size != y.size:
            raise _mismatch("rel", x, y)
        st = self._unary(REL, x.ptr, y.ptr, y.size)
        if st:
            self._call(st)

    def rel_deriv(self, x, y, dy, dx):
        if y.size != dx.size or dy.size != dx.size:
            raise _mismatch("rel_deriv", y, dy, dx)
        st = self._deriv(REL_DERIV, y.ptr, dy.ptr, dx.ptr, dx.size)
        if st:
            self._call(st)

    def sigmoid(self, x, y):
        if x.size != y.size:
            raise _mismatch("sigmoid", x, y)
        st = self._unary(SIGMOID, x.ptr, y.ptr, y.size)
        if st:
            self._call(st)

    def sigmoid_deriv(self, x, y, dy, dx):
        if y.size != dx.size or dy.size != dx.size:
            raise _mismatch("sigmoid_deriv", y, dy, dx)
        st = self._deriv(SIGMOID_DERIV, y.ptr, dy.ptr, dx.ptr, dx.size)
        if st:
            self._call(st)

    def tanh(self, x, y):
        if x.size != y.size:
            raise _mismatch("tanh", x, y)
        st = self._unary(TANH, x.ptr, y.ptr, y.size)
        if st:
            self._call(st)

    def tanh_deriv(self, x, y, dy, dx):
        if y.size != dx.size or dy.size != dx.size:
            raise _mismatch("tanh_deriv", y, dy, dx)
        st = self._deriv(TANH_DERIV, y.ptr, dy.ptr, dx.ptr, dx.size)
        if st:
            self._call(st)

    def el(self, x, y):
        if x.size != y.size:
            raise _mismatch("el", x, y)
        st = self._unary(EL, x.ptr, y.ptr, y.size)
        if st:
            self._call(st)

    def el_deriv(self, x, y, dy, dx):
        if y.size != dx.size or dy.size != dx.size:
            raise _mismatch("el_deriv", y, dy, dx)
        st = self._deriv(EL_DERIV, y.ptr, dy.ptr, dx.ptr, dx.size)
        if st:
            self._call(st)

    # ------------------------------------------------ fused layer-level steps
    # Extensions beyond the Handler interface. A layer may test for them with
    # hasattr() and fall back on the single operations, which give the same bits.
    _ACT_CODES = {"sigmoid": 0, "tanh": 1, "rel": 2, "linear": 3, "el": 4}

    def lstm_forward_step(self, activation, Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, Ca_prev, y,
                          pi, pf, po, bz, bi, bf, bo):
        """Everything lstm_layer.py:121-145 does at one time step after its four
        dot_add_mm calls; the arrays are the [t] (and Ca[t-1]) slices."""
        batch, n = Za.shape
        mats = (Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, Ca_prev, y)
        vecs = (pi, pf, po, bz, bi, bf, bo)
        if any(m.shape != (batch, n) for m in mats) or any(v.size != n for v in vecs):
            raise ValueError("lstm_forward_step: inconsistent shapes")
        self._call(self._lib.bship_lstm_fwd_step_f32(
            self._ACT_CODES[activation], batch, n, *[a.ptr for a in mats + vecs]))

    def lstm_backward_step(self, activation, dy, Zb, Ib, Fb, Ob, Cb, Ca_prev, Fb_next, dIa_next,
                           dFa_next, dCa_next, dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb,
                           pi, pf, po):
        """Everything lstm_layer.py:186-214 does at one time step between the
        dot_add_mm calls into dy[t] and the end of the loop body."""
        batch, n = dy.shape
        mats = (dy, Zb, Ib, Fb, Ob, Cb, Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next,
                dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb)
        vecs = (pi, pf, po)
        if any(m.shape != (batch, n) for m in mats) or any(v.size != n for v in vecs):
            raise ValueError("lstm_backward_step: inconsistent shapes")
        self._call(self._lib.bship_lstm_bwd_step_f32(
            self._ACT_CODES[activation], batch, n, *[a.ptr for a in mats + vecs]))

    def stack_adjacent(self, arrays):
        """One (k*rows, ...) array over k equally shaped arrays that lie back to back in
        device memory (as the four recurrent matrices of an LSTM do in brainstorm's
        parameter vector), or None if they do not."""
        first = arrays[0]
        for k, a in enumerate(arrays):
            if a.shape != first.shape or a.ptr != first.ptr + k * first.nbytes or not a.ptr:
                return None
        shape = (len(arrays) * first.shape[0],) + tuple(first.shape[1:])
        return DeviceArray(first.ptr, shape, [a._owner for a in arrays], self)

    def lstm_forward_step_packed(self, activation, rec, Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb,
                                 Ca_prev, y, pi, pf, po, bz, bi, bf, bo):
        """lstm_forward_step with the four recurrent products given as one matrix
        rec (batch, 4n) = y[t-1] . [Rz;Ri;Rf;Ro]^T instead of accumulated into Za..Oa."""
        batch, n = Za.shape
        mats = (Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, Ca_prev, y)
        vecs = (pi, pf, po, bz, bi, bf, bo)
        if (rec.shape != (batch, 4 * n) or any(m.shape != (batch, n) for m in mats)
                or any(v.size != n for v in vecs)):
            raise ValueError("lstm_forward_step_packed: inconsistent shapes")
        self._call(self._lib.bship_lstm_fwd_step_packed_f32(
            self._ACT_CODES[activation], batch, n, rec.ptr, *[a.ptr for a in mats + vecs]))

    def lstm_forward_sequence(self, activation, R_all, Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, y,
                              pi, pf, po, bz, bi, bf, bo):
        """The whole forward recurrence of lstm_layer.py:115-145 in one launch: Za, Ia, Fa, Oa hold the
        input products on entry; every array is (time + 1, batch, n) with its context slot last; R_all is
        the stacked (4n, n) recurrent matrix (stack_adjacent). Returns False, with nothing done, when the
        shape does not fit the kernel (n % 4, batch > 128, n > 1024, or fewer compute units than
        n / 4): the caller then takes the step-by-step path. Raises BshipError (status
        BSHIP_ERR_TIMEOUT) if the workgroups did not meet at a time step's barrier. Waits for the
        device."""
        steps = Za.shape[0] - 1
        batch, n = Za.shape[1], Za.shape[2]
        mats = (Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, y)
        vecs = (pi, pf, po, bz, bi, bf, bo)
        if (R_all.shape != (4 * n, n) or any(m.shape != (steps + 1, batch, n) for m in mats)
                or any(v.size != n for v in vecs)):
            raise ValueError("lstm_forward_sequence: inconsistent shapes")
        if n % 4 or batch > 128 or n > 1024:
            return False
        status = self._lib.bship_lstm_fwd_sequence_f32(
            self._ACT_CODES[activation], steps, batch, n, R_all.ptr, *[a.ptr for a in mats + vecs])
        if status in (_lib.ERR_UNSUPPORTED, _lib.ERR_OUT_OF_MEMORY):
            return False            # nothing was launched (the scratch for the operand buffers did not fit the pool)
        self._call(status)
        return True

    def lstm_backward_step_packed(self, activation, deltas, dy, packed_out, Zb, Ib, Fb, Ob, Cb,
                                  Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next, dZa, dZb, dIa,
                                  dIb, dFa, dFb, dOa, dOb, dCa, dCb, pi, pf, po):
        """lstm_backward_step for one stacked recurrent product: dy holds
        packed[t+1] . [Rz;Ri;Rf;Ro] on entry and deltas + that afterwards;
        packed_out (batch, 4n) receives [dZa|dIa|dFa|dOa] of this step."""
        batch, n = dy.shape
        mats = (deltas, dy, Zb, Ib, Fb, Ob, Cb, Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next,
                dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb)
        vecs = (pi, pf, po)
        if (packed_out.shape != (batch, 4 * n) or any(m.shape != (batch, n) for m in mats)
                or any(v.size != n for v in vecs)):
            raise ValueError("lstm_backward_step_packed: inconsistent shapes")
        self._call(self._lib.bship_lstm_bwd_step_packed_f32(
            self._ACT_CODES[activation], batch, n, deltas.ptr, dy.ptr, packed_out.ptr,
            *[a.ptr for a in mats[2:] + vecs]))

    def lstm_backward_step_thin(self, activation, deltas, dy_parts, dy, packed_t_out, Zb, Ib, Fb, Ob, Cb,
                                Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next, dZa, dZb, dIa,
                                dIb, dFa, dFb, dOa, dOb, dCa, dCb, pi, pf, po):
        """lstm_backward_step_packed behind dot_small_tn: dy_parts holds the partial products of
        packed[t+1] . [Rz;Ri;Rf;Ro], shape (batch, n) or (parts, batch, n); dy receives deltas + their
        sum; packed_t_out (4n, 128) receives [dZa|dIa|dFa|dOa] of this step transposed (the left
        operand of the next product)."""
        batch, n = dy.shape
        mats = (Zb, Ib, Fb, Ob, Cb, Ca_prev, Fb_next, dIa_next, dFa_next, dCa_next,
                dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb)
        vecs = (pi, pf, po)
        parts = 1 if len(dy_parts.shape) == 2 else dy_parts.shape[0]
        if (packed_t_out.shape != (4 * n, 128) or tuple(dy_parts.shape[-2:]) != (batch, n) or batch > 128
                or deltas.shape != (batch, n) or any(m.shape != (batch, n) for m in mats)
                or any(v.size != n for v in vecs)):
            raise ValueError("lstm_backward_step_thin: inconsistent shapes")
        self._call(self._lib.bship_lstm_bwd_step_thin_f32(
            self._ACT_CODES[activation], batch, n, deltas.ptr, dy_parts.ptr, parts, batch * n, dy.ptr,
            packed_t_out.ptr, *[a.ptr for a in mats + vecs]))

    def softmax_ce_forward(self, inputs, targets, probs, loss):
        """softmax_m(inputs, probs) and loss = -log(clip(probs[i, targets[i]], 1e-6, 1)) with the roundings of
        softmax_ce_layer.py:79-89 (index_m_by_v, clip_t, log_t, mult_st) in two launches instead of six."""
        rows, k = inputs.shape
        if probs.shape != (rows, k) or targets.size != rows or loss.size != rows:
            raise ValueError("softmax_ce_forward: inconsistent shapes")
        self._call(self._lib.bship_softmax_ce_fwd_f32(inputs.ptr, targets.ptr, probs.ptr, loss.ptr, rows, k))

    def softmax_ce_backward(self, probs, targets, dloss, t_bin, dinputs):
        """softmax_ce_layer.py:108-112 (binarize_v, mult_st, add_tt, mult_mv, add_tt) in one pass."""
        rows, k = probs.shape
        if (t_bin.shape != (rows, k) or dinputs.shape != (rows, k) or targets.size != rows
                or dloss.size != rows):
            raise ValueError("softmax_ce_backward: inconsistent shapes")
        self._call(self._lib.bship_softmax_ce_bwd_f32(probs.ptr, targets.ptr, dloss.ptr, t_bin.ptr,
                                                      dinputs.ptr, rows, k))

    def momentum_update(self, momentum, neg_learning_rate, gradients, velocity, parameters):
        """mult_st(momentum, velocity, velocity); mult_add_st(neg_learning_rate, gradients, velocity);
        add_tt(velocity, parameters, parameters) (steppers.py:104-112) in one pass."""
        if not (gradients.size == velocity.size == parameters.size):
            raise ValueError("momentum_update: inconsistent sizes")
        self._call(self._lib.bship_momentum_update_f32(momentum, neg_learning_rate, gradients.ptr, velocity.ptr,
                                                       parameters.ptr, parameters.size))

    def highway_forward(self, H, T, x, y):
        """y = T * (H - x) + x with the roundings of highway_layer.py:48-51, one pass."""
        if not (H.shape == T.shape == x.shape == y.shape):
            raise ValueError("highway_forward: inconsistent shapes")
        self._call(self._lib.bship_highway_fwd_f32(H.ptr, T.ptr, x.ptr, y.ptr, y.size))

    def highway_backward(self, H, T, x, dy, dx, dH, dT):
        """dx += (1-T)*dy; dH += T*dy; dT += (H-x)*dy (highway_layer.py:64-71), one pass."""
        if any(a.shape != x.shape for a in (H, T, dy, dx, dH, dT)):
            raise ValueError("highway_backward: inconsistent shapes")
        self._call(self._lib.bship_highway_bwd_f32(H.ptr, T.ptr, x.ptr, dy.ptr, dx.ptr, dH.ptr,
                                                   dT.ptr, x.size))

    def bias_act(self, activation, m, bias, out):
        """out = act(m + bias): add_mv followed by act_func[activation] in one pass
        (fully_connected_layer.py:61-62). m and out are (M, N), bias has N elements."""
        n_cols = m.shape[-1]
        if out.shape != m.shape or bias.size != n_cols:
            raise ValueError("bias_act: inconsistent shapes")
        self._call(self._lib.bship_bias_act_f32(self._ACT_CODES[activation], m.ptr, bias.ptr, out.ptr,
                                                m.size // n_cols if n_cols else 0, n_cols))

    def batchnorm_forward(self, training_pass, inputs, gamma, beta, mu, sigma, decay, epsilon,
                          sigma_b, centered, x_hat, out):
        """batch_normalization_layer.py:54-105 on flattened (M, N) buffers."""
        rows, n = inputs.shape
        if (any(a.shape != (rows, n) for a in (centered, x_hat, out))
                or any(v.size != n for v in (gamma, beta, mu, sigma, sigma_b))):
            raise ValueError("batchnorm_forward: inconsistent shapes")
        self._call(self._lib.bship_batchnorm_fwd_f32(
            int(bool(training_pass)), inputs.ptr, gamma.ptr, beta.ptr, mu.ptr, sigma.ptr,
            float(decay), float(epsilon), sigma_b.ptr, centered.ptr, x_hat.ptr, out.ptr, rows, n))

    def batchnorm_backward(self, out_deltas, x_hat, gamma, sigma_b, dgamma, dbeta, in_deltas):
        """batch_normalization_layer.py:107-152 on flattened (M, N) buffers."""
        rows, n = out_deltas.shape
        if (x_hat.shape != (rows, n) or in_deltas.shape != (rows, n)
                or any(v.size != n for v in (gamma, sigma_b, dgamma, dbeta))):
            raise ValueError("batchnorm_backward: inconsistent shapes")
        self._call(self._lib.bship_batchnorm_bwd_f32(out_deltas.ptr, x_hat.ptr, gamma.ptr, sigma_b.ptr,
                                                     dgamma.ptr, dbeta.ptr, in_deltas.ptr, rows, n))

    def dropout_forward(self, inputs, keep_probability, scale, mask, out):
        """generate_probability_mask(mask, keep_probability); out = inputs * mask;
        out = scale * out (dropout_layer.py:41-45) with one pass behind the mask."""
        if not (inputs.shape == mask.shape == out.shape):
            raise ValueError("dropout_forward: inconsistent shapes")
        fn = self._lib.bship_dropout_fwd_fast_on_f32 if self.fast_masks else self._lib.bship_dropout_fwd_on_f32
        self._call(fn(self.rnd._id, inputs.ptr, mask.ptr, out.ptr, out.size, float(keep_probability), float(scale)))
