"""TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.

CPU oracle for HipHandler: a restatement of brainstorm's NumpyHandler
(brainstorm/handlers/numpy_handler.py) driven by NumPy as a library, plus
``cpuop.c`` (a C restatement of brainstorm/handlers/_cpuop.pyx) for pooling,
im2col and col2im. Only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline may import this module; the product never does.

Every method cites the numpy_handler.py lines it follows. The arithmetic of
almost every operation IS a NumPy routine (np.add, np.fmod, np.tanh, np.sum,
np.dot ...), so driving NumPy with the same expression reproduces the
reference's results exactly, including dtype promotion and rounding order.

How the oracle itself is pinned (tests/test_oracle_*.py): closed forms and
invariants (softmax rows sum to 1 and are shift invariant, sigmoid symmetry,
one-hot structure, merge/split round trip), brute-force Python loops on tiny
inputs for pooling / im2col / col2im / convolution, adjointness of im2col and
col2im, the MT19937 known-answer vectors for the mask stream. The reference
ships no golden vectors for any handler operation.

Parity unpinned by the reference's own tests (no test there covers them):
generate_probability_mask, fill_gaussian, modulo_tt, copy_to_if, fill_if,
add_into_if, mult_add_mv, is_fully_finite, fill, copy_to. They are pinned here
by the library routine they reduce to or by the known-answer tests above.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

from brainstorm_amd.handler_api import Handler

_HERE = os.path.dirname(os.path.abspath(__file__))
_CPUOP_PATH = os.path.join(_HERE, "libcpuop_oracle.so")
_cpuop = None


def load_cpuop():
    """Loads oracle/libcpuop_oracle.so (built by `make -C oracle`)."""
    global _cpuop
    if _cpuop is None:
        if not os.path.exists(_CPUOP_PATH):
            raise ImportError("%s missing: run `make -C oracle`" % _CPUOP_PATH)
        _cpuop = ctypes.CDLL(_CPUOP_PATH)
    return _cpuop


def _ptr(a):
    assert a.flags['C_CONTIGUOUS'], "oracle C routines need C-contiguous arrays"
    return ctypes.c_void_p(a.ctypes.data)


class NumpyRefHandler(Handler):
    """NumpyHandler semantics (numpy_handler.py:13-309)."""

    array_type = np.ndarray

    def __init__(self, dtype=np.float32, seed=None):
        super(NumpyRefHandler, self).__init__()
        self.dtype = np.dtype(dtype).type
        self.context = 'numpy'
        self.EMPTY = np.zeros(0)
        if seed is None:
            seed = np.random.randint(0, 1000000000)
        # brainstorm.randomness.RandomState is numpy's RandomState plus a remembered seed
        # (randomness.py:10-22)
        self.rnd = np.random.RandomState(seed)

    def _suffix(self):
        return {np.float32: "f32", np.float64: "f64"}[self.dtype]

    # ---- allocation: numpy_handler.py 36-43 ----
    def allocate(self, size):
        return np.zeros(size, dtype=self.dtype)

    def ones(self, shape):
        return np.ones(shape=shape, dtype=self.dtype)

    def zeros(self, shape):
        return np.zeros(shape=shape, dtype=self.dtype)

    # ---- copy and fill: 47-65 ----
    def copy_to(self, src, dest):
        np.copyto(dest, src, casting='same_kind')          # 52

    def create_from_numpy(self, arr):
        return arr.copy()                                    # 55

    def fill(self, mem, val):
        mem.fill(val)                                        # 58

    def get_numpy_copy(self, arr):
        assert type(arr) == self.array_type                  # 61
        return arr.copy()

    def set_from_numpy(self, mem, arr):
        mem[:] = arr.astype(self.dtype)                      # 65

    def copy_to_if(self, src, dest, cond):
        dest[cond != 0] = src[cond != 0]                     # 174

    def fill_if(self, mem, val, cond):
        mem[cond != 0] = val                                 # 197

    def add_into_if(self, a, out, cond):
        out[cond != 0] += a[cond != 0]                       # 78

    def is_fully_finite(self, a):
        return np.all(np.isfinite(a))                        # 70

    # ---- tensor (op) tensor ----
    def add_tt(self, a, b, out):
        out[:] = a + b                                       # 87

    def subtract_tt(self, a, b, out):
        assert a.shape == b.shape == out.shape               # 265
        out[:] = a - b                                       # 266

    def mult_tt(self, a, b, out):
        np.multiply(a, b, out)                               # 246

    def divide_tt(self, a, b, out):
        out[:] = a / b                                       # 191

    def modulo_tt(self, a, b, out):
        np.fmod(a, b, out)                                   # 228

    def mult_add_tt(self, a, b, out):
        out[:] += a * b                                      # 234

    # ---- scalar (op) tensor ----
    def add_st(self, s, t, out):
        out[:] = t + s                                       # 84

    def mult_st(self, s, t, out):
        np.multiply(s, t, out)                               # 243

    def mult_add_st(self, s, t, out):
        out[:] += s * t                                      # 231

    # ---- unary ----
    def abs_t(self, a, out):
        np.abs(a, out=out)                                   # 75

    def sign_t(self, a, out):
        np.sign(a, out=out)                                  # 249

    def sqrt_t(self, a, out):
        np.sqrt(a, out)                                      # 259

    def log_t(self, a, out):
        np.log(a, out)                                       # 208

    def clip_t(self, a, a_min, a_max, out):
        np.clip(a, a_min, a_max, out)                        # 108

    # ---- matrix (op) vector ----
    def add_mv(self, m, v, out):
        out[:] = m + v                                       # 81

    def subtract_mv(self, m, v, out):
        out[:] = m - v                                       # 262

    def mult_mv(self, m, v, out):
        out[:] = m * v                                       # 237

    def divide_mv(self, m, v, out):
        out[:] = m / v                                       # 188

    def mult_add_mv(self, m, v, out):
        out[:] += m * v                                      # 240

    def broadcast_t(self, a, axis, out):
        assert (out.shape[:axis] + (1,) + out.shape[axis + 1:]) == a.shape   # 104
        out[:] = a[:]                                        # 105

    def merge_tt(self, a, b, out):
        # 221-225: out[..., :na] = a, out[..., na:] = b
        flat = out.reshape(-1, out.shape[-1])
        na = a.shape[-1]
        flat[:, :na] = a.reshape(-1, na)
        flat[:, na:] = b.reshape(-1, b.shape[-1])

    def split_add_tt(self, x, out_a, out_b):
        # 251-256
        fa = out_a.reshape(-1, out_a.shape[-1])
        fb = out_b.reshape(-1, out_b.shape[-1])
        fx = x.reshape(-1, x.shape[-1])
        na = fa.shape[-1]
        fa[:] += fx[:, :na]
        fb[:] += fx[:, na:]

    # ---- reductions ----
    def sum_t(self, a, axis, out):
        # 268-273: keepdims iff out has as many axes as a
        keepdims = axis is not None and len(out.shape) == len(a.shape)
        np.sum(a, axis=axis, out=out, keepdims=keepdims)

    def softmax_m(self, m, out):
        # 292-295
        row_max = np.amax(m, axis=1, keepdims=True)
        e = np.exp(m - row_max)
        out[:] = e / np.sum(e, axis=1, keepdims=True)

    # ---- indexing ----
    def binarize_v(self, v, out):
        # 99-101: rows of the identity picked by the labels
        eye = np.eye(out.shape[1], dtype=self.dtype)
        out[:] = eye[v.astype(np.int32)].reshape(out.shape)

    def index_m_by_v(self, m, v, out):
        out[:, 0] = m[np.arange(m.shape[0]), v.squeeze().astype(np.int32)]   # 203

    # ---- RNG ----
    def fill_gaussian(self, mean, std, out):
        out[:] = std * self.rnd.standard_normal(out.shape) + mean            # 194

    def generate_probability_mask(self, mask, probability):
        mask[:] = self.rnd.uniform(size=mask.shape) < probability            # 200

    # ---- dense ----
    def dot_mm(self, a, b, out, transa=False, transb=False):
        # 181-185
        out[:] = np.dot(a.T if transa else a, b.T if transb else b)

    def dot_add_mm(self, a, b, out, transa=False, transb=False):
        # 176-179
        out[:] += np.dot(a.T if transa else a, b.T if transb else b)

    def _im2col(self, image, kh, kw, pad, stride, col):
        fn = getattr(load_cpuop(), "bs_im2col_" + self._suffix())
        h, w, c = image.shape
        fn(_ptr(image), _ptr(col), h, w, c, kh, kw, pad, pad, pad, pad, stride[0], stride[1])

    def _col2im(self, col, kh, kw, pad, stride, image_deltas):
        fn = getattr(load_cpuop(), "bs_col2im_" + self._suffix())
        h, w, c = image_deltas.shape
        fn(_ptr(col), _ptr(image_deltas), h, w, c, kh, kw, pad, pad, pad, pad, stride[0], stride[1])

    def conv2d_forward_batch(self, inputs, weights, bias, outputs, padding, stride):
        # 149-171: per image, col = im2col(image); outputs[i] = col . W^T; then + bias
        n_filters = weights.shape[0]
        kh, kw = weights.shape[1], weights.shape[2]
        n_pix = outputs.shape[1] * outputs.shape[2]
        n_k = int(np.prod(weights.shape[1:]))
        w2d = weights.reshape(n_filters, n_k)
        for i in range(inputs.shape[0]):
            col = np.zeros((n_pix, n_k), dtype=self.dtype)
            self._im2col(inputs[i], kh, kw, padding, stride, col)
            np.dot(col, w2d.T, out=outputs[i].reshape((n_pix, n_filters)))
        outputs += bias.reshape((1, 1, 1, n_filters))

    def conv2d_backward_batch(self, inputs, weights, padding, stride, in_deltas, out_deltas,
                              weight_deltas, bias_deltas):
        # 110-147: weight/bias deltas are zeroed then summed over the images; in_deltas are
        # accumulated through col2im
        n_filters = weights.shape[0]
        kh, kw = weights.shape[1], weights.shape[2]
        n_pix = out_deltas.shape[1] * out_deltas.shape[2]
        n_k = int(np.prod(weights.shape[1:]))
        weight_deltas.fill(0.0)
        bias_deltas.fill(0.0)
        col = np.zeros((n_pix, n_k), dtype=self.dtype)
        dw2d = weight_deltas.reshape(n_filters, n_k)
        w2d = weights.reshape((n_filters, n_k))
        for i in range(inputs.shape[0]):
            self._im2col(inputs[i], kh, kw, padding, stride, col)
            dy = out_deltas[i].reshape((n_pix, n_filters))
            self.dot_add_mm(dy, col, out=dw2d, transa=True)
            bias_deltas += np.sum(dy, axis=0)
            np.dot(dy, w2d, out=col)
            self._col2im(col, kh, kw, padding, stride, in_deltas[i])

    # ---- pooling: 89-97, 210-219 -> cpuop.c ----
    def maxpool2d_forward_batch(self, inputs, window, outputs, padding, stride, argmax):
        fn = getattr(load_cpuop(), "bs_maxpool_fwd_" + self._suffix())
        n, h, w, c = inputs.shape
        fn(_ptr(inputs), _ptr(outputs), _ptr(argmax), ctypes.c_long(n), h, w, c, outputs.shape[1],
           outputs.shape[2], window[0], window[1], padding, stride[0], stride[1])

    def maxpool2d_backward_batch(self, inputs, window, outputs, padding, stride, argmax,
                                 in_deltas, out_deltas):
        fn = getattr(load_cpuop(), "bs_maxpool_bwd_" + self._suffix())
        n, h, w, c = inputs.shape
        fn(_ptr(argmax), _ptr(out_deltas), _ptr(in_deltas), ctypes.c_long(n), h, w, c,
           outputs.shape[1], outputs.shape[2])

    def avgpool2d_forward_batch(self, inputs, window, outputs, padding, stride):
        fn = getattr(load_cpuop(), "bs_avgpool_fwd_" + self._suffix())
        n, h, w, c = inputs.shape
        fn(_ptr(inputs), _ptr(outputs), ctypes.c_long(n), h, w, c, outputs.shape[1],
           outputs.shape[2], window[0], window[1], padding, stride[0], stride[1])

    def avgpool2d_backward_batch(self, inputs, window, outputs, padding, stride, in_deltas,
                                 out_deltas):
        fn = getattr(load_cpuop(), "bs_avgpool_bwd_" + self._suffix())
        n, h, w, c = inputs.shape
        fn(_ptr(out_deltas), _ptr(in_deltas), ctypes.c_long(n), h, w, c, outputs.shape[1],
           outputs.shape[2], window[0], window[1], padding, stride[0], stride[1])

    # ---- activation functions: 277-309 ----
    def rel(self, x, y):
        y[:] = x * (x > 0)                                   # 278

    def rel_deriv(self, x, y, dy, dx):
        dx[:] = dy * (y > 0)                                 # 281

    def sigmoid(self, x, y):
        # 283-287: two branches so that exp never overflows
        pos = x >= 0
        y[pos] = 1. / (1. + np.exp(-x[pos]))
        neg = x < 0
        y[neg] = np.exp(x[neg]) / (1. + np.exp(x[neg]))

    def sigmoid_deriv(self, x, y, dy, dx):
        dx[:] = dy * y * (1. - y)                            # 290

    def tanh(self, x, y):
        np.tanh(x, y)                                        # 298

    def tanh_deriv(self, x, y, dy, dx):
        dx[:] = dy * (1. - y * y)                            # 301

    def el(self, x, y):
        y[:] = x * (x >= 0.) + (np.exp(x) - 1.) * (x < 0.)   # 305

    def el_deriv(self, x, y, dy, dx):
        dx[:] = dy * (y >= 0.) + dy * (y + 1.) * (y < 0.)    # 309
