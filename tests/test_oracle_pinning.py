"""CPU-only: pins the oracle (oracle/numpy_ref_handler.py + oracle/cpuop.c).

The reference ships no golden vectors for handler operations, so every oracle
function is checked against something that does not share its code: a published
known-answer value, a closed form, an invariant of the mathematics, an
independent formulation with NumPy slicing, or a brute-force loop on tiny
inputs -- chosen so that a dropped term, a wrong sign or index, or a transposed
operand fails. Retyping the oracle's own expression would pin nothing and is
avoided.
"""
import itertools
import math

import numpy as np
import pytest

from oracle.numpy_ref_handler import NumpyRefHandler

F32, F64 = np.float32, np.float64


@pytest.fixture(scope="module")
def ref():
    return NumpyRefHandler(F32, seed=7)


@pytest.fixture(scope="module")
def ref64():
    return NumpyRefHandler(F64, seed=7)


# ------------------------------------------------------------- memory operations
def test_allocate_copy_fill_and_transfers(ref):
    # allocate == zeros, of the handler's dtype (numpy_handler.py:36-43)
    for shape in ((3, 4), 7, (2, 0, 5), ()):
        a, z = ref.allocate(shape), ref.zeros(shape)
        assert a.dtype == F32 and z.dtype == F32 and a.shape == z.shape == np.empty(shape).shape
        assert not a.any() and not z.any()
    o = ref.ones((2, 3))
    assert o.dtype == F32 and all(v == 1.0 for v in o.ravel().tolist())
    # copy_to(src, dest): dest receives src, src is untouched; a reshaped view writes through (47-52)
    src = np.arange(12, dtype=F32).reshape(3, 4)
    base = np.full(20, -1.0, F32)
    dest = base[4:16].reshape(3, 4)                       # a view into a larger flat buffer
    ref.copy_to(src, dest)
    assert base.tolist() == [-1.0] * 4 + [float(k) for k in range(12)] + [-1.0] * 4
    assert src.tolist() == [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9, 10, 11]]
    with pytest.raises(TypeError):                        # same_kind casting: float -> int is refused
        ref.copy_to(src, np.zeros((3, 4), np.int32))
    # fill sets every element of a view and nothing else (57-58)
    ref.fill(base[2:5], 2.5)
    assert base[:6].tolist() == [-1.0, -1.0, 2.5, 2.5, 2.5, 1.0]
    # set_from_numpy casts to the handler dtype: float64 values are ROUNDED to float32 (64-65)
    mem = ref.allocate((3,))
    ref.set_from_numpy(mem, np.array([0.1, 16777217.0, -1e-50], dtype=F64))
    assert mem.dtype == F32
    assert mem.view(np.uint32).tolist() == [0x3dcccccd, 0x4b800000, 0x80000000]   # 0.1f, 2^24 (ties to even), -0
    ref.set_from_numpy(mem, np.array([1, -2, 3], dtype=np.int32))
    assert mem.tolist() == [1.0, -2.0, 3.0]
    # create_from_numpy / get_numpy_copy give copies, not views (54-62)
    host = np.array([1.0, 2.0], F32)
    dev = ref.create_from_numpy(host)
    back = ref.get_numpy_copy(dev)
    host[0], dev[1] = 9.0, 8.0
    assert dev.tolist() == [1.0, 8.0] and back.tolist() == [1.0, 2.0]


def test_is_fully_finite(ref):
    a = np.array([[0.0, -0.0, 1e-45], [3.4e38, -3.4e38, 1.0]], F32)     # zeros, a denormal, the largest floats
    assert ref.is_fully_finite(a) is True or ref.is_fully_finite(a) == True  # noqa: E712
    for bad in (np.nan, np.inf, -np.inf):
        for pos in ((0, 0), (1, 2)):
            b = a.copy()
            b[pos] = bad
            assert not ref.is_fully_finite(b), (bad, pos)
    assert ref.is_fully_finite(np.zeros((0, 3), F32))


# ----------------------------------------------------------------------- MT19937
class TextbookMT19937:
    """Matsumoto & Nishimura's mt19937ar.c (init_genrand / genrand_int32 / genrand_res53)."""

    def __init__(self, seed):
        self.mt = [0] * 624
        self.mt[0] = seed & 0xffffffff
        for i in range(1, 624):
            self.mt[i] = (1812433253 * (self.mt[i - 1] ^ (self.mt[i - 1] >> 30)) + i) & 0xffffffff
        self.idx = 624

    def int32(self):
        if self.idx >= 624:
            mt = self.mt
            for k in range(624):
                y = (mt[k] & 0x80000000) | (mt[(k + 1) % 624] & 0x7fffffff)
                mt[k] = mt[(k + 397) % 624] ^ (y >> 1) ^ (0x9908b0df if y & 1 else 0)
            self.idx = 0
        y = self.mt[self.idx]
        self.idx += 1
        y ^= y >> 11
        y ^= (y << 7) & 0x9d2c5680
        y ^= (y << 15) & 0xefc60000
        y ^= y >> 18
        return y & 0xffffffff

    def double(self):
        a, b = self.int32() >> 5, self.int32() >> 6
        return (a * 67108864.0 + b) / 9007199254740992.0


def test_textbook_mt19937_known_answers():
    # First output of the default seed 5489, and the 10000th output that the C++ standard
    # requires of std::mt19937 (same algorithm, same seeding).
    g = TextbookMT19937(5489)
    outs = [g.int32() for _ in range(10000)]
    assert outs[0] == 3499211612
    assert outs[9999] == 4123659995


def test_mask_stream_is_the_textbook_stream(ref):
    for seed in (0, 1, 12345, 4294967295):
        g = TextbookMT19937(seed)
        want = np.array([g.double() for _ in range(1500)])
        got = np.random.RandomState(seed).uniform(size=1500)
        assert np.array_equal(got, want)                   # uniform(0,1) is the raw 53-bit double
    h = NumpyRefHandler(F32, seed=99)
    g = TextbookMT19937(99)
    for shape, p in [((7, 5), 0.8), ((3,), 0.5), ((40, 40), 0.25)]:
        mask = np.full(shape, 9.0, F32)
        h.generate_probability_mask(mask, p)
        want = np.array([1.0 if g.double() < p else 0.0 for _ in range(mask.size)], F32).reshape(shape)
        assert np.array_equal(mask, want)


def test_fill_gaussian_is_the_polar_method_on_the_textbook_stream():
    h = NumpyRefHandler(F64, seed=5)
    g = TextbookMT19937(5)
    cache = []

    def gauss():
        if cache:
            return cache.pop()
        while True:
            x1, x2 = 2.0 * g.double() - 1.0, 2.0 * g.double() - 1.0
            r2 = x1 * x1 + x2 * x2
            if 0.0 < r2 < 1.0:
                break
        f = math.sqrt(-2.0 * math.log(r2) / r2)
        cache.append(f * x1)
        return f * x2

    out = np.zeros((5, 3), F64)                 # 15 values: leaves one cached for the next call
    h.fill_gaussian(1.5, 0.25, out)
    want = np.array([0.25 * gauss() + 1.5 for _ in range(15)]).reshape(5, 3)
    np.testing.assert_allclose(out, want, rtol=1e-15)
    out2 = np.zeros(4, F64)
    h.fill_gaussian(0.0, 1.0, out2)
    np.testing.assert_allclose(out2, [gauss() for _ in range(4)], rtol=1e-15)


# ----------------------------------------------------------- elementwise closed forms
def test_arithmetic_ops_reduce_to_single_ieee_operations(ref):
    rng = np.random.RandomState(0)
    a, b = rng.standard_normal(1000).astype(F32), rng.standard_normal(1000).astype(F32)
    out = np.zeros(1000, F32)
    # each checked against float64 arithmetic rounded once: exact for one IEEE operation
    for op, f in [("add_tt", np.add), ("subtract_tt", np.subtract), ("mult_tt", np.multiply),
                  ("divide_tt", np.divide)]:
        getattr(ref, op)(a, b, out)
        assert np.array_equal(out, f(a.astype(F64), b.astype(F64)).astype(F32)), op
    # out += a*b rounds the product first: differs from a fused multiply-add on some inputs
    acc = rng.standard_normal(1000).astype(F32)
    want = (acc.astype(F64) + (a.astype(F64) * b.astype(F64)).astype(F32).astype(F64)).astype(F32)
    fused = (acc.astype(F64) + a.astype(F64) * b.astype(F64)).astype(F32)
    got = acc.copy()
    ref.mult_add_tt(a, b, got)
    assert np.array_equal(got, want) and not np.array_equal(want, fused)
    got = acc.copy()
    ref.mult_add_st(0.1, a, got)                # python scalar is rounded to float32 first
    want = (acc.astype(F64) + (F64(F32(0.1)) * a.astype(F64)).astype(F32).astype(F64)).astype(F32)
    assert np.array_equal(got, want)
    ref.add_st(0.1, a, out)
    assert np.array_equal(out, (a.astype(F64) + F64(F32(0.1))).astype(F32))
    ref.mult_st(-1.0, a, out)
    assert np.array_equal(out, -a)


def test_modulo_sign_follows_the_dividend(ref):
    a = np.array([-5.0, 5.0, -5.0, 5.5, -7.25, 1e10], F32)
    b = np.array([3.0, -3.0, -3.0, 2.0, 2.0, 3.0], F32)
    out = np.zeros(6, F32)
    ref.modulo_tt(a, b, out)
    assert np.array_equal(out, np.array([-2.0, 2.0, -2.0, 1.5, -1.25, math.fmod(float(F32(1e10)), 3.0)], F32))
    rng = np.random.RandomState(1)
    a, b = (rng.standard_normal(500) * 100).astype(F32), (rng.standard_normal(500) * 7).astype(F32)
    out = np.zeros(500, F32)
    ref.modulo_tt(a, b, out)
    want = np.array([math.fmod(float(x), float(y)) for x, y in zip(a, b)], F32)   # fmod is exact
    assert np.array_equal(out, want)


def test_unary_ops(ref):
    x = np.array([-2.0, -0.0, 0.0, 3.0, np.nan, -np.inf, np.inf], F32)
    out = np.zeros(7, F32)
    ref.sign_t(x, out)
    assert np.array_equal(out[:4], [-1.0, 0.0, 0.0, 1.0]) and np.isnan(out[4])
    assert not np.signbit(out[1])                            # sign(-0.0) is +0.0
    ref.abs_t(x, out)
    assert np.array_equal(out[[0, 1, 2, 3, 5, 6]], [2.0, 0.0, 0.0, 3.0, np.inf, np.inf])
    ref.clip_t(x, -1.0, 1.0, out)
    assert np.array_equal(out[[0, 1, 2, 3, 5, 6]], [-1.0, 0.0, 0.0, 1.0, -1.0, 1.0]) and np.isnan(out[4])
    u = np.random.RandomState(2).uniform(0.1, 10, 1000).astype(F32)
    out = np.zeros(1000, F32)
    ref.sqrt_t(u, out)
    assert np.array_equal(out, np.sqrt(u.astype(F64)).astype(F32))          # correctly rounded
    ref.log_t(u, out)
    np.testing.assert_allclose(out, np.log(u.astype(F64)), rtol=1e-6)
    np.testing.assert_allclose(np.exp(out.astype(F64)), u, rtol=1e-5)       # inverse of exp


def test_rel_gives_negative_zero_for_negatives(ref):
    x = np.array([-3.0, -0.0, 0.0, 2.0, -np.inf, np.nan], F32)
    y = np.ones(6, F32)
    with np.errstate(invalid="ignore"):
        ref.rel(x, y)
    assert y[3] == 2.0 and y[0] == 0.0 and np.signbit(y[0]) and np.signbit(y[1]) and not np.signbit(y[2])
    assert np.isnan(y[4]) and np.isnan(y[5])                 # -inf * 0 and nan * 0


def _sigmoid64(x):
    return 1.0 / (1.0 + np.exp(-x.astype(F64)))


def test_activations_closed_forms(ref, ref64):
    rng = np.random.RandomState(3)
    x = (rng.standard_normal(2000) * 6).astype(F32)
    y = np.zeros_like(x)
    ref.sigmoid(x, y)
    np.testing.assert_allclose(y, _sigmoid64(x), rtol=5e-7)
    y2 = np.zeros_like(x)
    ref.sigmoid(-x, y2)
    np.testing.assert_allclose(y.astype(F64) + y2, 1.0, atol=2e-7)          # s(x) + s(-x) = 1
    big = np.array([-200.0, 200.0, -90.0], F32)
    yb = np.zeros(3, F32)
    with np.errstate(over="raise", invalid="raise"):                                          # no overflow in either branch
        ref.sigmoid(big, yb)
    assert yb[0] == 0.0 and yb[1] == 1.0 and 0.0 < yb[2] < 1e-38
    ref.tanh(x, y)
    np.testing.assert_allclose(y, np.tanh(x.astype(F64)), rtol=3e-7)
    ref.el(x, y)
    xd = x.astype(F64)
    np.testing.assert_allclose(y, np.where(xd >= 0, xd, np.expm1(xd)), rtol=1e-5, atol=3e-7)
    # derivatives are written in terms of the OUTPUT y; check against finite differences of the
    # forward function in float64
    x64 = rng.standard_normal(200) * 2
    eps = 1e-6
    for fwd, deriv in [("sigmoid", "sigmoid_deriv"), ("tanh", "tanh_deriv"), ("rel", "rel_deriv"),
                       ("el", "el_deriv")]:
        y0, yp, ym = np.zeros(200), np.zeros(200), np.zeros(200)
        getattr(ref64, fwd)(x64, y0)
        getattr(ref64, fwd)(x64 + eps, yp)
        getattr(ref64, fwd)(x64 - eps, ym)
        dy = rng.standard_normal(200)
        dx = np.zeros(200)
        getattr(ref64, deriv)(None, y0, dy, dx)             # x is not needed
        np.testing.assert_allclose(dx, dy * (yp - ym) / (2 * eps), rtol=1e-5, atol=1e-8, err_msg=deriv)


def test_conditional_ops(ref):
    a = np.arange(6, dtype=F32)
    cond = np.array([0.0, 1.0, -2.0, 0.0, np.nan, -0.0], F32)     # non-zero (and NaN) select
    out = np.full(6, 10.0, F32)
    ref.copy_to_if(a, out, cond)
    assert np.array_equal(out, [10, 1, 2, 10, 4, 10])
    out = np.full(6, 10.0, F32)
    ref.add_into_if(a, out, cond)
    assert np.array_equal(out, [10, 11, 12, 10, 14, 10])
    ref.fill_if(out, -1.0, cond)
    assert np.array_equal(out, [10, -1, -1, 10, -1, 10])


# ------------------------------------------------------------- broadcast / reductions
def test_mv_ops_against_explicit_loops(ref):
    rng = np.random.RandomState(4)
    m = rng.standard_normal((5, 7)).astype(F32)
    row, col = rng.standard_normal((1, 7)).astype(F32), rng.standard_normal((5, 1)).astype(F32)
    ops = {"add_mv": lambda p, q: p + q, "subtract_mv": lambda p, q: p - q,
           "mult_mv": lambda p, q: p * q, "divide_mv": lambda p, q: p / q}
    for name, f in ops.items():
        for v, pick in ((row, lambda i, j: row[0, j]), (col, lambda i, j: col[i, 0])):
            out = np.zeros_like(m)
            getattr(ref, name)(m, v, out)
            want = np.array([[f(m[i, j], pick(i, j)) for j in range(7)] for i in range(5)], F32)
            assert np.array_equal(out, want), name
    out = rng.standard_normal((5, 7)).astype(F32)
    want = np.array([[F32(out[i, j] + F32(m[i, j] * col[i, 0])) for j in range(7)] for i in range(5)], F32)
    ref.mult_add_mv(m, col, out)
    assert np.array_equal(out, want)


def test_broadcast_merge_split(ref):
    rng = np.random.RandomState(5)
    a = rng.standard_normal((2, 1, 4)).astype(F32)
    out = np.zeros((2, 3, 4), F32)
    ref.broadcast_t(a, 1, out)
    for k in range(3):
        assert np.array_equal(out[:, k, :], a[:, 0, :])
    x, y = rng.standard_normal((3, 2, 5)).astype(F32), rng.standard_normal((3, 2, 3)).astype(F32)
    merged = np.zeros((3, 2, 8), F32)
    ref.merge_tt(x, y, merged)
    assert np.array_equal(merged, np.concatenate([x, y], axis=-1))
    oa, ob = np.ones_like(x), np.ones_like(y)
    ref.split_add_tt(merged, oa, ob)                       # round trip, and it ADDS
    assert np.array_equal(oa, x + 1) and np.array_equal(ob, y + 1)


def test_sum_t_shapes_and_consistency(ref):
    rng = np.random.RandomState(6)
    a = rng.standard_normal((37, 53)).astype(F32)
    s0, s0k = np.zeros(53, F32), np.zeros((1, 53), F32)
    s1, s1k = np.zeros(37, F32), np.zeros((37, 1), F32)
    tot = np.zeros((), F32)
    ref.sum_t(a, 0, s0); ref.sum_t(a, 0, s0k); ref.sum_t(a, 1, s1); ref.sum_t(a, 1, s1k); ref.sum_t(a, None, tot)
    a64 = a.astype(F64)
    np.testing.assert_allclose(s0, [a64[:, j].sum() for j in range(53)], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(s1, [a64[i, :].sum() for i in range(37)], rtol=1e-5, atol=1e-5)
    assert np.array_equal(s0k[0], s0) and np.array_equal(s1k[:, 0], s1)
    np.testing.assert_allclose(tot, s0.astype(F64).sum(), rtol=1e-5)
    np.testing.assert_allclose(tot, s1.astype(F64).sum(), rtol=1e-5)


def test_softmax_invariants(ref):
    rng = np.random.RandomState(7)
    m = (rng.standard_normal((20, 33)) * 5).astype(F32)
    out = np.zeros_like(m)
    ref.softmax_m(m, out)
    np.testing.assert_allclose(out.astype(F64).sum(axis=1), 1.0, atol=1e-6)           # rows sum to 1
    shifted = np.zeros_like(m)
    ref.softmax_m((m + F32(3.0)).astype(F32), shifted)
    np.testing.assert_allclose(shifted, out, rtol=2e-5)                              # shift invariant
    e = np.exp(m.astype(F64))
    np.testing.assert_allclose(out, e / e.sum(axis=1, keepdims=True), rtol=1e-5)      # definition
    assert np.array_equal(np.argmax(out, axis=1), np.argmax(m, axis=1))
    huge = np.array([[1000.0, 1000.0, -1000.0]], F32)                                # no overflow
    o = np.zeros_like(huge)
    ref.softmax_m(huge, o)
    np.testing.assert_allclose(o, [[0.5, 0.5, 0.0]])


def test_binarize_and_index(ref):
    rng = np.random.RandomState(8)
    labels = rng.randint(0, 6, (9, 1)).astype(F32)
    out = np.full((9, 6), 5.0, F32)
    ref.binarize_v(labels, out)
    for i in range(9):
        for j in range(6):
            assert out[i, j] == (1.0 if j == int(labels[i, 0]) else 0.0)
    m = rng.standard_normal((9, 6)).astype(F32)
    picked = np.zeros((9, 1), F32)
    ref.index_m_by_v(m, labels, picked)
    assert np.array_equal(picked[:, 0], [m[i, int(labels[i, 0])] for i in range(9)])
    assert np.array_equal(picked[:, 0], (m * out).sum(axis=1))        # gather == one-hot dot product


def test_dot_transposes(ref):
    rng = np.random.RandomState(9)
    a, b = rng.standard_normal((3, 4)).astype(F32), rng.standard_normal((4, 5)).astype(F32)

    def loops(x, y):
        return np.array([[sum(float(x[i, k]) * float(y[k, j]) for k in range(x.shape[1]))
                          for j in range(y.shape[1])] for i in range(x.shape[0])])

    want = loops(a, b)
    for ta, tb in itertools.product((False, True), repeat=2):
        out = np.ones((3, 5), F32)
        ref.dot_mm(np.ascontiguousarray(a.T) if ta else a, np.ascontiguousarray(b.T) if tb else b, out, ta, tb)
        np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-6)
        ref.dot_add_mm(np.ascontiguousarray(a.T) if ta else a, np.ascontiguousarray(b.T) if tb else b, out, ta, tb)
        np.testing.assert_allclose(out, 2 * want, rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------- pooling (cpuop.c)
def _out_size(n, k, pad, stride):
    return (n + 2 * pad - k) // stride + 1


def _windows(h, w, win, pad, stride, oh, ow):
    """Yields (yo, xo, [(iy, ix), ...]) with the in-image pixels of each window in scan order."""
    for yo in range(oh):
        for xo in range(ow):
            pix = [(iy, ix)
                   for iy in range(yo * stride[0] - pad, yo * stride[0] - pad + win[0])
                   for ix in range(xo * stride[1] - pad, xo * stride[1] - pad + win[1])
                   if 0 <= iy < h and 0 <= ix < w]
            yield yo, xo, pix


POOL_CASES = [((2, 5, 6, 3), (2, 2), 0, (2, 2)), ((1, 4, 4, 2), (3, 3), 1, (1, 1)), ((2, 5, 5, 1), (3, 2), 2, (2, 1)),
              ((1, 3, 3, 2), (1, 1), 2, (1, 1)), ((1, 7, 5, 2), (3, 3), 0, (2, 2)), ((1, 6, 6, 1), (2, 3), 1, (3, 3))]


@pytest.mark.parametrize("dtype", [F32, F64])
def test_maxpool_forward_backward_brute_force(dtype):
    h_ = NumpyRefHandler(dtype, seed=0)
    rng = np.random.RandomState(10)
    for shape, win, pad, stride in POOL_CASES:
        n, h, w, c = shape
        oh, ow = _out_size(h, win[0], pad, stride[0]), _out_size(w, win[1], pad, stride[1])
        x = rng.randint(-3, 4, shape).astype(dtype)                  # many ties
        out, arg = np.full((n, oh, ow, c), 9, dtype), np.full((n, oh, ow, c), 9, dtype)
        h_.maxpool2d_forward_batch(x, win, out, pad, stride, arg)
        for i, ch in itertools.product(range(n), range(c)):
            for yo, xo, pix in _windows(h, w, win, pad, stride, oh, ow):
                if not pix:
                    assert out[i, yo, xo, ch] == 0 and arg[i, yo, xo, ch] == -1      # empty window
                    continue
                vals = [x[i, iy, ix, ch] for iy, ix in pix]
                k = int(np.argmax(vals))                                             # first maximum
                iy, ix = pix[k]
                assert out[i, yo, xo, ch] == vals[k]
                assert arg[i, yo, xo, ch] == (iy * w + ix) * c + ch
        # backward: every output adds its delta to the pixel its argmax names
        dout = rng.standard_normal(out.shape).astype(dtype)
        din = rng.standard_normal(shape).astype(dtype)
        want = din.astype(F64).copy()
        for i, ch in itertools.product(range(n), range(c)):
            for yo, xo, pix in _windows(h, w, win, pad, stride, oh, ow):
                if pix:
                    loc = int(arg[i, yo, xo, ch]) // c
                    want[i, loc // w, loc % w, ch] += dout[i, yo, xo, ch]
        got = din.copy()
        h_.maxpool2d_backward_batch(x, win, out, pad, stride, arg, got, dout)
        np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)


def test_maxpool_nan_and_lowest_values(ref):
    # strict '>' from -FLT_MAX: NaN never wins, and a window of only -FLT_MAX / -inf counts as empty
    lo = np.finfo(F32).min
    x = np.array([np.nan, 1.0, np.nan, np.nan, lo, -np.inf, 2.0, 2.0], F32).reshape(1, 1, 8, 1)
    out, arg = np.zeros((1, 1, 4, 1), F32), np.zeros((1, 1, 4, 1), F32)
    ref.maxpool2d_forward_batch(x, (1, 2), out, 0, (1, 2), arg)
    assert np.array_equal(out.ravel(), [1.0, 0.0, 0.0, 2.0])
    assert np.array_equal(arg.ravel(), [1.0, -1.0, -1.0, 6.0])


@pytest.mark.parametrize("dtype", [F32, F64])
def test_avgpool_forward_backward_brute_force(dtype):
    h_ = NumpyRefHandler(dtype, seed=0)
    rng = np.random.RandomState(11)
    for shape, win, pad, stride in POOL_CASES:
        n, h, w, c = shape
        oh, ow = _out_size(h, win[0], pad, stride[0]), _out_size(w, win[1], pad, stride[1])
        x = rng.standard_normal(shape).astype(dtype)
        out = np.full((n, oh, ow, c), 9, dtype)
        h_.avgpool2d_forward_batch(x, win, out, pad, stride)
        dout = rng.standard_normal(out.shape).astype(dtype)
        din = rng.standard_normal(shape).astype(dtype)
        want_din = din.astype(F64).copy()
        for i, ch in itertools.product(range(n), range(c)):
            for yo, xo, pix in _windows(h, w, win, pad, stride, oh, ow):
                mean = np.mean([F64(x[i, iy, ix, ch]) for iy, ix in pix]) if pix else 0.0   # non-padding pixels only
                np.testing.assert_allclose(out[i, yo, xo, ch], mean, rtol=1e-5, atol=1e-6)
                for iy, ix in pix:
                    want_din[i, iy, ix, ch] += F64(dout[i, yo, xo, ch]) / len(pix)
        got = din.copy()
        h_.avgpool2d_backward_batch(x, win, out, pad, stride, got, dout)
        np.testing.assert_allclose(got, want_din, rtol=1e-5, atol=1e-5)


# ------------------------------------------------------- im2col / col2im / convolution
CONV_CASES = [(5, 4, 3, 3, 3, 0, (1, 1)), (5, 4, 3, 3, 3, 1, (2, 1)), (6, 7, 2, 5, 5, 2, (1, 1)), (4, 5, 1, 2, 3, 1, (2, 3)),
              (3, 3, 2, 1, 1, 0, (1, 1))]


def test_im2col_is_padded_window_extraction(ref64):
    rng = np.random.RandomState(12)
    for h, w, c, kh, kw, pad, stride in CONV_CASES:
        oh, ow = _out_size(h, kh, pad, stride[0]), _out_size(w, kw, pad, stride[1])
        img = rng.standard_normal((h, w, c))
        col = np.full((oh * ow, kh * kw * c), 9.0)
        ref64._im2col(img, kh, kw, pad, stride, col)
        padded = np.pad(img, ((pad, pad), (pad, pad), (0, 0)))
        for yo, xo in itertools.product(range(oh), range(ow)):
            patch = padded[yo * stride[0]:yo * stride[0] + kh, xo * stride[1]:xo * stride[1] + kw, :]
            assert np.array_equal(col[yo * ow + xo], patch.ravel())


def test_col2im_is_the_adjoint_of_im2col_and_accumulates(ref64):
    rng = np.random.RandomState(13)
    for h, w, c, kh, kw, pad, stride in CONV_CASES:
        oh, ow = _out_size(h, kh, pad, stride[0]), _out_size(w, kw, pad, stride[1])
        img = rng.standard_normal((h, w, c))
        cols = rng.standard_normal((oh * ow, kh * kw * c))
        col_of_img = np.zeros_like(cols)
        ref64._im2col(img, kh, kw, pad, stride, col_of_img)
        start = rng.standard_normal((h, w, c))
        back = start.copy()
        ref64._col2im(cols, kh, kw, pad, stride, back)
        # <im2col(x), y> == <x, col2im(y)>, and col2im adds to what is there
        np.testing.assert_allclose(np.sum(col_of_img * cols), np.sum(img * (back - start)), rtol=1e-10)


def _conv_brute_force(x, wts, bias, pad, stride):
    n, h, w, c = x.shape
    f, kh, kw, _ = wts.shape
    oh, ow = _out_size(h, kh, pad, stride[0]), _out_size(w, kw, pad, stride[1])
    out = np.zeros((n, oh, ow, f))
    for i, yo, xo, k in itertools.product(range(n), range(oh), range(ow), range(f)):
        acc = bias[k]
        for ky, kx, ch in itertools.product(range(kh), range(kw), range(c)):
            iy, ix = yo * stride[0] - pad + ky, xo * stride[1] - pad + kx
            if 0 <= iy < h and 0 <= ix < w:
                acc += x[i, iy, ix, ch] * wts[k, ky, kx, ch]
        out[i, yo, xo, k] = acc
    return out


def test_conv_forward_brute_force_and_backward_finite_differences(ref64):
    rng = np.random.RandomState(14)
    for h, w, c, kh, kw, pad, stride in CONV_CASES[:4]:
        n, f = 2, 3
        x, wts, bias = rng.standard_normal((n, h, w, c)), rng.standard_normal((f, kh, kw, c)), rng.standard_normal(f)
        want = _conv_brute_force(x, wts, bias, pad, stride)
        out = np.zeros_like(want)
        ref64.conv2d_forward_batch(x, wts, bias, out, pad, stride)
        np.testing.assert_allclose(out, want, rtol=1e-10, atol=1e-12)
        # loss = sum(out * g): analytic gradients vs central differences
        g = rng.standard_normal(out.shape)
        din = rng.standard_normal(x.shape)
        din0 = din.copy()
        dw, db = np.full_like(wts, 7.0), np.full_like(bias, 7.0)          # must be overwritten
        ref64.conv2d_backward_batch(x, wts, pad, stride, din, g, dw, db)

        def loss(xx, ww, bb):
            o = np.zeros_like(want)
            ref64.conv2d_forward_batch(xx, ww, bb, o, pad, stride)
            return np.sum(o * g)

        def num_grad(arr, which):
            grad = np.zeros_like(arr)
            it = np.nditer(arr, flags=["multi_index"])
            for _ in it:
                idx = it.multi_index
                old = arr[idx]
                arr[idx] = old + 1e-5
                lp = loss(x, wts, bias)
                arr[idx] = old - 1e-5
                lm = loss(x, wts, bias)
                arr[idx] = old
                grad[idx] = (lp - lm) / 2e-5
            return grad

        np.testing.assert_allclose(dw, num_grad(wts, "w"), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(db, num_grad(bias, "b"), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(din - din0, num_grad(x, "x"), rtol=1e-5, atol=1e-6)   # in_deltas are ADDED to


def test_philox_known_answers_and_mask_rule():
    """oracle/philox.py against the generator's published known-answer vectors (Random123's
    kat_vectors for philox4x32 with 10 rounds) and the mask rule against a direct restatement."""
    from oracle import philox
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
            (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kat:
        got = philox.philox4x32_10(np.array([ctr], np.uint32), key)[0]
        assert tuple(int(x) for x in got) == want
    # several counters at once give what each gives alone
    ctrs = np.array([[5, 0, 0, 0], [6, 0, 0, 0], [0xffffffff, 7, 0, 0]], np.uint32)
    many = philox.philox4x32_10(ctrs, (11, 22))
    for i in range(3):
        assert np.array_equal(many[i], philox.philox4x32_10(ctrs[i:i + 1], (11, 22))[0])
    # the mask: block offset+b serves elements 4b..4b+3; 64-bit offsets carry into the second counter word
    seed, offset, n, p = (3 << 32) | 9, (1 << 32) - 2, 19, 0.3
    mask, blocks = philox.probability_mask(n, p, seed, offset)
    assert blocks == 5 and mask.shape == (n,)
    for i in range(n):
        b = offset + i // 4
        words = philox.philox4x32_10(np.array([[b & 0xffffffff, b >> 32, 0, 0]], np.uint32), (9, 3))[0]
        assert mask[i] == (1.0 if int(words[i % 4]) < int(np.floor(0.3 * 2 ** 32)) else 0.0)
    assert philox.mask_threshold(1.0) == 2 ** 32 and philox.mask_threshold(0.0) == 0 and philox.mask_threshold(-1.0) == 0
    big, _ = philox.probability_mask(400000, 0.8, 1234, 0)
    assert abs(float(big.mean()) - 0.8) < 0.005
