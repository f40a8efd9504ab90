"""GPU parity: HipHandler against the CPU oracle, operation by operation.

Structured like brainstorm/tests/test_handlers_against_reference.py: every
ndarray argument is uploaded, the operation runs on both handlers, and EVERY
array argument is compared afterwards (so in-place side effects are pinned
too). Where the reference compares with allclose(rtol=1e-5), this file uses the
stricter bars the operation allows:

  exact   bit-for-bit (all arithmetic made of single IEEE float32 operations,
          integer/indexing operations, the MT19937 mask stream)
  ulp     transcendentals, see test_transcendentals for the stated bound
  rel     1e-5 relative for reductions, softmax and matrix products
"""
import itertools

import numpy as np
import pytest

from util import assert_bit_equal, assert_max_ulp, sum_tolerance, ulp_distance

pytestmark = pytest.mark.gpu

F32 = np.float32
# the reference's shapes (test_handlers_against_reference.py:24-25) ...
some_2d_shapes = ((1, 1), (4, 1), (1, 4), (5, 5), (3, 4), (4, 3))
some_nd_shapes = ((1, 1, 4), (1, 1, 3, 3), (3, 4, 2, 1))
# ... plus shapes that exercise whole tiles, tile tails and odd row lengths
# ((1201, 2049): 2404 tiles of 1024 floats, i.e. two whole groups of tiles that the kernels with two
# inputs deal to the XCDs in runs, and a rest that keeps its order)
big_shapes = ((64, 64), (37, 1031), (4096,), (3, 5000), (1000, 205), (100, 1200), (513, 2048), (1201, 2049))


def rand(rng, shape):
    return np.asarray(rng.standard_normal(shape), dtype=F32)


def operation_check(hip, ref, op_name, ref_args, compare="exact", **tol):
    """Runs op_name on both handlers; returns the list of (ref_array, hip_array_as_numpy)."""
    args = [hip.create_from_numpy(a) if isinstance(a, np.ndarray) else a for a in ref_args]
    getattr(ref, op_name)(*ref_args)
    getattr(hip, op_name)(*args)
    pairs = []
    for i, (r, a) in enumerate(zip(ref_args, args)):
        if not isinstance(r, np.ndarray):
            continue
        got = hip.get_numpy_copy(a)
        what = "%s arg %d shape %r" % (op_name, i, r.shape)
        if compare == "exact":
            assert_bit_equal(got, r, what)
        elif compare == "ulp":
            assert_max_ulp(got, r, tol["max_ulp"], what)
        elif compare == "rel":
            np.testing.assert_allclose(got, r, rtol=tol.get("rtol", 1e-5), atol=tol.get("atol", 0),
                                       err_msg=what)
        pairs.append((r, got))
    return pairs


# ------------------------------------------------------------------ elementwise
BINARY_OPS = ["add_tt", "subtract_tt", "mult_tt", "divide_tt", "modulo_tt", "mult_add_tt"]


@pytest.mark.parametrize("op", BINARY_OPS)
def test_binary_tt_exact(hip, ref, op):
    rng = np.random.RandomState(0)
    for shape in some_2d_shapes + some_nd_shapes + big_shapes:
        a, b, out = rand(rng, shape), rand(rng, shape), rand(rng, shape)
        operation_check(hip, ref, op, (a, b, out))


@pytest.mark.parametrize("op", BINARY_OPS)
def test_binary_tt_in_place(hip, ref, op):
    # out aliases an input, as the layers do (e.g. add_tt(dbi, tmp, dbi), lstm_layer.py:228)
    rng = np.random.RandomState(1)
    for shape in ((5, 5), (37, 1031)):
        a, b = rand(rng, shape), rand(rng, shape)
        want_a, want_b = a.copy(), b.copy()
        getattr(ref, op)(want_a, want_b, want_a)
        da, db = hip.create_from_numpy(a), hip.create_from_numpy(b)
        getattr(hip, op)(da, db, da)
        assert_bit_equal(da.get(), want_a, op + " out is a")
        want_a2, want_b2 = a.copy(), b.copy()
        getattr(ref, op)(want_a2, want_b2, want_b2)
        da, db = hip.create_from_numpy(a), hip.create_from_numpy(b)
        getattr(hip, op)(da, db, db)
        assert_bit_equal(db.get(), want_b2, op + " out is b")


def test_special_values_exact(hip, ref):
    special = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38,
                        -3.4e38, 1.17549435e-38, 0.5, -2.5, 7.0, 1e-20], dtype=F32)
    a, b = np.meshgrid(special, special)
    a, b = a.copy(), b.copy()
    with np.errstate(all="ignore"):
        for op in ("add_tt", "subtract_tt", "mult_tt", "divide_tt", "modulo_tt", "mult_add_tt"):
            operation_check(hip, ref, op, (a.copy(), b.copy(), np.ones_like(a)))
        for op in ("abs_t", "sign_t", "sqrt_t", "rel"):
            operation_check(hip, ref, op, (a.copy(), np.zeros_like(a)))
        operation_check(hip, ref, "clip_t", (a.copy(), -1.0, 1.0, np.zeros_like(a)))
        for op in ("rel_deriv", "sigmoid_deriv", "tanh_deriv", "el_deriv"):
            operation_check(hip, ref, op, (None, a.copy(), b.copy(), np.zeros_like(a)))


@pytest.mark.parametrize("op,scalar", [("add_st", 0.1), ("mult_st", 0.5), ("mult_add_st", 0.5),
                                       ("mult_st", -1.0), ("mult_add_st", -0.0125), ("add_st", 1e-8)])
def test_scalar_ops_exact(hip, ref, op, scalar):
    rng = np.random.RandomState(2)
    for shape in some_2d_shapes + some_nd_shapes + big_shapes:
        t, out = rand(rng, shape), rand(rng, shape)
        operation_check(hip, ref, op, (scalar, t, out))


@pytest.mark.parametrize("op", ["abs_t", "sign_t", "rel"])
def test_unary_exact(hip, ref, op):
    rng = np.random.RandomState(3)
    for shape in some_2d_shapes + some_nd_shapes + big_shapes:
        a = rand(rng, shape)
        a.ravel()[::7] = 0.0          # sign_t of zeros (test_handlers_against_reference.py:305-313)
        operation_check(hip, ref, op, (a, np.zeros_like(a)))


def test_sqrt_exact(hip, ref):
    # IEEE-correct square root: identical bits. Inputs as in the reference's test (x + 10)
    # and the U(0.1, 10) of the op sweep.
    rng = np.random.RandomState(4)
    for shape in some_2d_shapes + big_shapes:
        a = (rand(rng, shape) + 10).astype(F32)
        operation_check(hip, ref, "sqrt_t", (a, np.zeros_like(a)))
        a = rng.uniform(0.1, 10, shape).astype(F32)
        operation_check(hip, ref, "sqrt_t", (a, np.zeros_like(a)))


def test_clip_exact(hip, ref):
    rng = np.random.RandomState(5)
    for shape in some_2d_shapes + some_nd_shapes + big_shapes:
        a = rand(rng, shape)
        operation_check(hip, ref, "clip_t", (a, -1.0, 1.0, np.zeros_like(a)))
        operation_check(hip, ref, "clip_t", (np.abs(a), 1e-6, 1.0, np.zeros_like(a)))


@pytest.mark.parametrize("op", ["rel_deriv", "sigmoid_deriv", "tanh_deriv", "el_deriv"])
def test_derivs_exact(hip, ref, op):
    rng = np.random.RandomState(6)
    for shape in some_2d_shapes + some_nd_shapes + big_shapes:
        y, dy = rand(rng, shape), rand(rng, shape)
        # x is never read by a derivative (debug_handler.py:489 passes None)
        operation_check(hip, ref, op, (None, y, dy, np.zeros_like(y)))
    # in-place form used by the layers: f(y, y, dy, dy)   (base_handler.py:50-56)
    y, dy = rand(rng, (37, 1031)), rand(rng, (37, 1031))
    want = dy.copy()
    getattr(ref, op)(y, y, want, want)
    dyd, yd = hip.create_from_numpy(dy), hip.create_from_numpy(y)
    getattr(hip, op)(yd, yd, dyd, dyd)
    assert_bit_equal(dyd.get(), want, op + " in place")


@pytest.mark.parametrize("op", ["copy_to_if", "add_into_if"])
def test_cond_ops_exact(hip, ref, op):
    rng = np.random.RandomState(7)
    for shape in some_2d_shapes + some_nd_shapes + big_shapes:
        a, out = rand(rng, shape), rand(rng, shape)
        cond = (rng.uniform(size=shape) < 0.5).astype(F32) * rand(rng, shape)
        operation_check(hip, ref, op, (a, out, cond))


def test_fill_if_exact(hip, ref):
    rng = np.random.RandomState(8)
    for shape in some_2d_shapes + big_shapes:
        mem = rand(rng, shape)
        cond = (rng.uniform(size=shape) < 0.5).astype(F32)
        operation_check(hip, ref, "fill_if", (mem, 2.5, cond))


def test_fill_copy_allocate(hip, ref):
    rng = np.random.RandomState(9)
    for shape in some_2d_shapes + some_nd_shapes + big_shapes + ((0,), (1, 0, 7), ()):
        a = rand(rng, shape)
        operation_check(hip, ref, "fill", (a, -3.25))
        operation_check(hip, ref, "copy_to", (rand(rng, shape), a))
        for maker in ("allocate", "zeros", "ones"):
            got = getattr(hip, maker)(shape)
            want = getattr(ref, maker)(shape)
            assert got.shape == want.shape
            assert_bit_equal(hip.get_numpy_copy(got), want, maker)


def test_large_fill_uses_every_element(hip):
    # arrays of 2^22 elements and more take the write-through store path
    for n in ((1 << 22), (1 << 22) + 4099, 5000001):
        base = hip.allocate((n + 2,))
        hip.fill(base[1:n + 1], 2.5)                   # odd start address, untouched guards
        got = base.get()
        assert got[0] == 0.0 and got[-1] == 0.0
        assert np.array_equal(got[1:n + 1], np.full(n, 2.5, F32))
        big = hip.allocate((n,))                       # zero fill of the allocation itself
        assert not big.get().any()


def test_allocate_reuses_blocks_zeroed(hip):
    # a pool block that comes back must be handed out zero-filled again
    for _ in range(3):
        a = hip.allocate((1000, 33))
        hip.fill(a, 7.0)
        del a
        b = hip.allocate((1000, 33))
        assert not hip.get_numpy_copy(b).any()
        del b


def test_set_from_numpy_casts_and_broadcasts(hip, ref):
    mem = hip.allocate((3, 4))
    hip.set_from_numpy(mem, np.arange(12, dtype=np.float64).reshape(3, 4))
    assert_bit_equal(mem.get(), np.arange(12, dtype=F32).reshape(3, 4))
    hip.set_from_numpy(mem, np.arange(4, dtype=np.int32))       # numpy_handler.py:65 broadcasts
    assert_bit_equal(mem.get(), np.broadcast_to(np.arange(4, dtype=F32), (3, 4)))


# -------------------------------------------------------------- transcendentals
# The bars for float32 transcendentals against the float32 oracle (NumpyHandler's results):
#   tanh:            every element within 2 ulp;
#   sigmoid, log_t:  every element within 4 ulp, and at least 99.9 % of the elements of an array of
#                    10^4 or more within 2 ulp.
# and against the float64 evaluation of the reference formula rounded to float32: within 1 ulp, always.
# A flat "2 ulp to NumpyHandler" cannot be met by any implementation for sigmoid and log_t: NumPy's
# float32 SIMD exp/log are themselves up to 3 ulp from the correctly rounded value (which host CPU
# decides where), and the result here is within 1 ulp of it.
ORACLE_MAX_ULP = {"tanh": 2, "sigmoid": 4, "log_t": 4}
ORACLE_MIN_FRACTION_WITHIN_2 = 0.999


def _check_transcendental(hip, ref, op, x, exact_f64, label):
    want32 = np.zeros_like(x)
    getattr(ref, op)(x.copy(), want32)
    xd = hip.create_from_numpy(x)
    yd = hip.allocate(x.shape)
    getattr(hip, op)(xd, yd)
    got = yd.get()
    with np.errstate(all="ignore"):
        truth = exact_f64(x.astype(np.float64)).astype(F32)
    d_truth = ulp_distance(got, truth)
    d_oracle = ulp_distance(got, want32)
    oracle_err = ulp_distance(want32, truth)
    within2 = float(np.mean(d_oracle <= 2))
    print("%s %s: max ulp to float32 oracle %d (oracle itself %d from float64 truth), "
          "fraction within 2 ulp %.6f" % (op, label, d_oracle.max(), oracle_err.max(), within2))
    assert d_truth.max() <= 1, "%s %s: %d ulp from the float64 evaluation" % (op, label, d_truth.max())
    assert d_oracle.max() <= ORACLE_MAX_ULP[op], "%s %s: %d ulp from the float32 oracle" % (op, label, d_oracle.max())
    if x.size >= 10000:
        assert within2 >= ORACLE_MIN_FRACTION_WITHIN_2, "%s %s: only %.6f within 2 ulp" % (op, label, within2)
    # in place must give the same bits
    getattr(hip, op)(xd, xd)
    assert_bit_equal(xd.get(), got, op + " in place")


def _sigmoid64(x):
    e = np.exp(-np.abs(x))
    return np.where(x >= 0, 1.0 / (1.0 + e), e / (1.0 + e))


@pytest.mark.parametrize("shape", [(5, 5), (37, 1031), (1024, 1024)])
def test_transcendentals(hip, ref, shape):
    rng = np.random.RandomState(10)
    x = rand(rng, shape)
    _check_transcendental(hip, ref, "tanh", x, np.tanh, "N(0,1)")
    _check_transcendental(hip, ref, "sigmoid", x, _sigmoid64, "N(0,1)")
    _check_transcendental(hip, ref, "tanh", (x * 8).astype(F32), np.tanh, "N(0,64)")
    _check_transcendental(hip, ref, "sigmoid", (x * 30).astype(F32), _sigmoid64, "N(0,900)")
    u = rng.uniform(0.1, 10, shape).astype(F32)
    _check_transcendental(hip, ref, "log_t", u, np.log, "U(0.1,10)")
    _check_transcendental(hip, ref, "log_t", (x + 10).astype(F32), np.log, "N(10,1)")


def test_transcendentals_special_values(hip):
    # signed zeros, infinities, NaN, denormals, the clamping thresholds and beyond: the bits of the
    # float64 evaluation rounded to float32
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1e-40, -1e-40, 1.17549435e-38,
                  -1.17549435e-38, 1e-30, -1e-30, 1e-10, -1e-10, 0.17, -0.17, 0.1733, -0.1733, 0.3466, -0.3466,
                  8.9, 9.1, -9.1, 19.99, 20.0, 20.01, -20.01, 87.0, -87.0, 88.8, -88.8, 103.0, -103.0, 104.5,
                  -104.5, 199.0, -199.0, 201.0, -201.0, 1e10, -1e10, 3.4e38, -3.4e38, 1.0, -1.0, 0.5, 2.0],
                 dtype=F32)
    xd = hip.create_from_numpy(x)
    yd = hip.allocate(x.shape)
    x64 = x.astype(np.float64)
    with np.errstate(all="ignore"):
        hip.tanh(xd, yd)
        assert_bit_equal(yd.get(), np.tanh(x64).astype(F32), "tanh of special values")
        hip.sigmoid(xd, yd)
        assert_bit_equal(yd.get(), _sigmoid64(x64).astype(F32), "sigmoid of special values")
        hip.log_t(xd, yd)
        assert_bit_equal(yd.get(), np.log(x64).astype(F32), "log of special values")


def test_el(hip, ref):
    # el = x*(x>=0) + (exp(x)-1)*(x<0) in float32 steps (numpy_handler.py:305). exp(x)-1 cancels,
    # so an ulp of exp(x) (<= 2^-24 for x<0) is an ABSOLUTE error of the result: the bound is
    # 3 ulp of 1.0 = 3 * 2^-24 absolute (2 for NumPy's exp, 1 for the rounding of ours) or 2 ulp.
    rng = np.random.RandomState(11)
    for shape in ((5, 5), (37, 1031)):
        x = rand(rng, shape)
        want = np.zeros_like(x)
        ref.el(x, want)
        xd, yd = hip.create_from_numpy(x), hip.allocate(shape)
        hip.el(xd, yd)
        got = yd.get()
        ok = (np.abs(got.astype(np.float64) - want) <= 3 * 2.0 ** -24) | (ulp_distance(got, want).reshape(shape) <= 2)
        assert ok.all()


# ----------------------------------------------------------------- broadcast
MV_OPS = ["add_mv", "subtract_mv", "mult_mv", "divide_mv", "mult_add_mv"]


@pytest.mark.parametrize("op", MV_OPS)
def test_mv_row_and_column_exact(hip, ref, op):
    rng = np.random.RandomState(12)
    shapes = some_2d_shapes + ((64, 64), (37, 1031), (100, 1200), (1000, 205), (513, 2048), (100, 10),
                               (2048, 4096), (7, 16384))
    for shape in shapes:
        m, out = rand(rng, shape), rand(rng, shape)
        row = (rand(rng, (1, shape[1])) + 3).astype(F32)
        col = (rand(rng, (shape[0], 1)) + 3).astype(F32)
        operation_check(hip, ref, op, (m, row, out))
        operation_check(hip, ref, op, (m.copy(), col, out.copy()))
    # in place: out is m (FullyConnected: add_mv(y, bias, y))
    m = rand(rng, (100, 1200))
    row = rand(rng, (1, 1200))
    want = m.copy()
    getattr(ref, op)(want, row, want)
    md = hip.create_from_numpy(m)
    getattr(hip, op)(md, hip.create_from_numpy(row), md)
    assert_bit_equal(md.get(), want, op + " in place")


def test_mv_one_dimensional_vector_is_a_row(hip, ref):
    # conv bias arrives as a 1-D (F,) vector (pycuda_handler.py:256-257)
    rng = np.random.RandomState(13)
    m, v = rand(rng, (50, 32)), rand(rng, (32,))
    out = np.zeros_like(m)
    ref.add_mv(m, v, out)
    od = hip.allocate(m.shape)
    hip.add_mv(hip.create_from_numpy(m), hip.create_from_numpy(v), od)
    assert_bit_equal(od.get(), out)


def test_mult_mv_same_shape(hip, ref):
    rng = np.random.RandomState(14)
    m, v = rand(rng, (5, 7)), rand(rng, (5, 7))
    operation_check(hip, ref, "mult_mv", (m, v, np.zeros_like(m)))


def test_broadcast_t_exact(hip, ref):
    # the 7 cases of test_handlers_against_reference.py:242-257 and larger ones
    rng = np.random.RandomState(15)
    cases = [((1, 4), 0, (3, 4)), ((3, 1), 1, (3, 4)), ((1, 3, 4), 0, (2, 3, 4)),
             ((2, 1, 4), 1, (2, 5, 4)), ((2, 3, 1), 2, (2, 3, 6)), ((1, 1, 3, 3), 0, (4, 1, 3, 3)),
             ((3, 4, 2, 1), 3, (3, 4, 2, 5)), ((1, 1000), 0, (100, 1000)), ((20, 30, 1), 2, (20, 30, 17))]
    for a_shape, axis, out_shape in cases:
        operation_check(hip, ref, "broadcast_t", (rand(rng, a_shape), axis, np.zeros(out_shape, F32)))


def test_merge_split_exact(hip, ref):
    rng = np.random.RandomState(16)
    for rows, na, nb in [((4,), 1, 1), ((3, 2), 3, 5), ((2049,), 3, 1025), ((7, 5), 128, 64)]:
        a, b = rand(rng, rows + (na,)), rand(rng, rows + (nb,))
        out = np.zeros(rows + (na + nb,), F32)
        operation_check(hip, ref, "merge_tt", (a, b, out))
        x = rand(rng, rows + (na + nb,))
        operation_check(hip, ref, "split_add_tt", (x, a.copy(), b.copy()))


# ------------------------------------------------------------------ reductions
def _check_sum(hip, ref, a, axis, out_shape):
    want = np.zeros(out_shape, F32)
    ref.sum_t(a, axis, want)
    od = hip.create_from_numpy(np.full(out_shape, 99.0, F32))
    hip.sum_t(hip.create_from_numpy(a), axis, od)
    got = od.get()
    assert got.shape == want.shape
    truth = np.sum(a.astype(np.float64), axis=axis)
    tol = sum_tolerance(want, a, axis)
    err = np.abs(got.astype(np.float64).reshape(tol.shape) - want.astype(np.float64).reshape(tol.shape))
    assert np.all(err <= tol), "sum_t axis=%r shape %r: error %g over tolerance" % (
        axis, a.shape, float(np.max(err / tol)))
    # and no further from the float64 sum than the float32 oracle is (up to the same bound)
    err_truth = np.abs(got.astype(np.float64).reshape(tol.shape) - truth.reshape(tol.shape))
    assert np.all(err_truth <= tol)


def test_sum_t(hip, ref):
    rng = np.random.RandomState(17)
    shapes = some_2d_shapes + ((64, 64), (37, 1031), (100, 1200), (1000, 205), (10000, 10), (7, 16384),
                               (2048, 4096), (513, 2049), (100, 1), (1, 100), (3000, 17), (70000, 3))
    for shape in shapes:
        for a in (rand(rng, shape), np.abs(rand(rng, shape))):
            _check_sum(hip, ref, a, 0, (1, shape[1]))
            _check_sum(hip, ref, a, 0, (shape[1],))
            _check_sum(hip, ref, a, 1, (shape[0],))
            _check_sum(hip, ref, a, 1, (shape[0], 1))
            _check_sum(hip, ref, a, None, ())
    # Loss layer: 3-D array, axis None, 0-d output (loss_layer.py:44-46)
    _check_sum(hip, ref, rand(rng, (1, 100, 1)), None, ())
    _check_sum(hip, ref, rand(rng, (1 << 22,)), None, ())
    _check_sum(hip, ref, rand(rng, ((1 << 22) + 13,)), None, ())


def test_sum_t_over_an_axis_of_arrays_with_more_axes(hip, ref):
    # NumpyHandler takes whatever np.sum takes (numpy_handler.py:268-273): any axis of any array,
    # negative axes, out with or without the summed axis kept
    rng = np.random.RandomState(18)
    for shape in ((2, 3, 4), (5, 300, 7), (300, 5, 260), (3, 4, 5, 6), (1, 2049, 3), (4, 1, 9), (40, 3, 1)):
        a = rand(rng, shape)
        for axis in list(range(len(shape))) + [-1, -2]:
            want = np.sum(a.astype(np.float64), axis=axis)
            for out_shape in (want.shape, np.sum(a, axis=axis, keepdims=True).shape):
                _check_sum(hip, ref, a, axis, out_shape)
    with pytest.raises(ValueError):
        hip.sum_t(hip.allocate((2, 3, 4)), 3, hip.allocate((2, 3)))


def test_copy_to_broadcasts_like_numpy(hip, ref):
    # np.copyto(dest, src) broadcasts src (numpy_handler.py:47-52)
    rng = np.random.RandomState(19)
    cases = [((1, 7), (5, 7)), ((7,), (5, 7)), ((5, 1), (5, 7)), ((1,), (5, 7)), ((), (3, 4, 5)), ((1, 1), (3, 4)),
             ((3, 1, 1, 6), (3, 4, 5, 6)), ((4, 260), (3, 4, 260)), ((2, 1, 1028), (2, 300, 1028)), ((5, 7), (5, 7)),
             ((35,), (35,)),
             # repeated axes that are not neighbours: one broadcast per run of them, innermost first
             ((1, 4, 1), (3, 4, 5)), ((4, 1), (3, 4, 5)), ((2, 1, 3, 1), (2, 5, 3, 4)), ((1, 3, 1, 7, 1), (2, 3, 4, 7, 5)),
             ((1, 1, 5), (1, 1, 5)), ((1, 5), (1, 1, 5))]
    for src_shape, dest_shape in cases:
        operation_check(hip, ref, "copy_to", (rand(rng, src_shape), rand(rng, dest_shape)))
    for src_shape, dest_shape in [((3,), (5, 7)), ((2, 7), (5, 7)), ((5, 7, 1), (5, 7)), ((35,), (5, 7))]:
        with pytest.raises(ValueError):
            hip.copy_to(hip.allocate(src_shape), hip.allocate(dest_shape))
        with pytest.raises(ValueError):
            ref.copy_to(np.zeros(src_shape, F32), np.zeros(dest_shape, F32))


def test_sum_t_is_deterministic(hip):
    rng = np.random.RandomState(18)
    a = hip.create_from_numpy(rand(rng, (2048, 4096)))
    outs = []
    for _ in range(3):
        o = hip.allocate((4096,))
        hip.sum_t(a, 0, o)
        outs.append(o.get())
    assert_bit_equal(outs[0], outs[1])
    assert_bit_equal(outs[0], outs[2])


def test_softmax_m(hip, ref):
    rng = np.random.RandomState(19)
    shapes = some_2d_shapes + ((100, 10), (10000, 205), (64, 64), (37, 1031), (16, 4096), (5, 5000),
                               (3, 16384), (2, 70001), (2, 70000), (300, 256), (9, 1024), (9, 1025),
                               # rows 64 KiB or 128 KiB apart: workgroups take the rows in another order,
                               # all of them, some of them and (3 rows) none
                               (64, 16384), (100, 16384), (70, 32768),
                               # more rows than the device holds workgroups at once
                               (1100, 16384), (1030, 12288))
    for shape in shapes:
        for scale in (1.0, 20.0):
            m = (rand(rng, shape) * scale).astype(F32)
            pairs = operation_check(hip, ref, "softmax_m", (m, np.zeros_like(m)), compare="rel", rtol=1e-5, atol=1e-37)
            got = pairs[1][1]
            # invariant the domain gives: rows sum to one
            np.testing.assert_allclose(got.astype(np.float64).sum(axis=1), 1.0, rtol=0, atol=1e-5)
    # in place (softmax_ce_layer.py calls it out of place, but aliasing must be safe)
    m = rand(rng, (100, 205))
    want = np.zeros_like(m)
    ref.softmax_m(m, want)
    md = hip.create_from_numpy(m)
    hip.softmax_m(md, md)
    np.testing.assert_allclose(md.get(), want, rtol=1e-5)


def test_random_shapes_reductions_broadcasts_indexing(hip, ref):
    # the launch plans of these kernels depend on the shape (column lanes, row bands, wavefront or
    # workgroup per row, vector width by divisibility): 80 random shapes, log-uniform in both
    # dimensions, each through sum_t on all axes, softmax_m, the mv operations with both vector
    # shapes, binarize_v and index_m_by_v
    rng = np.random.RandomState(4242)
    for case in range(80):
        rows = int(np.exp(rng.uniform(0, np.log(3000))))
        cols = int(np.exp(rng.uniform(0, np.log(3000))))
        a = rand(rng, (rows, cols))
        _check_sum(hip, ref, a, 0, (1, cols))
        _check_sum(hip, ref, a, 1, (rows, 1))
        _check_sum(hip, ref, a, None, ())
        pairs = operation_check(hip, ref, "softmax_m", (a, np.zeros_like(a)), compare="rel", rtol=1e-5, atol=1e-37)
        np.testing.assert_allclose(pairs[1][1].astype(np.float64).sum(axis=1), 1.0, rtol=0, atol=1e-5)
        row, col = rand(rng, (1, cols)), rand(rng, (rows, 1))
        for op in ("add_mv", "mult_mv", "subtract_mv", "divide_mv"):
            operation_check(hip, ref, op, (a, row, np.zeros_like(a)))
            operation_check(hip, ref, op, (a, col, np.zeros_like(a)))
        operation_check(hip, ref, "mult_add_mv", (a, row, rand(rng, (rows, cols))))
        operation_check(hip, ref, "mult_add_mv", (a, col, rand(rng, (rows, cols))))
        labels = rng.randint(0, cols, (rows, 1)).astype(F32)
        operation_check(hip, ref, "binarize_v", (labels, np.full((rows, cols), 3.0, F32)))
        operation_check(hip, ref, "index_m_by_v", (a, labels, np.zeros((rows, 1), F32)))


def test_is_fully_finite(hip, ref):
    rng = np.random.RandomState(20)
    for shape in ((5, 5), (37, 1031), (1 << 20,)):
        a = rand(rng, shape)
        assert hip.is_fully_finite(hip.create_from_numpy(a)) is True
        for bad in (np.nan, np.inf, -np.inf):
            b = a.copy()
            b.ravel()[b.size // 3] = bad
            assert hip.is_fully_finite(hip.create_from_numpy(b)) is False
            assert bool(ref.is_fully_finite(b)) is False


# -------------------------------------------------------------------- indexing
def test_binarize_v_exact(hip, ref):
    rng = np.random.RandomState(21)
    for rows, k in [(1, 1), (5, 3), (100, 10), (10000, 205), (64, 64), (300, 1031), (512, 4096),
                    (2048, 2048), (4100, 1031), (1025, 4100)]:      # the last three: 2^22 elements and more
        v = rng.randint(0, k, (rows, 1)).astype(F32)
        operation_check(hip, ref, "binarize_v", (v, np.full((rows, k), 7.0, F32)))


def test_index_m_by_v_exact(hip, ref):
    rng = np.random.RandomState(22)
    for rows, k in [(1, 1), (5, 3), (100, 10), (10000, 205), (4096, 4096)]:
        m = rand(rng, (rows, k))
        v = rng.randint(0, k, (rows, 1)).astype(F32)
        operation_check(hip, ref, "index_m_by_v", (m, v, np.zeros((rows, 1), F32)))


def test_negative_labels_count_from_the_last_column(hip, ref):
    # NumPy's indexing wraps labels in [-K, -1] (numpy_handler.py:101, 203: eye[v], m[arange, v]);
    # the kernels do the same, also the fused softmax cross entropy
    rng = np.random.RandomState(23)
    rows, k = 37, 11
    v = rng.randint(-k, k, (rows, 1)).astype(F32)
    v[:4, 0] = [-1, -k, k - 1, 0]
    operation_check(hip, ref, "binarize_v", (v, np.full((rows, k), 7.0, F32)))
    operation_check(hip, ref, "index_m_by_v", (rand(rng, (rows, k)), v, np.zeros((rows, 1), F32)))
    x = rand(rng, (rows, k))
    vd, xd = hip.create_from_numpy(v), hip.create_from_numpy(x)
    probs, loss = hip.allocate((rows, k)), hip.allocate((rows, 1))
    hip.softmax_ce_forward(xd, vd, probs, loss)
    picked = hip.allocate((rows, 1))
    hip.index_m_by_v(probs, vd, picked)
    want = -np.log(np.clip(picked.get(), F32(1e-6), F32(1.0)).astype(np.float64))
    np.testing.assert_allclose(loss.get(), want, rtol=1e-6)
    t_bin, din = hip.allocate((rows, k)), hip.allocate((rows, k))
    hip.softmax_ce_backward(probs, vd, hip.create_from_numpy(np.ones((rows, 1), F32)), t_bin, din)
    onehot = np.zeros((rows, k), F32)
    ref.binarize_v(v, onehot)
    assert_bit_equal(din.get(), (-onehot + probs.get()) * F32(1.0), "softmax - onehot with wrapped labels")


def test_documented_deviations_from_numpy(hip, ref):
    """Two places where the device does something NumpyHandler cannot or does not:
    labels beyond [-K, K) (NumPy raises IndexError; a kernel cannot raise, the row selects no column:
    an all-zero one-hot row, a gathered 0) and sigmoid of NaN (NumPy's two masked assignments skip the
    element and leave y's old value, numpy_handler.py:283-287; the device writes NaN)."""
    k = 5
    v = np.array([[5.0], [-6.0], [1e10], [np.nan], [np.inf], [2.0]], F32)
    vd = hip.create_from_numpy(v)
    out = hip.create_from_numpy(np.full((6, k), 7.0, F32))
    hip.binarize_v(vd, out)
    want = np.zeros((6, k), F32)
    want[5, 2] = 1.0
    assert_bit_equal(out.get(), want, "one-hot rows of labels out of range")
    m = np.arange(30, dtype=F32).reshape(6, k) + 1
    got = hip.allocate((6, 1))
    hip.index_m_by_v(hip.create_from_numpy(m), vd, got)
    assert_bit_equal(got.get(), np.array([[0], [0], [0], [0], [0], [m[5, 2]]], F32), "gather with labels out of range")
    with pytest.raises(IndexError):
        ref.index_m_by_v(m, v[:1], np.zeros((1, 1), F32))
    # sigmoid(NaN)
    x = np.array([0.5, np.nan, -0.5], F32)
    y_ref = np.full(3, 9.0, F32)
    with np.errstate(invalid="ignore"):
        ref.sigmoid(x, y_ref)
    assert y_ref[1] == 9.0                       # the oracle (like NumpyHandler) leaves the old value
    y = hip.create_from_numpy(np.full(3, 9.0, F32))
    hip.sigmoid(hip.create_from_numpy(x), y)
    got = y.get()
    assert np.isnan(got[1]) and got[0] == y_ref[0] and got[2] == y_ref[2]


# ------------------------------------------------------------------------- RNG
def test_handlers_alive_together_keep_their_own_streams(hip):
    # every reference handler owns its random state (numpy_handler.py:21): two handlers with different
    # seeds, their calls interleaved (masks, a repeating pattern that starts the look-ahead, gaussians,
    # a reseed), each reproduce their own RandomState stream; the session's handler is not disturbed
    from brainstorm_amd import HipHandler
    hip.rnd.seed(99)
    rs0 = np.random.RandomState(99)
    m0 = hip.allocate((1000,))
    hip.generate_probability_mask(m0, 0.5)
    assert_bit_equal(m0.get(), (rs0.uniform(size=1000) < 0.5).astype(F32))
    a, b = HipHandler(seed=7), HipHandler(seed=8)            # constructing them reseeds nobody else
    ra, rb = np.random.RandomState(7), np.random.RandomState(8)
    assert a.rnd.get_seed() == 7 and b.rnd.get_seed() == 8
    ma, mb = a.allocate((3, 1200)), b.allocate((777,))
    for step in range(8):
        for _ in range(2):                                   # a: the same two requests every step (look-ahead)
            a.generate_probability_mask(ma, 0.8)
            assert_bit_equal(ma.get(), (ra.uniform(size=(3, 1200)) < 0.8).astype(F32), "handler a, step %d" % step)
        b.generate_probability_mask(mb, 0.3)
        assert_bit_equal(mb.get(), (rb.uniform(size=777) < 0.3).astype(F32), "handler b, step %d" % step)
        if step == 3:
            g = b.allocate((5,))
            b.fill_gaussian(1.0, 2.0, g)
            np.testing.assert_allclose(g.get(), 2.0 * rb.standard_normal(5) + 1.0, rtol=1e-6)
        if step == 5:
            a.rnd.seed(70)
            ra = np.random.RandomState(70)
        hip.generate_probability_mask(m0, 0.5)
        assert_bit_equal(m0.get(), (rs0.uniform(size=1000) < 0.5).astype(F32), "session handler, step %d" % step)
    for h, r in ((a, ra), (b, rb), (hip, rs0)):
        _, key, pos, has_gauss, _ = h.rnd.get_state()
        st = r.get_state()
        assert pos == st[2] and np.array_equal(key, st[1]) and has_gauss == st[3]
    del a, b                                                  # their generators are destroyed with them
    hip.generate_probability_mask(m0, 0.5)
    assert_bit_equal(m0.get(), (rs0.uniform(size=1000) < 0.5).astype(F32), "after the others are gone")


def test_generate_probability_mask_matches_randomstate(hip):
    # Sizes chosen so that consecutive calls start at even and odd positions of the 624-word
    # MT19937 block and cross block boundaries (a 53-bit double takes two words).
    from brainstorm_amd import HipHandler  # noqa: F401  (same library instance)
    for seed in (0, 1, 42, 4294967295):
        hip.rnd.seed(seed)
        rs = np.random.RandomState(seed)
        for shape, p in [((7, 5), 0.8), ((1,), 0.5), ((311,), 0.5), ((312,), 0.3), ((313,), 0.9),
                         ((1, 100, 784), 0.8), ((1, 100, 1200), 0.5), ((3,), 0.5), ((100000,), 0.123)]:
            mask = hip.allocate(shape)
            hip.generate_probability_mask(mask, p)
            want = (rs.uniform(size=shape) < p).astype(F32)
            assert_bit_equal(mask.get(), want, "mask seed %d shape %r" % (seed, shape))
        # the generator state itself must agree with NumPy's afterwards
        _, key, pos, _, _ = hip.rnd.get_state()
        st = rs.get_state()
        assert pos == st[2]
        np.testing.assert_array_equal(key, st[1])


def test_long_masks_drawn_in_parallel_segments_match_randomstate(hip):
    # Long draws (2^20 words = 524 288 doubles or more; inside recorded steps from about 61 000 words) are cut
    # into 4 ... 64 segments of whole 624-word blocks by jump-ahead and generated side by side: masks and
    # the state afterwards must still be those of one sequential RandomState, wherever in its block a draw
    # starts and ends.
    for seed in (3, 2718281828):
        hip.rnd.seed(seed)
        rs = np.random.RandomState(seed)
        for n, p in [(524287, 0.5), (524288, 0.5), (5, 0.5), (524289, 0.3), (311, 0.5), (624 * 900, 0.9),
                     (1000003, 0.2), (4096 * 1024, 0.65), (1, 0.5), (64 * 624 * 50, 0.5), (64 * 624 * 50 + 1, 0.5)]:
            mask = hip.allocate((n,))
            hip.generate_probability_mask(mask, p)
            want = (rs.uniform(size=(n,)) < p).astype(F32)
            assert_bit_equal(mask.get(), want, "mask seed %d, %d elements" % (seed, n))
            _, key, pos, _, _ = hip.rnd.get_state()
            st = rs.get_state()
            assert pos == st[2], "position after %d elements" % n
            np.testing.assert_array_equal(key, st[1], err_msg="key after %d elements" % n)
    # the gaussian stream takes its uniform numbers the same way
    out = hip.allocate((700000,))
    hip.fill_gaussian(0.5, 2.0, out)
    assert_max_ulp(out.get(), (2.0 * rs.standard_normal((700000,)) + 0.5).astype(F32), 1, "long fill_gaussian")
    _, key, pos, has_gauss, _ = hip.rnd.get_state()
    st = rs.get_state()
    assert (pos, has_gauss) == (st[2], st[3])
    np.testing.assert_array_equal(key, st[1])


def test_mask_prefetch_never_changes_the_stream(hip):
    # Repeating request patterns switch on the look-ahead generation on the second stream; whether a
    # request is served from it, misses it, or another consumer of the generator cuts in, the masks
    # and the generator state must be those of one sequential RandomState.
    lib = hip._lib
    hip.rnd.seed(11)
    rs = np.random.RandomState(11)

    def draw(shape, p, tag):
        mask = hip.allocate(shape)
        hip.generate_probability_mask(mask, p)
        want = (rs.uniform(size=shape) < p).astype(F32)
        assert_bit_equal(mask.get(), want, tag)

    def check_state(tag):
        _, key, pos, has_gauss, _ = hip.rnd.get_state()
        st = rs.get_state()
        assert (pos, has_gauss) == (st[2], st[3]), tag
        np.testing.assert_array_equal(key, st[1], err_msg=tag)

    pattern = [((100, 784), 0.8), ((100, 1200), 0.5), ((100, 1200), 0.5)]
    for step in range(7):                      # period 3: served ahead of time from the third step on
        for k, (shape, p) in enumerate(pattern):
            draw(shape, p, "step %d mask %d" % (step, k))
    draw((100, 1200), 0.5, "request out of turn")           # the queue expects (100, 784): rewind
    check_state("after a miss")
    for step in range(5):                      # period 1
        draw((313,), 0.3, "period one, %d" % step)
    check_state("reading the state while masks are queued")
    for step in range(4):
        draw((313,), 0.3, "period one again, %d" % step)
    out = hip.allocate((1001,))                # the gaussian stream cuts in while masks are queued
    hip.fill_gaussian(0.0, 1.0, out)
    assert_max_ulp(out.get(), rs.standard_normal((1001,)).astype(F32), 1, "gaussian after prefetch")
    for step in range(4):
        draw((313,), 0.3, "after the gaussian, %d" % step)
        draw((5, 7), 0.9, "after the gaussian, second mask %d" % step)
    hip.rnd.seed(12)                           # reseeding with masks queued
    rs = np.random.RandomState(12)
    for step in range(4):
        draw((64, 64), 0.5, "reseeded, %d" % step)
    check_state("end")


def test_fill_gaussian_matches_randomstate(hip):
    for seed in (0, 7):
        hip.rnd.seed(seed)
        rs = np.random.RandomState(seed)
        for shape, mean, std in [((5,), 0.0, 1.0), ((4,), 1.5, 0.1), ((1000, 37), -2.0, 3.0), ((1,), 0.0, 1.0),
                                 ((2,), 0.0, 1.0)]:
            out = hip.allocate(shape)
            hip.fill_gaussian(mean, std, out)
            want = (std * rs.standard_normal(shape) + mean).astype(F32)
            # float64 log/sqrt of the device maths library vs the host's: at most 1 float32 ulp
            assert_max_ulp(out.get(), want, 1, "fill_gaussian seed %d shape %r" % (seed, shape))
        # interleave with masks: both draw from the one stream
        mask = hip.allocate((11,))
        hip.generate_probability_mask(mask, 0.5)
        assert_bit_equal(mask.get(), (rs.uniform(size=(11,)) < 0.5).astype(F32))
        _, key, pos, has_gauss, _ = hip.rnd.get_state()
        st = rs.get_state()
        assert (pos, has_gauss) == (st[2], st[3])
        np.testing.assert_array_equal(key, st[1])


# ----------------------------------------------------------------------- dense
def test_dot_mm_and_dot_add_mm(hip, ref):
    rng = np.random.RandomState(23)
    dims = [(1, 1, 1), (4, 1, 3), (5, 5, 5), (3, 4, 2), (100, 784, 1200), (100, 1200, 10), (64, 205, 1000),
            (257, 129, 65)]
    for (m, k, n), ta, tb in itertools.product(dims, (False, True), (False, True)):
        a = rand(rng, (k, m) if ta else (m, k))
        b = rand(rng, (n, k) if tb else (k, n))
        out = rand(rng, (m, n))
        for op in ("dot_mm", "dot_add_mm"):
            want = out.copy()
            getattr(ref, op)(a, b, want, ta, tb)
            od = hip.create_from_numpy(out)
            getattr(hip, op)(hip.create_from_numpy(a), hip.create_from_numpy(b), od, ta, tb)
            # 1e-5 relative to the magnitude of a length-k inner product
            scale = np.sqrt(k) + np.abs(want)
            assert np.max(np.abs(od.get() - want) / scale) <= 1e-5, (op, m, k, n, ta, tb)


def test_dot_mm_with_operands_at_odd_elements(hip, ref):
    # time-step slices and hub slices start at any element of a flat buffer: A, B and C 4-byte but not
    # 16-byte aligned, each shape twice so that the second call runs the cached plan
    rng = np.random.RandomState(29)
    for (m, k, n), ta, tb in itertools.product([(100, 1000, 1000), (37, 129, 65), (5, 3, 2)], (False, True),
                                               (False, True)):
        a = rand(rng, (k, m) if ta else (m, k))
        b = rand(rng, (n, k) if tb else (k, n))
        out = rand(rng, (m, n))
        for offs in ((1, 2, 3), (3, 1, 1)):
            views = []
            for arr, off in zip((a, b, out), offs):
                flat = hip.allocate((arr.size + 4,))
                assert flat.ptr % 16 == 0
                v = flat[off:off + arr.size].reshape(arr.shape)
                hip.set_from_numpy(v, arr)
                views.append(v)
            for op in ("dot_mm", "dot_add_mm"):
                hip.set_from_numpy(views[2], out)
                want = out.copy()
                getattr(ref, op)(a, b, want, ta, tb)
                getattr(hip, op)(views[0], views[1], views[2], ta, tb)
                scale = np.sqrt(k) + np.abs(want)
                assert np.max(np.abs(views[2].get() - want) / scale) <= 1e-5, (op, m, k, n, ta, tb, offs)


def test_first_call_of_a_thin_product_touches_the_result_once(hip, ref):
    # the first call of a shape makes its plan (with BSHIP_GEMM_AUTOTUNE set, after trial runs into a
    # scratch result): an accumulating first call adds the product exactly once, and the later calls
    # (cached plan) repeat the first bit for bit
    rng = np.random.RandomState(31)
    for (m, k, n), ta, tb in itertools.product([(100, 4003, 1001), (7, 333, 4001), (2003, 77, 96)], (False, True),
                                               (False, True)):
        a = rand(rng, (k, m) if ta else (m, k))
        b = rand(rng, (n, k) if tb else (k, n))
        out = rand(rng, (m, n)) * F32(100.0)
        want = out.copy()
        ref.dot_add_mm(a, b, want, ta, tb)
        ad, bd = hip.create_from_numpy(a), hip.create_from_numpy(b)
        results = []
        for _ in range(3):
            od = hip.create_from_numpy(out)
            hip.dot_add_mm(ad, bd, od, ta, tb)
            results.append(od.get())
        scale = np.sqrt(k) + np.abs(want)
        assert np.max(np.abs(results[0] - want) / scale) <= 1e-5, (m, k, n, ta, tb)
        assert_bit_equal(results[1], results[0], "second call")
        assert_bit_equal(results[2], results[0], "third call")


# -------------------------------------------------------------- conv / pooling
def _out_size(n, k, pad, stride):
    return (n + 2 * pad - k) // stride + 1


POOL_CASES = [(n, h, w, c, win, pad, stride)
              for (n, h, w, c) in [(1, 4, 4, 1), (2, 5, 7, 3), (3, 32, 32, 32), (2, 15, 15, 64)]
              for win in [(1, 1), (2, 2), (3, 3), (2, 3), (3, 2), (4, 4)]
              for pad in (0, 1, 2)
              for stride in [(1, 1), (2, 2), (1, 2), (3, 3)]
              if win[0] <= h + 2 * pad and win[1] <= w + 2 * pad]


def test_maxpool_forward_backward_exact(hip, ref):
    rng = np.random.RandomState(24)
    for n, h, w, c, win, pad, stride in POOL_CASES:
        oh, ow = _out_size(h, win[0], pad, stride[0]), _out_size(w, win[1], pad, stride[1])
        x = rand(rng, (n, h, w, c))
        x[rng.uniform(size=x.shape) < 0.3] = 0.5          # ties: the first maximum must win
        out = np.zeros((n, oh, ow, c), F32)
        arg = np.zeros((n, oh, ow, c), F32)
        ref.maxpool2d_forward_batch(x, win, out, pad, stride, arg)
        xd = hip.create_from_numpy(x)
        outd, argd = hip.allocate(out.shape), hip.allocate(arg.shape)
        hip.maxpool2d_forward_batch(xd, win, outd, pad, stride, argd)
        what = "maxpool %r" % ((n, h, w, c, win, pad, stride),)
        assert_bit_equal(outd.get(), out, what + " values")
        assert_bit_equal(argd.get(), arg, what + " argmax")
        dout = rand(rng, out.shape)
        din = rand(rng, x.shape)
        want = din.copy()
        ref.maxpool2d_backward_batch(x, win, out, pad, stride, arg, want, dout)
        dind = hip.create_from_numpy(din)
        hip.maxpool2d_backward_batch(xd, win, outd, pad, stride, argd, dind, hip.create_from_numpy(dout))
        assert_bit_equal(dind.get(), want, what + " backward")


def test_avgpool_forward_backward_exact(hip, ref):
    rng = np.random.RandomState(25)
    for n, h, w, c, win, pad, stride in POOL_CASES:
        oh, ow = _out_size(h, win[0], pad, stride[0]), _out_size(w, win[1], pad, stride[1])
        x = rand(rng, (n, h, w, c))
        out = np.zeros((n, oh, ow, c), F32)
        ref.avgpool2d_forward_batch(x, win, out, pad, stride)
        xd = hip.create_from_numpy(x)
        outd = hip.allocate(out.shape)
        hip.avgpool2d_forward_batch(xd, win, outd, pad, stride)
        what = "avgpool %r" % ((n, h, w, c, win, pad, stride),)
        assert_bit_equal(outd.get(), out, what + " values")
        dout, din = rand(rng, out.shape), rand(rng, x.shape)
        want = din.copy()
        ref.avgpool2d_backward_batch(x, win, out, pad, stride, want, dout)
        dind = hip.create_from_numpy(din)
        hip.avgpool2d_backward_batch(xd, win, outd, pad, stride, dind, hip.create_from_numpy(dout))
        assert_bit_equal(dind.get(), want, what + " backward")


CONV_CASES = [(2, 5, 4, 3, 2, 3, 3, 0, (1, 1)), (2, 5, 4, 3, 2, 3, 3, 1, (2, 1)), (1, 3, 3, 1, 1, 1, 1, 0, (1, 1)),
              (4, 9, 9, 3, 4, 5, 5, 2, (1, 1)), (3, 9, 6, 1, 3, 3, 2, 1, (2, 3)),
              (10, 32, 32, 3, 32, 5, 5, 2, (1, 1)), (10, 15, 15, 32, 64, 5, 5, 2, (1, 1)),
              # channel counts that are no multiple of 4 with a col matrix that is: groups of four
              # col elements that straddle kernel positions and output pixels
              (2, 6, 6, 3, 4, 2, 2, 1, (2, 2)), (5, 8, 4, 2, 3, 3, 3, 1, (1, 1)), (9, 6, 6, 1, 2, 3, 3, 1, (1, 1)),
              # 3x3 and 5x5 windows with stride 1 and 16 or more channels (col2im with all terms of an element
              # loaded together): no padding, the usual padding, and a padding as wide as the window allows
              (3, 7, 6, 16, 4, 3, 3, 1, (1, 1)), (2, 9, 8, 20, 4, 5, 5, 0, (1, 1)), (2, 6, 7, 16, 4, 5, 5, 4, (1, 1)),
              # an image per compute unit and col rows of 9.6 KB: the backward pass's col2im streams the col matrix into LDS
              (256, 10, 32, 3, 4, 5, 5, 2, (1, 1))]


def test_conv2d_forward_backward(hip, ref):
    rng = np.random.RandomState(26)
    for n, h, w, c, f, kh, kw, pad, stride in CONV_CASES:
        oh, ow = _out_size(h, kh, pad, stride[0]), _out_size(w, kw, pad, stride[1])
        x = rand(rng, (n, h, w, c))
        wts = rand(rng, (f, kh, kw, c))
        bias = rand(rng, (f,))
        out = np.zeros((n, oh, ow, f), F32)
        ref.conv2d_forward_batch(x, wts, bias, out, pad, stride)
        xd, wd, bd = hip.create_from_numpy(x), hip.create_from_numpy(wts), hip.create_from_numpy(bias)
        outd = hip.allocate(out.shape)
        hip.conv2d_forward_batch(xd, wd, bd, outd, pad, stride)
        k = kh * kw * c
        scale = np.sqrt(k) + np.abs(out)
        assert np.max(np.abs(outd.get() - out) / scale) <= 1e-5, ("conv fwd", n, h, w, c, f)
        dout = rand(rng, out.shape)
        din = rand(rng, x.shape)
        want_din, dw, db = din.copy(), np.full_like(wts, 5.0), np.full_like(bias, 5.0)
        ref.conv2d_backward_batch(x, wts, pad, stride, want_din, dout, dw, db)
        dind = hip.create_from_numpy(din)
        dwd, dbd = hip.create_from_numpy(np.full_like(wts, 5.0)), hip.create_from_numpy(np.full_like(bias, 5.0))
        hip.conv2d_backward_batch(xd, wd, pad, stride, dind, hip.create_from_numpy(dout), dwd, dbd)
        assert np.max(np.abs(dind.get() - want_din) / (np.sqrt(f * kh * kw) + np.abs(want_din))) <= 1e-5
        assert np.max(np.abs(dwd.get() - dw) / (np.sqrt(n * oh * ow) + np.abs(dw))) <= 1e-5
        assert np.max(np.abs(dbd.get() - db) / (np.sqrt(n * oh * ow) + np.abs(db))) <= 1e-5


THIN_CASES = [  # n, h, w, c, f, kh, kw, pad: stride 1, kh*kw*c <= 128, f a multiple of 16 up to 64
    (10, 32, 32, 3, 32, 5, 5, 2), (3, 28, 28, 1, 16, 5, 5, 0), (2, 9, 7, 3, 16, 3, 3, 1), (5, 17, 13, 2, 48, 5, 3, 2),
    (1, 5, 5, 4, 64, 5, 5, 4), (4, 6, 150, 3, 32, 3, 3, 1), (2, 40, 3, 5, 16, 5, 5, 2), (7, 8, 8, 8, 32, 4, 4, 0),
    (300, 12, 12, 3, 32, 5, 5, 2), (2, 10, 10, 128, 16, 1, 1, 0), (3, 11, 9, 1, 32, 1, 1, 3),
    (2, 64, 64, 1, 16, 7, 7, 3), (1, 96, 96, 3, 16, 3, 3, 1), (2, 33, 65, 2, 32, 3, 5, 1), (5, 7, 100, 1, 64, 1, 9, 4)]


# of these, backward keeps to the im2col path: a row of out_deltas x f beyond 4096 floats
THIN_FORWARD_ONLY = {(4, 6, 150, 3, 32, 3, 3, 1), (5, 7, 100, 1, 64, 1, 9, 4)}


def test_thin_filter_convolutions_forward(hip, ref):
    # filters of at most 128 entries are convolved without a col matrix (bship_conv2d_fwd_thin_f32): against the
    # oracle at the bar of the products, and against the im2col path of the same handler
    rng = np.random.RandomState(261)
    assert hip.thin_convolutions
    for n, h, w, c, f, kh, kw, pad in THIN_CASES:
        oh, ow = _out_size(h, kh, pad, 1), _out_size(w, kw, pad, 1)
        x, wts, bias = rand(rng, (n, h, w, c)), rand(rng, (f, kh, kw, c)), rand(rng, (f,))
        out = np.zeros((n, oh, ow, f), F32)
        ref.conv2d_forward_batch(x, wts, bias, out, pad, (1, 1))
        xd, wd, bd = hip.create_from_numpy(x), hip.create_from_numpy(wts), hip.create_from_numpy(bias)
        outd = hip.create_from_numpy(np.full(out.shape, 7.0, F32))
        status = hip._lib.bship_conv2d_fwd_thin_f32(xd.ptr, h * w * c, wd.ptr, bd.ptr, outd.ptr, n, h, w, c, f, kh, kw,
                                                    pad, 1, 1)
        assert status == 0, (n, h, w, c, f, kh, kw, pad)
        got = outd.get()
        scale = np.sqrt(kh * kw * c) + np.abs(out)
        assert np.max(np.abs(got - out) / scale) <= 1e-5, ("thin conv", n, h, w, c, f, kh, kw, pad)
        hip.thin_convolutions = False
        try:
            other = hip.allocate(out.shape)
            hip.conv2d_forward_batch(xd, wd, bd, other, pad, (1, 1))
        finally:
            hip.thin_convolutions = True
        assert np.max(np.abs(got - other.get()) / scale) <= 2e-6
        hip.conv2d_forward_batch(xd, wd, bd, other, pad, (1, 1))          # and through the handler: the same kernel
        assert_bit_equal(other.get(), got, "handler route")
    # geometries the kernel does not take are refused with nothing done
    lib = hip._lib
    a = hip.allocate((2, 8, 8, 3))
    for f, kh, kw, c, stride in ((20, 3, 3, 3, 1), (80, 3, 3, 3, 1), (16, 7, 7, 3, 1), (16, 3, 3, 3, 2)):
        assert lib.bship_conv2d_fwd_thin_f32(a.ptr, 192, a.ptr, a.ptr, a.ptr, 2, 8, 8, c, f, kh, kw, 1, stride, stride) == -6


def test_thin_filter_convolutions_backward(hip, ref):
    # the same filters backward without a col matrix (bship_conv2d_bwd_thin_f32): weight and bias deltas
    # overwritten, input deltas accumulated; against the oracle at the bar of the products, against the im2col
    # path of the same handler, and the same bits on a second call (sums in a fixed order, no atomics)
    rng = np.random.RandomState(262)
    lib = hip._lib
    for n, h, w, c, f, kh, kw, pad in THIN_CASES:
        if kh * kw * c > 127:
            continue
        oh, ow = _out_size(h, kh, pad, 1), _out_size(w, kw, pad, 1)
        x, wts, dout, din = rand(rng, (n, h, w, c)), rand(rng, (f, kh, kw, c)), rand(rng, (n, oh, ow, f)), rand(rng, (n, h, w, c))
        want_din, dw, db = din.copy(), np.full_like(wts, 5.0), np.full((f,), 5.0, F32)
        ref.conv2d_backward_batch(x, wts, pad, (1, 1), want_din, dout, dw, db)
        xd, wd, doutd = hip.create_from_numpy(x), hip.create_from_numpy(wts), hip.create_from_numpy(dout)
        results = []
        for _ in range(2):
            dind = hip.create_from_numpy(din)
            dwd, dbd = hip.create_from_numpy(np.full_like(wts, 5.0)), hip.create_from_numpy(np.full((f,), 5.0, F32))
            status = lib.bship_conv2d_bwd_thin_f32(xd.ptr, h * w * c, wd.ptr, doutd.ptr, dind.ptr, h * w * c, dwd.ptr,
                                                   dbd.ptr, n, h, w, c, f, kh, kw, pad, 1, 1)
            if (n, h, w, c, f, kh, kw, pad) in THIN_FORWARD_ONLY:
                assert status == -6
                break
            assert status == 0, (n, h, w, c, f, kh, kw, pad, status)
            results.append((dind.get(), dwd.get(), dbd.get()))
        if not results:
            continue
        case = ("thin conv backward", n, h, w, c, f, kh, kw, pad)
        got_din, got_dw, got_db = results[0]
        assert np.max(np.abs(got_din - want_din) / (np.sqrt(f * kh * kw) + np.abs(want_din))) <= 1e-5, case
        assert np.max(np.abs(got_dw - dw) / (np.sqrt(n * oh * ow) + np.abs(dw))) <= 1e-5, case
        assert np.max(np.abs(got_db - db) / (np.sqrt(n * oh * ow) + np.abs(db))) <= 1e-5, case
        for first, second in zip(results[0], results[1]):
            assert_bit_equal(second, first, "second call")
        hip.thin_convolutions = False
        try:
            dind = hip.create_from_numpy(din)
            dwd, dbd = hip.allocate(wts.shape), hip.allocate((f,))
            hip.conv2d_backward_batch(xd, wd, pad, (1, 1), dind, doutd, dwd, dbd)
        finally:
            hip.thin_convolutions = True
        assert np.max(np.abs(got_din - dind.get()) / (np.sqrt(f * kh * kw) + np.abs(want_din))) <= 4e-6, case
        assert np.max(np.abs(got_dw - dwd.get()) / (np.sqrt(n * oh * ow) + np.abs(dw))) <= 4e-6, case
        dind = hip.create_from_numpy(din)
        hip.conv2d_backward_batch(xd, wd, pad, (1, 1), dind, doutd, dwd, dbd)   # through the handler: the same kernels
        assert_bit_equal(dind.get(), got_din, "handler route, input deltas")
        assert_bit_equal(dwd.get(), got_dw, "handler route, weight deltas")
        assert_bit_equal(dbd.get(), got_db, "handler route, bias deltas")
    a = hip.allocate((2, 8, 8, 3))
    for f, kh, kw, c, stride in ((20, 3, 3, 3, 1), (80, 3, 3, 3, 1), (16, 7, 7, 3, 1), (16, 3, 3, 3, 2), (16, 8, 8, 2, 1)):
        assert lib.bship_conv2d_bwd_thin_f32(a.ptr, 192, a.ptr, a.ptr, a.ptr, 192, a.ptr, a.ptr, 2, 8, 8, c, f, kh, kw, 1,
                                             stride, stride) == -6


def test_im2col_col2im_exact(hip, ref):
    # through the C ABI directly: the batched kernels against the oracle's per-image routines
    rng = np.random.RandomState(27)
    lib = hip._lib
    for n, h, w, c, f, kh, kw, pad, stride in CONV_CASES:
        oh, ow = _out_size(h, kh, pad, stride[0]), _out_size(w, kw, pad, stride[1])
        x = rand(rng, (n, h, w, c))
        col = np.zeros((n, oh * ow, kh * kw * c), F32)
        for i in range(n):
            ref._im2col(x[i], kh, kw, pad, stride, col[i])
        xd = hip.create_from_numpy(x)
        cold = hip.allocate(col.shape)
        hip._call(lib.bship_im2col_nhwc_f32(xd.ptr, cold.ptr, n, h, w, c, kh, kw, pad, stride[0], stride[1]))
        assert_bit_equal(cold.get(), col, "im2col")
        cols = rand(rng, col.shape)
        din = rand(rng, x.shape)
        want = din.copy()
        for i in range(n):
            ref._col2im(cols[i], kh, kw, pad, stride, want[i])
        dind = hip.create_from_numpy(din)
        colsd = hip.create_from_numpy(cols)
        hip._call(lib.bship_col2im_nhwc_f32(colsd.ptr, dind.ptr, n, h, w, c, kh, kw, pad,
                                            stride[0], stride[1]))
        assert_bit_equal(dind.get(), want, "col2im")


# Geometries for the LDS-banded kernels: several bands per image, several phases per workgroup
# (enough images that a workgroup walks down more than one group of image rows), strides,
# col rows that are and are not multiples of 4 floats, few images (single-phase bands).
BAND_CASES = [(260, 40, 32, 3, 5, 5, 2, (1, 1)), (210, 40, 256, 3, 3, 3, 1, (2, 2)), (1030, 28, 28, 1, 5, 5, 2, (1, 1)),
              (9, 40, 32, 3, 5, 5, 2, (1, 1)), (130, 17, 12, 8, 3, 3, 0, (1, 1)), (70, 30, 30, 6, 3, 3, 1, (3, 1)),
              (300, 19, 16, 12, 2, 2, 0, (2, 2)), (33, 15, 15, 32, 5, 5, 2, (1, 1)), (40, 11, 9, 5, 3, 3, 1, (1, 1)),
              (20, 10, 10, 3, 3, 3, 1, (1, 1)), (20, 12, 10, 3, 3, 3, 1, (2, 1)),
              # 4 output pixels = kh*kw*c stores: 245 of them (one lane each), 294 (too many: general kernel), 2 groups a row
              (12, 20, 16, 5, 7, 7, 3, (1, 1)), (12, 20, 16, 6, 7, 7, 3, (1, 1)), (50, 9, 8, 3, 2, 3, 1, (1, 2))]


def test_im2col_col2im_banded_exact(hip, ref):
    rng = np.random.RandomState(127)
    lib = hip._lib
    for n, h, w, c, kh, kw, pad, stride in BAND_CASES:
        oh, ow = _out_size(h, kh, pad, stride[0]), _out_size(w, kw, pad, stride[1])
        x = rand(rng, (n, h, w, c))
        col = np.zeros((n, oh * ow, kh * kw * c), F32)
        for i in range(n):
            ref._im2col(x[i], kh, kw, pad, stride, col[i])
        xd = hip.create_from_numpy(x)
        cold = hip.allocate(col.shape)
        hip.fill(cold, 7.0)
        hip._call(lib.bship_im2col_nhwc_f32(xd.ptr, cold.ptr, n, h, w, c, kh, kw, pad, stride[0], stride[1]))
        assert_bit_equal(cold.get(), col, "im2col %r" % ((n, h, w, c, kh, kw, pad, stride),))
        cols = rand(rng, col.shape)
        din = rand(rng, x.shape)
        want = din.copy()
        for i in range(n):
            ref._col2im(cols[i], kh, kw, pad, stride, want[i])
        dind = hip.create_from_numpy(din)
        colsd = hip.create_from_numpy(cols)
        hip._call(lib.bship_col2im_nhwc_f32(colsd.ptr, dind.ptr, n, h, w, c, kh, kw, pad,
                                            stride[0], stride[1]))
        assert_bit_equal(dind.get(), want, "col2im %r" % ((n, h, w, c, kh, kw, pad, stride),))


# Geometries for the streaming col2im kernel (3x3 and 5x5 windows, stride 1, 1 or 3 channels, col rows of at
# least 4.5 KB, one image or more per compute unit): an odd number of col rows (the last phase holds one), padding
# of 0 and of the kernel size minus one, images of a single phase, more images than workgroups by a
# remainder, exactly one image per workgroup, a single col row with lanes left over in the last adding
# wavefront; the last one stays with the banded kernel (col rows too short).
STREAM_CASES = [(300, 9, 32, 3, 5, 4), (257, 6, 88, 1, 5, 0), (530, 12, 32, 3, 5, 2), (260, 7, 100, 1, 5, 2),
                (256, 20, 84, 1, 5, 2), (256, 5, 100, 1, 5, 0), (290, 11, 16, 3, 5, 2), (270, 9, 64, 3, 3, 1),
                (260, 5, 104, 3, 3, 1), (300, 12, 12, 3, 5, 2)]


def test_col2im_streaming_exact(hip, ref):
    rng = np.random.RandomState(128)
    lib = hip._lib
    for n, h, w, c, k, pad in STREAM_CASES:
        oh, ow = _out_size(h, k, pad, 1), _out_size(w, k, pad, 1)
        cols = rand(rng, (n, oh * ow, k * k * c))
        din = rand(rng, (n, h, w, c))
        din[0, 0, :3, 0] = [-0.0, np.inf, np.nan]          # adding nothing must leave -0.0 alone
        cols[0, :2] = 0.0
        cols[0, :2, ::2] = -0.0
        want = din.copy()
        for i in range(n):
            ref._col2im(cols[i], k, k, pad, (1, 1), want[i])
        colsd = hip.create_from_numpy(cols)
        dind = hip.create_from_numpy(din)
        hip._call(lib.bship_col2im_nhwc_f32(colsd.ptr, dind.ptr, n, h, w, c, k, k, pad, 1, 1))
        assert_bit_equal(dind.get(), want, "col2im %r" % ((n, h, w, c, k, pad),))
        # the same images a pitch apart (every image followed by 8 floats that must stay as they are)
        image = h * w * c
        wide = np.full((n, image + 8), 5.0, F32)
        wide[:, :image] = din.reshape(n, image)
        wided = hip.create_from_numpy(wide)
        hip._call(lib.bship_col2im_nhwc_pitched_f32(colsd.ptr, wided.ptr, image + 8, n, h, w, c, k, k, pad, 1, 1))
        got = wided.get()
        assert_bit_equal(got[:, :image].reshape(din.shape), want, "pitched col2im %r" % ((n, h, w, c, k, pad),))
        assert (got[:, image:] == 5.0).all()


def test_im2col_col2im_random_geometries(hip, ref):
    # the banded kernels choose band sizes, LDS rings and phases from the geometry: many random
    # geometries (non-square kernels, strides up to 3, padding up to the kernel size minus one,
    # 1-20 channels, few and many images) against the oracle, bit for bit
    rng = np.random.RandomState(321)
    lib = hip._lib
    cases = []
    while len(cases) < 70:
        kh, kw = rng.randint(1, 6), rng.randint(1, 6)
        pad = rng.randint(0, min(kh, kw))
        sh, sw = rng.randint(1, 4), rng.randint(1, 4)
        h, w = rng.randint(1, 41), rng.randint(1, 41)
        if h + 2 * pad < kh or w + 2 * pad < kw:
            continue
        c = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 20]))
        n = int(rng.choice([1, 2, 3, 9, 17, 40, 130, 600]))
        oh, ow = _out_size(h, kh, pad, sh), _out_size(w, kw, pad, sw)
        if n * oh * ow * kh * kw * c > 6_000_000:
            continue
        cases.append((n, h, w, c, kh, kw, pad, (sh, sw)))
    for n, h, w, c, kh, kw, pad, stride in cases:
        oh, ow = _out_size(h, kh, pad, stride[0]), _out_size(w, kw, pad, stride[1])
        what = "%r" % ((n, h, w, c, kh, kw, pad, stride),)
        x = rand(rng, (n, h, w, c))
        col = np.zeros((n, oh * ow, kh * kw * c), F32)
        for i in range(n):
            ref._im2col(x[i], kh, kw, pad, stride, col[i])
        xd = hip.create_from_numpy(x)
        cold = hip.allocate(col.shape)
        hip._call(lib.bship_im2col_nhwc_f32(xd.ptr, cold.ptr, n, h, w, c, kh, kw, pad, stride[0], stride[1]))
        assert_bit_equal(cold.get(), col, "im2col " + what)
        cols = rand(rng, col.shape)
        din = rand(rng, x.shape)
        want = din.copy()
        for i in range(n):
            ref._col2im(cols[i], kh, kw, pad, stride, want[i])
        dind = hip.create_from_numpy(din)
        colsd = hip.create_from_numpy(cols)
        hip._call(lib.bship_col2im_nhwc_f32(colsd.ptr, dind.ptr, n, h, w, c, kh, kw, pad, stride[0], stride[1]))
        assert_bit_equal(dind.get(), want, "col2im " + what)


def test_many_small_fills_keep_call_order(hip):
    # small fills are collected and enqueued together: overlapping ones, more than fit one launch,
    # fills of unaligned views, and fills followed directly by a reader must all act in call order
    flat = hip.allocate((40000,))
    want = np.zeros((40000,), F32)
    hip.fill(flat, 1.0)
    want[:] = 1.0
    for k in range(40):                               # more fills than one collected launch holds
        lo, hi = 37 * k + 1, 37 * k + 1 + 5 * (k % 7) + 1
        hip.fill(flat[lo:hi], float(k + 2))
        want[lo:hi] = k + 2
    hip.fill(flat[3:30000], 5.0)                      # overlaps many of the above
    want[3:30000] = 5.0
    hip.fill(flat[10:20], 6.0)                        # overlaps the one just before
    want[10:20] = 6.0
    other = hip.allocate((7, 9))
    hip.fill(other, 9.0)
    hip.add_st(1.0, flat, flat)                       # a reader right behind the fills
    want += 1.0
    assert_bit_equal(flat.get(), want, "small fills in call order")
    assert_bit_equal(other.get(), np.full((7, 9), 9.0, F32), "small fill of another array")
    for n in (1 << 19, 1 << 23):                      # a collected and an immediate large fill between small ones
        big = hip.allocate((n,))
        hip.fill(big[5:100], 3.0)
        hip.fill(big, 2.0)
        hip.fill(big[7:9], 4.0)
        hip.fill(big[n - 3:], 8.0)
        wb = np.full((n,), 2.0, F32)
        wb[7:9] = 4.0
        wb[n - 3:] = 8.0
        assert_bit_equal(big.get(), wb, "large fill (%d elements) between small ones" % n)


# ---------------------------------------------------------- views of one buffer
def test_ops_on_unaligned_views(hip, ref):
    # Layer buffers are slices of one flat array (buffers.py:79-83) and may start at any element,
    # so only 4-byte alignment can be assumed.
    rng = np.random.RandomState(28)
    flat = rand(rng, (3 * 5000 + 16,))
    fd = hip.create_from_numpy(flat)
    for off in (1, 2, 3, 5):
        a, b, o = (flat[off:off + 5000], flat[5003 + off:5003 + off + 5000], flat[10012:10012 + 5000])
        want = flat.copy()
        wa, wb, wo = want[off:off + 5000], want[5003 + off:5003 + off + 5000], want[10012:10012 + 5000]
        ref.add_tt(wa, wb, wo)
        ref.sigmoid_deriv(None, wa, wb, wo[:5000])
        fd2 = hip.create_from_numpy(flat)
        da, db, do = fd2[off:off + 5000], fd2[5003 + off:5003 + off + 5000], fd2[10012:10012 + 5000]
        hip.add_tt(da, db, do)
        hip.sigmoid_deriv(None, da, db, do)
        assert_bit_equal(fd2.get(), want, "offset %d" % off)
        # 2-D views with odd row length, row vector add + row/col sums + softmax
        m = flat[off:off + 4800].reshape(40, 120)
        md = fd[off:off + 4800].reshape((40, 120))
        v = flat[9000 + off:9000 + off + 120].reshape(1, 120)
        vd = fd[9000 + off:9000 + off + 120].reshape((1, 120))
        want_o = np.zeros_like(m)
        ref.add_mv(m, v, want_o)
        od = hip.allocate((40, 120))
        hip.add_mv(md, vd, od)
        assert_bit_equal(od.get(), want_o)
        _check_sum(hip, ref, m.copy(), 0, (120,))
        s0 = hip.allocate((120,))
        hip.sum_t(md, 0, s0)
        np.testing.assert_allclose(s0.get(), m.sum(axis=0), rtol=1e-4, atol=1e-5)
        s1 = hip.allocate((40,))
        hip.sum_t(md, 1, s1)
        np.testing.assert_allclose(s1.get(), m.sum(axis=1), rtol=1e-4, atol=1e-5)
        sm = hip.allocate((40, 120))
        hip.softmax_m(md, sm)
        want_sm = np.zeros_like(m)
        ref.softmax_m(m, want_sm)
        np.testing.assert_allclose(sm.get(), want_sm, rtol=1e-5)
    assert_bit_equal(fd.get(), flat, "inputs untouched")


def test_device_array_views_alias(hip):
    base = hip.create_from_numpy(np.arange(2 * 3 * 4, dtype=F32).reshape(2, 3, 4))
    host = np.arange(24, dtype=F32).reshape(2, 3, 4)
    np.testing.assert_array_equal(base[1].get(), host[1])
    np.testing.assert_array_equal(base[-1, 1:].get(), host[-1, 1:])
    np.testing.assert_array_equal(base[0, 2].get(), host[0, 2])
    np.testing.assert_array_equal(base[1, 2, 3].get(), host[1, 2, 3])
    np.testing.assert_array_equal(base.reshape((6, 4))[2:5].get(), host.reshape(6, 4)[2:5])
    np.testing.assert_array_equal(base[:, :, :].get(), host)
    hip.fill(base[1, 1:], -1.0)                 # writes through a view reach the parent
    host[1, 1:] = -1.0
    np.testing.assert_array_equal(base.get(), host)
    flat = base.reshape(24)
    hip.fill(flat[3:5], 9.0)
    host.reshape(24)[3:5] = 9.0
    np.testing.assert_array_equal(base.get(), host)


# ---------------------------------------------------------- environment switches
_SWITCH_SCRIPT = r"""
import hashlib, sys
sys.path.insert(0, %r)
import numpy as np
from brainstorm_amd import HipHandler
h = HipHandler(seed=0)
rng = np.random.RandomState(5)
a = rng.standard_normal((1201, 2049)).astype(np.float32)
b = rng.standard_normal((1201, 2049)).astype(np.float32)
ad, bd, od = h.create_from_numpy(a), h.create_from_numpy(b), h.allocate(a.shape)
h.add_tt(ad, bd, od)
print("ADD", hashlib.sha256(od.get().tobytes()).hexdigest())
h.mult_add_tt(ad, bd, od)
print("MULTADD", hashlib.sha256(od.get().tobytes()).hexdigest())
m = rng.standard_normal((72, 16384)).astype(np.float32)
md, sd = h.create_from_numpy(m), h.allocate(m.shape)
h.softmax_m(md, sd)
print("SOFTMAX", hashlib.sha256(sd.get().tobytes()).hexdigest())
for name, shape in (("SOFTMAX_LONG", (1100, 16384)),):
    m = (rng.standard_normal(shape) * 3).astype(np.float32)
    md, sd = h.create_from_numpy(m), h.allocate(m.shape)
    h.softmax_m(md, sd)
    print(name, hashlib.sha256(sd.get().tobytes()).hexdigest())
cols = rng.standard_normal((260, 12 * 32, 75)).astype(np.float32)
dimg = rng.standard_normal((260, 12, 32, 3)).astype(np.float32)
cd, dd = h.create_from_numpy(cols), h.create_from_numpy(dimg)
h._call(h._lib.bship_col2im_nhwc_f32(cd.ptr, dd.ptr, 260, 12, 32, 3, 5, 5, 2, 1, 1))
print("COL2IM", hashlib.sha256(dd.get().tobytes()).hexdigest())
x = rng.standard_normal((100, 4003)).astype(np.float32)
w = rng.standard_normal((4003, 1001)).astype(np.float32)
out = h.allocate((100, 1001))
xd, wd = h.create_from_numpy(x), h.create_from_numpy(w)
h.dot_mm(xd, wd, out)
exact = x.astype(np.float64) @ w.astype(np.float64)
err = np.abs(out.get() - exact).max()
print("DOT_OK", bool(err <= 1e-5 * np.sqrt(4003) * 10))
# the first call of another thin shape accumulates: with the timed choice of the product's kernel its
# trial runs must not touch the result
x2 = x[:, :3001].copy(); w2 = w[:3001, :997].copy()
acc0 = rng.standard_normal((100, 997)).astype(np.float32) * np.float32(100)
acc = h.create_from_numpy(acc0)
h.dot_add_mm(h.create_from_numpy(x2), h.create_from_numpy(w2), acc)
err = np.abs(acc.get() - (acc0 + x2.astype(np.float64) @ w2.astype(np.float64))).max()
print("DOTADD_OK", bool(err <= 1e-5 * (np.sqrt(3001) * 10 + 400)))
"""


def _run_with(env_extra):
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", _SWITCH_SCRIPT % root], env=dict(os.environ, **env_extra),
                         capture_output=True, text=True, timeout=110)
    assert res.returncode == 0, res.stderr
    return dict(line.split(" ", 1) for line in res.stdout.strip().splitlines()), res.stderr


def test_launch_order_switches_leave_the_results_alone():
    # the order in which tiles and rows are dealt to the XCDs and the kind of store (write-through for
    # outputs of 2^18 to 2^26 elements, as the three here) are a matter of speed only: elementwise results
    # and softmax rows are the same bits with and without them, col2im with either of its kernels for
    # 3-channel images as well; the product's kernel choice may
    # change the summation order, so products are held to the float64 value with either setting
    default, _ = _run_with({})
    plain, _ = _run_with({"BSHIP_EW_RUN_KB": "0", "BSHIP_SM_CHUNK_KB": "0", "BSHIP_STORE_THROUGH_MIN": str(2 ** 40),
                          "BSHIP_COL2IM_STREAM_MIN": "0"})
    for key in ("ADD", "MULTADD", "SOFTMAX", "SOFTMAX_LONG", "COL2IM"):
        assert default[key] == plain[key], key
    for res in (default, plain):
        assert res["DOT_OK"] == "True" and res["DOTADD_OK"] == "True"
    # the optional timed choice of a thin product's kernel: same bars, a line per shape on stderr
    timed, err = _run_with({"BSHIP_GEMM_AUTOTUNE": "2"})
    assert timed["DOT_OK"] == "True" and timed["DOTADD_OK"] == "True"
    assert err.count("bship product plan") >= 2
