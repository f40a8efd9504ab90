"""GPU: the op sweep at its full benchmark size (float32 16384x16384, 2^28 elements per tensor).

The device tensors are the ones bench.py measures on: 16 copies of the seeded 4096x4096 inputs, one
after the other in memory. That gives size-independent checks that need no 2^28-element oracle run:
elementwise results must repeat bit for bit from copy to copy and equal the oracle's result on the
4096x4096 inputs; reductions have closed forms in terms of the small inputs; one-hot rows sum to one
and gather back to one; softmax rows sum to one. Everything goes through the C ABI.
"""
import numpy as np
import pytest

import bench
from util import assert_bit_equal, assert_max_ulp, ulp_distance

pytestmark = pytest.mark.gpu
F32 = np.float32
SIZE, BASE = 16384, 4096
REPS = (SIZE * SIZE) // (BASE * BASE)


@pytest.fixture(scope="module")
def sweep(hip):
    t = bench.device_tensors(hip, SIZE, BASE)
    src = bench.host_tensors(BASE)
    yield t, src
    t.clear()


def chunks(hip, arr):
    """The 16 copies as rows of a (16, 4096*4096) NumPy array."""
    return hip.get_numpy_copy(arr).reshape(REPS, BASE * BASE)


def check_repeats(hip, out, want_base, what, max_ulp=0, min_within_2=None):
    got = chunks(hip, out)
    for k in range(1, REPS):
        assert np.array_equal(got[k].view(np.uint32), got[0].view(np.uint32)), "%s: copy %d differs from copy 0" % (what, k)
    if max_ulp == 0:
        assert_bit_equal(got[0], want_base.ravel(), what)
    else:
        assert_max_ulp(got[0], want_base.ravel(), max_ulp, what)
    if min_within_2 is not None:
        within2 = float(np.mean(ulp_distance(got[0], want_base.ravel()) <= 2))
        assert within2 >= min_within_2, "%s: only %.6f of the elements within 2 ulp of the oracle" % (what, within2)


def test_elementwise_ops_at_2p28(hip, ref, sweep):
    t, src = sweep
    a, b, u, y = src["a"], src["b"], src["u"], src["y"]
    out = t["out"]
    cases = [
        ("add_tt", lambda: hip.add_tt(t["a"], t["b"], out), lambda w: ref.add_tt(a, b, w)),
        ("mult_tt", lambda: hip.mult_tt(t["a"], t["b"], out), lambda w: ref.mult_tt(a, b, w)),
        ("divide_tt", lambda: hip.divide_tt(t["a"], t["u"], out), lambda w: ref.divide_tt(a, u, w)),
        ("rel", lambda: hip.rel(t["a"], out), lambda w: ref.rel(a, w)),
        ("clip_t", lambda: hip.clip_t(t["a"], -1.0, 1.0, out), lambda w: ref.clip_t(a, -1.0, 1.0, w)),
        ("sqrt_t", lambda: hip.sqrt_t(t["u"], out), lambda w: ref.sqrt_t(u, w)),
        ("sigmoid_deriv", lambda: hip.sigmoid_deriv(None, t["y"], t["b"], out), lambda w: ref.sigmoid_deriv(None, y, b, w)),
        ("tanh_deriv", lambda: hip.tanh_deriv(None, t["y"], t["b"], out), lambda w: ref.tanh_deriv(None, y, b, w)),
        ("rel_deriv", lambda: hip.rel_deriv(None, t["y"], t["b"], out), lambda w: ref.rel_deriv(None, y, b, w)),
    ]
    for name, run, oracle in cases:
        want = np.zeros((BASE, BASE), F32)
        oracle(want)
        run()
        check_repeats(hip, out, want, name)
    # out += 0.5 * a, twice, starting from zero: exact in float32 order (0 + p) + p
    hip.fill(t["acc"], 0.0)
    hip.mult_add_st(0.5, t["a"], t["acc"])
    hip.mult_add_st(0.5, t["a"], t["acc"])
    want = np.zeros((BASE, BASE), F32)
    ref.mult_add_st(0.5, a, want)
    ref.mult_add_st(0.5, a, want)
    check_repeats(hip, t["acc"], want, "mult_add_st")
    # transcendentals: position independent, and at the bars of the small-size tests (test_gpu_parity.py):
    # tanh within 2 ulp of the float32 oracle everywhere; sigmoid and log_t within 4 ulp everywhere and
    # 99.9 % of the elements within 2 (NumPy's float32 exp/log are up to 3 ulp from the correctly rounded
    # value themselves; the device result is within 1 ulp of it)
    for name, run, oracle, bound in [
            ("tanh", lambda: hip.tanh(t["a"], out), lambda w: ref.tanh(a, w), 2),
            ("sigmoid", lambda: hip.sigmoid(t["a"], out), lambda w: ref.sigmoid(a, w), 4),
            ("log_t", lambda: hip.log_t(t["u"], out), lambda w: ref.log_t(u, w), 4)]:
        want = np.zeros((BASE, BASE), F32)
        oracle(want)
        run()
        check_repeats(hip, out, want, name, max_ulp=bound, min_within_2=0.999)
    # copy and fill
    hip.copy_to(t["a"], out)
    check_repeats(hip, out, a, "copy_to")
    hip.fill(out, 0.5)
    assert np.array_equal(hip.get_numpy_copy(out), np.full((SIZE, SIZE), 0.5, F32))


def test_broadcasts_at_2p28(hip, sweep):
    t, src = sweep
    a64 = src["a"].astype(np.float64)
    row = hip.get_numpy_copy(t["row"])          # (1, 16384)
    col = hip.get_numpy_copy(t["col"])          # (16384, 1)
    big = np.empty((SIZE, SIZE), F32)
    # row r of the big matrix is 4 consecutive rows of one copy of the small one
    tiled = np.tile(src["a"].reshape(BASE // 4, SIZE), (REPS, 1))
    for name, run, want in [
            ("add_mv row", lambda: hip.add_mv(t["a"], t["row"], t["out"]), lambda: tiled + row),
            ("mult_mv row", lambda: hip.mult_mv(t["a"], t["row"], t["out"]), lambda: tiled * row),
            ("add_mv col", lambda: hip.add_mv(t["a"], t["col"], t["out"]), lambda: tiled + col),
            ("mult_mv col", lambda: hip.mult_mv(t["a"], t["col"], t["out"]), lambda: tiled * col)]:
        run()
        got = hip.get_numpy_copy(t["out"])
        assert_bit_equal(got, want().astype(F32), name)
    del big, a64


def test_reductions_at_2p28(hip, sweep):
    t, src = sweep
    a64 = src["a"].astype(np.float64)
    tiled64 = a64.reshape(BASE // 4, SIZE)                   # one copy, as rows of the big matrix
    norm_rows = np.sqrt((tiled64 ** 2).sum(axis=1))
    # axis 1: every copy has the same row sums
    hip.sum_t(t["a"], 1, t["col_out"])
    got = hip.get_numpy_copy(t["col_out"]).reshape(REPS, BASE // 4)
    want = tiled64.sum(axis=1)
    for k in range(REPS):
        assert np.all(np.abs(got[k] - want) <= 1e-5 * np.maximum(np.abs(want), norm_rows)), "axis 1, copy %d" % k
    # axis 0: column sums are 16 times those of one copy
    hip.sum_t(t["a"], 0, t["row_out"])
    got = hip.get_numpy_copy(t["row_out"]).ravel()
    want = REPS * tiled64.sum(axis=0)
    norm = np.sqrt(REPS * (tiled64 ** 2).sum(axis=0))
    assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(np.abs(want), norm))
    # all: 16 times the sum of one copy, and consistent with the axis sums
    hip.sum_t(t["a"], None, t["scalar_out"])
    total = float(hip.get_numpy_copy(t["scalar_out"]))
    want_total = REPS * a64.sum()
    assert abs(total - want_total) <= 1e-5 * max(abs(want_total), np.sqrt(REPS * (a64 ** 2).sum()))
    # a closed form without rounding: ones sum to the element count
    hip.fill(t["out"], 1.0)
    hip.sum_t(t["out"], None, t["scalar_out"])
    assert float(hip.get_numpy_copy(t["scalar_out"])) == float(SIZE * SIZE)
    hip.sum_t(t["out"], 0, t["row_out"])
    assert np.array_equal(hip.get_numpy_copy(t["row_out"]), np.full((1, SIZE), float(SIZE), F32))
    hip.sum_t(t["out"], 1, t["col_out"])
    assert np.array_equal(hip.get_numpy_copy(t["col_out"]), np.full((SIZE, 1), float(SIZE), F32))


def test_softmax_and_labels_at_2p28(hip, ref, sweep):
    t, src = sweep
    hip.softmax_m(t["a"], t["out"])
    got = hip.get_numpy_copy(t["out"])
    rows = got.reshape(REPS, BASE // 4, SIZE)
    for k in range(1, REPS):
        assert np.array_equal(rows[k].view(np.uint32), rows[0].view(np.uint32)), "softmax copy %d" % k
    one = src["a"].reshape(BASE // 4, SIZE)
    want = np.zeros_like(one)
    ref.softmax_m(one, want)
    np.testing.assert_allclose(rows[0], want, rtol=1e-5, atol=1e-37)
    np.testing.assert_allclose(got.astype(np.float64).sum(axis=1), 1.0, rtol=0, atol=1e-5)
    assert float(got.min()) >= 0.0
    # one-hot rows: exactly one 1 per row, at the label; gathering it back gives ones
    labels = hip.get_numpy_copy(t["labels"]).astype(np.int64).ravel()
    hip.binarize_v(t["labels"], t["out"])
    hip.sum_t(t["out"], 1, t["col_out"])
    assert np.array_equal(hip.get_numpy_copy(t["col_out"]), np.ones((SIZE, 1), F32))
    hip.index_m_by_v(t["out"], t["labels"], t["picked"])
    assert np.array_equal(hip.get_numpy_copy(t["picked"]), np.ones((SIZE, 1), F32))
    hot = hip.get_numpy_copy(t["out"])
    assert np.array_equal(np.argmax(hot, axis=1), labels) and float(hot.sum(dtype=np.float64)) == SIZE
    # index_m_by_v on data
    hip.index_m_by_v(t["a"], t["labels"], t["picked"])
    tiled = np.tile(src["a"].reshape(BASE // 4, SIZE), (REPS, 1))
    assert_bit_equal(hip.get_numpy_copy(t["picked"]).ravel(), tiled[np.arange(SIZE), labels], "index_m_by_v")
