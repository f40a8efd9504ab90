"""The thin-operand matrix product (bship_dot_small_tn_f32), bship_transpose_f32 and the LSTM backward
step that consumes its partial products, against NumPy in float64, against the packed step kernel bit
for bit, and through the LSTM network against the oracle's primitive-by-primitive layer.

Bars: a product sums K terms in an order of its own (16 k per matrix-core step, four quarters, then the
caller's partial products), so it is held to float64 at 1e-5 of the largest magnitude, the bar of the
hipBLASLt products (numpy_handler.py:211-229 leaves the order to BLAS as well). The transpose and the
step kernel's elementwise arithmetic are exact.
"""
import numpy as np
import pytest

from brainstorm_amd._lib import BshipError
from brainstorm_amd.drivers import configs
from oracle.numpy_ref_handler import NumpyRefHandler
from util import assert_bit_equal

pytestmark = pytest.mark.gpu
F32 = np.float32


def scaled_err(got, want):
    scale = float(np.max(np.abs(want)))
    return float(np.max(np.abs(got.astype(np.float64) - want))) / (scale if scale > 0 else 1.0)


@pytest.mark.parametrize("rows,cols,pitch", [(1, 1, 1), (5, 37, 128), (100, 1000, 128), (33, 64, 40), (128, 31, 128),
                                             (1000, 4000, 1000)])
def test_transpose_is_exact_and_leaves_the_padding_alone(hip, rows, cols, pitch):
    rng = np.random.RandomState(rows + cols)
    a = rng.standard_normal((rows, cols)).astype(F32)
    out = hip.create_from_numpy(np.full((cols, pitch), 7.0, F32))
    hip.transpose(hip.create_from_numpy(a), out)
    got = hip.get_numpy_copy(out)
    assert_bit_equal(got[:, :rows], a.T, "transpose")
    assert np.all(got[:, rows:] == 7.0)


SHAPES = [  # M, K, N, splits
    (1, 1, 1, 1), (5, 37, 50, 1), (16, 16, 32, 1), (17, 100, 33, 2), (64, 64, 64, 1), (65, 130, 31, 3),
    (100, 1000, 4000, 1), (100, 4000, 1000, 4), (128, 256, 96, 8), (77, 500, 1, 1), (48, 15, 200, 4)]


@pytest.mark.parametrize("m,k,n,splits", SHAPES)
def test_dot_small_tn_matches_float64(hip, m, k, n, splits):
    rng = np.random.RandomState(m * 7 + k * 3 + n)
    a = rng.standard_normal((m, k)).astype(F32)
    b = rng.standard_normal((k, n)).astype(F32)
    a_t = hip.zeros((k, 128))
    hip.transpose(hip.create_from_numpy(a), a_t)
    out = hip.create_from_numpy(np.full((m, n) if splits == 1 else (splits, m, n), np.nan, F32))
    hip.dot_small_tn(a_t, m, hip.create_from_numpy(b), out, splits)
    got = hip.get_numpy_copy(out)
    assert np.all(np.isfinite(got)), "an element of the output was not written"
    if splits > 1:
        # the slabs are the products of whole 16-blocks of k, in order
        per = -(-(-(-k // 16)) // splits) * 16
        for s in range(splits):
            lo, hi = min(s * per, k), min((s + 1) * per, k)
            want = a[:, lo:hi].astype(np.float64) @ b[lo:hi].astype(np.float64)
            assert np.max(np.abs(got[s] - want)) <= 1e-5 * max(1.0, np.max(np.abs(want))), s
        got = got.astype(np.float64).sum(axis=0)
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert scaled_err(got, want) <= 1e-5


def test_dot_small_tn_and_transpose_on_pitched_operands(hip):
    # b, c and the transpose's source as column slices of wider matrices (row pitches above the widths),
    # straight through the C ABI
    rng = np.random.RandomState(9)
    m, k, n, ldb, ldc, lda = 70, 203, 45, 61, 50, 230
    a_wide = rng.standard_normal((m, lda)).astype(F32)
    b_wide = rng.standard_normal((k, ldb)).astype(F32)
    c_wide = np.full((2, m, ldc), -3.0, F32)
    da, db, dc = hip.create_from_numpy(a_wide), hip.create_from_numpy(b_wide), hip.create_from_numpy(c_wide)
    a_t = hip.zeros((k, 128))
    lib = hip._lib
    hip._call(lib.bship_transpose_f32(da.ptr + 4 * 11, m, k, lda, a_t.ptr, 128))            # a = a_wide[:, 11:11+k]
    assert_bit_equal(hip.get_numpy_copy(a_t)[:, :m], a_wide[:, 11:11 + k].T, "pitched transpose")
    hip._call(lib.bship_dot_small_tn_f32(a_t.ptr, db.ptr + 4 * 7, dc.ptr + 4 * 2, m, n, k, ldb, ldc, 2, m * ldc))
    got = hip.get_numpy_copy(dc)
    assert np.all(got[:, :, :2] == -3.0) and np.all(got[:, :, 2 + n:] == -3.0), "columns outside the slice were written"
    want = a_wide[:, 11:11 + k].astype(np.float64) @ b_wide[:, 7:7 + n].astype(np.float64)
    assert scaled_err(got[:, :, 2:2 + n].astype(np.float64).sum(axis=0), want) <= 1e-5


def test_dot_small_tn_with_nothing_to_add_writes_zeros(hip):
    out = hip.create_from_numpy(np.full((2, 5, 9), 3.0, F32))
    lib = hip._lib
    hip._call(lib.bship_dot_small_tn_f32(0, 0, out.ptr, 5, 7, 0, 7, 9, 2, 45))      # K = 0: no operands are read
    got = hip.get_numpy_copy(out)
    assert np.all(got[:, :, :7] == 0.0) and np.all(got[:, :, 7:] == 3.0)


def test_dot_small_tn_is_deterministic_and_rejects_what_it_does_not_take(hip):
    rng = np.random.RandomState(3)
    a = rng.standard_normal((100, 4000)).astype(F32)
    b = hip.create_from_numpy(rng.standard_normal((4000, 1000)).astype(F32))
    a_t = hip.zeros((4000, 128))
    hip.transpose(hip.create_from_numpy(a), a_t)
    outs = []
    for _ in range(3):
        out = hip.zeros((4, 100, 1000))
        hip.dot_small_tn(a_t, 100, b, out, 4)
        outs.append(hip.get_numpy_copy(out))
    assert_bit_equal(outs[1], outs[0], "second run")
    assert_bit_equal(outs[2], outs[0], "third run")
    with pytest.raises(ValueError):
        hip.dot_small_tn(hip.zeros((4000, 128)), 129, b, hip.zeros((129, 1000)))
    lib = hip._lib
    wide = hip.zeros((200, 8))
    assert lib.bship_dot_small_tn_f32(a_t.ptr, b.ptr, wide.ptr, 200, 8, 16, 8, 8, 1, 0) != 0     # more than 128 rows
    assert lib.bship_dot_small_tn_f32(a_t.ptr + 4, b.ptr, wide.ptr, 8, 8, 16, 8, 8, 1, 0) != 0   # operand not 16-byte aligned
    assert lib.bship_dot_small_tn_f32(a_t.ptr, b.ptr, wide.ptr, 8, 8, 16, 4, 8, 1, 0) != 0       # pitch below the width
    assert_bit_equal(hip.get_numpy_copy(wide), np.zeros((200, 8), F32), "refused calls write nothing")


@pytest.mark.parametrize("act", ["tanh", "sigmoid", "rel", "linear", "el"])
@pytest.mark.parametrize("batch,n,parts", [(5, 12, 1), (33, 100, 3), (128, 64, 8), (100, 250, 4)])
def test_thin_backward_step_equals_packed_step(hip, act, batch, n, parts):
    # same inputs through lstm_backward_step_packed (dy holding the finished product) and through the thin
    # step (the product cut into `parts` slabs whose ascending sum is that product exactly): every output
    # bit for bit, and the transposed operand equals packed_out transposed
    rng = np.random.RandomState(batch + n + parts)
    slabs = np.zeros((parts, batch, n), F32)
    slabs[0] = rng.standard_normal((batch, n)).astype(F32)
    for p in range(1, parts):                      # powers of two times the first slab's magnitude: sums are exact
        slabs[p] = np.ldexp(np.round(rng.standard_normal((batch, n)) * 4), -3).astype(F32)
    total = slabs[0].copy()
    for p in range(1, parts):
        total = (total + slabs[p]).astype(F32)
    mats_in = [rng.standard_normal((batch, n)).astype(F32) for _ in range(11)]       # deltas, Zb..dCa_next
    mats_in[1:6] = [rng.uniform(0.05, 0.95, (batch, n)).astype(F32) for _ in range(5)]
    vecs = [rng.standard_normal(n).astype(F32) for _ in range(3)]
    dca0 = rng.standard_normal((batch, n)).astype(F32)

    def run(thin):
        dev_in = [hip.create_from_numpy(m) for m in mats_in]
        outs = [hip.zeros((batch, n)) for _ in range(10)]
        hip.set_from_numpy(outs[8], dca0)                                           # dCa is read and written
        pv = [hip.create_from_numpy(v) for v in vecs]
        if thin:
            dy = hip.zeros((batch, n))
            packed_t = hip.zeros((4 * n, 128))
            dy_parts = hip.create_from_numpy(slabs if parts > 1 else slabs[0])
            hip.lstm_backward_step_thin(act, dev_in[0], dy_parts, dy, packed_t, *dev_in[1:], *outs, *pv)
            packed = hip.get_numpy_copy(packed_t)
            assert not packed[:, batch:].any()
            packed = np.ascontiguousarray(packed[:, :batch].T)
        else:
            dy = hip.create_from_numpy(total)
            packed_d = hip.zeros((batch, 4 * n))
            hip.lstm_backward_step_packed(act, dev_in[0], dy, packed_d, *dev_in[1:], *outs, *pv)
            packed = hip.get_numpy_copy(packed_d)
        return [hip.get_numpy_copy(dy), packed] + [hip.get_numpy_copy(o) for o in outs]

    for k, (got, want) in enumerate(zip(run(True), run(False))):
        assert_bit_equal(got, want, "output %d" % k)


@pytest.mark.parametrize("shape", [(3, 5, 11, 12), (5, 33, 20, 100), (4, 64, 13, 256), (3, 65, 13, 36), (6, 100, 30, 200),
                                   (3, 128, 7, 64)], ids=lambda s: "T%d_B%d_S%d_H%d" % s)
def test_lstm_thin_backward_against_oracle_layer(hip, shape):
    steps, batch, symbols, hidden = shape
    kw = dict(time_steps=steps, batch=batch, symbols=symbols, hidden=hidden)
    ref = NumpyRefHandler(F32, seed=3)
    net_r, data = configs.build_lstm(ref, **kw)
    net_r.provide_external_data(data)
    net_r.forward_pass(training_pass=True)
    net_r.backward_pass()
    hip.rnd.seed(3)
    net_h, data_h = configs.build_lstm(hip, fused="thin", **kw)
    net_h.provide_external_data(data_h)
    calls = []
    real = hip.dot_small_tn
    hip.dot_small_tn = lambda *a: calls.append(1) or real(*a)
    try:
        net_h.forward_pass(training_pass=True)
        net_h.backward_pass()
    finally:
        del hip.dot_small_tn
    assert len(calls) == steps, "the backward pass did not go through dot_small_tn"
    g_h = hip.get_numpy_copy(net_h.gradients)
    for name, (a, b, _) in net_r.parameter_slices().items():
        assert scaled_err(g_h[a:b], net_r.gradients[a:b]) <= 1e-4, name
    for key in ("dZa", "dIa", "dFa", "dOa", "dCa"):
        assert scaled_err(net_h.get("lstm", "internals", key), net_r.get("lstm", "internals", key)) <= 1e-4, key
    assert scaled_err(net_h.get("Input", "output_deltas", "default"),
                      net_r.get("Input", "output_deltas", "default")) <= 1e-4
