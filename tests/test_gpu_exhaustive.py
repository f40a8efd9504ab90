"""Every float32 bit pattern through tanh, sigmoid and log_t.

The kernels evaluate in float64 and round once; the statement checked here is that for ALL 2^32
inputs the result is within 1 ulp of the float64 evaluation (NumPy, float64) rounded to float32,
that all but a vanishing fraction are exactly that value, and that NaNs, infinities and the sign of
zero agree. About 15 s per function with 8 host threads.
"""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F32 = np.float32
CHUNK = 1 << 25


def _sigmoid64(x):
    e = np.exp(-np.abs(x))
    return np.where(x >= 0, 1.0 / (1.0 + e), e / (1.0 + e))


def _ordered(a):
    i = a.view(np.int32).astype(np.int64)
    return np.where(i < 0, -(i & 0x7fffffff), i)


def _compare(got, x, exact_f64):
    with np.errstate(all="ignore"):
        truth = exact_f64(x.astype(np.float64)).astype(F32)
    nan_g, nan_t = np.isnan(got), np.isnan(truth)
    d = np.abs(_ordered(got) - _ordered(truth))
    d[nan_g & nan_t] = 0
    d[nan_g ^ nan_t] = 1 << 40
    wrong_zero = (got == 0) & (truth == 0) & (np.signbit(got) != np.signbit(truth))
    i = int(d.argmax())
    return int(d[i]), int(np.count_nonzero(d)), int(np.count_nonzero(wrong_zero)), (x[i], got[i], truth[i])


@pytest.mark.parametrize("op,exact_f64", [("tanh", np.tanh), ("sigmoid", _sigmoid64), ("log_t", np.log)])
def test_all_float32_inputs(op, exact_f64):
    from brainstorm_amd import HipHandler
    hip = HipHandler(seed=0)
    xd, yd = hip.allocate((CHUNK,)), hip.allocate((CHUNK,))
    worst, differing, wrong_zeros, example = 0, 0, 0, None
    with ThreadPoolExecutor(8) as pool:
        pending = []
        for c in range((1 << 32) // CHUNK):
            x = (np.arange(CHUNK, dtype=np.uint64) + c * CHUNK).astype(np.uint32).view(F32)
            hip.set_from_numpy(xd, x)
            getattr(hip, op)(xd, yd)
            pending.append(pool.submit(_compare, hip.get_numpy_copy(yd), x, exact_f64))
            if len(pending) == 8:
                for p in pending:
                    w, n, z, e = p.result()
                    if w > worst:
                        worst, example = w, e
                    differing += n
                    wrong_zeros += z
                pending = []
        for p in pending:
            w, n, z, e = p.result()
            if w > worst:
                worst, example = w, e
            differing += n
            wrong_zeros += z
    print("%s: max %d ulp from the rounded float64 evaluation, %d of 2^32 inputs differ from it, "
          "%d zeros of the wrong sign" % (op, worst, differing, wrong_zeros))
    assert worst <= 1, "%s: %d ulp at x=%r (got %r, float64 evaluation %r)" % ((op, worst) + tuple(example))
    assert differing <= 1000, "%s: %d inputs are not the rounded float64 evaluation" % (op, differing)
    assert wrong_zeros == 0


def _exact_compare(got, x, op):
    from oracle.numpy_ref_handler import NumpyRefHandler
    ref = NumpyRefHandler(F32, seed=0)
    want = np.zeros_like(x)
    with np.errstate(all="ignore"):
        getattr(ref, op)(x, want)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    bad = np.flatnonzero(~same)
    return int(bad.size), (None if bad.size == 0 else (x[bad[0]], got[bad[0]], want[bad[0]]))


@pytest.mark.parametrize("op", ["abs_t", "sign_t", "sqrt_t", "rel"])
def test_all_float32_inputs_bit_exact(op):
    """The operations that have one right answer in float32: the same bits as the oracle for every input."""
    from brainstorm_amd import HipHandler
    hip = HipHandler(seed=0)
    xd, yd = hip.allocate((CHUNK,)), hip.allocate((CHUNK,))
    differing, example = 0, None
    with ThreadPoolExecutor(8) as pool:
        pending = []
        for c in range((1 << 32) // CHUNK):
            x = (np.arange(CHUNK, dtype=np.uint64) + c * CHUNK).astype(np.uint32).view(F32)
            hip.set_from_numpy(xd, x)
            getattr(hip, op)(xd, yd)
            pending.append(pool.submit(_exact_compare, hip.get_numpy_copy(yd), x, op))
            if len(pending) == 8 or c == (1 << 32) // CHUNK - 1:
                for p in pending:
                    n, e = p.result()
                    differing += n
                    example = example or e
                pending = []
    assert differing == 0, "%s: %d of 2^32 inputs differ, e.g. x=%r got %r want %r" % ((op, differing) + tuple(example))
