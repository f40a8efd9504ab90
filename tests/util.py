"""Comparison helpers shared by the parity tests."""
import numpy as np


def ulp_distance(a, b):
    """Elementwise distance in float32 units in the last place (NaN vs NaN counts as 0)."""
    a = np.ascontiguousarray(a, dtype=np.float32).ravel()
    b = np.ascontiguousarray(b, dtype=np.float32).ravel()
    ai = a.view(np.int32).astype(np.int64)
    bi = b.view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, -(ai & 0x7fffffff), ai)
    bi = np.where(bi < 0, -(bi & 0x7fffffff), bi)
    d = np.abs(ai - bi)
    both_nan = np.isnan(a) & np.isnan(b)
    one_nan = np.isnan(a) ^ np.isnan(b)
    d = np.where(both_nan, 0, d)
    d = np.where(one_nan, np.iinfo(np.int64).max, d)
    return d


def bit_equal(a, b):
    """True if the float32 arrays are identical bit for bit (any NaN equals any NaN)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    if a.shape != b.shape:
        return False
    same = a.view(np.uint32) == b.view(np.uint32)
    return bool(np.all(same | (np.isnan(a) & np.isnan(b))))


def assert_bit_equal(got, want, what=""):
    got = np.ascontiguousarray(got, dtype=np.float32)
    want = np.ascontiguousarray(want, dtype=np.float32)
    assert got.shape == want.shape, "%s: shape %r != %r" % (what, got.shape, want.shape)
    if not bit_equal(got, want):
        ok = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        bad = np.flatnonzero(~ok.ravel())
        i = bad[0]
        raise AssertionError("%s: %d of %d elements differ; first at flat index %d: got %r want %r"
                             % (what, bad.size, got.size, i, got.ravel()[i], want.ravel()[i]))


def assert_max_ulp(got, want, max_ulp, what=""):
    d = ulp_distance(got, want)
    if d.size == 0:
        return
    worst = int(d.max())
    i = int(d.argmax())
    assert worst <= max_ulp, "%s: max ulp distance %d > %d (flat index %d: got %r want %r)" % (
        what, worst, max_ulp, i, np.asarray(got).ravel()[i], np.asarray(want).ravel()[i])


def sum_tolerance(want, terms, axis):
    """Allowed absolute error of a float32 sum: 1e-5 relative to max(|sum|, ||terms||_2).

    The 2-norm of the terms is the natural magnitude of a sum of mixed-sign data (its standard
    deviation for random signs); for same-sign data |sum| >= ||terms||_2 and the bound is the
    plain 1e-5 relative error. Without it a sum of N(0,1) data that happens to land near zero
    could not be compared relatively at all.
    """
    t = np.asarray(terms, dtype=np.float64)
    norm = np.sqrt(np.sum(t * t, axis=axis))
    return 1e-5 * np.maximum(np.abs(np.asarray(want, dtype=np.float64)).reshape(norm.shape), norm)
