"""GPU: bship_sum_noalloc_f32, the entry point for callers that cannot allocate device
memory. It must give the bits of bship_sum_f32 (same kernels, partial sums in a static
device buffer instead of a pool block), also on a second, smaller call that finds the
first call's partial sums in the buffer, and it must not touch the pool.

Collected last (file name): a failure here must not hide other tests under `pytest -x`.
"""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

from util import assert_bit_equal, sum_tolerance

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def pool_stats(lib):
    a, b, c = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.bship_pool_stats(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)) == 0
    return a.value, b.value, c.value


def both_sums(hip, x, axis):
    """(bship_sum_noalloc_f32, bship_sum_f32) of the host matrix x through the C ABI."""
    lib = hip._lib
    M, N = x.shape
    out_n = N if axis == 0 else M if axis == 1 else 1
    xd = hip.create_from_numpy(x)
    got = hip.allocate((out_n,))
    want = hip.allocate((out_n,))
    hip.fill(got, -7.0)
    hip.synchronize()
    before = pool_stats(lib)
    st = lib.bship_sum_noalloc_f32(xd.ptr, got.ptr, M, N, axis)
    assert st == 0, lib.bship_last_error()
    assert pool_stats(lib) == before, "the pool was used"
    st = lib.bship_sum_f32(xd.ptr, want.ptr, M, N, axis)
    assert st == 0, lib.bship_last_error()
    return got.get(), want.get()


@pytest.mark.parametrize("axis", [0, -1, 1])
def test_two_calls_in_a_row_second_smaller(hip, axis):
    rng = np.random.RandomState(11 + axis)
    # first call: several row bands / chunks, so the partial sums go through the static buffer
    big = rng.standard_normal((3001, 1028)).astype(np.float32)
    small = rng.standard_normal((1100, 260)).astype(np.float32) + 1.0
    for x in (big, small):
        got, want = both_sums(hip, x, axis)
        assert_bit_equal(got, want, "axis %d, shape %r" % (axis, x.shape))
        # and both are the sum (1e-5 of the terms' scale)
        truth = np.sum(x.astype(np.float64), axis=None if axis == -1 else axis)
        tol = sum_tolerance(truth, x, None if axis == -1 else axis)
        assert np.all(np.abs(got.astype(np.float64).reshape(np.shape(truth)) - truth) <= tol)


def test_unaligned_odd_and_degenerate_shapes(hip):
    lib = hip._lib
    rng = np.random.RandomState(5)
    for shape in ((1, 77), (77, 1), (2049, 3), (513, 1001), (4, 8)):
        x = rng.standard_normal(shape).astype(np.float32)
        for axis in (0, 1, -1):
            got, want = both_sums(hip, x, axis)
            assert_bit_equal(got, want, "axis %d, shape %r" % (axis, shape))
    # a view that starts at an odd element of its buffer
    flat = hip.create_from_numpy(rng.standard_normal(1 + 2000 * 516).astype(np.float32))
    a, b = hip.allocate((516,)), hip.allocate((516,))
    assert lib.bship_sum_noalloc_f32(flat.ptr + 4, a.ptr, 2000, 516, 0) == 0
    assert lib.bship_sum_f32(flat.ptr + 4, b.ptr, 2000, 516, 0) == 0
    assert_bit_equal(a.get(), b.get())
    # empty sums are zero; bad arguments are refused like bship_sum_f32's
    hip.fill(a, 3.0)
    assert lib.bship_sum_noalloc_f32(flat.ptr, a.ptr, 0, 516, 0) == 0
    assert np.array_equal(a.get(), np.zeros(516, np.float32))
    assert lib.bship_sum_noalloc_f32(flat.ptr, a.ptr, 4, 4, 2) == -3
    assert lib.bship_sum_noalloc_f32(None, a.ptr, 4, 4, 0) == -2
    assert lib.bship_sum_noalloc_f32(flat.ptr, flat.ptr, 4, 4, 0) == -3


REFUSAL_SCRIPT = r"""
import ctypes, sys
sys.path.insert(0, %r)
from brainstorm_amd import _lib
lib = _lib.load()
assert lib.bship_init(0) == 0
M, N = 8192, 4096
a, out = ctypes.c_void_p(), ctypes.c_void_p()
assert lib.bship_malloc(M * N * 4, ctypes.byref(a)) == 0
assert lib.bship_malloc(N * 4, ctypes.byref(out)) == 0
st = lib.bship_sum_noalloc_f32(a, out, M, N, 0)
msg = lib.bship_last_error().decode()
assert st == -3 and "floats of partial sums" in msg, (st, msg)
assert lib.bship_sum_f32(a, out, M, N, 0) == 0          # the pool-backed entry point takes it
assert lib.bship_sum_noalloc_f32(a, out, M, N, -1) == 0   # and a shape that fits still works
assert lib.bship_sync() == 0
print("refused:", msg)
"""


def test_partial_sums_beyond_the_buffer_are_refused():
    # 64 workgroups per compute unit instead of 3 make (8192, 4096) need 128 row bands = 524288
    # floats of partial sums, twice what the static buffer holds. The launch shape is read from
    # the environment when the library starts, hence a process of its own.
    env = dict(os.environ, BSHIP_COLSUM_BLOCKS_PER_CU="64")
    res = subprocess.run([sys.executable, "-c", REFUSAL_SCRIPT % ROOT], env=env, capture_output=True, text=True,
                         timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "refused:" in res.stdout
