"""GPU: error paths through the C ABI and the behaviour of the caching pool.
Every failure is forced from the host (bad arguments, a pool cap); no kernel is
made to fault."""
import ctypes
import os

import numpy as np
import pytest

from brainstorm_amd import _lib

pytestmark = pytest.mark.gpu


def pool_stats(lib):
    a, b, c = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.bship_pool_stats(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)) == 0
    return a.value, b.value, c.value


def test_bad_arguments_return_errors_not_crashes(hip):
    lib = hip._lib
    x = hip.allocate((8,))
    assert lib.bship_binary_f32(99, x.ptr, x.ptr, x.ptr, 8) == -4           # BSHIP_ERR_BAD_OP
    assert b"unknown op" in lib.bship_last_error()
    assert lib.bship_binary_f32(0, None, x.ptr, x.ptr, 8) == -2             # BSHIP_ERR_NULL_POINTER
    assert lib.bship_sum_f32(x.ptr, x.ptr, 2, 4, 3) == -3                   # bad axis
    assert lib.bship_sum_f32(x.ptr, x.ptr, -1, 4, 0) == -3                  # negative dimension
    assert lib.bship_fill_f32(x.ptr + 2, 1.0, 1) == -7                      # not 4-byte aligned
    assert lib.bship_free(x.ptr + 4) == -7                                  # not a pool block
    assert lib.bship_maxpool_fwd_nhwc_f32(x.ptr, x.ptr, x.ptr, 1, 2, 2, 1, 1, 1, 0, 2, 0, 1, 1) == -3
    # row-pitched forms: family / operation codes, pitches and strides are checked before any launch
    pitched = lib.bship_elementwise_pitched_f32
    assert pitched(99, 0, 0.0, 0.0, x.ptr, 4, 1, x.ptr, 4, 1, x.ptr, 4, 2, 4) == -4         # unknown family
    assert pitched(0, 99, 0.0, 0.0, x.ptr, 4, 1, x.ptr, 4, 1, x.ptr, 4, 2, 4) == -4         # unknown operation
    assert pitched(0, 0, 0.0, 0.0, x.ptr, 4, 1, x.ptr, 4, 1, x.ptr, 3, 2, 4) == -3          # pitch below the row length
    assert pitched(0, 0, 0.0, 0.0, x.ptr, 4, 2, x.ptr, 4, 1, x.ptr, 4, 2, 4) == -3          # column stride not 0 or 1
    assert pitched(0, 0, 0.0, 0.0, None, 4, 1, x.ptr, 4, 1, x.ptr, 4, 2, 4) == -2           # missing operand
    assert pitched(0, 0, 0.0, 0.0, x.ptr, 4, 1, x.ptr, 4, 1, x.ptr, 4, 0, 4) == 0           # no rows: nothing to do
    assert lib.bship_sum_pitched_f32(x.ptr, 3, x.ptr, 2, 4, 0) == -3                        # pitch below the row length
    assert lib.bship_softmax_ce_bwd_f32(x.ptr, None, x.ptr, x.ptr, x.ptr, 2, 4) == -2
    assert lib.bship_momentum_update_f32(0.9, -0.1, x.ptr, x.ptr + 2, x.ptr, 8) == -7
    assert lib.bship_init(hip.device) == 0                                   # idempotent
    assert lib.bship_init(hip.device + 1000) != 0                            # another device: refused
    with pytest.raises(_lib.BshipError):
        hip._call(lib.bship_unary_f32(42, x.ptr, x.ptr, 8))
    with pytest.raises(ValueError):
        hip.dot_mm(hip.allocate((2, 3)), hip.allocate((4, 5)), hip.allocate((2, 5)))
    with pytest.raises(ValueError):
        hip.add_mv(hip.allocate((2, 3)), hip.allocate((1, 4)), hip.allocate((2, 3)))
    with pytest.raises(NotImplementedError):
        hip.sum_t(hip.allocate((2, 3, 4)), (0, 1), hip.allocate((4,)))
    # the handler is still usable afterwards
    hip.fill(x, 3.0)
    assert np.array_equal(x.get(), np.full(8, 3.0, np.float32))


def test_zero_sized_operations_do_nothing(hip):
    e = hip.allocate((0, 5))
    v = hip.allocate((1, 5))
    hip.add_tt(e, e, e)
    hip.sigmoid(e, e)
    hip.add_mv(e, v, e)
    hip.softmax_m(e, e)
    hip.sum_t(e, 1, hip.allocate((0,)))
    out = hip.create_from_numpy(np.full((5,), 7.0, np.float32))
    hip.sum_t(e, 0, out)                      # an empty sum is zero
    assert np.array_equal(out.get(), np.zeros(5, np.float32))
    hip.generate_probability_mask(e, 0.5)
    assert hip.is_fully_finite(e) is True
    assert hip.get_numpy_copy(e).shape == (0, 5)


def test_pool_caches_and_reuses_blocks(hip):
    lib = hip._lib
    hip.synchronize()
    in_use0, cached0, allocs0 = pool_stats(lib)
    a = hip.allocate((1000, 1000))                       # 4 MB -> one 4 MiB block
    in_use1, _, allocs1 = pool_stats(lib)
    assert in_use1 - in_use0 == 4 << 20 and allocs1 >= allocs0
    ptr = a.ptr
    view = a[10:20]                                      # a view keeps the block alive
    del a
    assert pool_stats(lib)[0] == in_use1
    del view
    in_use2, cached2, allocs2 = pool_stats(lib)
    assert in_use2 == in_use0 and cached2 >= 4 << 20
    b = hip.allocate((1000, 1000))                       # same size class: the cached block comes back
    assert b.ptr == ptr and pool_stats(lib)[2] == allocs2
    assert not b.get().any()                             # ... zero-filled
    del b
    assert lib.bship_pool_trim() == 0
    assert pool_stats(lib)[1] == 0


def test_pool_limit_raises_memory_error(hip):
    lib = hip._lib
    hip.synchronize()
    in_use = pool_stats(lib)[0]
    os.environ["BSHIP_POOL_LIMIT_BYTES"] = str(in_use + (8 << 20))
    try:
        ok = hip.allocate((1 << 20,))                    # 4 MiB fits
        with pytest.raises(MemoryError):
            hip.allocate((4 << 20,))                     # 16 MiB does not
        del ok
    finally:
        del os.environ["BSHIP_POOL_LIMIT_BYTES"]
    big = hip.allocate((4 << 20,))                       # fine again without the cap
    hip.fill(big, 1.0)
    assert float(big[-1:].get()[0]) == 1.0


def test_small_transfers_behind_a_long_queue(hip):
    # Read-backs and uploads of a few bytes poll pinned memory for at most 1 ms and then wait for the
    # stream the ordinary way. Several milliseconds of queued work in front of them take that second
    # path; the values must be the same. Every kernel here runs to its normal end.
    n = 1 << 28
    a = hip.allocate((n,))
    hip.fill(a, 1.0)
    hip.synchronize()
    for _ in range(12):                               # about 12 x 0.33 ms
        hip.mult_st(1.0001, a, a)
    one = hip.get_numpy_copy(a[12345:12346])          # read-back of one float behind the queue
    want = np.float32(1.0)
    for _ in range(12):
        want = np.float32(want * np.float32(1.0001))
    assert one[0] == want
    for _ in range(12):
        hip.mult_st(1.0001, a, a)
    small = hip.allocate((3,))
    hip.set_from_numpy(small, np.array([1.5, -2.5, 3.5], np.float32))       # upload behind the queue
    assert small.get().tolist() == [1.5, -2.5, 3.5]
    assert hip.is_fully_finite(a)
    del a
