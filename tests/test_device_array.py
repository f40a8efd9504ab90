"""CPU-only: DeviceArray view arithmetic (no device memory is touched).

The array contract is the one brainstorm/tests/test_array.py states for its DebugArray (integer
multi-indexing gives the same type with reduced shape, out-of-range raises IndexError) plus what
the buffer manager and the recurrent layers do with arrays: slices, negative indices, reshape,
zero-sized arrays (buffers.py:67-83, lstm_layer.py:106-117)."""
import itertools

import numpy as np
import pytest

from brainstorm_amd.device_array import DeviceArray

BASE_PTR = 0x7f0000001000


def make(shape):
    return DeviceArray(BASE_PTR, tuple(shape), None, None), np.zeros(shape, dtype=np.float32)


def offset_of(view, base):
    return (view.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // 4


def npview(host, key):
    """host[key] as an array view even when every axis is indexed (NumPy would return a scalar)."""
    key = key if isinstance(key, tuple) else (key,)
    if not any(k is Ellipsis for k in key):
        key = key + (Ellipsis,)
    return host[key]


def check_same(dev, host, host_base):
    assert dev.shape == host.shape
    assert dev.size == host.size
    if host.size:
        assert (dev.ptr - BASE_PTR) // 4 == offset_of(host, host_base)


KEYS = [0, 1, -1, slice(None), slice(1, 3), slice(-2, None), slice(0, 0), slice(None, -1),
        (0, 1), (1, 2, 3), (-1, -1), (1, slice(None)), (1, slice(1, 2)), (-1, slice(1, None)),
        (slice(None), slice(None)), (slice(1, 2), slice(None)), (0, 2, slice(1, 3)), (Ellipsis,),
        (1, Ellipsis), (slice(2, 5), Ellipsis)]


@pytest.mark.parametrize("shape", [(5,), (4, 3), (3, 4, 5), (2, 1, 3, 4), (6, 1)])
def test_dense_views_match_numpy(shape):
    dev, host = make(shape)
    for key in KEYS:
        try:
            want = npview(host, key)
        except IndexError:
            with pytest.raises(IndexError):
                dev[key]
            continue
        if want.size > 1 and not want.flags["C_CONTIGUOUS"]:
            with pytest.raises(NotImplementedError):
                dev[key]
            continue
        check_same(dev[key], want, host)


def test_integer_multi_indexing_like_debug_array():
    # brainstorm/tests/test_array.py:16-63
    dev, host = make((2, 3, 4, 5))
    for key in itertools.product(range(2), range(3)):
        check_same(dev[key], npview(host, key), host)
    check_same(dev[1, 2, 3], npview(host, (1, 2, 3)), host)
    assert dev[1, 2, 3, 4].shape == ()
    for bad in (2, (0, 3), (0, 0, 4), (0, 0, 0, 5), -3):
        with pytest.raises(IndexError):
            dev[bad]
    with pytest.raises(IndexError):
        dev[0, 0, 0, 0, 0]


def test_views_of_views_and_reshape_alias():
    dev, host = make((101, 100, 8))
    v, h = dev[:-1], host[:-1]
    check_same(v, h, host)
    check_same(v.reshape((100 * 100, 8)), h.reshape(100 * 100, 8), host)
    check_same(dev[-1], host[-1], host)                      # context slot of a time-major buffer
    check_same(dev[3].reshape(800), host[3].reshape(800), host)
    check_same(dev.reshape(-1, 8)[200:300], host.reshape(-1, 8)[200:300], host)
    check_same(dev.reshape((101, 800))[5:7].reshape((2, 100, 8)), host[5:7], host)
    with pytest.raises(ValueError):
        dev.reshape((7, 7))
    with pytest.raises(ValueError):
        dev.reshape((-1, -1))


def test_row_pitched_views_are_refused():
    dev, _ = make((4, 6))
    for key in [(slice(None), slice(1, 3)), (slice(0, 2), 0), (slice(None), 2)]:
        with pytest.raises(NotImplementedError):
            dev[key]
    dev[:, 0:6]                     # the full feature range of a hub stays dense
    dev[2:3, 1:3]                   # a single row is dense whatever its columns
    with pytest.raises(NotImplementedError):
        dev[::2]


def test_zero_sized_and_zero_dimensional():
    empty = DeviceArray(0, (1, 0, 7), None, None)
    assert empty.size == 0 and empty[0].shape == (0, 7) and empty[:, :, 2:4].shape == (1, 0, 2)
    assert empty.reshape((0,)).shape == (0,)
    scalar = DeviceArray(BASE_PTR, (), None, None)
    assert scalar.size == 1 and scalar.ndim == 0 and scalar.reshape((1, 1)).shape == (1, 1)
    with pytest.raises(IndexError):
        scalar[0]
    dev, host = make((3, 4))
    check_same(dev[1:1], host[1:1], host)
    assert dev.nbytes == 48 and len(dev) == 3


# ------------------------------------------------------------------ randomised against NumPy
from hypothesis import given, settings, strategies as st


class _PitchedHandler:
    pitched_views = True


def _index_strategy(ndim):
    def one(n_axes):
        item = st.one_of(st.integers(-7, 6),
                         st.builds(slice, st.one_of(st.none(), st.integers(-7, 7)),
                                   st.one_of(st.none(), st.integers(-7, 7))))
        return st.lists(item, min_size=0, max_size=n_axes).map(tuple)
    with_ellipsis = st.tuples(one(ndim), one(ndim)).map(lambda ab: ab[0] + (Ellipsis,) + ab[1])
    return st.one_of(one(ndim), with_ellipsis, st.integers(-7, 6))


@settings(max_examples=600, deadline=None)
@given(st.data())
def test_random_index_chains_match_numpy(data):
    """Two index operations in a row on random shapes: NumPy decides what the view is (its
    offset, shape and strides); DeviceArray must return the same dense view, or the same
    row-pitched view when the handler allows those, or refuse exactly the views that are neither
    (and raise IndexError exactly where NumPy does)."""
    shape = tuple(data.draw(st.lists(st.integers(0, 5), min_size=1, max_size=4)))
    pitched = data.draw(st.booleans())
    host_base = np.arange(int(np.prod(shape)), dtype=np.float32).reshape(shape)
    dev = DeviceArray(BASE_PTR, shape, None, _PitchedHandler() if pitched else None)
    host = host_base
    for _ in range(2):
        key = data.draw(_index_strategy(host.ndim))
        try:
            want = npview(host, key)
        except IndexError:
            with pytest.raises(IndexError):
                dev[key]
            return
        dense = want.size == 0 or want.ndim == 0 or want.flags["C_CONTIGUOUS"]
        # a row-pitched view: the longest dense suffix of axes is one run, the axes in front of it
        # advance like the rows of one matrix
        representable = dense
        if not dense and pitched:
            strides = [s // 4 for s in want.strides]
            run, k = 1, want.ndim
            while k > 0 and (want.shape[k - 1] == 1 or strides[k - 1] == run):
                run *= want.shape[k - 1]
                k -= 1
            pitch, below, ok = None, 1, True
            for n, s in zip(reversed(want.shape[:k]), reversed(strides[:k])):
                if n != 1:
                    if pitch is None:
                        ok = ok and s % below == 0
                        pitch = s // below
                    else:
                        ok = ok and s == pitch * below
                below *= n
            representable = ok
        if not representable:
            with pytest.raises(NotImplementedError):
                dev[key]
            return
        got = dev[key]
        assert got.shape == want.shape and got.size == want.size
        if want.size:
            assert (got._address() - BASE_PTR) // 4 == int(want.reshape(-1)[0]) if dense else \
                (got._address() - BASE_PTR) // 4 == int(want[(0,) * want.ndim])
            if dense:
                assert type(got) is DeviceArray
            else:
                assert got.pitch == pitch and got.run == run and got.rows * got.run == got.size
                # element strides agree with NumPy's wherever an axis has more than one entry
                for n, mine, theirs in zip(want.shape, got._strides(), want.strides):
                    assert n == 1 or mine == theirs // 4
        dev, host = got, want
        if type(dev) is not DeviceArray:
            return                                   # chains continue on dense views only here


def test_feature_slice_of_a_hub_reshaped_to_images():
    # buffer_structure.py:232-245: hub[:, :, a:b] of a (T, B, F) hub, reshaped to the layer's own
    # feature shape; the H*W*C elements of one image are one contiguous run
    T, B, F = 3, 4, 50
    host = np.arange(T * B * F, dtype=np.float32).reshape(T, B, F)
    dev = DeviceArray(BASE_PTR, (T, B, F), None, _PitchedHandler())
    sl = dev[:, :, 6:30]
    assert (sl.shape, sl.run, sl.pitch, sl.rows) == ((T, B, 24), 24, F, T * B)
    img = sl.reshape((T, B, 2, 3, 4))
    want = host[:, :, 6:30].reshape(T, B, 2, 3, 4)
    assert (img.shape, img.run, img.pitch, img.rows) == ((T, B, 2, 3, 4), 24, F, T * B)
    assert img._strides() == [s // 4 for s in want.strides]
    flat = img.reshape((T * B, 2, 3, 4))                       # flatten_time
    assert flat.shape == (T * B, 2, 3, 4) and flat.run == 24 and flat.rows == T * B
    assert img.reshape((T * B, 24)).shape == (T * B, 24)
    one = img[1]                                                # a time step: still pitched
    assert one.shape == (B, 2, 3, 4) and one.run == 24 and one.pitch == F
    assert (one._address() - BASE_PTR) // 4 == int(want[1, 0, 0, 0, 0])
    row = img[1, 2]                                             # one image: dense
    assert type(row) is DeviceArray and row.shape == (2, 3, 4)
    assert (row.ptr - BASE_PTR) // 4 == int(want[1, 2, 0, 0, 0])
    with pytest.raises(NotImplementedError):
        img[:, :, :, :, 1:3]                                    # a channel slice of the images: no single pitch
    with pytest.raises(NotImplementedError):
        sl.reshape((T, B, 4, 6))[:, :, 1:3, 1:3]
    for bad in ((T * B * 2, 12), (T, B * 24), (24, T * B)):    # would split or merge runs across the pitch
        with pytest.raises(NotImplementedError):
            sl.reshape(bad)
