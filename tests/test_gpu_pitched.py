"""GPU: row-pitched views (feature slices of a hub that several layers write side by side,
buffer_structure.py:232-245). NumPy addresses such slices with strides, so the oracle runs the very
same calls on NumPy views; the GPU handler (pitched_views=True) must give the same results in the
slice AND leave the rest of the hub untouched."""
import numpy as np
import pytest

from brainstorm_amd import HipHandler
from brainstorm_amd.device_array import PitchedDeviceArray, PitchedViewError
from brainstorm_amd.drivers.layers import FullyConnected
from oracle.numpy_ref_handler import NumpyRefHandler
from util import assert_bit_equal

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def php():
    return HipHandler(seed=1, pitched_views=True)


def test_default_handler_refuses_pitched_slices(hip):
    a = hip.allocate((4, 6, 10))
    with pytest.raises(NotImplementedError, match="pitched_views"):
        a[:, :, 2:5]
    assert a[:, :, 0:10].shape == (4, 6, 10)          # the full slice is dense


def test_view_algebra(php):
    rng = np.random.RandomState(0)
    x = rng.standard_normal((3, 4, 10)).astype(F32)
    a = php.create_from_numpy(x)
    v = a[:, :, 2:5]
    assert isinstance(v, PitchedDeviceArray) and v.shape == (3, 4, 3) and v.pitch == 10
    with pytest.raises(PitchedViewError):
        v.ptr
    assert_bit_equal(v.get(), x[:, :, 2:5], "slice")
    assert_bit_equal(v[1].get(), x[1, :, 2:5], "time step")
    assert_bit_equal(v[-1, 2].get(), x[-1, 2, 2:5], "one row is dense")
    assert not isinstance(v[-1, 2], PitchedDeviceArray)
    assert_bit_equal(v[1:3, :, 1:2].get(), x[1:3, :, 3:4], "slice of a slice")
    assert_bit_equal(v.reshape((12, 3)).get(), x[:, :, 2:5].reshape(12, 3), "flatten time")
    assert_bit_equal(a.reshape((12, 10))[:, 7:8].get(), x.reshape(12, 10)[:, 7:8], "column")
    with pytest.raises(NotImplementedError):
        v.reshape((4, 9))
    with pytest.raises(NotImplementedError):
        a[:, 1:3, 2:5]                                  # more than one pitch


OPS = [
    ("add_tt", lambda h, a, b, o, r, c, s: h.add_tt(a, b, o)),
    ("mult_add_tt", lambda h, a, b, o, r, c, s: h.mult_add_tt(a, b, o)),
    ("in place", lambda h, a, b, o, r, c, s: h.subtract_tt(a, b, a)),
    ("mult_add_st", lambda h, a, b, o, r, c, s: h.mult_add_st(0.3, a, o)),
    ("fill", lambda h, a, b, o, r, c, s: h.fill(o, 2.5)),
    ("copy_to", lambda h, a, b, o, r, c, s: h.copy_to(a, o)),
    ("tanh_deriv", lambda h, a, b, o, r, c, s: h.tanh_deriv(None, a, b, o)),
    ("rel", lambda h, a, b, o, r, c, s: h.rel(a, o)),
    ("clip_t", lambda h, a, b, o, r, c, s: h.clip_t(a, -0.5, 0.5, o)),
    ("add_mv row", lambda h, a, b, o, r, c, s: h.add_mv(a, r, o)),
    ("mult_add_mv col", lambda h, a, b, o, r, c, s: h.mult_add_mv(a, c, o)),
    ("sum_t axis 0", lambda h, a, b, o, r, c, s: h.sum_t(a, 0, r)),
    ("sum_t axis 1", lambda h, a, b, o, r, c, s: h.sum_t(a, 1, c)),
    ("dot_mm", lambda h, a, b, o, r, c, s: h.dot_mm(a, b, s, transb=True)),
    ("dot_add_mm into a slice", lambda h, a, b, o, r, c, s: h.dot_add_mm(s, b, o)),
    ("generate_probability_mask", lambda h, a, b, o, r, c, s: h.generate_probability_mask(o, 0.5)),
    ("add_into_if", lambda h, a, b, o, r, c, s: h.add_into_if(a, o, b)),
]


@pytest.mark.parametrize("name,call", OPS, ids=[n for n, _ in OPS])
def test_operations_on_pitched_slices(php, name, call):
    rng = np.random.RandomState(5)
    rows, width = 12, 23
    hub = rng.standard_normal((rows, width)).astype(F32)
    extra = {"r": rng.standard_normal((1, 5)).astype(F32), "c": rng.standard_normal((rows, 1)).astype(F32),
             "s": rng.standard_normal((rows, rows)).astype(F32)}
    ref = NumpyRefHandler(F32, seed=3)
    php.rnd.seed(3)
    want_hub = hub.copy()
    want_extra = {k: v.copy() for k, v in extra.items()}
    call(ref, want_hub[:, 2:7], want_hub[:, 9:14], want_hub[:, 15:20], want_extra["r"], want_extra["c"], want_extra["s"])
    dev_hub = php.create_from_numpy(hub)
    dev_extra = {k: php.create_from_numpy(v) for k, v in extra.items()}
    call(php, dev_hub[:, 2:7], dev_hub[:, 9:14], dev_hub[:, 15:20], dev_extra["r"], dev_extra["c"], dev_extra["s"])
    exact = name not in ("sum_t axis 0", "sum_t axis 1", "dot_mm", "dot_add_mm into a slice")
    for got, want, tag in [(dev_hub.get(), want_hub, "hub")] + [(dev_extra[k].get(), want_extra[k], k) for k in extra]:
        if exact:
            assert_bit_equal(got, want, name + ": " + tag)
        else:
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5, err_msg=name + ": " + tag)


def test_matrix_products_take_pitched_operands_as_they_are(php):
    # the pitch of a feature slice is the leading dimension of the product: no dense temporaries
    rng = np.random.RandomState(11)
    rows, width = 9, 40
    hub = rng.standard_normal((rows, width)).astype(F32)
    w = rng.standard_normal((7, 6)).astype(F32)
    dev_hub, dev_w = php.create_from_numpy(hub), php.create_from_numpy(w)
    allocations = []
    real_allocate, real_scratch = php.allocate, php._scratch
    php.allocate = lambda shape: allocations.append(shape) or real_allocate(shape)
    php._scratch = lambda shape: allocations.append(shape) or real_scratch(shape)
    try:
        php.dot_mm(dev_hub[:, 3:9], dev_w, dev_hub[:, 20:27], transb=True)      # (9,6) . (7,6)^T -> (9,7)
        php.dot_add_mm(dev_hub[:, 20:27], dev_w, dev_hub[:, 30:36])             # += (9,7) . (7,6)
    finally:
        php.allocate, php._scratch = real_allocate, real_scratch
    assert allocations == [], allocations
    want = hub.copy()
    want[:, 20:27] = want[:, 3:9] @ w.T
    want[:, 30:36] += want[:, 20:27] @ w
    np.testing.assert_allclose(dev_hub.get(), want, rtol=1e-5, atol=1e-5)
    untouched = np.ones(width, bool)
    untouched[20:27] = untouched[30:36] = False
    assert_bit_equal(dev_hub.get()[:, untouched], hub[:, untouched], "columns outside the written slices")


def test_two_layers_writing_one_hub(php):
    # two fully connected layers put their outputs side by side into one hub, a third reads the whole
    # hub: the multi-source hub of buffer_structure.py:232-245, forward and backward
    rng = np.random.RandomState(7)
    t, b, fin, fa, fb, fout = 3, 5, 6, 4, 7, 3
    x = rng.standard_normal((t, b, fin)).astype(F32)
    params = {"a": (rng.standard_normal((fa, fin)).astype(F32), rng.standard_normal((fa,)).astype(F32)),
              "b": (rng.standard_normal((fb, fin)).astype(F32), rng.standard_normal((fb,)).astype(F32)),
              "c": (rng.standard_normal((fout, fa + fb)).astype(F32), rng.standard_normal((fout,)).astype(F32))}
    dout = rng.standard_normal((t, b, fout)).astype(F32)

    class Bufs:
        pass

    def run(h):
        up = h.create_from_numpy
        xin, hub, hub_d, out = up(x), h.allocate((t, b, fa + fb)), h.allocate((t, b, fa + fb)), h.allocate((t, b, fout))
        din, out_d = h.allocate((t, b, fin)), up(dout)
        layers = {}
        for name, size, act, inp, outp, ind, outd in (
                ("a", fa, "tanh", xin, hub[:, :, :fa], din, hub_d[:, :, :fa]),
                ("b", fb, "rel", xin, hub[:, :, fa:], din, hub_d[:, :, fa:]),
                ("c", fout, "sigmoid", hub, out, hub_d, out_d)):
            layer = FullyConnected(size, act)
            layer.handler = h
            bufs = Bufs()
            bufs.parameters = {"W": up(params[name][0]), "bias": up(params[name][1])}
            bufs.gradients = {"W": h.allocate(params[name][0].shape), "bias": h.allocate(params[name][1].shape)}
            bufs.inputs, bufs.outputs = {"default": inp}, {"default": outp}
            bufs.input_deltas, bufs.output_deltas = {"default": ind}, {"default": outd}
            layers[name] = (layer, bufs)
        for name in "abc":
            layers[name][0].forward_pass(layers[name][1], True)
        for name in "cba":
            layers[name][0].backward_pass(layers[name][1])
        get = h.get_numpy_copy
        return [get(hub), get(out), get(hub_d), get(din)] + [get(layers[n][1].gradients[k]) for n in "abc" for k in ("W", "bias")]

    got, want = run(php), run(NumpyRefHandler(F32, seed=0))
    for g, w in zip(got, want):
        np.testing.assert_allclose(g, w, rtol=1e-4, atol=1e-5)
