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


NATIVE_OPS = [
    ("add_tt", lambda h, a, b, o, r, c: h.add_tt(a, b, o)),
    ("subtract_tt in place", lambda h, a, b, o, r, c: h.subtract_tt(a, b, a)),
    ("mult_tt", lambda h, a, b, o, r, c: h.mult_tt(a, b, o)),
    ("divide_tt", lambda h, a, b, o, r, c: h.divide_tt(a, b, o)),
    ("modulo_tt", lambda h, a, b, o, r, c: h.modulo_tt(a, b, o)),
    ("mult_add_tt", lambda h, a, b, o, r, c: h.mult_add_tt(a, b, o)),
    ("add_st", lambda h, a, b, o, r, c: h.add_st(1.5, a, o)),
    ("mult_st in place", lambda h, a, b, o, r, c: h.mult_st(-0.7, a, a)),
    ("mult_add_st", lambda h, a, b, o, r, c: h.mult_add_st(0.3, a, o)),
    ("abs_t", lambda h, a, b, o, r, c: h.abs_t(a, o)),
    ("sign_t", lambda h, a, b, o, r, c: h.sign_t(a, o)),
    ("sqrt_t of abs", lambda h, a, b, o, r, c: (h.abs_t(a, o), h.sqrt_t(o, o))),
    ("sigmoid", lambda h, a, b, o, r, c: h.sigmoid(a, o)),
    ("tanh", lambda h, a, b, o, r, c: h.tanh(a, o)),
    ("log_t of abs", lambda h, a, b, o, r, c: (h.abs_t(a, o), h.log_t(o, o))),
    ("rel in place", lambda h, a, b, o, r, c: h.rel(a, a)),
    ("el", lambda h, a, b, o, r, c: h.el(a, o)),
    ("sigmoid_deriv", lambda h, a, b, o, r, c: h.sigmoid_deriv(None, a, b, o)),
    ("tanh_deriv in place", lambda h, a, b, o, r, c: h.tanh_deriv(None, a, b, b)),
    ("rel_deriv", lambda h, a, b, o, r, c: h.rel_deriv(None, a, b, o)),
    ("el_deriv", lambda h, a, b, o, r, c: h.el_deriv(None, a, b, o)),
    ("clip_t", lambda h, a, b, o, r, c: h.clip_t(a, -0.5, 0.5, o)),
    ("fill", lambda h, a, b, o, r, c: h.fill(o, 2.5)),
    ("copy_to", lambda h, a, b, o, r, c: h.copy_to(a, o)),
    ("copy_to_if", lambda h, a, b, o, r, c: (h.rel(b, b), h.copy_to_if(a, o, b))),
    ("fill_if", lambda h, a, b, o, r, c: (h.rel(b, b), h.fill_if(o, 7.0, b))),
    ("add_into_if", lambda h, a, b, o, r, c: (h.rel(b, b), h.add_into_if(a, o, b))),
    ("add_mv row", lambda h, a, b, o, r, c: h.add_mv(a, r, o)),
    ("subtract_mv col", lambda h, a, b, o, r, c: h.subtract_mv(a, c, o)),
    ("mult_mv with a matrix", lambda h, a, b, o, r, c: h.mult_mv(a, b, o)),
    ("divide_mv row in place", lambda h, a, b, o, r, c: h.divide_mv(a, r, a)),
    ("mult_add_mv col", lambda h, a, b, o, r, c: h.mult_add_mv(a, c, o)),
    ("mult_mv with a column of the hub", lambda h, a, b, o, r, c: h.mult_mv(a, b[:, 4:5], o)),
    ("sum_t axis 0", lambda h, a, b, o, r, c: h.sum_t(a, 0, r)),
    ("sum_t axis 1", lambda h, a, b, o, r, c: h.sum_t(a, 1, c)),
    ("sum_t of all", lambda h, a, b, o, r, c: h.sum_t(a, None, c[0:1].reshape(()))),
    ("softmax_m", lambda h, a, b, o, r, c: h.softmax_m(a, o)),
    ("softmax_m in place", lambda h, a, b, o, r, c: h.softmax_m(a, a)),
    ("binarize_v", lambda h, a, b, o, r, c: (h.fill(c, 3.0), h.binarize_v(c, o))),
    ("binarize_v by a column of the hub", lambda h, a, b, o, r, c: (h.fill(a[:, 2:3], 1.0), h.binarize_v(a[:, 2:3], o))),
    ("index_m_by_v", lambda h, a, b, o, r, c: (h.fill(c, 2.0), h.index_m_by_v(a, c, c))),
    ("index_m_by_v into a column of the hub", lambda h, a, b, o, r, c: (h.fill(c, 4.0), h.index_m_by_v(a, c, o[:, 1:2]))),
]


@pytest.mark.parametrize("rows,width,cuts", [(37, 790, (3, 260, 517, 774)), (5, 40, (1, 8, 15, 22)),
                                             (300, 4100, (4, 1028, 2052, 3076)), (9, 7600, (5, 2530, 5055, 7580)),
                                             # 260 x 1027 = 267 020 elements per slice: above the 2^18 from which
                                             # the kernels store write-through, rows at odd offsets
                                             (260, 4200, (3, 1030, 2057, 3084))],
                         ids=["257 columns at odd offsets", "7 columns", "1024 columns, aligned", "2525 columns",
                              "1027 columns at odd offsets, write-through size"])
@pytest.mark.parametrize("name,call", NATIVE_OPS, ids=[n for n, _ in NATIVE_OPS])
def test_row_pitched_kernels(php, name, call, rows, width, cuts):
    # the kernels that take row-pitched operands as they are: same bits as NumPy on strided views,
    # nothing outside the slice changes, and no dense temporaries are made
    rng = np.random.RandomState(8)
    hub = rng.standard_normal((rows, width)).astype(F32)
    cols = cuts[1] - cuts[0]
    r = rng.uniform(0.5, 2.0, (1, cols)).astype(F32)
    c = rng.uniform(0.5, 2.0, (rows, 1)).astype(F32)
    ref = NumpyRefHandler(F32, seed=3)
    want_hub, want_r, want_c = hub.copy(), r.copy(), c.copy()
    call(ref, want_hub[:, cuts[0]:cuts[1]], want_hub[:, cuts[1]:cuts[2]], want_hub[:, cuts[2]:cuts[3]], want_r, want_c)
    dev_hub, dev_r, dev_c = php.create_from_numpy(hub), php.create_from_numpy(r), php.create_from_numpy(c)
    temporaries = []
    real_scratch = php._scratch
    php._scratch = lambda shape: temporaries.append(shape) or real_scratch(shape)
    try:
        call(php, dev_hub[:, cuts[0]:cuts[1]], dev_hub[:, cuts[1]:cuts[2]], dev_hub[:, cuts[2]:cuts[3]], dev_r, dev_c)
    finally:
        php._scratch = real_scratch
    assert temporaries == [], temporaries
    for got, want, tag in ((dev_hub.get(), want_hub, "hub"), (dev_r.get(), want_r, "row vector"),
                           (dev_c.get(), want_c, "column vector")):
        if name.startswith("sum_t") or name.startswith("softmax_m"):
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5, err_msg=name + ": " + tag)
        elif name in ("sigmoid", "tanh", "log_t of abs"):
            # NumPy's float32 formula and the device result are each within 2 units in the last place
            # of the exact value (test_gpu_parity.py); the dense kernel's bits are checked below
            np.testing.assert_array_max_ulp(got, want, maxulp=4)
        elif name == "el":
            # exp(x) - 1 cancels near 0, so one unit of exp is many units of the result
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=2e-7, err_msg=name + ": " + tag)
        else:
            assert_bit_equal(got, want, name + ": " + tag)
    # the path through dense temporaries gives the same bits
    php.native_pitched = False
    try:
        dev_hub2, dev_r2, dev_c2 = php.create_from_numpy(hub), php.create_from_numpy(r), php.create_from_numpy(c)
        call(php, dev_hub2[:, cuts[0]:cuts[1]], dev_hub2[:, cuts[1]:cuts[2]], dev_hub2[:, cuts[2]:cuts[3]], dev_r2, dev_c2)
    finally:
        php.native_pitched = True
    if not name.startswith("sum_t"):
        assert_bit_equal(dev_hub2.get(), dev_hub.get(), name + ": temporaries vs row-pitched kernels")


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


# ------------------------------------------------------------------ images, masks, broadcast, merge / split
class _NoTemporaries:
    """Fails the test if the handler makes a dense temporary (allocate or _scratch) inside the block."""

    def __init__(self, handler, allowed=0):
        self.h, self.allowed, self.made = handler, allowed, []

    def __enter__(self):
        self.real = (self.h.allocate, self.h._scratch)
        self.h.allocate = lambda shape: self.made.append(shape) or self.real[0](shape)
        self.h._scratch = lambda shape: self.made.append(shape) or self.real[1](shape)
        return self

    def __exit__(self, *exc):
        self.h.allocate, self.h._scratch = self.real
        if exc[0] is None:
            assert len(self.made) <= self.allowed, self.made


def _hub_pair(php, rng, n, width):
    host = rng.standard_normal((n, width)).astype(F32)
    return host, php.create_from_numpy(host)


@pytest.mark.parametrize("n,h,w,c,win,pad,stride", [(5, 9, 9, 4, 3, 0, 2), (3, 8, 8, 3, 2, 1, 2), (4, 7, 6, 8, 3, 1, 1),
                                                    (2, 32, 32, 32, 3, 0, 2)])
def test_pooling_on_image_slices_of_hubs(php, n, h, w, c, win, pad, stride):
    # inputs, outputs, argmax and both delta arrays are feature slices of wider hubs, reshaped to
    # images (buffer_structure.py:232-245): same bits as the oracle, nothing else in the hubs changes
    rng = np.random.RandomState(31)
    ref = NumpyRefHandler(F32, seed=0)
    oh, ow = (h + 2 * pad - win) // stride + 1, (w + 2 * pad - win) // stride + 1
    fi, fo = h * w * c, oh * ow * c
    off_i, off_o = 5, 3
    hubs = {k: _hub_pair(php, rng, n, width) for k, width in
            (("in", fi + 11), ("out", fo + 7), ("arg", fo + 9), ("din", fi + 11), ("dout", fo + 7))}

    def views(which):
        sl = {"in": (off_i, fi, (n, h, w, c)), "din": (off_i, fi, (n, h, w, c)), "out": (off_o, fo, (n, oh, ow, c)),
              "arg": (off_o, fo, (n, oh, ow, c)), "dout": (off_o, fo, (n, oh, ow, c))}
        return {k: hubs[k][which][:, a:a + f].reshape(shape) for k, (a, f, shape) in sl.items()}

    dev, host = views(1), views(0)
    assert all(type(v) is PitchedDeviceArray for v in dev.values())
    # the oracle's C routines take contiguous arrays: run them on copies and put the results back
    x, out, arg = (np.ascontiguousarray(host[k]) for k in ("in", "out", "arg"))
    din, dout = np.ascontiguousarray(host["din"]), np.ascontiguousarray(host["dout"])
    ref.maxpool2d_forward_batch(x, (win, win), out, pad, (stride, stride), arg)
    ref.maxpool2d_backward_batch(x, (win, win), out, pad, (stride, stride), arg, din, dout)
    out_avg = out.copy()
    ref.avgpool2d_forward_batch(x, (win, win), out_avg, pad, (stride, stride))
    din_avg = din.copy()
    ref.avgpool2d_backward_batch(x, (win, win), out_avg, pad, (stride, stride), din_avg, dout)
    with _NoTemporaries(php):
        php.maxpool2d_forward_batch(dev["in"], (win, win), dev["out"], pad, (stride, stride), dev["arg"])
        php.maxpool2d_backward_batch(dev["in"], (win, win), dev["out"], pad, (stride, stride), dev["arg"],
                                     dev["din"], dev["dout"])
    want = {k: hubs[k][0].copy() for k in hubs}
    want["out"][:, off_o:off_o + fo] = out.reshape(n, fo)
    want["arg"][:, off_o:off_o + fo] = arg.reshape(n, fo)
    want["din"][:, off_i:off_i + fi] = din.reshape(n, fi)
    for k in hubs:
        assert_bit_equal(hubs[k][1].get(), want[k], "max pooling, hub %s" % k)
    with _NoTemporaries(php):
        php.avgpool2d_forward_batch(dev["in"], (win, win), dev["out"], pad, (stride, stride))
        php.avgpool2d_backward_batch(dev["in"], (win, win), dev["out"], pad, (stride, stride), dev["din"], dev["dout"])
    want["out"][:, off_o:off_o + fo] = out_avg.reshape(n, fo)
    want["din"][:, off_i:off_i + fi] = din_avg.reshape(n, fi)
    for k in hubs:
        assert_bit_equal(hubs[k][1].get(), want[k], "average pooling, hub %s" % k)


@pytest.mark.parametrize("n,h,w,c,f,k,pad", [(4, 8, 8, 3, 5, 3, 1), (3, 6, 7, 8, 4, 5, 2), (2, 32, 32, 3, 8, 5, 2)])
def test_convolution_on_image_slices_of_hubs(php, n, h, w, c, f, k, pad):
    rng = np.random.RandomState(32)
    ref = NumpyRefHandler(F32, seed=0)
    oh, ow = h + 2 * pad - k + 1, w + 2 * pad - k + 1
    fi, fo = h * w * c, oh * ow * f
    hubs = {key: _hub_pair(php, rng, n, width) for key, width in
            (("in", fi + 6), ("out", fo + 10), ("din", fi + 6), ("dout", fo + 10))}
    wts, bias = rng.standard_normal((f, k, k, c)).astype(F32), rng.standard_normal((f,)).astype(F32)
    dev = {"in": hubs["in"][1][:, 2:2 + fi].reshape((n, h, w, c)), "din": hubs["din"][1][:, 2:2 + fi].reshape((n, h, w, c)),
           "out": hubs["out"][1][:, 7:7 + fo].reshape((n, oh, ow, f)), "dout": hubs["dout"][1][:, 7:7 + fo].reshape((n, oh, ow, f))}
    x = np.ascontiguousarray(hubs["in"][0][:, 2:2 + fi].reshape(n, h, w, c))
    din = np.ascontiguousarray(hubs["din"][0][:, 2:2 + fi].reshape(n, h, w, c))
    dout = np.ascontiguousarray(hubs["dout"][0][:, 7:7 + fo].reshape(n, oh, ow, f))
    out = np.zeros((n, oh, ow, f), F32)
    dw, db = np.zeros_like(wts), np.zeros_like(bias)
    ref.conv2d_forward_batch(x, wts, bias, out, pad, (1, 1))
    ref.conv2d_backward_batch(x, wts, pad, (1, 1), din, dout, dw, db)
    wd, bd = php.create_from_numpy(wts), php.create_from_numpy(bias)
    dwd, dbd = php.allocate(wts.shape), php.allocate(bias.shape)
    php.conv2d_forward_batch(dev["in"], wd, bd, dev["out"], pad, (1, 1))
    php.conv2d_backward_batch(dev["in"], wd, pad, (1, 1), dev["din"], dev["dout"], dwd, dbd)
    want = {key: hubs[key][0].copy() for key in hubs}
    want["out"][:, 7:7 + fo] = out.reshape(n, fo)
    want["din"][:, 2:2 + fi] = din.reshape(n, fi)
    scale = np.sqrt(k * k * c)
    for key in hubs:
        got = hubs[key][1].get()
        assert np.max(np.abs(got - want[key])) <= 1e-5 * scale * max(1.0, np.max(np.abs(want[key]))), key
    untouched = np.ones(fo + 10, bool)
    untouched[7:7 + fo] = False
    assert_bit_equal(hubs["out"][1].get()[:, untouched], hubs["out"][0][:, untouched], "outside the output slice")
    assert_bit_equal(hubs["in"][1].get(), hubs["in"][0], "inputs")
    np.testing.assert_allclose(dwd.get(), dw, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(dbd.get(), db, rtol=1e-4, atol=1e-4)


def test_masks_broadcast_merge_split_on_slices(php):
    rng = np.random.RandomState(33)
    ref = NumpyRefHandler(F32, seed=9)
    php.rnd.seed(9)
    t, b, width = 3, 7, 61
    hub, dhub = rng.standard_normal((t, b, width)).astype(F32), None
    dhub = php.create_from_numpy(hub)
    want = hub.copy()
    # masks: a 3-d feature slice, the same slice seen as images, and again (the look-ahead sees a pattern)
    for _ in range(4):
        with _NoTemporaries(php):
            php.generate_probability_mask(dhub[:, :, 4:28], 0.7)
            php.generate_probability_mask(dhub[:, :, 30:54].reshape((t, b, 2, 3, 4)), 0.4)
        ref.generate_probability_mask(want[:, :, 4:28], 0.7)
        ref.generate_probability_mask(want[:, :, 30:54].reshape(t, b, 2, 3, 4), 0.4)
        assert_bit_equal(dhub.get(), want, "masks in slices")
    # broadcast_t: over the batch axis into a slice, over the last axis, and from a pitched source
    src = rng.standard_normal((t, 1, 24)).astype(F32)
    col = rng.standard_normal((t, b, 1)).astype(F32)
    dsrc, dcol = php.create_from_numpy(src), php.create_from_numpy(col)
    with _NoTemporaries(php):
        php.broadcast_t(dsrc, 1, dhub[:, :, 4:28])
        php.broadcast_t(dcol, 2, dhub[:, :, 30:54])
        php.broadcast_t(dhub[:, :, 57:58], 2, dhub[:, :, 0:3])
    ref.broadcast_t(src, 1, want[:, :, 4:28])
    ref.broadcast_t(col, 2, want[:, :, 30:54])
    ref.broadcast_t(want[:, :, 57:58].copy(), 2, want[:, :, 0:3])
    assert_bit_equal(dhub.get(), want, "broadcast_t into slices")
    # merge_tt and split_add_tt with every operand a slice
    with _NoTemporaries(php):
        php.merge_tt(dhub[:, :, 4:14], dhub[:, :, 30:37], dhub[:, :, 40:57])
        php.split_add_tt(dhub[:, :, 40:57], dhub[:, :, 4:14], dhub[:, :, 20:27])
    ref.merge_tt(want[:, :, 4:14], want[:, :, 30:37], want[:, :, 40:57])
    ref.split_add_tt(want[:, :, 40:57], want[:, :, 4:14], want[:, :, 20:27])
    assert_bit_equal(dhub.get(), want, "merge_tt / split_add_tt on slices")
    # dense operands mixed with slices
    a, bb = rng.standard_normal((t, b, 10)).astype(F32), rng.standard_normal((t, b, 7)).astype(F32)
    da, db = php.create_from_numpy(a), php.create_from_numpy(bb)
    with _NoTemporaries(php):
        php.merge_tt(da, db, dhub[:, :, 40:57])
        php.split_add_tt(dhub[:, :, 40:57], da, db)
    ref.merge_tt(a, bb, want[:, :, 40:57])
    ref.split_add_tt(want[:, :, 40:57], a, bb)
    assert_bit_equal(dhub.get(), want, "merge_tt with dense sources")
    assert_bit_equal(da.get(), a, "split_add_tt into a dense array")
    assert_bit_equal(db.get(), bb, "split_add_tt into a dense array")
