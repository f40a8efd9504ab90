"""GPU: the fused layer-level entry points (LSTM time steps, Highway, BatchNorm, bias +
activation) against the sequence of single
handler operations they replace. Both run on the GPU with the same matrix-product
kernels, so every buffer must agree bit for bit; the unfused sequence itself is
held to the CPU oracle in test_gpu_configs.py."""
import numpy as np
import pytest

from brainstorm_amd.drivers import configs
from util import assert_bit_equal

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(autouse=True)
def single_operations_stay_single(hip):
    # the comparison is against the primitive launches: the fusing window would turn them into the
    # very kernels under test
    before = hip.fusing
    hip.set_fusing(False)
    yield
    hip.set_fusing(before)


def run_lstm(hip, fused, **kw):
    hip.rnd.seed(5)
    net, data = configs.build_lstm(hip, fused=fused, **kw)
    net.provide_external_data(data)
    net.forward_pass(training_pass=True)
    net.backward_pass()
    return net


@pytest.mark.parametrize("shape", [dict(time_steps=7, batch=5, symbols=11, hidden=13),
                                   dict(time_steps=20, batch=33, symbols=50, hidden=257)])
def test_fused_lstm_network_is_bit_identical(hip, shape):
    plain = run_lstm(hip, False, **shape)
    fused = run_lstm(hip, True, **shape)
    assert fused.layers["lstm"]._use_fused()
    for group in ("outputs", "internals", "output_deltas"):
        for key in getattr(plain.buffers["lstm"], group):
            assert_bit_equal(fused.get("lstm", group, key), plain.get("lstm", group, key),
                             "lstm.%s.%s" % (group, key))
    assert_bit_equal(hip.get_numpy_copy(fused.gradients), hip.get_numpy_copy(plain.gradients), "gradients")
    assert_bit_equal(fused.get("Input", "output_deltas", "default"),
                     plain.get("Input", "output_deltas", "default"), "input deltas")


@pytest.mark.parametrize("activation", ["tanh", "sigmoid", "rel", "el", "linear"])
def test_fused_steps_match_single_operations(hip, activation):
    rng = np.random.RandomState(17)
    batch, n = 37, 129                       # odd sizes: views start at unaligned addresses

    def mats(count, scale=1.0):
        flat = hip.create_from_numpy((scale * rng.standard_normal((count, batch, n))).astype(F32))
        return [flat[k] for k in range(count)]

    def vecs(count):
        return [hip.create_from_numpy(rng.standard_normal((1, n)).astype(F32)) for _ in range(count)]

    pi, pf, po = vecs(3)
    bz, bi, bf, bo = [v.reshape((n,)) for v in vecs(4)]
    h = hip

    # ---- forward
    acc = [m for m in mats(4)]                                  # Za, Ia, Fa, Oa as the products left them
    ca_prev = mats(1)[0]
    init = [h.get_numpy_copy(a) for a in acc]
    Za, Ia, Fa, Oa = acc
    Zb, Ib, Fb, Ob, Ca, Cb, y = mats(7)
    h.lstm_forward_step(activation, Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, ca_prev, y,
                        pi, pf, po, bz, bi, bf, bo)
    got = [h.get_numpy_copy(a) for a in (Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, y)]

    for a, v in zip(acc, init):
        h.set_from_numpy(a, v)
    h.add_mv(Za, bz.reshape((1, n)), Za)
    h.act_func[activation](Za, Zb)
    h.mult_add_mv(ca_prev, pi, Ia)
    h.add_mv(Ia, bi.reshape((1, n)), Ia)
    h.sigmoid(Ia, Ib)
    h.mult_add_mv(ca_prev, pf, Fa)
    h.add_mv(Fa, bf.reshape((1, n)), Fa)
    h.sigmoid(Fa, Fb)
    h.mult_tt(Ib, Zb, Ca)
    h.mult_add_tt(Fb, ca_prev, Ca)
    h.mult_add_mv(Ca, po, Oa)
    h.add_mv(Oa, bo.reshape((1, n)), Oa)
    h.sigmoid(Oa, Ob)
    h.act_func[activation](Ca, Cb)
    h.mult_tt(Ob, Cb, y)
    names = "Za Zb Ia Ib Fa Fb Oa Ob Ca Cb y".split()
    for name, g, a in zip(names, got, (Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, y)):
        assert_bit_equal(g, h.get_numpy_copy(a), "forward " + name)

    # ---- backward, on the forward state just computed
    dy, fb_next, dia_next, dfa_next, dca_next = mats(5, 0.5)
    dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb = mats(10)
    dca_init = h.get_numpy_copy(dCa)
    h.lstm_backward_step(activation, dy, Zb, Ib, Fb, Ob, Cb, ca_prev, fb_next, dia_next, dfa_next,
                         dca_next, dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb, pi, pf, po)
    outs = (dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb)
    got = [h.get_numpy_copy(a) for a in outs]

    h.set_from_numpy(dCa, dca_init)
    h.mult_add_mv(dia_next, pi, dCa)
    h.mult_add_mv(dfa_next, pf, dCa)
    h.mult_tt(dy, Cb, dOb)
    h.sigmoid_deriv(Oa, Ob, dOb, dOa)
    h.mult_add_mv(dOa, po, dCa)
    h.mult_tt(dy, Ob, dCb)
    h.act_func_deriv[activation](Ca, Cb, dCb, dCb)
    h.add_tt(dCa, dCb, dCa)
    h.mult_add_tt(dca_next, fb_next, dCa)
    h.mult_tt(dCa, ca_prev, dFb)
    h.sigmoid_deriv(Fa, Fb, dFb, dFa)
    h.mult_tt(dCa, Zb, dIb)
    h.sigmoid_deriv(Ia, Ib, dIb, dIa)
    h.mult_tt(dCa, Ib, dZb)
    h.act_func_deriv[activation](Za, Zb, dZb, dZa)
    names = "dZa dZb dIa dIb dFa dFb dOa dOb dCa dCb".split()
    for name, g, a in zip(names, got, outs):
        assert_bit_equal(g, h.get_numpy_copy(a), "backward " + name)


def test_packed_lstm_network_matches_to_rounding(hip):
    # one stacked recurrent product per step instead of four: same values up to the
    # summation order inside the matrix products
    shape = dict(time_steps=20, batch=33, symbols=50, hidden=257)
    plain = run_lstm(hip, False, **shape)
    packed = run_lstm(hip, "packed", **shape)
    assert packed.layers["lstm"]._stacked_recurrent(*list(packed.buffers["lstm"].parameters.values())[7:11]) is not None
    for group in ("outputs", "internals", "output_deltas"):
        for key in getattr(plain.buffers["lstm"], group):
            want = plain.get("lstm", group, key)
            got = packed.get("lstm", group, key)
            scale = float(np.max(np.abs(want))) or 1.0
            assert float(np.max(np.abs(got - want))) <= 1e-5 * scale, (group, key)
    g_want, g_got = hip.get_numpy_copy(plain.gradients), hip.get_numpy_copy(packed.gradients)
    for name, (a, b, _) in plain.parameter_slices().items():
        scale = float(np.max(np.abs(g_want[a:b]))) or 1.0
        assert float(np.max(np.abs(g_got[a:b] - g_want[a:b]))) <= 1e-5 * scale, name


def test_stack_adjacent(hip):
    flat = hip.allocate((4 * 6 + 5,))
    parts = [flat[k * 6:(k + 1) * 6].reshape((2, 3)) for k in range(4)]
    whole = hip.stack_adjacent(parts)
    assert whole.shape == (8, 3) and whole.ptr == parts[0].ptr
    assert hip.stack_adjacent([parts[0], parts[2]]) is None
    assert hip.stack_adjacent([parts[0], flat[6:11].reshape((5,))]) is None


def test_fused_step_argument_errors(hip):
    a = hip.allocate((4, 8))
    v = hip.allocate((1, 8))
    b = hip.allocate((8,))
    with pytest.raises(ValueError):
        hip.lstm_forward_step("tanh", a, a, a, a, a, a, a, a, a, a, hip.allocate((4, 9)), a,
                              v, v, v, b, b, b, b)
    with pytest.raises(KeyError):
        hip.lstm_forward_step("softplus", a, a, a, a, a, a, a, a, a, a, a, a, v, v, v, b, b, b, b)
    lib = hip._lib
    p = a.ptr
    assert lib.bship_lstm_fwd_step_f32(9, 4, 8, *([p] * 19)) == -4
    assert lib.bship_lstm_fwd_step_f32(1, 4, 8, *([p] * 18 + [None])) == -2
    assert lib.bship_lstm_bwd_step_f32(1, -1, 8, *([p] * 24)) == -3
    assert lib.bship_lstm_bwd_step_f32(1, 0, 8, *([p] * 24)) == 0


# ------------------------------------------------------------------ Highway / BatchNorm / bias
def run_highway(hip, fused, training=True, **kw):
    hip.rnd.seed(6)
    net, data = configs.build_highway(hip, fused=fused, **kw)
    net.provide_external_data(data)
    net.forward_pass(training_pass=training)
    net.backward_pass()
    return net


@pytest.mark.parametrize("shape", [dict(blocks=2, batch=37, width=101), dict(blocks=3, batch=256, width=512)])
@pytest.mark.parametrize("training", [True, False])
def test_fused_highway_batchnorm_network_is_bit_identical(hip, shape, training):
    plain = run_highway(hip, False, training, **shape)
    fused = run_highway(hip, True, training, **shape)
    for name in plain.layers:
        for group in ("outputs", "internals", "output_deltas"):
            for key in getattr(plain.buffers[name], group):
                if training is False and name.startswith("bn") and key == "sigma_b":
                    continue        # not written by an inference pass
                assert_bit_equal(fused.get(name, group, key), plain.get(name, group, key),
                                 "%s.%s.%s" % (name, group, key))
    assert_bit_equal(hip.get_numpy_copy(fused.parameters), hip.get_numpy_copy(plain.parameters), "parameters")
    if training:                    # the backward pass uses the batch deviation of a training pass
        assert_bit_equal(hip.get_numpy_copy(fused.gradients), hip.get_numpy_copy(plain.gradients), "gradients")


@pytest.mark.parametrize("rows,cols", [(1, 5), (37, 129), (300, 64), (2048, 260)])
def test_fused_batchnorm_matches_single_operations(hip, rows, cols):
    from brainstorm_amd.drivers.layers import BatchNorm
    rng = np.random.RandomState(rows * 1000 + cols)
    h = hip

    class Bufs:
        pass

    def make(fused):
        r = np.random.RandomState(99)
        pad = h.allocate((1,))          # shifts what follows off 16-byte alignment in one variant
        b = Bufs()
        flat = h.create_from_numpy(r.standard_normal((6, 1, rows, cols)).astype(F32))
        b.inputs = {"default": flat[0]}
        b.outputs = {"default": flat[1]}
        b.internals = {"sigma_b": h.create_from_numpy(r.standard_normal((cols,)).astype(F32)),
                       "centered": flat[2], "x_hat": flat[3]}
        b.output_deltas = {"default": flat[4]}
        b.input_deltas = {"default": flat[5]}
        vec = lambda lo, hi: h.create_from_numpy(r.uniform(lo, hi, (cols,)).astype(F32))
        from collections import OrderedDict
        b.parameters = OrderedDict([("gamma", vec(0.5, 2)), ("beta", vec(-1, 1)), ("mu", vec(-1, 1)),
                                    ("sigma", vec(0.5, 2))])
        b.gradients = OrderedDict([("gamma", vec(-1, 1)), ("beta", vec(-1, 1))])
        layer = BatchNorm(fused=fused)
        layer.handler = h
        return layer, b, pad

    for training in (True, False):
        results = []
        for fused in (False, True):
            layer, b, _ = make(fused)
            layer.forward_pass(b, training_pass=training)
            if training:
                layer.backward_pass(b)
            got = {}
            for group in ("outputs", "internals", "input_deltas", "parameters", "gradients"):
                for key, arr in getattr(b, group).items():
                    got[group + "." + key] = h.get_numpy_copy(arr)
            results.append(got)
        for key in results[0]:
            assert_bit_equal(results[1][key], results[0][key], "training=%s %s" % (training, key))


@pytest.mark.parametrize("activation", ["tanh", "sigmoid", "rel", "el", "linear"])
@pytest.mark.parametrize("rows,cols", [(3, 7), (65, 1028)])
def test_bias_act_matches_single_operations(hip, activation, rows, cols):
    rng = np.random.RandomState(3)
    x = rng.standard_normal((rows, cols)).astype(F32)
    bias = hip.create_from_numpy(rng.standard_normal((cols,)).astype(F32))
    a = hip.create_from_numpy(x)
    b = hip.create_from_numpy(x)
    hip.bias_act(activation, a, bias, a)
    hip.add_mv(b, bias.reshape((1, cols)), b)
    hip.inplace_act_func[activation](b)
    assert_bit_equal(a.get(), b.get(), activation)


@pytest.mark.parametrize("n", [1, 5, 1024, 4099, 300001])
def test_highway_steps_match_single_operations(hip, n):
    rng = np.random.RandomState(n)
    h = hip
    flat = h.create_from_numpy(rng.standard_normal((8, n)).astype(F32))   # rows start at odd offsets
    H, T, x, dy, dx, dH, dT, y = [flat[k] for k in range(8)]
    init = flat.get()
    h.highway_forward(H, T, x, y)
    h.highway_backward(H, T, x, dy, dx, dH, dT)
    got = flat.get()
    h.set_from_numpy(flat, init)
    tmp = h.zeros(x.shape)
    h.subtract_tt(H, x, out=tmp)
    h.mult_tt(T, tmp, out=tmp)
    h.add_tt(tmp, x, out=y)
    tmp = h.ones(dx.shape)
    h.subtract_tt(tmp, T, out=tmp)
    h.mult_add_tt(tmp, dy, out=dx)
    h.mult_add_tt(T, dy, out=dH)
    h.subtract_tt(H, x, out=tmp)
    h.mult_add_tt(tmp, dy, out=dT)
    assert_bit_equal(got, flat.get(), "highway n=%d" % n)


def test_fused_layer_argument_errors(hip):
    a = hip.allocate((4, 8))
    v = hip.allocate((8,))
    with pytest.raises(ValueError):
        hip.highway_forward(a, a, a, hip.allocate((4, 9)))
    with pytest.raises(ValueError):
        hip.bias_act("rel", a, hip.allocate((7,)), a)
    with pytest.raises(ValueError):
        hip.batchnorm_forward(True, a, v, v, v, v, 0.9, 1e-5, v, a, a, hip.allocate((8, 4)))
    lib = hip._lib
    assert lib.bship_bias_act_f32(7, a.ptr, v.ptr, a.ptr, 4, 8) == -4
    assert lib.bship_highway_fwd_f32(a.ptr, None, a.ptr, a.ptr, 32) == -2
    assert lib.bship_batchnorm_bwd_f32(a.ptr, a.ptr, v.ptr, v.ptr, v.ptr, v.ptr, a.ptr, 0, 8) == -3
    assert lib.bship_batchnorm_fwd_f32(1, a.ptr, v.ptr, v.ptr, v.ptr, v.ptr, 0.9, 1e-5, v.ptr, a.ptr,
                                       a.ptr, a.ptr, 4, 0) == 0


def test_fused_mlp_training_is_bit_identical(hip):
    # dropout (with masks served from the look-ahead queue once the pattern repeats), bias+activation,
    # softmax cross entropy and the momentum update through the fused entry points: same masks, same parameters after 12 steps
    from brainstorm_amd.drivers.net import MomentumStepper
    results = []
    for fused in (False, True):
        hip.rnd.seed(31)
        net, data = configs.build_mlp(hip, fused=fused, batch=37, in_size=50, hidden=129)
        net.provide_external_data(data)
        stepper = MomentumStepper(0.1, 0.9, fused=fused)
        stepper.start(net)
        for _ in range(12):
            stepper.run()
        results.append((hip.get_numpy_copy(net.parameters),
                        [net.get(k, "internals", "mask") for k in ("drop1", "drop2", "drop3")],
                        net.get("loss", "outputs", "loss"), hip.rnd.get_state()))
    (p0, m0, l0, s0), (p1, m1, l1, s1) = results
    assert_bit_equal(p1, p0, "parameters")
    for a, b in zip(m1, m0):
        assert_bit_equal(a, b, "mask")
    assert_bit_equal(l1, l0, "loss")
    assert s0[2] == s1[2] and np.array_equal(s0[1], s1[1])


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_dropout_forward_matches_single_operations(hip, n):
    rng = np.random.RandomState(n)
    x = hip.create_from_numpy(rng.standard_normal((n + 1,)).astype(F32))[1:]    # odd start address
    for keep in (0.8, 0.5):
        hip.rnd.seed(n)
        rs = np.random.RandomState(n)
        for rep in range(5):                       # repeats: later rounds come from the queue
            mask, out = hip.allocate((n,)), hip.allocate((n,))
            hip.dropout_forward(x, keep, 1 / keep, mask, out)
            want_mask = (rs.uniform(size=(n,)) < keep).astype(F32)
            assert_bit_equal(mask.get(), want_mask, "mask n=%d rep %d" % (n, rep))
            want = (x.get() * want_mask) * F32(1 / keep)
            assert_bit_equal(out.get(), want.astype(F32), "out n=%d rep %d" % (n, rep))


@pytest.mark.parametrize("rows,k", [(1, 1), (100, 10), (37, 205), (10000, 205), (513, 4096)])
def test_softmax_ce_fused_matches_single_operations(hip, rows, k):
    # softmax_ce_layer.py:79-89 and 108-112 through the single operations and through the fused entry points
    rng = np.random.RandomState(rows + k)
    x = (rng.standard_normal((rows, k)) * 3).astype(F32)
    tg = rng.randint(0, k, (rows, 1)).astype(F32)
    dl = rng.standard_normal((rows, 1)).astype(F32)
    di = rng.standard_normal((rows, k)).astype(F32)
    up = hip.create_from_numpy
    res = []
    for fused in (False, True):
        xd, td, dld, did = up(x), up(tg), up(dl), up(di)
        probs, loss, t_bin = hip.allocate((rows, k)), hip.allocate((rows, 1)), hip.allocate((rows, k))
        if fused:
            hip.softmax_ce_forward(xd, td, probs, loss)
            hip.softmax_ce_backward(probs, td, dld, t_bin, did)
        else:
            hip.softmax_m(xd, probs)
            hip.fill(loss, 0.)
            hip.index_m_by_v(probs, td, loss)
            hip.clip_t(loss, 1e-6, 1.0, loss)
            hip.log_t(loss, loss)
            hip.mult_st(-1, loss, loss)
            hip.binarize_v(td, t_bin)
            hip.mult_st(-1, t_bin, t_bin)
            hip.add_tt(t_bin, probs, t_bin)
            hip.mult_mv(t_bin, dld, t_bin)
            hip.add_tt(t_bin, did, did)
        res.append([a.get() for a in (probs, loss, t_bin, did)])
    for name, a, b in zip(("probs", "loss", "t_bin", "dinputs"), res[0], res[1]):
        assert_bit_equal(b, a, "%s (%d, %d)" % (name, rows, k))
    # and what it means: loss = -log(p[target]) clipped, dinputs += (p - onehot) * dloss
    p = res[1][0].astype(np.float64)
    want_loss = -np.log(np.clip(p[np.arange(rows), tg[:, 0].astype(int)], 1e-6, 1.0))
    np.testing.assert_allclose(res[1][1][:, 0], want_loss, rtol=2e-6, atol=1e-7)
    onehot = np.zeros((rows, k)); onehot[np.arange(rows), tg[:, 0].astype(int)] = 1
    np.testing.assert_allclose(res[1][3], di + (p - onehot) * dl, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("n", [1, 5, 4099, 2395210])
def test_momentum_update_matches_single_operations(hip, n):
    rng = np.random.RandomState(n)
    g, v, p = (rng.standard_normal((n + 1,)).astype(F32) for _ in range(3))
    res = []
    for fused in (False, True):
        gd, vd, pd = (hip.create_from_numpy(a)[1:] for a in (g, v, p))       # odd start addresses
        for _ in range(3):
            if fused:
                hip.momentum_update(0.9, -0.01, gd, vd, pd)
            else:
                hip.mult_st(0.9, vd, out=vd)
                hip.mult_add_st(-0.01, gd, out=vd)
                hip.add_tt(vd, pd, out=pd)
        res.append((vd.get(), pd.get()))
    assert_bit_equal(res[1][0], res[0][0], "velocity")
    assert_bit_equal(res[1][1], res[0][1], "parameters")
    m, lr = F32(0.9), F32(-0.01)
    vv, pp = v[1:].copy(), p[1:].copy()
    for _ in range(3):
        vv = m * vv
        vv = vv + lr * g[1:]
        pp = vv + pp
    assert_bit_equal(res[1][0], vv, "velocity against NumPy float32")
    assert_bit_equal(res[1][1], pp, "parameters against NumPy float32")
