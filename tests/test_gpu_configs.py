"""GPU parity of the four network workloads: the same op-trace drivers
(brainstorm_amd/drivers) run on HipHandler and on the float32 CPU oracle with
identical seeded inputs, weights and dropout masks.

What is compared and to which bar:
  * dropout masks and max-pooling argmax: bit-exact;
  * loss: 1e-5 relative;
  * every other buffer (activations, deltas, the flat gradient vector, parameters
    after momentum steps): max |hip - oracle| <= TOL * max |oracle| per buffer. The
    two sides sum the same float32 products in different orders inside the matrix
    products (hipBLASLt tiles vs OpenBLAS), so single elements of a long
    back-propagated chain cannot be held to 1e-5 of their own magnitude; the bar
    is 1e-5 of the buffer's scale for single passes and 1e-4 for gradients that
    went through a 100-step recurrence or through training steps.
  * deltas behind a ReLU: `rel_deriv` is a discrete decision (y > 0). A pre-activation
    within rounding distance of zero can land on different sides on the two handlers
    (about one unit in a million at width 4096 x batch 2048); such a unit's delta then
    differs by its full size. The Highway test therefore compares the backward pass
    from one common forward state (the oracle's activations uploaded to the GPU).
"""
import numpy as np
import pytest

from brainstorm_amd.drivers import configs
from brainstorm_amd.drivers.net import MomentumStepper
from oracle.numpy_ref_handler import NumpyRefHandler
from util import assert_bit_equal

pytestmark = pytest.mark.gpu
F32 = np.float32


def scaled_err(got, want):
    scale = float(np.max(np.abs(want)))
    return float(np.max(np.abs(got.astype(np.float64) - want))) / (scale if scale > 0 else 1.0)


def both(builder, hip, seed_rng, **kw):
    ref = NumpyRefHandler(F32, seed=seed_rng)
    hip.rnd.seed(seed_rng)
    net_h, data = builder(hip, **kw)
    net_r, data_r = builder(ref, **kw)
    for k in data:
        assert np.array_equal(data[k], data_r[k])
    net_h.provide_external_data(data)
    net_r.provide_external_data(data_r)
    return net_h, net_r


def compare_all(net_h, net_r, tol, exact=()):
    worst = {}
    for name in net_r.layers:
        bh, br = net_h.buffers[name], net_r.buffers[name]
        for group in ("outputs", "internals", "output_deltas"):
            for key, want in getattr(br, group).items():
                got = net_h.handler.get_numpy_copy(getattr(bh, group)[key])
                tag = "%s.%s.%s" % (name, group, key)
                if (name, key) in exact:
                    assert_bit_equal(got, want, tag)
                else:
                    worst[tag] = scaled_err(got, want)
    bad = {k: v for k, v in worst.items() if v > tol}
    assert not bad, "buffers over %g: %r" % (tol, bad)
    return max(worst.values())


def device_equal(hip, a, b):
    """True if the device arrays a and b hold the same finite values everywhere (sum |a - b| == 0,
    computed on the device: the deep network's buffers are too large to compare on the host)."""
    n = a.size
    if n == 0:
        return True
    diff = hip._scratch((n,))
    hip.subtract_tt(a.reshape((n,)), b.reshape((n,)), diff)
    hip.abs_t(diff, diff)
    total = hip.allocate(())
    hip.sum_t(diff, None, total)
    return float(total.get()) == 0.0


@pytest.mark.parametrize("fused", [False, True], ids=["primitives", "fused"])
def test_mlp_training_steps(hip, fused):
    # fused=True: dropout, bias + activation, softmax cross entropy and the momentum update through
    # the fused entry points, held to the oracle's primitive sequence at the same bars
    net_h, net_r = both(lambda h, **kw: configs.build_mlp(h, fused=fused and h is hip, **kw), hip, 21)
    net_h.forward_pass(training_pass=True)
    net_r.forward_pass(training_pass=True)
    net_h.backward_pass()
    net_r.backward_pass()
    exact = {("drop1", "mask"), ("drop2", "mask"), ("drop3", "mask")}
    worst = compare_all(net_h, net_r, 1e-5, exact)
    loss_h, loss_r = net_h.get("loss", "outputs", "loss")[0], net_r.get("loss", "outputs", "loss")[0]
    assert abs(loss_h - loss_r) <= 1e-5 * abs(loss_r)
    g_err = scaled_err(net_h.handler.get_numpy_copy(net_h.gradients), net_r.gradients)
    assert g_err <= 1e-5, g_err
    # 20 momentum steps (lr 0.1, momentum 0.9 as in examples/mnist_pi.py:46) with fresh masks
    st_h, st_r = MomentumStepper(0.1, 0.9, fused=fused), MomentumStepper(0.1, 0.9)
    st_h.start(net_h)
    st_r.start(net_r)
    for _ in range(20):
        st_h.run()
        st_r.run()
    for k in ("drop1", "drop2", "drop3"):
        assert_bit_equal(net_h.get(k, "internals", "mask"), net_r.get(k, "internals", "mask"), k)
    p_err = scaled_err(net_h.handler.get_numpy_copy(net_h.parameters), net_r.parameters)
    assert p_err <= 1e-4, p_err
    loss_h, loss_r = net_h.get("loss", "outputs", "loss")[0], net_r.get("loss", "outputs", "loss")[0]
    assert abs(loss_h - loss_r) <= 1e-4 * abs(loss_r)
    print("mlp (fused=%s): worst buffer %.2e, gradient %.2e, parameters after 20 steps %.2e"
          % (fused, worst, g_err, p_err))


@pytest.mark.parametrize("fused", [False, True], ids=["primitives", "fused"])
def test_mlp_recorded_training_steps(hip, fused):
    # the step recorded into a HIP graph and replayed (masks drawn next to the replay, in parallel
    # segments of the same MT19937 stream), against the oracle's eager steps: same masks, same bars
    net_h, net_r = both(lambda h, **kw: configs.build_mlp(h, fused=fused and h is hip, **kw), hip, 27)
    st_h, st_r = MomentumStepper(0.1, 0.9, fused=fused), MomentumStepper(0.1, 0.9)
    st_h.start(net_h)
    st_r.start(net_r)
    st_h.run()                     # one ordinary step first: nothing is set up inside the recording
    st_r.run()
    try:
        for step in range(12):
            st_h.run_recorded()
            st_r.run()
            if step in (0, 5, 11):
                for k in ("drop1", "drop2", "drop3"):
                    assert_bit_equal(net_h.get(k, "internals", "mask"), net_r.get(k, "internals", "mask"),
                                     "%s after replay %d" % (k, step))
                loss_h = net_h.get("loss", "outputs", "loss")[0]
                loss_r = net_r.get("loss", "outputs", "loss")[0]
                assert abs(loss_h - loss_r) <= 1e-4 * abs(loss_r), (step, loss_h, loss_r)
        worst = compare_all(net_h, net_r, 1e-4, {("drop1", "mask"), ("drop2", "mask"), ("drop3", "mask")})
        p_err = scaled_err(hip.get_numpy_copy(net_h.parameters), net_r.parameters)
        assert p_err <= 1e-4, p_err
    finally:
        st_h.release_recorded()
    print("mlp recorded (fused=%s): worst buffer %.2e, parameters after 13 steps %.2e" % (fused, worst, p_err))


def test_lstm_full_size_forward_backward(hip):
    # the full configuration: T=100, batch 100, 205 symbols, 1000 cells, full BPTT
    net_h, net_r = both(configs.build_lstm, hip, 22)
    net_h.forward_pass(training_pass=True)
    net_r.forward_pass(training_pass=True)
    loss_h, loss_r = net_h.get("loss", "outputs", "loss")[0], net_r.get("loss", "outputs", "loss")[0]
    assert abs(loss_h - loss_r) <= 1e-5 * abs(loss_r), (loss_h, loss_r)
    for key in ("Za", "Ib", "Ca", "Cb"):
        err = scaled_err(net_h.get("lstm", "internals", key), net_r.get("lstm", "internals", key))
        assert err <= 1e-5, (key, err)
    assert scaled_err(net_h.get("lstm", "outputs", "default"), net_r.get("lstm", "outputs", "default")) <= 1e-5
    net_h.backward_pass()
    net_r.backward_pass()
    g_h, g_r = net_h.handler.get_numpy_copy(net_h.gradients), net_r.gradients
    worst = 0.0
    for name, (a, b, _) in net_r.parameter_slices().items():
        err = scaled_err(g_h[a:b], g_r[a:b])
        worst = max(worst, err)
        assert err <= 1e-4, (name, err)
    d_err = scaled_err(net_h.get("Input", "output_deltas", "default"), net_r.get("Input", "output_deltas", "default"))
    assert d_err <= 1e-4, d_err
    print("lstm: worst gradient block %.2e, input deltas %.2e" % (worst, d_err))
    # the same network through the fused time-step kernels with one stacked recurrent
    # product per step: held to the oracle at the same bars
    hip.rnd.seed(22)
    net_p, data = configs.build_lstm(hip, fused="packed")
    net_p.provide_external_data(data)
    net_p.forward_pass(training_pass=True)
    net_p.backward_pass()
    loss_p = net_p.get("loss", "outputs", "loss")[0]
    assert abs(loss_p - loss_r) <= 1e-5 * abs(loss_r), (loss_p, loss_r)
    for key in ("Za", "Ib", "Ca", "Cb"):
        err = scaled_err(net_p.get("lstm", "internals", key), net_r.get("lstm", "internals", key))
        assert err <= 1e-5, (key, err)
    g_p = hip.get_numpy_copy(net_p.gradients)
    worst_p = 0.0
    for name, (a, b, _) in net_r.parameter_slices().items():
        err = scaled_err(g_p[a:b], g_r[a:b])
        worst_p = max(worst_p, err)
        assert err <= 1e-4, (name, err)
    d_err = scaled_err(net_p.get("Input", "output_deltas", "default"), net_r.get("Input", "output_deltas", "default"))
    assert d_err <= 1e-4, d_err
    print("lstm, fused steps + stacked recurrent product: worst gradient block %.2e, input deltas %.2e"
          % (worst_p, d_err))
    # the backward recurrent product through the thin-operand kernel and its step kernel
    hip.rnd.seed(22)
    net_t, data = configs.build_lstm(hip, fused="thin")
    net_t.provide_external_data(data)
    net_t.forward_pass(training_pass=True)
    net_t.backward_pass()
    g_t = hip.get_numpy_copy(net_t.gradients)
    worst_t = 0.0
    for name, (a, b, _) in net_r.parameter_slices().items():
        err = scaled_err(g_t[a:b], g_r[a:b])
        worst_t = max(worst_t, err)
        assert err <= 1e-4, (name, err)
    d_err = scaled_err(net_t.get("Input", "output_deltas", "default"), net_r.get("Input", "output_deltas", "default"))
    assert d_err <= 1e-4, d_err
    print("lstm, thin backward product: worst gradient block %.2e, input deltas %.2e" % (worst_t, d_err))
    # and with the whole forward recurrence in one launch (weights resident in LDS, one grid barrier
    # per time step): every internal and the outputs at the oracle's bar
    hip.rnd.seed(22)
    net_s, data = configs.build_lstm(hip, fused="sequence")
    net_s.provide_external_data(data)
    net_s.forward_pass(training_pass=True)
    loss_s = net_s.get("loss", "outputs", "loss")[0]
    assert abs(loss_s - loss_r) <= 1e-5 * abs(loss_r), (loss_s, loss_r)
    worst_s = 0.0
    for key in ("Za", "Zb", "Ia", "Ib", "Fa", "Fb", "Oa", "Ob", "Ca", "Cb"):
        err = scaled_err(net_s.get("lstm", "internals", key), net_r.get("lstm", "internals", key))
        worst_s = max(worst_s, err)
        assert err <= 1e-5, (key, err)
    assert scaled_err(net_s.get("lstm", "outputs", "default"), net_r.get("lstm", "outputs", "default")) <= 1e-5
    print("lstm, whole-sequence forward kernel: worst internal %.2e" % worst_s)

    def whole_pass_against_oracle(label, fused, fusing):
        before = hip.fusing
        hip.set_fusing(fusing)
        try:
            hip.rnd.seed(22)
            net, data = configs.build_lstm(hip, fused=fused)
            net.provide_external_data(data)
            net.forward_pass(training_pass=True)
            net.backward_pass()
            loss = net.get("loss", "outputs", "loss")[0]
            assert abs(loss - loss_r) <= 1e-5 * abs(loss_r), (label, loss, loss_r)
            for key in ("Za", "Zb", "Ia", "Ib", "Fa", "Fb", "Oa", "Ob", "Ca", "Cb"):
                err = scaled_err(net.get("lstm", "internals", key), net_r.get("lstm", "internals", key))
                assert err <= 1e-5, (label, key, err)
            g = hip.get_numpy_copy(net.gradients)
            worst = 0.0
            for name, (a, b, _) in net_r.parameter_slices().items():
                err = scaled_err(g[a:b], g_r[a:b])
                worst = max(worst, err)
                assert err <= 1e-4, (label, name, err)
            err = scaled_err(net.get("Input", "output_deltas", "default"), net_r.get("Input", "output_deltas", "default"))
            assert err <= 1e-4, (label, err)
            print("lstm, %s: worst gradient block %.2e, input deltas %.2e" % (label, worst, err))
        finally:
            hip.set_fusing(before)

    # the layer asking for the per-step kernels itself, products as the reference issues them
    whole_pass_against_oracle("fused time steps, four products per step", "steps", False)
    # an unchanged caller: primitive calls only, through the fusing window ...
    whole_pass_against_oracle("primitive calls through the fusing window", False, True)
    # ... and with the window stacking the four recurrent products of a step into one
    whole_pass_against_oracle("primitive calls, window stacking the recurrent products", False, "stacked")


@pytest.mark.parametrize("fused", [False, True], ids=["primitives", "fused"])
def test_highway_batchnorm_blocks(hip, fused):
    # two blocks at the configuration's width and batch (the oracle's matrix products bound the size);
    # fused=True: BatchNorm, Highway, bias + activation and softmax cross entropy through the fused
    # entry points, against the oracle's primitive sequence
    net_h, net_r = both(lambda h, **kw: configs.build_highway(h, fused=fused and h is hip, **kw), hip, 23,
                        blocks=2)
    net_h.forward_pass(training_pass=True)
    net_r.forward_pass(training_pass=True)
    worst_fwd = 0.0
    for name in net_r.layers:
        for group in ("outputs", "internals"):
            for key, want in getattr(net_r.buffers[name], group).items():
                err = scaled_err(net_h.get(name, group, key), want)
                worst_fwd = max(worst_fwd, err)
                assert err <= 1e-5, (name, group, key, err)
    loss_h, loss_r = net_h.get("loss", "outputs", "loss")[0], net_r.get("loss", "outputs", "loss")[0]
    assert abs(loss_h - loss_r) <= 1e-5 * abs(loss_r)
    # the running statistics (parameters mu, sigma) moved identically
    assert scaled_err(net_h.handler.get_numpy_copy(net_h.parameters), net_r.parameters) <= 1e-6
    # Backward from the SAME forward state: rel_deriv is a discrete decision (y > 0), and with
    # 2 x 8M ReLU units a few pre-activations lie within rounding distance of zero and land on
    # different sides on the two handlers; each such unit changes a whole row of upstream deltas.
    # Giving both sides the oracle's activations removes that (and nothing else) from the comparison.
    for name in net_r.layers:
        for group in ("outputs", "internals"):
            for key, want in getattr(net_r.buffers[name], group).items():
                net_h.handler.set_from_numpy(getattr(net_h.buffers[name], group)[key], want)
    net_h.backward_pass()
    net_r.backward_pass()
    worst = compare_all(net_h, net_r, 1e-5)
    g_h, g_r = net_h.handler.get_numpy_copy(net_h.gradients), net_r.gradients
    for name, (a, b, _) in net_r.parameter_slices().items():
        assert scaled_err(g_h[a:b], g_r[a:b]) <= 1e-5, name
    print("highway (fused=%s): worst forward buffer %.2e, worst backward buffer %.2e" % (fused, worst_fwd, worst))


@pytest.fixture
def trimmed_pool(hip):
    """Gives the pool's cached blocks back to the driver after a test that used tens of gigabytes."""
    yield
    import gc
    gc.collect()
    assert hip._lib.bship_pool_trim() == 0


def test_highway_full_depth(hip, trimmed_pool):
    """The bandwidth-stress configuration at its full depth: 50 x {BatchNorm -> FC_H(rel) || FC_T(sigmoid)
    -> Highway} at width 4096 and batch 2048 (35 GB of buffers, 1.68 G parameters), one training step
    (forward, backward, momentum update) through the primitives and through the fused entry points.
    The oracle cannot run 50 blocks in test time, so depth is held by what does not need it:
      * the first two blocks equal the oracle's two-block network (same seed -> same weights);
      * every BatchNorm output has per-feature mean beta and variance gamma^2 var/(var + eps), at
        every depth (batch_normalization_layer.py:68-105), and every buffer is finite;
      * the fused network equals the primitive one on every buffer, gradient and parameter;
      * the momentum update of the whole unaligned parameter vector equals its closed form
        (steppers.py:104-112) bit for bit.
    """
    blocks, lr, mom = 50, 0.1, 0.9
    hip.rnd.seed(23)
    net_p, data = configs.build_highway(hip, blocks=blocks, quick_init_from_block=2)
    params0 = hip.get_numpy_copy(net_p.parameters)
    net_f, _ = configs.build_highway(hip, blocks=blocks, fused=True, parameters=params0)
    steppers = []
    for net, fused in ((net_p, False), (net_f, True)):
        net.provide_external_data(data)
        st = MomentumStepper(lr, mom, fused=fused)
        st.start(net)
        st.run()
        steppers.append(st)
        assert hip.is_fully_finite(net.full_buffer), "non-finite values (fused=%s)" % fused
    loss = net_p.get("loss", "outputs", "loss")[0]
    assert np.isfinite(loss) and 0.0 < loss < 20.0, loss

    # fused == primitives on everything, compared on the device
    assert device_equal(hip, net_f.full_buffer, net_p.full_buffer), "fused network differs from the primitive one"
    assert device_equal(hip, steppers[1].velocity, steppers[0].velocity)
    assert_bit_equal(net_f.get("loss", "outputs", "loss"), net_p.get("loss", "outputs", "loss"), "loss")
    del net_f, steppers

    # BatchNorm statistics at every depth (gamma = 1, beta = 0 at initialisation)
    eps = 1.0e-5
    for k in range(blocks):
        y = net_p.get("bn%d" % k, "outputs", "default")[0].astype(np.float64)
        s_b = net_p.get("bn%d" % k, "internals", "sigma_b").astype(np.float64)       # sqrt(var + eps)
        assert np.all(s_b > 0.05) and np.all(s_b < 50.0), ("scale drifts", k, s_b.min(), s_b.max())
        assert np.max(np.abs(y.mean(axis=0))) <= 2e-6, (k, np.max(np.abs(y.mean(axis=0))))
        want_var = 1.0 - eps / (s_b * s_b)
        assert np.max(np.abs(y.var(axis=0) - want_var)) <= 2e-5, (k, np.max(np.abs(y.var(axis=0) - want_var)))

    # the first two blocks against the oracle
    ref = NumpyRefHandler(F32, seed=23)
    net_r, data_r = configs.build_highway(ref, blocks=2)
    assert np.array_equal(data_r["default"], data["default"])
    n2 = net_r.parameters.size - (10 * 4096 + 10)                                     # without its output layer
    assert np.array_equal(params0[:n2], net_r.parameters[:n2])
    net_r.provide_external_data(data_r)
    net_r.forward_pass(training_pass=True)
    worst = 0.0
    for name in net_r.layers:
        if name in ("Input", "out", "ce", "loss"):
            continue
        for group in ("outputs", "internals"):
            for key, want in getattr(net_r.buffers[name], group).items():
                err = scaled_err(net_p.get(name, group, key), want)
                worst = max(worst, err)
                assert err <= 1e-5, (name, group, key, err)

    # the update: v = 0 * 0.9 + (-lr (1 - mom)) * g ; p = v + p, in float32, over all 1.68 G parameters
    # (BatchNorm's running statistics mu and sigma are rewritten by the forward pass and have no
    # gradient: they are left out here and covered by the comparisons above)
    step = F32(-(lr * (1 - mom)))
    n, chunk = params0.size, 1 << 27
    statistics = np.zeros(n, bool)
    for name, (a, b, _) in net_p.parameter_slices().items():
        if name.endswith(".mu") or name.endswith(".sigma"):
            statistics[a:b] = True
    for a in range(0, n, chunk):
        b = min(n, a + chunk)
        g = hip.get_numpy_copy(net_p.gradients[a:b])
        assert not g[statistics[a:b]].any()
        want = (F32(mom) * np.zeros(b - a, F32) + step * g) + params0[a:b]
        got = hip.get_numpy_copy(net_p.parameters[a:b])
        keep = ~statistics[a:b]
        assert_bit_equal(got[keep], want[keep], "parameters %d:%d" % (a, b))
    print("highway, 50 blocks: loss %.4f, first two blocks vs oracle %.2e" % (loss, worst))


@pytest.mark.parametrize("fused", [False, True], ids=["primitives", "fused"])
def test_cnn_forward_backward(hip, fused):
    net_h, net_r = both(lambda h, **kw: configs.build_cnn(h, fused=fused and h is hip, **kw), hip, 24)
    net_h.forward_pass(training_pass=True)
    net_r.forward_pass(training_pass=True)
    # Pooling must agree exactly GIVEN the same input: feed the oracle's conv outputs to the GPU pool
    for conv, pool in (("conv1", "pool1"), ("conv2", "pool2")):
        x = net_r.get(conv, "outputs", "default")
        bh = net_h.buffers[pool]
        saved = net_h.handler.get_numpy_copy(bh.inputs["default"])
        net_h.handler.set_from_numpy(bh.inputs["default"], x)
        net_h.layers[pool].forward_pass(bh, True)
        assert_bit_equal(net_h.get(pool, "outputs", "default"), net_r.get(pool, "outputs", "default"), pool)
        assert_bit_equal(net_h.get(pool, "internals", "argmax"), net_r.get(pool, "internals", "argmax"), pool + " argmax")
        net_h.handler.set_from_numpy(bh.inputs["default"], saved)
        net_h.layers[pool].forward_pass(bh, True)
    loss_h, loss_r = net_h.get("loss", "outputs", "loss")[0], net_r.get("loss", "outputs", "loss")[0]
    assert abs(loss_h - loss_r) <= 1e-5 * abs(loss_r)
    for name in ("conv1", "conv2", "fc", "out"):
        assert scaled_err(net_h.get(name, "outputs", "default"), net_r.get(name, "outputs", "default")) <= 1e-5, name
    net_h.backward_pass()
    net_r.backward_pass()
    g_h, g_r = net_h.handler.get_numpy_copy(net_h.gradients), net_r.gradients
    worst = 0.0
    for name, (a, b, _) in net_r.parameter_slices().items():
        err = scaled_err(g_h[a:b], g_r[a:b])
        worst = max(worst, err)
        assert err <= 5e-5, (name, err)
    print("cnn (fused=%s): worst gradient block %.2e" % (fused, worst))


def test_device_resident_inputs(hip):
    # provide_external_data takes arrays of the handler's own type (network.py:399-400): the one-hot
    # input of the LSTM workload is built on the device from the 40 kB of symbol ids with binarize_v
    # instead of uploading the 8 MB one-hot tensor every batch (data_iterators.py:222-231 does it on the host)
    kw = dict(time_steps=100, batch=100, symbols=205, hidden=16)
    net_a, data = configs.build_lstm(hip, **kw)
    net_b, _ = configs.build_lstm(hip, **kw)
    net_a.provide_external_data(data)
    t, b, s = data["default"].shape
    ids = hip.create_from_numpy(data["targets"].reshape(t * b, 1))
    onehot = hip.allocate((t * b, s))
    hip.binarize_v(ids, onehot)
    net_b.provide_external_data({"default": onehot.reshape((t, b, s)), "targets": ids.reshape((t, b, 1))})
    for key in ("default", "targets"):
        assert_bit_equal(net_b.get("Input", "outputs", key), net_a.get("Input", "outputs", key), key)
    net_a.forward_pass(training_pass=True)
    net_b.forward_pass(training_pass=True)
    assert_bit_equal(net_b.get("loss", "outputs", "loss"), net_a.get("loss", "outputs", "loss"), "loss")
