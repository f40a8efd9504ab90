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


def test_mlp_training_steps(hip):
    net_h, net_r = both(configs.build_mlp, hip, 21)
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
    st_h, st_r = MomentumStepper(0.1, 0.9), MomentumStepper(0.1, 0.9)
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
    print("mlp: worst buffer %.2e, gradient %.2e, parameters after 20 steps %.2e" % (worst, g_err, p_err))


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


def test_highway_batchnorm_blocks(hip):
    # two blocks at the configuration's width and batch (the oracle's matrix products bound the size)
    net_h, net_r = both(configs.build_highway, hip, 23, blocks=2)
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
    print("highway: worst forward buffer %.2e, worst backward buffer %.2e" % (worst_fwd, worst))


def test_cnn_forward_backward(hip):
    net_h, net_r = both(configs.build_cnn, hip, 24)
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
    print("cnn: worst gradient block %.2e" % worst)


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
