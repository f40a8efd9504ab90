"""CPU-only: the op-trace drivers (brainstorm_amd/drivers) run on the float64
oracle and are checked the way brainstorm checks its layers
(brainstorm/tests/test_layers.py:389-418): analytic gradients and input deltas
against central finite differences of the loss, plus closed forms where the
reference's sequence is deliberately not the true gradient (Dropout) and the
"backward passes add to deltas" rule (test_layers.py:490-531)."""
import numpy as np
import pytest

from brainstorm_amd.drivers.layers import (BatchNorm, Convolution2D, Dropout, FullyConnected, Highway,
                                           Input, Loss, Lstm, Pooling2D, SoftmaxCE)
from brainstorm_amd.drivers.net import MomentumStepper, Net
from oracle.numpy_ref_handler import NumpyRefHandler

F64 = np.float64


def make_net(middle, in_shape, classes, seed=0, time_steps=2, batch=3):
    """Input -> middle layers -> FullyConnected(classes, linear) -> SoftmaxCE -> Loss, float64."""
    h = NumpyRefHandler(F64, seed=11)
    rng = np.random.RandomState(seed)
    layers = [("Input", Input({"default": in_shape, "targets": (1,)}), {})] + middle
    last = middle[-1][0] if middle else "Input"
    layers += [("out", FullyConnected(classes, "linear"), {"default": last + ".default"}),
               ("ce", SoftmaxCE(), {"default": "out.default", "targets": "Input.targets"}),
               ("loss", Loss(), {"default": "ce.loss"})]
    net = Net(h, layers)
    data = {"default": rng.standard_normal((time_steps, batch) + tuple(in_shape)),
            "targets": rng.randint(0, classes, (time_steps, batch, 1)).astype(F64)}
    net.provide_external_data(data)
    params = rng.standard_normal(net.parameter_count()) * 0.5
    for name, (a, b, _) in net.parameter_slices().items():
        if name.endswith(("gamma", "sigma")):
            params[a:b] = 1.0 + 0.1 * rng.standard_normal(b - a)
    net.set_parameters(params)
    return net, data, params


def loss_of(net, data, params):
    net.set_parameters(params)
    net.provide_external_data(data)
    net.forward_pass(training_pass=True)
    return float(net.get("loss", "outputs", "loss")[0])


def check_gradients(net, data, params, skip=(), eps=1e-6, rtol=1e-4, atol=1e-7):
    net.set_parameters(params)
    net.provide_external_data(data)
    net.forward_pass(training_pass=True)
    net.backward_pass()
    grads = net.handler.get_numpy_copy(net.gradients)
    dinput = net.get("Input", "output_deltas", "default")
    for name, (a, b, _) in net.parameter_slices().items():
        if name.split(".")[-1] in skip:
            continue
        idx = np.unique(np.linspace(a, b - 1, min(b - a, 12)).astype(int))
        for i in idx:
            p = params.copy()
            p[i] += eps
            lp = loss_of(net, data, p)
            p[i] -= 2 * eps
            lm = loss_of(net, data, p)
            np.testing.assert_allclose(grads[i], (lp - lm) / (2 * eps), rtol=rtol, atol=atol,
                                       err_msg="gradient of %s[%d]" % (name, i - a))
    flat = data["default"].ravel()
    for i in np.unique(np.linspace(0, flat.size - 1, 10).astype(int)):
        d = {k: v.copy() for k, v in data.items()}
        d["default"].ravel()[i] += eps
        lp = loss_of(net, d, params)
        d["default"].ravel()[i] -= 2 * eps
        lm = loss_of(net, d, params)
        np.testing.assert_allclose(dinput.ravel()[i], (lp - lm) / (2 * eps), rtol=rtol, atol=atol,
                                   err_msg="input delta %d" % i)


@pytest.mark.parametrize("activation", ["rel", "tanh", "sigmoid", "linear", "el"])
def test_fully_connected_and_softmax_ce(activation):
    net, data, params = make_net([("fc", FullyConnected(5, activation), {"default": "Input.default"})], (4,), 3)
    check_gradients(net, data, params)


def test_softmax_ce_closed_form():
    # d loss / d logits = (softmax - onehot) / batch
    net, data, params = make_net([], (4,), 3, time_steps=1, batch=5)
    net.forward_pass(training_pass=True)
    net.backward_pass()
    probs = net.get("ce", "outputs", "predictions")
    np.testing.assert_allclose(probs.sum(axis=-1), 1.0, rtol=1e-12)
    onehot = np.eye(3)[data["targets"].astype(int)[..., 0]]
    np.testing.assert_allclose(net.get("out", "output_deltas", "default"), (probs - onehot) / 5, rtol=1e-10)
    want_loss = -np.log(np.clip(np.sum(probs * onehot, axis=-1), 1e-6, 1.0)).sum() / 5
    np.testing.assert_allclose(net.get("loss", "outputs", "loss")[0], want_loss, rtol=1e-12)


@pytest.mark.parametrize("activation", ["tanh", "sigmoid"])
def test_lstm_full_bptt(activation):
    net, data, params = make_net([("lstm", Lstm(4, activation), {"default": "Input.default"})], (3,), 3,
                                 time_steps=5, batch=2)
    check_gradients(net, data, params, rtol=2e-4)


def test_lstm_forward_ignores_garbage_in_internals():
    # test_layers.py:421-487: results must not depend on what the buffers held before
    net, data, params = make_net([("lstm", Lstm(4), {"default": "Input.default"})], (3,), 3, time_steps=4, batch=2)
    net.forward_pass(training_pass=True)
    net.backward_pass()
    want_loss = net.get("loss", "outputs", "loss").copy()
    want_grad = net.handler.get_numpy_copy(net.gradients)
    rng = np.random.RandomState(1)
    for name in ("Za", "Zb", "Ib", "Ca", "Cb", "dZa", "dCa", "dIa"):
        buf = net.buffers["lstm"].internals[name]
        buf[:] = rng.standard_normal(buf.shape)
    net.buffers["lstm"].outputs["default"][:] = 7.0
    net.forward_pass(training_pass=True)
    net.backward_pass()
    np.testing.assert_allclose(net.get("loss", "outputs", "loss"), want_loss, rtol=1e-12)
    np.testing.assert_allclose(net.handler.get_numpy_copy(net.gradients), want_grad, rtol=1e-10, atol=1e-14)


def test_batch_norm():
    net, data, params = make_net([("bn", BatchNorm(), {"default": "Input.default"})], (5,), 3, time_steps=2, batch=6)
    # the forward pass moves the running statistics mu/sigma; they carry no gradient
    check_gradients(net, data, params, skip=("mu", "sigma"), rtol=2e-4)
    net.set_parameters(params)
    net.provide_external_data(data)
    net.forward_pass(training_pass=True)
    x = data["default"].reshape(12, 5)
    out = net.get("bn", "outputs", "default").reshape(12, 5)
    sl = net.parameter_slices()
    gamma, beta = params[slice(*sl["bn.gamma"][:2])], params[slice(*sl["bn.beta"][:2])]
    want = (x - x.mean(axis=0)) / np.sqrt(x.var(axis=0) + 1e-5) * gamma + beta
    np.testing.assert_allclose(out, want, rtol=1e-10)
    new = net.handler.get_numpy_copy(net.parameters)
    mu0, sg0 = params[slice(*sl["bn.mu"][:2])], params[slice(*sl["bn.sigma"][:2])]
    np.testing.assert_allclose(new[slice(*sl["bn.mu"][:2])], 0.9 * mu0 + 0.1 * (-x.mean(axis=0)), rtol=1e-12)
    np.testing.assert_allclose(new[slice(*sl["bn.sigma"][:2])], 0.9 * sg0 + 0.1 * np.sqrt(x.var(axis=0) + 1e-5),
                               rtol=1e-12)


def test_highway_block():
    middle = [("H", FullyConnected(4, "rel"), {"default": "Input.default"}),
              ("T", FullyConnected(4, "sigmoid"), {"default": "Input.default"}),
              ("hw", Highway(), {"H": "H.default", "T": "T.default", "x": "Input.default"})]
    net, data, params = make_net(middle, (4,), 3)
    check_gradients(net, data, params)       # three sinks share Input's delta buffer: they must ADD
    net.set_parameters(params)
    net.provide_external_data(data)
    net.forward_pass(training_pass=True)
    H, T = net.get("H", "outputs", "default"), net.get("T", "outputs", "default")
    np.testing.assert_allclose(net.get("hw", "outputs", "default"), T * H + (1 - T) * data["default"], rtol=1e-12)


@pytest.mark.parametrize("pool", ["max", "avg"])
def test_convolution_and_pooling(pool):
    middle = [("conv", Convolution2D(3, (3, 3), padding=1, activation="tanh"), {"default": "Input.default"}),
              ("pool", Pooling2D(pool, (3, 3), stride=(2, 2)), {"default": "conv.default"})]
    net, data, params = make_net(middle, (6, 5, 2), 3, time_steps=1, batch=2)
    check_gradients(net, data, params, rtol=2e-4)


def test_dropout_is_the_reference_sequence():
    h = NumpyRefHandler(F64, seed=3)
    net = Net(h, [("Input", Input({"default": (6,)}), {}), ("drop", Dropout(0.25), {"default": "Input.default"})])
    x = np.random.RandomState(0).standard_normal((2, 4, 6))
    net.provide_external_data({"default": x})
    h.rnd.seed(3)
    net.forward_pass(training_pass=True)
    mask = (np.random.RandomState(3).uniform(size=x.shape) < 0.75).astype(F64)
    np.testing.assert_array_equal(net.get("drop", "internals", "mask"), mask)
    np.testing.assert_allclose(net.get("drop", "outputs", "default"), x * mask / 0.75, rtol=1e-15)
    net.backward_pass()
    net.buffers["drop"].output_deltas["default"][:] = 2.0
    net.buffers["drop"].input_deltas["default"][:] = 1.0
    net.layers["drop"].backward_pass(net.buffers["drop"])
    # adds dy*mask WITHOUT the 1/(1-p) factor (dropout_layer.py:49-52)
    np.testing.assert_array_equal(net.get("Input", "output_deltas", "default"), 1.0 + 2.0 * mask)
    net.forward_pass(training_pass=False)
    np.testing.assert_array_equal(net.get("drop", "outputs", "default"), x)


def test_momentum_stepper_closed_form():
    net, data, params = make_net([("fc", FullyConnected(5, "tanh"), {"default": "Input.default"})], (4,), 3)
    stepper = MomentumStepper(learning_rate=0.1, momentum=0.9)
    stepper.start(net)
    v = np.zeros_like(params)
    p = params.copy()
    for _ in range(3):
        net.set_parameters(p)
        net.forward_pass(training_pass=True)
        net.backward_pass()
        g = net.handler.get_numpy_copy(net.gradients)
        stepper.run()
        v = 0.9 * v - 0.1 * (1 - 0.9) * g          # learning rate scaled by (1 - momentum)
        p = p + v
        np.testing.assert_allclose(net.handler.get_numpy_copy(net.parameters), p, rtol=1e-12, atol=1e-15)


def test_backward_clears_then_adds():
    net, data, params = make_net([("fc", FullyConnected(5, "rel"), {"default": "Input.default"})], (4,), 3)
    net.forward_pass(training_pass=True)
    net.backward_pass()
    first = net.get("Input", "output_deltas", "default").copy()
    net.backward_pass()                                  # cleared before every backward pass
    np.testing.assert_allclose(net.get("Input", "output_deltas", "default"), first, rtol=1e-12)
    net.layers["fc"].backward_pass(net.buffers["fc"])   # a second layer pass alone adds on top
    assert not np.allclose(net.get("Input", "output_deltas", "default"), first)


def test_backward_only_buffers_lie_together_and_one_fill_clears_them():
    # gradients, deltas and the backward-only internals of every layer form one contiguous region of the
    # flat buffer (the reference sorts its buffers into hubs by kind and clears each backward-only hub with
    # one fill, structure/buffers.py:147-150); forward buffers keep their values through a backward pass
    net, data, params = make_net([("lstm", Lstm(4), {"default": "Input.default"})], (3,), 2, time_steps=3)
    assert len(net._backward_only) == 1
    region = net._backward_only[0]
    backward = [net.gradients] + [v for b in net.buffers.values() for v in b.output_deltas.values()]
    is_backward = lambda layer, k: net.specs[layer][2][k].backward_only
    backward += [v for layer, b in net.buffers.items() for k, v in b.internals.items() if is_backward(layer, k)]
    assert all(np.shares_memory(region, v) for v in backward)
    forward = [v for b in net.buffers.values() for v in b.outputs.values()] + [net.parameters]
    forward += [v for layer, b in net.buffers.items() for k, v in b.internals.items() if not is_backward(layer, k)]
    assert not any(np.shares_memory(region, v) for v in forward)
    net.forward_pass(training_pass=True)
    before = {name: {k: np.array(v, copy=True) for k, v in b.outputs.items()} for name, b in net.buffers.items()}
    net.backward_pass()
    assert np.any(net.handler.get_numpy_copy(net.gradients) != 0.0)
    for name, outs in before.items():
        for k, v in outs.items():
            np.testing.assert_array_equal(net.handler.get_numpy_copy(net.buffers[name].outputs[k]), v)
    net.handler.fill(region, 0.0)
    assert not np.any(net.handler.get_numpy_copy(net.gradients))
    for name, outs in before.items():
        for k, v in outs.items():
            np.testing.assert_array_equal(net.handler.get_numpy_copy(net.buffers[name].outputs[k]), v)
