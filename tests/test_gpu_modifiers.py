"""GPU: arithmetic operators of DeviceArray, the modifier-like op sequences that use them (modifier_ops.py),
and the contract-checking wrapper around HipHandler, each against the CPU oracle on the same inputs."""
import numpy as np
import pytest

from brainstorm_amd.checked_handler import CheckedHandler, ContractError
import modifier_ops
from brainstorm_amd.drivers import configs
from brainstorm_amd.drivers.net import MomentumStepper
from oracle.numpy_ref_handler import NumpyRefHandler
from util import assert_bit_equal

pytestmark = pytest.mark.gpu
F32 = np.float32


def test_device_array_operators_match_numpy(hip):
    rng = np.random.RandomState(1)
    x = rng.standard_normal((37, 129)).astype(F32)
    y = rng.uniform(0.5, 2.0, (37, 129)).astype(F32)
    a, b = hip.create_from_numpy(x), hip.create_from_numpy(y)
    assert_bit_equal((a * b).get(), x * y, "a * b")
    assert_bit_equal((a * 0.3).get(), x * F32(0.3), "a * s")
    assert_bit_equal((0.3 * a).get(), F32(0.3) * x, "s * a")
    assert_bit_equal((a + b).get(), x + y, "a + b")
    assert_bit_equal((a + 2).get(), x + F32(2), "a + s")
    assert_bit_equal((a - b).get(), x - y, "a - b")
    assert_bit_equal((a / b).get(), x / y, "a / b")
    assert_bit_equal((b ** 0.5).get(), y ** 0.5, "b ** 0.5")
    assert_bit_equal((a ** 2).get(), x ** 2, "a ** 2")
    assert_bit_equal(a.get(), x, "operands are left alone")
    with pytest.raises(NotImplementedError):
        a ** 3
    with pytest.raises(ValueError):
        a * hip.allocate((129, 37))
    with pytest.raises(TypeError):
        a * "two"


def test_modifiers_match_the_oracle(hip):
    ref = NumpyRefHandler(F32, seed=0)
    rng = np.random.RandomState(2)
    w = rng.standard_normal((300, 5, 41)).astype(F32)
    g = rng.standard_normal(w.shape).astype(F32)
    mask = (rng.uniform(size=w.shape) < 0.5).astype(F32)

    def both(what, make, exact=True, with_grad=False):
        outs = []
        for h in (hip, ref):
            view = h.create_from_numpy(w.copy())
            mod = make()
            if with_grad:
                grad = h.create_from_numpy(g.copy())
                mod(h, view, grad)
                outs.append(h.get_numpy_copy(grad))
            else:
                mod(h, view)
                outs.append(h.get_numpy_copy(view))
        if exact:
            assert_bit_equal(outs[0], outs[1], what)
        return outs

    for with_operators in (True, False):
        got, want = both("cap_row_norms", lambda: modifier_ops.cap_row_norms(2.0, with_operators), exact=False)
        np.testing.assert_allclose(got, want, rtol=1e-5)         # row sums of squares: 1e-5 relative
        assert np.sqrt((got.reshape(300, -1).astype(np.float64) ** 2).sum(axis=1)).max() <= 2.0 * (1 + 1e-5)
    both("clamp", lambda: modifier_ops.clamp(-0.5, 0.25))
    both("keep_where", lambda: modifier_ops.keep_where(mask))
    both("hold_values", lambda: modifier_ops.hold_values(g))
    both("shrink_l1", lambda: modifier_ops.shrink_l1(0.01), with_grad=True)
    both("shrink_l2", lambda: modifier_ops.shrink_l2(0.01), with_grad=True)


def test_mlp_with_norm_constraint_trains_like_the_oracle(hip):
    # the shape of examples/mnist_pi.py including a row-norm cap on every weight matrix after each update
    nets = []
    for h in (hip, NumpyRefHandler(F32, seed=9)):
        if h is hip:
            hip.rnd.seed(9)
        net, data = configs.build_mlp(h, batch=50, in_size=64, hidden=96)
        net.provide_external_data(data)
        net.weight_modifiers = {(name, "W"): [modifier_ops.cap_row_norms(0.3)] for name in ("fc1", "fc2", "out")}
        stepper = MomentumStepper(0.1, 0.9)
        stepper.start(net)
        for _ in range(10):
            stepper.run()
        nets.append(net)
    p_h, p_r = hip.get_numpy_copy(nets[0].parameters), nets[1].parameters
    assert float(np.max(np.abs(p_h - p_r))) <= 1e-4 * float(np.max(np.abs(p_r)))
    for k in ("drop1", "drop2", "drop3"):
        assert_bit_equal(nets[0].get(k, "internals", "mask"), nets[1].get(k, "internals", "mask"), k)


def test_checked_hip_handler(hip):
    checked = CheckedHandler(hip, check_finite=True)
    assert checked.array_type is hip.array_type
    a = checked.create_from_numpy(np.ones((4, 6), F32))
    with pytest.raises(ContractError):
        checked.add_tt(a, checked.allocate((6, 4)), a)           # would write out of bounds unchecked
    with pytest.raises(ContractError):
        checked.add_mv(a, checked.allocate((1, 5)), a)
    with pytest.raises(ValueError, match="log_t"):
        checked.log_t(checked.zeros((2, 2)), checked.allocate((2, 2)))       # log(0) = -inf
    # a training step of every driver passes the contracts, fused entry points included
    for builder, kw in ((configs.build_mlp, dict(batch=5, in_size=7, hidden=6, fused=True)),
                        (configs.build_lstm, dict(time_steps=4, batch=3, symbols=5, hidden=6, fused="packed")),
                        (configs.build_highway, dict(blocks=2, batch=6, width=5, fused=True)),
                        (configs.build_cnn, dict(batch=2, size=8))):
        net, data = builder(checked, **kw)
        net.provide_external_data(data)
        stepper = MomentumStepper(0.01, 0.9)
        stepper.start(net)
        stepper.run()
        assert np.isfinite(net.get("loss", "outputs", "loss")).all()
