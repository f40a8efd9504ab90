"""The whole-sequence LSTM forward kernel (bship_lstm_fwd_sequence_f32) against the oracle's
primitive-by-primitive layer (lstm_layer.py:103-145 through NumpyRefHandler) and against a float64
model of the recurrence for the activations and context slots the benchmark network does not use.

Bars: the kernel adds the recurrent products in its own order (four K-quarters, 16 k per
matrix-core step), so pre-activations differ from the oracle's float32 BLAS sums in the last bits:
<= 1e-5 of the largest magnitude per buffer, the bar of the other matrix-product paths.
"""
import os
import subprocess
import sys

import numpy as np
import pytest

from brainstorm_amd import HipHandler
from brainstorm_amd._lib import ERR_TIMEOUT, BshipError
from brainstorm_amd.drivers import configs
from oracle.numpy_ref_handler import NumpyRefHandler

pytestmark = pytest.mark.gpu
F32 = np.float32
INTERNALS = ("Za", "Zb", "Ia", "Ib", "Fa", "Fb", "Oa", "Ob", "Ca", "Cb")
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def scaled_err(got, want):
    scale = float(np.max(np.abs(want)))
    return float(np.max(np.abs(got.astype(np.float64) - want))) / (scale if scale > 0 else 1.0)


# (time steps, batch, symbols, cells): one row tile, a ragged tile, exactly one row set, two row sets with
# 3 + 2, 4 + 3 and 4 + 4 tiles, cells that leave K-quarters empty or ragged, the largest layer (256 workgroups)
SHAPES = [(3, 5, 11, 12), (4, 16, 9, 64), (5, 33, 20, 100), (4, 64, 13, 256), (3, 65, 13, 36),
          (6, 100, 30, 200), (3, 128, 7, 64), (2, 77, 5, 4), (2, 100, 7, 1024)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "T%d_B%d_S%d_H%d" % s)
def test_sequence_kernel_matches_oracle_layer(hip, shape):
    steps, batch, symbols, hidden = shape
    kw = dict(time_steps=steps, batch=batch, symbols=symbols, hidden=hidden)
    ref = NumpyRefHandler(F32, seed=3)
    net_r, data = configs.build_lstm(ref, **kw)
    net_r.provide_external_data(data)
    net_r.forward_pass(training_pass=True)
    hip.rnd.seed(3)
    net_h, data_h = configs.build_lstm(hip, fused="sequence", **kw)
    net_h.provide_external_data(data_h)
    calls = []
    real = hip.lstm_forward_sequence
    hip.lstm_forward_sequence = lambda *a: calls.append(real(*a)) or calls[-1]
    try:
        net_h.forward_pass(training_pass=True)
    finally:
        del hip.lstm_forward_sequence
    assert calls == [True], "the layer did not take the whole-sequence kernel: %r" % calls
    for key in INTERNALS:
        err = scaled_err(net_h.get("lstm", "internals", key), net_r.get("lstm", "internals", key))
        assert err <= 1e-5, (key, err)
    assert scaled_err(net_h.get("lstm", "outputs", "default"), net_r.get("lstm", "outputs", "default")) <= 1e-5
    loss_h, loss_r = net_h.get("loss", "outputs", "loss")[0], net_r.get("loss", "outputs", "loss")[0]
    assert abs(loss_h - loss_r) <= 1e-5 * abs(loss_r)
    # and the backward pass that follows reads what the kernel left: gradients at the oracle's bar
    net_h.backward_pass()
    net_r.backward_pass()
    g_h = hip.get_numpy_copy(net_h.gradients)
    for name, (a, b, _) in net_r.parameter_slices().items():
        assert scaled_err(g_h[a:b], net_r.gradients[a:b]) <= 1e-4, name


def _model(act, R, inputs, y0, c0, peep, bias):
    """Peephole LSTM recurrence in float64 (lstm_layer.py:115-145 as formulas)."""
    f = {"sigmoid": lambda x: 1 / (1 + np.exp(-x)), "tanh": np.tanh, "rel": lambda x: x * (x > 0),
         "linear": lambda x: x, "el": lambda x: np.where(x >= 0, x, np.exp(np.minimum(x, 0)) - 1)}[act]
    sig = lambda x: 1 / (1 + np.exp(-x))
    n = R.shape[1]
    Rz, Ri, Rf, Ro = (R[k * n:(k + 1) * n].astype(np.float64) for k in range(4))
    pi, pf, po = (p.astype(np.float64) for p in peep)
    bz, bi, bf, bo = (b.astype(np.float64) for b in bias)
    y, c = y0.astype(np.float64), c0.astype(np.float64)
    ys, cs = [], []
    for za, ia, fa, oa in zip(*inputs):
        z = f(za + y @ Rz.T + bz)
        i = sig(ia + y @ Ri.T + c * pi + bi)
        fg = sig(fa + y @ Rf.T + c * pf + bf)
        c = i * z + fg * c
        o = sig(oa + y @ Ro.T + c * po + bo)
        y = o * f(c)
        ys.append(y)
        cs.append(c)
    return np.array(ys), np.array(cs)


@pytest.mark.parametrize("act", ["sigmoid", "tanh", "rel", "linear", "el"])
def test_sequence_kernel_activations_and_context(hip, act):
    # non-zero context slots (y[-1], Ca[-1]) and every activation, against the float64 model
    steps, batch, n = 7, 70, 48
    rng = np.random.RandomState(11)
    R = (rng.standard_normal((4 * n, n)) * 0.2).astype(F32)
    host = {k: np.zeros((steps + 1, batch, n), F32) for k in INTERNALS + ("y",)}
    for k in ("Za", "Ia", "Fa", "Oa"):
        host[k][:steps] = rng.standard_normal((steps, batch, n)).astype(F32)
    host["y"][steps] = rng.uniform(-1, 1, (batch, n)).astype(F32)
    host["Ca"][steps] = rng.standard_normal((batch, n)).astype(F32)
    vecs = [(rng.standard_normal(n) * 0.5).astype(F32) for _ in range(7)]
    want_y, want_c = _model(act, R, [host[k][:steps] for k in ("Za", "Ia", "Fa", "Oa")], host["y"][steps],
                            host["Ca"][steps], vecs[:3], vecs[3:])
    dev = {k: hip.create_from_numpy(v) for k, v in host.items()}
    ok = hip.lstm_forward_sequence(act, hip.create_from_numpy(R), *[dev[k] for k in INTERNALS], dev["y"],
                                   *[hip.create_from_numpy(v) for v in vecs])
    assert ok is True
    got_y, got_c = hip.get_numpy_copy(dev["y"]), hip.get_numpy_copy(dev["Ca"])
    assert scaled_err(got_y[:steps], want_y) <= 1e-5
    assert scaled_err(got_c[:steps], want_c) <= 1e-5
    # the context slots are inputs only
    assert np.array_equal(got_y[steps], host["y"][steps]) and np.array_equal(got_c[steps], host["Ca"][steps])


@pytest.mark.parametrize("batch,n", [(8, 10), (129, 16), (8, 1028)],
                         ids=["n_not_multiple_of_4", "batch_over_128", "n_over_1024"])
def test_sequence_kernel_declines_shapes_it_does_not_fit(hip, batch, n):
    steps = 2
    mats = [hip.allocate((steps + 1, batch, n)) for _ in range(11)]
    for m in mats:
        hip.fill(m, 0.25)
    vecs = [hip.zeros((n,)) for _ in range(7)]
    assert hip.lstm_forward_sequence("tanh", hip.zeros((4 * n, n)), *mats, *vecs) is False
    for m in mats:                                   # nothing was touched
        assert float(hip.get_numpy_copy(m).min()) == 0.25 == float(hip.get_numpy_copy(m).max())
    # the layer then takes the step-by-step path (checked for n % 4 != 0 through the network)
    if n == 10:
        kw = dict(time_steps=3, batch=batch, symbols=6, hidden=n)
        ref = NumpyRefHandler(F32, seed=5)
        net_r, data = configs.build_lstm(ref, **kw)
        net_r.provide_external_data(data)
        net_r.forward_pass(training_pass=True)
        hip.rnd.seed(5)
        net_h, data_h = configs.build_lstm(hip, fused="sequence", **kw)
        net_h.provide_external_data(data_h)
        net_h.forward_pass(training_pass=True)
        assert scaled_err(net_h.get("lstm", "outputs", "default"), net_r.get("lstm", "outputs", "default")) <= 1e-5


def test_sequence_kernel_with_reused_operand_buffers(hip, monkeypatch):
    # a scratch limit of 1 MB leaves two operand buffers for 1000 units: they are rewritten every other step
    # and the caches invalidated at every barrier; same results as with one buffer per step
    steps, batch, n = 9, 100, 1000
    rng = np.random.RandomState(4)
    R = hip.create_from_numpy((rng.standard_normal((4 * n, n)) * 0.03).astype(F32))
    host = {k: np.zeros((steps + 1, batch, n), F32) for k in INTERNALS + ("y",)}
    for k in ("Za", "Ia", "Fa", "Oa"):
        host[k][:steps] = (rng.standard_normal((steps, batch, n)) * 0.5).astype(F32)
    vecs = [hip.create_from_numpy((rng.standard_normal(n) * 0.3).astype(F32)) for _ in range(7)]

    def run():
        dev = {k: hip.create_from_numpy(v) for k, v in host.items()}
        assert hip.lstm_forward_sequence("tanh", R, *[dev[k] for k in INTERNALS], dev["y"], *vecs) is True
        return {k: hip.get_numpy_copy(v) for k, v in dev.items()}

    want = run()
    monkeypatch.setenv("BSHIP_LSTM_SEQ_SCRATCH_MB", "1")
    got = run()
    for k in want:
        assert np.array_equal(got[k], want[k]), k


_TIMEOUT_SCRIPT = r"""
import sys
import numpy as np
sys.path.insert(0, %r)
from brainstorm_amd import HipHandler
from brainstorm_amd._lib import BshipError
h = HipHandler(seed=0)
steps, batch, n = 4, 20, 256
mats = [h.zeros((steps + 1, batch, n)) for _ in range(11)]
vecs = [h.zeros((n,)) for _ in range(7)]
try:
    h.lstm_forward_sequence("tanh", h.zeros((4 * n, n)), *mats, *vecs)
    print("NO ERROR")
except BshipError as e:
    print("STATUS", e.status)
# every workgroup has left the device: ordinary work goes on
a = h.create_from_numpy(np.arange(6, dtype=np.float32).reshape(2, 3))
h.add_tt(a, a, a)
print("AFTER", h.get_numpy_copy(a).sum())
"""


def test_barrier_timeout_is_reported_and_the_device_stays_usable():
    # A spin limit of 0 makes every workgroup give up at its first barrier without polling: the kernel
    # exits normally, the call reports BSHIP_ERR_TIMEOUT, later calls work.
    env = dict(os.environ, BSHIP_GRID_BARRIER_SPINS="0")
    res = subprocess.run([sys.executable, "-c", _TIMEOUT_SCRIPT % REPO], env=env, capture_output=True, text=True,
                         timeout=110)
    assert res.returncode == 0, res.stderr
    assert "STATUS %d" % ERR_TIMEOUT in res.stdout, res.stdout + res.stderr
    assert "AFTER 30.0" in res.stdout, res.stdout


_FALLBACK_SCRIPT = r"""
import sys
import numpy as np
sys.path.insert(0, %r)
from brainstorm_amd import HipHandler
from brainstorm_amd.drivers import configs
from oracle.numpy_ref_handler import NumpyRefHandler
shape = dict(time_steps=6, batch=20, symbols=9, hidden=64)
h = HipHandler(seed=0)
net, data = configs.build_lstm(h, fused="sequence", **shape)
net.provide_external_data(data)
net.forward_pass(training_pass=True)
net.backward_pass()
print("FALLBACKS", net.layers["lstm"].sequence_fallbacks)
ref, _ = configs.build_lstm(NumpyRefHandler(np.float32, seed=0), **shape)
ref.provide_external_data(data)
ref.forward_pass(training_pass=True)
ref.backward_pass()
worst = 0.0
for group, key in (("outputs", "default"), ("internals", "Ca"), ("internals", "Ob"), ("internals", "dZa")):
    got, want = net.get("lstm", group, key), ref.get("lstm", group, key)
    worst = max(worst, float(np.max(np.abs(got - want)) / max(np.max(np.abs(want)), 1e-30)))
got, want = h.get_numpy_copy(net.gradients), ref.gradients
worst = max(worst, float(np.max(np.abs(got - want)) / np.max(np.abs(want))))
print("WORST %%.3e" %% worst)
"""


def test_the_layer_takes_the_step_loop_when_the_sequence_kernel_times_out():
    # every barrier of the sequence kernel fails at once (spin limit 0, forced from the host; the kernel exits
    # normally): the layer forms the input products again and runs the recurrence step by step
    env = dict(os.environ, BSHIP_GRID_BARRIER_SPINS="0")
    res = subprocess.run([sys.executable, "-c", _FALLBACK_SCRIPT % REPO], env=env, capture_output=True, text=True,
                         timeout=110)
    assert res.returncode == 0, res.stderr
    assert "FALLBACKS 1" in res.stdout, res.stdout + res.stderr
    worst = float(res.stdout.split("WORST")[1].split()[0])
    assert worst <= 1e-5, res.stdout


def test_unparsable_spin_limits_are_ignored():
    # "abc" or "12x" must not become a spin limit of 0 (which fails every barrier)
    for value in ("abc", "12x", "-3", ""):
        env = dict(os.environ, BSHIP_GRID_BARRIER_SPINS=value)
        res = subprocess.run([sys.executable, "-c", _TIMEOUT_SCRIPT % REPO], env=env, capture_output=True, text=True,
                             timeout=110)
        assert res.returncode == 0, res.stderr
        assert "NO ERROR" in res.stdout, (value, res.stdout + res.stderr)
