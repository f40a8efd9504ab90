"""GPU: the fusing window. A caller that issues the reference layers' primitive operations only
(fused=False drivers) must get, with the window on, the same bits in every buffer as with the
window off - on all four network workloads, over several training steps, with in-place and
aliased calls, and when a sequence is cut short by a read-back. The window-off runs are what
test_gpu_configs.py holds to the CPU oracle."""
import numpy as np
import pytest

from brainstorm_amd.drivers import configs
from brainstorm_amd.drivers.net import MomentumStepper
from util import assert_bit_equal

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(autouse=True)
def restore_fusing(hip):
    before = hip.fusing
    yield
    hip.set_fusing(before)


def train(hip, builder, fusing, steps, seed=11, **kw):
    hip.set_fusing(fusing)
    hip.rnd.seed(seed)
    net, data = builder(hip, **kw)
    net.provide_external_data(data)
    stepper = MomentumStepper(0.05, 0.9)
    stepper.start(net)
    hip.fusing_stats(reset=True)
    losses = []
    for _ in range(steps):
        stepper.run()
        losses.append(net.get("loss", "outputs", "loss").copy())
    stats = hip.fusing_stats()
    everything = hip.get_numpy_copy(net.full_buffer)
    velocity = hip.get_numpy_copy(stepper.velocity)
    return everything, velocity, np.concatenate([l.ravel() for l in losses]), stats


WORKLOADS = [
    ("mlp", configs.build_mlp, dict(batch=23, in_size=37, hidden=41), 4,
     dict(fused_launches=4 * (3 + 2 + 1 + 1 + 1))),
    ("mlp_full", configs.build_mlp, dict(), 3, dict(fused_launches=3 * 8)),
    ("lstm", configs.build_lstm, dict(time_steps=9, batch=7, symbols=11, hidden=13), 3,
     dict(fused_launches=3 * (9 + 9 + 1 + 1 + 1))),
    ("lstm_wide", configs.build_lstm, dict(time_steps=12, batch=33, symbols=50, hidden=257), 2,
     dict(fused_launches=2 * (12 + 12 + 1 + 1 + 1))),
    ("highway", configs.build_highway, dict(blocks=3, batch=37, width=129), 3,
     dict(fused_launches=3 * (3 * (2 + 2 + 2) + 1 + 1 + 1))),
    ("cnn", configs.build_cnn, dict(batch=6, size=16), 3, dict(fused_launches=3 * (1 + 1 + 1 + 1))),
]


@pytest.mark.parametrize("name,builder,kw,steps,expect", WORKLOADS, ids=[w[0] for w in WORKLOADS])
def test_unchanged_callers_get_the_same_bits(hip, name, builder, kw, steps, expect):
    plain = train(hip, builder, False, steps, **kw)
    fused = train(hip, builder, True, steps, **kw)
    assert plain[3]["calls"] == 0                      # nothing went through the window when it was off
    assert fused[3]["fused_launches"] == expect["fused_launches"], fused[3]
    assert_bit_equal(fused[2], plain[2], name + ": losses")
    assert_bit_equal(fused[0], plain[0], name + ": parameters, gradients and every buffer")
    assert_bit_equal(fused[1], plain[1], name + ": velocity")


def test_lstm_full_size_through_the_window(hip):
    # the char-LSTM workload at its full size: T=100, batch 100, 1000 units, one forward and backward pass
    results = []
    for fusing in (False, True):
        hip.set_fusing(fusing)
        hip.rnd.seed(2)
        net, data = configs.build_lstm(hip)
        net.provide_external_data(data)
        hip.fusing_stats(reset=True)
        net.forward_pass(training_pass=True)
        net.backward_pass()
        stats = hip.fusing_stats()
        results.append((hip.get_numpy_copy(net.gradients), net.get("lstm", "outputs", "default"),
                        net.get("lstm", "internals", "dZa"), net.get("loss", "outputs", "loss"), stats))
        del net
    plain, fused = results
    assert fused[4]["fused_launches"] == 100 + 100 + 1 + 1
    assert fused[4]["overtaken"] >= 300           # the input-, forget- and output-gate products of every forward step
    for k, what in enumerate(("gradients", "outputs", "dZa", "loss")):
        assert_bit_equal(fused[k], plain[k], what)


def test_a_sequence_cut_by_a_read_back(hip):
    rng = np.random.RandomState(3)
    batch, n = 19, 67
    x = rng.standard_normal((batch, n)).astype(F32)
    b = rng.standard_normal((1, n)).astype(F32)
    p = rng.standard_normal((1, n)).astype(F32)
    c = rng.standard_normal((batch, n)).astype(F32)

    def run(fusing, cut):
        hip.set_fusing(fusing)
        Za, Ia, Cp = hip.create_from_numpy(x), hip.create_from_numpy(x * 0.5), hip.create_from_numpy(c)
        bias, peep = hip.create_from_numpy(b), hip.create_from_numpy(p)
        Zb, Ib = hip.allocate((batch, n)), hip.allocate((batch, n))
        seen = []
        # the first five calls of an LSTM time step (lstm_layer.py:122-128) ...
        hip.add_mv(Za, bias, Za)
        hip.tanh(Za, Zb)
        if cut:
            seen.append(hip.get_numpy_copy(Zb))       # ... read back in the middle
        hip.mult_add_mv(Cp, peep, Ia)
        hip.add_mv(Ia, bias, Ia)
        hip.sigmoid(Ia, Ib)
        # ... and then something else
        hip.mult_tt(Ib, Zb, Za)
        return [hip.get_numpy_copy(a) for a in (Za, Zb, Ia, Ib)] + seen

    want = run(False, True)
    for cut in (True, False):
        got = run(True, cut)
        for k, (g, w) in enumerate(zip(got, want)):
            assert_bit_equal(g, w, "array %d (cut=%r)" % (k, cut))


def test_in_place_and_aliased_calls(hip):
    rng = np.random.RandomState(4)
    m, n = 29, 131
    x = rng.standard_normal((m, n)).astype(F32)
    v = rng.standard_normal((1, n)).astype(F32)

    def run(fusing):
        hip.set_fusing(fusing)
        out = []
        # bias + activation in place and out of place
        a, bias = hip.create_from_numpy(x), hip.create_from_numpy(v)
        hip.add_mv(a, bias, a)
        hip.sigmoid(a, a)
        out.append(hip.get_numpy_copy(a))
        a, t = hip.create_from_numpy(x), hip.allocate((m, n))
        hip.add_mv(a, bias, t)
        hip.rel(t, t)
        out += [hip.get_numpy_copy(a), hip.get_numpy_copy(t)]
        # the momentum update's three calls on ONE array (velocity = gradients = parameters): not the fused form
        w = hip.create_from_numpy(x)
        hip.mult_st(0.9, w, w)
        hip.mult_add_st(-0.1, w, w)
        hip.add_tt(w, w, w)
        out.append(hip.get_numpy_copy(w))
        # Highway's forward calls with H = x (reads may alias) and with y = the temporary (must not fuse)
        H, T = hip.create_from_numpy(x), hip.create_from_numpy(np.abs(x) % 1)
        y = hip.allocate((m, n))
        tmp = hip.zeros((m, n))
        hip.subtract_tt(H, H, tmp)
        hip.mult_tt(T, tmp, tmp)
        hip.add_tt(tmp, H, y)
        del tmp
        out.append(hip.get_numpy_copy(y))
        tmp = hip.zeros((m, n))
        hip.subtract_tt(H, T, tmp)
        hip.mult_tt(T, tmp, tmp)
        hip.add_tt(tmp, T, tmp)
        out.append(hip.get_numpy_copy(tmp))
        # softmax cross entropy backward with the deltas aliasing the one-hot buffer
        probs = hip.create_from_numpy(np.abs(x))
        labels = hip.create_from_numpy(rng.randint(0, n, (m, 1)).astype(F32))
        dloss = hip.create_from_numpy(rng.standard_normal((m, 1)).astype(F32))
        tb = hip.allocate((m, n))
        hip.binarize_v(labels, tb)
        hip.mult_st(-1, tb, tb)
        hip.add_tt(tb, probs, tb)
        hip.mult_mv(tb, dloss, tb)
        hip.add_tt(tb, tb, tb)
        out.append(hip.get_numpy_copy(tb))
        return out

    rng_state = rng.get_state()
    want = run(False)
    rng.set_state(rng_state)
    got = run(True)
    for k, (g, w) in enumerate(zip(got, want)):
        assert_bit_equal(g, w, "result %d" % k)


def test_errors_of_held_calls_surface(hip):
    hip.set_fusing(True)
    a, v = hip.allocate((4, 6)), hip.allocate((1, 6))
    hip.add_mv(a, v, a)                          # held
    assert hip.fusing_stats()["calls"] >= 1
    hip.synchronize()                            # enqueues it; nothing to report
    assert np.array_equal(hip.get_numpy_copy(a), np.zeros((4, 6), F32))


@pytest.mark.parametrize("kw", [dict(time_steps=9, batch=7, symbols=11, hidden=13),
                                dict(time_steps=12, batch=33, symbols=50, hidden=257),
                                dict(time_steps=6, batch=100, symbols=30, hidden=512)])
def test_stacked_products_agree_to_rounding(hip, kw):
    # fusing="stacked": one product over [Rz;Ri;Rf;Ro] per time step instead of four; only the order in which the
    # products sum changes, so every buffer agrees with the window-off run to rounding
    results = {}
    for mode in (False, "stacked"):
        hip.set_fusing(mode)
        hip.rnd.seed(7)
        net, data = configs.build_lstm(hip, **kw)
        net.provide_external_data(data)
        stepper = MomentumStepper(0.05, 0.9)
        stepper.start(net)
        hip.fusing_stats(reset=True)
        for _ in range(2):
            stepper.run()
        stats = hip.fusing_stats()
        results[mode] = ({(group, key): net.get("lstm", group, key) for group in ("outputs", "internals", "output_deltas")
                          for key in getattr(net.buffers["lstm"], group)},
                         hip.get_numpy_copy(net.gradients), hip.get_numpy_copy(net.parameters), stats)
        del net, stepper
    plain, stacked = results[False], results["stacked"]
    T = kw["time_steps"]
    assert stacked[3]["fused_launches"] == 2 * (2 * T + 3)
    for key, want in plain[0].items():
        scale = float(np.max(np.abs(want))) or 1.0
        assert float(np.max(np.abs(stacked[0][key] - want))) <= 2e-5 * scale, key
    for k, what in ((1, "gradients"), (2, "parameters")):
        scale = float(np.max(np.abs(plain[k])))
        assert float(np.max(np.abs(stacked[k] - plain[k]))) <= 2e-5 * scale, what


# ---------------------------------------------------------------- call streams that almost match
OPS = {"add_tt", "subtract_tt", "mult_tt", "divide_tt", "mult_add_tt", "add_st", "mult_st", "mult_add_st", "add_mv",
       "subtract_mv", "mult_mv", "divide_mv", "mult_add_mv", "sigmoid", "tanh", "rel", "el", "softmax_m", "sigmoid_deriv",
       "tanh_deriv", "rel_deriv", "el_deriv", "fill", "copy_to", "sum_t", "dot_mm", "dot_add_mm", "clip_t", "abs_t",
       "sign_t", "sqrt_t", "log_t", "binarize_v", "index_m_by_v", "broadcast_t", "generate_probability_mask",
       "maxpool2d_forward_batch", "maxpool2d_backward_batch", "conv2d_forward_batch", "conv2d_backward_batch"}


class MutatingHandler(object):
    """Passes a network's handler calls on, except at the numbered calls of `plan`: "drop" leaves the call
    out, "twice" issues it twice, "late" issues it after the call that follows it, "read" reads one of its
    array operands back first, "alias" lets it write over its first operand (same size only). The window
    must give every such stream the bits it has when each call is launched as it comes."""

    def __init__(self, real, plan):
        self.__dict__["_real"], self.__dict__["_plan"] = real, plan
        self.__dict__["count"], self.__dict__["_held"] = 0, None

    def __getattr__(self, name):
        attr = getattr(self._real, name)
        if name not in OPS:
            return attr

        def call(*args, **kwargs):
            index = self.count
            self.__dict__["count"] = index + 1
            action = self._plan.get(index)
            arrays = [a for a in args if hasattr(a, "ptr") and a.size]
            if action == "read" and arrays:
                self._real.get_numpy_copy(arrays[len(arrays) // 2])
            if action == "alias" and len(arrays) >= 2 and arrays[0].size == arrays[-1].size and args[-1] is arrays[-1]:
                args = args[:-1] + (arrays[0].reshape(arrays[-1].shape),)
            if action == "drop":
                return None
            if action == "late" and self._held is None:
                self.__dict__["_held"] = (attr, args, kwargs)
                return None
            result = attr(*args, **kwargs)
            if action == "twice":
                attr(*args, **kwargs)
            if self._held is not None:
                late, late_args, late_kwargs = self._held
                self.__dict__["_held"] = None
                late(*late_args, **late_kwargs)
            return result
        return call

    def __setattr__(self, name, value):
        setattr(self._real, name, value)


def train_mutated(hip, builder, fusing, steps, plan, seed=11, **kw):
    hip.set_fusing(fusing)
    hip.rnd.seed(seed)
    proxy = MutatingHandler(hip, plan)
    net, data = builder(proxy, **kw)
    net.provide_external_data(data)
    stepper = MomentumStepper(0.05, 0.9)
    stepper.start(net)
    hip.fusing_stats(reset=True)
    for _ in range(steps):
        stepper.run()
    fused_launches = hip.fusing_stats()["fused_launches"]
    return hip.get_numpy_copy(net.full_buffer), hip.get_numpy_copy(stepper.velocity), proxy.count, fused_launches


MUTATED = [("mlp", configs.build_mlp, dict(batch=23, in_size=37, hidden=41)),
           ("lstm", configs.build_lstm, dict(time_steps=5, batch=7, symbols=11, hidden=13)),
           ("highway", configs.build_highway, dict(blocks=2, batch=37, width=129)),
           ("cnn", configs.build_cnn, dict(batch=3, size=16))]


@pytest.mark.parametrize("name,builder,kw", MUTATED, ids=[w[0] for w in MUTATED])
def test_call_streams_that_almost_match_keep_their_bits(hip, name, builder, kw):
    # the layers' sequences with calls missing, doubled, out of place, read back in the middle or writing
    # over an operand: the patterns match in part, then do not - held calls must come out as they were called
    calls = train_mutated(hip, builder, False, 2, {}, **kw)[2]
    rng = np.random.RandomState(97)
    actions = ("drop", "twice", "late", "read", "alias")
    still_fused = 0
    for trial in range(40):
        sites = rng.choice(calls, size=1 + trial % 12, replace=False)
        plan = {int(i): actions[rng.randint(len(actions))] for i in sites}
        plain = train_mutated(hip, builder, False, 2, plan, **kw)
        fused = train_mutated(hip, builder, True, 2, plan, **kw)
        assert plain[2] == fused[2] and plain[3] == 0
        still_fused += fused[3]
        case = "%s trial %d %r" % (name, trial, sorted(plan.items()))
        assert_bit_equal(fused[0], plain[0], case + ": buffers")
        assert_bit_equal(fused[1], plain[1], case + ": velocity")
    assert still_fused > 40          # the undisturbed parts of the streams went through the fused kernels


def test_stacked_window_on_call_streams_that_almost_match(hip):
    # fusing="stacked" also holds the recurrent products and reuses a packed copy of the deltas from step to
    # step; with calls missing, doubled, delayed, read back or aliased nothing stale may get into a product.
    # Other summation order inside the stacked products: agreement to 1e-4 of the buffers' scale, not the same bits.
    kw = dict(time_steps=5, batch=7, symbols=11, hidden=13)
    calls = train_mutated(hip, configs.build_lstm, False, 2, {}, **kw)[2]
    rng = np.random.RandomState(5)
    actions = ("drop", "twice", "late", "read", "alias")
    for trial in range(60):
        sites = rng.choice(calls, size=1 + trial % 12, replace=False)
        plan = {int(i): actions[rng.randint(len(actions))] for i in sites}
        plain = train_mutated(hip, configs.build_lstm, False, 2, plan, **kw)
        stacked = train_mutated(hip, configs.build_lstm, "stacked", 2, plan, **kw)
        case = "trial %d %r" % (trial, sorted(plan.items()))
        for a, b in ((plain[0], stacked[0]), (plain[1], stacked[1])):
            finite = np.isfinite(a)
            assert np.array_equal(finite, np.isfinite(b)), case
            if finite.any():
                assert np.max(np.abs(a[finite] - b[finite])) <= 1e-4 * max(1.0, np.max(np.abs(a[finite]))), case
