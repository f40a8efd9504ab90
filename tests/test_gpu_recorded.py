"""Recorded steps (HIP graphs): every replay must give what eager execution gives.

Each recording is replayed several times, with eager work and synchronisation between the
replays and inputs that change, and every replay is compared with the eager result.
"""
import numpy as np
import pytest

from util import assert_bit_equal

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture()
def hip():
    from brainstorm_amd import HipHandler
    return HipHandler(seed=1234)


@pytest.fixture()
def ref():
    from oracle.numpy_ref_handler import NumpyRefHandler
    return NumpyRefHandler(seed=1234)


def _sequence(h, x, w, bias, hid, act, colsum, prob, out):
    """A layer-like sequence with a matrix product, broadcasts, reductions and a temporary."""
    h.dot_mm(x, w, hid)
    h.add_mv(hid, bias, hid)
    h.sigmoid(hid, act)
    tmp = h.allocate(act.shape)               # allocated (and dropped) inside the sequence
    h.mult_tt(act, act, tmp)
    h.sum_t(tmp, 0, colsum)
    h.softmax_m(hid, prob)
    h.mult_add_st(0.5, prob, out)
    h.clip_t(out, -0.75, 0.75, out)


def test_replays_equal_eager_execution(hip):
    rng = np.random.RandomState(5)
    m, k, n = 96, 300, 200
    shapes = dict(x=(m, k), w=(k, n), bias=(1, n), hid=(m, n), act=(m, n), colsum=(1, n), prob=(m, n), out=(m, n))
    dev = {name: hip.allocate(shape) for name, shape in shapes.items()}
    eager = {name: hip.allocate(shape) for name, shape in shapes.items()}

    def load(arrays, seed):
        r = np.random.RandomState(seed)
        for name in ("x", "w", "bias", "out"):
            hip.set_from_numpy(arrays[name], r.standard_normal(shapes[name]).astype(F32))

    load(dev, 0)
    _sequence(hip, **dev)                      # lazy set-up (plans, workspaces) happens outside the recording
    step = hip.record(lambda: _sequence(hip, **dev))
    for replay in range(4):
        load(dev, 100 + replay)
        load(eager, 100 + replay)
        step.replay()
        # eager work of the same kinds between the replays, with a wait
        _sequence(hip, **eager)
        scratch = hip.allocate((257, 129))
        hip.fill(scratch, float(replay))
        hip.synchronize()
        for name in ("hid", "act", "colsum", "prob", "out"):
            assert_bit_equal(hip.get_numpy_copy(dev[name]), hip.get_numpy_copy(eager[name]),
                             "%s, replay %d" % (name, replay))
        assert_bit_equal(hip.get_numpy_copy(scratch), np.full((257, 129), replay, F32), "eager scratch")
    step.release()
    # the handler keeps working after the recording is gone
    load(dev, 7)
    load(eager, 7)
    _sequence(hip, **dev)
    _sequence(hip, **eager)
    assert_bit_equal(hip.get_numpy_copy(dev["out"]), hip.get_numpy_copy(eager["out"]), "after release")


def test_calls_that_wait_are_refused_while_recording(hip):
    a = hip.allocate((8, 8))
    host = np.zeros((8, 8), F32)

    def bad_step():
        hip.fill(a, 1.0)
        hip.get_numpy_copy(a)

    with pytest.raises(Exception) as err:
        hip.record(bad_step)
    assert "recorded" in str(err.value)
    # the failed recording leaves the handler usable, eagerly and for a new recording
    hip.fill(a, 2.0)
    assert_bit_equal(hip.get_numpy_copy(a), np.full((8, 8), 2.0, F32), "after failed recording")
    for call in (lambda: hip.set_from_numpy(a, host), hip.synchronize, lambda: hip.is_fully_finite(a),
                 lambda: hip.fill_gaussian(0.0, 1.0, a)):
        with pytest.raises(Exception):
            hip.record(call)
    step = hip.record(lambda: hip.add_st(1.0, a, a))
    step.replay()
    step.replay()
    assert_bit_equal(hip.get_numpy_copy(a), np.full((8, 8), 4.0, F32), "two replays of add_st")


def test_masks_of_recorded_steps_continue_the_random_stream(hip, ref):
    shape_a, shape_b = (100, 1200), (37, 61)
    ma, mb, x, y, md = (hip.allocate(shape_a), hip.allocate(shape_b), hip.allocate(shape_a),
                        hip.allocate(shape_a), hip.allocate(shape_a))
    hip.fill(x, 2.0)
    ra, rb, rd = np.zeros(shape_a, F32), np.zeros(shape_b, F32), np.zeros(shape_a, F32)

    def step_fn():
        hip.generate_probability_mask(ma, 0.8)
        hip.generate_probability_mask(mb, 0.5)
        hip.dropout_forward(x, 0.7, 1.25, md, y)

    def ref_step():
        ref.generate_probability_mask(ra, 0.8)
        ref.generate_probability_mask(rb, 0.5)
        ref.generate_probability_mask(rd, 0.7)

    def check(what):
        assert_bit_equal(hip.get_numpy_copy(ma), ra, what + ": first mask")
        assert_bit_equal(hip.get_numpy_copy(mb), rb, what + ": second mask")
        assert_bit_equal(hip.get_numpy_copy(md), rd, what + ": dropout mask")
        assert_bit_equal(hip.get_numpy_copy(y), (F32(1.25) * (F32(2.0) * rd)).astype(F32), what + ": dropout output")

    # eager steps first (the prefetch of eager masks gets going), then the recording
    for i in range(3):
        step_fn()
        ref_step()
        check("eager step %d" % i)
    step = hip.record(step_fn)
    for i in range(3):
        step.replay()
        ref_step()
        check("replay %d" % i)
    # another use of the generator between replays: the pending masks are given up, nothing is skipped
    other, rother = hip.allocate((50, 50)), np.zeros((50, 50), F32)
    hip.generate_probability_mask(other, 0.3)
    ref.generate_probability_mask(rother, 0.3)
    assert_bit_equal(hip.get_numpy_copy(other), rother, "eager mask between replays")
    for i in range(2):
        step.replay()
        ref_step()
        check("replay after eager use %d" % i)
    # eager steps again, and a gaussian draw, continue from the right position
    step_fn()
    ref_step()
    check("eager step after replays")
    g, rg = hip.allocate((33, 5)), np.zeros((33, 5), F32)
    hip.fill_gaussian(0.0, 1.0, g)
    ref.fill_gaussian(0.0, 1.0, rg)
    assert_bit_equal(hip.get_numpy_copy(g), rg, "gaussian draw after replays")
    step.replay()
    ref_step()
    check("replay after gaussian draw")
    step.release()
    step_fn()
    ref_step()
    check("eager step after release")


def test_two_recordings_with_masks_share_the_random_stream(hip, ref):
    # two recorded steps that both draw masks, replayed in turn: each replay takes the next numbers of the one
    # stream (the pending masks of the other recording are given up, nothing is skipped or used twice)
    sa, sb, sc = (100, 784), (64, 1200), (3, 7)
    ma, mb, mc = hip.allocate(sa), hip.allocate(sb), hip.allocate(sc)
    ra, rb, rc = np.zeros(sa, F32), np.zeros(sb, F32), np.zeros(sc, F32)

    def step_a():
        hip.generate_probability_mask(ma, 0.8)
        hip.generate_probability_mask(mc, 0.5)

    def step_b():
        hip.generate_probability_mask(mb, 0.3)

    def ref_a():
        ref.generate_probability_mask(ra, 0.8)
        ref.generate_probability_mask(rc, 0.5)

    def ref_b():
        ref.generate_probability_mask(rb, 0.3)

    rec_a, rec_b = hip.record(step_a), hip.record(step_b)
    for k, which in enumerate("aabababbba"):
        if which == "a":
            rec_a.replay()
            ref_a()
            assert_bit_equal(hip.get_numpy_copy(ma), ra, "replay %d (a): first mask" % k)
            assert_bit_equal(hip.get_numpy_copy(mc), rc, "replay %d (a): second mask" % k)
        else:
            rec_b.replay()
            ref_b()
            assert_bit_equal(hip.get_numpy_copy(mb), rb, "replay %d (b)" % k)
    rec_a.release()
    step_b()
    ref_b()
    assert_bit_equal(hip.get_numpy_copy(mb), rb, "eager step after one recording was released")
    rec_b.replay()
    ref_b()
    assert_bit_equal(hip.get_numpy_copy(mb), rb, "replay of the other recording afterwards")
    rec_b.release()
    _, key, pos, _, _ = hip.rnd.get_state()
    st = ref.rnd.get_state()
    assert pos == st[2]
    np.testing.assert_array_equal(key, st[1])


def test_recorded_training_steps_equal_eager_ones():
    from brainstorm_amd import HipHandler
    from brainstorm_amd.drivers import configs
    from brainstorm_amd.drivers.net import MomentumStepper

    def train(recorded, fused, builder=configs.build_mlp):
        h = HipHandler(seed=77)
        net, data = builder(h, fused=fused)
        net.provide_external_data(data)
        stepper = MomentumStepper(0.1, 0.9, fused=fused)
        stepper.start(net)
        stepper.run()
        losses = []
        for _ in range(6):
            if recorded:
                stepper.run_recorded()
            else:
                stepper.run()
            losses.append(float(net.get("loss", "outputs", "loss").sum()))
        params = h.get_numpy_copy(net.parameters)
        stepper.release_recorded()
        return losses, params

    for fused in (False, True):
        want_losses, want_params = train(False, fused)
        got_losses, got_params = train(True, fused)
        assert got_losses == want_losses, (fused, got_losses, want_losses)
        assert_bit_equal(got_params, want_params, "parameters after recorded steps (fused=%r)" % fused)
    # the convolutional workload: im2col / col2im, pooling and products with a bias epilogue inside the recording
    for fused in (False, True):
        want_losses, want_params = train(False, fused, configs.build_cnn)
        got_losses, got_params = train(True, fused, configs.build_cnn)
        assert got_losses == want_losses, (fused, got_losses, want_losses)
        assert_bit_equal(got_params, want_params,
                         "parameters after recorded steps of the convolutional workload (fused=%r)" % fused)


def test_graph_entry_points_report_misuse(hip):
    import ctypes
    lib = hip._lib
    gid = ctypes.c_int(-1)
    assert lib.bship_graph_end(ctypes.byref(gid)) != 0              # nothing is being recorded
    assert b"no step" in lib.bship_last_error()
    assert lib.bship_graph_launch(12345) != 0                       # unknown recording
    assert lib.bship_graph_destroy(12345) != 0
    assert lib.bship_graph_begin() == 0
    assert lib.bship_graph_begin() != 0                             # already recording
    assert lib.bship_graph_launch(1) != 0                           # not while recording
    a = hip.allocate((4, 4))
    hip.add_st(1.0, a, a)
    assert lib.bship_graph_end(ctypes.byref(gid)) == 0 and gid.value > 0
    assert lib.bship_graph_launch(gid.value) == 0
    assert lib.bship_graph_destroy(gid.value) == 0
    assert lib.bship_graph_destroy(gid.value) != 0                  # already destroyed
    assert lib.bship_graph_launch(gid.value) != 0
    assert_bit_equal(hip.get_numpy_copy(a), np.full((4, 4), 1.0, F32), "one replay of add_st")
    # an empty recording is refused, and the handler stays usable
    assert lib.bship_graph_begin() == 0
    status = lib.bship_graph_end(ctypes.byref(gid))
    if status == 0:
        assert lib.bship_graph_launch(gid.value) == 0
        assert lib.bship_graph_destroy(gid.value) == 0
    hip.add_st(1.0, a, a)
    assert_bit_equal(hip.get_numpy_copy(a), np.full((4, 4), 2.0, F32), "eager call after the recordings")
