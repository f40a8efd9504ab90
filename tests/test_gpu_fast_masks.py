"""The optional fast mask stream (Philox4x32-10): the device masks are exactly what oracle/philox.py
computes from (seed, block counter), calls and replays advance the counter, and the fused dropout
uses the same masks. This stream is NOT NumpyHandler's; the default handler keeps that one."""
import numpy as np
import pytest

from util import assert_bit_equal

pytestmark = pytest.mark.gpu
F32 = np.float32


def test_fast_masks_match_the_oracle_generator():
    from brainstorm_amd import HipHandler
    from oracle import philox
    hip = HipHandler(seed=4711, fast_masks=True)
    assert hip.fast_mask_state() == (4711, 0)
    offset = 0
    flat = hip.allocate((70000,))
    for shape, p in [((100, 1200), 0.8), ((3, 5), 0.5), ((1,), 0.2), ((37, 1031), 0.5), ((4096, 1024), 0.65),
                     ((7,), 1.0), ((9,), 0.0), ((2, 3, 5), 0.9)]:
        m = hip.allocate(shape)
        hip.generate_probability_mask(m, p)
        want, blocks = philox.probability_mask(int(np.prod(shape)), p, 4711, offset)
        assert_bit_equal(hip.get_numpy_copy(m), want.reshape(shape), "fast mask %r p=%r" % (shape, p))
        offset += blocks
        assert hip.fast_mask_state() == (4711, offset)
    for start, n in [(1, 13), (3, 4097), (2, 64)]:          # views that are only 4-byte aligned
        view = flat[start:start + n]
        hip.generate_probability_mask(view, 0.5)
        want, blocks = philox.probability_mask(n, 0.5, 4711, offset)
        assert_bit_equal(hip.get_numpy_copy(view), want, "fast mask of an unaligned view")
        offset += blocks
    # fused dropout: the same mask, out = scale * (in * mask)
    x = np.random.RandomState(1).standard_normal((100, 1201)).astype(F32)
    xd, md, yd = hip.create_from_numpy(x), hip.allocate(x.shape), hip.allocate(x.shape)
    hip.dropout_forward(xd, 0.7, 1.25, md, yd)
    want, blocks = philox.probability_mask(x.size, 0.7, 4711, offset)
    want = want.reshape(x.shape)
    assert_bit_equal(hip.get_numpy_copy(md), want, "fused dropout mask")
    assert_bit_equal(hip.get_numpy_copy(yd), F32(1.25) * (x * want), "fused dropout output")
    offset += blocks
    # a recorded step draws fresh masks on every replay
    a, b = hip.allocate((100, 300)), hip.allocate((50, 7))

    def step():
        hip.generate_probability_mask(a, 0.5)
        hip.generate_probability_mask(b, 0.8)

    rec = hip.record(step)
    for replay in range(3):
        rec.replay()
        wa, ba = philox.probability_mask(a.size, 0.5, 4711, offset)
        wb, bb = philox.probability_mask(b.size, 0.8, 4711, offset + ba)
        assert_bit_equal(hip.get_numpy_copy(a), wa.reshape(a.shape), "replay %d, first mask" % replay)
        assert_bit_equal(hip.get_numpy_copy(b), wb.reshape(b.shape), "replay %d, second mask" % replay)
        offset += ba + bb
    rec.release()
    assert hip.fast_mask_state() == (4711, offset)
    # the gaussian stream is still NumPy's
    g = hip.allocate((33,))
    hip.fill_gaussian(0.0, 1.0, g)
    assert_bit_equal(hip.get_numpy_copy(g), np.random.RandomState(4711).standard_normal(33).astype(F32), "fill_gaussian")
    # re-seeding the handler's random state restarts the mask stream too
    hip.rnd.seed(99)
    assert hip.fast_mask_state() == (99, 0)
    hip.generate_probability_mask(a, 0.5)
    wa, _ = philox.probability_mask(a.size, 0.5, 99, 0)
    assert_bit_equal(hip.get_numpy_copy(a), wa.reshape(a.shape), "mask after re-seeding")


def test_default_handler_keeps_numpys_stream():
    from brainstorm_amd import HipHandler
    hip = HipHandler(seed=5)
    m = hip.allocate((50, 40))
    hip.generate_probability_mask(m, 0.5)
    want = (np.random.RandomState(5).uniform(size=(50, 40)) < 0.5).astype(F32)
    assert_bit_equal(hip.get_numpy_copy(m), want, "default mask stream")


def test_mlp_trains_with_fast_masks():
    from brainstorm_amd import HipHandler
    from brainstorm_amd.drivers import configs
    from brainstorm_amd.drivers.net import MomentumStepper
    runs = []
    for recorded in (False, True):
        h = HipHandler(seed=3, fast_masks=True)
        net, data = configs.build_mlp(h, fused=True)
        net.provide_external_data(data)
        stepper = MomentumStepper(0.1, 0.9)
        stepper.start(net)
        stepper.run()
        losses = []
        for _ in range(8):
            (stepper.run_recorded if recorded else stepper.run)()
            losses.append(float(net.get("loss", "outputs", "loss").sum()))
        stepper.release_recorded()
        runs.append(losses)
    assert runs[0] == runs[1]                      # recorded and eager steps see the same masks
    assert runs[0][-1] < runs[0][0]                # and the network learns
