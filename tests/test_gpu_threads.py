"""GPU: handlers driven from different Python threads. Every random call names its generator and the
library selects and draws under one lock, so two handlers with different seeds each reproduce their own
numpy.random.RandomState stream whatever the interleaving (every reference handler owns its `rnd`,
numpy_handler.py:21)."""
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.mark.parametrize("fusing", [True, False])
def test_two_handlers_on_two_threads_keep_their_own_streams(hip, fusing):
    from brainstorm_amd import HipHandler
    before = hip.fusing
    handlers = [HipHandler(seed=101, fusing=fusing), HipHandler(seed=202, fusing=fusing)]
    failures = []
    start = threading.Barrier(2)

    def work(h, seed):
        try:
            rs = np.random.RandomState(seed)
            x = np.arange(37 * 11, dtype=F32).reshape(37, 11)
            xd = h.create_from_numpy(x)
            start.wait()
            for k in range(150):
                p = 0.2 + 0.6 * ((k * 7) % 10) / 10.0
                mask, out = h.allocate((37, 11)), h.allocate((37, 11))
                # a dropout layer's three calls (dropout_layer.py:41-45): with the fusing window on they become one launch
                h.generate_probability_mask(mask, p)
                h.mult_tt(xd, mask, out)
                h.mult_st(2.0, out, out)
                want = (rs.uniform(size=(37, 11)) < p).astype(F32)
                got = h.get_numpy_copy(mask)
                if not np.array_equal(got, want):
                    failures.append("seed %d draw %d: mask differs" % (seed, k))
                    return
                if not np.array_equal(h.get_numpy_copy(out), F32(2.0) * (x * want)):
                    failures.append("seed %d draw %d: product differs" % (seed, k))
                    return
                if k % 50 == 49:
                    g = h.allocate((5, 3))
                    h.fill_gaussian(0.5, 2.0, g)
                    np.testing.assert_allclose(h.get_numpy_copy(g), (rs.standard_normal((5, 3)) * 2.0 + 0.5).astype(F32),
                                               rtol=1e-6)
        except Exception as exc:                      # noqa: BLE001 - reported by the main thread
            failures.append("seed %d: %r" % (seed, exc))

    threads = [threading.Thread(target=work, args=(h, s)) for h, s in zip(handlers, (101, 202))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
    hip.set_fusing(before)
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not failures, failures
