"""CPU: the fusing window's matcher and its mapping to fused entry points, driven by the real
HipHandler and the real op-trace drivers over a host-only library that logs launches instead of
making them (tests/window_trace/trace_lib.cpp, built here with g++ from the library's own
window_core.h and window_sink.h).

The claim under test: a caller that issues primitive operations only (fused=False drivers, the
reference layers' sequences) gets, with the window on, exactly the launches that a handler-aware
caller asks for (fused=... drivers) with the window off - same entry points, same operands, same
order - and nothing but reordered matrix products otherwise.
"""
import numpy as np
import pytest


def canonical(log, base, size):
    """Addresses inside the network's buffer become offsets into it, every other address the number
    of its first appearance in the log; generator numbers are dropped."""
    seen = {}
    out = []
    for line in log:
        tokens = []
        for tok in line.split():
            if tok.startswith("@"):
                addr = int(tok[1:])
                if addr < 0:
                    tok = "@null"
                elif base <= addr < base + size:
                    tok = "@net+%d" % (addr - base)
                else:
                    tok = "@other%d" % seen.setdefault(addr, len(seen))
            elif tok[0] == "g" and tok[1:].lstrip("-").isdigit():
                tok = "g"
            tokens.append(tok)
        if tokens[:2] == ["bias_act", "3"]:
            # bias + 'linear' activation, which a handler-aware layer asks for, is the bias addition alone
            tokens = ["mv", "0"] + tokens[2:] + ["0", "0"]
        out.append(" ".join(tokens))
    return out


def run_step(trace, builder, fusing, fused, steps=1, **kw):
    """The launch log of `steps` training steps (after one untraced step) and the window's counters."""
    from brainstorm_amd import HipHandler
    from brainstorm_amd.drivers.net import MomentumStepper
    h = HipHandler(seed=3, fusing=fusing)
    net, data = builder(h, fused=fused, **kw) if fused is not None else builder(h, **kw)
    net.provide_external_data(data)
    stepper = MomentumStepper(0.1, 0.9, fused=bool(fused))
    stepper.start(net)
    stepper.run()
    base = net.full_buffer.ptr - 0x100000000
    trace.trace_reset()
    for _ in range(steps):
        stepper.run()
    log = canonical(trace.trace_log().decode().splitlines(), base, net.full_buffer.size * 4)
    stats = h.fusing_stats()
    del stepper, net
    return log, stats, base


def names(log):
    return [line.split()[0] for line in log]


def normalised(log, skip=()):
    return [line for line in log if line.split()[0] not in skip]


def test_mlp_unchanged_calls_become_the_fused_launches(trace):
    from brainstorm_amd.drivers import configs
    kw = dict(batch=5, in_size=7, hidden=6)
    plain, _, _ = run_step(trace, configs.build_mlp, fusing=False, fused=False, **kw)
    window, stats, _ = run_step(trace, configs.build_mlp, fusing=True, fused=False, **kw)
    aware, _, _ = run_step(trace, configs.build_mlp, fusing=False, fused=True, **kw)
    assert window == aware
    assert len(window) < len(plain)
    for name in ("dropout_fwd", "bias_act", "softmax_ce_fwd", "softmax_ce_bwd", "momentum"):
        assert name in names(window) and name not in names(plain)
    assert names(window).count("dropout_fwd") == 3 and names(window).count("bias_act") == 2
    assert stats["fused_launches"] == 3 + 2 + 1 + 1 + 1


def test_lstm_unchanged_calls_become_the_fused_launches(trace):
    from brainstorm_amd.drivers import configs
    kw = dict(time_steps=5, batch=3, symbols=4, hidden=6)
    plain, _, _ = run_step(trace, configs.build_lstm, fusing=False, fused=False, **kw)
    window, stats, _ = run_step(trace, configs.build_lstm, fusing=True, fused=False, **kw)
    aware, _, _ = run_step(trace, configs.build_lstm, fusing=False, fused="steps", **kw)
    assert window == aware
    assert names(window).count("lstm_fwd_step") == 5 and names(window).count("lstm_bwd_step") == 5
    assert stats["overtaken"] == 5 * 3           # the products of the input, forget and output gates
    # every launch of the unfused run that is not part of a time step's elementwise work is still there, in order
    keep = ("gemm", "d2d", "sum")
    assert [l for l in plain if l.split()[0] in keep] == [l for l in window if l.split()[0] in keep]


def test_highway_and_batchnorm_sequences_need_their_temporaries_freed(trace):
    from brainstorm_amd.drivers import configs
    kw = dict(blocks=2, batch=6, width=5)
    window, stats, _ = run_step(trace, configs.build_highway, fusing=True, fused=False, **kw)
    aware, _, _ = run_step(trace, configs.build_highway, fusing=False, fused=True, **kw)
    assert window == aware
    assert "SCALARS-DIFFER" not in "\n".join(window)
    got = names(window)
    for name, count in (("batchnorm_fwd", 2), ("batchnorm_bwd", 2), ("highway_fwd", 2), ("highway_bwd", 2),
                        ("bias_act", 4)):
        assert got.count(name) == count, name


def test_cnn_keeps_its_order(trace):
    from brainstorm_amd.drivers import configs
    kw = dict(batch=2, size=8)
    window, stats, _ = run_step(trace, configs.build_cnn, fusing=True, fused=False, **kw)
    aware, _, _ = run_step(trace, configs.build_cnn, fusing=False, fused=True, **kw)
    # the same launches; a product may have gone ahead of a held call that it shares nothing with (the
    # column sum of the bias gradient in the convolution's backward pass is held as a possible start of
    # a batch normalisation pass when the next product arrives)
    assert sorted(window) == sorted(aware)
    others = lambda log: [l for l in log if not l.startswith("gemm")]
    products = lambda log: [l for l in log if l.startswith("gemm")]
    assert others(window) == others(aware) and products(window) == products(aware)
    assert stats["overtaken"] >= 1


def test_a_sequence_cut_short_is_issued_as_it_was_called(trace):
    from brainstorm_amd import HipHandler
    h = HipHandler(seed=1, fusing=True)
    a, b, v, c = h.allocate((4, 6)), h.allocate((4, 6)), h.allocate((1, 6)), h.allocate((4, 6))
    trace.trace_reset()
    h.add_mv(a, v, a)                # could become bias + activation, or an LSTM step
    assert trace.trace_held() == 1
    h.tanh(a, b)                     # the LSTM step's second call (out of place)
    h.mult_add_mv(c, v, a)           # ... and its third
    assert trace.trace_held() == 3
    got = h.get_numpy_copy(a)        # reading back: everything held is issued first, in call order
    assert got.shape == (4, 6)
    log = trace.trace_log().decode().splitlines()
    assert names(log) == ["mv", "unary", "mv", "d2h"]
    # in place the same two calls are one fused launch
    trace.trace_reset()
    h.add_mv(a, v, a)
    h.tanh(a, a)
    assert trace.trace_held() == 0
    assert names(trace.trace_log().decode().splitlines()) == ["bias_act"]


def test_operands_that_share_memory_are_not_fused(trace):
    from brainstorm_amd import HipHandler
    h = HipHandler(seed=1, fusing=True)
    n = 8
    v, g, p = h.allocate((n,)), h.allocate((n,)), h.allocate((2 * n,))
    trace.trace_reset()
    # the momentum update with parameters that overlap the velocity: three separate launches
    h.mult_st(0.9, v, v)
    h.mult_add_st(-0.1, g, v)
    h.add_tt(v, v, v)
    assert names(trace.trace_log().decode().splitlines()) == ["scalar", "scalar", "binary"]
    trace.trace_reset()
    h.mult_st(0.9, v, v)
    h.mult_add_st(-0.1, g, v)
    h.add_tt(v, p[:n], p[:n])
    assert names(trace.trace_log().decode().splitlines()) == ["momentum"]


def test_highway_with_a_temporary_that_stays_alive_is_not_fused(trace):
    from brainstorm_amd import HipHandler
    h = HipHandler(seed=1, fusing=True)
    H, T, x, y = (h.allocate((3, 5)) for _ in range(4))
    tmp = h.zeros((3, 5))
    trace.trace_reset()
    h.subtract_tt(H, x, tmp)
    h.mult_tt(T, tmp, tmp)
    h.add_tt(tmp, x, y)
    assert trace.trace_held() == 3               # complete, waiting for the temporary
    h.fill(y, 0.0)                               # another call instead of the free
    log = names(trace.trace_log().decode().splitlines())
    assert log == ["binary", "binary", "binary", "fill"]
    trace.trace_reset()
    h.subtract_tt(H, x, tmp)
    h.mult_tt(T, tmp, tmp)
    h.add_tt(tmp, x, y)
    del tmp                                      # what the layer does when it returns
    assert names(trace.trace_log().decode().splitlines()) == ["highway_fwd"]


def test_products_that_touch_held_operands_do_not_overtake(trace):
    from brainstorm_amd import HipHandler
    h = HipHandler(seed=1, fusing=True)
    a, w, out, v = h.allocate((4, 6)), h.allocate((6, 6)), h.allocate((4, 6)), h.allocate((1, 6))
    trace.trace_reset()
    h.add_mv(a, v, a)                            # held
    h.dot_mm(a, w, out)                          # reads what the held call writes
    assert names(trace.trace_log().decode().splitlines()) == ["mv", "gemm"]
    trace.trace_reset()
    h.add_mv(a, v, a)                            # held
    h.dot_mm(out, w, out if False else h.allocate((4, 6)))     # the allocation enqueues what is held
    trace.trace_reset()
    b = h.allocate((4, 6))
    h.add_mv(a, v, a)
    h.dot_add_mm(out, w, b)                      # shares nothing with the held call: goes first
    h.tanh(a, a)
    assert names(trace.trace_log().decode().splitlines()) == ["gemm", "bias_act"]


def test_stacked_mode_runs_one_product_per_lstm_time_step(trace):
    from brainstorm_amd.drivers import configs
    T, B, n = 5, 3, 6
    kw = dict(time_steps=T, batch=B, symbols=4, hidden=n)
    plain, _, _ = run_step(trace, configs.build_lstm, fusing=True, fused=False, **kw)
    stacked, stats, _ = run_step(trace, configs.build_lstm, fusing="stacked", fused=False, **kw)
    got = names(stacked)
    assert got.count("lstm_fwd_step_packed") == T and got.count("lstm_bwd_step_packed") == T
    assert "lstm_fwd_step" not in got and "lstm_bwd_step" not in got
    # forward: the four recurrent products of a step are one product with 4n result columns
    fwd_products = [l.split() for l in stacked if l.startswith("gemm 0 1 %d %d %d " % (B, 4 * n, n))]
    assert len(fwd_products) == T
    # backward: the first step has no packed deltas to read (copy + four products), every later step one product over K = 4n
    bwd_products = [l.split() for l in stacked if l.startswith("gemm 0 0 %d %d %d " % (B, n, 4 * n))]
    assert len(bwd_products) == T - 1
    assert got.count("d2d") == 1
    # the packed copy that a backward step reads is the one the step before it wrote
    steps = [l.split() for l in stacked if l.startswith("lstm_bwd_step_packed")]
    assert steps[0][4] == "@null"                                # no deltas: dy was complete
    for before, product, after in zip(steps, bwd_products, steps[1:]):
        assert product[7] == before[6]                            # A of the product = packed_out of the step before
        assert after[4] != "@null" and after[6] != before[6]     # deltas added by the kernel, the other buffer written
    # everything that is not part of a time step is unchanged
    keep = ("sum", "softmax_ce_fwd", "softmax_ce_bwd", "momentum", "fill")
    same = lambda log: [l for l in log if l.split()[0] in keep and "@other" not in l]    # temporaries are numbered per run
    assert same(plain) == same(stacked) and len(same(plain)) > 10
    assert len([l for l in stacked if l.startswith("gemm")]) == len([l for l in plain if l.startswith("gemm")]) - 3 * T - 3 * (T - 1)


def test_stacked_mode_forgets_the_packed_deltas_when_something_else_runs(trace):
    # two backward steps with an unrelated call between them: the second one must form its four products itself
    from brainstorm_amd import HipHandler
    from brainstorm_amd.drivers import configs
    h = HipHandler(seed=1, fusing="stacked")
    net, data = configs.build_lstm(h, time_steps=3, batch=2, symbols=3, hidden=4)
    net.provide_external_data(data)
    net.forward_pass(training_pass=True)
    layer, buffers = net.layers["lstm"], net.buffers["lstm"]

    class Nosy(type(h)):
        """The same handler, poking an unrelated array after every backward time step."""
    other = h.allocate((4,))
    calls = {"n": 0}
    original = h.tanh_deriv

    def tanh_deriv(x, y, dy, dx):
        original(x, y, dy, dx)
        calls["n"] += 1
        if calls["n"] % 2 == 0:                  # the step's last call (the block input's derivative)
            h.fill(other, 3.0)
    h.tanh_deriv = tanh_deriv
    h.act_func_deriv["tanh"] = tanh_deriv
    trace.trace_reset()
    net.backward_pass()
    log = names(trace.trace_log().decode().splitlines())
    assert log.count("lstm_bwd_step_packed") == 3
    assert log.count("d2d") == 3                 # no step could use the packed copy of the one before
    h.set_fusing(True)
