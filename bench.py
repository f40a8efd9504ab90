#!/usr/bin/env python
"""Benchmark of the handler hot path on one MI355X.

A "step" is one pass of the handler-operation sweep (the operations named by
the op-sweep configuration: elementwise, activations and derivatives,
reductions, softmax, matrix-vector broadcasts, label indexing) over synthetic
float32 tensors that are already resident in HBM. The headline value is the
sweep's aggregate algorithmic throughput in GB/s: the sum over operations of
the minimum number of bytes each must move (bytes read + bytes written,
ALG_BYTES below) divided by the wall time of the step.

Prints ONE JSON line. Besides the required keys it carries
  roofline      for the kernel that takes the largest share of a step (two-input elementwise):
                algorithmic bytes / mean kernel time (HIP events on the library's
                stream, taken inside the timed steps) against 8 TB/s HBM peak
  cpu_baseline  the CPU oracle (NumpyHandler semantics, NumPy) timed on this
                machine's host cores on a bounded sample (the 4096x4096 sweep)
  ops           per-operation GB/s and fraction of peak

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--size S] [--no-cpu]
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
F32_MATRIX_PEAK_TFLOPS = 157.3   # MI355X dense float32 matrix cores, published
F32 = np.float32


# HBM bytes per launch at the default 16384x16384 workload, measured with
# `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` (two runs of this script) and scaled by what
# the same counters read for the sweep's 1 GiB copy_to (factors 2.000 and 0.999); the table and
# the commands are in profiles/op_sweep_2p28_hbm_traffic.md. MiB per launch.
MEASURED_TRAFFIC_MIB_2P28 = {
    "add_tt": 3071.3, "mult_tt": 3071.3, "divide_tt": 3071.3, "mult_add_st": 3071.3,
    "sigmoid_deriv": 3071.3, "tanh_deriv": 3071.3, "rel_deriv": 3071.3,
    "sigmoid": 2047.4, "tanh": 2047.4, "log_t": 2047.4, "rel": 2048.0, "clip_t": 2047.4,
    "sqrt_t": 2047.3, "copy_to": 2048.0, "fill": 1023.4, "softmax_m": 2050.4,
    "add_mv_row": 2047.4, "mult_mv_row": 2047.4, "add_mv_col": 2049.4, "mult_mv_col": 2049.6,
    "sum_t_axis0": 1024.8, "sum_t_axis1": 1024.5, "sum_t_all": 1024.1, "binarize_v": 1024.3,
}


def alg_bytes(rows, cols):
    """Minimum HBM traffic of each sweep operation on a (rows, cols) float32 tensor."""
    n = rows * cols
    return {
        "add_tt": 12 * n, "mult_tt": 12 * n, "divide_tt": 12 * n,
        "mult_add_st": 12 * n,
        "sigmoid": 8 * n, "tanh": 8 * n, "rel": 8 * n,
        "sigmoid_deriv": 12 * n, "tanh_deriv": 12 * n, "rel_deriv": 12 * n,
        "clip_t": 8 * n, "sqrt_t": 8 * n, "log_t": 8 * n,
        "sum_t_axis0": 4 * n + 4 * cols, "sum_t_axis1": 4 * n + 4 * rows, "sum_t_all": 4 * n + 4,
        "softmax_m": 8 * n,
        "add_mv_row": 8 * n + 4 * cols, "mult_mv_row": 8 * n + 4 * cols,
        "add_mv_col": 8 * n + 4 * rows, "mult_mv_col": 8 * n + 4 * rows,
        "binarize_v": 4 * n + 4 * rows,
        "index_m_by_v": 12 * rows,          # label + gathered element + result per row
        "copy_to": 8 * n, "fill": 4 * n,
    }


def sweep_ops(h, t):
    """(name, thunk) for every operation of the sweep on handler h and tensor set t."""
    return [
        ("add_tt", lambda: h.add_tt(t["a"], t["b"], t["out"])),
        ("mult_tt", lambda: h.mult_tt(t["a"], t["b"], t["out"])),
        ("divide_tt", lambda: h.divide_tt(t["a"], t["u"], t["out"])),
        ("mult_add_st", lambda: h.mult_add_st(0.5, t["a"], t["acc"])),
        ("sigmoid", lambda: h.sigmoid(t["a"], t["out"])),
        ("tanh", lambda: h.tanh(t["a"], t["out"])),
        ("rel", lambda: h.rel(t["a"], t["out"])),
        ("sigmoid_deriv", lambda: h.sigmoid_deriv(None, t["y"], t["b"], t["out"])),
        ("tanh_deriv", lambda: h.tanh_deriv(None, t["y"], t["b"], t["out"])),
        ("rel_deriv", lambda: h.rel_deriv(None, t["y"], t["b"], t["out"])),
        ("clip_t", lambda: h.clip_t(t["a"], -1.0, 1.0, t["out"])),
        ("sqrt_t", lambda: h.sqrt_t(t["u"], t["out"])),
        ("log_t", lambda: h.log_t(t["u"], t["out"])),
        ("sum_t_axis0", lambda: h.sum_t(t["a"], 0, t["row_out"])),
        ("sum_t_axis1", lambda: h.sum_t(t["a"], 1, t["col_out"])),
        ("sum_t_all", lambda: h.sum_t(t["a"], None, t["scalar_out"])),
        ("softmax_m", lambda: h.softmax_m(t["a"], t["out"])),
        ("add_mv_row", lambda: h.add_mv(t["a"], t["row"], t["out"])),
        ("mult_mv_row", lambda: h.mult_mv(t["a"], t["row"], t["out"])),
        ("add_mv_col", lambda: h.add_mv(t["a"], t["col"], t["out"])),
        ("mult_mv_col", lambda: h.mult_mv(t["a"], t["col"], t["out"])),
        ("binarize_v", lambda: h.binarize_v(t["labels"], t["out"])),
        ("index_m_by_v", lambda: h.index_m_by_v(t["a"], t["labels"], t["picked"])),
        ("copy_to", lambda: h.copy_to(t["a"], t["out"])),
        ("fill", lambda: h.fill(t["out"], 0.5)),
    ]


def host_tensors(size, seed=0):
    """The op-sweep inputs: N(0,1) tensors, U(0.1,10) denominators, integer labels; seed 0."""
    rng = np.random.RandomState(seed)
    shape = (size, size)
    t = {
        "a": rng.standard_normal(shape).astype(F32),
        "b": rng.standard_normal(shape).astype(F32),
        "u": rng.uniform(0.1, 10, shape).astype(F32),
        "row": rng.standard_normal((1, size)).astype(F32),
        "col": rng.standard_normal((size, 1)).astype(F32),
        "labels": rng.randint(0, size, (size, 1)).astype(F32),
    }
    t["y"] = np.tanh(t["b"])          # a plausible activation output for the derivatives
    return t


def add_outputs(h, t, size):
    t["out"] = h.allocate((size, size))
    t["acc"] = h.allocate((size, size))
    t["row_out"] = h.allocate((1, size))
    t["col_out"] = h.allocate((size, 1))
    t["scalar_out"] = h.allocate(())
    t["picked"] = h.allocate((size, 1))
    return t


def device_tensors(hip, size, base=4096):
    """Tensors of (size, size) on the device, tiled from the seeded (base, base) host inputs
    with the handler's own broadcast_t so that no multi-GiB host arrays are needed."""
    base = min(base, size)
    src = host_tensors(base)
    reps = (size * size) // (base * base)
    t = {}
    for name in ("a", "b", "u", "y"):
        small = hip.create_from_numpy(src[name].reshape(1, base * base))
        big = hip.allocate((reps, base * base))
        hip.broadcast_t(small, 0, big)
        t[name] = big.reshape((size, size))
    rng = np.random.RandomState(1)
    t["row"] = hip.create_from_numpy(rng.standard_normal((1, size)).astype(F32))
    t["col"] = hip.create_from_numpy(rng.standard_normal((size, 1)).astype(F32))
    t["labels"] = hip.create_from_numpy(rng.randint(0, size, (size, 1)).astype(F32))
    return add_outputs(hip, t, size)


def run_gpu(size, steps, warmup, hip=None):
    from brainstorm_amd import HipHandler
    hip = hip or HipHandler(seed=0)
    lib = hip._lib
    name, cus = hip.device_info()
    t = device_tensors(hip, size)
    ops = sweep_ops(hip, t)
    nops = len(ops)
    assert steps * (nops + 1) <= 1024, "too many steps for the event slots"
    for _ in range(warmup):
        for _, fn in ops:
            fn()
    hip.synchronize()
    t0 = time.perf_counter()
    slot = 0
    for _ in range(steps):
        # one event before every operation and one after the last: kernel times are read
        # after the timed region, nothing waits inside it
        for _, fn in ops:
            lib.bship_event_record(slot)
            slot += 1
            fn()
        lib.bship_event_record(slot)
        slot += 1
    hip.synchronize()
    elapsed = time.perf_counter() - t0
    ms = ctypes.c_float()
    per_op_ms = {n: [] for n, _ in ops}
    for s in range(steps):
        base = s * (nops + 1)
        for i, (n, _) in enumerate(ops):
            hip._call(lib.bship_event_elapsed_ms(base + i, base + i + 1, ctypes.byref(ms)))
            per_op_ms[n].append(ms.value)
    return hip, name, cus, elapsed, {n: float(np.mean(v)) for n, v in per_op_ms.items()}


def run_image_ops(hip, n_img=2048, reps=10):
    """The image operations (im2col/col2im of the convolutions, max/avg pooling) at the shapes of
    the CNN workload with a batch large enough to leave the caches: us per launch and the fraction
    of peak for the bytes each must move at least (inputs read once, outputs written once)."""
    lib = hip._lib
    ms = ctypes.c_float()

    def timed(fn):
        for _ in range(2):
            fn()
        lib.bship_event_record(0)
        for _ in range(reps):
            fn()
        lib.bship_event_record(1)
        hip._call(lib.bship_event_elapsed_ms(0, 1, ctypes.byref(ms)))
        return ms.value * 1e3 / reps

    def filled(shape, seed=[0]):
        # N(0,1) data (a seeded 4 MiB block repeated on the device): which pixel of a window is the
        # largest decides what the pooling kernels touch, so constant inputs would not be representative
        seed[0] += 1
        n, base = int(np.prod(shape)), 1 << 20
        src = hip.create_from_numpy(np.random.RandomState(seed[0]).standard_normal((1, base)).astype(F32))
        reps = (n + base - 1) // base
        big = hip.allocate((reps, base))
        hip.broadcast_t(src, 0, big)
        return big.reshape((reps * base,))[:n].reshape(shape)

    out = {}

    def report(name, us, nbytes):
        gbps = nbytes / us / 1e3
        out[name] = {"us": round(us, 1), "gbps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4)}

    for h, w, c, k, pad, tag in ((32, 32, 3, 5, 2, "conv1_32x32x3_k5"), (15, 15, 32, 5, 2, "conv2_15x15x32_k5")):
        x = filled((n_img, h, w, c))
        oh, ow = h + 2 * pad - k + 1, w + 2 * pad - k + 1
        col = hip.allocate((n_img * oh * ow, k * k * c))
        dx = hip.allocate((n_img, h, w, c))
        report("im2col_" + tag, timed(lambda: hip._call(lib.bship_im2col_nhwc_f32(
            x.ptr, col.ptr, n_img, h, w, c, k, k, pad, 1, 1))), 4 * (x.size + col.size))
        report("col2im_" + tag, timed(lambda: hip._call(lib.bship_col2im_nhwc_f32(
            col.ptr, dx.ptr, n_img, h, w, c, k, k, pad, 1, 1))), 4 * (2 * x.size + col.size))
        del col, dx, x
    # The CNN workload's first convolution (5 x 5 x 3 filters, 32 of them) forward and backward: without a col
    # matrix (thin filters: the handler's choice) and through im2col + the matrix-product library + col2im.
    # Matrix-core work: TFLOP/s of the 2 * pixels * 75 * 32 flops forward and twice that backward, and their
    # fraction of the float32 matrix peak.
    for batch, n_reps in ((n_img, reps), (100, 20 * reps)):
        x, dy = filled((batch, 32, 32, 3)), filled((batch, 32, 32, 32))
        wts, bias = filled((32, 5, 5, 3)), filled((32,))
        y, dx, dw, db = hip.allocate((batch, 32, 32, 32)), hip.allocate((batch, 32, 32, 3)), hip.allocate((32, 5, 5, 3)), hip.allocate((32,))
        flops = 2.0 * batch * 32 * 32 * 75 * 32
        for thin, route in ((True, "thin"), (False, "im2col")):
            hip.thin_convolutions = thin
            try:
                for name, work, fn in (("fwd", flops, lambda: hip.conv2d_forward_batch(x, wts, bias, y, 2, (1, 1))),
                                       ("bwd", 2 * flops, lambda: hip.conv2d_backward_batch(x, wts, 2, (1, 1), dx, dy, dw, db))):
                    for _ in range(2):
                        fn()
                    lib.bship_event_record(0)
                    for _ in range(n_reps):
                        fn()
                    lib.bship_event_record(1)
                    hip._call(lib.bship_event_elapsed_ms(0, 1, ctypes.byref(ms)))
                    us = ms.value * 1e3 / n_reps
                    out["conv1_%s_%s_batch%d" % (name, route, batch)] = {
                        "us": round(us, 1), "tflops": round(work / us / 1e6, 1),
                        "frac_of_f32_matrix_peak": round(work / us / 1e6 / F32_MATRIX_PEAK_TFLOPS, 4)}
            finally:
                hip.thin_convolutions = True
        del x, dy, y, dx
    for h, w, c, k, s, tag in ((32, 32, 32, 3, 2, "pool1_32x32x32_k3s2"), (15, 15, 64, 3, 2, "pool2_15x15x64_k3s2")):
        x = filled((n_img, h, w, c))
        oh, ow = (h - k) // s + 1, (w - k) // s + 1
        o, am, do = hip.allocate((n_img, oh, ow, c)), hip.allocate((n_img, oh, ow, c)), filled((n_img, oh, ow, c))
        dx = hip.allocate((n_img, h, w, c))
        report("maxpool_fwd_" + tag, timed(lambda: hip.maxpool2d_forward_batch(x, (k, k), o, 0, (s, s), am)),
               4 * (x.size + 2 * o.size))
        report("maxpool_bwd_" + tag, timed(lambda: hip.maxpool2d_backward_batch(x, (k, k), o, 0, (s, s), am, dx, do)),
               4 * (2 * x.size + 2 * o.size))
        report("avgpool_fwd_" + tag, timed(lambda: hip.avgpool2d_forward_batch(x, (k, k), o, 0, (s, s))),
               4 * (x.size + o.size))
        report("avgpool_bwd_" + tag, timed(lambda: hip.avgpool2d_backward_batch(x, (k, k), o, 0, (s, s), dx, do)),
               4 * (2 * x.size + o.size))
        del x, o, am, do, dx
    return out


def run_host_call_cost(hip, calls=20000):
    """What one handler call costs on the host, in us: `add_tt` on 100x1200 arrays issued back to back
    (a call no pattern of the fusing window begins with: it goes into the window and out again), with the
    window on and off, and for comparison the same entry point through ctypes alone."""
    lib = hip._lib
    a, b, o = hip.allocate((100, 1200)), hip.allocate((100, 1200)), hip.allocate((100, 1200))
    out = {"calls": calls, "arrays": "100x1200 float32"}

    def issue(fn):
        for _ in range(200):
            fn()
        hip.synchronize()
        t0 = time.perf_counter()
        for _ in range(calls):
            fn()
        dt = time.perf_counter() - t0
        hip.synchronize()
        return round(dt / calls * 1e6, 3)

    before = hip.fusing
    try:
        for on, tag in ((True, "window_on"), (False, "window_off")):
            hip.set_fusing(on)
            out["add_tt_%s_us" % tag] = issue(lambda: hip.add_tt(a, b, o))
        from brainstorm_amd._lib import ADD
        ap, bp, op, n = a.ptr, b.ptr, o.ptr, o.size
        out["bship_binary_f32_through_ctypes_us"] = issue(lambda: lib.bship_binary_f32(ADD, ap, bp, op, n))
    finally:
        hip.set_fusing(before)
    return out


def run_pitched_ops(rows=8192, cols=8192, reps=10):
    """Operations on row-pitched views: three (rows, cols) feature slices of one (rows, 3*cols) hub,
    as the layers writing side by side into a hub see them (buffer_structure.py:232-245). For each
    operation the fraction of peak with the row-pitched kernels and with the dense-temporaries path."""
    from brainstorm_amd import HipHandler
    hip = HipHandler(seed=0, pitched_views=True)
    lib = hip._lib
    ms = ctypes.c_float()
    hub = hip.allocate((rows, 3 * cols))
    hip.fill(hub, 0.25)
    a, b, o = hub[:, :cols], hub[:, cols:2 * cols], hub[:, 2 * cols:]
    row, col = hip.allocate((1, cols)), hip.allocate((rows, 1))
    n = rows * cols
    cases = [("add_tt", 12 * n, lambda: hip.add_tt(a, b, o)),
             ("tanh", 8 * n, lambda: hip.tanh(a, o)),
             ("mult_add_st", 12 * n, lambda: hip.mult_add_st(0.5, a, o)),
             ("add_mv_row", 8 * n, lambda: hip.add_mv(a, row, o)),
             ("mult_mv_col", 8 * n, lambda: hip.mult_mv(a, col, o)),
             ("sum_t_axis0", 4 * n, lambda: hip.sum_t(a, 0, row)),
             ("sum_t_axis1", 4 * n, lambda: hip.sum_t(a, 1, col)),
             ("copy_to", 8 * n, lambda: hip.copy_to(a, o)),
             ("generate_probability_mask", 4 * n, lambda: hip.generate_probability_mask(o, 0.5)),
             ("broadcast_t_rows", 4 * n, lambda: hip.broadcast_t(row, 0, o)),
             ("merge_tt", 8 * n, lambda: hip.merge_tt(a[:, :cols // 2], b[:, :cols // 2], o)),
             ("split_add_tt", 12 * n, lambda: hip.split_add_tt(o, a[:, :cols // 2], b[:, :cols // 2]))]
    # pooling on image slices: batch 2048 of 32x32x32 images and their 15x15x32 pooled outputs, each a
    # feature slice of a hub that is half as wide again (the image operations' own benchmark shapes)
    n_img, h, w, c, k, s = 2048, 32, 32, 32, 3, 2
    oh = (h - k) // s + 1
    fi, fo = h * w * c, oh * oh * c
    hub_in, hub_din = hip.allocate((n_img, fi + fi // 2)), hip.allocate((n_img, fi + fi // 2))
    hub_out, hub_arg, hub_dout = (hip.allocate((n_img, fo + fo // 2)) for _ in range(3))
    noise = hip.allocate((1, 1 << 22))            # N(0,1) values: which pixel wins decides what max pooling touches
    hip.fill_gaussian(0.0, 1.0, noise)
    hip.broadcast_t(noise, 0, hub_in.reshape((hub_in.size // (1 << 22), 1 << 22)))
    hip.copy_to(hub_in.reshape((hub_in.size,))[:hub_dout.size].reshape(hub_dout.shape), hub_dout)
    x, dx = (t[:, :fi].reshape((n_img, h, w, c)) for t in (hub_in, hub_din))
    y, am, dy = (t[:, :fo].reshape((n_img, oh, oh, c)) for t in (hub_out, hub_arg, hub_dout))
    ni, no = n_img * fi, n_img * fo
    cases += [("maxpool_fwd_32x32x32_k3s2", 4 * (ni + 2 * no), lambda: hip.maxpool2d_forward_batch(x, (k, k), y, 0, (s, s), am)),
              ("maxpool_bwd_32x32x32_k3s2", 4 * (2 * ni + 2 * no),
               lambda: hip.maxpool2d_backward_batch(x, (k, k), y, 0, (s, s), am, dx, dy)),
              ("avgpool_fwd_32x32x32_k3s2", 4 * (ni + no), lambda: hip.avgpool2d_forward_batch(x, (k, k), y, 0, (s, s))),
              ("avgpool_bwd_32x32x32_k3s2", 4 * (2 * ni + no),
               lambda: hip.avgpool2d_backward_batch(x, (k, k), y, 0, (s, s), dx, dy))]
    out = {}
    for native in (True, False):
        hip.native_pitched = native
        for name, nbytes, fn in cases:
            for _ in range(2):
                fn()
            lib.bship_event_record(0)
            for _ in range(reps):
                fn()
            lib.bship_event_record(1)
            hip._call(lib.bship_event_elapsed_ms(0, 1, ctypes.byref(ms)))
            gbps = nbytes / (ms.value / reps * 1e-3) / 1e9
            out.setdefault(name, {})["row_pitched_kernels" if native else "dense_temporaries"] = {
                "gbps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4)}
    hip.native_pitched = True
    return out


def time_net(handler, builder, steps, warmup, sync, recorded=False, fusing=None, **kw):
    """Training steps per second of one network workload (forward + backward + momentum update,
    inputs uploaded once; the per-step loss read-back of a Trainer is included). recorded: the
    step's handler calls are recorded once (after an ordinary step) and replayed with one launch.
    fusing: the handler's fusing window on or off for this run (None: as the handler is). The
    random stream is restarted first, so every variant of a network sees the same dropout masks;
    "loss" is the loss of the last step, which variants that promise the same bits must share."""
    from brainstorm_amd.drivers.net import MomentumStepper
    before = getattr(handler, "fusing", None)
    if fusing is not None:
        handler.set_fusing(fusing)
    if hasattr(handler.rnd, "seed"):
        handler.rnd.seed(0)
    net, data = builder(handler, **kw)
    net.provide_external_data(data)
    stepper = MomentumStepper(0.1, 0.9, fused=bool(kw.get("fused")))
    stepper.start(net)
    if recorded:
        stepper.run()
    step = stepper.run_recorded if recorded else stepper.run
    for _ in range(warmup - (1 if recorded else 0)):
        step()
        net.get("loss", "outputs", "loss")
    sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
        loss = net.get("loss", "outputs", "loss")      # device-to-host copy + wait, as trainer.py:100 does
    sync()
    dt = (time.perf_counter() - t0) / steps
    if recorded:
        stepper.release_recorded()
    if fusing is not None:
        handler.set_fusing(before)
    samples = data["default"].shape[0] * data["default"].shape[1]
    return {"ms_per_step": round(dt * 1e3, 3), "samples_per_s": round(samples / dt, 1),
            "loss": float(np.asarray(loss).ravel()[0])}


def time_net_fast_masks(builder, steps, warmup):
    from brainstorm_amd import HipHandler
    handler = HipHandler(seed=0, fast_masks=True)
    return time_net(handler, builder, steps, warmup, handler.synchronize, recorded=True, fused=True)


def same_bits(nets, names):
    """The variants `names` of one network promise the same bits: their last losses must be one number
    (a timing of a path that computes something else is not a timing of that network)."""
    losses = {n: nets[n]["loss"] for n in names}
    if len({np.float32(v).tobytes() for v in losses.values()}) != 1 or not all(np.isfinite(v) for v in losses.values()):
        raise AssertionError("variants that must agree bit for bit do not: %r" % losses)


def close_to(nets, name, reference, rel):
    a, b = nets[name]["loss"], nets[reference]["loss"]
    if not (np.isfinite(a) and abs(a - b) <= rel * abs(b)):
        raise AssertionError("%s: loss %r is not within %g of %s's %r" % (name, a, rel, reference, b))


def run_nets_gpu(hip):
    """Step times of the four network workloads. The first line of each group is what an UNCHANGED caller
    gets: the reference layers' primitive call sequences (fused=False drivers) on the default handler, whose
    fusing window turns them into the fused kernels (same bits). "_window_off": the same calls launched
    one by one. "_fused...": a handler-aware caller that asks for the fused entry points itself."""
    from brainstorm_amd.drivers import configs
    mlp, lstm, cnn, hw = ("mlp_784-1200-1200-10_batch100", "lstm_205-1000-205_T100_batch100", "cnn_32x32x3_batch100",
                          "highway_bn_50x4096_batch2048")
    sync = hip.synchronize
    nets = {
        mlp: time_net(hip, configs.build_mlp, 600, 20, sync, fusing=True),
        mlp + "_window_off": time_net(hip, configs.build_mlp, 600, 20, sync, fusing=False),
        # dropout, bias + activation, softmax cross entropy and the update through the fused entry points
        mlp + "_fused": time_net(hip, configs.build_mlp, 600, 20, sync, fused=True),
        # the step recorded into a HIP graph and replayed
        mlp + "_recorded": time_net(hip, configs.build_mlp, 600, 20, sync, recorded=True),
        mlp + "_fused_recorded": time_net(hip, configs.build_mlp, 600, 20, sync, recorded=True, fused=True),
        # NOT the reference's masks: dropout masks from the optional counter-based generator
        # (HipHandler(fast_masks=True)), one parallel launch per mask instead of the MT19937 walk
        mlp + "_fused_recorded_fast_masks": time_net_fast_masks(configs.build_mlp, 600, 20),
        lstm: time_net(hip, configs.build_lstm, 5, 2, sync, fusing=True),
        lstm + "_window_off": time_net(hip, configs.build_lstm, 5, 2, sync, fusing=False),
        # the same unchanged caller with the window also stacking the four recurrent products of a time step
        # into one (HipHandler(fusing="stacked")): another summation order inside the products, not the same bits
        lstm + "_window_stacked": time_net(hip, configs.build_lstm, 5, 2, sync, fusing="stacked"),
        # the ~4000 launches of a step (window off) recorded into a HIP graph and replayed
        lstm + "_window_off_recorded": time_net(hip, configs.build_lstm, 5, 2, sync, recorded=True, fusing=False),
        # the elementwise part of each time step in one launch, asked for by the layer
        lstm + "_fused_steps": time_net(hip, configs.build_lstm, 5, 2, sync, fused=True),
        # ... and the four recurrent matrix products of a step as one over the stacked matrices
        lstm + "_fused_packed": time_net(hip, configs.build_lstm, 5, 2, sync, fused="packed"),
        # ... with the backward recurrent product through the thin-operand kernel (dot_small_tn)
        lstm + "_fused_thin": time_net(hip, configs.build_lstm, 5, 2, sync, fused="thin"),
        # ... and the whole forward recurrence as one persistent launch (weights resident in LDS, one grid
        # barrier per time step); the backward pass is the packed one
        lstm + "_fused_sequence": time_net(hip, configs.build_lstm, 5, 2, sync, fused="sequence"),
        # the convolutional workload (conv 5x5x32, max pool 3x3/2, conv 5x5x64, max pool, 1000, 10)
        cnn: time_net(hip, configs.build_cnn, 200, 10, sync, fusing=True),
        cnn + "_window_off": time_net(hip, configs.build_cnn, 200, 10, sync, fusing=False),
        cnn + "_recorded": time_net(hip, configs.build_cnn, 200, 10, sync, recorded=True),
        cnn + "_fused": time_net(hip, configs.build_cnn, 200, 10, sync, fused=True),
        cnn + "_fused_recorded": time_net(hip, configs.build_cnn, 200, 10, sync, recorded=True, fused=True),
        # the bandwidth-stress workload: 50 Highway + batch normalisation blocks of width 4096
        hw: time_net(hip, configs.build_highway, 3, 1, sync, fusing=True),
        hw + "_window_off": time_net(hip, configs.build_highway, 3, 1, sync, fusing=False),
        hw + "_fused": time_net(hip, configs.build_highway, 3, 1, sync, fused=True),
    }
    # a timing of a broken path must fail: same-bits variants share their last loss, the others are close to it
    same_bits(nets, [mlp, mlp + "_window_off", mlp + "_fused", mlp + "_recorded", mlp + "_fused_recorded"])
    same_bits(nets, [lstm, lstm + "_window_off", lstm + "_window_off_recorded", lstm + "_fused_steps"])
    for variant in ("_window_stacked", "_fused_packed", "_fused_thin", "_fused_sequence"):      # other summation orders in the products
        close_to(nets, lstm + variant, lstm, 1e-4)
    same_bits(nets, [cnn, cnn + "_window_off", cnn + "_recorded", cnn + "_fused", cnn + "_fused_recorded"])
    same_bits(nets, [hw, hw + "_window_off", hw + "_fused"])
    return nets


def run_nets_cpu(ref):
    from brainstorm_amd.drivers import configs
    return {
        "mlp_784-1200-1200-10_batch100": time_net(ref, configs.build_mlp, 10, 1, lambda: None),
        "lstm_205-1000-205_T100_batch100": time_net(ref, configs.build_lstm, 1, 0, lambda: None),
    }


def run_cpu(size, budget_s):
    """Times the CPU oracle on the (size, size) sweep: whole passes until ~budget_s is spent."""
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from oracle.numpy_ref_handler import NumpyRefHandler
    ref = NumpyRefHandler(F32, seed=0)
    t = add_outputs(ref, host_tensors(size), size)
    ops = sweep_ops(ref, t)
    for _, fn in ops[:2]:
        fn()                                   # touch the output pages once
    per_op = {n: [] for n, _ in ops}
    passes = 0
    start = time.perf_counter()
    while passes < 1 or (time.perf_counter() - start < budget_s and passes < 20):
        for n, fn in ops:
            t0 = time.perf_counter()
            fn()
            per_op[n].append(time.perf_counter() - t0)
        passes += 1
    return passes, {n: float(np.median(v)) for n, v in per_op.items()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=16384, help="tensors are size x size float32")
    ap.add_argument("--cpu-size", type=int, default=4096)
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-nets", action="store_true", help="skip the MLP/LSTM samples/s runs")
    ap.add_argument("--no-image-ops", action="store_true", help="skip the im2col/col2im/pooling measurements")
    ap.add_argument("--no-pitched", action="store_true", help="skip the operations on row-pitched views")
    ap.add_argument("--no-2p26", action="store_true",
                    help="skip the second, untimed-for-the-metric pass of the sweep on 8192x8192 tensors")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the handler path has no multi-GPU part "
                 "(got --gpus %d); run it with --gpus 1" % args.gpus)
    if args.size % 4096 and args.size > 4096:
        sys.exit("--size must be a multiple of 4096")

    hip, dev_name, cus, elapsed, op_ms = run_gpu(args.size, args.steps, args.warmup)
    ab = alg_bytes(args.size, args.size)
    total_bytes = sum(ab[n] for n in op_ms)
    ms_per_step = elapsed / args.steps * 1e3
    value = total_bytes / (elapsed / args.steps) / 1e9
    ops = {}
    for n, ms in op_ms.items():
        gbps = ab[n] / (ms * 1e-3) / 1e9
        ops[n] = {"ms": round(ms, 4), "gbps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4)}
    # the two-input elementwise kernel (12 bytes per element) takes the largest share of a step; its
    # instances (add_tt, mult_tt, ..., the derivatives) run within 1 % of each other, so the first of
    # them in sweep order stands for the kernel instead of whichever happened to be slowest this run
    most_bytes = max(ab[n] for n in op_ms)
    dominant = next(n for n in op_ms if ab[n] == most_bytes)
    roofline = {
        "kernel": dominant, "bound": "hbm",
        "achieved": ops[dominant]["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": ops[dominant]["frac"],
        "traffic": (int(MEASURED_TRAFFIC_MIB_2P28[dominant] * 2 ** 20)
                    if args.size == 16384 and dominant in MEASURED_TRAFFIC_MIB_2P28 else None),
        "alg_bytes_per_launch": ab[dominant], "ms_per_launch": ops[dominant]["ms"],
    }
    # the graded kernel furthest below the roofline in the timed sweep (index_m_by_v is a latency-bound gather
    # of one element per row and is reported in microseconds, not graded against the bandwidth)
    lowest = min((n for n in ops if n != "index_m_by_v"), key=lambda n: ops[n]["frac"])
    roofline["lowest"] = {"kernel": lowest, "frac": ops[lowest]["frac"]}
    out = {
        "metric": "handler-op HBM GB/s", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "handler op sweep (%d operations) on float32 %dx%d tensors (2^%d "
                               "elements each), inputs resident in HBM"
                               % (len(op_ms), args.size, args.size,
                                  int(round(np.log2(args.size * args.size)))),
                   "device": dev_name, "compute_units": cus},
        "roofline": roofline,
    }
    if not args.no_2p26 and args.size != 8192:
        # the same sweep at 2^26 elements per tensor, the smallest size the throughput targets are
        # quoted at (launch overheads and two-stage reductions weigh four times more there)
        _, _, _, _, small_ms = run_gpu(8192, args.steps, args.warmup, hip)
        sab = alg_bytes(8192, 8192)
        out["ops_2p26"] = {n: {"ms": round(ms, 4), "gbps": round(sab[n] / (ms * 1e-3) / 1e9, 1),
                               "frac": round(sab[n] / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
                           for n, ms in small_ms.items()}
    if not args.no_image_ops:
        out["image_ops"] = run_image_ops(hip)
    if not args.no_pitched:
        out["pitched_ops"] = run_pitched_ops()
    if "ops_2p26" in out or "pitched_ops" in out:
        out["note_256mb_tensors"] = ("ops_2p26 and pitched_ops work on 8192x8192 tensors: an output of 256 MB fits the "
                                     "last-level cache, which takes the kernels' write-through stores, so their frac "
                                     "(algorithmic bytes per second over the HBM peak) is not HBM traffic and can pass "
                                     "what HBM alone delivers; value and roofline are measured on 1 GB tensors, where "
                                     "it cannot")
    if not args.no_nets:
        # second part of the metric: training samples/s of the MLP and LSTM workloads
        out["nets"] = run_nets_gpu(hip)
        out["host_call_cost"] = run_host_call_cost(hip)
    if not args.no_cpu:
        passes, cpu_s = run_cpu(args.cpu_size, args.cpu_seconds)
        cab = alg_bytes(args.cpu_size, args.cpu_size)
        cpu_total = sum(cpu_s.values())
        out["cpu_baseline"] = {
            "value": round(sum(cab[n] for n in cpu_s) / cpu_total / 1e9, 3), "unit": "GB/s",
            "cores": 1, "kind": "port",
            "sample": "%d passes of the same %d-operation sweep on %dx%d float32 tensors with the "
                      "NumPy oracle (median per operation; NumPy elementwise and reduction "
                      "routines run on one core); host has %d cores, numpy %s"
                      % (passes, len(cpu_s), args.cpu_size, args.cpu_size, os.cpu_count(), np.__version__),
            "ops_gbps": {n: round(cab[n] / s / 1e9, 3) for n, s in cpu_s.items()},
        }
        if not args.no_nets:
            from oracle.numpy_ref_handler import NumpyRefHandler
            out["cpu_baseline"]["nets"] = run_nets_cpu(NumpyRefHandler(F32, seed=0))
    # the per-operation tables go last, the headline sweep's at the very end, so that a reader who keeps
    # only the end of the line still has the figures the headline value is made of
    for key in ("image_ops", "pitched_ops", "note_256mb_tensors", "ops_2p26"):
        if key in out:
            out[key] = out.pop(key)
    out["ops"] = ops
    print(json.dumps(out))


if __name__ == "__main__":
    main()
