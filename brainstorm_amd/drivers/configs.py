"""The four network workloads of the benchmark configurations, on synthetic data.

Each builder returns ``(net, data)`` for a given handler: the network (op-trace
drivers, see layers.py) with seeded parameters already uploaded, and the
dictionary of seeded NumPy inputs to hand to ``net.provide_external_data``.
Everything is derived from ``numpy.random.RandomState(seed)`` in a fixed order,
so two handlers built with the same arguments see identical inputs and weights.

  mlp      784-1200-1200-10, ReLU, dropout 0.2 / 0.5 / 0.5, softmax cross entropy
           (shape of examples/mnist_pi.py:28-37); batch 100
  lstm     one peephole LSTM layer (1000 units, tanh) -> FullyConnected(205) ->
           softmax cross entropy on one-hot sequences over 205 symbols
           (examples/hutter_lstm.py:31-36); T=100, batch 100
  highway  N x {BatchNorm -> FC_H(rel) || FC_T(sigmoid) -> Highway}, width 4096,
           batch 2048, then FC(10) -> softmax cross entropy
  cnn      conv5x5x32 ReLU -> maxpool 3x3/2 -> conv5x5x64 ReLU -> maxpool 3x3/2 ->
           FC1000 ReLU -> FC10 -> softmax cross entropy on 32x32x3 images
           (examples/cifar10_cnn.py:28-41); batch 100
"""
from __future__ import annotations

import numpy as np

from .layers import (BatchNorm, Convolution2D, Dropout, FullyConnected, Highway, Input, Loss, Lstm,
                     Pooling2D, SoftmaxCE)
from .net import Net

F32 = np.float32


def _init_parameters(net, rng, std, special=None, quick=None):
    """Gaussian weights, zero biases; `special` maps a parameter-name suffix to a constant.

    `quick(layer_name)` -> None or an int: weights of layers for which it returns an int are drawn
    from a float32 PCG64 stream seeded with that int instead of `rng`, several layers at a time on
    host threads (what makes a 1.7 G-parameter network quick to set up; RandomState's float64
    polar method is sequential and takes minutes for it).
    """
    flat = np.zeros(net.parameter_count(), dtype=F32)
    jobs = []
    for name, (a, b, shape) in net.parameter_slices().items():
        layer, leaf = name.split(".")
        if special and leaf in special:
            flat[a:b] = special[leaf]
        elif len(shape) >= 2:
            stream = quick(layer) if quick else None
            if stream is None:
                flat[a:b] = (rng.standard_normal(b - a) * std).astype(F32)
            else:
                jobs.append((stream, a, b))
        # 1-D parameters (biases) stay zero

    def draw(job):
        stream, a, b = job
        np.random.Generator(np.random.PCG64(stream)).standard_normal(out=flat[a:b], dtype=F32)
        flat[a:b] *= F32(std)

    if jobs:
        import concurrent.futures
        with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
            list(pool.map(draw, jobs))
    return flat


def _finish(net, data, flat):
    first = data[next(iter(data))]
    net.resize(first.shape[0], first.shape[1])
    net.set_parameters(flat)
    return net, data


def build_mlp(handler, seed=1, batch=100, in_size=784, hidden=1200, classes=10, fused=False):
    rng = np.random.RandomState(seed)
    data = {"default": rng.uniform(0, 1, (1, batch, in_size)).astype(F32),
            "targets": rng.randint(0, classes, (1, batch, 1)).astype(F32)}
    net = Net(handler, [
        ("Input", Input({"default": (in_size,), "targets": (1,)}), {}),
        ("drop1", Dropout(0.2, fused=fused), {"default": "Input.default"}),
        ("fc1", FullyConnected(hidden, "rel", fused=fused), {"default": "drop1.default"}),
        ("drop2", Dropout(0.5, fused=fused), {"default": "fc1.default"}),
        ("fc2", FullyConnected(hidden, "rel", fused=fused), {"default": "drop2.default"}),
        ("drop3", Dropout(0.5, fused=fused), {"default": "fc2.default"}),
        ("out", FullyConnected(classes, "linear", fused=fused), {"default": "drop3.default"}),
        ("ce", SoftmaxCE(fused=fused), {"default": "out.default", "targets": "Input.targets"}),
        ("loss", Loss(), {"default": "ce.loss"}),
    ])
    return _finish(net, data, _init_parameters(net, rng, 0.01))


def build_lstm(handler, seed=2, time_steps=100, batch=100, symbols=205, hidden=1000, fused=False):
    rng = np.random.RandomState(seed)
    ids = rng.randint(0, symbols, (time_steps, batch, 1))
    onehot = np.zeros((time_steps, batch, symbols), dtype=F32)     # like data_iterators.OneHot
    np.put_along_axis(onehot, ids, 1.0, axis=2)
    data = {"default": onehot, "targets": ids.astype(F32)}
    net = Net(handler, [
        ("Input", Input({"default": (symbols,), "targets": (1,)}), {}),
        ("lstm", Lstm(hidden, "tanh", fused=fused), {"default": "Input.default"}),
        ("out", FullyConnected(symbols, "linear", fused=bool(fused)), {"default": "lstm.default"}),
        ("ce", SoftmaxCE(fused=bool(fused)), {"default": "out.default", "targets": "Input.targets"}),
        ("loss", Loss(), {"default": "ce.loss"}),
    ])
    return _finish(net, data, _init_parameters(net, rng, 0.05))


def build_highway(handler, seed=3, blocks=50, batch=2048, width=4096, classes=10, fused=False,
                  quick_init_from_block=None, parameters=None):
    """quick_init_from_block: blocks from this index on (and the output layer) take their weights
    from per-layer PCG64 streams (see _init_parameters), so the first blocks of a deep network have
    the weights of the shallow network with the same seed. parameters: a flat float32 vector to
    use instead of drawing one."""
    rng = np.random.RandomState(seed)
    data = {"default": rng.standard_normal((1, batch, width)).astype(F32),
            "targets": rng.randint(0, classes, (1, batch, 1)).astype(F32)}
    layers = [("Input", Input({"default": (width,), "targets": (1,)}), {})]
    prev = "Input.default"
    for k in range(blocks):
        layers += [
            ("bn%d" % k, BatchNorm(fused=fused), {"default": prev}),
            ("H%d" % k, FullyConnected(width, "rel", fused=fused), {"default": "bn%d.default" % k}),
            ("T%d" % k, FullyConnected(width, "sigmoid", fused=fused), {"default": "bn%d.default" % k}),
            ("hw%d" % k, Highway(fused=fused), {"H": "H%d.default" % k, "T": "T%d.default" % k,
                                     "x": "bn%d.default" % k}),
        ]
        prev = "hw%d.default" % k
    layers += [
        ("out", FullyConnected(classes, "linear", fused=fused), {"default": prev}),
        ("ce", SoftmaxCE(fused=fused), {"default": "out.default", "targets": "Input.targets"}),
        ("loss", Loss(), {"default": "ce.loss"}),
    ]
    net = Net(handler, layers)
    if parameters is not None:
        return _finish(net, data, parameters)

    def quick(layer):
        if quick_init_from_block is None:
            return None
        if layer == "out":
            return 1000 * seed + 999
        block = int(layer[1:])                       # "H12", "T12"
        return None if block < quick_init_from_block else 1000 * seed + 2 * block + (layer[0] == "T")

    flat = _init_parameters(net, rng, 1.0 / np.sqrt(width), special={"gamma": 1.0, "sigma": 1.0}, quick=quick)
    return _finish(net, data, flat)


def build_cnn(handler, seed=4, batch=100, size=32, classes=10, fused=False):
    rng = np.random.RandomState(seed)
    data = {"default": rng.standard_normal((1, batch, size, size, 3)).astype(F32),
            "targets": rng.randint(0, classes, (1, batch, 1)).astype(F32)}
    net = Net(handler, [
        ("Input", Input({"default": (size, size, 3), "targets": (1,)}), {}),
        ("conv1", Convolution2D(32, (5, 5), padding=2, activation="rel"), {"default": "Input.default"}),
        ("pool1", Pooling2D("max", (3, 3), stride=(2, 2)), {"default": "conv1.default"}),
        ("conv2", Convolution2D(64, (5, 5), padding=2, activation="rel"), {"default": "pool1.default"}),
        ("pool2", Pooling2D("max", (3, 3), stride=(2, 2)), {"default": "conv2.default"}),
        ("fc", FullyConnected(1000, "rel", fused=fused), {"default": "pool2.default"}),
        ("out", FullyConnected(classes, "linear", fused=fused), {"default": "fc.default"}),
        ("ce", SoftmaxCE(fused=fused), {"default": "out.default", "targets": "Input.targets"}),
        ("loss", Loss(), {"default": "ce.loss"}),
    ])
    return _finish(net, data, _init_parameters(net, rng, 0.05))
