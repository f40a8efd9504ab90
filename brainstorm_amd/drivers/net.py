"""A minimal network runner for the op-trace drivers.

It reproduces what brainstorm's Network and BufferManager do AROUND the layer
passes, as far as handler calls are concerned (structure/network.py:381-445,
structure/buffers.py:69-150, training/steppers.py:83-114):

  * one flat ``handler.allocate((total,))`` sliced and reshaped into every
    buffer (parameters and gradients are contiguous flat vectors);
  * ``provide_external_data`` = ``set_from_numpy`` into the Input layer's outputs;
  * forward: clear the context slots (``fill`` of ``buf[T - context:]``), then
    the layers in order;
  * backward: ``fill(…, 0)`` of every backward-only buffer (deltas, gradients,
    backward-only internals), then the layers in reverse;
  * MomentumStepper: ``mult_st``, ``mult_add_st``, ``add_tt`` on the flat vectors.

It is not a re-implementation of brainstorm's graph/layout compiler: layers are
given in execution order with explicit connections.
"""
from __future__ import annotations

from collections import OrderedDict

import numpy as np

from .layers import Buf, Input, _prod


class BufferNamespace:
    """The seven groups of views a layer pass receives."""

    def __init__(self):
        self.inputs = OrderedDict()
        self.outputs = OrderedDict()
        self.parameters = OrderedDict()
        self.gradients = OrderedDict()
        self.internals = OrderedDict()
        self.input_deltas = OrderedDict()
        self.output_deltas = OrderedDict()


class Net:
    """layers: list of (name, layer, connections) in execution order; connections maps an input
    name of the layer to "source_layer.output_name". The first layer must be an Input."""

    def __init__(self, handler, layers):
        self.handler = handler
        self.layers = OrderedDict()
        self.connections = {}
        self.specs = {}            # layer name -> (outputs, parameters, internals)
        for name, layer, conn in layers:
            layer.handler = handler
            in_shapes = {}
            for in_name, src in conn.items():
                src_layer, src_out = src.split(".")
                in_shapes[in_name] = self.specs[src_layer][0][src_out]
            self.specs[name] = layer.setup(in_shapes)
            self.layers[name] = layer
            self.connections[name] = conn
        assert isinstance(next(iter(self.layers.values())), Input)
        self.time_size = self.batch_size = None
        self.full_buffer = None
        self.buffers = None
        self.parameters = self.gradients = None
        self._backward_only = []
        self._with_context = []

    # ---------------------------------------------------------------- layout
    def _layout(self, time_size, batch_size):
        """[(key, shape, backward_only, context)], parameters first, then gradients."""
        items = []
        for name, (_, params, _) in self.specs.items():
            for p, shape in params.items():
                items.append((("param", name, p), tuple(shape), False, 0))
        n_params = len(items)
        for key, shape, _, _ in list(items[:n_params]):
            items.append((("grad",) + key[1:], shape, True, 0))
        rest = []
        for name, (outputs, _, internals) in self.specs.items():
            for o, buf in outputs.items():
                rest.append((("out", name, o), buf.shape(time_size, batch_size), False, buf.context))
                rest.append((("delta", name, o), buf.shape(time_size, batch_size), True, buf.context))
            for i, buf in internals.items():
                rest.append((("internal", name, i), buf.shape(time_size, batch_size), buf.backward_only,
                             buf.context if buf.scales == "TB" else 0))
        # the backward-only buffers lie together, behind the gradients, so that one fill clears them all
        # (the reference sorts its buffers into hubs by kind as well, structure/layout.py, and clears
        # each backward-only hub with one fill, structure/buffers.py:147-150)
        items += [it for it in rest if it[2]] + [it for it in rest if not it[2]]
        return items

    def resize(self, time_size, batch_size):
        if (time_size, batch_size) == (self.time_size, self.batch_size):
            return
        old_params = None
        if self.parameters is not None:
            old_params = self.handler.get_numpy_copy(self.parameters)
        items = self._layout(time_size, batch_size)
        total = sum(_prod(shape) for _, shape, _, _ in items)
        self.full_buffer = self.handler.allocate((total,))
        views, offset = {}, 0
        self._backward_only, self._with_context = [], []
        runs = []                                  # [first, end) of adjacent backward-only buffers
        for key, shape, backward_only, context in items:
            n = _prod(shape)
            view = self.full_buffer[offset:offset + n].reshape(shape)
            views[key] = view
            if backward_only and n:
                if runs and runs[-1][1] == offset:
                    runs[-1][1] = offset + n
                else:
                    runs.append([offset, offset + n])
            if context:
                self._with_context.append((view, context))
            offset += n
        n_param = sum(_prod(s) for k, s, _, _ in items if k[0] == "param")
        self.parameters = self.full_buffer[0:n_param]
        self.gradients = self.full_buffer[n_param:2 * n_param]
        self._backward_only = [self.full_buffer[first:end] for first, end in runs]
        self.time_size, self.batch_size = time_size, batch_size
        self.buffers = OrderedDict()
        for name, (outputs, params, internals) in self.specs.items():
            b = BufferNamespace()
            for p in params:
                b.parameters[p] = views[("param", name, p)]
                b.gradients[p] = views[("grad", name, p)]
            for o in outputs:
                b.outputs[o] = views[("out", name, o)]
                b.output_deltas[o] = views[("delta", name, o)]
            for i in internals:
                b.internals[i] = views[("internal", name, i)]
            for in_name, src in self.connections[name].items():
                src_layer, src_out = src.split(".")
                src_view = views[("out", src_layer, src_out)]
                src_delta = views[("delta", src_layer, src_out)]
                if self.specs[src_layer][0][src_out].context:
                    # a sink sees the time steps only, not the source's context slots
                    # (structure/buffer_structure.py:238-243)
                    src_view, src_delta = src_view[:time_size], src_delta[:time_size]
                b.inputs[in_name] = src_view
                b.input_deltas[in_name] = src_delta
            self.buffers[name] = b
        if old_params is not None:
            self.handler.set_from_numpy(self.parameters, old_params)

    # --------------------------------------------------------------- running
    def set_parameters(self, flat):
        self.handler.set_from_numpy(self.parameters, np.asarray(flat).reshape(self.parameters.shape))

    def provide_external_data(self, data):
        first = data[next(iter(data))]
        self.resize(first.shape[0], first.shape[1])
        input_name = next(iter(self.layers))
        for name, buf in self.buffers[input_name].outputs.items():
            if isinstance(data[name], self.handler.array_type):
                self.handler.copy_to(data[name], buf)
            else:
                self.handler.set_from_numpy(buf, data[name])

    def forward_pass(self, training_pass=False):
        for buf, context in self._with_context:           # BufferManager.clear_context
            self.handler.fill(buf[self.time_size - context:], 0.)
        for name, layer in list(self.layers.items())[1:]:
            layer.forward_pass(self.buffers[name], training_pass)

    def backward_pass(self):
        for buf in self._backward_only:                    # BufferManager.clear_backward_buffers
            self.handler.fill(buf, 0.)
        for name, layer in reversed(list(self.layers.items())[1:]):
            layer.backward_pass(self.buffers[name])
        self.apply_gradient_modifiers()                    # network.py:445

    def apply_weight_modifiers(self):
        """After every update (network.py:490-495): ``weight_modifiers`` maps (layer, parameter) to a list of
        callables ``hook(handler, view)``."""
        for (layer, view), hooks in getattr(self, "weight_modifiers", {}).items():
            for hook in hooks:
                hook(self.handler, self.buffers[layer].parameters[view])

    def apply_gradient_modifiers(self):
        """At the end of the backward pass (network.py:497-509): ``gradient_modifiers`` maps (layer, parameter)
        to a list of callables ``hook(handler, parameters, gradients)``."""
        for (layer, view), hooks in getattr(self, "gradient_modifiers", {}).items():
            for hook in hooks:
                hook(self.handler, self.buffers[layer].parameters[view], self.buffers[layer].gradients[view])

    def get(self, layer, group, name):
        return self.handler.get_numpy_copy(getattr(self.buffers[layer], group)[name])

    def parameter_count(self):
        return sum(_prod(s) for _, params, _ in self.specs.values() for s in params.values())

    def parameter_slices(self):
        """name -> (start, stop, shape) of every parameter in the flat vector."""
        out, offset = OrderedDict(), 0
        for name, (_, params, _) in self.specs.items():
            for p, shape in params.items():
                out[name + "." + p] = (offset, offset + _prod(shape), tuple(shape))
                offset += _prod(shape)
        return out


class MomentumStepper:
    """training/steppers.py:83-114"""

    def __init__(self, learning_rate=0.1, momentum=0.0, scale_learning_rate=True, fused=False):
        self.learning_rate = learning_rate
        self.momentum = momentum
        self.scale_learning_rate = scale_learning_rate
        self.fused = bool(fused)      # the three update operations through the handler's momentum_update (same bits)
        self.net = None
        self.velocity = None

    def start(self, net):
        self.net = net
        self.velocity = net.handler.zeros(net.parameters.shape)

    def run(self):
        learning_rate = self.learning_rate
        momentum = self.momentum
        if self.scale_learning_rate:
            learning_rate *= (1 - momentum)
        self.net.forward_pass(training_pass=True)
        self.net.backward_pass()
        h = self.net.handler
        if self.fused and hasattr(h, "momentum_update"):
            h.momentum_update(momentum, -learning_rate, self.net.gradients, self.velocity, self.net.parameters)
        else:
            h.mult_st(momentum, self.velocity, out=self.velocity)
            h.mult_add_st(-learning_rate, self.net.gradients, out=self.velocity)
            h.add_tt(self.velocity, self.net.parameters, out=self.net.parameters)
        self.net.apply_weight_modifiers()                  # the trainer does this after every update (trainer.py:101)

    def run_recorded(self):
        """The same step through a recording: the first call records ``run`` with the handler's
        ``record`` (the network must have done at least one ordinary step before, so that nothing is
        set up lazily inside the recording) and replays it; later calls only replay. Input data has
        to be in place in the network's buffers (``provide_external_data``) before each call, and
        the batch shape must not change."""
        if getattr(self, "_recorded", None) is None:
            self._recorded = self.net.handler.record(self.run)
        self._recorded.replay()

    def release_recorded(self):
        if getattr(self, "_recorded", None) is not None:
            self._recorded.release()
            self._recorded = None
