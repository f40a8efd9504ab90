"""Op-trace drivers: the handler-call sequences of the brainstorm layers that
the benchmark configurations use.

brainstorm's layers contain no arithmetic of their own; each forward or
backward pass is a fixed sequence of handler calls on views of the network's
buffers. The classes below issue the same calls, in the same order, on views
of the same shapes as the reference layers, so that a handler can be driven --
and compared with the CPU oracle -- exactly the way brainstorm drives it. They
are callers of the handler, not part of it: they work with any object that
implements the handler interface (HipHandler, or the NumPy oracle in tests).

Each class names the reference file and lines whose sequence it reproduces,
including its quirks (they are part of the observable behaviour):
  - backward passes ADD into input deltas (several sinks share one buffer),
    while FullyConnected/Convolution gradients are overwritten;
  - Dropout's backward does not rescale by 1/(1-p);
  - BatchNorm stores the NEGATIVE running mean and centres with add_mv;
  - Lstm reads time step t-1 = -1 (the context slot) at t = 0, relies on
    ``allocate`` returning zeros, and adds the same dCa[-1]*dIa[0] term to both
    the input-gate and the forget-gate peephole gradients.
"""
from __future__ import annotations

from collections import OrderedDict


def _prod(shape):
    n = 1
    for s in shape:
        n *= int(s)
    return n


# brainstorm/utils.py:150-170 -- reshapes only, the views alias their parents
def flatten_time(a):
    return a.reshape((a.shape[0] * a.shape[1],) + tuple(a.shape[2:]))


def flatten_time_and_features(a):
    return a.reshape((a.shape[0] * a.shape[1], _prod(a.shape[2:])))


def flatten_all_but_last(a):
    return a.reshape((_prod(a.shape[:-1]), a.shape[-1]))


class Buf:
    """Description of one buffer of a layer: per-sample feature shape, whether it scales with
    time and batch ('TB'), extra context time steps, and whether only the backward pass uses it."""

    def __init__(self, feature_shape, scales="TB", context=0, backward_only=False):
        self.feature_shape = tuple(int(s) for s in feature_shape)
        self.scales = scales
        self.context = context
        self.backward_only = backward_only

    def shape(self, time_size, batch_size):
        if self.scales == "TB":
            return (time_size + self.context, batch_size) + self.feature_shape
        return self.feature_shape


class Layer:
    """setup(in_shapes) -> (outputs, parameters, internals), each an OrderedDict name -> Buf
    (parameters: name -> shape tuple). forward_pass / backward_pass receive a namespace with
    .inputs .outputs .parameters .gradients .internals .input_deltas .output_deltas, each an
    OrderedDict of views (like brainstorm's BufferView, structure/buffer_views.py)."""

    handler = None

    def setup(self, in_shapes):
        raise NotImplementedError

    def forward_pass(self, buffers, training_pass=True):
        raise NotImplementedError

    def backward_pass(self, buffers):
        raise NotImplementedError


class Input(Layer):
    """layers/input_layer.py: only provides the external data as outputs."""

    def __init__(self, out_shapes):
        self.out_shapes = out_shapes

    def setup(self, in_shapes):
        outputs = OrderedDict((name, Buf(shape)) for name, shape in self.out_shapes.items())
        return outputs, OrderedDict(), OrderedDict()

    def forward_pass(self, buffers, training_pass=True):
        pass

    def backward_pass(self, buffers):
        pass


class FullyConnected(Layer):
    """layers/fully_connected_layer.py:52-78"""

    def __init__(self, size, activation="rel", fused=False):
        self.size = int(size)
        self.activation = activation
        self.fused = bool(fused)        # bias + activation through handler.bias_act when it exists

    def setup(self, in_shapes):
        in_size = _prod(in_shapes["default"].feature_shape)
        outputs = OrderedDict(default=Buf((self.size,)))
        parameters = OrderedDict([("W", (self.size, in_size)), ("bias", (self.size,))])
        return outputs, parameters, OrderedDict()

    def forward_pass(self, buffers, training_pass=True):
        _h = self.handler
        W, bias = buffers.parameters["W"], buffers.parameters["bias"]
        inputs = flatten_time_and_features(buffers.inputs["default"])
        outputs = flatten_time_and_features(buffers.outputs["default"])
        _h.dot_mm(inputs, W, outputs, transb=True)
        if self.fused and hasattr(_h, "bias_act"):
            _h.bias_act(self.activation, outputs, bias, outputs)
            return
        _h.add_mv(outputs, bias.reshape((1, bias.shape[0])), outputs)
        _h.inplace_act_func[self.activation](outputs)

    def backward_pass(self, buffers):
        _h = self.handler
        W = buffers.parameters["W"]
        dW, dbias = buffers.gradients["W"], buffers.gradients["bias"]
        inputs = flatten_time_and_features(buffers.inputs["default"])
        outputs = flatten_time_and_features(buffers.outputs["default"])
        in_deltas = flatten_time_and_features(buffers.input_deltas["default"])
        out_deltas = flatten_time_and_features(buffers.output_deltas["default"])
        _h.inplace_act_func_deriv[self.activation](outputs, out_deltas)
        _h.dot_add_mm(out_deltas, W, out=in_deltas)
        _h.dot_mm(out_deltas, inputs, out=dW, transa=True)
        _h.sum_t(out_deltas, axis=0, out=dbias)


class Dropout(Layer):
    """layers/dropout_layer.py:36-52"""

    def __init__(self, drop_prob=0.5, fused=False):
        self.drop_prob = drop_prob
        self.fused = bool(fused)        # mask, product and scaling through handler.dropout_forward

    def setup(self, in_shapes):
        shape = in_shapes["default"].feature_shape
        return OrderedDict(default=Buf(shape)), OrderedDict(), OrderedDict(mask=Buf(shape))

    def forward_pass(self, buffers, training_pass=True):
        _h = self.handler
        if training_pass and self.fused and hasattr(_h, "dropout_forward"):
            _h.dropout_forward(buffers.inputs["default"], 1 - self.drop_prob, 1 / (1 - self.drop_prob),
                               buffers.internals["mask"], buffers.outputs["default"])
        elif training_pass:
            _h.generate_probability_mask(buffers.internals["mask"], 1 - self.drop_prob)
            _h.mult_tt(buffers.inputs["default"], buffers.internals["mask"], out=buffers.outputs["default"])
            _h.mult_st(1 / (1 - self.drop_prob), buffers.outputs["default"], out=buffers.outputs["default"])
        else:
            _h.copy_to(buffers.inputs["default"], buffers.outputs["default"])

    def backward_pass(self, buffers):
        self.handler.mult_add_tt(buffers.output_deltas["default"], buffers.internals["mask"],
                                 buffers.input_deltas["default"])


class SoftmaxCE(Layer):
    """layers/softmax_ce_layer.py:65-114; inputs 'default' and integer 'targets' (..., 1)."""

    def __init__(self, fused=False):
        # fused: use the handler's softmax_ce_forward / softmax_ce_backward when it has them (same bits)
        self.fused = bool(fused)

    def setup(self, in_shapes):
        in_shape = in_shapes["default"].feature_shape
        tar_shape = in_shapes["targets"].feature_shape
        assert tar_shape[-1] == 1 and tar_shape[:-1] == in_shape[:-1]
        outputs = OrderedDict([("predictions", Buf(in_shape)), ("loss", Buf(tar_shape))])
        internals = OrderedDict(t_bin=Buf(in_shape, backward_only=True))
        return outputs, OrderedDict(), internals

    def forward_pass(self, buffers, training_pass=True):
        _h = self.handler
        loss = buffers.outputs["loss"]
        flat_inputs = flatten_all_but_last(buffers.inputs["default"])
        flat_probs = flatten_all_but_last(buffers.outputs["predictions"])
        flat_loss = flatten_all_but_last(loss)
        flat_targets = flatten_all_but_last(buffers.inputs["targets"])
        if self.fused and hasattr(_h, "softmax_ce_forward"):
            _h.softmax_ce_forward(flat_inputs, flat_targets, flat_probs, flat_loss)
            return
        _h.softmax_m(flat_inputs, flat_probs)
        # cross entropy with index targets: -ln(p[target])
        _h.fill(loss, 0.)
        _h.index_m_by_v(flat_probs, flat_targets, flat_loss)
        _h.clip_t(flat_loss, 1e-6, 1.0, flat_loss)
        _h.log_t(loss, loss)
        _h.mult_st(-1, loss, loss)

    def backward_pass(self, buffers):
        _h = self.handler
        flat_probs = flatten_all_but_last(buffers.outputs["predictions"])
        flat_targets = flatten_all_but_last(buffers.inputs["targets"])
        flat_t_bin = flatten_all_but_last(buffers.internals["t_bin"])
        flat_dloss = flatten_all_but_last(buffers.output_deltas["loss"])
        flat_dinputs = flatten_all_but_last(buffers.input_deltas["default"])
        # d loss / d input = (softmax - onehot) * dloss
        if self.fused and hasattr(_h, "softmax_ce_backward"):
            _h.softmax_ce_backward(flat_probs, flat_targets, flat_dloss, flat_t_bin, flat_dinputs)
            return
        _h.binarize_v(flat_targets, flat_t_bin)
        _h.mult_st(-1, flat_t_bin, flat_t_bin)
        _h.add_tt(flat_t_bin, flat_probs, flat_t_bin)
        _h.mult_mv(flat_t_bin, flat_dloss, flat_t_bin)
        _h.add_tt(flat_t_bin, flat_dinputs, flat_dinputs)


class Loss(Layer):
    """layers/loss_layer.py:38-58: sums its input into one number, scaled by importance/batch."""

    def __init__(self, importance=1.0):
        self.importance = importance

    def setup(self, in_shapes):
        return OrderedDict(loss=Buf((1,), scales="")), OrderedDict(), OrderedDict()

    def forward_pass(self, buffers, training_pass=True):
        batch_size = buffers.inputs["default"].shape[1]
        self.handler.sum_t(buffers.inputs["default"], None, buffers.outputs["loss"].reshape(tuple()))
        self.handler.mult_st(self.importance / batch_size, buffers.outputs["loss"], buffers.outputs["loss"])

    def backward_pass(self, buffers):
        batch_size = buffers.inputs["default"].shape[1]
        self.handler.add_st(self.importance / batch_size, buffers.input_deltas["default"],
                            buffers.input_deltas["default"])


class Lstm(Layer):
    """layers/lstm_layer.py:27-278 (peephole LSTM, full back-propagation through time)."""

    PARAMS = ("Wz", "Wi", "Wf", "Wo", "pi", "pf", "po", "Rz", "Ri", "Rf", "Ro", "bz", "bi", "bf", "bo")
    INTERNALS = ("Za", "Zb", "Ia", "Ib", "Fa", "Fb", "Oa", "Ob", "Ca", "Cb")

    def __init__(self, size, activation="tanh", fused=False):
        self.size = int(size)
        self.activation = activation
        # fused="steps" (or True): the elementwise part of each time step goes through the
        # handler's lstm_forward_step / lstm_backward_step (one launch each, same bits) when it
        # has them. fused="packed": additionally the four recurrent products of a step become
        # one product over the stacked matrices [Rz;Ri;Rf;Ro] (same values up to the summation
        # order inside the matrix product). fused="sequence": as "packed", and the whole forward
        # recurrence is one launch of the handler's lstm_forward_sequence when it has one and the
        # shape fits it. fused="thin": as "sequence", and for batches of at most 128 rows the backward
        # recurrent product goes through the handler's dot_small_tn (a product kernel for a thin left
        # operand kept transposed, its K range cut into partial products that the step kernel adds).
        self.fused = "steps" if fused is True else (fused or False)
        assert self.fused in (False, "steps", "packed", "sequence", "thin")

    def _use_fused(self):
        return bool(self.fused) and hasattr(self.handler, "lstm_forward_step")

    def _stacked_recurrent(self, Rz, Ri, Rf, Ro):
        if self.fused not in ("packed", "sequence", "thin") or not hasattr(self.handler, "stack_adjacent"):
            return None
        return self.handler.stack_adjacent([Rz, Ri, Rf, Ro])

    def setup(self, in_shapes):
        in_size = _prod(in_shapes["default"].feature_shape)
        n = self.size
        outputs = OrderedDict(default=Buf((n,), context=1))
        shapes = {"W": (n, in_size), "p": (1, n), "R": (n, n), "b": (n,)}
        parameters = OrderedDict((name, shapes[name[0]]) for name in self.PARAMS)
        internals = OrderedDict()
        for name in self.INTERNALS:
            internals[name] = Buf((n,), context=1)
        for name in self.INTERNALS:
            internals["d" + name] = Buf((n,), context=1, backward_only=True)
        return outputs, parameters, internals

    def forward_pass(self, buffers, training_pass=True):
        _h = self.handler
        n = self.size
        (Wz, Wi, Wf, Wo, pi, pf, po, Rz, Ri, Rf, Ro, bz, bi, bf, bo) = buffers.parameters.values()
        (Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb) = list(buffers.internals.values())[:10]
        x = buffers.inputs["default"]
        y = buffers.outputs["default"]
        time_size = x.shape[0]

        flat_x = flatten_time_and_features(x)
        _h.dot_mm(flat_x, Wz, flatten_time(Za[:-1]), transb=True)
        _h.dot_mm(flat_x, Wi, flatten_time(Ia[:-1]), transb=True)
        _h.dot_mm(flat_x, Wf, flatten_time(Fa[:-1]), transb=True)
        _h.dot_mm(flat_x, Wo, flatten_time(Oa[:-1]), transb=True)

        R_all = self._stacked_recurrent(Rz, Ri, Rf, Ro)
        if (R_all is not None and self.fused in ("sequence", "thin") and hasattr(_h, "lstm_forward_sequence")
                and Za.shape[0] == time_size + 1):
            try:
                if _h.lstm_forward_sequence(self.activation, R_all, Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb, y,
                                            pi, pf, po, bz, bi, bf, bo):
                    return
            except RuntimeError as err:
                # the workgroups did not meet at a time step's barrier within the kernel's bound (other work
                # kept some of them off the device): every workgroup has left, the buffers hold an unfinished
                # pass. The kernel accumulates in place, so the input products are formed again, then the
                # step-by-step path below runs the recurrence.
                if getattr(err, "status", None) != getattr(_h, "ERR_TIMEOUT", None):
                    raise
                self.sequence_fallbacks = getattr(self, "sequence_fallbacks", 0) + 1
                _h.dot_mm(flat_x, Wz, flatten_time(Za[:-1]), transb=True)
                _h.dot_mm(flat_x, Wi, flatten_time(Ia[:-1]), transb=True)
                _h.dot_mm(flat_x, Wf, flatten_time(Fa[:-1]), transb=True)
                _h.dot_mm(flat_x, Wo, flatten_time(Oa[:-1]), transb=True)
        if R_all is not None:
            rec = _h.allocate((x.shape[1], 4 * n))
            for t in range(time_size):
                _h.dot_mm(y[t - 1], R_all, rec, transb=True)
                _h.lstm_forward_step_packed(self.activation, rec, Za[t], Zb[t], Ia[t], Ib[t], Fa[t],
                                            Fb[t], Oa[t], Ob[t], Ca[t], Cb[t], Ca[t - 1], y[t],
                                            pi, pf, po, bz, bi, bf, bo)
            return
        if self._use_fused():
            for t in range(time_size):
                y_prev = y[t - 1]
                _h.dot_add_mm(y_prev, Rz, Za[t], transb=True)
                _h.dot_add_mm(y_prev, Ri, Ia[t], transb=True)
                _h.dot_add_mm(y_prev, Rf, Fa[t], transb=True)
                _h.dot_add_mm(y_prev, Ro, Oa[t], transb=True)
                _h.lstm_forward_step(self.activation, Za[t], Zb[t], Ia[t], Ib[t], Fa[t], Fb[t],
                                     Oa[t], Ob[t], Ca[t], Cb[t], Ca[t - 1], y[t],
                                     pi, pf, po, bz, bi, bf, bo)
            return

        for t in range(time_size):
            # block input
            _h.dot_add_mm(y[t - 1], Rz, Za[t], transb=True)
            _h.add_mv(Za[t], bz.reshape((1, n)), Za[t])
            _h.act_func[self.activation](Za[t], Zb[t])
            # input gate
            _h.dot_add_mm(y[t - 1], Ri, Ia[t], transb=True)
            _h.mult_add_mv(Ca[t - 1], pi, Ia[t])
            _h.add_mv(Ia[t], bi.reshape((1, n)), Ia[t])
            _h.sigmoid(Ia[t], Ib[t])
            # forget gate
            _h.dot_add_mm(y[t - 1], Rf, Fa[t], transb=True)
            _h.mult_add_mv(Ca[t - 1], pf, Fa[t])
            _h.add_mv(Fa[t], bf.reshape((1, n)), Fa[t])
            _h.sigmoid(Fa[t], Fb[t])
            # cell
            _h.mult_tt(Ib[t], Zb[t], Ca[t])
            _h.mult_add_tt(Fb[t], Ca[t - 1], Ca[t])
            # output gate
            _h.dot_add_mm(y[t - 1], Ro, Oa[t], transb=True)
            _h.mult_add_mv(Ca[t], po, Oa[t])
            _h.add_mv(Oa[t], bo.reshape((1, n)), Oa[t])
            _h.sigmoid(Oa[t], Ob[t])
            # block output
            _h.act_func[self.activation](Ca[t], Cb[t])
            _h.mult_tt(Ob[t], Cb[t], y[t])

    def backward_pass(self, buffers):
        _h = self.handler
        (Wz, Wi, Wf, Wo, pi, pf, po, Rz, Ri, Rf, Ro, bz, bi, bf, bo) = buffers.parameters.values()
        (dWz, dWi, dWf, dWo, dpi, dpf, dpo, dRz, dRi, dRf, dRo, dbz, dbi, dbf, dbo) = \
            buffers.gradients.values()
        (Za, Zb, Ia, Ib, Fa, Fb, Oa, Ob, Ca, Cb,
         dZa, dZb, dIa, dIb, dFa, dFb, dOa, dOb, dCa, dCb) = buffers.internals.values()
        x = buffers.inputs["default"]
        dx = buffers.input_deltas["default"]
        y = buffers.outputs["default"]
        deltas = buffers.output_deltas["default"]

        # arbitrary content where the handler can allocate that: every time step of dy is written before
        # it is read; dy[-1], the slot behind the last step, is read below without ever being written
        empty = getattr(_h, "empty", _h.allocate)
        dy = empty(y.shape)
        _h.fill(dy[-1], 0.0)
        _h.fill(dCa, 0.0)
        time_size = x.shape[0]
        fused = self._use_fused()
        R_all = self._stacked_recurrent(Rz, Ri, Rf, Ro)
        batch = x.shape[1]
        packed_all = None
        thin = R_all is not None and self.fused == "thin" and hasattr(_h, "dot_small_tn") and batch <= 128
        if thin:
            # the same, transposed ((4n, 128), columns beyond the batch stay zero), and the partial
            # products of as many K ranges as fill the device with workgroups of 64 rows x 32 columns
            n = self.size
            packed_t = [_h.allocate((4 * n, 128)) for _ in range(2)]
            groups = -(-n // 32) * (2 if batch > 64 else 1)
            splits = max(1, min(8, _h.device_info()[1] // groups))
            parts = _h.allocate((splits, batch, n) if splits > 1 else (batch, n))
        elif R_all is not None:
            # [dZa|dIa|dFa|dOa] of the step after the current one; zero beyond the end. When the input
            # weights, their gradients, the recurrent gradients and the bias gradients are stacked in
            # memory like R_all, the packed deltas of all steps are kept and the products and sums over
            # time below become one each instead of one per gate (same terms, summed in the order of
            # one product instead of four); otherwise two buffers alternate.
            stacks = [_h.stack_adjacent(list(group)) for group in
                      ((Wz, Wi, Wf, Wo), (dWz, dWi, dWf, dWo), (dRz, dRi, dRf, dRo), (dbz, dbi, dbf, dbo))]
            if all(a is not None for a in stacks):
                W_all, dW_all, dR_all, db_all = stacks
                packed_all = empty((time_size + 1, batch, 4 * self.size))
                _h.fill(packed_all[time_size], 0.0)
                packed = None
            else:
                packed = [_h.allocate((x.shape[1], 4 * self.size)) for _ in range(2)]
        # the backward product packed[t+1] . R_all reads the weights against their rows; with a handler
        # that can transpose, it is given R_all^T and transb instead (same product; on MI355X the
        # library's kernel for that layout takes 16 us per step instead of 20)
        R_all_t = None
        if R_all is not None and not thin and hasattr(_h, "transpose"):
            R_all_t = _h.allocate((self.size, 4 * self.size))
            _h.transpose(R_all, R_all_t)
        for t in range(time_size - 1, -1, -1):
            if thin:
                _h.dot_small_tn(packed_t[(t + 1) % 2], batch, R_all, parts, splits)
                _h.lstm_backward_step_thin(self.activation, deltas[t], parts, dy[t], packed_t[t % 2],
                                           Zb[t], Ib[t], Fb[t], Ob[t], Cb[t], Ca[t - 1],
                                           Fb[t + 1], dIa[t + 1], dFa[t + 1], dCa[t + 1],
                                           dZa[t], dZb[t], dIa[t], dIb[t], dFa[t], dFb[t],
                                           dOa[t], dOb[t], dCa[t], dCb[t], pi, pf, po)
                continue
            if R_all is not None:
                dy_t = dy[t]
                packed_next = packed_all[t + 1] if packed_all is not None else packed[(t + 1) % 2]
                packed_now = packed_all[t] if packed_all is not None else packed[t % 2]
                if R_all_t is not None:
                    _h.dot_mm(packed_next, R_all_t, dy_t, transb=True)
                else:
                    _h.dot_mm(packed_next, R_all, dy_t)
                _h.lstm_backward_step_packed(self.activation, deltas[t], dy_t, packed_now,
                                             Zb[t], Ib[t], Fb[t], Ob[t], Cb[t], Ca[t - 1],
                                             Fb[t + 1], dIa[t + 1], dFa[t + 1], dCa[t + 1],
                                             dZa[t], dZb[t], dIa[t], dIb[t], dFa[t], dFb[t],
                                             dOa[t], dOb[t], dCa[t], dCb[t], pi, pf, po)
                continue
            if fused:
                dy_t = dy[t]
                _h.copy_to(deltas[t], dy_t)
                _h.dot_add_mm(dIa[t + 1], Ri, dy_t)
                _h.dot_add_mm(dFa[t + 1], Rf, dy_t)
                _h.dot_add_mm(dOa[t + 1], Ro, dy_t)
                _h.dot_add_mm(dZa[t + 1], Rz, dy_t)
                _h.lstm_backward_step(self.activation, dy_t, Zb[t], Ib[t], Fb[t], Ob[t], Cb[t],
                                      Ca[t - 1], Fb[t + 1], dIa[t + 1], dFa[t + 1], dCa[t + 1],
                                      dZa[t], dZb[t], dIa[t], dIb[t], dFa[t], dFb[t], dOa[t],
                                      dOb[t], dCa[t], dCb[t], pi, pf, po)
                continue
            # accumulate recurrent deltas
            _h.copy_to(deltas[t], dy[t])
            _h.dot_add_mm(dIa[t + 1], Ri, dy[t])
            _h.dot_add_mm(dFa[t + 1], Rf, dy[t])
            _h.dot_add_mm(dOa[t + 1], Ro, dy[t])
            _h.dot_add_mm(dZa[t + 1], Rz, dy[t])
            # peepholes into the cell
            _h.mult_add_mv(dIa[t + 1], pi, dCa[t])
            _h.mult_add_mv(dFa[t + 1], pf, dCa[t])
            # output gate
            _h.mult_tt(dy[t], Cb[t], dOb[t])
            _h.sigmoid_deriv(Oa[t], Ob[t], dOb[t], dOa[t])
            _h.mult_add_mv(dOa[t], po, dCa[t])
            # cell
            _h.mult_tt(dy[t], Ob[t], dCb[t])
            _h.act_func_deriv[self.activation](Ca[t], Cb[t], dCb[t], dCb[t])
            _h.add_tt(dCa[t], dCb[t], dCa[t])
            _h.mult_add_tt(dCa[t + 1], Fb[t + 1], dCa[t])
            # forget gate
            _h.mult_tt(dCa[t], Ca[t - 1], dFb[t])
            _h.sigmoid_deriv(Fa[t], Fb[t], dFb[t], dFa[t])
            # input gate
            _h.mult_tt(dCa[t], Zb[t], dIb[t])
            _h.sigmoid_deriv(Ia[t], Ib[t], dIb[t], dIa[t])
            # block input
            _h.mult_tt(dCa[t], Ib[t], dZb[t])
            _h.act_func_deriv[self.activation](Za[t], Zb[t], dZb[t], dZa[t])

        flat_inputs = flatten_time_and_features(x)
        flat_dinputs = flatten_time_and_features(dx)
        flat_dIa = flatten_time(dIa[:-1])
        flat_dFa = flatten_time(dFa[:-1])
        flat_dOa = flatten_time(dOa[:-1])
        flat_dZa = flatten_time(dZa[:-1])

        # input deltas and input-weight gradients
        if packed_all is not None:
            flat_packed = flatten_time(packed_all[:-1])
            _h.dot_add_mm(flat_packed, W_all, flat_dinputs)
            _h.dot_add_mm(flat_packed, flat_inputs, dW_all, transa=True)
            dbias_tmp = _h.allocate(db_all.shape)
            _h.sum_t(flat_packed, axis=0, out=dbias_tmp)
            _h.add_tt(db_all, dbias_tmp, db_all)
        else:
            _h.dot_add_mm(flat_dIa, Wi, flat_dinputs)
            _h.dot_add_mm(flat_dFa, Wf, flat_dinputs)
            _h.dot_add_mm(flat_dOa, Wo, flat_dinputs)
            _h.dot_add_mm(flat_dZa, Wz, flat_dinputs)
            _h.dot_add_mm(flat_dIa, flat_inputs, dWi, transa=True)
            _h.dot_add_mm(flat_dFa, flat_inputs, dWf, transa=True)
            _h.dot_add_mm(flat_dOa, flat_inputs, dWo, transa=True)
            _h.dot_add_mm(flat_dZa, flat_inputs, dWz, transa=True)

            dbias_tmp = _h.allocate(dbz.shape)
            _h.sum_t(flat_dIa, axis=0, out=dbias_tmp)
            _h.add_tt(dbi, dbias_tmp, dbi)
            _h.sum_t(flat_dFa, axis=0, out=dbias_tmp)
            _h.add_tt(dbf, dbias_tmp, dbf)
            _h.sum_t(flat_dOa, axis=0, out=dbias_tmp)
            _h.add_tt(dbo, dbias_tmp, dbo)
            _h.sum_t(flat_dZa, axis=0, out=dbias_tmp)
            _h.add_tt(dbz, dbias_tmp, dbz)

        flat_outputs = flatten_time(y[:-2])
        flat_cell = flatten_time(Ca[:-2])
        flat_cell2 = flatten_time(Ca[:-1])
        dWco_tmp = empty(flat_cell2.shape)            # written by the products below before it is read
        dWc_tmp = _h.allocate(dpo.shape)
        # output-gate peephole
        _h.mult_tt(flat_cell2, flat_dOa, dWco_tmp)
        _h.sum_t(dWco_tmp, axis=0, out=dWc_tmp)
        _h.add_tt(dpo, dWc_tmp, dpo)

        flat_dIa = flatten_time(dIa[1:-1])
        flat_dFa = flatten_time(dFa[1:-1])
        flat_dOa = flatten_time(dOa[1:-1])
        flat_dZa = flatten_time(dZa[1:-1])
        # recurrent-weight gradients
        if packed_all is not None:
            _h.dot_add_mm(flatten_time(packed_all[1:-1]), flat_outputs, dR_all, transa=True)
            _h.dot_add_mm(packed_all[0], dy[-1], dR_all, transa=True)
        else:
            _h.dot_add_mm(flat_dIa, flat_outputs, dRi, transa=True)
            _h.dot_add_mm(flat_dFa, flat_outputs, dRf, transa=True)
            _h.dot_add_mm(flat_dOa, flat_outputs, dRo, transa=True)
            _h.dot_add_mm(flat_dZa, flat_outputs, dRz, transa=True)
            _h.dot_add_mm(dIa[0], dy[-1], dRi, transa=True)
            _h.dot_add_mm(dFa[0], dy[-1], dRf, transa=True)
            _h.dot_add_mm(dOa[0], dy[-1], dRo, transa=True)
            _h.dot_add_mm(dZa[0], dy[-1], dRz, transa=True)

        # input- and forget-gate peepholes
        dWcif_tmp = empty(flat_cell.shape)
        _h.mult_tt(flat_cell, flat_dIa, dWcif_tmp)
        _h.sum_t(dWcif_tmp, axis=0, out=dWc_tmp)
        _h.add_tt(dpi, dWc_tmp, dpi)
        _h.mult_tt(flat_cell, flat_dFa, dWcif_tmp)
        _h.sum_t(dWcif_tmp, axis=0, out=dWc_tmp)
        _h.add_tt(dpf, dWc_tmp, dpf)

        dWcif_tmp = _h.allocate(dIa[0].shape)
        _h.mult_tt(dCa[-1], dIa[0], dWcif_tmp)
        _h.sum_t(dWcif_tmp, axis=0, out=dWc_tmp)
        _h.add_tt(dpi, dWc_tmp, dpi)
        _h.mult_tt(dCa[-1], dIa[0], dWcif_tmp)       # the reference uses dIa here as well
        _h.sum_t(dWcif_tmp, axis=0, out=dWc_tmp)
        _h.add_tt(dpf, dWc_tmp, dpf)


class BatchNorm(Layer):
    """layers/batch_normalization_layer.py:54-152"""

    def __init__(self, decay=0.9, epsilon=1.0e-5, fused=False):
        self.decay = decay
        self.epsilon = epsilon
        self.fused = bool(fused)        # whole passes through handler.batchnorm_* when they exist

    def setup(self, in_shapes):
        shape = in_shapes["default"].feature_shape
        f = (shape[-1],)
        parameters = OrderedDict([("gamma", f), ("beta", f), ("mu", f), ("sigma", f)])
        internals = OrderedDict([("sigma_b", Buf(f, scales="")), ("centered", Buf(shape)), ("x_hat", Buf(shape))])
        return OrderedDict(default=Buf(shape)), parameters, internals

    def forward_pass(self, buffers, training_pass=True):
        _h = self.handler
        sigma_b = buffers.internals["sigma_b"]
        gamma, beta, mu, sigma = buffers.parameters.values()
        inputs = flatten_all_but_last(buffers.inputs["default"])
        centered = flatten_all_but_last(buffers.internals["centered"])
        x_hat = flatten_all_but_last(buffers.internals["x_hat"])
        out = flatten_all_but_last(buffers.outputs["default"])
        m = inputs.shape[0]
        if self.fused and hasattr(_h, "batchnorm_forward"):
            _h.batchnorm_forward(training_pass, inputs, gamma, beta, mu, sigma, self.decay,
                                 self.epsilon, sigma_b, centered, x_hat, out)
            return

        if training_pass:
            mu_b = sigma_b                       # reused as scratch for the NEGATIVE batch mean
            _h.sum_t(inputs, 0, mu_b)
            _h.mult_st(-1.0 / m, mu_b, mu_b)
            # running average of the (negative) mean
            _h.mult_st(self.decay, mu, mu)
            _h.mult_add_st(1.0 - self.decay, mu_b, mu)
            mu = mu_b
        _h.add_mv(inputs, mu.reshape((1, mu.size)), centered)

        if training_pass:
            sigma2 = sigma_b
            centered2 = x_hat                    # scratch
            _h.mult_tt(centered, centered, centered2)
            _h.sum_t(centered2, 0, sigma2)
            _h.mult_st(1.0 / m, sigma2, sigma2)              # biased variance
            _h.add_st(self.epsilon, sigma2, sigma2)
            _h.sqrt_t(sigma2, sigma_b)
            _h.mult_st(self.decay, sigma, sigma)
            _h.mult_add_st(1.0 - self.decay, sigma_b, sigma)
            sigma = sigma_b
        _h.divide_mv(centered, sigma.reshape((1, sigma.size)), x_hat)
        _h.mult_mv(x_hat, gamma.reshape((1, gamma.size)), out)
        _h.add_mv(out, beta.reshape((1, beta.size)), out)

    def backward_pass(self, buffers):
        _h = self.handler
        sigma_b = buffers.internals["sigma_b"]
        gamma = buffers.parameters["gamma"]
        dgamma, dbeta = buffers.gradients["gamma"], buffers.gradients["beta"]
        x_hat = flatten_all_but_last(buffers.internals["x_hat"])
        outdeltas = flatten_all_but_last(buffers.output_deltas["default"])
        indeltas = flatten_all_but_last(buffers.input_deltas["default"])
        m = outdeltas.shape[0]
        if self.fused and hasattr(_h, "batchnorm_backward"):
            _h.batchnorm_backward(outdeltas, x_hat, gamma, sigma_b, dgamma, dbeta, indeltas)
            return

        big_tmp = _h.allocate(x_hat.shape)
        small_tmp = _h.allocate(gamma.shape)
        # dgamma
        _h.mult_tt(outdeltas, x_hat, big_tmp)
        _h.sum_t(big_tmp, axis=0, out=small_tmp)
        _h.add_tt(small_tmp, dgamma, dgamma)
        _h.mult_st(1 / m, small_tmp, small_tmp)
        _h.mult_mv(x_hat, small_tmp.reshape((1, gamma.size)), big_tmp)        # term1
        # dbeta
        _h.sum_t(outdeltas, axis=0, out=small_tmp)
        _h.add_tt(small_tmp, dbeta, dbeta)
        _h.mult_st(1 / m, small_tmp, small_tmp)
        # deltas
        _h.subtract_tt(outdeltas, big_tmp, big_tmp)                           # term2
        _h.subtract_mv(big_tmp, small_tmp.reshape((1, dbeta.size)), big_tmp)  # term3
        _h.divide_tt(gamma, sigma_b, small_tmp)                               # gamma / sigma_b
        _h.mult_mv(big_tmp, small_tmp.reshape((1, small_tmp.size)), big_tmp)  # term4
        _h.add_tt(big_tmp, indeltas, indeltas)


class Highway(Layer):
    """layers/highway_layer.py:40-71: y = T*H + (1-T)*x with inputs 'H', 'T', 'x'."""

    def __init__(self, fused=False):
        self.fused = bool(fused)        # one pass each way through handler.highway_* when they exist

    def setup(self, in_shapes):
        return OrderedDict(default=Buf(in_shapes["x"].feature_shape)), OrderedDict(), OrderedDict()

    def forward_pass(self, buffers, training_pass=True):
        _h = self.handler
        x, H, T = buffers.inputs["x"], buffers.inputs["H"], buffers.inputs["T"]
        y = buffers.outputs["default"]
        if self.fused and hasattr(_h, "highway_forward"):
            _h.highway_forward(H, T, x, y)
            return
        tmp = _h.zeros(x.shape)
        _h.subtract_tt(H, x, out=tmp)
        _h.mult_tt(T, tmp, out=tmp)
        _h.add_tt(tmp, x, out=y)

    def backward_pass(self, buffers):
        _h = self.handler
        x, H, T = buffers.inputs["x"], buffers.inputs["H"], buffers.inputs["T"]
        dx, dH, dT = buffers.input_deltas["x"], buffers.input_deltas["H"], buffers.input_deltas["T"]
        dy = buffers.output_deltas["default"]
        if self.fused and hasattr(_h, "highway_backward"):
            _h.highway_backward(H, T, x, dy, dx, dH, dT)
            return
        tmp = _h.ones(dx.shape)
        _h.subtract_tt(tmp, T, out=tmp)
        _h.mult_add_tt(tmp, dy, out=dx)
        _h.mult_add_tt(T, dy, out=dH)
        _h.subtract_tt(H, x, out=tmp)
        _h.mult_add_tt(tmp, dy, out=dT)


def _conv_out(size, kernel, padding, stride):
    return (size + 2 * padding - kernel) // stride + 1


class Convolution2D(Layer):
    """layers/convolution_layer_2d.py:78-112; images are (T, B, H, W, C)."""

    def __init__(self, num_filters, kernel_size, stride=(1, 1), padding=0, activation="rel"):
        self.num_filters = num_filters
        self.kernel_size = tuple(kernel_size)
        self.stride = tuple(stride)
        self.padding = padding
        self.activation = activation

    def setup(self, in_shapes):
        h, w, c = in_shapes["default"].feature_shape
        kh, kw = self.kernel_size
        out_shape = (_conv_out(h, kh, self.padding, self.stride[0]),
                     _conv_out(w, kw, self.padding, self.stride[1]), self.num_filters)
        parameters = OrderedDict([("W", (self.num_filters, kh, kw, c)), ("bias", (self.num_filters,))])
        return OrderedDict(default=Buf(out_shape)), parameters, OrderedDict()

    def forward_pass(self, buffers, training_pass=True):
        _h = self.handler
        W, bias = buffers.parameters["W"], buffers.parameters["bias"]
        outputs = buffers.outputs["default"]
        _h.conv2d_forward_batch(flatten_time(buffers.inputs["default"]), W, bias, flatten_time(outputs),
                                self.padding, self.stride)
        _h.inplace_act_func[self.activation](outputs)

    def backward_pass(self, buffers):
        _h = self.handler
        W = buffers.parameters["W"]
        dW, dbias = buffers.gradients["W"], buffers.gradients["bias"]
        out_deltas = buffers.output_deltas["default"]
        _h.inplace_act_func_deriv[self.activation](buffers.outputs["default"], out_deltas)
        _h.conv2d_backward_batch(flatten_time(buffers.inputs["default"]), W, self.padding, self.stride,
                                 flatten_time(buffers.input_deltas["default"]), flatten_time(out_deltas),
                                 dW, dbias)


class Pooling2D(Layer):
    """layers/pooling_layer_2d.py:74-121"""

    def __init__(self, type, kernel_size, stride=(1, 1), padding=0):
        assert type in ("max", "avg")
        self.type = type
        self.kernel_size = tuple(kernel_size)
        self.stride = tuple(stride)
        self.padding = padding

    def setup(self, in_shapes):
        h, w, c = in_shapes["default"].feature_shape
        out_shape = (_conv_out(h, self.kernel_size[0], self.padding, self.stride[0]),
                     _conv_out(w, self.kernel_size[1], self.padding, self.stride[1]), c)
        internals = OrderedDict()
        if self.type == "max":
            internals["argmax"] = Buf(out_shape)
        return OrderedDict(default=Buf(out_shape)), OrderedDict(), internals

    def forward_pass(self, buffers, training_pass=True):
        _h = self.handler
        flat_inputs = flatten_time(buffers.inputs["default"])
        flat_outputs = flatten_time(buffers.outputs["default"])
        if self.type == "max":
            _h.maxpool2d_forward_batch(flat_inputs, self.kernel_size, flat_outputs, self.padding,
                                       self.stride, flatten_time(buffers.internals["argmax"]))
        else:
            _h.avgpool2d_forward_batch(flat_inputs, self.kernel_size, flat_outputs, self.padding, self.stride)

    def backward_pass(self, buffers):
        _h = self.handler
        flat_inputs = flatten_time(buffers.inputs["default"])
        flat_outputs = flatten_time(buffers.outputs["default"])
        flat_in_deltas = flatten_time(buffers.input_deltas["default"])
        flat_out_deltas = flatten_time(buffers.output_deltas["default"])
        if self.type == "max":
            _h.maxpool2d_backward_batch(flat_inputs, self.kernel_size, flat_outputs, self.padding,
                                        self.stride, flatten_time(buffers.internals["argmax"]),
                                        flat_in_deltas, flat_out_deltas)
        else:
            _h.avgpool2d_backward_batch(flat_inputs, self.kernel_size, flat_outputs, self.padding,
                                        self.stride, flat_in_deltas, flat_out_deltas)
