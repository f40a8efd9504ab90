"""CPU: calls whose operands do not fit each other are refused before anything is launched.

NumPy raises ValueError where `out[:] = a + b` cannot be formed (numpy_handler.py:86-87); the
device kernels get one element count and raw addresses, so HipHandler has to refuse such calls
itself. Every case below must raise on the CPU oracle AND on HipHandler, and the launch log of
the host-only trace library must stay empty."""
import numpy as np
import pytest

from oracle.numpy_ref_handler import NumpyRefHandler

F32 = np.float32


def cases(h):
    A = lambda *shape: h.allocate(shape)
    a46, b64, a47, v5, c41, c51 = A(4, 6), A(6, 4), A(4, 7), A(1, 5), A(4, 1), A(5, 1)
    img, pooled = A(2, 8, 8, 3), A(2, 3, 3, 3)
    return [
        ("add_tt", lambda: h.add_tt(a46, a47, a46)),
        ("add_tt short output", lambda: h.add_tt(a47, a47, a46)),
        ("subtract_tt", lambda: h.subtract_tt(a46, a47, a46)),
        ("mult_tt", lambda: h.mult_tt(a47, a46, a46)),
        ("divide_tt", lambda: h.divide_tt(a46, a46, a47)),
        ("modulo_tt", lambda: h.modulo_tt(a46, a47, a46)),
        ("mult_add_tt", lambda: h.mult_add_tt(a46, a47, a46)),
        ("add_st", lambda: h.add_st(1.0, a47, a46)),
        ("mult_st", lambda: h.mult_st(2.0, a47, a46)),
        ("mult_add_st", lambda: h.mult_add_st(2.0, a47, a46)),
        ("abs_t", lambda: h.abs_t(a47, a46)),
        ("sign_t", lambda: h.sign_t(a47, a46)),
        ("sqrt_t", lambda: h.sqrt_t(a47, a46)),
        ("log_t", lambda: h.log_t(a47, a46)),
        ("clip_t", lambda: h.clip_t(a47, 0.0, 1.0, a46)),
        ("sigmoid", lambda: h.sigmoid(a47, a46)),
        ("tanh", lambda: h.tanh(a47, a46)),
        ("rel", lambda: h.rel(a47, a46)),
        ("el", lambda: h.el(a47, a46)),
        ("sigmoid_deriv", lambda: h.sigmoid_deriv(None, a47, a46, a46)),
        ("tanh_deriv", lambda: h.tanh_deriv(None, a46, a47, a46)),
        ("rel_deriv", lambda: h.rel_deriv(None, a46, a46, a47)),
        ("el_deriv", lambda: h.el_deriv(None, a47, a46, a46)),
        ("add_mv row", lambda: h.add_mv(a46, v5, a46)),
        ("mult_mv column", lambda: h.mult_mv(a46, c51, a46)),
        ("subtract_mv output", lambda: h.subtract_mv(a46, c41, a47)),
        ("divide_mv", lambda: h.divide_mv(a46, v5, a46)),
        ("mult_add_mv", lambda: h.mult_add_mv(a46, v5, a46)),
        ("sum_t axis 0", lambda: h.sum_t(a46, 0, v5)),
        ("sum_t axis 1", lambda: h.sum_t(a46, 1, c51)),
        ("sum_t everything", lambda: h.sum_t(a46, None, v5)),
        ("softmax_m", lambda: h.softmax_m(a46, a47)),
        ("binarize_v", lambda: h.binarize_v(c51, a46)),
        ("index_m_by_v", lambda: h.index_m_by_v(a46, c41, c51)),
        ("copy_to", lambda: h.copy_to(a47, a46)),
        ("copy_to flat", lambda: h.copy_to(A(24), a46)),
        ("copy_to_if", lambda: h.copy_to_if(a47, a46, a46)),
        ("fill_if", lambda: h.fill_if(a46, 1.0, a47)),
        ("add_into_if", lambda: h.add_into_if(a47, a46, a46)),
        ("merge_tt", lambda: h.merge_tt(a46, a47, A(4, 12))),
        ("split_add_tt", lambda: h.split_add_tt(A(4, 12), a46, a47)),
        ("dot_mm", lambda: h.dot_mm(a46, a47, A(4, 7))),
        ("dot_add_mm", lambda: h.dot_add_mm(a46, b64, a46)),
        # from here on HipHandler only: the reference's image routines (Cython, `_cpuop.pyx`) trust their
        # shapes like the kernels do, and so does the oracle's C restatement
        ("maxpool2d_forward_batch", lambda: h.maxpool2d_forward_batch(img, (3, 3), A(2, 4, 4, 3), 0, (2, 2), A(2, 4, 4, 3))),
        ("maxpool2d_backward_batch", lambda: h.maxpool2d_backward_batch(img, (3, 3), pooled, 0, (2, 2), pooled, A(2, 8, 8, 2), pooled)),
        ("avgpool2d_forward_batch", lambda: h.avgpool2d_forward_batch(img, (3, 3), A(2, 3, 4, 3), 0, (2, 2))),
        ("conv2d_forward_batch", lambda: h.conv2d_forward_batch(img, A(5, 3, 3, 3), A(5), A(2, 8, 8, 5), 0, (1, 1))),
        ("conv2d_forward_batch channels", lambda: h.conv2d_forward_batch(img, A(5, 3, 3, 2), A(5), A(2, 6, 6, 5), 0, (1, 1))),
    ]


def test_mismatched_operands_raise_and_launch_nothing(trace):
    from brainstorm_amd import HipHandler
    for fusing in (False, True):
        hip = HipHandler(seed=1, fusing=fusing)
        ref = NumpyRefHandler(F32, seed=1)
        hip_cases, ref_cases = cases(hip), cases(ref)
        trace.trace_reset()
        for (name, on_hip), (_, on_ref) in zip(hip_cases, ref_cases):
            if "pool" not in name and "conv" not in name:
                with pytest.raises((ValueError, AssertionError, IndexError)), np.errstate(all="ignore"):
                    on_ref()
            with pytest.raises((ValueError, AssertionError)):
                on_hip()
            assert trace.trace_held() == 0, name
        assert trace.trace_log() == b"", trace.trace_log()


def test_matching_operands_of_other_shapes_still_run(trace):
    # the reference checks no shapes (base_handler.py:14-28): what counts is that NumPy can form the result.
    from brainstorm_amd import HipHandler
    hip = HipHandler(seed=1, fusing=False)
    a, flat = hip.allocate((4, 6)), hip.allocate((24,))
    trace.trace_reset()
    hip.add_mv(a, hip.allocate((6,)), a)                 # a 1-D vector is a row
    hip.sum_t(a, 0, hip.allocate((6,)))                  # keepdims or not is the output's business
    hip.sum_t(a, 1, hip.allocate((4, 1)))
    hip.sum_t(a.reshape((2, 2, 6)), None, hip.allocate(()))
    hip.copy_to(hip.allocate((1, 6)), a)                 # broadcast rows
    hip.copy_to(hip.allocate((2, 1, 3, 1)), hip.allocate((2, 5, 3, 4)))    # repeated axes that are not neighbours
    hip.mult_st(2.0, flat, flat)
    log = [line.split()[0] for line in trace.trace_log().decode().splitlines()]
    assert log == ["mv", "sum", "sum", "sum", "broadcast", "broadcast", "broadcast", "scalar"], log
