"""ctypes binding of libbship.so (declarations in include/bship.h).

The library is loaded from the package directory (or ``$BSHIP_LIB``). There is
no fallback: if the library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, c_char_p, c_double, c_float, c_int, c_int64,
                    c_size_t, c_uint32, c_void_p)

HERE = os.path.dirname(os.path.abspath(__file__))
DEFAULT_LIB_PATH = os.path.join(HERE, "libbship.so")

# op codes of include/bship.h
ADD, SUB, MUL, DIV, FMOD = 0, 1, 2, 3, 4
ADD_ST, MULT_ST, MULT_ADD_ST = 0, 1, 2
ABS, SIGN, SQRT, LOG, SIGMOID, TANH, REL, EL = 0, 1, 2, 3, 4, 5, 6, 7
SIGMOID_DERIV, TANH_DERIV, REL_DERIV, EL_DERIV = 0, 1, 2, 3
COPY_IF, FILL_IF, ADD_IF = 0, 1, 2
(PITCHED_BINARY, PITCHED_MULT_ADD, PITCHED_SCALAR, PITCHED_UNARY, PITCHED_DERIV, PITCHED_CLIP, PITCHED_COND,
 PITCHED_FILL) = range(8)

ERR_OUT_OF_MEMORY = -5
ERR_UNSUPPORTED = -6
ERR_TIMEOUT = -9

_P = c_void_p          # device pointers travel as plain integers
_I64 = c_int64

# name -> argtypes; every function returns an int status except the two noted.
SIGNATURES = {
    "bship_init": [c_int],
    "bship_shutdown": [],
    "bship_sync": [],
    "bship_device_info": [ctypes.c_char_p, c_size_t, POINTER(c_int)],
    "bship_event_record": [c_int],
    "bship_event_elapsed_ms": [c_int, c_int, POINTER(c_float)],
    "bship_graph_begin": [],
    "bship_graph_end": [POINTER(c_int)],
    "bship_graph_launch": [c_int],
    "bship_graph_destroy": [c_int],
    "bship_malloc": [c_size_t, POINTER(c_void_p)],
    "bship_malloc_scratch": [c_size_t, POINTER(c_void_p)],
    "bship_free": [_P],
    "bship_pool_trim": [],
    "bship_pool_stats": [POINTER(c_size_t), POINTER(c_size_t), POINTER(c_size_t)],
    "bship_h2d": [_P, c_void_p, c_size_t],
    "bship_d2h": [c_void_p, _P, c_size_t],
    "bship_d2d": [_P, _P, c_size_t],
    "bship_copy2d_f32": [_P, _I64, _P, _I64, _I64, _I64],
    "bship_fill_f32": [_P, c_float, c_size_t],
    "bship_binary_f32": [c_int, _P, _P, _P, c_size_t],
    "bship_mult_add_tt_f32": [_P, _P, _P, c_size_t],
    "bship_scalar_f32": [c_int, c_float, _P, _P, c_size_t],
    "bship_unary_f32": [c_int, _P, _P, c_size_t],
    "bship_deriv_f32": [c_int, _P, _P, _P, c_size_t],
    "bship_clip_f32": [_P, c_float, c_float, _P, c_size_t],
    "bship_cond_f32": [c_int, _P, c_float, _P, _P, c_size_t],
    "bship_mv_f32": [c_int, _P, _P, _P, _I64, _I64, c_int, c_int],
    "bship_elementwise_pitched_f32": [c_int, c_int, c_float, c_float, _P, _I64, c_int, _P, _I64, c_int,
                                      _P, _I64, _I64, _I64],
    "bship_broadcast_f32": [_P, _P, _I64, _I64, _I64],
    "bship_broadcast_pitched_f32": [_P, _I64, _I64, _P, _I64, _I64, _I64, _I64, _I64],
    "bship_merge_f32": [_P, _P, _P, _I64, _I64, _I64],
    "bship_split_add_f32": [_P, _P, _P, _I64, _I64, _I64],
    "bship_sum_f32": [_P, _P, _I64, _I64, c_int],
    "bship_sum_pitched_f32": [_P, _I64, _P, _I64, _I64, c_int],
    "bship_sum_noalloc_f32": [_P, _P, _I64, _I64, c_int],
    "bship_softmax_rows_pitched_f32": [_P, _I64, _P, _I64, _I64, _I64],
    "bship_binarize_pitched_f32": [_P, _I64, _P, _I64, _I64, _I64],
    "bship_index_m_by_v_pitched_f32": [_P, _I64, _P, _I64, _P, _I64, _I64, _I64],
    "bship_softmax_rows_f32": [_P, _P, _I64, _I64],
    "bship_isfinite_f32": [_P, c_size_t, POINTER(c_int)],
    "bship_binarize_f32": [_P, _P, _I64, _I64],
    "bship_index_m_by_v_f32": [_P, _P, _P, _I64, _I64],
    "bship_rng_create": [POINTER(c_int)],
    "bship_rng_select": [c_int],
    "bship_rng_destroy": [c_int],
    "bship_rng_seed": [c_uint32],
    "bship_prob_mask_f32": [_P, c_size_t, c_double],
    "bship_prob_mask_pitched_f32": [_P, _I64, _I64, _I64, c_double],
    "bship_fill_gaussian_f32": [_P, c_size_t, c_double, c_double],
    "bship_fast_rng_seed": [ctypes.c_ulonglong],
    "bship_fast_rng_get_state": [POINTER(ctypes.c_ulonglong), POINTER(ctypes.c_ulonglong)],
    "bship_prob_mask_fast_f32": [_P, c_size_t, c_double],
    "bship_dropout_fwd_fast_f32": [_P, _P, _P, c_size_t, c_double, c_float],
    "bship_rng_get_state": [POINTER(c_uint32), POINTER(c_int), POINTER(c_int), POINTER(c_double)],
    "bship_rng_seed_on": [c_int, c_uint32],
    "bship_rng_get_state_on": [c_int, POINTER(c_uint32), POINTER(c_int), POINTER(c_int), POINTER(c_double)],
    "bship_prob_mask_on_f32": [c_int, _P, c_size_t, c_double],
    "bship_prob_mask_pitched_on_f32": [c_int, _P, _I64, _I64, _I64, c_double],
    "bship_fill_gaussian_on_f32": [c_int, _P, c_size_t, c_double, c_double],
    "bship_dropout_fwd_on_f32": [c_int, _P, _P, _P, c_size_t, c_double, c_float],
    "bship_fast_rng_seed_on": [c_int, ctypes.c_ulonglong],
    "bship_fast_rng_get_state_on": [c_int, POINTER(ctypes.c_ulonglong), POINTER(ctypes.c_ulonglong)],
    "bship_prob_mask_fast_on_f32": [c_int, _P, c_size_t, c_double],
    "bship_dropout_fwd_fast_on_f32": [c_int, _P, _P, _P, c_size_t, c_double, c_float],
    "bship_fusing_set": [c_int],
    "bship_fusing_get": [POINTER(c_int)],
    "bship_fusing_flush": [],
    "bship_fusing_stats": [POINTER(ctypes.c_ulonglong)] * 5 + [c_int],
    "bship_gemm_f32": [c_int, c_int, _I64, _I64, _I64, c_float, _P, _I64, _P, _I64, c_float, _P, _I64],
    "bship_gemm_bias_f32": [c_int, c_int, _I64, _I64, _I64, _P, _I64, _P, _I64, _P, _P, _I64],
    "bship_conv2d_fwd_thin_f32": [_P, _I64, _P, _P, _P, _I64] + [c_int] * 9,
    "bship_conv2d_bwd_thin_f32": [_P, _I64, _P, _P, _P, _I64, _P, _P, _I64] + [c_int] * 9,
    "bship_im2col_nhwc_f32": [_P, _P, _I64] + [c_int] * 8,
    "bship_col2im_nhwc_f32": [_P, _P, _I64] + [c_int] * 8,
    "bship_maxpool_fwd_nhwc_f32": [_P, _P, _P, _I64] + [c_int] * 10,
    "bship_maxpool_bwd_nhwc_f32": [_P, _P, _P, _I64] + [c_int] * 10,
    "bship_avgpool_fwd_nhwc_f32": [_P, _P, _I64] + [c_int] * 10,
    "bship_avgpool_bwd_nhwc_f32": [_P, _P, _I64] + [c_int] * 10,
    "bship_im2col_nhwc_pitched_f32": [_P, _I64, _P, _I64] + [c_int] * 8,
    "bship_col2im_nhwc_pitched_f32": [_P, _P, _I64, _I64] + [c_int] * 8,
    "bship_maxpool_fwd_nhwc_pitched_f32": [_P, _I64, _P, _I64, _P, _I64, _I64] + [c_int] * 10,
    "bship_maxpool_bwd_nhwc_pitched_f32": [_P, _I64, _P, _I64, _P, _I64, _I64] + [c_int] * 10,
    "bship_avgpool_fwd_nhwc_pitched_f32": [_P, _I64, _P, _I64, _I64] + [c_int] * 10,
    "bship_avgpool_bwd_nhwc_pitched_f32": [_P, _I64, _P, _I64, _I64] + [c_int] * 10,
    "bship_lstm_fwd_step_f32": [c_int, _I64, _I64] + [_P] * 19,
    "bship_lstm_bwd_step_f32": [c_int, _I64, _I64] + [_P] * 24,
    "bship_lstm_fwd_step_packed_f32": [c_int, _I64, _I64] + [_P] * 20,
    "bship_lstm_bwd_step_packed_f32": [c_int, _I64, _I64] + [_P] * 26,
    "bship_lstm_fwd_sequence_f32": [c_int, _I64, _I64, _I64] + [_P] * 19,
    "bship_dot_small_tn_f32": [_P, _P, _P, _I64, _I64, _I64, _I64, _I64, c_int, _I64],
    "bship_transpose_f32": [_P, _I64, _I64, _I64, _P, _I64],
    "bship_lstm_bwd_step_thin_f32": [c_int, _I64, _I64, _P, _P, c_int, _I64] + [_P] * 25,
    "bship_softmax_ce_fwd_f32": [_P, _P, _P, _P, _I64, _I64],
    "bship_softmax_ce_bwd_f32": [_P, _P, _P, _P, _P, _I64, _I64],
    "bship_momentum_update_f32": [c_float, c_float, _P, _P, _P, c_size_t],
    "bship_highway_fwd_f32": [_P, _P, _P, _P, c_size_t],
    "bship_highway_bwd_f32": [_P] * 7 + [c_size_t],
    "bship_dropout_fwd_f32": [_P, _P, _P, c_size_t, c_double, c_float],
    "bship_bias_act_f32": [c_int, _P, _P, _P, _I64, _I64],
    "bship_batchnorm_fwd_f32": [c_int, _P, _P, _P, _P, _P, c_double, c_double, _P, _P, _P, _P, _I64, _I64],
    "bship_batchnorm_bwd_f32": [_P] * 7 + [_I64, _I64],
}
# functions that do not return a status
SPECIAL_RESTYPES = {"bship_version": (c_int, []), "bship_last_error": (c_char_p, [])}

EXPORTED_SYMBOLS = tuple(sorted(list(SIGNATURES) + list(SPECIAL_RESTYPES)))


class BshipError(RuntimeError):
    """A libbship call returned a non-zero status."""

    def __init__(self, status, message):
        super().__init__("libbship error %d: %s" % (status, message))
        self.status = status


def lib_path() -> str:
    return os.environ.get("BSHIP_LIB") or DEFAULT_LIB_PATH


_LIB = None


def load():
    """Loads libbship.so once and declares every prototype."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(
            "libbship.so not found at %s; build it with `python -m brainstorm_amd.build` "
            "(hipcc, gfx950). There is no CPU fallback." % path)
    lib = ctypes.CDLL(path)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int
    for name, (restype, argtypes) in SPECIAL_RESTYPES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = restype
    _LIB = lib
    return lib


# entry points that the handler calls through brainstorm_amd._fastcall (csrc/fastcall.c)
FAST_ENTRY_POINTS = ("bship_binary_f32", "bship_mult_add_tt_f32", "bship_scalar_f32", "bship_unary_f32",
                     "bship_deriv_f32", "bship_clip_f32", "bship_mv_f32", "bship_fill_f32", "bship_gemm_f32",
                     "bship_d2d", "bship_sum_f32")


def entry_point_addresses(lib):
    """name -> address of the entry points of FAST_ENTRY_POINTS that `lib` exports."""
    out = {}
    for name in FAST_ENTRY_POINTS:
        try:
            fn = getattr(lib, name)
        except AttributeError:
            continue
        out[name] = ctypes.cast(fn, c_void_p).value
    return out


def raise_for_status(lib, status):
    msg = lib.bship_last_error()
    msg = msg.decode("utf-8", "replace") if msg else ""
    if status == ERR_OUT_OF_MEMORY:
        raise MemoryError("libbship: " + msg)
    raise BshipError(status, msg)
