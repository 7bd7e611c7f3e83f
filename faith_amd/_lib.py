"""ctypes binding of libfaith_amd.so (the C ABI declared in include/faith_amd.h).

There is no fallback: if the library is missing or a symbol is absent, import
of this module raises.  Build it with ``python -m faith_amd.build``.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libfaith_amd.so")

OK = 0
ERR_NULL, ERR_SHAPE, ERR_UNSUPPORTED, ERR_ALIGN, ERR_LAUNCH = -1, -2, -3, -4, -5
Q_1, Q_2, Q_INF = 1, 2, 0
LAYOUT_NATURAL, LAYOUT_TRANSPOSED = 0, 1
OP_RELU, OP_TANH, OP_EXP, OP_RECIPROCAL, OP_SQR, OP_SQRT = 1, 2, 3, 4, 5, 6

_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float

# name -> argument types, in the order of include/faith_amd.h
SIGNATURES = {
    "faith_tune_set": [_I, _I],
    "faith_copy_f32": [_P, _P, ctypes.c_longlong, _P],
    "faith_mfma_clock": [_P, _I, _I, _P],
    "faith_concretize": [_P] * 6 + [_I, _I, _I, _F, _I, _I, _I, _P],
    "faith_relu_verification": [_P] * 10 + [_I, _I, _I, _F, _I, _I, _I, _P],
    "faith_tanh_verification": [_P] * 10 + [_I, _I, _I, _F, _I, _I, _I, _P],
    "faith_unary_verification": [_I] + [_P] * 10 + [_I, _I, _I, _F, _I, _I, _I, _P],
    "faith_multiply_verification": [_P] * 12 + [_I, _I, _I, _F, _I, _I, _P],
    "faith_affine_verification": [_P] * 5 + [_F] + [_P] * 9 + [ctypes.c_longlong, ctypes.c_longlong, _I, _P],
    "faith_rows_gather": [_P] * 5 + [_I] * 4 + [_P],
    "faith_rows_put": [_P] * 7 + [_I] * 4 + [_P],
    "faith_rows_spread": [_P] * 3 + [_I] * 3 + [ctypes.c_longlong, _P],
    "faith_concretize_rows": [_P] * 7 + [_I] * 5 + [_F, _I, _I, _P],
    "faith_input_coefficients": [_P] * 3 + [_F] + [_I] * 5 + [_P],
    "faith_flag_below": [_P, _P, _I, ctypes.c_longlong, _F, _I, _P],
    "faith_verdict": [_P] * 4 + [_I, ctypes.c_longlong, _I, _P],
    "faith_rowsum_verification": [_P] * 8 + [ctypes.c_longlong, ctypes.c_longlong, _I, _P],
    "faith_rowmean_verification": [_P] * 8 + [ctypes.c_longlong, ctypes.c_longlong, _I, _P],
    "faith_layer_norm_verification": [_P] * 14 + [ctypes.c_longlong, ctypes.c_longlong, _I, _P],
    "faith_softmax_verification": [_P] * 9 + [_F, _I, _I, _I, _F, _I, _I, _P],
    "faith_softmax_fits": [_I, _I],          # a predicate: returns 1 / 0, not a status (call it through lib)
    "faith_interval_unary": [_I, _P, _P, _P, _P, ctypes.c_longlong, _P],
    "faith_interval_product": [_P] * 6 + [ctypes.c_longlong, _P],
    "faith_matmul_verification": [_P] * 10 + [_I] * 5 + [_P],
    "faith_matmul_concretize_verification": [_P] * 12 + [_I] * 5 + [_F, _I, _I, _P],
    "faith_matmul_group_verification": [_P] * 4 + [_I] + [_P] * 6 + [_I] * 5 + [_P],
    "faith_matmul_relu_fits": [ctypes.c_longlong] + [_I] * 4,           # answers 0 / 1 / 2 as well
    "faith_matmul_relu_verification": [_P] * 10 + [_I] * 5 + [_F, _I, _I, _P],
    "faith_matmul_layer_norm_fits": [ctypes.c_longlong] + [_I] * 4,     # answers 0 / 1 / 2 instead of a status: call it through `lib`
    "faith_matmul_layer_norm_verification": [_P] * 11 + [_I] + [_P] * 6 + [_I] * 5 + [_P],
    "faith_matmul_rows_verification": [_P] * 10 + [ctypes.c_longlong, ctypes.c_longlong, _I, _I, _P],
    "faith_matmul_group_rows_verification": [_P] * 4 + [_I] + [_P] * 6 + [ctypes.c_longlong, ctypes.c_longlong, _I, _I, _P],
    "faith_dot_product_verification_QK": [_P] * 16 + [_I] * 5 + [_F, _I, _I, _I, _P],
    "faith_dot_product_verification_QK_static": [_P] * 12 + [_I] * 5 + [_F, _I, _I, _I, _P],
    "faith_dot_product_verification_V": [_P] * 16 + [_I] * 5 + [_F, _I, _I, _I, _P],
    "faith_attention_scores": [_P] * 16 + [_I] * 6 + [_F, _I, _I, _P],
    "faith_attention_scores_compact": [_P] * 16 + [_I] * 6 + [_P],
    "faith_attention_context_compact": [_P] * 17 + [_I] * 7 + [_F, _I, _I, _P],
    "faith_attention_context": [_P] * 16 + [_I] * 6 + [_F, _I, _I, _P],
    "faith_convolution_verification": [_P] * 10 + [_I] * 9 + [_P],
}


class FaithError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, fn, code, msg):
        super().__init__(f"{fn} failed with status {code}: {msg}")
        self.code = code


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: the HIP library is not built "
            "(run `python -m faith_amd.build`); there is no CPU fallback")
    lib = ctypes.CDLL(LIB_PATH)
    lib.faith_last_error.restype = ctypes.c_char_p
    lib.faith_last_error.argtypes = []
    lib.faith_version.restype = _I
    lib.faith_version.argtypes = []
    lib.faith_static_scratch_bytes.restype = ctypes.c_longlong
    lib.faith_static_scratch_bytes.argtypes = []
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is missing
        fn.restype = _I
        fn.argtypes = argtypes
    return lib


lib = _load()


_ENTRY = {name: getattr(lib, name) for name in SIGNATURES}


def call(name, *args):
    """Invoke an entry point; raise FaithError on a non-zero status."""
    rc = _ENTRY[name](*args)
    if rc:
        raise FaithError(name, rc, lib.faith_last_error().decode())
