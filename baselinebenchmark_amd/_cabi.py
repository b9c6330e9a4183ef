"""ctypes binding of libsage_mi355x.so (C ABI declared in include/sage_mi355x.h).

Follows the reference's own native-boundary pattern, hipcc -> .so -> ctypes -> extern "C" with raw
data_ptr()s (backends/_hygon/ops/attnres/attnres_hip.py:20-58), except that the library is built
ahead of time (``python -m baselinebenchmark_amd.build``) and a missing library is an error: there
is no fallback path of any kind.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

import os

# SAGE_MI355X_LIB selects another build of the same library (the timing build); there is still no fallback.
LIB_PATH = Path(os.environ.get("SAGE_MI355X_LIB") or Path(__file__).resolve().parent / "csrc" / "libsage_mi355x.so")

SAGE_OK, SAGE_EINVAL, SAGE_ETYPE, SAGE_ENOTIMPL, SAGE_ELAUNCH, SAGE_EWORKSPACE = 0, -1, -2, -3, -4, -5
DT_F16, DT_BF16 = 0, 1
PV_FP16, PV_FP8 = 0, 1
PANEL_ROWS = 128

_I, _L, _P = c_int, c_int64, c_void_p

# name -> (restype, argtypes); one entry per declaration in include/sage_mi355x.h
SIGNATURES = {
    "sage_backend_name": (c_char_p, []),
    "sage_last_error": (c_char_p, []),
    "sage_quant_int8": (c_int, [_P, _P, _P, _P, _I, _I, _I, _I, _L, _L, _L, _L, _L, _L, _L, _L, _I, c_float, _I,
                                _P, _P, _L, _P]),
    "sage_k_mean_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "sage_k_mean": (c_int, [_P, _P, _P, c_size_t, _I, _I, _I, _I, _L, _L, _L, _I, _P, _P]),
    "sage_prep_v_workspace_bytes": (c_size_t, [_I, _I, _I, _I, _I]),
    "sage_v_panel_bytes": (c_size_t, [_I, _I, _I, _I, _I]),
    "sage_prep_v": (c_int, [_P, _P, _P, _P, c_size_t, _I, _I, _I, _I, _L, _L, _L, _I, _I, _P, _P, _L, _P]),
    "sage_varlen_plan_ints": (c_size_t, [_I, _I]),
    "sage_varlen_plan_offsets": (None, [_I, _I, ctypes.POINTER(c_int64)]),
    "sage_varlen_plan": (c_int, [_P, _P, _I, _I, _I, _I, _I, _P, c_size_t, _P]),
    "sage_attn_fwd": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I,
                              _L, _L, _L, _L, _L, _L, _L, _L, _L, _I, _I, _I, _I, _I, _P, _P, _P, _I, _L, _L, _L, _P]),
    "sage_attn_fwd_qfused": (c_int, [_P, _I, c_double, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I,
                                     _L, _L, _L, _L, _L, _L, _L, _L, _L, _I, _I, _I, _I, _I, _P, _P, _P, _I, _L, _L, _P]),
    "sage_attn_fwd_masked": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I,
                                     _L, _L, _L, _L, _L, _L, _L, _L, _L, _I, _I, _I, _I, _P, _I, _L, _L, _L, _L, _P]),
    "sage_sageattn_workspace_bytes": (c_size_t, [_I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I]),
    "sage_sageattn_workspace_bytes_for": (c_size_t, [_I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I, _I]),
    "sage_sageattn": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, _I, _I, _I, _I, _I, _I,
                              _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L,
                              _I, _I, _I, c_double, _I, _I, _I, _P, _P, _I, _I, _P]),
    "sage_sageattn_static_capacity": (c_size_t, []),
    "sage_sageattn_static": (c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I,
                                     _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L,
                                     _I, _I, _I, c_double, _I, _I, _I, _P, _P, _I, _I, _P]),
    "sage_sageattn_masked": (c_int, [_P, _P, _P, _P, _P, _P, c_size_t, _I, _I, _I, _I, _I, _I,
                                     _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L, _L,
                                     _I, _I, _I, c_double, _I, _I, _I, _P, _P, _I, _I,
                                     _P, _I, _L, _L, _L, _L, _P]),
}

_lib = None


class SageLibraryMissing(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """Load the library once.  Raises SageLibraryMissing if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise SageLibraryMissing(
            f"{LIB_PATH} is missing: build it with `python -m baselinebenchmark_amd.build` "
            "(there is no fallback implementation)")
    handle = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = handle
    return _lib


_ERRORS = {SAGE_EINVAL: ValueError, SAGE_ETYPE: TypeError, SAGE_ENOTIMPL: NotImplementedError,
           SAGE_ELAUNCH: RuntimeError, SAGE_EWORKSPACE: RuntimeError}


def check(rc: int) -> None:
    """Map a negative return code to the exception class the reference raises for that kind of error
    (backends/_enflame/ops/sage_attention/attn_qk_int8_per_block_native.py:212-276,
    backends/_hygon/ops/sageattention/sageattention_hip.py:30-74)."""
    if rc != SAGE_OK:
        msg = lib().sage_last_error().decode()
        raise _ERRORS.get(rc, RuntimeError)(msg)
