"""ctypes binding of libbased_hip.so (the C ABI declared in include/based_hip.h).

The library is loaded lazily; there is no fallback path.  If the shared object is missing
the first use raises, so a GPU run can never silently go through something else.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbased_hip.so")  # the in-tree build is the only library ever loaded

BASED_BF16 = 0
BASED_F32 = 1
PREFILL_SEGMENT_STATE_BYTES = 43008  # BASED_PREFILL_SEGMENT_STATE_BYTES of include/based_hip.h

_I64 = C.c_int64
_P = C.c_void_p

# name -> (restype, argtypes); must list every symbol declared in include/based_hip.h
SIGNATURES = {
    "based_hip_version": (C.c_int, []),
    "based_hip_last_error": (C.c_char_p, []),
    "based_linear_attn_step": (
        C.c_int,
        [_P, _P, _P, _P, _P, _P] + [_I64] * 3 + [_I64] * 8 + [C.c_float, C.c_int, _P],
    ),
    "based_linear_attn_step_deferred": (
        C.c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, _P] + [_I64] * 3 + [_I64] * 8 + [C.c_float, C.c_int, C.c_int, _P],
    ),
    "based_linear_attn_flush_deferred": (C.c_int, [_P, _P, _P, _P] + [_I64] * 3 + [_P]),
    "based_linear_attn_prefill": (
        C.c_int,
        [_P, _P, _P, _P, _P, _P] + [_I64] * 4 + [_I64] * 12 + [C.c_float, C.c_int, _P],
    ),
    "based_linear_attn_prefill_plan": (
        C.c_int,
        [_I64] * 4 + [C.c_int, C.POINTER(_I64), C.POINTER(_I64)],
    ),
    "based_linear_attn_prefill_split": (
        C.c_int,
        [_P, _P, _P, _P, _P, _P] + [_I64] * 4 + [_I64] * 12 + [C.c_float, C.c_int, _I64, _P, _I64, _P],
    ),
    "based_linear_attn_prefill_split_static": (
        C.c_int,
        [_P, _P, _P, _P, _P, _P] + [_I64] * 4 + [_I64] * 12 + [C.c_float, C.c_int, _I64, _P],
    ),
    "based_swa_prefill": (
        C.c_int,
        [_P, _P, _P, _P] + [_I64] * 3 + [_I64] * 12 + [C.c_int, C.c_float]
        + [_P, _P, _I64] + [_P, _P] + [_I64] * 4 + [C.c_int, _P],
    ),
    "based_gated_conv_prefill": (
        C.c_int,
        [_P, _P, _P, _P, _P] + [_I64] * 3 + [C.c_int] + [_I64] * 4 + [C.c_int, C.c_int, _P],
    ),
    "based_gated_conv_step": (
        C.c_int,
        [_P, _P, _P, _P, _P] + [_I64] * 2 + [C.c_int] + [_I64] * 2 + [C.c_int, C.c_int, _P],
    ),
    "based_swa_prefill_anydim": (
        C.c_int,
        [_P, _P, _P, _P] + [_I64] * 4 + [_I64] * 12 + [C.c_int, C.c_float] + [_P, _P] + [_I64] * 4 + [C.c_int, _P],
    ),
    "based_swa_prefill_wide": (
        C.c_int,
        [_P, _P, _P, _P] + [_I64] * 4 + [_I64] * 12 + [C.c_int, C.c_float] + [_P, _P, _I64, _I64, C.c_int]
        + [_P, _P] + [_I64] * 4 + [C.c_int, _P],
    ),
    "based_swa_step_wide": (
        C.c_int,
        [_P] * 6 + [_P, _I64] + [_I64] * 4 + [_I64] * 8 + [_I64] * 3 + [C.c_int, C.c_float]
        + [_P, _P, _I64, _I64, C.c_int] + [C.c_int, _P],
    ),
    "based_greedy_step": (C.c_int, [_P, _I64, _I64, _I64, _P, _I64, _P, _I64, _I64, _P, _P, _I64, C.c_int, _P]),
    "based_swa_step_anydim": (
        C.c_int,
        [_P] * 6 + [_P, _I64] + [_I64] * 4 + [_I64] * 8 + [_I64] * 3 + [C.c_int, C.c_float, C.c_int, _P],
    ),
    "based_short_conv_prefill": (
        C.c_int,
        [_P, _P, _P, _P, _P] + [_I64] * 3 + [C.c_int] + [_I64] * 4 + [C.c_int, C.c_int, _P],
    ),
    "based_short_conv_step": (
        C.c_int,
        [_P, _P, _P, _P, _P] + [_I64] * 2 + [C.c_int] + [_I64] * 2 + [C.c_int, C.c_int, _P],
    ),
    "based_add_rms_norm": (
        C.c_int,
        [_P, _P, _P, _P, _P] + [_I64] * 6 + [C.c_float, C.c_int, C.c_int, _P],
    ),
    "based_swiglu": (C.c_int, [_P, _P] + [_I64] * 4 + [C.c_int, _P]),
    "based_decode_linear": (C.c_int, [_P, _I64, _P, _I64, _P, _I64, _P, _P, _I64, _I64, _I64, _I64, C.c_int,
                                      _P, _I64, _P, _I64, _P, C.c_float, C.c_int, _P, C.c_int, _P, _P, C.c_int, _P]),
    "based_swa_step": (
        C.c_int,
        [_P, _P, _P, _P, _P, _P, _P, _I64] + [_I64] * 3 + [_I64] * 8 + [_I64] * 3
        + [C.c_int, C.c_float] + [_P, _P, _I64] + [C.c_int, _P],
    ),
}

_lib = None
_lock = threading.Lock()


class BasedHipError(RuntimeError):
    """Raised when the native library is missing or a launch is refused by the runtime."""


def lib():
    """Returns the loaded library, loading and typing it on first use."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise BasedHipError(
                        f"{LIB_PATH} not found: build it with `python -m based_amd.build` "
                        "(there is no non-HIP fallback)"
                    )
                handle = C.CDLL(LIB_PATH)
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype = res
                    fn.argtypes = args
                _lib = handle
    return _lib


_SHAPE_CODES = (1, 2, 3)  # BASED_ERR_SHAPE / DTYPE / ALIGN -> ValueError, like the reference's
                          # "implementation not supported" ValueError (linear_attention.py:217-218)


def check(code: int) -> None:
    if code == 0:
        return
    msg = lib().based_hip_last_error().decode("utf-8", "replace")
    if code in _SHAPE_CODES or code == 4:
        raise ValueError(msg)
    raise BasedHipError(msg)
