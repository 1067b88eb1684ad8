"""ctypes binding of libof3pair.so (declared in include/of3pair.h).

There is no fallback: if the library has not been built, or a call returns a non-zero
status, the caller gets an exception.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

from . import build as _build
from .build import LIB_PATH

OF3_OK, OF3_EINVAL, OF3_ENOSPC, OF3_EHIP, OF3_ESTATIC = 0, -1, -2, -3, -4
OF3_STATIC_SCRATCH_BYTES = 48 << 20
OF3_DTYPE_F32, OF3_DTYPE_BF16 = 0, 1

_I64x3 = ctypes.POINTER(c_int64)

# name -> (restype, argtypes); mirrors include/of3pair.h one to one
SIGNATURES = {
    "of3_version": (c_int, []),
    "of3_last_hip_error": (c_int, []),
    "of3_status_string": (c_char_p, [c_int]),
    "of3_padded_n": (c_int64, [c_int64]),
    "of3_trimul_workspace_bytes": (c_int64, [c_int64] * 4),
    "of3_trimul_workspace_bytes_for": (c_int64, [c_int] + [c_int64] * 4),
    "of3_trimul_proj": (c_int, [c_void_p, _I64x3, c_void_p, _I64x3] + [c_void_p] * 8 + [c_int64] * 4 + [c_int, c_void_p]),
    "of3_trimul_contract": (c_int, [c_void_p] * 3 + [c_int64] * 3 + [c_int, c_void_p]),
    "of3_trimul_contract_variant": (c_int, [c_int64] * 3),
    "of3_trimul_out": (c_int, [c_void_p, c_void_p, _I64x3] + [c_void_p] * 7 + [c_int64] * 4 + [c_int, c_void_p]),
    "of3_trimul_fwd": (c_int, [c_void_p, _I64x3, c_void_p, _I64x3] + [c_void_p] * 11 + [c_int64] * 4
                       + [c_int, c_int, c_void_p, c_int64, c_int, c_void_p]),
    "of3_trimul_fwd_static": (c_int, [c_void_p, _I64x3, c_void_p, _I64x3] + [c_void_p] * 11 + [c_int64] * 4
                              + [c_int, c_int, c_int, c_void_p]),
    "of3_triattn_workspace_bytes": (c_int64, [c_int64] * 5),
    "of3_triattn_workspace_bytes_for": (c_int64, [c_int] + [c_int64] * 5),
    "of3_triattn_proj": (c_int, [c_void_p, _I64x3, c_void_p, _I64x3] + [c_void_p] * 11 + [c_int64] * 5
                         + [c_float, c_void_p]),
    "of3_triattn_flash": (c_int, [c_void_p] * 6 + [c_int64] * 4 + [c_void_p]),
    "of3_triattn_out": (c_int, [c_void_p, c_void_p, _I64x3] + [c_void_p] * 5 + [c_int64] * 5 + [c_int, c_void_p]),
    "of3_triattn_fwd": (c_int, [c_void_p, _I64x3, c_void_p, _I64x3] + [c_void_p] * 9 + [c_int64] * 5
                        + [c_float, c_int, c_void_p, c_int64, c_int, c_void_p]),
    "of3_transition_fwd": (c_int, [c_void_p, _I64x3, c_void_p, _I64x3] + [c_void_p] * 6 + [c_int64] * 4
                           + [c_int, c_int, c_void_p]),
    "of3_transition_workspace_bytes_for": (c_int64, [c_int] + [c_int64] * 4),
    "of3_transition_fwd_ws": (c_int, [c_void_p, _I64x3, c_void_p, _I64x3] + [c_void_p] * 6 + [c_int64] * 4
                              + [c_int, c_void_p, c_int64, c_int, c_void_p]),
    "of3_pair_bias_fwd": (c_int, [c_void_p, _I64x3] + [c_void_p] * 4 + [c_int64] * 4 + [c_int, c_void_p]),
    "of3_attn_pair_bias_workspace_bytes": (c_int64, [c_int64] * 5),
    "of3_attn_pair_bias_workspace_bytes_for": (c_int64, [c_int] + [c_int64] * 5),
    "of3_transition_rows_workspace_bytes_for": (c_int64, [c_int] + [c_int64] * 3),
    "of3_attn_pair_bias_fwd": (c_int, [c_void_p] * 12 + [c_int64] * 5 + [ctypes.c_float, c_int, c_void_p, c_int64, c_int,
                                                                    c_void_p]),
    "of3_transition_rows_workspace_bytes": (c_int64, [c_int64] * 3),
    "of3_transition_rows_fwd": (c_int, [c_void_p] * 8 + [c_int64] * 3 + [c_int, c_void_p, c_int64, c_int, c_void_p]),
    "of3_layer_norm_fwd": (c_int, [c_void_p] * 4 + [c_int64] * 2 + [c_int, c_void_p]),
    "of3_template_tail_fwd": (c_int, [c_void_p] * 5 + [c_int64] * 5 + [c_int, c_int, c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libof3pair.so is not built (%s); build it with `python -m of3pair.build`" % LIB_PATH)
        if LIB_PATH == _build.LIB_PATH and _build.is_stale():
            raise RuntimeError(
                "libof3pair.so is older than its sources (%s was edited after the build); rebuild it with "
                "`python -m of3pair.build`" % _build.CSRC)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def strides3(values):
    return (c_int64 * 3)(*[int(v) for v in values])


def check(status: int, what: str):
    """Error convention of the reference's alternative-kernel wrappers: unsupported shapes
    raise ValueError (tmu.py:707-712, attention.py:346-350); anything else is a RuntimeError."""
    if status == OF3_OK:
        return
    lib = load()
    msg = "%s: %s" % (what, lib.of3_status_string(status).decode())
    if status in (OF3_EINVAL, OF3_ESTATIC):
        raise ValueError(msg)
    if status == OF3_EHIP:
        msg += " (hipError %d)" % lib.of3_last_hip_error()
    raise RuntimeError(msg)
