"""ctypes binding of libdeepep_amd.so — the C-ABI declared in include/deepep_amd.h.

There is no fallback: if the library is missing or a symbol is absent, loading raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdeepep_amd.so")

_P = ctypes.c_void_p
_I = ctypes.c_int
_Z = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/deepep_amd.h one to one.
SIGNATURES = {
    "dpep_last_error": (ctypes.c_char_p, ()),
    "dpep_version": (_I, ()),
    "dpep_workspace_create": (_I, (_Z, ctypes.POINTER(_P))),
    "dpep_workspace_destroy": (_I, (_P,)),
    "dpep_workspace_capacity": (_I, (_P, ctypes.POINTER(_Z))),
    "dpep_workspace_tune": (_I, (_P, ctypes.c_char_p, ctypes.c_longlong)),
    "dpep_layout_workspace_bytes": (_Z, (_I, _I, _I)),
    "dpep_layout": (_I, (_P, _P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P)),
    "dpep_layout_static": (_I, (_P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P)),
    "dpep_layout_wait": (_I, (_P, _P, _I, ctypes.POINTER(ctypes.c_int32), ctypes.c_longlong)),
    "dpep_dispatch_store_policy": (_I, (_I,)),
    "dpep_dispatch_copy": (_I, (_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P, _P, _P)),
    "dpep_dispatch_quant_fp8": (_I, (_P, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P)),
    "dpep_layout_dispatch_small": (_I, (_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P)),
    "dpep_cast_to_fp8": (_I, (_P, _I, _I, _P, _P, _P)),
    "dpep_cast_back": (_I, (_P, _P, _I, _I, _I, _P, _P)),
    "dpep_combine": (_I, (_P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P)),
    "dpep_combine_fp16": (_I, (_P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P)),
    "dpep_combine_served": (_I, (_P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P)),
    "dpep_mx_quant": (_I, (_P, _I, _I, _P, _P, _P)),
    "dpep_megamoe_schedule_check": (_I, (_I, _I, _I, _I, _I)),
    "dpep_megamoe_schedule_check_column_waves": (_I, (_I, _I, _I, _I, _I)),
    "dpep_megamoe_workspace_bytes": (_Z, (_I, _I, _I, _I, _I, _I)),
    "dpep_megamoe_padded_dim": (_I, (_I,)),
    "dpep_megamoe_prepared_shape": (_I, (_I, _I, _I, ctypes.POINTER(_I), ctypes.POINTER(_I), ctypes.POINTER(_I))),
    "dpep_megamoe_prepare_weights": (_I, (_P, _P, _I, _I, _I, _I, _P, _P, _P)),
    "dpep_megamoe_fill_report": (_I, (_P, _I, _I, _I, _I, _I, _I, ctypes.POINTER(ctypes.c_int32),
                                      ctypes.POINTER(ctypes.c_int64), _P)),
    "dpep_megamoe_forward": (_I, (_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I,
                                  _P, _P, _P)),
}

_lock = threading.Lock()
_lib = None


def load():
    """Load the shared library once and attach the prototypes.  Raises if it is not built."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise ImportError(
                    f"{LIB_PATH} is missing: build it with `python -m deepep_amd.build` "
                    "(there is no CPU or eager fallback for the dispatch/combine path)"
                )
            lib = ctypes.CDLL(LIB_PATH)
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)  # AttributeError if the export is missing
                fn.restype = restype
                fn.argtypes = list(argtypes)
            _lib = lib
    return _lib


class NativeError(RuntimeError):
    pass


def check(status: int, what: str) -> None:
    """Status -> exception, following csrc/ops: invalid argument -> ValueError, runtime -> RuntimeError."""
    if status == 0:
        return
    message = load().dpep_last_error().decode("utf-8", "replace")
    if not message.startswith(what):
        message = f"{what}: {message}"
    if status == -1:
        raise ValueError(message)
    raise NativeError(message)
