"""ctypes binding of libpikv_hip.so (the C ABI declared in include/pikv_hip.h).

The library is the only compute path of this package: if it is missing, or a
call returns a non-zero status, an exception is raised.  There is no CPU or
PyTorch fallback.  The reference's binding precedent is PiKVKernels.__init__
(core/single/pikv_kernels.py:36-52), which resolves the shared library next to
the package and silently falls back to torch when it is absent; here the
absence is an error.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("PIKV_HIP_LIB", os.path.join(_HERE, "libpikv_hip.so"))

# element types / schemes / policies (mirrors include/pikv_hip.h)
F32, BF16 = 0, 1
Q_I8_SYM, Q_I8_ASYM, Q_I4_ASYM, Q_I4_SYM = 0, 1, 2, 3
EVICT_H2O, EVICT_LRU = 0, 1
SCORE_TILE = 64
MAX_PLANES = 10

_p, _i, _l, _f, _d = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_double

# name -> (restype, argtypes)
SIGNATURES = {
    "pikv_status_string": (C.c_char_p, [_i]),
    "pikv_abi_version": (_i, []),
    "pikv_router_fused": (_i, [_p, _p, _i, _p, _p, _p, _f, _f, _i, _l, _i, _i, _i, _l,
                               _p, _p, _p, _p, _p, _p, _p, _l, _p]),
    "pikv_router_tail": (_i, [_p, _p, _p, _p, _p, _f, _f, _i, _i, _l, _i, _i, _l,
                              _p, _p, _p, _p, _p, _p, _l, _p]),
    "pikv_capacity_slots": (_i, [_p, _l, _i, _l, _p, _p, _p, _l, _p]),
    "pikv_capacity_slots_static": (_i, [_p, _l, _i, _l, _p, _p, _p]),
    "pikv_capacity_slots_static_max": (_l, []),
    "pikv_router_workspace_bytes": (_l, [_l, _i, _i]),
    "pikv_router_fused_workspace_bytes": (_l, [_l, _i, _i, _i]),
    "pikv_quant_scatter": (_i, [_p, _p, _i, _l, _i, _i, _i, _i, _p, _p, _p, _p, _p, _i,
                                _p, _p, _p, _p, _p, _p, _p, _p, _f, _p]),
    "pikv_cache_advance": (_i, [_p, _p, _p, _i, _l, _p]),
    "pikv_quant_gather": (_i, [_p, _p, _i, _i, _i, _i, _p, _p, _p, _l, _p, _p, _p, _p, _i,
                               _p, _p, _p, _p, _p, _p, _p, _p, _f, _p]),
    "pikv_quantize_rows": (_i, [_p, _i, _l, _i, _i, _i, _l, _p, _p, _p, _p]),
    "pikv_quant8_minshift": (_i, [_p, _i, _l, _i, _p, _p, _p, _p, _p]),
    "pikv_gather_dequant": (_i, [_p, _p, _p, _i, _i, _i, _p, _l, _l, _p, _i, _p]),
    "pikv_gather_dequant_scores": (_i, [_p, _p, _p, _i, _i, _i, _i, _i, _p, _i, _f,
                                        _p, _p, _i, _l, _l, _p, _p, _p, _p]),
    "pikv_h2o_accumulate": (_i, [_p, _p, _p, _i, _p, _p, _i, _l, _l, _f, _f, _i,
                                 _p, _p, _p, _p, _p]),
    "pikv_attend_values": (_i, [_p, _p, _l, _p, _p, _p, _i, _i, _i, _i, _i, _p, _p, _i, _l,
                                _f, _f, _p, _p, _p, _p, _l, _p]),
    "pikv_attend_workspace_bytes": (_l, [_i, _i, _i, _l]),
    "pikv_decode_attend": (_i, [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _p, _i, _f, _p, _p, _i, _l,
                                _f, _f, _p, _p, _p, _p, _l, _p]),
    "pikv_decode_attend_workspace_bytes": (_l, [_i, _i, _i, _l]),
    "pikv_evict_select": (_i, [_i, _p, _p, _p, _p, _p, _p, _i, _l, _p, _p, _p, _p, _l, _p]),
    "pikv_evict_workspace_bytes": (_l, [_i, _l]),
    "pikv_h2o_budget": (_i, [_p, _i, _d, _d, _p, _p, _p]),
    "pikv_compact_rows": (_i, [C.POINTER(_p), C.POINTER(_l), _i, _p, _p, _p, _p, _i, _p]),
    "pikv_fakequant_colblocks": (_i, [_p, _l, _i, _i, _i, _i, _p, _p, _p, _p, _l, _p]),
    "pikv_fakequant_workspace_bytes": (_l, [_l, _i, _i]),
    "pikv_fakequant_preset": (_i, [_p, _l, _i, _i, _i, _i, _p, _p, _p, _p, _l, _p]),
}

_lib = None
_lock = threading.Lock()


class PiKVNativeError(RuntimeError):
    """The native library is missing or returned an error status."""


def lib() -> C.CDLL:
    """Load libpikv_hip.so once; raise if it is not built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise PiKVNativeError(
                        f"{LIB_PATH} not found: build it with `python -m pikv_amd.build` "
                        "(there is no CPU fallback)")
                handle = C.CDLL(LIB_PATH)
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype = res
                    fn.argtypes = args
                _lib = handle
    return _lib


def status_string(code: int) -> str:
    return lib().pikv_status_string(int(code)).decode()


def check(code: int, what: str) -> None:
    if code != 0:
        raise PiKVNativeError(f"{what} failed: {status_string(code)} (status {code})")


def call(name: str, *args) -> None:
    """Call an int-status entry point and raise on a non-zero status."""
    check(getattr(lib(), name)(*args), name)
