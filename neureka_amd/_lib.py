"""ctypes binding of ``libneureka_hip.so`` (the C ABI declared in ``include/neureka_hip.h``).

The same symbols a JVM host would bind through Panama or JNI.  There is no fallback: if the library is
missing, or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libneureka_hip.so")

F32, F64 = 0, 1
OP = {"add": 0, "subtract": 1, "multiply": 2, "divide": 3, "modulo": 4, "power": 5, "idy": 6}
FUN = {name: i for i, name in enumerate(
    ["abs", "cos", "gasu", "gatu", "gaus", "fast_gaus", "gelu", "idy", "ln", "quad", "relu", "selu", "sig", "silu",
     "sin", "softplus", "softsign", "tanh", "fast_tanh", "exp", "log10", "sqrt", "cbrt"])}
FUSE_LOAD, FUSE_CONST, FUSE_FUN, FUSE_DFUN, FUSE_BIN = 0, 1, 2, 3, 4
ROW_MAJOR, COLUMN_MAJOR = 0, 1

# every symbol include/neureka_hip.h declares: name -> (restype, argtypes)
_u64, _i64, _i32, _p = C.c_uint64, C.c_int64, C.c_int, C.c_void_p
_cfg = C.POINTER(C.c_int32)
SYMBOLS = {
    "nk_last_error": (C.c_char_p, []),
    "nk_last_path": (C.c_char_p, []),
    "nk_device_count": (_i32, [C.POINTER(C.c_int)]),
    "nk_device_open": (_i32, [_i32, C.POINTER(_u64)]),
    "nk_device_close": (_i32, [_u64]),
    "nk_device_sync": (_i32, [_u64]),
    "nk_device_props": (_i32, [_u64, C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(_u64),
                               C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "nk_device_memory": (_i32, [_u64, C.POINTER(_u64), C.POINTER(_u64)]),
    "nk_device_stats": (_i32, [_u64, C.POINTER(_u64), C.POINTER(_u64)]),
    "nk_alloc": (_i32, [_u64, _u64, C.POINTER(_u64)]),
    "nk_free": (_i32, [_u64, _u64]),
    "nk_pool_trim": (_i32, [_u64]),
    "nk_pool_stats": (_i32, [_u64, C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_u64)]),
    "nk_pool_config": (_i32, [_u64, _u64, _i32]),
    "nk_h2d": (_i32, [_u64, _u64, _u64, _p, _u64]),
    "nk_d2h": (_i32, [_u64, _p, _u64, _u64, _u64]),
    "nk_d2d": (_i32, [_u64, _u64, _u64, _u64, _u64, _u64]),
    "nk_fill": (_i32, [_u64, _u64, _u64, _p, _i32, _u64]),
    "nk_event_create": (_i32, [_u64, C.POINTER(_u64)]),
    "nk_event_record": (_i32, [_u64, _u64]),
    "nk_event_elapsed_ms": (_i32, [_u64, _u64, _u64, C.POINTER(C.c_float)]),
    "nk_event_destroy": (_i32, [_u64, _u64]),
    "nk_activation": (_i32, [_u64, _i32, _i32, _i32, _i32, _u64, _cfg, _u64, _cfg, _i64]),
    "nk_elementwise": (_i32, [_u64, _i32, _i32, _i32, _i32, _u64, _cfg, _u64, _cfg, _u64, _cfg, _i64]),
    "nk_scalarization": (_i32, [_u64, _i32, _i32, _i32, _i32, _u64, _cfg, _u64, _cfg, C.c_double, _i64]),
    "nk_scalar_fill": (_i32, [_u64, _i32, _i32, _u64, _cfg, C.c_double, _i64]),
    "nk_broadcast": (_i32, [_u64, _i32, _i32, _i32, _i32, _u64, _cfg, _u64, _cfg, _u64, _cfg, _i64]),
    "nk_convolution": (_i32, [_u64, _i32, _i32, _i32, _u64, _cfg, _u64, _cfg, _u64, _cfg, _i64]),
    "nk_matmul": (_i32, [_u64, _i32, _i32, _i64, _i64, _i64, _u64, _u64, _u64]),
    "nk_matmul_set": (_i32, [_u64, _i32, _i32, _i64, _i64, _i64, _u64, _u64, _u64]),
    "nk_scalarization_int": (_i32, [_u64, _i32, _i32, _i32, _i32, _u64, _cfg, _u64, _cfg, _i64, _i64]),
    "nk_sum": (_i32, [_u64, _i32, _u64, _i64, _u64]),
    "nk_sum_static": (_i32, [_u64, _i32, _u64, _i64, _u64]),
    "nk_reduce_index": (_i32, [_u64, _i32, _i32, _u64, _i64, _u64]),
    "nk_dot": (_i32, [_u64, _i32, _u64, _u64, _i64, _u64]),
    "nk_fused": (_i32, [_u64, C.POINTER(C.c_int32), _i32, C.POINTER(C.c_double), _i32, _i32, _i32, _u64, _cfg, _i32,
                        C.POINTER(_u64), C.POINTER(_cfg), _i64]),
}


class HipError(RuntimeError):
    """A call into libneureka_hip.so returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"[{status}] {message}")
        self.status = status


_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """Loads the in-tree library and binds every declared symbol; raises if anything is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()' "
            "or make -C neureka_amd/csrc). There is no CPU fallback."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SYMBOLS.items():
        fn = getattr(lib, name)          # AttributeError if the export is missing
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != 0:
        raise HipError(status, load().nk_last_error().decode("utf-8", "replace"))


def last_path() -> str:
    return load().nk_last_path().decode()


def cfg_ptr(inline):
    """``inline`` is a contiguous int32 numpy array (NDConfiguration.asInlineArray())."""
    return inline.ctypes.data_as(_cfg)
