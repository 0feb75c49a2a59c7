"""ctypes wrapper of the CPU oracle (``neureka_cpu_oracle.c``) — TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this
module.  Operands are flat numpy backing arrays plus inline view descriptors
(``shape | strides | indicesMap | offset | spread``, int32[5*rank]), the same things the HIP library is
given, so that a test feeds both sides identical bytes.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Sequence

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libneureka_cpu_oracle.so")

FUN = {name: i for i, name in enumerate(
    ["abs", "cos", "gasu", "gatu", "gaus", "fast_gaus", "gelu", "idy", "ln", "quad", "relu", "selu", "sig", "silu",
     "sin", "softplus", "softsign", "tanh", "fast_tanh", "exp", "log10", "sqrt", "cbrt"])}
OP = {"add": 0, "subtract": 1, "multiply": 2, "divide": 3, "modulo": 4, "power": 5, "idy": 6}
KIND = {"activation": 0, "elementwise": 1, "scalarization": 2, "broadcast": 3, "convolve": 4, "deconvolve": 5,
        "deconvolve_fast": 6}

_lib = None


def build() -> None:
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        l = C.CDLL(_SO)
        l.orc_fun_f64.restype = C.c_double
        l.orc_fun_f64.argtypes = [C.c_int, C.c_int, C.c_double]
        l.orc_fun_f32.restype = C.c_float
        l.orc_fun_f32.argtypes = [C.c_int, C.c_int, C.c_float]
        l.orc_bin_f64.restype = C.c_double
        l.orc_bin_f64.argtypes = [C.c_int, C.c_int, C.c_int, C.c_double, C.c_double]
        l.orc_bin_f32.restype = C.c_float
        l.orc_bin_f32.argtypes = [C.c_int, C.c_int, C.c_int, C.c_float, C.c_float]
        l.orc_long_string_hash.restype = C.c_int64
        l.orc_long_string_hash.argtypes = [C.c_char_p]
        l.orc_initial_scramble.restype = C.c_int64
        l.orc_initial_scramble.argtypes = [C.c_int64]
        l.orc_index_of_index.restype = C.c_int
        l.orc_fill_gaussian.argtypes = [C.c_int, C.c_void_p, C.c_int64, C.c_int, C.c_int]
        l.orc_split_leaves.restype = C.c_int
        l.orc_run_threaded.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.c_void_p, C.c_double, C.c_int, C.c_int, C.c_int]
        l.orc_gemm_threaded.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int]
        l.orc_gemm_partial.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int]
        l.orc_sum_tree.restype = C.c_double
        l.orc_sum_tree.argtypes = [C.c_int, C.c_void_p, C.c_int]
        l.orc_reduce_index.restype = C.c_int
        l.orc_reduce_index.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int]
        l.orc_dot.restype = C.c_double
        l.orc_dot.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int]
        l.orc_scalarization_int.restype = C.c_int
        l.orc_scalarization_int.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int]
        l.orc_simple_conv2d.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        _lib = l
    return _lib


def _cfg(cfg) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(cfg, dtype=np.int32))


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _is64(a: np.ndarray) -> int:
    if a.dtype == np.float64: return 1
    if a.dtype == np.float32: return 0
    raise TypeError(f"oracle handles float32/float64, got {a.dtype}")


def dense_cfg(shape: Sequence[int]) -> np.ndarray:
    """Inline descriptor of a fresh row-major tensor."""
    shape = [int(s) for s in shape]
    strides, p = [0] * len(shape), 1
    for k in reversed(range(len(shape))):
        strides[k] = p
        p *= shape[k]
    return np.array(shape + strides + strides + [0] * len(shape) + [1] * len(shape), dtype=np.int32)


def index_of_index(cfg, index: int) -> int:
    cfg = _cfg(cfg)
    return lib().orc_index_of_index(_p(cfg), len(cfg) // 5, int(index))


def fun(name: str, x, derive: bool = False):
    """Scalar function on a numpy array, elementwise, in the array's dtype."""
    x = np.asarray(x)
    out = np.empty_like(x)
    f = lib().orc_fun_f64 if x.dtype == np.float64 else lib().orc_fun_f32
    flat_in, flat_out = x.reshape(-1), out.reshape(-1)
    for i in range(flat_in.size):
        flat_out[i] = f(FUN[name], int(derive), float(flat_in[i]))
    return out


def _size(cfg: np.ndarray) -> int:
    return int(np.prod(cfg[: len(cfg) // 5]))


def run(kind: str, op: int, d: int, drn: np.ndarray, drn_cfg, a=None, a_cfg=None, b=None, b_cfg=None, value: float = 0.0,
        workers: int = 1, first: int = 0, limit: int = None) -> np.ndarray:
    """Runs one kernel over [first, limit) of the drain's flat index (default: all of it), split over
    `workers` threads the way the reference's executor splits it.  Writes into `drn` and returns it."""
    drn_cfg = _cfg(drn_cfg)
    rank = len(drn_cfg) // 5
    a_cfg = None if a_cfg is None else _cfg(a_cfg)
    b_cfg = None if b_cfg is None else _cfg(b_cfg)
    if limit is None:
        limit = _size(drn_cfg)
    lib().orc_run_threaded(KIND[kind], op, d, _is64(drn), rank, _p(drn), _p(drn_cfg), _p(a), _p(a_cfg), _p(b), _p(b_cfg),
                           float(value), int(first), int(limit), int(workers))
    return drn


def activation(name: str, d: int, drn, drn_cfg, src, src_cfg, **kw):
    return run("activation", FUN[name], d, drn, drn_cfg, src, src_cfg, **kw)


def elementwise(op: str, d: int, drn, drn_cfg, a, a_cfg, b, b_cfg, **kw):
    return run("elementwise", OP[op], d, drn, drn_cfg, a, a_cfg, b, b_cfg, **kw)


def scalarization(op: str, d: int, drn, drn_cfg, src, src_cfg, value: float, **kw):
    return run("scalarization", OP[op], d, drn, drn_cfg, src, src_cfg, value=value, **kw)


ITYPE = {np.dtype(np.int32): 2, np.dtype(np.int64): 3, np.dtype(np.int16): 4, np.dtype(np.int8): 5}


class JavaArithmeticException(ArithmeticError):
    """Where the CPU device throws java.lang.ArithmeticException (integer division by zero)."""


def scalarization_int(op: str, d: int, drn: np.ndarray, drn_cfg, src: np.ndarray, src_cfg, value: int) -> np.ndarray:
    """CPUScalarBroadcast on int32 / int64 / int16 / int8 data; `value` is narrowed to the element type."""
    drn_cfg, src_cfg = _cfg(drn_cfg), _cfg(src_cfg)
    assert drn.dtype == src.dtype and drn.dtype in ITYPE
    value = int(value)
    value = (value + (1 << 63)) % (1 << 64) - (1 << 63)
    thrown = lib().orc_scalarization_int(ITYPE[drn.dtype], OP[op], d, len(drn_cfg) // 5, _p(drn), _p(drn_cfg), _p(src), _p(src_cfg),
                                         value, 0, _size(drn_cfg))
    if thrown:
        raise JavaArithmeticException("/ by zero")
    return drn


def scalar_fill(drn, drn_cfg, value: float):
    drn_cfg = _cfg(drn_cfg)
    lib().orc_scalar_fill(_is64(drn), len(drn_cfg) // 5, _p(drn), _p(drn_cfg), C.c_double(value), 0, _size(drn_cfg))
    return drn


def broadcast(op: str, d: int, drn, drn_cfg, a, a_cfg, b, b_cfg, **kw):
    return run("broadcast", OP[op], d, drn, drn_cfg, a, a_cfg, b, b_cfg, **kw)


def convolve(drn, drn_cfg, a, a_cfg, b, b_cfg, **kw):
    return run("convolve", 0, -1, drn, drn_cfg, a, a_cfg, b, b_cfg, **kw)


def deconvolve(drn, drn_cfg, a, a_cfg, b, b_cfg, fast: bool = False, **kw):
    return run("deconvolve_fast" if fast else "deconvolve", 0, 0, drn, drn_cfg, a, a_cfg, b, b_cfg, **kw)


def simple_conv2d(image: np.ndarray, kernel: np.ndarray, width: int, height: int, kw: int, kh: int, batch: int = 1) -> np.ndarray:
    out = np.zeros(batch * (width - kw + 1) * (height - kh + 1), dtype=image.dtype)
    for bi in range(batch):
        lib().orc_simple_conv2d(_is64(image), _p(image), _p(kernel), _p(out), width, height, kw, kh, bi)
    return out


def sum_tree(data: np.ndarray):
    """CPUSum: tiles of 128 summed front to back, recursively; returns a scalar of the array's dtype."""
    return data.dtype.type(lib().orc_sum_tree(_is64(data), _p(data), data.size))


def reduce_index(kind: str, data: np.ndarray) -> int:
    """CPUReduce: index of the minimum ('min') or maximum ('max') as the reference's tile recursion finds it."""
    return lib().orc_reduce_index({"min": 0, "max": 1}[kind], _is64(data), _p(data), data.size)


def dot(a: np.ndarray, b: np.ndarray):
    """DOT.unrolled04 of two vectors."""
    return a.dtype.type(lib().orc_dot(_is64(a), _p(a), _p(b), a.size))


def gemm(row_major: bool, A: np.ndarray, B: np.ndarray, M: int, K: int, N: int, C_init=None, workers: int = 1) -> np.ndarray:
    """C += A @ B on flat arrays in the given layout, with the reference's loop order."""
    out = np.zeros(M * N, dtype=A.dtype) if C_init is None else C_init
    lib().orc_gemm_threaded(_is64(A), int(row_major), _p(out), _p(A), A.size, K, _p(B), B.size, int(workers))
    return out


def long_string_hash(s: str) -> int:
    return lib().orc_long_string_hash(s.encode())


def seeded(dtype, n: int, seed) -> np.ndarray:
    """``Tensor.of(type).withShape(n).andSeed(seed)`` for Float/Double."""
    if isinstance(seed, str):
        seed = long_string_hash(seed)
    out = np.zeros(n, dtype=dtype)
    lib().orc_fill_gaussian(_is64(out), _p(out), C.c_int64(seed), 0, n)
    return out


def split_leaves(first: int, limit: int, workers: int, threshold: int = 32):
    buf = np.zeros(2 * 4096, dtype=np.int32)
    n = lib().orc_split_leaves(first, limit, workers, threshold, _p(buf), 4096)
    return sorted((int(buf[2 * i]), int(buf[2 * i + 1])) for i in range(min(n, 4096)))
