"""neureka_amd — an MI355X-native ``HipDevice`` for Neureka's hot path.

``libneureka_hip.so`` (hand-written gfx950 HIP kernels behind a C ABI, ``include/neureka_hip.h``) is the
product; this package is the host-side mirror of the reference's device/backend interface that drives
the same C ABI a JVM host would bind.  Importing the package does not touch the GPU; the library is
loaded on first use and a missing library is an error, never a fallback.
"""
from .ndim import IllegalArgumentException, IllegalStateException, Layout, NDConfiguration
from ._lib import HipError, LIB_PATH
from .device import HipData, HipDevice
from .backend import BackendContext, ExecutionCall, HipBackend, backend
from .tensor import Tensor
from .function import Function, OptimizedFunction, execute

__all__ = [
    "IllegalArgumentException", "IllegalStateException", "Layout", "NDConfiguration", "HipError", "LIB_PATH",
    "HipData", "HipDevice", "BackendContext", "ExecutionCall", "HipBackend", "backend", "Tensor", "Function",
    "OptimizedFunction", "execute",
]
