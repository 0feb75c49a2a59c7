"""``HipDevice``: the device object that satisfies Neureka's ``Device`` contract on an MI355X.

Mirrors ``src/main/java/neureka/devices/opencl/OpenCLDevice.java`` (store/restore/free/has, buffer
ownership through reference-counted data objects, virtual tensors, blocking reads and writes) on top of
the C ABI of ``libneureka_hip.so``.  Method names follow ``neureka.devices.Device``
(``src/main/java/neureka/devices/Device.java:73-410``) and ``AbstractDevice`` (``AbstractDevice.java:86-206``).
"""
from __future__ import annotations

import ctypes as C
import weakref
from typing import Dict, List, Optional, Sequence

import numpy as np

from . import _lib
from .ndim import IllegalArgumentException, IllegalStateException, NDConfiguration


_INT_CODES = {np.dtype(np.int32): 2, np.dtype(np.int64): 3, np.dtype(np.int16): 4, np.dtype(np.int8): 5}


_ITEM_SIZES = {np.float32: 4, np.float64: 8, np.int32: 4, np.int64: 8, np.int16: 2, np.int8: 1, np.uint8: 1}
_FLOAT_CODES = {np.float32: _lib.F32, np.float64: _lib.F64, np.dtype(np.float32): _lib.F32, np.dtype(np.float64): _lib.F64}


def _dtype_code(dtype) -> int:
    code = _FLOAT_CODES.get(dtype)
    if code is not None:
        return code
    dt = np.dtype(dtype)
    if dt == np.float32:
        return _lib.F32
    if dt == np.float64:
        return _lib.F64
    raise IllegalArgumentException(f"HipDevice computes in float32 and float64 (integer types: scalar broadcast only), not {dt}")


class HipData:
    """A device buffer with a usage count: ``AbstractDeviceData`` (devices/AbstractDeviceData.java:7-59) /
    ``OpenCLDevice.CLData`` (OpenCLDevice.java:950-966).  Tensors that share storage (slices, permuted
    views) share one HipData; the buffer is released when the count drops to zero."""

    def __init__(self, device: "HipDevice", ptr: int, dtype, size: int):
        self.device = device
        self.ptr = ptr
        self.dtype = np.dtype(dtype)
        self.size = size            # elements
        self._usage = 0
        self._freed = False
        device._data_objects += 1

    def owner(self) -> "HipDevice":
        return self.device

    def usages(self) -> int:
        return self._usage

    def incrementUsageCount(self) -> None:
        self._usage += 1

    def decrementUsageCount(self) -> None:
        self._usage -= 1
        if self._usage <= 0:
            self.release()

    def release(self) -> None:
        if not self._freed:
            self._freed = True
            self.device._data_objects -= 1
            if not self.device._disposed:
                _lib.check(self.device._lib.nk_free(self.device.handle, self.ptr))

    def __del__(self):  # the role of CustomDeviceCleaner (devices/CustomDeviceCleaner.java:21-121)
        try:
            self.release()
        except Exception:
            pass


class HipDevice:
    """One MI355X: one in-order HIP stream, blocking host transfers, asynchronous kernel launches."""

    _open: Dict[int, "HipDevice"] = {}

    # ---- discovery ---------------------------------------------------------------------------
    @staticmethod
    def count() -> int:
        n = C.c_int(0)
        _lib.check(_lib.load().nk_device_count(C.byref(n)))
        return n.value

    @staticmethod
    def get(index: int = 0) -> "HipDevice":
        dev = HipDevice._open.get(index)
        if dev is None or dev._disposed:
            dev = HipDevice(index)
            HipDevice._open[index] = dev
        return dev

    def __init__(self, index: int = 0):
        self._lib = _lib.load()
        h = C.c_uint64(0)
        _lib.check(self._lib.nk_device_open(index, C.byref(h)))
        self.handle = h.value
        self.index = index
        self._disposed = False
        self._data_objects = 0
        # tensors currently outsourced to this device, held weakly (id -> weak reference): a tensor nobody holds any
        # more leaves the table by itself and its HipData releases the buffer once no tensor shares it -- the role of
        # the DeviceCleaner on weak reachability (devices/AbstractDevice.java:59,109; OpenCLDevice.java:301)
        self._stored: Dict[int, weakref.ref] = {}
        name = C.create_string_buffer(256)
        cu, mhz, lds, wave = C.c_int(0), C.c_int(0), C.c_int(0), C.c_int(0)
        mem = C.c_uint64(0)
        _lib.check(self._lib.nk_device_props(self.handle, name, 256, C.byref(cu), C.byref(mhz), C.byref(mem), C.byref(lds), C.byref(wave)))
        self._name = name.value.decode()
        self._cu, self._mhz, self._mem, self._lds, self._wave = cu.value, mhz.value, mem.value, lds.value, wave.value

    # properties: OpenCLDevice.java:738-809
    def name(self) -> str: return self._name
    def maxComputeUnits(self) -> int: return self._cu
    def maxClockFrequenzy(self) -> int: return self._mhz       # spelling of the reference (OpenCLDevice.java:768)
    def globalMemSize(self) -> int: return self._mem
    def localMemSize(self) -> int: return self._lds
    def wavefrontSize(self) -> int: return self._wave
    def __repr__(self) -> str: return f"HipDevice[{self.index}: {self._name}, {self._cu} CUs]"

    # ---- Device contract ---------------------------------------------------------------------
    def numberOfStored(self) -> int:
        return len(self._stored)

    def numberOfDataObjects(self) -> int:
        return self._data_objects

    def isEmpty(self) -> bool:
        return not self._stored

    def has(self, tensor) -> bool:
        ref = self._stored.get(id(tensor))
        return ref is not None and ref() is tensor

    def _register(self, tensor) -> None:
        key = id(tensor)
        stored = self._stored

        def gone(ref, key=key, stored=stored):
            if stored.get(key) is ref:       # the id may have been taken by a younger tensor meanwhile
                del stored[key]
        stored[key] = weakref.ref(tensor, gone)

    def contains(self, tensor) -> bool:
        return self.has(tensor)

    def store(self, tensor) -> "HipDevice":
        """``Tensor.to(device)`` lands here: AbstractDevice.update (AbstractDevice.java:86-107) +
        OpenCLDevice._updateInternal/_add (OpenCLDevice.java:346-405,661-674)."""
        self._check_open()
        if self.has(tensor):
            return self
        parent = tensor._parent
        if parent is not None:
            root = tensor._root()
            if not self.has(root):
                raise IllegalStateException("Data parent is not outsourced!")
            tensor._set_data(root._data, self)      # share the root's buffer
        else:
            host = tensor._data
            if isinstance(host, HipData):
                if host.device is self:
                    tensor._set_data(host, self)
                    self._register(tensor)
                    return self
                raise IllegalStateException("tensor already lives on another device")
            data = self._upload(host, tensor.dtype, tensor.isVirtual())
            tensor._set_data(data, self)
        self._register(tensor)
        return self

    def restore(self, tensor) -> "HipDevice":
        """Brings a tensor back to host memory (OpenCLDevice.java:315-334)."""
        if not self.has(tensor):
            raise IllegalArgumentException("The passed tensor cannot be restored from this device as it is not stored on the device.")
        host = self._read_all(tensor._data)
        self.free(tensor)
        tensor._set_data(host, None)
        return self

    def free(self, tensor) -> "HipDevice":
        """Drops the device's claim on the tensor (OpenCLDevice.java:609-620)."""
        if not self.has(tensor):
            raise IllegalArgumentException("tensor is not stored on this device")
        del self._stored[id(tensor)]
        data = tensor._data
        tensor._data = None
        tensor._device = None
        if isinstance(data, HipData):
            data.decrementUsageCount()
        return self

    def approve(self, call) -> "HipDevice":
        """Device.approve (Device.java:205-214): every operand must be on this device."""
        for t in call.inputs:
            if t is not None and t._device is not self:
                raise IllegalStateException("ExecutionCall holds a tensor that is not stored on the executing HipDevice")
        return self

    def sync(self) -> None:
        _lib.check(self._lib.nk_device_sync(self.handle))

    def dispose(self) -> None:
        """OpenCLDevice.dispose (OpenCLDevice.java:299-304): finishes the queue and drops every buffer."""
        if self._disposed:
            return
        for ref in list(self._stored.values()):
            t = ref()
            if t is not None:
                t._data = None
                t._device = None
        self._stored.clear()
        _lib.check(self._lib.nk_device_close(self.handle))
        self._disposed = True

    def liveBuffers(self) -> int:
        n, b = C.c_uint64(0), C.c_uint64(0)
        _lib.check(self._lib.nk_device_stats(self.handle, C.byref(n), C.byref(b)))
        return n.value

    def freeMemory(self) -> int:
        """Bytes of device memory the driver reports as free (blocks at rest in the pool count as used)."""
        f, t = C.c_uint64(0), C.c_uint64(0)
        _lib.check(self._lib.nk_device_memory(self.handle, C.byref(f), C.byref(t)))
        return f.value

    def poolStats(self) -> dict:
        """The buffer pool behind ``allocate`` / ``HipData.release``: blocks at rest, their bytes, allocations that
        went to the driver and allocations served from a block at rest."""
        v = [C.c_uint64(0) for _ in range(4)]
        _lib.check(self._lib.nk_pool_stats(self.handle, *[C.byref(x) for x in v]))
        return dict(zip(("resting_blocks", "resting_bytes", "driver_allocations", "reuses"), (x.value for x in v)))

    def trimPool(self) -> None:
        _lib.check(self._lib.nk_pool_trim(self.handle))

    def configurePool(self, max_resting_bytes: Optional[int] = None, poison: bool = False) -> None:
        limit = self._mem // 2 if max_resting_bytes is None else int(max_resting_bytes)
        _lib.check(self._lib.nk_pool_config(self.handle, limit, 1 if poison else 0))

    # ---- data access: AbstractDevice._readAll/_readItem/_readArray/_writeItem/_writeArray ------------
    def allocate(self, dtype, size: int) -> HipData:
        """Device.allocate (OpenCLDevice.java:520-530)."""
        self._check_open()
        itemsize = _ITEM_SIZES.get(dtype)
        if itemsize is None:
            itemsize = np.dtype(dtype).itemsize
        ptr = C.c_uint64(0)
        _lib.check(self._lib.nk_alloc(self.handle, int(size) * itemsize, C.byref(ptr)))
        return HipData(self, ptr.value, dtype, int(size))

    def allocateFromOne(self, dtype, size: int, value) -> HipData:
        """Device.allocateFromOne: a buffer filled with one value by the device (OpenCLDevice.java:478-486)."""
        data = self.allocate(dtype, size)
        self._fill(data, 0, size, value)
        return data

    def allocateFromAll(self, array: np.ndarray) -> HipData:
        array = np.ascontiguousarray(array)
        data = self.allocate(array.dtype, array.size)
        self._write(data, 0, array)
        return data

    def _upload(self, host: np.ndarray, dtype, virtual: bool) -> HipData:
        host = np.ascontiguousarray(host, dtype=dtype)
        if virtual:     # a virtual tensor keeps a single element on the device
            return self.allocateFromOne(dtype, 1, host.reshape(-1)[0])
        return self.allocateFromAll(host.reshape(-1))

    def _fill(self, data: HipData, start: int, count: int, value) -> None:
        pat = np.array([value], dtype=data.dtype)
        _lib.check(self._lib.nk_fill(self.handle, data.ptr, start * data.dtype.itemsize, pat.ctypes.data_as(C.c_void_p),
                                     data.dtype.itemsize, count))

    def _write(self, data: HipData, start: int, array: np.ndarray) -> None:
        array = np.ascontiguousarray(array, dtype=data.dtype)
        _lib.check(self._lib.nk_h2d(self.handle, data.ptr, start * data.dtype.itemsize, array.ctypes.data_as(C.c_void_p), array.nbytes))

    def _read(self, data: HipData, start: int, count: int) -> np.ndarray:
        out = np.empty(count, dtype=data.dtype)
        _lib.check(self._lib.nk_d2h(self.handle, out.ctypes.data_as(C.c_void_p), data.ptr, start * data.dtype.itemsize, out.nbytes))
        return out

    def _read_all(self, data: HipData) -> np.ndarray:
        return self._read(data, 0, data.size)

    def _actualize(self, tensor) -> None:
        """virtual -> full buffer, filled by the device (OpenCLDevice.java:573-593)."""
        old: HipData = tensor._data
        value = self._read(old, 0, 1)[0]
        new = self.allocateFromOne(tensor.dtype, tensor.ndc.size, value)
        tensor._replace_data(new)

    def _virtualize(self, tensor) -> None:
        old: HipData = tensor._data
        value = self._read(old, tensor.ndc.indexOfIndex(0) if not tensor.ndc.isVirtual() else 0, 1)[0]
        new = self.allocateFromOne(tensor.dtype, 1, value)
        tensor._replace_data(new)

    # ---- the protected contract of AbstractDevice (devices/AbstractDevice.java:188-206), as OpenCLDevice fills it in
    #      (devices/opencl/OpenCLDevice.java:527-660); indices are positions in the tensor's buffer ------------------
    def _readAll(self, tensor, clone: bool = True) -> np.ndarray:
        return self._read_all(tensor._data)

    def _readItem(self, tensor, index: int):
        return self._read(tensor._data, index, 1)[0]

    def _readArray(self, tensor, start: int, size: int) -> np.ndarray:
        return self._read(tensor._data, start, size)

    def _writeItem(self, tensor, item, start: int, size: int) -> None:
        """One value repeated over [start, start + size): a device fill (OpenCLDevice.java:537-541)."""
        self._fill(tensor._data, start, size, item)

    def _writeArray(self, tensor, array, offset: int, start: int, size: int) -> None:
        """array[offset : offset + size] -> buffer[start : start + size] (OpenCLDevice.java:542-552)."""
        self._write(tensor._data, start, np.asarray(array).reshape(-1)[offset:offset + size])

    def _swap(self, former, replacement) -> None:
        """The replacement takes over the former tensor's device data (OpenCLDevice.java:635-640)."""
        replacement._set_data(former._data, self)

    def _sizeOccupiedBy(self, tensor) -> int:
        return tensor._data.size

    def _dataTypeOf(self, raw) -> np.dtype:
        return np.dtype(raw.dtype)

    def update(self, tensor, added: bool) -> bool:
        """Component.update(OwnerChangeRequest) (OpenCLDevice.java:340-371): a tensor that gains this device as a
        component is stored on it, one that loses it is restored to the host."""
        if added:
            if not self.has(tensor):
                self.store(tensor)
        elif self.has(tensor):
            self.restore(tensor)
        return True

    def _check_open(self) -> None:
        if self._disposed:
            raise IllegalStateException("HipDevice has been disposed")

    # ---- fused functions: Device.optimizedFunctionOf (Device.java:216-243) -------------------------
    def optimizedFunctionOf(self, function, name: str):
        from .function import OptimizedFunction
        return OptimizedFunction(self, function, name)

    # ---- kernel launches (thin wrappers over the C ABI; operands are device tensors) ----------------
    @staticmethod
    def _ops(*tensors):
        out = []
        rank = len(tensors[0].ndc.shape)
        for t in tensors:
            if len(t.ndc.shape) != rank:
                raise IllegalArgumentException(f"operands of one kernel must have one rank, got {[t.rank for t in tensors]}")
            # a virtual tensor keeps one element on the device and is addressed through all-zero tables
            inline, pointer = (NDConfiguration.virtualOf(t.shape) if t._virtual else t.ndc).inlineArguments()
            out.append((t._data.ptr, inline, pointer))
        return out

    def launch_activation(self, fun: str, d: int, drn, src) -> None:
        (p0, k0, c0), (p1, k1, c1) = self._ops(drn, src)
        _lib.check(self._lib.nk_activation(self.handle, _lib.FUN[fun], d, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, p1, c1, drn.ndc.size))

    def launch_activation_item(self, fun: str, d: int, drn, src) -> None:
        """f (or f') of the one element a virtual tensor keeps on the device, written to the drain's one element.
        `drn` / `src` are virtual tensors or bare one-element buffers."""
        one = NDConfiguration.ofShape((1,)).asInlineArray()
        dt = drn.dtype
        p0 = C.c_uint64(drn.ptr if isinstance(drn, HipData) else drn._data.ptr)
        p1 = C.c_uint64(src.ptr if isinstance(src, HipData) else src._data.ptr)
        _lib.check(self._lib.nk_activation(self.handle, _lib.FUN[fun], d, _dtype_code(dt), 1, p0, _lib.cfg_ptr(one), p1, _lib.cfg_ptr(one), 1))

    def launch_elementwise(self, op: str, d: int, drn, a, b) -> None:
        (p0, k0, c0), (p1, k1, c1), (p2, k2, c2) = self._ops(drn, a, b)
        _lib.check(self._lib.nk_elementwise(self.handle, _lib.OP[op], d, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, p1, c1, p2, c2, drn.ndc.size))

    def launch_scalarization(self, op: str, d: int, drn, src, value) -> None:
        (p0, k0, c0), (p1, k1, c1) = self._ops(drn, src)
        if drn.dtype in _INT_CODES:              # CLScalarBroadcast's "int", "long", "short", "char" kernels
            if src.dtype != drn.dtype:
                raise IllegalArgumentException(f"scalarization of {src.dtype} data into a {drn.dtype} drain")
            wrapped = (int(value) + (1 << 63)) % (1 << 64) - (1 << 63)
            _lib.check(self._lib.nk_scalarization_int(self.handle, _lib.OP[op], d, _INT_CODES[drn.dtype], drn.ndc.rank, p0, c0, p1, c1,
                                                      wrapped, drn.ndc.size))
            return
        _lib.check(self._lib.nk_scalarization(self.handle, _lib.OP[op], d, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, p1, c1, float(value), drn.ndc.size))

    def launch_scalar_fill(self, drn, value: float) -> None:
        ((p0, k0, c0),) = self._ops(drn)
        _lib.check(self._lib.nk_scalar_fill(self.handle, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, float(value), drn.ndc.size))

    def launch_broadcast(self, op: str, d: int, drn, a, b) -> None:
        (p0, k0, c0), (p1, k1, c1), (p2, k2, c2) = self._ops(drn, a, b)
        _lib.check(self._lib.nk_broadcast(self.handle, _lib.OP[op], d, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, p1, c1, p2, c2, drn.ndc.size))

    def launch_convolution(self, d: int, drn, a, b) -> None:
        (p0, k0, c0), (p1, k1, c1), (p2, k2, c2) = self._ops(drn, a, b)
        _lib.check(self._lib.nk_convolution(self.handle, d, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, p1, c1, p2, c2, drn.ndc.size))

    def launch_matmul(self, row_major: bool, M: int, K: int, N: int, a, b, c, accumulate: bool = True) -> None:
        """c += a @ b (GEMM.java:282-304), or with accumulate=False c = a @ b, what the OpenCL device's kernel does
        (CLMatMul.java:50) and what the registered implementation calls: the drain it is handed is freshly zeroed."""
        fn = self._lib.nk_matmul if accumulate else self._lib.nk_matmul_set
        _lib.check(fn(self.handle, _dtype_code(c.dtype), _lib.ROW_MAJOR if row_major else _lib.COLUMN_MAJOR,
                      M, K, N, a._data.ptr, b._data.ptr, c._data.ptr))

    def launch_sum(self, src, out) -> None:
        """CLSum.run (operations/linear/internal/opencl/CLSum.java:24-62): out[0] = sum of the dense tensor `src`."""
        _lib.check(self._lib.nk_sum(self.handle, _dtype_code(src.dtype), src._data.ptr, src.ndc.size, out._data.ptr))

    def launch_dot(self, a, b, out) -> None:
        """CLDot (implementations/linear/CLDot.java:20-56)."""
        _lib.check(self._lib.nk_dot(self.handle, _dtype_code(a.dtype), a._data.ptr, b._data.ptr, a.ndc.size, out._data.ptr))

    def reduce_index(self, kind: str, src) -> int:
        """CLReduce: index of the minimum / maximum of the dense tensor `src` (operations/other/Min.java:47-49 reads it
        back with ``index.item(0)``)."""
        slot = self.allocate(np.int32, 1)
        try:
            _lib.check(self._lib.nk_reduce_index(self.handle, {"min": 0, "max": 1}[kind], _dtype_code(src.dtype), src._data.ptr,
                                                 src.ndc.size, slot.ptr))
            return int(self._read(slot, 0, 1)[0])
        finally:
            slot.release()

    def launch_fused(self, program: Sequence[int], consts: Sequence[float], drn, srcs) -> None:
        ops = self._ops(drn, *srcs)
        prog = (C.c_int32 * len(program))(*program)
        cs = (C.c_double * max(1, len(consts)))(*consts)
        ptrs = (C.c_uint64 * max(1, len(srcs)))(*[o[0] for o in ops[1:]])
        cfgs = (C.POINTER(C.c_int32) * max(1, len(srcs)))(*[o[2] for o in ops[1:]])
        _lib.check(self._lib.nk_fused(self.handle, prog, len(program) // 2, cs, len(consts), _dtype_code(drn.dtype), drn.ndc.rank,
                                      ops[0][0], ops[0][2], len(srcs), ptrs, cfgs, drn.ndc.size))

    def prepared(self, entry: str, *args):
        """Binds one C-ABI call with its arguments converted once; the returned callable repeats exactly
        that launch (used where the per-call cost of building descriptors would distort a measurement).
        Tensors are passed as (pointer, descriptor) pairs by the caller-facing helpers below."""
        fn = getattr(self._lib, entry)
        keep = args                      # keeps descriptor arrays alive
        def call():
            _lib.check(fn(*keep))
        return call

    def prepared_launch(self, kind: str, *a):
        """kind: 'broadcast' | 'elementwise' (op, d, drn, x, y) | 'activation' (fun, d, drn, x) |
        'scalarization_int' (op, d, drn, x, value) | 'fused' (program, consts, drn, srcs) | 'convolution' (d, drn, x, y) | 'matmul' (row_major, M, K, N, x, y, z)"""
        h = C.c_uint64(self.handle)
        if kind in ("broadcast", "elementwise"):
            op, d, drn, x, y = a
            (p0, k0, c0), (p1, k1, c1), (p2, k2, c2) = ops = self._ops(drn, x, y)
            call = self.prepared("nk_" + kind, h, _lib.OP[op], d, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, p1, c1, p2, c2, C.c_int64(drn.ndc.size))
        elif kind == "activation":
            fun, d, drn, x = a
            (p0, k0, c0), (p1, k1, c1) = ops = self._ops(drn, x)
            call = self.prepared("nk_activation", h, _lib.FUN[fun], d, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, p1, c1, C.c_int64(drn.ndc.size))
        elif kind == "scalarization_int":
            op, d, drn, x, value = a
            (p0, k0, c0), (p1, k1, c1) = ops = self._ops(drn, x)
            call = self.prepared("nk_scalarization_int", h, _lib.OP[op], d, _INT_CODES[drn.dtype], drn.ndc.rank, p0, c0, p1, c1,
                                 C.c_int64(int(value)), C.c_int64(drn.ndc.size))
        elif kind == "convolution":
            d, drn, x, y = a
            (p0, k0, c0), (p1, k1, c1), (p2, k2, c2) = ops = self._ops(drn, x, y)
            call = self.prepared("nk_convolution", h, d, _dtype_code(drn.dtype), drn.ndc.rank, p0, c0, p1, c1, p2, c2, C.c_int64(drn.ndc.size))
        elif kind in ("matmul", "matmul_set"):
            rm, M, K, N, x, y, z = a
            ops = None
            call = self.prepared("nk_matmul" if kind == "matmul" else "nk_matmul_set", h, _dtype_code(z.dtype), _lib.ROW_MAJOR if rm else _lib.COLUMN_MAJOR, C.c_int64(M), C.c_int64(K), C.c_int64(N),
                                 C.c_uint64(x._data.ptr), C.c_uint64(y._data.ptr), C.c_uint64(z._data.ptr))
        elif kind == "fused":
            program, consts, drn, srcs = a
            ops = self._ops(drn, *srcs)
            prog = (C.c_int32 * len(program))(*program)
            cs = (C.c_double * max(1, len(consts)))(*consts)
            ptrs = (C.c_uint64 * max(1, len(srcs)))(*[o[0] for o in ops[1:]])
            cfgs = (C.POINTER(C.c_int32) * max(1, len(srcs)))(*[o[2] for o in ops[1:]])
            call = self.prepared("nk_fused", h, prog, len(program) // 2, cs, len(consts), _dtype_code(drn.dtype), drn.ndc.rank,
                                 ops[0][0], ops[0][2], len(srcs), ptrs, cfgs, C.c_int64(drn.ndc.size))
            ops = (ops, prog, cs, ptrs, cfgs)
        else:
            raise IllegalArgumentException(f"unknown launch kind '{kind}'")
        call._keepalive = ops
        return call

    # timing on the device stream
    def event(self) -> int:
        e = C.c_uint64(0)
        _lib.check(self._lib.nk_event_create(self.handle, C.byref(e)))
        return e.value

    def record(self, event: int) -> None:
        _lib.check(self._lib.nk_event_record(self.handle, event))

    def elapsed_ms(self, start: int, stop: int) -> float:
        ms = C.c_float(0)
        _lib.check(self._lib.nk_event_elapsed_ms(self.handle, start, stop, C.byref(ms)))
        return ms.value
