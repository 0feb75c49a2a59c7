"""A minimal ``Tensor``: just enough of ``neureka.Tensor`` to drive the HipDevice hot path the way the
reference's call sites do (``Tensor.to(device)``, ``a + b``, ``a.conv(k)``, ``a.matMul(b)``, ``T()``,
slicing, ``backward``).  It holds a view descriptor and either a host array or a device buffer; all
arithmetic runs on a ``HipDevice`` through the backend registry; there is no host arithmetic path.

Reference call sites mirrored here (paths relative to src/main/java/neureka/):
  Tensor.java:1738-1741 (plus), :2007-2010 (conv), TensorImpl.java:862-865 (to), :872-882 (backward),
  math/implementations/FunctionNode.java:89-137 (device selection), autograd/GraphNode.java:409-439.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np

from .device import HipData, HipDevice
from .ndim import IllegalArgumentException, IllegalStateException, Layout, NDConfiguration


def physical_indices(ndc: NDConfiguration) -> np.ndarray:
    """Physical element index of every flat index 0..size-1 (vectorised indexOfIndex)."""
    n = ndc.size
    if ndc.isVirtual():
        return np.zeros(n, dtype=np.int64)
    rest = np.arange(n, dtype=np.int64)
    phys = np.zeros(n, dtype=np.int64)
    for k in range(ndc.rank):
        q = rest // ndc.indicesMap[k]
        rest = rest % ndc.indicesMap[k]
        phys += (q * ndc.spread[k] + ndc.offset[k]) * ndc.strides[k]
    return phys


class Tensor:
    def __init__(self, dtype, ndc: NDConfiguration, data, virtual: bool = False):
        self.dtype = np.dtype(dtype)
        self.ndc = ndc
        self._data = data                    # np.ndarray (host, flat) | HipData | None
        self._virtual = virtual
        self._device: Optional[HipDevice] = None
        self._parent: Optional["Tensor"] = None
        self._intermediate = False
        self._rqs_gradient = False
        self.gradient: Optional["Tensor"] = None
        self._node: Optional["GraphNode"] = None

    # ---- construction ----------------------------------------------------------------------
    @staticmethod
    def of(dtype, shape: Sequence[int], values) -> "Tensor":
        """``Tensor.of(type, shape, data)``: a list cycles to fill the shape (as ``Tensor.of([11,11], 3d..19d)``
        does), a single number gives a virtual tensor (``Tensor.of(shape, value)``)."""
        shape = tuple(int(s) for s in shape)
        dt = np.dtype(dtype)
        size = int(np.prod(shape))
        if np.isscalar(values):
            t = Tensor(dt, NDConfiguration.ofShape(shape), np.array([values], dtype=dt), virtual=True)
            return t
        arr = np.asarray(values, dtype=dt).reshape(-1)
        if arr.size != size:
            arr = np.resize(arr, size)
        return Tensor(dt, NDConfiguration.ofShape(shape), np.ascontiguousarray(arr))

    @staticmethod
    def _on_device(device: HipDevice, dtype, shape, layout: Layout = Layout.ROW_MAJOR, zeroed: bool = True) -> "Tensor":
        """A dense tensor in device memory.  ``zeroed=False`` leaves the buffer as the pool hands it out: for drains
        whose every element the next kernel writes, where the zeros of ``all(0)`` would never be read."""
        ndc = NDConfiguration.ofShape(shape, layout)
        t = Tensor(dtype, ndc, None)
        data = device.allocateFromOne(dtype, ndc.size, 0) if zeroed else device.allocate(dtype, ndc.size)
        t._set_data(data, device)
        device._register(t)
        return t

    # ---- shape -----------------------------------------------------------------------------------
    @property
    def shape(self) -> Tuple[int, ...]: return self.ndc.shape
    @property
    def rank(self) -> int: return self.ndc.rank
    @property
    def size(self) -> int: return self.ndc.size
    def getNDConf(self) -> NDConfiguration: return self.ndc
    def isVirtual(self) -> bool: return self._virtual
    def isOutsourced(self) -> bool: return self._device is not None
    def getDevice(self) -> Optional[HipDevice]: return self._device
    def isSlice(self) -> bool: return self._parent is not None

    def isPartialSlice(self) -> bool:
        root = self._root()
        return root is not self and root.size != self.size

    def _root(self) -> "Tensor":
        t = self
        while t._parent is not None:
            t = t._parent
        return t

    # ---- data plumbing -----------------------------------------------------------------------
    def _set_data(self, data, device: Optional[HipDevice]) -> None:
        old = self._data
        self._data = data
        self._device = device
        if isinstance(data, HipData):
            data.incrementUsageCount()
        if isinstance(old, HipData) and old is not data:
            old.decrementUsageCount()

    def __del__(self):
        # a tensor that is dropped without Device.free gives up its share of the buffer (the usage count the
        # DeviceCleaner decrements in the reference: OpenCLDevice.java:950-966)
        try:
            data = self._data
            if isinstance(data, HipData):
                self._data = None
                data.decrementUsageCount()
        except Exception:
            pass

    def _replace_data(self, data: HipData) -> None:
        self._set_data(data, self._device)

    def to(self, device: HipDevice) -> "Tensor":
        device.store(self)
        return self

    def setIsVirtual(self, virtual: bool) -> "Tensor":
        """TensorImpl.setIsVirtual: actualize / virtualize through the owning device (AbstractDevice.java:136-160)."""
        if virtual == self._virtual:
            return self
        if self._device is not None:
            (self._device._virtualize if virtual else self._device._actualize)(self)
        else:
            if virtual:
                self._data = np.array([self._data[self.ndc.indexOfIndex(0)]], dtype=self.dtype)
            else:
                self._data = np.full(self.size, self._data[0], dtype=self.dtype)
        self._virtual = virtual
        return self

    def getData(self) -> np.ndarray:
        """The raw backing array (``mut.data.get()``), downloaded when the tensor is outsourced."""
        if self._device is not None:
            return self._device._read_all(self._data)
        return self._data

    @property
    def items(self) -> np.ndarray:
        """Items in logical (row-major nd-index) order, through the view descriptor."""
        raw = self.getData()
        if self._virtual:
            return np.full(self.size, raw[0], dtype=self.dtype)
        return raw[physical_indices(self.ndc)]

    def item(self, i: int = 0):
        if self._virtual:
            i_phys = 0
        else:
            i_phys = self.ndc.indexOfIndex(i)
        if self._device is not None:
            return self._device._read(self._data, i_phys, 1)[0]
        return self._data[i_phys]

    def setItems(self, values) -> "Tensor":
        """Writes items in logical order (``mut.setItems`` / ``t.mut[0..n] = other``)."""
        values = np.asarray(values, dtype=self.dtype).reshape(-1)
        self.setIsVirtual(False)
        if self._device is not None:
            raw = self._device._read_all(self._data)
            raw[physical_indices(self.ndc)[: values.size]] = values
            self._device._write(self._data, 0, raw)
        else:
            self._data[physical_indices(self.ndc)[: values.size]] = values
        return self

    # ---- views ----------------------------------------------------------------------------------
    def _view(self, ndc: NDConfiguration) -> "Tensor":
        self.setIsVirtual(False)
        v = Tensor(self.dtype, ndc, None)
        v._parent = self
        if self._device is not None:
            v._set_data(self._root()._data, self._device)
            self._device._register(v)
        else:
            v._data = self._data
        return v

    def permute(self, *axes: int) -> "Tensor":
        """other/Permute.java:67-79."""
        return self._view(self.ndc.newReshaped(axes))

    def T(self) -> "Tensor":
        return self.permute(*reversed(range(self.rank)))

    def getAt(self, *ranges) -> "Tensor":
        """Slicing with ``slice`` objects or ints per axis: other/Slice.java:80-183."""
        if len(ranges) != self.rank:
            raise IllegalArgumentException("one range per axis is required")
        new_shape, new_offset, new_spread = [], [], []
        for axis, r in enumerate(ranges):
            if isinstance(r, int):
                r = slice(r, r + 1, 1)
            start, stop, step = r.indices(self.shape[axis])
            n = len(range(start, stop, step))
            if n <= 0:
                raise IllegalArgumentException("Cannot create slice because ranges are out of the bounds of the targeted tensor.")
            new_shape.append(n)
            new_offset.append(start)
            new_spread.append(step if n > 1 else 1)
        return self._view(self.ndc.sliced(new_shape, new_offset, new_spread))

    __getitem__ = lambda self, key: self.getAt(*(key if isinstance(key, tuple) else (key,)))

    def deepCopy(self) -> "Tensor":
        """A dense row-major copy made by the device (identity activation through the view)."""
        from .function import execute
        return execute("idy", [self])

    def toLayoutCopy(self, layout: Layout) -> "Tensor":
        """``relayout`` to a dense tensor of the requested layout (MatMulAlgorithm._checkAndPrepareLayout)."""
        if self.ndc.getLayout() is layout:
            return self
        dev = self._require_device()
        out = Tensor._on_device(dev, self.dtype, self.shape, layout, zeroed=False)
        dev.launch_activation("idy", -1, out, self)
        return out

    def _require_device(self) -> HipDevice:
        if self._device is None:
            raise IllegalStateException("tensor is not stored on a HipDevice; this package has no host arithmetic path")
        return self._device

    # ---- arithmetic ------------------------------------------------------------------------------
    def _bin(self, op: str, other) -> "Tensor":
        from .function import execute
        if not isinstance(other, Tensor):
            other = Tensor.of(self.dtype, (1,), int(other) if np.issubdtype(self.dtype, np.integer) else float(other))
        return execute(op, [self, other])

    def plus(self, o): return self._bin("add", o)
    def minus(self, o): return self._bin("subtract", o)
    def times(self, o): return self._bin("multiply", o)
    def div(self, o): return self._bin("divide", o)
    def mod(self, o): return self._bin("modulo", o)
    def power(self, o): return self._bin("power", o)
    __add__, __sub__, __mul__, __truediv__, __mod__, __pow__ = plus, minus, times, div, mod, power

    def assign(self, other) -> "Tensor":
        """``mut.assign(other)`` / ``I[0] <- I[1]``: the operation "left_inline" (operations/other/AssignLeft.java)."""
        from .function import execute
        if not isinstance(other, Tensor):
            other = Tensor.of(self.dtype, self.shape, int(other) if np.issubdtype(self.dtype, np.integer) else float(other))
        return execute("left_inline", [self, other])

    def conv(self, k: "Tensor") -> "Tensor":
        from .function import execute
        return execute("mul_conv", [self, k])

    def matMul(self, b: "Tensor") -> "Tensor":
        from .function import execute
        return execute("matMul", [self, b])

    __matmul__ = matMul

    def sum(self) -> "Tensor":
        """Tensor.sum(): the operation "sumItems" (operations/other/Sum.java)."""
        from .function import execute
        return execute("sumItems", [self])

    def min(self) -> "Tensor":
        from .function import execute
        return execute("min", [self])

    def max(self) -> "Tensor":
        from .function import execute
        return execute("max", [self])

    def dot(self, b: "Tensor") -> "Tensor":
        from .function import execute
        return execute("dot", [self, b])

    def __getattr__(self, name):
        # activation shorthands: t.tanh(), t.sig(), t.relu() ...
        from .backend import ACTIVATIONS
        if name in ACTIVATIONS:
            from .function import execute
            return lambda: execute(name, [self])
        raise AttributeError(name)

    # ---- autograd ----------------------------------------------------------------------------------
    def setRqsGradient(self, flag: bool) -> "Tensor":
        self._rqs_gradient = flag
        return self

    def rqsGradient(self) -> bool:
        return self._rqs_gradient

    def backward(self, error=None) -> "Tensor":
        """TensorImpl._backward (TensorImpl.java:872-882) -> GraphNode.backward (autograd/GraphNode.java:409-439)."""
        if error is None:
            error = Tensor.of(self.dtype, self.shape, 1.0)
        elif not isinstance(error, Tensor):
            error = Tensor.of(self.dtype, self.shape, float(error))
        if self._device is not None and not error.isOutsourced():
            error.to(self._device)
        _backward(self, error)
        return self

    def applyGradient(self) -> "Tensor":
        """Gradients are *added* on apply (autograd settings of Tensor_Convolution_Spec.groovy:303-366)."""
        if self.gradient is not None:
            from .function import execute
            dev = self._require_device()
            if not self.gradient.isOutsourced():
                self.gradient.to(dev)
            dev.launch_elementwise("add", -1, self, self, self.gradient)
            self.gradient = None
        return self

    def __repr__(self) -> str:
        where = "host" if self._device is None else repr(self._device)
        return f"Tensor({self.dtype}, shape={list(self.shape)}, {self.ndc.kind()}, on {where})"


def make_fit(tensors: Sequence[Tensor]) -> List[Tensor]:
    """``Permute.makeFit`` (other/Permute.java:81-109): pads lower-rank operands with extent-1 axes, in
    front or behind depending on where the largest operand carries its own extent-1 axes."""
    largest = max(tensors, key=lambda t: t.rank)
    shape = largest.shape
    prefix = 0
    for s in shape:
        if s == 1: prefix += 1
        else: break
    postfix = 0
    for s in reversed(shape):
        if s == 1: postfix += 1
        else: break
    rank = largest.rank
    out = []
    for t in tensors:
        if t.rank != rank:
            padding = rank - t.rank
            if postfix <= prefix:
                form = [-1] * padding + list(range(rank - padding))
            else:
                form = list(range(rank - padding)) + [-1] * padding
            if t.isOutsourced():
                t = t.permute(*form)
            else:       # a host operand: the padded tensor shares the host array, no parent relation needed
                padded = Tensor(t.dtype, t.ndc.newReshaped(form), t._data, t._virtual)
                padded._rqs_gradient = t._rqs_gradient
                t = padded
        out.append(t)
    return out


class GraphNode:
    """What an operation records for reverse-mode AD (autograd/GraphNode.java:121-277): its parents and,
    per parent, the ADAction that turns an error of the result into an error of that parent."""

    def __init__(self, parents: Sequence[Tensor], actions):
        self.parents = list(parents)
        self.actions = list(actions)         # callables error -> Tensor, or None for non-differentiated parents


def _backward(result: Tensor, error: Tensor) -> None:
    from .function import execute
    if result._rqs_gradient:
        if result.gradient is None:
            result.gradient = error
        else:
            result.gradient = execute("add", [result.gradient, error], record=False)
    node = result._node
    if node is None:
        return
    for parent, action in zip(node.parents, node.actions):
        if action is None:
            continue
        if parent._rqs_gradient or parent._node is not None:
            _backward(parent, action(error))
