"""View descriptors: the host-side mirror of Neureka's ``NDConfiguration``.

A descriptor is the 5-tuple ``shape, strides, indicesMap, spread, offset`` (each ``int[rank]``) of
``src/main/java/neureka/ndim/config/NDConfiguration.java:186-345``.  The device format is
``asInlineArray()`` = ``shape | strides | indicesMap | offset | spread`` (``:335-345``), which is what every
kernel entry point of ``libneureka_hip.so`` takes.

Only integer bookkeeping lives here; nothing in this module touches the GPU.
"""
from __future__ import annotations

import enum
from dataclasses import dataclass
from typing import Sequence, Tuple

import ctypes as C
import functools
import numpy as np

MAX_RANK = 8


class Layout(enum.Enum):
    """``NDConfiguration.Layout`` (NDConfiguration.java:95-144)."""

    ROW_MAJOR = "ROW_MAJOR"
    COLUMN_MAJOR = "COLUMN_MAJOR"
    SYMMETRIC = "SYMMETRIC"
    UNSPECIFIC = "UNSPECIFIC"

    def isCompatible(self, other: "Layout") -> bool:
        if self is Layout.UNSPECIFIC or other is Layout.UNSPECIFIC:
            return False
        if self is Layout.SYMMETRIC or other is Layout.SYMMETRIC:
            return True
        return self is other

    def newStridesFor(self, shape: Sequence[int]) -> Tuple[int, ...]:
        """Strides of a dense tensor of this layout (NDConfiguration.java:109-132)."""
        n = len(shape)
        order = [n - 1 - i for i in range(n)]
        if self is Layout.COLUMN_MAJOR and n > 1:
            order[0], order[1] = order[1], order[0]
        strides = [0] * n
        prod = 1
        for i in order:
            strides[i] = prod
            prod *= shape[i]
        return tuple(strides)

    def rearrange(self, tln: Sequence[int], shape: Sequence[int], newForm: Sequence[int]) -> Tuple[int, ...]:
        """NDConfiguration.java:135-143."""
        shpTln = self.newStridesFor(shape)
        return tuple(shpTln[i] if f < 0 else tln[f] for i, f in enumerate(newForm))


def _rearrange(array: Sequence[int], pointers: Sequence[int]) -> Tuple[int, ...]:
    """``NDConfiguration.Utility.rearrange`` (NDConfiguration.java:427-434)."""
    return tuple(abs(p) if p < 0 else array[p] for p in pointers)


@dataclass(frozen=True)
class NDConfiguration:
    shape: Tuple[int, ...]
    strides: Tuple[int, ...]
    indicesMap: Tuple[int, ...]
    spread: Tuple[int, ...]
    offset: Tuple[int, ...]
    virtual: bool = False

    # ---- factories ------------------------------------------------------------------------
    @staticmethod
    def of(shape, strides, indicesMap, spread, offset) -> "NDConfiguration":
        """``AbstractNDC.construct`` (ndim/config/AbstractNDC.java:68-139): same validation and errors."""
        shape, strides, indicesMap, spread, offset = (tuple(int(v) for v in a) for a in (shape, strides, indicesMap, spread, offset))
        rank = len(shape)
        if not (len(strides) == len(indicesMap) == len(spread) == len(offset) == rank):
            raise ValueError("all five arrays of a NDConfiguration must have the same length")
        if rank < 1 or rank > MAX_RANK:
            raise ValueError(f"rank {rank} outside [1, {MAX_RANK}]")
        for dim in shape:
            if dim == 0:
                raise IllegalStateException(
                    "Trying to create tensor configuration containing shape with dimension 0.\n"
                    "Shape dimensions must be greater than 0!\n"
                )
        for i in range(rank):
            if shape[i] == 1 and spread[i] > 1:
                raise IllegalStateException(
                    f"Trying to create an 'NDConfiguration' with a nonsensical spread/step value for dimension {i}, "
                    f"using shape {list(shape)} and spread {list(spread)}."
                )
        return NDConfiguration(shape, strides, indicesMap, spread, offset)

    @staticmethod
    def ofShape(shape: Sequence[int], layout: Layout = Layout.ROW_MAJOR) -> "NDConfiguration":
        """A fresh dense tensor: ``NDConstructor.of(shape)`` (ndim/NDConstructor.java).  Configurations are immutable and,
        as in the reference (``AbstractNDC._cached``, ndim/config/AbstractNDC.java:39-66), one instance serves every
        tensor of a shape and layout."""
        if type(shape) is not tuple:
            shape = tuple(int(s) for s in shape)
        return _dense_configuration(shape, layout)

    @staticmethod
    def virtualOf(shape: Sequence[int]) -> "NDConfiguration":
        """``VirtualNDConfiguration`` (ndim/config/types/views/virtual/VirtualNDConfiguration.java:34-64)."""
        shape = tuple(int(s) for s in shape)
        z = (0,) * len(shape)
        return NDConfiguration(shape, z, z, z, z, virtual=True)

    # ---- queries --------------------------------------------------------------------------
    @property
    def rank(self) -> int:
        return len(self.shape)

    @property
    def size(self) -> int:
        s = 1
        for d in self.shape:
            s *= d
        return s

    def isVirtual(self) -> bool:
        return self.virtual

    def isCompact(self) -> bool:
        """NDConfiguration.java:392-397."""
        return all(s in (0, 1) for s in self.spread) and all(o == 0 for o in self.offset)

    def getLayout(self) -> Layout:
        """NDConfiguration.java:157-173."""
        if not self.isCompact():
            return Layout.UNSPECIFIC
        rm = Layout.ROW_MAJOR.newStridesFor(self.shape)
        has_rm_indices = rm == self.indicesMap
        is_rm = rm == self.strides and has_rm_indices
        is_cm = Layout.COLUMN_MAJOR.newStridesFor(self.shape) == self.strides and has_rm_indices
        if is_rm and is_cm:
            return Layout.SYMMETRIC
        if is_rm:
            return Layout.ROW_MAJOR
        if is_cm:
            return Layout.COLUMN_MAJOR
        return Layout.UNSPECIFIC

    def isSimple(self) -> bool:
        """NDConfiguration.java:376-383."""
        simple = self.getLayout().newStridesFor(self.shape)
        return self.strides == simple and self.indicesMap == simple and self.isCompact()

    def kind(self) -> str:
        """Name of the specialised class ``AbstractNDC.construct`` would pick (AbstractNDC.java:96-139)."""
        if self.virtual:
            return "VirtualNDConfiguration"
        rank = self.rank
        rm = Layout.ROW_MAJOR.newStridesFor(self.shape)
        ones, zeros = (1,) * rank, (0,) * rank
        is_simple = self.strides == rm and self.indicesMap == rm and self.offset == zeros and self.spread == ones
        is_transposed = self.offset == zeros and self.spread == ones
        dims = {1: "1D", 2: "2D", 3: "3D"}.get(rank, "ND")
        if is_simple:
            if rank == 1 and self.shape[0] == 1:
                return "Simple0DConfiguration"
            return f"Simple{dims}Configuration"
        if is_transposed:
            return f"Permuted{dims}Configuration"
        if rank == 1 and self.shape[0] == 1:
            return "Sliced0DConfiguration"
        return f"Sliced{dims}Configuration"

    # ---- index maths (ndim/config/types/sliced/SlicedNDConfiguration.java:94-111) -----------------
    def indicesOfIndex(self, index: int) -> Tuple[int, ...]:
        if self.virtual:
            return (0,) * self.rank
        out = []
        for m in self.indicesMap:
            out.append(index // m)
            index %= m
        return tuple(out)

    def indexOfIndices(self, indices: Sequence[int]) -> int:
        if self.virtual:
            return 0
        return sum((indices[i] * self.spread[i] + self.offset[i]) * self.strides[i] for i in range(self.rank))

    def indexOfIndex(self, index: int) -> int:
        return self.indexOfIndices(self.indicesOfIndex(index))

    def asInlineArray(self) -> np.ndarray:
        """``shape | strides | indicesMap | offset | spread`` (NDConfiguration.java:335-345).  The array is built once
        per configuration and handed out read-only."""
        return self.inlineArguments()[0]

    def inlineArguments(self):
        """(the inline array, a ctypes ``int32*`` to it): what a kernel launch passes for this configuration."""
        cached = self.__dict__.get("_inline")
        if cached is None:
            arr = np.array(self.shape + self.strides + self.indicesMap + self.offset + self.spread, dtype=np.int32)
            arr.flags.writeable = False
            cached = (arr, arr.ctypes.data_as(C.POINTER(C.c_int32)))
            object.__setattr__(self, "_inline", cached)      # a cache beside the (frozen) fields, not one of them
        return cached

    # ---- derived views ---------------------------------------------------------------------
    def newReshaped(self, newForm: Sequence[int]) -> "NDConfiguration":
        """Permutation / padding view: ``AbstractNDC._simpleReshape`` (AbstractNDC.java:182-203).  For a
        non-simple source the reference wraps the result in a ``SimpleReshapeView`` whose 5-tuple is the
        same (``types/views/SimpleReshapeView.java:30-45``)."""
        newForm = tuple(int(f) for f in newForm)
        for f in newForm:
            if f < -1 and not self._isSimpleConfiguration():
                raise ValueError("SimpleReshapeView may not view a NDConfiguration beyond reshaping and or padding!")
        layout = self.getLayout()
        newShape = _rearrange(self.shape, newForm)
        newStrides = layout.rearrange(self.strides, newShape, newForm)
        newIndicesMap = layout.newStridesFor(newShape)
        newSpread = tuple(1 if f < 0 else self.spread[f] for f in newForm)
        newOffset = tuple(0 if f < 0 else self.offset[f] for f in newForm)
        return NDConfiguration.of(newShape, newStrides, newIndicesMap, newSpread, newOffset)

    def _isSimpleConfiguration(self) -> bool:
        rm = Layout.ROW_MAJOR.newStridesFor(self.shape)
        return self.strides == rm and self.indicesMap == rm and self.offset == (0,) * self.rank and self.spread == (1,) * self.rank

    def sliced(self, newShape: Sequence[int], newOffset: Sequence[int], newSpread: Sequence[int]) -> "NDConfiguration":
        """``Slice._slice`` (backend/main/operations/other/Slice.java:80-94): the parent's strides are kept,
        the flat->nd table is rebuilt for the new shape, offsets are inherited, zero steps become 1."""
        newShape = tuple(int(s) for s in newShape)
        newStrides = self.strides
        newIndicesMap = self.getLayout().newStridesFor(newShape)
        spread = tuple(1 if int(s) == 0 else int(s) for s in newSpread)
        offset = tuple(int(o) + self.offset[i] for i, o in enumerate(newOffset))
        return NDConfiguration.of(newShape, newStrides, newIndicesMap, spread, offset)


class IllegalStateException(RuntimeError):
    """Stands for ``java.lang.IllegalStateException`` where the reference throws one."""


class IllegalArgumentException(ValueError):
    """Stands for ``java.lang.IllegalArgumentException`` where the reference throws one."""


@functools.lru_cache(maxsize=4096)
def _dense_configuration(shape: Tuple[int, ...], layout: Layout) -> NDConfiguration:
    shape = tuple(int(s) for s in shape)
    strides = layout.newStridesFor(shape)
    # the flat->nd table is always the row-major one for RM and CM tensors (NDConfiguration.getLayout :157-173)
    imap = Layout.ROW_MAJOR.newStridesFor(shape)
    return NDConfiguration.of(shape, strides, imap, (1,) * len(shape), (0,) * len(shape))
