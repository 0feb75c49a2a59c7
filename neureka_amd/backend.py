"""The plugin seam: ``ExecutionCall``, the device-agnostic ``Algorithm`` objects and ``HipBackend``, the
registration table that hangs ``ImplementationFor<HipDevice>`` objects on them.

Mirrors, for the hot path only:
  - ``backend/api/ExecutionCall.java`` / ``Call.java`` (slot 0 = drain, ``Arg.DerivIdx``)
  - ``backend/main/algorithms/{BiElementwise,Broadcast,BiScalarBroadcast,ElementwiseAlgorithm,NDConvolution,MatMulAlgorithm}.java``
    (suitability scores and call preparation = output allocation)
  - ``backend/api/template/algorithms/AbstractDeviceAlgorithm.java:127-156`` (executeDeviceAlgorithm) and
    ``:427-449`` (executeOnCommonDevice)
  - ``backend/ocl/CLBackend.java:200-325`` (the op x algorithm -> implementation table)
(paths relative to src/main/java/neureka/ of the reference).
"""
from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np

from .device import HipDevice
from .ndim import IllegalArgumentException, IllegalStateException, Layout

# suitability scores: backend/api/fun/SuitabilityPredicate.java:21-29
PERFECT, EXCELLENT, VERY_GOOD, GOOD, BAD, UNSUITABLE = 1.0, 0.875, 0.75, 0.625, 0.25, 0.0

ACTIVATIONS = ["abs", "cos", "gasu", "gatu", "gaus", "fast_gaus", "gelu", "idy", "ln", "quad", "relu", "selu", "sig",
               "silu", "sin", "softplus", "softsign", "tanh", "fast_tanh", "exp", "log10", "sqrt", "cbrt"]
OPERATORS = {"+": "add", "-": "subtract", "*": "multiply", "/": "divide", "%": "modulo", "**": "power", "^": "power",
             "x": "mul_conv", "@": "matMul"}


@dataclass
class ExecutionCall:
    device: Optional[HipDevice]
    operation: "Operation"
    inputs: List[Optional[object]]
    derivIdx: int = -1
    algorithm: Optional["Algorithm"] = None

    def input(self, i: int):
        return self.inputs[i]

    @property
    def arity(self) -> int:
        return len(self.inputs)

    def getDerivativeIndex(self) -> int:
        return self.derivIdx

    def withInputAt(self, i: int, t) -> "ExecutionCall":
        inputs = list(self.inputs)
        inputs[i] = t
        return ExecutionCall(self.device, self.operation, inputs, self.derivIdx, self.algorithm)

    def withAddedInputAt(self, i: int, t) -> "ExecutionCall":
        inputs = list(self.inputs)
        inputs.insert(i, t)
        return ExecutionCall(self.device, self.operation, inputs, self.derivIdx, self.algorithm)

    def withInputs(self, inputs: Sequence) -> "ExecutionCall":
        return ExecutionCall(self.device, self.operation, list(inputs), self.derivIdx, self.algorithm)


class Algorithm:
    """A device-agnostic algorithm with per-device implementations (backend/api/DeviceAlgorithm.java:40-66)."""

    name = "algorithm"

    def __init__(self):
        self._impls: Dict[type, Callable[[ExecutionCall], object]] = {}

    def setImplementationFor(self, device_class: type, impl) -> "Algorithm":
        self._impls[device_class] = impl
        return self

    def getImplementationFor(self, device) -> Optional[Callable]:
        for cls in type(device).__mro__:
            if cls in self._impls:
                return self._impls[cls]
        return None

    def isSuitableFor(self, call: ExecutionCall) -> float:
        return UNSUITABLE

    def prepare(self, call: ExecutionCall) -> ExecutionCall:
        return call


def _new_output(device: HipDevice, dtype, shape, layout: Layout = Layout.ROW_MAJOR, overwritten: bool = False):
    """``Tensor.of(type).withShape(shape).all(0)`` + ``setIsVirtual(false)`` + ``device.store`` as the call
    preparations do it (e.g. Broadcast.java:90-94).  The reference fills the fresh drain with zeros (on the OpenCL
    device: a clEnqueueFillBuffer of the whole output, OpenCLDevice.java:478-486) and the kernel then writes every
    element.  ``overwritten=True`` says that the implementation the drain goes to does exactly that, so the zeros
    would never be read and the fill (a second pass over the output, as long as the kernel itself for a broadcast)
    is left out; the result is the same bit for bit.  Drains a kernel adds to, or writes in part, keep the fill."""
    from .tensor import Tensor
    t = Tensor._on_device(device, dtype, shape, layout, zeroed=not overwritten)
    t._intermediate = True
    return t


class BiElementwise(Algorithm):
    name = "elementwise"

    def isSuitableFor(self, call):       # BiElementwise.java:17-24
        ts = [t for t in call.inputs if t is not None]
        if all(t.shape == ts[0].shape for t in ts):
            return GOOD
        return UNSUITABLE

    def prepare(self, call):             # BiElementwise.java:42-61
        if call.arity < 3:
            call = call.withAddedInputAt(0, None)
        if call.input(0) is None:
            call = call.withInputAt(0, _new_output(call.device, call.input(1).dtype, call.input(1).shape, overwritten=True))
        return call


class Broadcast(Algorithm):
    name = "broadcast"

    def isSuitableFor(self, call):       # Broadcast.java:18-46
        ts = [t for t in call.inputs if t is not None]
        max_rank = max(t.rank for t in ts)
        for i in range(max_rank):
            current = -1
            for t in ts:
                if i < t.rank:
                    if current == -1:
                        current = t.shape[i]
                    elif current != t.shape[i] and current != 1 and t.shape[i] != 1:
                        return UNSUITABLE
        return GOOD

    def prepare(self, call):             # Broadcast.java:60-97
        from .tensor import make_fit
        if call.arity < 3:
            call = call.withAddedInputAt(0, None)
        offset = 1 if call.input(0) is None else 0
        if call.input(offset).rank != call.input(1 + offset).rank:
            a, b = make_fit([call.input(offset), call.input(1 + offset)])
            call = call.withInputs([None, a, b])
        if call.input(0) is None:
            s1, s2 = call.input(1).shape, call.input(2).shape
            out_shape = tuple(s2[i] if s1[i] == 1 else s1[i] for i in range(len(s1)))
            # the forward kernel writes every element; a drain of the reducing backward kernel arrives from the caller
            call = call.withInputAt(0, _new_output(call.device, call.input(1).dtype, out_shape, overwritten=call.derivIdx < 0))
        return call


class BiScalarBroadcast(Algorithm):
    name = "scalarization"

    def isSuitableFor(self, call):       # BiScalarBroadcast.java:16-29
        ts = call.inputs
        if len(ts) not in (2, 3):
            return UNSUITABLE
        offset = len(ts) - 2
        if ts[1 + offset] is None or ts[offset] is None:
            return UNSUITABLE
        if ts[1 + offset].size > 1 and not ts[1 + offset].isVirtual():
            return UNSUITABLE
        return VERY_GOOD

    def prepare(self, call):             # BiScalarBroadcast.java:30-45
        offset = 1 if call.input(0) is None else 0
        if call.arity == 2:
            offset = 0
        src = call.input(offset)
        out = _new_output(call.device, src.dtype, src.shape, overwritten=True)
        if call.arity == 3:
            return call.withInputAt(0, out)
        return call.withAddedInputAt(0, out)


class ElementwiseAlgorithm(Algorithm):
    name = "activation"

    def isSuitableFor(self, call):
        return GOOD

    def prepare(self, call):             # ElementwiseAlgorithm.java:39-53: a fresh row-major output
        if call.arity < 2:
            call = call.withAddedInputAt(0, None)
        if call.input(0) is None:
            call = call.withInputAt(0, _new_output(call.device, call.input(1).dtype, call.input(1).shape, overwritten=True))
        return call


def _two_slots(call: ExecutionCall) -> List[Optional[object]]:
    """(drain or None, source): the activation calls arrive with one input or with an empty drain slot in front."""
    return [None] + list(call.inputs) if call.arity == 1 else list(call.inputs)


class ScalarAlgorithm(Algorithm):
    """"scalar activation": a function of a virtual tensor is a virtual tensor (algorithms/ScalarAlgorithm.java:15-58)."""
    name = "scalar activation"

    def isSuitableFor(self, call):       # ScalarAlgorithm.java:24-34
        ts = _two_slots(call)
        if len(ts) != 2 or ts[1] is None or not ts[1].isVirtual():
            return UNSUITABLE
        if ts[0] is not None and (not ts[0].isVirtual() or ts[0].shape != ts[1].shape):
            return UNSUITABLE
        return EXCELLENT

    def prepare(self, call):             # ScalarAlgorithm.java:36-46: a virtual output of the source's shape and type
        from .tensor import Tensor
        ts = _two_slots(call)
        if ts[0] is None:
            out = Tensor.of(ts[1].dtype, ts[1].shape, 0.0).to(call.device)
            out._intermediate = True
            ts[0] = out
        return call.withInputs(ts)


class ScalarBroadcast(Algorithm):
    """"scalar broadcast": a function of a virtual tensor written to every element of a full drain
    (algorithms/ScalarBroadcast.java:21-82)."""
    name = "scalar broadcast"

    def isSuitableFor(self, call):       # ScalarBroadcast.java:32-42
        ts = _two_slots(call)
        if len(ts) != 2 or ts[1] is None or not ts[1].isVirtual():
            return UNSUITABLE
        if ts[0] is not None and (ts[0].isVirtual() or ts[0].shape != ts[1].shape):
            return UNSUITABLE
        return VERY_GOOD

    def prepare(self, call):             # ScalarBroadcast.java:44-58: a full (actual) output of the source's shape
        ts = _two_slots(call)
        if ts[0] is None:
            ts[0] = _new_output(call.device, ts[1].dtype, ts[1].shape, overwritten=True)
        return call.withInputs(ts)


class AssignScalar(BiScalarBroadcast):
    """The BiScalarBroadcast of AssignLeft (operations/other/AssignLeft.java:32-71): the last operand is one value
    (virtual or of size 1) that is written to every element of the drain's view."""

    def isSuitableFor(self, call):       # AssignLeft.java:35-51
        if call.arity > 3:
            raise IllegalArgumentException("AssignLeft operation only supports up to 3 arguments!")
        if call.arity < 2:
            raise IllegalArgumentException("AssignLeft operation needs at least 2 arguments!")
        last = call.input(call.arity - 1)
        return PERFECT if last.isVirtual() or last.size == 1 else UNSUITABLE

    def prepare(self, call):             # AssignLeft.java:59-68
        offset = 1 if call.input(0) is None else 0
        call.input(offset).setIsVirtual(False)
        return replace(call, inputs=[call.input(offset), call.input(offset + 1)], derivIdx=-1)


class AssignElementwise(ElementwiseAlgorithm):
    """The ElementwiseAlgorithm of AssignLeft (AssignLeft.java:74-98): drain view <- source view, element by element."""

    def isSuitableFor(self, call):       # AssignLeft.java:76-81
        return EXCELLENT if call.arity in (2, 3) else UNSUITABLE

    def prepare(self, call):             # AssignLeft.java:88-95
        offset = 1 if call.input(0) is None else 0
        return replace(call, inputs=[call.input(offset), call.input(offset + 1)], derivIdx=-1)


class NDConvolution(Algorithm):
    name = "convolution"

    def isSuitableFor(self, call):
        return GOOD

    def prepare(self, call):             # linear/Convolution.java:91-103, ConvUtil.shapeOfCon (ConvUtil.java:61-66)
        inputs = call.inputs if len(call.inputs) > 2 else [None] + list(call.inputs)
        if inputs[0] is None:
            s1, s2 = inputs[1].shape, inputs[2].shape
            shp = tuple([abs(p - q) + 1 for p, q in zip(s1, s2)])
            inputs = [_new_output(call.device, inputs[1].dtype, shp, overwritten=True)] + list(inputs[1:])
        if inputs is call.inputs:
            return call
        return ExecutionCall(call.device, call.operation, inputs, call.derivIdx, call.algorithm)


class MatMulAlgorithm(Algorithm):
    name = "simple_matmul"

    def isSuitableFor(self, call):
        return GOOD

    @staticmethod
    def _is_rm_or_cm(layout: Layout) -> bool:
        return layout in (Layout.ROW_MAJOR, Layout.COLUMN_MAJOR)

    def prepare(self, call):             # MatMulAlgorithm.java:64-155
        if call.arity == 2:
            call = call.withAddedInputAt(0, None)
        if call.input(0) is None:
            a, b = call.input(1), call.input(2)
            la, lb = a.ndc.getLayout(), b.ndc.getLayout()
            if self._is_rm_or_cm(la):
                if lb is not Layout.SYMMETRIC and lb is not la:
                    b = b.toLayoutCopy(la)
                lc = la
            elif self._is_rm_or_cm(lb):
                if la is not Layout.SYMMETRIC and la is not lb:
                    a = a.toLayoutCopy(lb)
                lc = lb
            else:
                lc = Layout.ROW_MAJOR
                a, b = a.toLayoutCopy(lc), b.toLayoutCopy(lc)
            # the registered implementation writes C = A @ B (nk_matmul_set), it does not add to the drain
            out = _new_output(call.device, a.dtype, (a.shape[0], b.shape[1]), lc, overwritten=True)
            call = call.withInputs([out, a, b])
        # _autoClone: anything that is not a dense RM or CM matrix is copied before the kernel sees it
        inputs = []
        for t in call.inputs:
            lay = t.ndc.getLayout()
            if t.rank != 2 or lay not in (Layout.ROW_MAJOR, Layout.COLUMN_MAJOR, Layout.SYMMETRIC) or t.isPartialSlice():
                t = t.deepCopy()
            inputs.append(t)
        return call.withInputs(inputs)


def _dense(t):
    """The reductions read a tensor's buffer front to back: views and virtual tensors are materialised first."""
    if t.isVirtual():
        t.setIsVirtual(False)
    if not t.ndc.isSimple() or t.isPartialSlice() or t.ndc.getLayout() is Layout.COLUMN_MAJOR:
        t = t.deepCopy()
    return t


class SumAlgorithm(Algorithm):
    """algorithms/SumAlgorithm.java:10-52."""
    name = "sum_algorithm"

    def isSuitableFor(self, call):
        return GOOD

    def prepare(self, call):
        return call.withInputs([_dense(call.input(0))])


class ReduceAlgorithm(Algorithm):
    """The min_algorithm / max_algorithm of operations/other/Min.java:33-74 and Max.java."""
    name = "reduce_algorithm"

    def isSuitableFor(self, call):
        return GOOD

    def prepare(self, call):
        return call.withInputs([_dense(call.input(0))])


class DotProductAlgorithm(Algorithm):
    """algorithms/DotProductAlgorithm.java:23-117: vectors only (after trimming extent-1 axes), dense copies."""
    name = "dot_algorithm"

    def isSuitableFor(self, call):
        return GOOD if all(sum(1 for d in t.shape if d > 1) <= 1 for t in call.inputs if t is not None) else UNSUITABLE

    def prepare(self, call):
        from .ndim import NDConfiguration
        from .tensor import Tensor
        ins = []
        for t in call.inputs:
            t = _dense(t)
            if t.rank > 1:               # dimTrim: the same buffer seen as a vector
                v = Tensor(t.dtype, NDConfiguration.ofShape((t.ndc.size,)), None)
                v._set_data(t._data, call.device)
                t = v
            ins.append(t)
        return call.withInputs(ins)


class Operation:
    """An operation with its algorithms (backend/api/Operation.java; template/operations/AbstractOperation.java:178-211)."""

    def __init__(self, identifier: str, operator: str, algorithms: Sequence[Algorithm]):
        self.identifier = identifier
        self.operator = operator
        self.algorithms = list(algorithms)

    def getAlgorithm(self, cls: type) -> Optional[Algorithm]:
        for a in self.algorithms:
            if isinstance(a, cls):
                return a
        return None

    def getAlgorithmFor(self, call: ExecutionCall) -> Algorithm:
        best, score = None, 0.0
        for a in self.algorithms:
            s = a.isSuitableFor(call)
            if s > score:
                best, score = a, s
        if best is None:
            raise IllegalStateException(f"No suitable algorithm found for operation '{self.identifier}'")
        return best


def execute_device_algorithm(call: ExecutionCall):
    """AbstractDeviceAlgorithm.executeDeviceAlgorithm (AbstractDeviceAlgorithm.java:127-156)."""
    for t in call.inputs:
        if t is None:
            raise IllegalArgumentException("Device arguments may not be null!")
    impl = call.algorithm.getImplementationFor(call.device)
    if impl is None:
        raise IllegalStateException(
            f"No '{type(call.device).__name__}' implementation found for algorithm '{call.algorithm.name}' "
            f"of operation '{call.operation.identifier}'")
    call.device.approve(call)
    result = impl(call)
    return call.input(0) if result is None else result


def execute_on_common_device(call: ExecutionCall, run: Callable[[ExecutionCall], object]):
    """AbstractDeviceAlgorithm.executeOnCommonDevice (:427-449): operands that are not on the device are
    stored for the duration of the call and restored afterwards."""
    device = call.device
    guests = [t for t in call.inputs if t is not None and not t.isOutsourced()]
    for t in guests:
        device.store(t)
    try:
        return run(call)
    finally:
        for t in guests:
            if device.has(t):
                device.restore(t)


class BackendContext:
    """Operations by identifier + the extensions registered on them (backend/api/BackendContext.java:170-346)."""

    def __init__(self):
        self.operations: Dict[str, Operation] = {}
        for op_id, sym in [("add", "+"), ("subtract", "-"), ("multiply", "*"), ("divide", "/"), ("modulo", "%"), ("power", "**")]:
            self.operations[op_id] = Operation(op_id, sym, [BiElementwise(), Broadcast(), BiScalarBroadcast()])
        for op_id, sym in [("mul_conv", "x"), ("inv_convolve_mul_left", "«x"), ("inv_convolve_mul_right", "x»")]:
            self.operations[op_id] = Operation(op_id, sym, [NDConvolution()])
        self.operations["matMul"] = Operation("matMul", "@", [MatMulAlgorithm()])
        self.operations["sumItems"] = Operation("sumItems", "sumItems", [SumAlgorithm()])
        self.operations["min"] = Operation("min", "min", [ReduceAlgorithm()])
        self.operations["max"] = Operation("max", "max", [ReduceAlgorithm()])
        self.operations["dot"] = Operation("dot", "dot", [DotProductAlgorithm()])
        for f in ACTIVATIONS:      # functions/AbstractActivationOperation.java:38-50
            self.operations[f] = Operation(f, f, [ElementwiseAlgorithm(), ScalarBroadcast(), ScalarAlgorithm()])
        self.operations["left_inline"] = Operation("left_inline", "<", [AssignScalar(), AssignElementwise()])
        self.operations["random"] = Operation("random", "rand", [ElementwiseAlgorithm()])
        self.extensions: List[object] = []

    def getOperation(self, identifier: str) -> Operation:
        op = self.operations.get(identifier)
        if op is None:
            raise IllegalArgumentException(f"unknown operation '{identifier}'")
        return op

    def set(self, extension) -> "BackendContext":
        """BackendContext.set(BackendExtension) (:289-322): every registration must find its target."""
        extension.load(_Registry(self, extension.device_class()))
        self.extensions.append(extension)
        return self

    def find(self, key: str):
        best, conf = None, 0.0
        for ext in self.extensions:
            dev, c = ext.find(key)
            if c > conf:
                best, conf = dev, c
        return best if conf > 0.42 else None     # devices/Query.java:66-75


class _Registry:
    """The registration DSL (backend/api/ini/BackendRegistry.java:24-51)."""

    def __init__(self, ctx: BackendContext, device_class: type):
        self.ctx, self.device_class = ctx, device_class

    def forOperation(self, identifier: str) -> "_Registry":
        self._op = self.ctx.operations.get(identifier)
        if self._op is None:
            raise IllegalStateException(f"No operation '{identifier}' found for registration")
        return self

    def set(self, algorithm_class: type, impl) -> "_Registry":
        alg = self._op.getAlgorithm(algorithm_class)
        if alg is None:
            raise IllegalStateException(f"Operation '{self._op.identifier}' has no algorithm {algorithm_class.__name__}")
        alg.setImplementationFor(self.device_class, impl)
        return self


# ---- ImplementationFor<HipDevice> ------------------------------------------------------------------
def hip_bi_elementwise(op: str):
    """CLBiElementwise (implementations/elementwise/CLBiElementwise.java:11-24)."""
    def run(call: ExecutionCall):
        call.device.launch_elementwise(op, call.derivIdx, call.input(0), call.input(1), call.input(2))
        return call.input(0)
    return run


def hip_broadcast(op: str):
    """CLBroadcast (implementations/broadcast/CLBroadcast.java:12-24)."""
    def run(call: ExecutionCall):
        call.device.launch_broadcast(op, call.derivIdx, call.input(0), call.input(1), call.input(2))
        return call.input(0)
    return run


def hip_scalar_broadcast(op: str):
    """CLScalarBroadcast<Op>.run (e.g. implementations/broadcast/CLScalarBroadcastAddition.java:15-34)."""
    def run(call: ExecutionCall):
        value = call.input(2).item(0)
        value = int(value) if np.issubdtype(call.input(0).dtype, np.integer) else float(value)
        call.device.launch_scalarization(op, call.derivIdx, call.input(0), call.input(1), value)
        return call.input(0)
    return run


def hip_elementwise_function(fun: str):
    """CLElementwiseFunction (implementations/elementwise/CLElementwiseFunction.java:27-41)."""
    def run(call: ExecutionCall):
        call.device.launch_activation(fun, call.derivIdx, call.input(0), call.input(1))
        return call.input(0)
    return run


def hip_scalar_function(fun: str):
    """CLScalarFunction (implementations/scalar/CLScalarFunction.java:11-29): drain item 0 = f(source item 0), both
    tensors virtual.  The reference evaluates f on the host and writes the item; here the one stored element goes
    through the activation kernel on the device, so no value crosses the bus and f is the device's f."""
    def run(call: ExecutionCall):
        call.device.launch_activation_item(fun, call.derivIdx, call.input(0), call.input(1))
        return call.input(0)
    return run


def hip_scalar_broadcast_function(fun: str):
    """ScalarBroadcast (algorithms/ScalarBroadcast.java:21-82): value = f(source item 0), written through the drain's view.
    f is evaluated by the device's own activation kernel on the one stored element, in the drain's type: what the CPU
    device does (CPUScalarBroadcastFunction.java:43-67: ``f.invoke(double)`` for Double, ``f.invoke(float)`` for Float
    tensors), which is the parity target.  The OpenCL device's lambda (ScalarBroadcast.java:64-81) evaluates f in double
    on the host and hands ``(float) value`` to its kernel for every type, so it drops digits of an f64 result; that
    rounding is an oddity of that lambda, not of the operation, and is not repeated here."""
    def run(call: ExecutionCall):
        dev, drn, src = call.device, call.input(0), call.input(1)
        slot = dev.allocate(drn.dtype, 1)
        try:
            dev.launch_activation_item(fun, call.derivIdx, slot, src)
            value = float(dev._read(slot, 0, 1)[0])         # the reference reads the item too (blocking)
        finally:
            slot.release()
        dev.launch_scalar_fill(drn, value)
        return drn
    return run


def hip_scalar_broadcast_identity(call: ExecutionCall):
    """CLScalarBroadcastIdentity (implementations/broadcast/CLScalarBroadcastIdentity.java:18-32): the drain is passed
    as drain and as source, the kernel writes the value."""
    drn = call.input(0)
    value = call.input(1).item(0)
    value = int(value) if np.issubdtype(drn.dtype, np.integer) else float(value)
    call.device.launch_scalarization("idy", call.derivIdx, drn, drn, value)
    return drn


def hip_assign_elementwise(call: ExecutionCall):
    """CLElementwiseFunction(ScalarFun.IDENTITY) as AssignLeft registers it (backend/ocl/CLBackend.java:232-234); the
    drain is made actual first as CPUElementwiseAssignFun does (implementations/elementwise/CPUElementwiseAssignFun.java:30)."""
    drn, src = call.input(0), call.input(1)
    if drn.shape != src.shape:
        raise IllegalArgumentException(f"cannot assign a tensor of shape {list(src.shape)} to one of shape {list(drn.shape)}")
    drn.setIsVirtual(False)
    call.device.launch_activation("idy", -1, drn, src)
    return drn


def hip_randomization(call: ExecutionCall):
    """CLRandomization (implementations/elementwise/CLRandomization.java:8-13) is a stub that throws; so is this."""
    raise IllegalStateException("Not yet implemented")


def hip_convolution(call: ExecutionCall):
    """CLConvolution (implementations/convolution/CLConvolution.java:11-23)."""
    call.device.launch_convolution(call.derivIdx, call.input(0), call.input(1), call.input(2))
    return call.input(0)


def hip_matmul(call: ExecutionCall):
    """CLMatMul / CPUMatMul (implementations/matmul/CPUMatMul.java:17-96): layout check, then the product, written
    over the drain as the OpenCL device's kernel does (CLMatMul.java:50; the drain arrives zeroed: MatMulAlgorithm.java:74-85)."""
    c, a, b = call.input(0), call.input(1), call.input(2)
    la, lb = a.ndc.getLayout(), b.ndc.getLayout()
    if not (la.isCompatible(lb) and la.isCompatible(c.ndc.getLayout()) and lb.isCompatible(c.ndc.getLayout())):
        raise IllegalArgumentException("Data layout inconsistency between provided tensors encountered. All tensors must be of the same layout.")
    if not (a.dtype == b.dtype == c.dtype):
        raise IllegalArgumentException("Type inconsistency between provided tensors encountered. All tensors must be of the same type.")
    row_major = all(l in (Layout.ROW_MAJOR, Layout.SYMMETRIC) for l in (la, lb))
    if a.shape[1] != b.shape[0]:
        raise IllegalArgumentException(f"'A' matrix rows {a.shape[1]} did not match 'B' matrix columns {b.shape[0]}.")
    call.device.launch_matmul(row_major, a.shape[0], a.shape[1], b.shape[1], a, b, c, accumulate=False)
    return c


def hip_sum(call: ExecutionCall):
    """CLSum (operations/linear/internal/opencl/CLSum.java:12-62)."""
    from .tensor import Tensor
    src = call.input(0)
    out = Tensor._on_device(call.device, src.dtype, (1,), zeroed=False)
    call.device.launch_sum(src, out)
    return out


def hip_reduce(kind: str):
    """CLReduce + the execution of operations/other/Min.java:43-52: the kernel finds the index, the item is read
    back and wrapped into a tensor of one element that remembers the index for the backward pass."""
    def run(call: ExecutionCall):
        from .tensor import Tensor
        src = call.input(0)
        i = call.device.reduce_index(kind, src)
        out = Tensor.of(src.dtype, (1,), src.item(i)).to(call.device)
        out._found_index = i
        return out
    return run


def hip_dot(call: ExecutionCall):
    """CLDot (implementations/linear/CLDot.java:17-56)."""
    from .tensor import Tensor
    a, b = call.input(0), call.input(1)
    if a.rank != 1 or b.rank != 1:
        raise IllegalArgumentException("Input tensors must be vectors.")
    if a.shape[0] != b.shape[0]:
        raise IllegalArgumentException("Input vectors must have the same length.")
    out = Tensor._on_device(call.device, a.dtype, (1,), zeroed=False)
    call.device.launch_dot(a, b, out)
    return out


class HipBackend:
    """``BackendExtension`` for HipDevice (model: backend/ocl/CLBackend.java:56-325)."""

    KEYWORDS = ("hip", "rocm", "amd", "radeon", "gpu", "first gpu", "mi355x", "instinct")

    def device_class(self) -> type:
        return HipDevice

    def find(self, key: str):
        """DeviceOption(device, confidence): keyword match on the search key (CLBackend.java:56-94; devices/Query.java:22-24)."""
        k = key.lower().strip()
        if HipDevice.count() == 0:
            return None, 0.0
        dev = HipDevice.get(0)
        if any(w == k or w in k.split() for w in self.KEYWORDS) or k in dev.name().lower():
            return dev, 1.0
        return dev, 0.0

    def load(self, registry: _Registry) -> None:
        for op in ("add", "subtract", "multiply", "divide", "modulo", "power"):
            (registry.forOperation(op)
                .set(BiScalarBroadcast, hip_scalar_broadcast(op))
                .set(Broadcast, hip_broadcast(op))
                .set(BiElementwise, hip_bi_elementwise(op)))
        for op in ("mul_conv", "inv_convolve_mul_left", "inv_convolve_mul_right"):
            registry.forOperation(op).set(NDConvolution, hip_convolution)
        registry.forOperation("matMul").set(MatMulAlgorithm, hip_matmul)
        registry.forOperation("sumItems").set(SumAlgorithm, hip_sum)
        registry.forOperation("min").set(ReduceAlgorithm, hip_reduce("min"))
        registry.forOperation("max").set(ReduceAlgorithm, hip_reduce("max"))
        registry.forOperation("dot").set(DotProductAlgorithm, hip_dot)
        (registry.forOperation("left_inline")                                    # CLBackend.java:232-234
            .set(BiScalarBroadcast, hip_scalar_broadcast_identity)
            .set(ElementwiseAlgorithm, hip_assign_elementwise))
        registry.forOperation("random").set(ElementwiseAlgorithm, hip_randomization)     # CLBackend.java:252-253
        for f in ACTIVATIONS:                                                    # CLBackend.java:255-324
            (registry.forOperation(f)
                .set(ElementwiseAlgorithm, hip_elementwise_function(f))
                .set(ScalarAlgorithm, hip_scalar_function(f)))
            # ScalarBroadcast carries its device implementation itself (ScalarBroadcast.java:64-81): it is attached
            # to the algorithm object, not through a registry row
            self.context_operation(registry, f).getAlgorithm(ScalarBroadcast).setImplementationFor(
                HipDevice, hip_scalar_broadcast_function(f))

    @staticmethod
    def context_operation(registry: _Registry, identifier: str) -> "Operation":
        return registry.ctx.getOperation(identifier)

    def dispose(self) -> None:
        for dev in list(HipDevice._open.values()):
            dev.dispose()


_context: Optional[BackendContext] = None


def backend() -> BackendContext:
    """The process-wide context with HipBackend registered (Neureka.get().backend(), Neureka.java:113-147)."""
    global _context
    if _context is None:
        _context = BackendContext().set(HipBackend())
    return _context
