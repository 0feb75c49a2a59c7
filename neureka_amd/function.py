"""Expression strings, operation dispatch and reverse-mode wiring for the hot path.

  - ``Function.of("tanh(sig(I[0])*I[1]+I[2])")``: a small parser in the spirit of
    ``math/parsing/FunctionParser.java``; nested expressions execute operation by operation through
    temporaries, exactly as ``AbstractDeviceAlgorithm.flatten`` makes the reference do
    (``backend/api/template/algorithms/AbstractDeviceAlgorithm.java:177-204``).
  - ``execute(op, inputs)``: ``Operation.execute`` (``backend/api/Operation.java:200-237``): pick the algorithm,
    prepare the call (allocate the drain), run the HipDevice implementation, record the ADActions.
  - ``OptimizedFunction``: what ``Device.optimizedFunctionOf`` returns (``devices/Device.java:216-243``): the
    whole expression as one fused kernel launch (``nk_fused``).
(paths relative to src/main/java/neureka/ of the reference)
"""
from __future__ import annotations

import re

import numpy as np
from typing import List, Optional, Sequence, Union

from . import _lib
from .backend import (ACTIVATIONS, BiElementwise, BiScalarBroadcast, Broadcast, ExecutionCall, ScalarAlgorithm,
                      ScalarBroadcast, backend, execute_device_algorithm, execute_on_common_device)
from .ndim import IllegalArgumentException, IllegalStateException
from .tensor import GraphNode, Tensor, make_fit


def _device_for(inputs: Sequence[Tensor]):
    """FunctionNode._deviceFor (math/implementations/FunctionNode.java:109-137)."""
    for t in inputs:
        if t is not None and t.isOutsourced():
            return t.getDevice()
    raise IllegalStateException("none of the operands is stored on a HipDevice; this package has no host arithmetic path")


def execute(op_id: str, inputs: Sequence[Tensor], d: int = -1, record: bool = True) -> Tensor:
    ctx = backend()
    operation = ctx.getOperation(op_id)
    device = _device_for(inputs)
    if op_id == "left_inline":               # operations/other/AssignLeft.java:103-114: inline, no autograd
        if d >= 0:
            raise IllegalArgumentException("Assignment does not support autograd!")
        record = False
    parents = list(inputs)                   # the tensors the caller holds: gradients attach to these
    if len(inputs) > 1 and op_id != "dot" and any(len(t.ndc.shape) != len(inputs[0].ndc.shape) for t in inputs):
        inputs = make_fit(list(inputs))      # FunctionNode.execute pads ranks first (FunctionNode.java:92-93)
    call = ExecutionCall(device, operation, list(inputs), d)
    call.algorithm = operation.getAlgorithmFor(call)

    def run(c: ExecutionCall):
        c = c.algorithm.prepare(c)
        for t in c.inputs[1:]:
            if t.isVirtual() and not isinstance(c.algorithm, (BiScalarBroadcast, ScalarAlgorithm, ScalarBroadcast)):
                t.setIsVirtual(False)       # sources are de-virtualised before the kernels (CPUBiElementWise.java:103-104)
        return execute_device_algorithm(c), c

    result, prepared = execute_on_common_device(call, run)
    if record and d < 0 and any(t.rqsGradient() or t._node is not None for t in parents):
        result._node = _graph_node(op_id, prepared, parents, result)
    return result


# ---- ADActions -------------------------------------------------------------------------------------
def _graph_node(op_id: str, call: ExecutionCall, inputs: List[Tensor], result: Tensor) -> GraphNode:
    alg = call.algorithm
    actions = []
    for d, parent in enumerate(inputs):
        if not (parent.rqsGradient() or parent._node is not None):
            actions.append(None)
            continue
        actions.append(_ad_action(op_id, alg, call, inputs, d, result))
    return GraphNode(inputs, actions)


def _ad_action(op_id: str, alg, call: ExecutionCall, inputs: List[Tensor], d: int, result: Optional[Tensor] = None):
    device = call.device
    prepared_in = call.inputs[1:]            # operands as the kernel saw them (rank-fitted)
    if op_id == "mul_conv":
        # linear/Convolution.java:56-89: "I[0] x>> I[1] x>> I[2]" on (error, derivative, zeros like the target);
        # ConvUtil.executeRecursively rearranges to (zeros, derivative, error) and runs the kernel with d >= 0
        other = prepared_in[1 - d]
        target_shape = prepared_in[d].shape
        def act(error: Tensor) -> Tensor:
            # "zeros like the target" in the reference; the gradient kernels assign every element of the drain
            # (AbstractCPUConvolution.java:319-408 ends each element with t0_value[i] = value), so the fill is left out
            zeros = Tensor._on_device(device, other.dtype, target_shape, zeroed=False)
            c = ExecutionCall(device, backend().getOperation("inv_convolve_mul_right"), [zeros, other, error], 0)
            c.algorithm = c.operation.algorithms[0]
            return execute_on_common_device(c, lambda cc: execute_device_algorithm(cc))
        return act
    if op_id == "sumItems":
        # SumAlgorithm.java:27-31: the error of one element becomes a tensor of the summed shape filled with it
        shape, dtype = inputs[0].shape, inputs[0].dtype
        return lambda error: Tensor.of(dtype, shape, error.item(0)).to(device).setIsVirtual(False)
    if op_id in ("min", "max"):
        # Min.java:53-60: zeros like the input with the error at the index that was found
        shape, dtype, found = inputs[0].shape, inputs[0].dtype, result._found_index
        def act(error: Tensor) -> Tensor:
            g = np.zeros(int(np.prod(shape)), dtype=dtype)
            g[found] = error.item(0)
            return Tensor.of(dtype, shape, g).to(device)
        return act
    if op_id == "dot":
        # DotProductAlgorithm.java:40-47: error (one element) times a copy of the other operand
        other = inputs[(1 + d) % 2]
        return lambda error: execute("multiply", [error, other.deepCopy()], record=False)
    if op_id == "matMul":
        # MatMulAlgorithm.java:37-59: d' = (1 + d) % 2 picks the operand to transpose
        a, b = prepared_in
        if d == 0:
            return lambda error: execute("matMul", [error, b.T().deepCopy()], record=False)
        return lambda error: execute("matMul", [a.T().deepCopy(), error], record=False)
    if op_id in ACTIVATIONS:
        src = prepared_in[0]
        def act(error: Tensor) -> Tensor:
            local = execute(op_id, [src], d=0, record=False)
            return execute("multiply", [error, local], record=False)
        return act
    broadcasting = isinstance(alg, Broadcast) or (isinstance(alg, BiScalarBroadcast) and prepared_in[0].shape != prepared_in[1].shape)
    if broadcasting and op_id in ("add", "subtract"):
        alg = call.operation.getAlgorithm(Broadcast)
        # operator/Addition.java:90-109 (_autogradBroadcast): the reducing backward kernel on
        # (zeros like operand d, zeros like the other operand, error)
        tgt, other = prepared_in[d], prepared_in[1 - d]
        def act(error: Tensor) -> Tensor:
            # the reducing kernel assigns every element of the drain (CPUBroadcast.java:209-257); the "derivative"
            # operand is an input of the kernel and keeps its zeros
            to_be_derived = Tensor._on_device(device, tgt.dtype, tgt.shape, zeroed=False)
            derivative = Tensor._on_device(device, other.dtype, other.shape)
            c = ExecutionCall(device, call.operation, [to_be_derived, derivative, error], d, alg)
            return execute_on_common_device(c, lambda cc: execute_device_algorithm(cc))
        return act
    if op_id in ("add", "subtract", "multiply", "divide", "modulo", "power"):
        # default ADAction: error * d f / d operand (FallbackAlgorithm.ADAction); for a broadcast multiply
        # this keeps the output's shape, as operator/Multiplication.java:55-69 does
        def act(error: Tensor) -> Tensor:
            a, b = prepared_in
            if op_id == "multiply":
                local = b if d == 0 else a
            else:
                c = ExecutionCall(device, call.operation, [None, a, b], d, call.operation.getAlgorithm(BiElementwise))
                c = c.algorithm.prepare(c)
                local = execute_on_common_device(c, lambda cc: execute_device_algorithm(cc))
            return execute("multiply", [error, local], record=False)
        return act
    raise IllegalStateException(f"no ADAction for operation '{op_id}'")


REDUCTIONS = ("min", "max", "sumItems")       # functions of one argument that are not elementwise


# ---- expression parsing ---------------------------------------------------------------------------
class Node:
    def __init__(self, kind: str, value=None, children: Optional[List["Node"]] = None):
        self.kind, self.value, self.children = kind, value, children or []    # kind: input | const | fun | op

    def __repr__(self):
        if self.kind in ("input", "const"):
            return f"I[{self.value}]" if self.kind == "input" else repr(self.value)
        if self.kind == "fun":
            return f"{self.value}({self.children[0]!r})"
        return f"({self.children[0]!r} {self.value} {self.children[1]!r})"


_TOKEN = re.compile(r"\s*(?:(\d+\.\d*(?:[eE][-+]?\d+)?|\d+(?:[eE][-+]?\d+)?)|([iI]\[?\s*\d+\s*\]?)|([A-Za-z_][A-Za-z_0-9]*)|(\*\*|<-|[-+*/%^()@,]))")
_BIN_OPS = {"<-": ("left_inline", 0), "+": ("add", 1), "-": ("subtract", 1), "*": ("multiply", 2), "/": ("divide", 2), "%": ("modulo", 2),
            "x": ("mul_conv", 2), "@": ("matMul", 2), "^": ("power", 3), "**": ("power", 3)}


def _tokenize(expr: str) -> List[tuple]:
    out, pos = [], 0
    expr = expr.strip()
    while pos < len(expr):
        m = _TOKEN.match(expr, pos)
        if not m:
            raise IllegalArgumentException(f"cannot parse '{expr}' at position {pos}")
        num, inp, name, sym = m.groups()
        if num is not None: out.append(("num", float(num)))
        elif inp is not None: out.append(("input", int(re.sub(r"\D", "", inp))))
        elif name is not None: out.append(("name", name))
        else: out.append(("sym", sym))
        pos = m.end()
    return out


class _Parser:
    def __init__(self, tokens): self.t, self.i = tokens, 0
    def peek(self): return self.t[self.i] if self.i < len(self.t) else (None, None)
    def next(self): tok = self.peek(); self.i += 1; return tok

    def expr(self, min_prec: int = 0) -> Node:
        left = self.atom()
        while True:
            kind, val = self.peek()
            sym = val if kind == "sym" else ("x" if (kind, val) == ("name", "x") else None)
            if sym not in _BIN_OPS or _BIN_OPS[sym][1] < min_prec:
                return left
            self.next()
            op, prec = _BIN_OPS[sym]
            right = self.expr(prec if op == "left_inline" else prec + 1)     # a <- b <- c nests to the right
            left = Node("op", op, [left, right])

    def atom(self) -> Node:
        kind, val = self.next()
        if kind == "num": return Node("const", val)
        if kind == "input": return Node("input", val)
        if kind == "sym" and val == "(":
            n = self.expr()
            if self.next() != ("sym", ")"): raise IllegalArgumentException("missing ')'")
            return n
        if kind == "sym" and val == "-":
            return Node("op", "multiply", [Node("const", -1.0), self.atom()])
        if kind == "name":
            if val not in ACTIVATIONS and val not in REDUCTIONS: raise IllegalArgumentException(f"unknown function '{val}'")
            if self.next() != ("sym", "("): raise IllegalArgumentException(f"'(' expected after {val}")
            arg = self.expr()
            if self.next() != ("sym", ")"): raise IllegalArgumentException("missing ')'")
            return Node("fun", val, [arg])
        raise IllegalArgumentException(f"unexpected token {val!r}")


class Function:
    """``Function.of(expression)``; calling it executes operation by operation on the operands' device."""

    def __init__(self, expression: str, doAD: bool = True):
        self.expression = expression
        self.doAD = doAD
        p = _Parser(_tokenize(expression))
        self.root = p.expr()
        if p.i != len(p.t):
            raise IllegalArgumentException(f"trailing input in '{expression}'")

    @staticmethod
    def of(expression: str, doAD: bool = True) -> "Function":
        return Function(expression, doAD)

    def numberOfArgs(self) -> int:
        def walk(n): return max([n.value + 1] if n.kind == "input" else [0] + [walk(c) for c in n.children])
        return walk(self.root)

    def isFlat(self) -> bool:
        return all(c.kind in ("input", "const") for c in self.root.children)

    def call(self, *inputs: Tensor) -> Tensor:
        if len(inputs) == 1 and isinstance(inputs[0], (list, tuple)):
            inputs = tuple(inputs[0])
        return self._eval(self.root, inputs)

    __call__ = call
    execute = call

    def _eval(self, n: Node, inputs) -> Union[Tensor, float]:
        if n.kind == "input":
            if n.value >= len(inputs):
                raise IllegalArgumentException(f"function '{self.expression}' needs input {n.value}, {len(inputs)} given")
            return inputs[n.value]
        if n.kind == "const":
            ref = next(t for t in inputs if isinstance(t, Tensor))
            return Tensor.of(ref.dtype, (1,), n.value)
        args = [self._eval(c, inputs) for c in n.children]
        return execute(n.value, args, record=self.doAD)

    def derive(self, inputs: Sequence[Tensor], index: int) -> Tensor:
        """d f / d I[index] for a flat unary function (``func.derive([t], 0)`` of Calculus_Stress_Test.groovy:255-256)."""
        if self.root.kind == "fun" and self.root.children[0].kind == "input" and self.root.children[0].value == index:
            return execute(self.root.value, [inputs[index]], d=0, record=False)
        raise IllegalArgumentException("derive() is provided for flat activation functions only")


def _const(v: float) -> Node:
    return Node("const", float(v))


def _is_const(n: Node, v: float) -> bool:
    return n.kind == "const" and n.value == v


def _mul(a: Node, b: Node) -> Node:
    if _is_const(a, 0.0) or _is_const(b, 0.0): return _const(0.0)
    if _is_const(a, 1.0): return b
    if _is_const(b, 1.0): return a
    return Node("op", "multiply", [a, b])


def _add(a: Node, b: Node) -> Node:
    if _is_const(a, 0.0): return b
    if _is_const(b, 0.0): return a
    return Node("op", "add", [a, b])


def _sub(a: Node, b: Node) -> Node:
    if _is_const(b, 0.0): return a
    if _is_const(a, 0.0): return _mul(_const(-1.0), b)
    return Node("op", "subtract", [a, b])


def derivative_of(n: Node, index: int) -> Node:
    """The expression tree of d n / d I[index] (the role of Function.getDerivative in
    devices/opencl/utility/CLFunctionCompiler.java:155-157), with 0 and 1 folded away.  ``dfun`` nodes stand for
    the derivative of a unary function at their argument."""
    if n.kind == "input":
        return _const(1.0 if n.value == index else 0.0)
    if n.kind == "const":
        return _const(0.0)
    if n.kind == "fun":
        u = n.children[0]
        return _mul(Node("dfun", n.value, [u]), derivative_of(u, index))
    if n.kind == "dfun":
        raise IllegalArgumentException("second derivatives of fused functions are not supported")
    u, v = n.children
    du, dv = derivative_of(u, index), derivative_of(v, index)
    if n.value == "add": return _add(du, dv)
    if n.value == "subtract": return _sub(du, dv)
    if n.value == "multiply": return _add(_mul(du, v), _mul(u, dv))
    if n.value == "divide":          # du / v - u * dv / v^2
        return _sub(Node("op", "divide", [du, v]) if not _is_const(du, 0.0) else _const(0.0),
                    _mul(dv, Node("op", "divide", [u, Node("op", "multiply", [v, v])])))
    if n.value == "power":           # d(u^v) = v * u^(v-1) * du + u^v * ln(u) * dv
        first = _mul(_mul(v, Node("op", "power", [u, Node("op", "subtract", [v, _const(1.0)])])), du)
        second = _mul(_mul(Node("op", "power", [u, v]), Node("fun", "ln", [u])), dv)
        return _add(first, second)
    if n.value == "modulo":          # operator/Modulo.java:183-185: the derivative of the first operand
        return du
    raise IllegalArgumentException(f"operator '{n.value}' has no fused derivative")


# what one launch of nk_fused takes (include/neureka_hip.h: NK_FUSE_MAX_*)
FUSE_MAX_SRC, FUSE_MAX_OPS, FUSE_MAX_STACK, FUSE_MAX_CONST, FUSE_MAX_SAVED = 6, 32, 8, 8, 4


def _fuse_cost(n: Node):
    """(op-codes, stack depth, leaves, constants) of the postfix program of the tree; leaves are inputs and temporaries."""
    if n.kind in ("input", "temp"):
        return 1, 1, {(n.kind, n.value)}, set()
    if n.kind == "const":
        return 1, 1, set(), {n.value}
    if n.kind in ("fun", "dfun"):
        ops, depth, leaves, consts = _fuse_cost(n.children[0])
        return ops + 1, depth, leaves, consts
    o1, d1, l1, c1 = _fuse_cost(n.children[0])
    o2, d2, l2, c2 = _fuse_cost(n.children[1])
    return o1 + o2 + 1, max(d1, d2 + 1), l1 | l2, c1 | c2


def _fuse_saved(n: Node) -> int:
    """How many intermediate results the program of the tree holds at once while it evaluates another sub-expression.
    The kernel works on one accumulator: an operand that is a plain source or constant is read where it is used,
    a computed operand that has to wait for the evaluation of its right-hand neighbour is saved (the rule nk_fused
    applies when it translates the postfix program)."""
    LAZY, ACC, SAVED = 0, 1, 2
    stack, saved, peak = [], 0, 0

    def save_acc():
        nonlocal saved, peak
        for i, kind in enumerate(stack):
            if kind == ACC:
                stack[i] = SAVED
                saved += 1
        peak = max(peak, saved)

    def walk(m: Node):
        nonlocal saved
        if not m.children:
            stack.append(LAZY)
        elif m.kind in ("fun", "dfun"):
            walk(m.children[0])
            if stack[-1] == LAZY:
                save_acc()
                stack[-1] = ACC
        else:
            walk(m.children[0]); walk(m.children[1])
            rhs, lhs = stack.pop(), stack.pop()
            if lhs == LAZY and rhs == LAZY:
                save_acc()
            elif lhs == SAVED:
                saved -= 1
            stack.append(ACC)
    walk(n)
    return peak


def _fuse_fits(n: Node) -> bool:
    ops, depth, leaves, consts = _fuse_cost(n)
    return (ops <= FUSE_MAX_OPS and depth <= FUSE_MAX_STACK and len(leaves) <= FUSE_MAX_SRC and len(consts) <= FUSE_MAX_CONST
            and _fuse_saved(n) <= FUSE_MAX_SAVED)


def plan_fused(root: Node):
    """Cuts an expression that is too large for one launch of nk_fused (more than 6 sources, 32 op-codes, 8 stack
    entries, 8 constants or 4 saved intermediates) into stages: the largest sub-expressions are evaluated into temporaries first, which
    later stages read as sources.  Every intermediate of a fused program is rounded to the tensor's element type as
    the unfused kernels round it, so a temporary holds exactly what the single program would have had on its stack
    (CLFunctionCompiler generates one OpenCL kernel whatever the size, CLFunctionCompiler.java:101-199).
    Returns [(program, consts, leaves)], leaves = [("input", k) | ("temp", stage)] in source-slot order; the last
    stage writes the result."""
    stages = []

    def lower(n: Node):
        leaves, consts, program = [], [], []

        def walk(m: Node):
            if m.kind in ("input", "temp"):
                key = (m.kind, m.value)
                if key not in leaves:
                    leaves.append(key)
                program.extend([_lib.FUSE_LOAD, leaves.index(key)])
            elif m.kind == "const":
                if m.value not in consts:
                    consts.append(m.value)
                program.extend([_lib.FUSE_CONST, consts.index(m.value)])
            elif m.kind in ("fun", "dfun"):
                if m.value not in _lib.FUN:
                    raise IllegalArgumentException(f"function '{m.value}' cannot be fused into an elementwise kernel")
                walk(m.children[0])
                program.extend([_lib.FUSE_FUN if m.kind == "fun" else _lib.FUSE_DFUN, _lib.FUN[m.value]])
            else:
                if m.value not in _lib.OP:
                    raise IllegalArgumentException(f"operator '{m.value}' cannot be fused into an elementwise kernel")
                walk(m.children[0]); walk(m.children[1])
                program.extend([_lib.FUSE_BIN, _lib.OP[m.value]])
        walk(n)
        return program, consts, leaves

    def reduce(n: Node) -> Node:
        if not n.children:
            return n
        children = [reduce(c) for c in n.children]            # every child fits one launch by itself now
        m = Node(n.kind, n.value, children)
        while not _fuse_fits(m):
            big = max((i for i, c in enumerate(children) if c.children), key=lambda i: _fuse_cost(children[i])[0])
            stages.append(lower(children[big]))
            children[big] = Node("temp", len(stages) - 1)
            m = Node(n.kind, n.value, children)
        return m

    final = reduce(root)
    if final.kind == "temp":                                  # (cannot happen: a temporary is only made of a child)
        final = Node("fun", "idy", [final])
    stages.append(lower(final))
    return stages


class OptimizedFunction:
    """One fused kernel for a whole elementwise expression (the counterpart of CLFunctionCompiler,
    devices/opencl/utility/CLFunctionCompiler.java:27-238): the expression tree is lowered to the postfix
    op-codes of ``nk_fused``; operands must share one shape (views are fine).  Expressions beyond what one launch
    takes run as several launches through temporaries (plan_fused)."""

    def __init__(self, device, function: Function, name: str):
        self.device, self.function, self.name = device, function, name
        self.n_src = function.numberOfArgs()
        self.stages = plan_fused(function.root)
        # the single-launch form, sources in input order: what callers that prepare the launch themselves use
        self.program: List[int] = []
        self.consts: List[float] = []
        if len(self.stages) == 1 and self.n_src <= FUSE_MAX_SRC:
            self._lower(function.root, self.program, self.consts)
        self._derivatives = {}               # input index -> stages of the derivative kernel

    @staticmethod
    def _lower(n: Node, program: List[int], consts: List[float]) -> None:
        if n.kind == "input":
            program += [_lib.FUSE_LOAD, n.value]
        elif n.kind == "const":
            if n.value not in consts:
                consts.append(n.value)
            program += [_lib.FUSE_CONST, consts.index(n.value)]
        elif n.kind in ("fun", "dfun"):
            if n.value not in _lib.FUN:
                raise IllegalArgumentException(f"function '{n.value}' cannot be fused into an elementwise kernel")
            OptimizedFunction._lower(n.children[0], program, consts)
            program += [_lib.FUSE_FUN if n.kind == "fun" else _lib.FUSE_DFUN, _lib.FUN[n.value]]
        else:
            if n.value not in _lib.OP:
                raise IllegalArgumentException(f"operator '{n.value}' cannot be fused into an elementwise kernel")
            OptimizedFunction._lower(n.children[0], program, consts)
            OptimizedFunction._lower(n.children[1], program, consts)
            program += [_lib.FUSE_BIN, _lib.OP[n.value]]

    def derivative_stages(self, index: int):
        """Stages of the kernel(s) for d f / d I[index] (CLFunctionCompiler compiles it next to the activation)."""
        if index not in self._derivatives:
            self._derivatives[index] = plan_fused(derivative_of(self.function.root, index))
        return self._derivatives[index]

    def derivative_program(self, index: int):
        """Op-codes and constants of d f / d I[index] when it is one launch with the sources in input order."""
        program, consts = [], []
        self._lower(derivative_of(self.function.root, index), program, consts)
        return program, consts

    def _run_stages(self, stages, srcs: List[Tensor]) -> Tensor:
        temps = {}
        out = None
        try:
            for k, (program, consts, leaves) in enumerate(stages):
                operands = [srcs[v] if kind == "input" else temps[v] for kind, v in leaves]
                if not operands:                     # a constant expression: the drain's shape comes from the first input
                    operands = [srcs[0]]
                out = Tensor._on_device(self.device, srcs[0].dtype, srcs[0].shape, zeroed=False)
                self.device.launch_fused(program, consts, out, operands)
                temps[k] = out
        finally:
            for k, t in temps.items():
                if t is not out and self.device.has(t):
                    self.device.free(t)
        return out

    def _with_guests(self, srcs: List[Tensor], run):
        """Operands that are not on the device are stored for the call and restored afterwards
        (AbstractDeviceAlgorithm.executeOnCommonDevice, AbstractDeviceAlgorithm.java:427-449)."""
        guests = [t for t in srcs if not t.isOutsourced()]
        for t in guests:
            self.device.store(t)
        try:
            for t in srcs:
                t.setIsVirtual(False)
            return run()
        finally:
            for t in guests:
                if self.device.has(t):
                    self.device.restore(t)

    def derive(self, inputs: Sequence[Tensor], index: int) -> Tensor:
        """d f / d I[index] at the inputs, in one launch."""
        srcs = list(inputs[: self.n_src])
        stages = self.derivative_stages(index)
        return self._with_guests(srcs, lambda: self._run_stages(stages, srcs))

    def call(self, *inputs: Tensor) -> Tensor:
        if len(inputs) == 1 and isinstance(inputs[0], (list, tuple)):
            inputs = tuple(inputs[0])
        if len(inputs) < self.n_src:
            raise IllegalArgumentException(f"'{self.name}' needs {self.n_src} inputs, {len(inputs)} given")
        srcs = list(inputs[: self.n_src])
        for t in srcs:
            if t.shape != srcs[0].shape:
                raise IllegalArgumentException("operands of a fused function must share one shape")

        out = self._with_guests(srcs, lambda: self._run_stages(self.stages, srcs))
        if self.function.doAD and any(t.rqsGradient() or t._node is not None for t in srcs):
            # reverse mode: error * (d f / d I[d]), the derivative in one fused launch (operands that live on the
            # host are stored again for that launch)
            def action(d):
                return lambda error: execute("multiply", [error, self.derive(srcs, d)], record=False)
            out._node = GraphNode(srcs, [action(d) if (t.rqsGradient() or t._node is not None) else None for d, t in enumerate(srcs)])
        return out

    __call__ = call
