"""CPU-only tests of the host-side mirror: view descriptors, the expression parser, the C ABI surface
(library loads, every declared symbol is exported).  No compute calls, no GPU."""
import ctypes
import os
import re

import numpy as np
import pytest

from neureka_amd import IllegalArgumentException, IllegalStateException, Layout, NDConfiguration, _lib
from neureka_amd.function import Function, OptimizedFunction
from neureka_amd.tensor import Tensor, physical_indices

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "neureka_hip.h")).read()
    declared = set(re.findall(r"\b(nk_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [name for name in sorted(declared) if not hasattr(lib, name)]
    assert not missing, f"declared in include/neureka_hip.h but not exported: {missing}"
    assert declared == set(_lib.SYMBOLS), "the ctypes table and the header disagree"
    _lib.load()


def test_specialised_class_choice_matches_ndconfiguration_spec(golden):
    for shape, strides, imap, spread, offset, expected in golden["ndconfiguration_spec"]["rows"]:
        ndc = NDConfiguration.of(shape, strides, imap, spread, offset)
        assert ndc.kind() == expected, (shape, strides, imap, spread, offset)
        inline = ndc.asInlineArray().tolist()
        assert inline == shape + strides + imap + offset + spread      # device order: offset before spread


def test_index_maths_matches_oracle(golden, orc):
    for shape, strides, imap, spread, offset, _ in golden["ndconfiguration_spec"]["rows"]:
        ndc = NDConfiguration.of(shape, strides, imap, spread, offset)
        phys = physical_indices(ndc)
        for i in range(ndc.size):
            assert ndc.indexOfIndex(i) == orc.index_of_index(ndc.asInlineArray(), i) == phys[i]


def test_construct_rejects_what_the_reference_rejects():
    with pytest.raises(IllegalStateException):
        NDConfiguration.of([2, 0], [1, 1], [1, 1], [1, 1], [0, 0])
    with pytest.raises(IllegalStateException):
        NDConfiguration.of([1, 3], [3, 1], [3, 1], [2, 1], [0, 0])     # step > 1 on an axis of extent 1


def test_layouts():
    assert Layout.ROW_MAJOR.newStridesFor([2, 3, 4]) == (12, 4, 1)
    assert Layout.COLUMN_MAJOR.newStridesFor([3, 4]) == (1, 3)
    # rank 3: only the two innermost axes trade places in the fill order (NDConfiguration.java:114-119)
    assert Layout.COLUMN_MAJOR.newStridesFor([2, 3, 4]) == (12, 1, 3)
    assert NDConfiguration.ofShape([3, 4]).getLayout() is Layout.ROW_MAJOR
    assert NDConfiguration.ofShape([3, 4], Layout.COLUMN_MAJOR).getLayout() is Layout.COLUMN_MAJOR
    assert NDConfiguration.ofShape([1, 1]).getLayout() is Layout.SYMMETRIC
    assert NDConfiguration.ofShape([3, 4]).isSimple()
    assert not NDConfiguration.ofShape([3, 4]).newReshaped([1, 0]).isSimple()
    assert Layout.SYMMETRIC.isCompatible(Layout.COLUMN_MAJOR) and not Layout.ROW_MAJOR.isCompatible(Layout.COLUMN_MAJOR)
    assert not Layout.UNSPECIFIC.isCompatible(Layout.UNSPECIFIC)


def test_views_of_the_benchmark_configs():
    """The descriptors the north-star configs name."""
    t = NDConfiguration.ofShape([16384, 4096]).newReshaped([1, 0])
    assert (t.shape, t.strides, t.indicesMap, t.spread, t.offset) == ((4096, 16384), (1, 4096), (16384, 1), (1, 1), (0, 0))
    assert t.kind() == "Permuted2DConfiguration" and t.getLayout() is Layout.COLUMN_MAJOR   # a transposed RM matrix IS a CM matrix (NDConfiguration.java:157-173)
    s = NDConfiguration.ofShape([8192, 16384]).sliced([4096, 8192], [0, 1], [2, 1])
    assert (s.shape, s.strides, s.indicesMap, s.spread, s.offset) == ((4096, 8192), (16384, 1), (8192, 1), (2, 1), (0, 1))
    assert s.kind() == "Sliced2DConfiguration"
    v = NDConfiguration.virtualOf([3, 4])
    assert v.asInlineArray().tolist() == [3, 4] + [0] * 8 and v.indexOfIndex(7) == 0


def test_views_against_numpy():
    base = np.arange(6 * 5 * 4, dtype=np.float32)
    t = Tensor.of(np.float32, [6, 5, 4], base)
    assert (t.T().items == base.reshape(6, 5, 4).transpose(2, 1, 0).reshape(-1)).all()
    assert (t.permute(1, 0, 2).items == base.reshape(6, 5, 4).transpose(1, 0, 2).reshape(-1)).all()
    sl = t[1:6:2, 2:5, 3]
    assert sl.shape == (3, 3, 1)
    assert (sl.items == base.reshape(6, 5, 4)[1:6:2, 2:5, 3:4].reshape(-1)).all()
    # slice of a transposed view: the offsets and steps travel with their axes (SimpleReshapeView)
    st = t[1:3, 0:5, 0:4].T()
    assert (st.items == base.reshape(6, 5, 4)[1:3].transpose(2, 1, 0).reshape(-1)).all()
    with pytest.raises(IllegalArgumentException):
        t[0:0, 0:5, 0:4]


def test_slice_then_transpose_matches_reference_string():
    """Tensor_Slice_Permute_Spec: A = [6,8] range, A[1..3, 4..5].T() starts at physical offsets 12, 20, 28, 13."""
    a = Tensor.of(np.float64, [6, 8], np.arange(48))
    v = a[1:4, 4:6].T()
    assert physical_indices(v.ndc).tolist()[:4] == [12, 20, 28, 13]


def test_view_chains_give_the_items_the_reference_prints():
    """tests/golden/reference_views.json: slices, transposed slices and padded reshapes of Tensor_Slice_Permute_Spec and
    Tensor_Slicing_Spec; the descriptors this package builds must address exactly the items those specifications print."""
    import json
    from helpers import apply_view_chain, view_row_parent
    rows = json.load(open(os.path.join(ROOT, "tests", "golden", "reference_views.json")))["rows"]
    assert len(rows) >= 12
    for row in rows:
        parent = view_row_parent(row)
        v = apply_view_chain(Tensor.of(parent.dtype, row["shape"], parent), row["chain"])
        assert list(v.shape) == row["want_shape"], row["name"]
        assert v.items.tolist() == row["want"], row["name"]


def test_parser_and_fused_lowering():
    f = Function.of("tanh(sig(I[0])*I[1]+I[2])")
    assert repr(f.root) == "tanh(((sig(I[0]) multiply I[1]) add I[2]))"
    assert f.numberOfArgs() == 3 and not f.isFlat()
    assert Function.of("I[0] x I[1]").root.value == "mul_conv"
    assert Function.of("i0 @ i1").root.value == "matMul"
    assert repr(Function.of("gaus(i0)*100 % i0").root) == "((gaus(I[0]) multiply 100.0) modulo I[0])"
    assert repr(Function.of("i0+i1*i2").root) == "(I[0] add (I[1] multiply I[2]))"
    opt = OptimizedFunction(None, f, "chain")
    L, Cn, Fn, B = _lib.FUSE_LOAD, _lib.FUSE_CONST, _lib.FUSE_FUN, _lib.FUSE_BIN
    assert opt.program == [L, 0, Fn, _lib.FUN["sig"], L, 1, B, _lib.OP["multiply"], L, 2, B, _lib.OP["add"], Fn, _lib.FUN["tanh"]]
    with pytest.raises(IllegalArgumentException):
        Function.of("nope(i0)")
    with pytest.raises(IllegalArgumentException):
        OptimizedFunction(None, Function.of("i0 x i1"), "conv")


def test_expressions_beyond_one_launch_are_cut_into_stages():
    """plan_fused: more than 6 sources, 32 op-codes, 8 stack entries, 8 constants or 4 waiting results per launch make several stages
    through temporaries; each stage respects the limits, and interpreting the stages gives the tree's own value
    (float32 after every operation, as the kernels round)."""
    from neureka_amd.function import FUSE_MAX_CONST, FUSE_MAX_OPS, FUSE_MAX_SAVED, FUSE_MAX_SRC, FUSE_MAX_STACK, plan_fused
    rng = np.random.default_rng(8)
    f32 = np.float32
    inv_fun = {v: k for k, v in _lib.FUN.items()}; inv_op = {v: k for k, v in _lib.OP.items()}
    np_fun = {"relu": lambda x: np.where(x >= 0, x, x * f32(0.01)), "quad": lambda x: x * x, "abs": np.abs, "idy": lambda x: x}
    np_op = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply}

    def tree_value(n, xs):
        if n.kind == "input": return xs[n.value]
        if n.kind == "const": return np.full_like(xs[0], n.value)
        if n.kind == "fun": return np_fun[n.value](tree_value(n.children[0], xs)).astype(f32)
        return np_op[n.value](tree_value(n.children[0], xs), tree_value(n.children[1], xs)).astype(f32)

    def run_stages(stages, xs):
        temps = {}
        for k, (program, consts, leaves) in enumerate(stages):
            ops = len(program) // 2
            assert ops <= FUSE_MAX_OPS and len(leaves) <= FUSE_MAX_SRC and len(consts) <= FUSE_MAX_CONST
            srcs = [xs[v] if kind == "input" else temps[v] for kind, v in leaves]
            stack, computed, deepest, waiting = [], [], 0, 0
            for code, arg in zip(program[0::2], program[1::2]):
                if code == _lib.FUSE_LOAD: stack.append(srcs[arg]); computed.append(False)
                elif code == _lib.FUSE_CONST: stack.append(np.full_like(xs[0], consts[arg])); computed.append(False)
                elif code == _lib.FUSE_FUN:
                    stack.append(np_fun[inv_fun[arg]](stack.pop()).astype(f32)); computed[-1] = True
                else:
                    b = stack.pop(); a = stack.pop()
                    stack.append(np_op[inv_op[arg]](a, b).astype(f32))
                    computed.pop(); computed[-1] = True
                deepest = max(deepest, len(stack))
                if computed[-1]:                         # results under a fresh result wait in the kernel's save slots
                    waiting = max(waiting, sum(computed[:-1]))
            assert len(stack) == 1 and deepest <= FUSE_MAX_STACK and waiting <= FUSE_MAX_SAVED, (deepest, waiting)
            temps[k] = stack[0]
        return temps[len(stages) - 1]

    small = Function.of("tanh(sig(I[0])*I[1]+I[2])")
    assert len(plan_fused(small.root)) == 1
    cases = ["relu(i0*i1+i2)*quad(i3-i4)+abs(i5*i6)-i7*i8+i9",                                   # ten sources
             "+".join(f"quad(i{k % 3}*{k + 1}.5-i{(k + 1) % 3})" for k in range(14)),                # 14 constants, ~100 op-codes
             "i0" + "".join(f"{'+-'[k % 2]}(i1*{k}.25)" for k in range(40)),                           # a long chain
             "(" * 12 + "i0" + "".join(f"+i{1 + k % 2})*i{k % 3}" for k in range(12)),               # nested to the left
             "+".join(f"(i{k % 3}*i{(k + 1) % 3}" for k in range(12)) + ")" * 12,                    # nested to the right: a deep stack
             "i0*i1+(i1*i2+(i2*i3+(i3*i4+(i4*i5+(i5*i0+i0*i2)))))"]                                  # 27 op-codes, 8 deep, six results wait
    for expr in cases:
        fn = Function.of(expr)
        stages = plan_fused(fn.root)
        assert len(stages) > 1, expr
        xs = [rng.uniform(-2, 2, 64).astype(f32) for _ in range(fn.numberOfArgs())]
        assert run_stages(stages, xs).tobytes() == tree_value(fn.root, xs).tobytes(), expr
    opt = OptimizedFunction(None, Function.of(cases[0]), "big")
    assert opt.program == [] and len(opt.stages) > 1                                            # no single-launch form


def test_no_host_arithmetic_path():
    a = Tensor.of(np.float32, [2, 2], [1, 2, 3, 4])
    with pytest.raises(IllegalStateException):
        a + a


def test_symbolic_derivative_of_fused_expressions():
    """derivative_of builds d f / d I[i] with 0 and 1 folded away; checked against central differences in
    float64 with a small evaluator of the same trees."""
    import math
    from neureka_amd.function import Function, derivative_of

    funs = {"tanh": math.tanh, "sig": lambda x: 1 / (1 + math.exp(-x)), "sin": math.sin, "cos": math.cos, "exp": math.exp,
            "ln": math.log, "quad": lambda x: x * x, "sqrt": math.sqrt}
    dfuns = {"tanh": lambda x: 1 - math.tanh(x) ** 2, "sig": lambda x: (1 / (1 + math.exp(-x))) * (1 - 1 / (1 + math.exp(-x))),
             "sin": math.cos, "cos": lambda x: -math.sin(x), "exp": math.exp, "ln": lambda x: 1 / x, "quad": lambda x: 2 * x,
             "sqrt": lambda x: 0.5 / math.sqrt(x)}
    ops = {"add": lambda a, b: a + b, "subtract": lambda a, b: a - b, "multiply": lambda a, b: a * b, "divide": lambda a, b: a / b,
           "power": lambda a, b: a ** b}

    def ev(n, x):
        if n.kind == "input": return x[n.value]
        if n.kind == "const": return n.value
        if n.kind == "fun": return funs[n.value](ev(n.children[0], x))
        if n.kind == "dfun": return dfuns[n.value](ev(n.children[0], x))
        return ops[n.value](ev(n.children[0], x), ev(n.children[1], x))

    x = [0.7, 1.3, 0.4]
    for expr in ("tanh(sig(I[0])*I[1]+I[2])", "I[0]*I[0]*I[1]", "sin(I[0])/cos(I[1])", "(I[0]+2)**I[1]", "exp(I[0]-I[2])*3", "quad(I[1])-ln(I[0])",
                 "sqrt(I[0]*I[1])/I[2]"):
        root = Function.of(expr).root
        for i in range(3):
            d = derivative_of(root, i)
            h = 1e-6
            xp, xm = list(x), list(x)
            xp[i] += h; xm[i] -= h
            numeric = (ev(root, xp) - ev(root, xm)) / (2 * h)
            assert abs(ev(d, x) - numeric) <= 1e-6 * max(1.0, abs(numeric)), (expr, i)
    # folding: the derivative with respect to an absent input is the constant 0, of I[0]+I[1] the constant 1
    assert repr(derivative_of(Function.of("sig(I[0])*I[1]").root, 2)) == "0.0"
    assert repr(derivative_of(Function.of("I[0]+I[1]").root, 1)) == "1.0"


def test_every_registration_row_of_the_opencl_backend_has_a_hip_counterpart():
    """CLBackend.java:200-325 as data (tests/golden/clbackend_registration_rows.json): every (operation, algorithm) row
    must resolve to an implementation for HipDevice, and ScalarBroadcast must carry one on every activation."""
    import json
    import importlib
    B = importlib.import_module("neureka_amd.backend")
    from neureka_amd.device import HipDevice
    rows = json.load(open(os.path.join(ROOT, "tests", "golden", "clbackend_registration_rows.json")))
    ctx = B.BackendContext().set(B.HipBackend())           # registration touches no device
    probe = object.__new__(HipDevice)                      # an instance only for the class lookup
    for op_id, alg_name in rows["rows"]:
        alg = ctx.getOperation(op_id).getAlgorithm(getattr(B, alg_name))
        assert alg is not None, (op_id, alg_name)
        assert alg.getImplementationFor(probe) is not None, f"no HipDevice implementation for {op_id} x {alg_name}"
    for f in B.ACTIVATIONS:
        alg = ctx.getOperation(f).getAlgorithm(B.ScalarBroadcast)
        assert alg is not None and alg.getImplementationFor(probe) is not None, f
    # every row must hit an existing (operation, algorithm) pair, as BackendContext.set demands (BackendContext.java:309-318)
    with pytest.raises(IllegalStateException):
        B._Registry(ctx, HipDevice).forOperation("add").set(B.NDConvolution, lambda call: None)
    with pytest.raises(IllegalStateException):
        B.hip_randomization(None)


def test_integration_text_binds_every_export_and_every_registration_row():
    """The Java binding text a maintainer copies must declare a MethodHandle for every export of the header and name
    every operation class the OpenCL backend registers."""
    header = open(os.path.join(ROOT, "include", "neureka_hip.h")).read()
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    declared = sorted(set(re.findall(r"\b(nk_[a-z0-9_]+)\s*\(", header)))
    bound = set(re.findall(r'MethodHandle\s+(nk_[a-z0-9_]+)\s*=\s*h\("(nk_[a-z0-9_]+)"', text))
    assert all(a == b for a, b in bound)
    missing = [n for n in declared if n not in {a for a, _ in bound}]
    assert not missing, f"exports without a MethodHandle in the binding text: {missing}"
    for cls in ("Addition", "Subtraction", "Multiplication", "Division", "Modulo", "Power", "AssignLeft", "Convolution", "XConvLeft",
                "XConvRight", "MatMul", "DotProduct", "Sum", "Randomization", "Absolute", "Cosinus", "GaSU", "GaTU", "Gaussian",
                "GaussianFast", "GeLU", "Identity", "Logarithm", "Quadratic", "ReLU", "SeLU", "Sigmoid", "SiLU", "Sinus", "Softplus",
                "Softsign", "Tanh", "TanhFast", "Exp", "Cbrt", "Log10", "Sqrt"):
        assert re.search(rf"\b{cls}\.class", text), f"{cls} is not registered in the binding text"
    for method in ("_readAll", "_readItem", "_readArray", "_writeItem", "_writeArray", "_swap", "_sizeOccupiedBy", "_actualize",
                   "_virtualize", "_dataTypeOf", "allocateFromOne", "allocateFromAll", "optimizedOperationOf", "dispose"):
        assert re.search(rf"\b{method}\(", text), f"HipDevice.{method} is missing from the binding text"
    # the Java sources exist as files, and the document prints them as they are
    blocks = dict(re.findall(r"`(java/[A-Za-z/]+\.java)`\n\n```java\n(.*?)\n```", text, re.S))
    files = []
    for folder, _, names in os.walk(os.path.join(ROOT, "java")):
        files += [os.path.relpath(os.path.join(folder, n), ROOT) for n in names if n.endswith(".java")]
    assert sorted(files) == sorted(blocks) and len(files) == 5, (sorted(files), sorted(blocks))
    for path in files:
        assert open(os.path.join(ROOT, path)).read().rstrip("\n") == blocks[path], f"{path} differs from its block in INTEGRATION.md"
    compiler = open(os.path.join(ROOT, "java", "neureka", "devices", "hip", "HipFunctionCompiler.java")).read()
    for piece in ("static Node treeOf(", "static Node derivativeOf(", "static List<Stage> plan(", "private static Stage lower(", "public Operation optimize()",
                  "setImplementationFor( HipDevice.class"):
        assert piece in compiler, piece
    # the limits and op-codes of the Java planner are the header's
    for name, value in re.findall(r"#define (NK_FUSE_MAX_[A-Z]+) (\d+)", header):
        assert re.search(rf"\b{name[len('NK_FUSE_'):]} = {value}\b", compiler), name


def test_assignment_parses_and_nests_to_the_right():
    assert repr(Function.of("I[0]<-I[1]").root) == "(I[0] left_inline I[1])"           # Function_Parsing_Spec.groovy:67
    assert repr(Function.of("I[0] <- (I[0] * -3)").root) == "(I[0] left_inline (I[0] multiply (-1.0 multiply 3.0)))"
    assert repr(Function.of("I[2]<-I[0]<-I[1]").root) == "(I[2] left_inline (I[0] left_inline I[1]))"
    assert repr(Function.of("I[0] <- I[1] + I[2]").root) == "(I[0] left_inline (I[1] add I[2]))"


def test_the_counted_traffic_record_belongs_to_the_sources_in_the_tree():
    """bench.py reports `roofline.traffic` from profiles/rows_binary_lean_kernel_broadcast_c2.json only while the digest
    in that record is the digest of the headline kernel's sources: a change to those sources without a new counter run
    fails here, not silently in the driver's bench line."""
    import json
    import os
    from neureka_amd.profile_summary import HEADLINE_PATH, kernel_sources_digest
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "profiles", "rows_binary_lean_kernel_broadcast_c2.json")) as f:
        rec = json.load(f)
    assert rec["path"] == HEADLINE_PATH
    assert rec["sources_sha256"] == kernel_sources_digest(), "the headline kernel's sources changed: regenerate profiles/ (neureka_amd/profile_summary.py)"
    algorithmic = 4 * (1024 * 2048 * 512 + 1024 * 512 + 2048 * 512)
    assert algorithmic <= rec["traffic_bytes"] <= 1.05 * algorithmic
    import bench
    traffic, note = bench.counted_traffic(HEADLINE_PATH)
    assert traffic == rec["traffic_bytes"] and "FETCH_SIZE" in note
    assert bench.counted_traffic("some_other_plan")[0] is None


def test_java_binding_is_consistent_with_the_header_as_far_as_text_can_tell():
    """No JDK exists here, so the Java files cannot be compiled; what text allows is checked: every `Nk.` member the other
    classes use is declared in Nk.java, every MethodHandle there has the argument count and kinds (int / long / double /
    address) of the ctypes binding of the same symbol, and brackets balance in every file outside strings and comments."""
    import ctypes as C
    import os
    import re
    from neureka_amd import _lib
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "java")
    files = {}
    for folder, _, names in os.walk(root):
        for name in names:
            if name.endswith(".java"):
                with open(os.path.join(folder, name)) as f:
                    files[name] = f.read()
    assert {"Nk.java", "HipDevice.java", "HipBackend.java", "Hip.java", "HipFunctionCompiler.java"} <= set(files)
    nk = files["Nk.java"]
    handles = dict(re.findall(r'MethodHandle\s+(nk_\w+)\s*=\s*h\("nk_\w+",\s*([^;]*?)\);', nk))
    assert set(handles) == set(_lib.SYMBOLS), sorted(set(handles) ^ set(_lib.SYMBOLS))
    kind = {C.c_int: "I", C.c_uint64: "J", C.c_int64: "J", C.c_size_t: "J", C.c_double: "D", C.c_float: "F"}
    for name, layouts in handles.items():
        res, *args = [a.strip() for a in layouts.split(",")]
        restype, argtypes = _lib.SYMBOLS[name]
        want = [kind.get(t, "P") for t in argtypes]              # every pointer type (void*, T*, char*) is an address
        assert args == want, (name, args, want)
        assert res == ("P" if restype is C.c_char_p else "I"), (name, res)
    members = set(handles) | set(re.findall(r"static\s+[\w<>\[\]?]+\s+(\w+)\s*\(", nk))
    for name, text in files.items():
        for used in re.findall(r"\bNk\.(\w+)", text):
            assert used in members, f"{name} uses Nk.{used}, which Nk.java does not declare"
        stripped = re.sub(r'"(?:\\.|[^"\\])*"|\'(?:\\.|[^\'\\])\'|//[^\n]*|/\*.*?\*/', "", text, flags=re.S)
        for open_, close in ("{}", "()", "[]"):
            assert stripped.count(open_) == stripped.count(close), f"{name}: unbalanced {open_}{close}"
