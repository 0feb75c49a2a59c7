"""The rows of the OpenCL backend's registration table that are thin wrappers over kernels tested elsewhere --
AssignLeft (scalar and tensor assignment into views), ScalarAlgorithm (a function of a virtual tensor),
ScalarBroadcast (f(value) written through a view) -- driven through the operations and compared with the oracle's
CPUElementwiseAssignFun / CPUScalarBroadcastIdentity / CPUScalarBroadcastFunction restatements; plus the ownership
rules of the device (tensors held weakly, buffers released when the last tensor that shares them is dropped)."""
import gc
import importlib

import numpy as np
import pytest

from helpers import assert_bits, assert_close
from neureka_amd import Function, IllegalArgumentException, IllegalStateException, Tensor, _lib

pytestmark = pytest.mark.gpu
B = importlib.import_module("neureka_amd.backend")
F = {"f32": np.float32, "f64": np.float64}


def say(*a):
    print("[case]", *a, flush=True)


def on(device, array):
    array = np.asarray(array)
    return Tensor.of(array.dtype, array.shape, array.reshape(-1)).to(device)


def cfg(t):
    return t.ndc.asInlineArray()


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_assign_a_tensor_and_a_scalar_into_a_sliced_view(device, orc, dt):
    rng = np.random.default_rng(81)
    base = rng.uniform(-1, 1, (12, 20)).astype(F[dt])
    src = rng.uniform(-1, 1, (5, 9)).astype(F[dt])
    say("assign tensor into view", dt)
    t = on(device, base)
    view = t[1:11:2, 2:11]
    s = on(device, src)
    got = view.assign(s)
    assert got is view and _lib.last_path() != ""
    want = base.reshape(-1).copy()
    orc.activation("idy", -1, want, cfg(view), src.reshape(-1), cfg(s))          # CPUElementwiseAssignFun = identity through both views
    assert_bits(t.getData(), want, "tensor assignment")
    assert np.count_nonzero(want != base.reshape(-1)) == 45
    # a transposed source view, through the expression "I[0] <- I[1]"
    say("assign transposed view through the parser", dt)
    src2 = rng.uniform(-1, 1, (9, 5)).astype(F[dt])
    s2 = on(device, src2).T()
    Function.of("I[0] <- I[1]")(view, s2)
    want2 = want.copy()
    orc.activation("idy", -1, want2, cfg(view), src2.reshape(-1), cfg(s2))
    assert_bits(t.getData(), want2, "assignment of a transposed view")
    # a scalar: the BiScalarBroadcast of AssignLeft (CPUScalarBroadcastIdentity writes the value to the drain's view)
    say("assign scalar into view", dt)
    algorithm = B.backend().getOperation("left_inline").getAlgorithmFor(
        B.ExecutionCall(device, B.backend().getOperation("left_inline"), [view, Tensor.of(F[dt], view.shape, -0.0)]))
    assert isinstance(algorithm, B.AssignScalar)
    view.assign(-0.0)
    want3 = want2.copy()
    orc.scalarization("idy", -1, want3, cfg(view), want3.copy(), cfg(view), -0.0)
    assert_bits(t.getData(), want3, "scalar assignment")
    assert np.signbit(t.getData()[1 * 20 + 2])                                  # the -0.0 arrived as -0.0
    # a virtual drain becomes actual before it is written (AssignLeft.java:61)
    v = Tensor.of(F[dt], (3, 4), 7.0).to(device)
    v.assign(2.5)
    assert not v.isVirtual() and (v.items == 2.5).all()
    with pytest.raises(IllegalArgumentException):
        from neureka_amd.function import execute
        execute("left_inline", [view, s], d=0)                                   # "Assignment does not support autograd!"
    with pytest.raises(IllegalArgumentException):
        view.assign(on(device, np.zeros((2, 2), dtype=F[dt])))


def test_assign_integers(device, orc):
    say("assign int scalar")
    base = np.arange(40, dtype=np.int32).reshape(5, 8)
    t = on(device, base)
    view = t[1:4, ::3]
    view.assign(-9)
    want = base.reshape(-1).copy()
    want = orc.scalarization_int("idy", -1, want, cfg(view), want.copy(), cfg(view), -9)
    assert (t.getData() == want).all() and (want == -9).sum() == 9


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_function_of_a_virtual_tensor_stays_virtual(device, orc, dt):
    """ScalarAlgorithm + CLScalarFunction: f(item 0) written to item 0 of a virtual result, forward and derivative."""
    x = F[dt](0.625)
    for name in B.ACTIVATIONS:
        say("scalar activation", name, dt)
        t = Tensor.of(F[dt], (3, 5), float(x)).to(device)
        op = B.backend().getOperation(name)
        call = B.ExecutionCall(device, op, [t])
        assert isinstance(op.getAlgorithmFor(call), B.ScalarAlgorithm)
        for d in (-1, 0):
            from neureka_amd.function import execute
            r = execute(name, [t], d=d, record=False)
            assert r.isVirtual() and r.shape == (3, 5) and r._data.size == 1
            want = orc.fun(name, np.array([x], dtype=F[dt]), derive=d >= 0)
            assert_close(r.getData(), want, f"{name} d={d}")
            assert (r.items == r.getData()[0]).all()
    # autograd through a virtual operand
    t = Tensor.of(np.float32, (2, 2), 0.5).to(device).setRqsGradient(True)
    y = t.tanh()
    y.backward(Tensor.of(np.float32, (2, 2), 2.0))
    want = 2.0 * (1 - np.tanh(0.5) ** 2)
    assert np.allclose(t.gradient.items, want, rtol=1e-5)


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_scalar_broadcast_writes_f_of_the_value_through_the_drain_view(device, orc, dt):
    """ScalarBroadcast: a full drain (here a strided view) and a virtual source of the same shape."""
    say("scalar broadcast", dt)
    base = np.zeros((6, 8), dtype=F[dt])
    t = on(device, base)
    view = t[1:6:2, 2:7]
    src = Tensor.of(F[dt], view.shape, 0.3).to(device)
    for name, d in (("tanh", -1), ("sig", 0), ("quad", -1), ("relu", 0)):
        op = B.backend().getOperation(name)
        call = B.ExecutionCall(device, op, [view, src], d)
        call.algorithm = op.getAlgorithmFor(call)
        assert isinstance(call.algorithm, B.ScalarBroadcast), name
        out = B.execute_device_algorithm(call.algorithm.prepare(call))
        assert out is view
        value = orc.fun(name, np.array([0.3], dtype=F[dt]), derive=d >= 0)[0]
        want = np.zeros(48, dtype=F[dt])
        orc.scalar_fill(want, cfg(view), float(value))
        got = t.getData()
        assert_close(got, want, f"{name} d={d}")
        assert (got != 0).sum() == (15 if value != 0 else 0)
    # without a drain the algorithm allocates a full output of the source's shape
    op = B.backend().getOperation("exp")
    call = B.ExecutionCall(device, op, [src])
    out = B.execute_device_algorithm(op.getAlgorithm(B.ScalarBroadcast).prepare(replace_algorithm(call, op.getAlgorithm(B.ScalarBroadcast))))
    assert not out.isVirtual() and out.shape == view.shape
    assert_close(out.items, np.full(15, orc.fun("exp", np.array([0.3], dtype=F[dt]))[0], dtype=F[dt]), "exp fill")


def replace_algorithm(call, algorithm):
    call.algorithm = algorithm
    return call


def test_randomization_is_the_stub_it_is_in_the_reference(device):
    op = B.backend().getOperation("random")
    t = on(device, np.zeros(4, dtype=np.float32))
    call = B.ExecutionCall(device, op, [t, t], -1, op.algorithms[0])
    with pytest.raises(IllegalStateException, match="Not yet implemented"):
        B.execute_device_algorithm(call)


def test_dropped_results_release_their_buffers(device):
    """A training loop that drops its results must not grow the device: tensors are held weakly, a buffer goes when
    the last tensor that shares it is gone (the reference's DeviceCleaner on weak reachability)."""
    say("ownership")
    a = on(device, np.ones((64, 64), dtype=np.float32))
    b = on(device, np.ones((64, 64), dtype=np.float32))
    y = a + b; del y; gc.collect()
    stored, objects, live = device.numberOfStored(), device.numberOfDataObjects(), device.liveBuffers()
    for _ in range(100):
        y = a + b
        z = y.tanh()
        del y, z
    gc.collect()
    assert (device.numberOfStored(), device.numberOfDataObjects(), device.liveBuffers()) == (stored, objects, live)
    # a view keeps its root's buffer alive, and only as long as the view lives
    root = on(device, np.arange(12, dtype=np.float32).reshape(3, 4))
    view = root[1:3, 1:3]
    live_with_root = device.liveBuffers()
    del root; gc.collect()
    assert device.liveBuffers() == live_with_root and view.items.tolist() == [5, 6, 9, 10]
    del view; gc.collect()
    assert device.liveBuffers() == live_with_root - 1
    # autograd temporaries (zeros like the operands of the reducing backward) go with the graph
    p = on(device, np.ones((8, 1, 4), dtype=np.float32)).setRqsGradient(True)
    q = on(device, np.ones((1, 6, 4), dtype=np.float32)).setRqsGradient(True)
    (p + q).backward(); gc.collect()
    base = device.liveBuffers()
    for _ in range(20):
        p.gradient = q.gradient = None
        (p + q).backward()
    gc.collect()
    assert device.liveBuffers() == base
    assert device.has(a) and not device.has(Tensor.of(np.float32, (1,), 0.0))


def test_calls_from_several_host_threads_are_serialised(device, orc):
    """Four host threads call the C ABI on one device handle at once -- allocation and release, whole-tensor sums whose
    partial results share the device's grow-on-demand workspace, matrix products whose parts do, elementwise launches.
    The library serialises the calls of a handle, so every result is the single-threaded one and the registry of
    allocations ends where it began."""
    import ctypes as C
    import threading
    say("threads")
    lib, h = device._lib, device.handle
    rng = np.random.default_rng(90)
    live_before = device.liveBuffers()
    errors = []

    def worker(seed):
        try:
            r = np.random.default_rng(seed)
            for it in range(12):
                n = int(r.integers(40000, 3000000))
                x = r.integers(-8, 9, n).astype(np.float32)            # integer-valued: every summation order is exact
                buf, out = C.c_uint64(), C.c_uint64()
                _lib.check(lib.nk_alloc(h, 4 * n, C.byref(buf))); _lib.check(lib.nk_alloc(h, 4, C.byref(out)))
                _lib.check(lib.nk_h2d(h, buf, 0, x.ctypes.data_as(C.c_void_p), 4 * n))
                _lib.check(lib.nk_sum(h, 0, buf, n, out))
                got = np.zeros(1, dtype=np.float32)
                _lib.check(lib.nk_d2h(h, got.ctypes.data_as(C.c_void_p), out, 0, 4))
                assert got[0] == np.float32(x.astype(np.float64).sum()), (seed, it, n)
                M, K, N = 128, int(r.choice([2048, 4096, 8192])), 128      # few tiles, long inner dimension: parts in the workspace
                a = r.integers(-2, 3, (M, K)).astype(np.float32); b = r.integers(-2, 3, (K, N)).astype(np.float32)
                pa, pb, pc = C.c_uint64(), C.c_uint64(), C.c_uint64()
                for ptr, arr in ((pa, a), (pb, b)):
                    _lib.check(lib.nk_alloc(h, arr.nbytes, C.byref(ptr)))
                    _lib.check(lib.nk_h2d(h, ptr, 0, arr.ctypes.data_as(C.c_void_p), arr.nbytes))
                _lib.check(lib.nk_alloc(h, 4 * M * N, C.byref(pc)))
                _lib.check(lib.nk_matmul_set(h, 0, _lib.ROW_MAJOR, M, K, N, pa, pb, pc))
                c = np.zeros((M, N), dtype=np.float32)
                _lib.check(lib.nk_d2h(h, c.ctypes.data_as(C.c_void_p), pc, 0, c.nbytes))
                assert (c == a.astype(np.float64) @ b.astype(np.float64)).all(), (seed, it, K)
                for ptr in (buf, out, pa, pb, pc): _lib.check(lib.nk_free(h, ptr))
        except BaseException as e:                                          # reported by the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(100 + i,)) for i in range(4)]
    for t in threads: t.start()
    for t in threads: t.join()
    assert not errors, errors[0]
    assert device.liveBuffers() == live_before


def test_fused_function_on_host_operands_keeps_autograd(device):
    """A fused function whose operands live on the host (stored for the call, restored afterwards) records its graph
    node like the unfused path does: same result, same gradients."""
    say("fused with guests")
    rng = np.random.default_rng(83)
    xs = [rng.standard_normal((6, 7)).astype(np.float32) for _ in range(3)]
    expr = "tanh(sig(I[0])*I[1]+I[2])"

    def run(fused: bool, guests: bool):
        ts = [Tensor.of(np.float32, x.shape, x).setRqsGradient(True) for x in xs]
        if not guests:
            for t in ts: t.to(device)
        f = Function.of(expr)
        y = device.optimizedFunctionOf(f, "chain")(*ts) if fused else f(*ts)
        y.backward(Tensor.of(np.float32, y.shape, 1.0))
        return y.items, [t.gradient.items for t in ts]

    y0, g0 = run(False, False)
    for fused, guests in ((True, False), (True, True)):
        y, g = run(fused, guests)
        assert np.allclose(y, y0, rtol=1e-5, atol=1e-7), (fused, guests)
        for a, b in zip(g, g0):
            assert np.allclose(a, b, rtol=2e-5, atol=1e-6), (fused, guests)
    # modulo has a fused derivative now: d (u % v) / d u = 1 (operator/Modulo.java:183-185)
    a = on(device, np.array([5.5, -3.25, 7.0], dtype=np.float32)).setRqsGradient(True)
    m = on(device, np.array([2.0, 2.0, 4.0], dtype=np.float32))
    out = device.optimizedFunctionOf(Function.of("(I[0] % I[1]) * 3"), "mod")(a, m)
    out.backward()
    assert out.items.tolist() == [4.5, -3.75, 9.0] and a.gradient.items.tolist() == [3.0, 3.0, 3.0]
