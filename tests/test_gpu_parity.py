"""Parity of the HIP path (through the C ABI of libneureka_hip.so) with the CPU oracle, on the same
seeded inputs.  Bit-exact for + - * and copies (and every kernel that keeps the reference's summation
order); rtol 1e-5 (f32) / 1e-12 (f64) for transcendental activations; norm-wise 1e-5 / 1e-12 for
re-ordered reductions.  Every test prints what it is about to run before touching the GPU."""
import ctypes as C
import gc

import numpy as np
import pytest

from helpers import ATOL, RTOL, assert_bits, assert_close, fill_it, java_array_hash
from neureka_amd import Function, HipError, IllegalArgumentException, IllegalStateException, Layout, NDConfiguration, Tensor, _lib
from neureka_amd.tensor import physical_indices

pytestmark = pytest.mark.gpu

F = {"f32": np.float32, "f64": np.float64}
ACTS = ["abs", "cos", "gasu", "gatu", "gaus", "fast_gaus", "gelu", "idy", "ln", "quad", "relu", "selu", "sig", "silu",
        "sin", "softplus", "softsign", "tanh", "fast_tanh", "exp", "log10", "sqrt", "cbrt"]
POSITIVE_ONLY = {"ln", "log10", "sqrt", "cbrt"}


def say(*a):
    print("[case]", *a, flush=True)


def on(device, array, shape=None):
    array = np.asarray(array)
    return Tensor.of(array.dtype, shape if shape is not None else array.shape, array.reshape(-1)).to(device)


def cfg(t):
    return t.ndc.asInlineArray()


# ---- device contract -----------------------------------------------------------------------------------
def test_memory_roundtrip_fill_and_accounting(device):
    say("memory roundtrip")
    before = device.liveBuffers()
    data = device.allocate(np.float32, 1000)
    host = np.arange(1000, dtype=np.float32)
    device._write(data, 0, host)
    assert (device._read_all(data) == host).all()
    device._write(data, 10, np.full(5, -1, dtype=np.float32))           # partial write (setItems at an offset)
    assert (device._read(data, 8, 9) == [8, 9, -1, -1, -1, -1, -1, 15, 16]).all()
    device._fill(data, 100, 50, 7.5)
    got = device._read_all(data)
    assert (got[100:150] == 7.5).all() and got[99] == 99 and got[150] == 150
    d64 = device.allocateFromOne(np.float64, 33, -0.0)
    assert np.signbit(device._read_all(d64)).all()
    assert device.liveBuffers() == before + 2
    ptr = data.ptr
    data.release(); d64.release()
    assert device.liveBuffers() == before
    with pytest.raises(HipError):                                      # double free is reported, not ignored
        _lib.check(device._lib.nk_free(device.handle, ptr))
    with pytest.raises(HipError):                                      # out-of-range transfer is refused on the host
        small = device.allocate(np.float32, 4)
        try:
            device._read(small, 2, 10)
        finally:
            small.release()


def test_large_fills_every_pattern_size(device):
    """Fills of a MiB and more go through 16-byte stores with the pattern repeated, the rest of the last 16 bytes
    through the element kernel; a start that is not on a 16-byte boundary keeps the element kernel.  Every element
    type's pattern, the elements before and after the filled range untouched."""
    say("large fills")
    for dt, value in ((np.int8, -7), (np.int16, -12345), (np.float32, -0.0), (np.float32, 3.25), (np.float64, -1e-300), (np.int64, -(2 ** 62) - 5)):
        n = (3 << 20) // np.dtype(dt).itemsize + 37
        for start, count in ((0, n), (16 // np.dtype(dt).itemsize, n - 2 * (16 // np.dtype(dt).itemsize) - 3), (1, n - 2)):
            data = device.allocate(dt, n)
            device._fill(data, 0, n, 1)
            device._fill(data, start, count, value)
            got = device._read_all(data)
            want = np.ones(n, dtype=dt); want[start:start + count] = value
            assert got.tobytes() == want.tobytes(), (np.dtype(dt).name, start, count)
            data.release()


def test_store_restore_free_virtual_and_slices(device):
    say("device contract")
    stored, objs = device.numberOfStored(), device.numberOfDataObjects()
    t = Tensor.of(np.float64, [3, 4], np.arange(12.0))
    assert not t.isOutsourced() and not device.has(t)
    t.to(device)
    assert t.isOutsourced() and device.has(t) and device.numberOfStored() == stored + 1
    assert (t.items == np.arange(12.0)).all()
    s = t[1:3, 1:4]                                                      # a slice shares the parent's buffer
    assert device.has(s) and s._data is t._data and device.numberOfDataObjects() == objs + 1
    assert (s.items == np.arange(12.0).reshape(3, 4)[1:3, 1:4].reshape(-1)).all()
    v = Tensor.of(np.float32, [1000, 1000], 4.0).to(device)              # virtual: one element on the device
    assert v.isVirtual() and v._data.size == 1 and (v.items[:3] == 4.0).all()
    v.setIsVirtual(False)
    assert v._data.size == 1000000 and (v.getData() == 4.0).all()
    device.restore(t)
    assert not t.isOutsourced() and (t.items == np.arange(12.0)).all()
    with pytest.raises(IllegalArgumentException):
        device.restore(t)                                                # OpenCLDevice.java:317-322
    orphan = Tensor.of(np.float32, [4], [1, 2, 3, 4])
    child = orphan[1:3]
    with pytest.raises(IllegalStateException, match="Data parent is not outsourced!"):
        device.store(child)                                              # AbstractDevice.java:96-97
    device.free(s); device.free(v)
    assert device.numberOfStored() == stored and device.numberOfDataObjects() == objs


def test_protected_device_contract(device):
    """_readItem/_readArray/_writeItem/_writeArray/_swap/_sizeOccupiedBy/update as AbstractDevice declares them
    (devices/AbstractDevice.java:188-206), partial reads and writes included (Cross_Device_IO_Spec)."""
    say("protected device contract")
    t = Tensor.of(np.float64, [3, 4], np.arange(12.0)).to(device)
    assert device._sizeOccupiedBy(t) == 12 and device._dataTypeOf(t._data) == np.float64
    assert device._readItem(t, 7) == 7.0 and device._readArray(t, 4, 3).tolist() == [4.0, 5.0, 6.0]
    device._writeItem(t, -1.5, 2, 3)                       # one value over three positions
    device._writeArray(t, [100.0, 200.0, 300.0, 400.0], 1, 9, 2)      # array[1:3] -> positions 9, 10
    assert device._readAll(t).tolist() == [0, 1, -1.5, -1.5, -1.5, 5, 6, 7, 8, 200, 300, 11]
    other = Tensor(np.float64, NDConfiguration.ofShape((12,)), None)
    device._swap(t, other)
    assert other.isOutsourced() and other.items.tolist() == device._readAll(t).tolist()
    host = Tensor.of(np.float32, [4], [1, 2, 3, 4])
    assert device.update(host, True) and host.isOutsourced()
    assert device.update(host, False) and not host.isOutsourced() and host.items.tolist() == [1, 2, 3, 4]
    device.free(t)


def test_bad_arguments_are_reported(device):
    say("argument errors")
    a = on(device, np.ones(8, dtype=np.float32))
    out = on(device, np.zeros(8, dtype=np.float32))
    lib, h = device._lib, device.handle
    c8 = cfg(a)
    big = NDConfiguration.ofShape([16]).asInlineArray()
    with pytest.raises(HipError, match="exceeds the buffer"):           # a view larger than its buffer never reaches the GPU
        _lib.check(lib.nk_activation(h, 0, -1, 0, 1, out._data.ptr, _lib.cfg_ptr(big), a._data.ptr, _lib.cfg_ptr(big), 16))
    with pytest.raises(HipError, match="n = 5"):
        _lib.check(lib.nk_activation(h, 0, -1, 0, 1, out._data.ptr, _lib.cfg_ptr(c8), a._data.ptr, _lib.cfg_ptr(c8), 5))
    with pytest.raises(HipError, match="unknown function id"):
        _lib.check(lib.nk_activation(h, 99, -1, 0, 1, out._data.ptr, _lib.cfg_ptr(c8), a._data.ptr, _lib.cfg_ptr(c8), 8))
    with pytest.raises(HipError, match="rank"):
        _lib.check(lib.nk_activation(h, 0, -1, 0, 9, out._data.ptr, _lib.cfg_ptr(c8), a._data.ptr, _lib.cfg_ptr(c8), 8))
    with pytest.raises(HipError, match="unknown device handle"):
        _lib.check(lib.nk_device_sync(987654))


# ---- elementwise family --------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("n", [1, 5, 7907, 1 << 16])
def test_binary_elementwise_bit_exact(device, orc, dt, n):
    say("elementwise", dt, n)
    rng = np.random.default_rng(n)
    a = rng.uniform(-1, 1, n).astype(F[dt]); b = rng.uniform(-1, 1, n).astype(F[dt])
    ta, tb = on(device, a), on(device, b)
    c = orc.dense_cfg([n])
    for op in ("add", "subtract", "multiply", "divide", "modulo"):
        for d in (-1, 0, 1):
            out = on(device, np.zeros(n, dtype=F[dt]))
            device.launch_elementwise(op, d, out, ta, tb)
            want = orc.elementwise(op, d, np.zeros(n, dtype=F[dt]), c, a, c, b, c)
            if op in ("add", "subtract", "multiply") or d < 0 or (d == 0):
                assert_bits(out.getData(), want, f"{op} d={d}")
            else:
                assert_close(out.getData(), want, f"{op} d={d}")
    out = on(device, np.zeros(n, dtype=F[dt]))
    ap = np.abs(a) + 0.5
    device.launch_elementwise("power", -1, out, on(device, ap), tb)
    assert_close(out.getData(), orc.elementwise("power", -1, np.zeros(n, dtype=F[dt]), c, ap, c, b, c), "power")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_all_activations_and_derivatives(device, orc, dt):
    n = 7907
    x = orc.seeded(F[dt], n, "Tempeh")
    c = orc.dense_cfg([n])
    for name in ACTS:
        xi = (np.abs(x) + F[dt](0.01)).astype(F[dt]) if name in POSITIVE_ONLY else x
        tx = on(device, xi)
        for d in (-1, 0):
            say("activation", name, d, dt)
            out = on(device, np.zeros(n, dtype=F[dt]))
            device.launch_activation(name, d, out, tx)
            want = orc.activation(name, d, np.zeros(n, dtype=F[dt]), c, xi, c)
            got = out.getData()
            if dt == "f32" and name in ("abs", "idy", "quad", "relu", "fast_gaus", "softsign", "gasu", "fast_tanh") and (d < 0 or name != "fast_tanh"):
                assert_bits(got, want, f"{name} d={d}")     # pure float arithmetic in the reference: identical
            else:
                assert_close(got, want, f"{name} d={d}")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_binary_operators_on_special_values(device, orc, dt):
    """Every pair from a set of special values through + - * / % ** and their partial derivatives."""
    T = F[dt]
    vals = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -2.5, 3.0, np.inf, -np.inf, np.nan, 1e30, -1e-30], dtype=T)
    a = np.repeat(vals, vals.size); b = np.tile(vals, vals.size)
    c = orc.dense_cfg([a.size])
    ta, tb = on(device, a), on(device, b)
    for op in ("add", "subtract", "multiply", "divide", "modulo", "power"):
        for d in (-1, 0, 1):
            say("operator specials", op, d, dt)
            out = on(device, np.zeros(a.size, dtype=T))
            device.launch_elementwise(op, d, out, ta, tb)
            with np.errstate(all="ignore"):
                want = orc.elementwise(op, d, np.zeros(a.size, dtype=T), c, a, c, b, c)
            if op in ("add", "subtract", "multiply", "divide", "modulo") and d < 0:
                assert_bits(out.getData(), want, f"{op}")
            else:
                assert_close(out.getData(), want, f"{op} d={d}")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_activations_on_special_values(device, orc, dt):
    """Zeros of both signs, infinities, NaN, huge, tiny and subnormal arguments: NaN where the CPU device gives NaN,
    the same infinity where it gives one, within tolerance elsewhere."""
    T = F[dt]
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 100.0, -100.0, 1e30, -1e30, 1e-30, -1e-30, 1e-40, 20.0, -20.0, 0.1249, 0.1251, -0.125, 88.0, -88.0,
                  709.0, -709.0], dtype=T)
    c = orc.dense_cfg([x.size])
    tx = on(device, x)
    for name in ACTS:
        for d in (-1, 0):
            say("activation specials", name, d, dt)
            out = on(device, np.zeros(x.size, dtype=T))
            device.launch_activation(name, d, out, tx)
            with np.errstate(all="ignore"):
                want = orc.activation(name, d, np.zeros(x.size, dtype=T), c, x, c)
                assert_close(out.getData(), want, f"{name} d={d} on {x.tolist()}")


def test_activation_golden_vectors_on_device(device, orc, golden):
    g = golden["activation_vectors"]
    for row in g["rows"]:
        say("golden activation", row["fun"], row["derive"], row["type"])
        dt = F[row["type"]]
        x = orc.seeded(dt, g["size"], g["seed"])
        fn = Function.of(f"{row['fun']}(I[0])")
        t = on(device, x)
        res = fn.derive([t], 0) if row["derive"] else fn(t)
        assert_close(res.items, np.array(row["expected"], dtype=dt), str(row))
        # the same through a slice of a larger tensor, as the reference test does (t2 = zeros(5)[1..3])
        big = on(device, np.zeros(5, dtype=dt))
        sl = big[1:4]
        sl.setItems(x)
        res2 = fn.derive([sl], 0) if row["derive"] else fn(sl)
        assert_close(res2.items, np.array(row["expected"], dtype=dt), str(row) + " (slice)")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_scalarization_and_fill(device, orc, dt):
    say("scalarization", dt)
    n = 4099
    rng = np.random.default_rng(4)
    a = rng.uniform(-2, 2, n).astype(F[dt])
    ta = on(device, a)
    c = orc.dense_cfg([n])
    for op, val in (("add", 0.1), ("subtract", 3.0), ("multiply", 100.0), ("divide", 3.0), ("modulo", 0.7), ("idy", -2.5)):
        out = on(device, np.zeros(n, dtype=F[dt]))
        device.launch_scalarization(op, -1, out, ta, val)
        assert_bits(out.getData(), orc.scalarization(op, -1, np.zeros(n, dtype=F[dt]), c, a, c, val), op)
    out = on(device, np.zeros(n, dtype=F[dt]))
    device.launch_scalarization("power", -1, out, on(device, np.abs(a) + 0.5), 2.5)
    assert_close(out.getData(), orc.scalarization("power", -1, np.zeros(n, dtype=F[dt]), c, np.abs(a) + F[dt](0.5), c, 2.5), "power")
    # fill through a strided view: only the viewed elements change
    base = on(device, np.zeros((6, 8), dtype=F[dt]))
    view = base[1:6:2, 2:7]
    device.launch_scalar_fill(view, 0.1)
    want = np.zeros(48, dtype=F[dt])
    orc.scalar_fill(want, cfg(view), 0.1)
    assert_bits(base.getData(), want, "fill view")
    assert np.count_nonzero(want) == 15


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_compiled_in_functions_and_operators_on_row_views(device, orc, dt):
    """One function, or one heavy operator, of a source runs in a kernel with it compiled in ("rows_vec_single",
    "rows_vec_pair") -- also on views whose rows are dense but lie apart (row slices, rows of a length that is no
    multiple of the vector) and into a drain that is such a view: every function and derivative, every heavy operator
    with a tensor and with a constant as its second operand, against the oracle on the same descriptors."""
    T = F[dt]
    rng = np.random.default_rng(77)
    parent = rng.uniform(0.05, 2.0, (37, 203)).astype(T)
    other = rng.uniform(0.05, 2.0, (37, 203)).astype(T)
    tp, to = on(device, parent), on(device, other)
    sl = np.s_[3:33, :]
    vp, vo = tp[sl], to[sl]
    hp, ho = np.ascontiguousarray(parent[sl]).reshape(-1), np.ascontiguousarray(other[sl]).reshape(-1)
    dense = orc.dense_cfg([30, 203])
    for name in ACTS:
        for d in (-1, 0):
            say("compiled-in function on a row view", name, d, dt)
            drain_parent = on(device, np.full((37, 203), -7.0, dtype=T))
            drain = drain_parent[sl]
            device.launch_activation(name, d, drain, vp)
            assert _lib.last_path() == "rows_vec_single", _lib.last_path()
            want = orc.activation(name, d, np.zeros(hp.size, dtype=T), dense, hp, dense)
            got = drain_parent.getData().reshape(37, 203)
            assert (got[:3] == -7.0).all() and (got[33:] == -7.0).all(), "rows outside the view changed"
            assert_close(got[sl].reshape(-1), want, f"{name} d={d}")
    for op, ds in (("modulo", (-1, 0, 1)), ("power", (-1, 0, 1)), ("divide", (0, 1))):
        for d in ds:
            say("compiled-in operator on row views", op, d, dt)
            out = Tensor._on_device(device, T, (30, 203))
            device.launch_elementwise(op, d, out, vp, vo)
            assert _lib.last_path() == "rows_vec_pair", _lib.last_path()
            want = orc.elementwise(op, d, np.zeros(hp.size, dtype=T), dense, hp, dense, ho, dense)
            (assert_bits if op == "modulo" and d < 0 else assert_close)(out.getData(), want, f"{op} d={d}")
            say("compiled-in operator with a constant", op, d, dt)
            device.launch_scalarization(op, d, out, vp, 1.75)
            assert _lib.last_path() == "rows_vec_pair", _lib.last_path()
            want = orc.scalarization(op, d, np.zeros(hp.size, dtype=T), dense, hp, dense, 1.75)
            (assert_bits if op == "modulo" and d < 0 else assert_close)(out.getData(), want, f"{op} d={d} with a constant")


VIEWS = {
    "permuted": lambda t: t.T(),
    "sliced": lambda t: t[::2, 1:t.shape[1] // 2 + 1],
    "sliced_rows": lambda t: t[1:t.shape[0] - 1, :],
    "perm3": None,
}


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_views_take_the_fast_paths_and_match(device, orc, dt):
    """Non-contiguous NDConfigurations: transposed, strided-slice and row-band views as sources, a dense
    drain; bit-exact against the oracle walking the same descriptors; the kernel path is asserted."""
    rng = np.random.default_rng(8)
    R, Cc = 70, 130
    base_a = rng.uniform(-1, 1, (R, Cc)).astype(F[dt]); base_b = rng.uniform(-1, 1, (R, Cc)).astype(F[dt])
    ta, tb = on(device, base_a), on(device, base_b)
    for name, expect_path in (("permuted", "tile_transpose"), ("sliced", "rows"), ("sliced_rows", "rows")):
        say("view", name, dt)
        va, vb = VIEWS[name](ta), VIEWS[name](tb)
        out = Tensor._on_device(device, F[dt], va.shape)
        device.launch_elementwise("multiply", -1, out, va, vb)
        assert _lib.last_path().startswith(expect_path), (name, _lib.last_path())
        want = orc.elementwise("multiply", -1, np.zeros(out.size, dtype=F[dt]), cfg(out), base_a.reshape(-1), cfg(va), base_b.reshape(-1), cfg(vb))
        assert_bits(out.getData(), want, name)
        # one view, one dense operand; and a view as the DRAIN
        dense = on(device, rng.uniform(-1, 1, va.shape).astype(F[dt]))
        device.launch_elementwise("add", -1, out, va, dense)
        want = orc.elementwise("add", -1, np.zeros(out.size, dtype=F[dt]), cfg(out), base_a.reshape(-1), cfg(va), dense.getData(), cfg(dense))
        assert_bits(out.getData(), want, name + " mixed")
        target = on(device, np.zeros((R, Cc), dtype=F[dt]))
        vt = VIEWS[name](target)
        device.launch_activation("idy", -1, vt, dense)
        want = orc.activation("idy", -1, np.zeros(R * Cc, dtype=F[dt]), cfg(vt), dense.getData(), cfg(dense))
        assert_bits(target.getData(), want, name + " as drain")
    # rank 3 permutation with the contiguous axis moved to the front
    say("view perm3", dt)
    b3 = rng.uniform(-1, 1, (9, 20, 33)).astype(F[dt])
    t3 = on(device, b3)
    v3 = t3.permute(2, 0, 1)
    out = Tensor._on_device(device, F[dt], v3.shape)
    device.launch_activation("quad", -1, out, v3)
    assert_bits(out.getData(), orc.activation("quad", -1, np.zeros(out.size, dtype=F[dt]), cfg(out), b3.reshape(-1), cfg(v3)), "perm3")


def test_slices_of_transposed_tensors_walk_in_row_major_order(device, orc):
    """A slice of a transposed (column-major) matrix carries the column-major indicesMap [1, rows] (Slice.java:88),
    with which idx[0] = i / 1 leaves the view for every flat index beyond the first column.  The one result the
    reference defines there is that of a CPU workload from index 0 (every operand starts at nd-index 0 and advances
    in row-major order): what the oracle computes in one piece, what numpy computes -- as source, as drain, for every
    kernel family that unravels a flat index, and never an access outside the view."""
    rng = np.random.default_rng(77)
    for dt in ("f32", "f64"):
        T = F[dt]
        for R, Cn in ((8, 15), (130, 517), (1024, 2050)):
            say("slice of a transposed tensor", dt, R, Cn)
            a = rng.standard_normal((R, Cn)).astype(T); b = rng.standard_normal((Cn, R)).astype(T)
            ta, tb = on(device, a), on(device, b)
            va, vb = ta[1::2, 3::2], tb.T()[1::2, 3::2]
            assert cfg(vb).tolist()[4:6] == [1, va.shape[0]]                      # the column-major table
            na, nb = a[1::2, 3::2], b.T[1::2, 3::2]
            so = va.shape
            n = int(np.prod(so))
            dense = orc.dense_cfg(list(so))
            # both kinds of source, dense drain
            out = Tensor._on_device(device, T, so)
            device.launch_elementwise("subtract", -1, out, va, vb)
            assert _lib.last_path() != "literal", _lib.last_path()
            assert_bits(out.getData().reshape(so), na - nb, "a - b^T, slices")
            assert_bits(out.getData(), orc.elementwise("subtract", -1, np.zeros(n, dtype=T), dense, a.reshape(-1), cfg(va), b.reshape(-1), cfg(vb)), "oracle")
            device.launch_scalarization("multiply", -1, out, vb, 3.0)
            assert_bits(out.getData().reshape(so), nb * T(3.0), "3 b^T")
            device.launch_activation("relu", -1, out, vb)
            assert_bits(out.getData(), orc.activation("relu", -1, np.zeros(n, dtype=T), dense, b.reshape(-1), cfg(vb)), "relu")
            fn = Function.of("I[0]*I[1]+I[0]")
            got = device.optimizedFunctionOf(fn, "fma")(vb, va)
            assert_bits(got.getData().reshape(so), nb * na + nb, "fused")
            # the drain is such a view: only its elements change
            parent = rng.standard_normal((Cn, R)).astype(T)
            tp = on(device, parent)
            drain = tp.T()[1::2, 3::2]
            device.launch_elementwise("add", -1, drain, va, vb)
            want = parent.copy(); want.T[1::2, 3::2] = na + nb
            assert_bits(tp.getData().reshape(Cn, R), want, "drain view")
            device.launch_scalar_fill(drain, 7.0)
            want.T[1::2, 3::2] = 7.0
            assert_bits(tp.getData().reshape(Cn, R), want, "fill of a drain view")
            # broadcast backward into such a drain: the error [r, c] summed over axis 0 into a row [1, c] of the view
            e = rng.integers(-3, 4, so).astype(T)
            te = on(device, e)
            row = tb.T()[1:2, 3::2]                                                # column-major table [1, 1]
            assert cfg(row).tolist()[4:6] == [1, 1]
            zeros = Tensor._on_device(device, T, (so[0], 1))
            device.launch_broadcast("add", 0, row, zeros, te)
            want_b = b.copy(); want_b.T[1:2, 3::2] = e.sum(axis=0, keepdims=True)
            assert_bits(tb.getData().reshape(Cn, R), want_b, "backward into a drain view")
        # integers: the indexed kernel
        say("slice of a transposed int32 tensor")
        x = rng.integers(-1000, 1000, (15, 8)).astype(np.int32)
        tx = on(device, x)
        vx = tx.T()[1::2, 3::2]
        out = Tensor._on_device(device, np.int32, vx.shape)
        device.launch_scalarization("multiply", -1, out, vx, 3)
        assert (out.getData().reshape(vx.shape) == x.T[1::2, 3::2] * 3).all()
    # convolution into a drain view
    say("convolution into a slice of a transposed tensor")
    img = rng.integers(-3, 4, (1, 1, 12, 17)).astype(np.float32); ker = rng.integers(-2, 3, (1, 1, 3, 3)).astype(np.float32)
    ti, tk = on(device, img), on(device, ker)
    parent = np.zeros((1, 1, 30, 20), dtype=np.float32)
    tp = on(device, parent)
    drain = tp.permute(0, 1, 3, 2)[0:1, 0:1, 0:10, 0:15]
    device.launch_convolution(-1, drain, ti, tk)
    full = np.zeros((10, 15), dtype=np.float32)
    for ky in range(3):
        for kx in range(3):
            full += img[0, 0, ky:ky + 10, kx:kx + 15] * ker[0, 0, ky, kx]
    want = parent.copy(); want.transpose(0, 1, 3, 2)[0, 0, 0:10, 0:15] = full
    assert_bits(tp.getData().reshape(parent.shape), want, "convolution drain view")


def test_reference_view_chains_on_device(device, orc, golden):
    """tests/golden/reference_views.json on the device: every view chain of Tensor_Slice_Permute_Spec and Tensor_Slicing_Spec
    (slices, transposed slices -- whose descriptors carry the column-major unravel table --, padded reshapes) read
    through the kernels: a copy through the view (the identity activation), the view times two (scalarization), the view
    as drain of an assignment, and the product of the two transposed blocks through the operator x."""
    import json
    import os
    from helpers import apply_view_chain, view_row_parent
    data = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_views.json")))
    views = []
    for row in data["rows"]:
        say("view chain", row["name"])
        parent = view_row_parent(row)
        t = Tensor.of(parent.dtype, row["shape"], parent).to(device)
        v = apply_view_chain(t, row["chain"])
        views.append(v)
        assert list(v.shape) == row["want_shape"]
        want = np.asarray(row["want"], dtype=parent.dtype)
        if np.issubdtype(parent.dtype, np.integer):
            out = Tensor._on_device(device, parent.dtype, v.shape)
            device.launch_scalarization("multiply", -1, out, v, 2)
            assert out.getData().tolist() == (want * 2).tolist(), row["name"]
            continue
        assert_bits(v.deepCopy().getData(), want, row["name"] + ": copy through the view")
        out = Tensor._on_device(device, parent.dtype, v.shape)
        device.launch_scalarization("multiply", -1, out, v, 2.0)
        assert_bits(out.getData(), want * 2, row["name"] + ": twice the view")
        dense = orc.dense_cfg(list(v.shape))
        assert_bits(orc.activation("idy", -1, np.zeros(v.size, dtype=parent.dtype), dense, parent, cfg(v)), want, row["name"] + ": oracle")
        # the view as a drain: only its elements change
        fresh = Tensor.of(parent.dtype, v.shape, -want).to(device)
        v.assign(fresh)
        after = parent.copy()
        orc.activation("idy", -1, after, cfg(v), -want, dense)
        assert_bits(t.getData(), after, row["name"] + ": assignment into the view")
        assert_bits(v.items, -want, row["name"] + ": items after the assignment")
    for prod in data["products"]:
        say("product of transposed slices")
        rows = data["rows"]
        ta = apply_view_chain(on(device, view_row_parent(rows[prod["left_row"]]).reshape(rows[prod["left_row"]]["shape"])), rows[prod["left_row"]]["chain"])
        tb = apply_view_chain(on(device, view_row_parent(rows[prod["right_row"]]).reshape(rows[prod["right_row"]]["shape"])), rows[prod["right_row"]]["chain"])
        c = ta.permute(0, 1, -1).conv(tb.permute(-1, 0, 1))          # convDot: [2,2,1] x [1,2,2] (Tensor.java:1949-1966)
        assert list(c.shape) == prod["want_shape"] and c.items.tolist() == prod["want"]


def test_exotic_descriptor_falls_back_to_the_literal_formula(device, orc):
    """A descriptor whose indicesMap is not the row-major table of its shape cannot be reduced to
    base + strides: the literal kernel evaluates NDConfiguration.indexOfIndex (the formula the 20 rows of
    NDConfiguration_Spec pin, and the one `items` reads results back with) for every operand.
    (The reference's CPU kernels walk such operands with iterator increments from each thread's range
    start, which makes their result depend on the thread partition; that is not a parity target.)"""
    say("literal fallback")
    ndc = NDConfiguration.of([2, 3], [3, 1], [3, 2], [1, 1], [0, 0])        # flat 2 -> (0, 1), flat 1 -> (0, 0)
    src = np.arange(1, 13, dtype=np.float32)
    tsrc = on(device, src)
    weird = Tensor(np.float32, ndc, None); weird._set_data(tsrc._data, device)
    out = on(device, np.zeros((2, 3), dtype=np.float32))
    dense6 = on(device, np.arange(6, dtype=np.float32).reshape(2, 3))
    with pytest.raises(IllegalArgumentException):                      # operands of one launch share one rank
        device.launch_elementwise("add", -1, on(device, np.zeros(6, dtype=np.float32)), weird, dense6)
    device.launch_elementwise("add", -1, out, weird, dense6)
    assert _lib.last_path() == "literal"
    phys = [orc.index_of_index(ndc.asInlineArray(), i) for i in range(6)]
    assert phys == physical_indices(ndc).tolist() == [0, 0, 1, 3, 3, 4]
    assert_bits(out.getData(), src[phys] + np.arange(6, dtype=np.float32), "literal")
    # the same descriptor as the drain
    backing = on(device, np.full(12, -1, dtype=np.float32))             # kept: a dropped tensor gives up its buffer
    out2 = Tensor(np.float32, ndc, None); out2._set_data(backing._data, device)
    device.launch_activation("idy", -1, out2, dense6)
    # a unary kernel addresses its source with the DRAIN's nd-index (CPUElementwiseFunction.java:103-104):
    # flat 0..5 -> nd (0,0),(0,0),(0,1),(1,0),(1,0),(1,1) -> the dense source's elements 0,0,1,3,3,4
    got = out2.getData()
    assert got.tolist() == [0, 1, -1, 3, 4, -1, -1, -1, -1, -1, -1, -1]
    # virtual source: all-zero tables address element 0
    virt = Tensor.of(np.float32, [2, 3], 2.5).to(device)
    device.launch_elementwise("multiply", -1, out, virt, dense6)
    assert_bits(out.getData(), dense6.getData() * np.float32(2.5), "virtual")


# ---- broadcast ----------------------------------------------------------------------------------------------
def test_broadcast_forward_golden_on_device(device, golden):
    g = golden["broadcast_stress"]
    for row in g["rows"]:
        say("golden broadcast", row["op"], row["shape1"], row["shape2"])
        a = Tensor.of(np.float64, row["shape1"], g["t1_range"]).to(device)
        b = Tensor.of(np.float64, row["shape2"], g["t2_range"]).to(device)
        fn = {"modulo": lambda x, y: x % y, "multiply": lambda x, y: x * y, "add": lambda x, y: x + y,
              "subtract": lambda x, y: x - y, "divide": lambda x, y: x / y}[row["op"]]
        out = fn(a, b)
        assert list(out.shape) == row["shape"]
        def fmt(v):
            if np.isnan(v): return "NaN"
            if np.isinf(v): return "-inf" if v < 0 else "inf"
            r = round(float(v), 5)
            return repr(r) if r != 0 else ("-0.0" if np.signbit(v) else "0.0")
        assert [fmt(v) for v in out.items] == row["expected"], row


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_broadcast_forward_bit_exact(device, orc, dt):
    rng = np.random.default_rng(21)
    cases = [([64, 1, 96], [1, 40, 96]), ([1, 40, 1], [64, 40, 96]), ([33, 1], [1, 77]), ([5, 6, 7], [5, 6, 7]),
             ([3, 1, 5, 1], [1, 4, 1, 6]), ([1], [1]), ([128, 1, 4], [1, 9, 4])]
    for s1, s2 in cases:
        say("broadcast fwd", s1, s2, dt)
        so = [q if p == 1 else p for p, q in zip(s1, s2)]
        a = rng.uniform(-1, 1, s1).astype(F[dt]); b = rng.uniform(-1, 1, s2).astype(F[dt])
        ta, tb = on(device, a), on(device, b)
        for op, f in (("add", np.add), ("subtract", np.subtract), ("multiply", np.multiply)):
            out = Tensor._on_device(device, F[dt], so)
            device.launch_broadcast(op, -1, out, ta, tb)
            want = orc.broadcast(op, -1, np.zeros(out.size, dtype=F[dt]), orc.dense_cfg(so), a.reshape(-1), orc.dense_cfg(s1), b.reshape(-1), orc.dense_cfg(s2))
            assert_bits(out.getData(), want, f"{op} {s1} {s2}")
            assert_bits(out.getData().reshape(so), f(a, b), f"{op} numpy")


def test_rows_shorter_than_a_vector_merge_with_the_axis_above(device, orc):
    """f32 rows of two or three elements (channels-last data and a per-channel operand): the innermost axis and the one
    above it become one long row; operands that are dense across both move in vectors, an operand pinned on the upper
    axis repeats with the short row as its period and is gathered at column mod period.  Broadcast in both operand
    orders, a bias over a flat image, rank 4, a million rows; + * / bit for bit, power and modulo against the oracle.
    A drain with gaps, or a source with another stride, keeps the element-wise path."""
    T = np.float32
    rng = np.random.default_rng(28)
    for s1, s2 in (([4096, 1, 3], [1, 64, 3]), ([1, 64, 3], [4096, 1, 3]),            # rows of 192
                         ([300, 500, 3], [1, 1, 3]), ([1, 1, 3], [300, 500, 3]),            # one row of 450 000
                         ([7, 1, 1, 2], [1, 5, 33, 2]),                                            # rows of 330, period 2
                         ([5000, 1, 3], [5000, 77, 3]),                                            # rows of 231
                         ([9, 1, 1, 3], [9, 4, 11, 3]),                                              # rows of 132
                         ([1, 3], [1000003, 3]),                                                   # one row of 3 000 009
                         ([77, 1, 2], [1, 34, 2]),                                                   # rows of 68, period 2
                         ([33, 1, 3], [33, 4, 3]),                                                   # rows of 12: one thread per row
                         ([1, 1, 3], [70001, 4, 3])):                                                # one row of 840 012
        so = [q if p == 1 else p for p, q in zip(s1, s2)]
        a = rng.uniform(-1, 1, s1).astype(T); b = rng.uniform(-1, 1, s2).astype(T)
        ta, tb = on(device, a), on(device, b)
        for op, f in (("add", np.add), ("multiply", np.multiply), ("divide", np.divide), ("subtract", np.subtract)):
            say("short rows", s1, s2, op)
            out = Tensor._on_device(device, T, so)
            device.launch_broadcast(op, -1, out, ta, tb)
            assert _lib.last_path() == "rows_vec_binary_periodic", (_lib.last_path(), s1, s2)
            assert_bits(out.getData().reshape(so), f(a, b), f"{op} {s1} {s2}")
    say("rows of five and seven merge when the whole tensor becomes one row")
    for s1, s2, path in (([70001, 5], [1, 5], "rows_vec_binary_periodic"), ([1, 1, 7], [333, 99, 7], "rows_vec_binary_periodic"), ([512, 1, 5], [1, 9, 5], "rows_vec_binary")):
        so = [q if p == 1 else p for p, q in zip(s1, s2)]
        a = rng.uniform(-1, 1, s1).astype(T); b = rng.uniform(-1, 1, s2).astype(T)
        out = Tensor._on_device(device, T, so)
        device.launch_broadcast("subtract", -1, out, on(device, a), on(device, b))
        assert _lib.last_path() == path, (_lib.last_path(), s1, s2)
        assert_bits(out.getData().reshape(so), a - b, f"subtract {s1} {s2}")
    say("short rows, power and modulo")
    s1, s2 = [513, 1, 3], [1, 21, 3]
    so = [513, 21, 3]
    a = rng.uniform(0.5, 2, s1).astype(T); b = rng.uniform(0.5, 2, s2).astype(T)
    for op in ("power", "modulo"):
        out = Tensor._on_device(device, T, so)
        device.launch_broadcast(op, -1, out, on(device, a), on(device, b))
        assert _lib.last_path() == "rows_vec_periodic", _lib.last_path()
        want = orc.broadcast(op, -1, np.zeros(out.size, dtype=T), orc.dense_cfg(so), a.reshape(-1), orc.dense_cfg(s1), b.reshape(-1), orc.dense_cfg(s2))
        assert_close(out.getData(), want, op)
    say("short rows in place and with a ragged merged row")
    for n_rows in (7, 1001, 4096):                                       # 21 and 3003 elements: no whole number of vectors
        x = rng.uniform(-1, 1, [n_rows, 3]).astype(T); bias = rng.uniform(-1, 1, [1, 3]).astype(T)
        tx = on(device, x)
        device.launch_broadcast("add", -1, tx, tx, on(device, bias))     # x += bias
        assert "periodic" in _lib.last_path(), (_lib.last_path(), n_rows)
        assert_bits(tx.getData().reshape(n_rows, 3), x + bias, f"in place {n_rows}")
        out = Tensor._on_device(device, T, [n_rows, 3])
        device.launch_broadcast("multiply", -1, out, on(device, bias), on(device, x))
        assert "periodic" in _lib.last_path(), (_lib.last_path(), n_rows)
        assert_bits(out.getData().reshape(n_rows, 3), bias * x, f"ragged {n_rows}")
    say("short rows that stay element-wise")
    wide = on(device, np.zeros((64, 8, 4), dtype=T))
    view = wide[:, :, 0:3]                                                   # a drain with gaps
    device.launch_broadcast("add", -1, view, on(device, rng.uniform(-1, 1, [64, 1, 3]).astype(T)), on(device, rng.uniform(-1, 1, [1, 8, 3]).astype(T)))
    assert _lib.last_path() in ("rows_binary", "rows", "canon"), _lib.last_path()


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_ragged_rows_run_on_vectors_and_stay_bit_exact(device, orc, dt):
    """Rows whose length is not a multiple of the 16-byte vector: the last vector of a row is moved back to end with the
    row (its neighbour's elements are computed twice).  Broadcast, same-shape elementwise, an activation and a fused
    chain, bit for bit; and in place (the drain is one of the sources), where computing twice would not be the
    same thing, the element-wise path must be taken."""
    rng = np.random.default_rng(23)
    T = F[dt]
    V = 16 // np.dtype(T).itemsize
    for s1, s2 in (([37, 1, 511], [1, 9, 511]), ([5, 1, 7], [1, 6, 7]), ([3, 1023], [3, 1023]), ([64, 1, 5], [1, 33, 5]), ([2, 1, V + 1], [1, 3, V + 1])):
        so = [q if p == 1 else p for p, q in zip(s1, s2)]
        a = rng.uniform(-1, 1, s1).astype(T); b = rng.uniform(-1, 1, s2).astype(T)
        ta, tb = on(device, a), on(device, b)
        for op, f in (("add", np.add), ("multiply", np.multiply), ("divide", np.divide)):
            say("ragged broadcast", s1, s2, op, dt)
            out = Tensor._on_device(device, T, so)
            device.launch_broadcast(op, -1, out, ta, tb)
            assert _lib.last_path() == "rows_vec_binary", _lib.last_path()
            assert_bits(out.getData().reshape(so), f(a, b), f"{op} {s1} {s2}")
    n = [7, 333]
    x = rng.uniform(-2, 2, n).astype(T); y = rng.uniform(-2, 2, n).astype(T)
    tx, ty = on(device, x), on(device, y)
    say("ragged activation", dt)
    out = Tensor._on_device(device, T, n)
    device.launch_activation("softsign", -1, out, tx)
    assert _lib.last_path() == "rows_vec_single"
    assert_bits(out.getData(), orc.activation("softsign", -1, np.zeros(x.size, dtype=T), orc.dense_cfg(n), x.reshape(-1), orc.dense_cfg(n)), "softsign")
    say("ragged in place", dt)
    device.launch_elementwise("add", -1, tx, tx, ty)                       # x += y
    assert _lib.last_path() == "rows_binary", _lib.last_path()
    assert_bits(tx.getData().reshape(n), x + y, "in place")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_square_and_first_power_are_exact_products(device, orc, dt):
    """x ** 2 and x ** 1 with a scalar exponent leave the power kernels: the square is the correctly rounded product
    (what Math.pow returns: the exact product of two floats fits a double), the first power is x itself
    (Math.pow's specification).  Special values included; other exponents still go through pow."""
    T = F[dt]
    rng = np.random.default_rng(27)
    x = np.concatenate([rng.uniform(-3, 3, 1000), [0.0, -0.0, np.inf, -np.inf, np.nan, 1e30, -1e30, 1e-30, 3e-39]]).astype(T)
    tx = on(device, x)
    cfg1 = orc.dense_cfg([x.size])
    for value in (2.0, 1.0, 3.0, 0.0, -1.0):
        say("x **", value, dt)
        out = Tensor._on_device(device, T, (x.size,))
        device.launch_scalarization("power", -1, out, tx, value)
        with np.errstate(all="ignore"):
            want = orc.scalarization("power", -1, np.zeros_like(x), cfg1, x, cfg1, value)
            if value == 2.0:
                assert_bits(out.getData(), x * x, "square")
            if value == 1.0:
                assert_bits(out.getData(), x, "first power")
        assert_close(out.getData(), want, f"x ** {value}")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_sources_that_take_every_nth_column(device, orc, dt):
    """Step slices along the innermost axis: the rows kernels gather the source element by element and still write the
    drain in whole vectors."""
    rng = np.random.default_rng(26)
    T = F[dt]
    a = rng.uniform(-2, 2, (33, 200)).astype(T); b = rng.uniform(-2, 2, (33, 200)).astype(T)
    ta, tb = on(device, a), on(device, b)
    for sl in (np.s_[:, ::2], np.s_[1:30, 1::3], np.s_[::2, 4:196:8]):
        va, vb = ta[sl], tb[sl]
        say("every n-th column", sl, dt)
        out = Tensor._on_device(device, T, va.shape)
        device.launch_activation("softsign", -1, out, va)
        assert _lib.last_path() in ("rows_vec", "rows"), _lib.last_path()
        x = np.ascontiguousarray(a[sl]); dense = orc.dense_cfg(list(x.shape))
        assert_bits(out.getData(), orc.activation("softsign", -1, np.zeros(x.size, dtype=T), dense, x.reshape(-1), dense), "softsign")
        device.launch_elementwise("multiply", -1, out, va, vb)
        assert _lib.last_path() in ("rows_vec", "rows"), _lib.last_path()
        assert_bits(out.getData().reshape(x.shape), a[sl] * b[sl], "multiply")
        device.launch_elementwise("subtract", -1, out, va, on(device, np.ascontiguousarray(b[sl])))     # one strided, one dense
        assert_bits(out.getData().reshape(x.shape), a[sl] - b[sl], "subtract")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_deep_index_spaces_and_row_constant_sources(device, orc, dt):
    """Four and five outer axes that do not merge (alternating broadcast axes, slices on every axis) and sources that
    are constant along a row (outer products, per-row scales): the vector kernels with every outer axis resolved,
    bit for bit against numpy / the oracle."""
    rng = np.random.default_rng(24)
    T = F[dt]
    for s1, s2 in (([6, 1, 5, 1, 8], [1, 4, 1, 3, 8]), ([3, 1, 4, 1, 2, 12], [1, 2, 1, 3, 1, 12]), ([6, 1, 5, 1, 3], [1, 4, 1, 3, 3]),
                   ([40, 9, 1], [1, 1, 64]), ([7, 1], [1, 36]), ([1, 36], [7, 1]), ([5, 3, 16], [5, 3, 1]), ([5, 3, 1], [5, 1, 1])):
        so = [max(p, q) for p, q in zip(s1, s2)]
        a = rng.uniform(-1, 1, s1).astype(T); b = rng.uniform(-1, 1, s2).astype(T)
        ta, tb = on(device, a), on(device, b)
        for op, f in (("add", np.add), ("subtract", np.subtract), ("multiply", np.multiply), ("divide", np.divide)):
            say("deep / row-constant broadcast", s1, s2, op, dt)
            out = Tensor._on_device(device, T, so)
            device.launch_broadcast(op, -1, out, ta, tb)
            assert _lib.last_path() in ("rows_vec_binary", "rows_binary", "rows_vec", "rows", "rows_vec_binary_periodic"), _lib.last_path()
            assert_bits(out.getData().reshape(so), f(a, b), f"{op} {s1} {s2}")
    say("activation and fused chain on a view with five live axes", dt)
    parent = rng.uniform(-2, 2, (5, 6, 7, 5, 40)).astype(T)
    tp = on(device, parent)
    view = tp[1:4, 0:6:2, 2:7, 1:5:3, 4:36]
    want_items = parent[1:4, 0:6:2, 2:7, 1:5:3, 4:36]
    out = Tensor._on_device(device, T, view.shape)
    device.launch_activation("softsign", -1, out, view)
    assert _lib.last_path() in ("rows_vec", "rows_vec_single"), _lib.last_path()
    dense = orc.dense_cfg(list(view.shape))
    want = orc.activation("softsign", -1, np.zeros(out.size, dtype=T), dense, np.ascontiguousarray(want_items).reshape(-1), dense)
    assert_bits(out.getData(), want, "softsign on a deep view")
    from neureka_amd.function import Function
    fused = device.optimizedFunctionOf(Function.of("tanh(sig(I[0])*I[1]+I[2])"), "chain")
    got = fused(view, view, view)
    x = np.ascontiguousarray(want_items).reshape(-1)
    t1 = orc.activation("sig", -1, np.zeros_like(x), dense, x, dense)
    t2 = orc.elementwise("multiply", -1, np.zeros_like(x), dense, t1, dense, x, dense)
    t3 = orc.elementwise("add", -1, np.zeros_like(x), dense, t2, dense, x, dense)
    assert_close(got.items, orc.activation("tanh", -1, np.zeros_like(x), dense, t3, dense), "fused chain on a deep view")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_broadcast_backward_bit_exact(device, orc, dt):
    rng = np.random.default_rng(22)
    full = [6, 5, 7]
    e = rng.uniform(-1, 1, full).astype(F[dt])
    te = on(device, e)
    for tgt in ([6, 1, 7], [1, 5, 1], [1, 1, 1], [6, 5, 7], [6, 5, 1]):
        for op in ("add", "subtract", "multiply"):
            for d in (0, 1):
                say("broadcast bwd", tgt, op, d, dt)
                other = rng.uniform(-1, 1, full).astype(F[dt]) if op == "multiply" else np.zeros(full, dtype=F[dt])
                tother = on(device, other)
                drn = Tensor._on_device(device, F[dt], tgt)
                device.launch_broadcast(op, d, drn, tother, te)
                want = orc.broadcast(op, d, np.zeros(drn.size, dtype=F[dt]), orc.dense_cfg(tgt), other.reshape(-1), orc.dense_cfg(full), e.reshape(-1), orc.dense_cfg(full))
                assert_bits(drn.getData(), want, f"{tgt} {op} {d}")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_broadcast_backward_split_sums(device, orc, dt):
    """Gradients with few elements and long sums (a bias, a row sum, a full reduction) or with the innermost axis
    reduced: blocks split the sums.  Same terms as the reference, another order: |delta| <= tol * sum |terms| against the
    oracle's sequential sums (tol 1e-5 / 1e-12), exact on integer-valued data."""
    T = F[dt]
    tol = 1e-5 if dt == "f32" else 1e-12
    rng = np.random.default_rng(25)
    cases = [([48, 40, 128], [1, 1, 128], "broadcast_backward_split_vec"), ([48, 40, 128], [48, 1, 1], "broadcast_backward_split_rows_vec"),
             ([48, 40, 128], [1, 40, 1], "broadcast_backward_split_rows_vec"), ([48, 40, 128], [1, 1, 1], "broadcast_backward_split_rows_vec"),
             ([6, 10, 2048], [6, 10, 1], "broadcast_backward_split_rows_vec"), ([6, 10, 512], [6, 10, 1], "broadcast_backward_split_rows_vec"),
             ([7, 9, 515], [7, 9, 1], "broadcast_backward_split_rows"), ([5, 3, 1027], [5, 3, 1], "broadcast_backward_split_rows"),
             ([1100, 700], [1, 700], "broadcast_backward_split_vec"), ([1100, 701], [1, 701], "broadcast_backward_split"),
             ([30, 2100], [30, 1], "broadcast_backward_split_rows_vec"), ([1100, 2000], [1, 2000], "broadcast_backward_split_vec"),
             ([19, 300, 1, 70], [1, 300, 1, 1], "broadcast_backward_split_rows")]
    for full, tgt, path in cases:
        for integer in (True, False):
            for op, d in (("add", 0), ("subtract", 1), ("multiply", 0), ("multiply", 1), ("divide", 1)):
                if integer and op == "divide":
                    continue
                if op == "divide":      # the error is the divisor here: keep it away from zero, or single terms dwarf the sum
                    e = (rng.uniform(0.5, 1.5, full) * rng.choice([-1.0, 1.0], full)).astype(T)
                else:
                    e = (rng.integers(-3, 4, full) if integer else rng.uniform(-1, 1, full)).astype(T)
                te = on(device, e)
                say("broadcast bwd split", full, tgt, op, d, dt, "integer" if integer else "uniform")
                if op in ("multiply", "divide"):
                    other = (rng.integers(1, 4, full) if integer else rng.uniform(0.5, 1.5, full)).astype(T)
                else:
                    other = np.zeros(full, dtype=T)
                drn = Tensor._on_device(device, T, tgt)
                device.launch_broadcast(op, d, drn, on(device, other), te)
                assert _lib.last_path().startswith(path), (_lib.last_path(), path)
                dense_t, dense_f = orc.dense_cfg(tgt), orc.dense_cfg(full)
                want = orc.broadcast(op, d, np.zeros(drn.size, dtype=T), dense_t, other.reshape(-1), dense_f, e.reshape(-1), dense_f)
                if integer:
                    assert_bits(drn.getData(), want, f"{full} {tgt} {op} {d}")
                else:
                    # the same sum over the absolute values of the terms bounds the rounding error of any order
                    mag = orc.broadcast(op, d, np.zeros(drn.size), dense_t, np.abs(other).astype(np.float64).reshape(-1), dense_f,
                                        np.abs(e).astype(np.float64).reshape(-1), dense_f)
                    err_abs = np.abs(drn.getData().astype(np.float64) - want)
                    worst = int(np.argmax(err_abs / (np.abs(mag) + 1e-300)))
                    assert (err_abs <= tol * np.abs(mag) + 1e-30).all(), (full, tgt, op, d, worst, float(drn.getData()[worst]), float(want[worst]), float(mag[worst]))
    # a source that does not move along the 16-byte vector has its own instantiations: the other operand in its own
    # shape, as autograd passes it (extent 1 where the drain keeps the innermost axis), and a virtual tensor (one
    # element, all-zero tables) where the innermost axis is reduced
    for full, tgt, oth, path in (([48, 40, 128], [1, 1, 128], [48, 40, 1], "broadcast_backward_split_vec"),
                                 ([1100, 700], [1, 700], [1100, 1], "broadcast_backward_split_vec"),
                                 ([48, 40, 128], [48, 1, 1], None, "broadcast_backward_split_rows_vec"),
                                 ([30, 2100], [30, 1], None, "broadcast_backward_split_rows_vec")):
        e = rng.integers(-3, 4, full).astype(T)
        te = on(device, e)
        for op, d in (("add", 0), ("subtract", 1), ("multiply", 0), ("multiply", 1)):
            say("broadcast bwd split, constant source", full, tgt, oth, op, d, dt)
            if oth is None:
                other = np.full(full, 3, dtype=T)
                tother = Tensor.of(T, full, 3.0).to(device)
                assert tother.isVirtual()
                other_cfg = orc.dense_cfg(full)
            else:
                other = rng.integers(1, 4, oth).astype(T)
                tother = on(device, other)
                other_cfg = orc.dense_cfg(oth)
            drn = Tensor._on_device(device, T, tgt)
            device.launch_broadcast(op, d, drn, tother, te)
            assert _lib.last_path().startswith(path), (_lib.last_path(), path)
            want = orc.broadcast(op, d, np.zeros(drn.size, dtype=T), orc.dense_cfg(tgt), other.reshape(-1), other_cfg, e.reshape(-1), orc.dense_cfg(full))
            assert_bits(drn.getData(), want, f"constant source {full} {tgt} {oth} {op} {d}")
    say("broadcast bwd split on a sliced error and a transposed drain", dt)
    parent = rng.integers(-3, 4, (50, 44, 140)).astype(T)
    err = on(device, parent)[1:49, 2:42, 6:134]
    for tgt in ([1, 1, 128], [48, 1, 1]):
        drn = Tensor._on_device(device, T, tgt)
        device.launch_broadcast("add", 0, drn, on(device, np.zeros([48, 40, 128], dtype=T)), err)
        assert _lib.last_path().startswith("broadcast_backward_split")
        axes = tuple(k for k in range(3) if tgt[k] == 1)
        assert_bits(drn.getData().reshape(tgt), parent[1:49, 2:42, 6:134].sum(axis=axes, keepdims=True).astype(T), f"sliced error {tgt}")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_broadcast_backward_split_sums_in_pairs(device, orc, dt):
    """Long sums over a contiguous innermost axis with src1 pinned along a kept axis (per-slab sums of an operand that the
    forward broadcast repeated over the slabs): a block owns two drain elements half that axis apart and reads src1
    once for both.  Exact on integer-valued data; norm-wise within 1e-5 / 1e-12 on uniform data; one and several
    segments per sum; a kept axis in the middle."""
    T = F[dt]
    tol = 1e-5 if dt == "f32" else 1e-12
    rng = np.random.default_rng(27)
    for full, tgt, oth in (([1024, 16, 512], [1024, 1, 1], [1, 16, 512]),       # four segments per pair of sums
                           ([4096, 4, 2048], [4096, 1, 1], [1, 4, 2048]),       # one segment: straight into the drain
                           ([3, 512, 8192], [3, 512, 1], [3, 1, 8192])):        # the second axis pairs
        for integer in (True, False):
            for op, d in (("add", 0), ("subtract", 1), ("multiply", 1), ("divide", 1)):
                if integer and op == "divide":
                    continue
                if op == "divide":
                    e = (rng.uniform(0.5, 1.5, full) * rng.choice([-1.0, 1.0], full)).astype(T)
                else:
                    e = (rng.integers(-3, 4, full) if integer else rng.uniform(-1, 1, full)).astype(T)
                other = (rng.integers(1, 4, oth) if integer else rng.uniform(0.5, 1.5, oth)).astype(T)
                say("broadcast bwd split pairs", full, tgt, op, d, dt, "integer" if integer else "uniform")
                drn = Tensor._on_device(device, T, tgt)
                device.launch_broadcast(op, d, drn, on(device, other), on(device, e))
                assert _lib.last_path() == "broadcast_backward_split_rows_vec_pairs", _lib.last_path()
                dense_t, dense_o, dense_f = orc.dense_cfg(tgt), orc.dense_cfg(oth), orc.dense_cfg(full)
                want = orc.broadcast(op, d, np.zeros(drn.size, dtype=T), dense_t, other.reshape(-1), dense_o, e.reshape(-1), dense_f, workers=8)
                if integer:
                    assert_bits(drn.getData(), want, f"{full} {tgt} {op} {d}")
                else:
                    mag = orc.broadcast(op, d, np.zeros(drn.size), dense_t, np.abs(other).astype(np.float64).reshape(-1), dense_o,
                                        np.abs(e).astype(np.float64).reshape(-1), dense_f, workers=8)
                    err_abs = np.abs(drn.getData().astype(np.float64) - want)
                    assert (err_abs <= tol * np.abs(mag) + 1e-30).all(), (full, tgt, op, d, float(err_abs.max()))


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_broadcast_backward_two_drain_elements_per_thread(device, orc, dt):
    """Large gradients along whose kept axis src1 is pinned (the operand the forward broadcast repeated): a thread owns
    the drain elements i and i + extent / 2 of that axis and loads every value of src1 once for both sums.  Random,
    non-zero src1 of the other operand's shape, every form of the term that reads src1, pair axis first, in the middle
    and next to the vector axis, a drain view with gaps: bit-identical to the CPU state machine."""
    T = F[dt]
    rng = np.random.default_rng(26)
    cases = [([1024, 6, 512], [1024, 1, 512], [1, 6, 512]),            # pair axis 0
             ([6, 1024, 512], [1, 1024, 512], [6, 1, 512]),            # pair axis 1, reduced axis outermost
             ([4, 1024, 5, 512], [1, 1024, 1, 512], [4, 1, 5, 1]),     # two reduced axes around the pair axis
             ([512, 3, 2, 512], [512, 1, 2, 512], [1, 3, 1, 512])]     # the first of two pinned axes pairs
    for full, tgt, oth in cases:
        e = rng.uniform(0.5, 1.5, full).astype(T) * rng.choice([-1.0, 1.0], full).astype(T)
        te = on(device, e)
        for op, d in (("add", 0), ("subtract", 1), ("multiply", 0), ("multiply", 1), ("divide", 0), ("divide", 1), ("power", 0)):
            say("broadcast bwd pairs", full, tgt, op, d, dt)
            other = rng.uniform(0.5, 1.5, oth).astype(T)
            drn = Tensor._on_device(device, T, tgt)
            device.launch_broadcast(op, d, drn, on(device, other), te)
            assert _lib.last_path() == "broadcast_backward_vec_pairs", _lib.last_path()
            want = orc.broadcast(op, d, np.zeros(drn.size, dtype=T), orc.dense_cfg(tgt), other.reshape(-1), orc.dense_cfg(oth), e.reshape(-1), orc.dense_cfg(full), workers=8)
            if op in ("add", "subtract", "multiply"): assert_bits(drn.getData(), want, f"{full} {tgt} {op} {d}")
            else: assert_close(drn.getData(), want, f"{full} {tgt} {op} {d}")
    say("broadcast bwd pairs into a drain with gaps", dt)
    full, oth = [1024, 6, 512], [1, 6, 512]
    e = rng.uniform(-1, 1, full).astype(T); other = rng.uniform(-1, 1, oth).astype(T)
    backing = on(device, np.zeros((1024, 2, 1024), dtype=T))
    view = backing[:, 1:2, 256:768]                                     # shape [1024, 1, 512] inside a wider tensor
    device.launch_broadcast("add", 0, view, on(device, other), on(device, e))
    assert _lib.last_path() == "broadcast_backward_vec_pairs", _lib.last_path()
    want = orc.broadcast("add", 0, np.zeros(1024 * 512, dtype=T), orc.dense_cfg([1024, 1, 512]), other.reshape(-1), orc.dense_cfg(oth), e.reshape(-1), orc.dense_cfg(full), workers=8)
    got = backing.getData().reshape(1024, 2, 1024)
    assert_bits(got[:, 1, 256:768].reshape(-1), want, "drain view")
    assert (got[:, 0, :] == 0).all() and (got[:, 1, :256] == 0).all() and (got[:, 1, 768:] == 0).all()


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_broadcast_backward_vector_path_and_views(device, orc, dt):
    """Drains whose last axis is kept and a multiple of the vector width (16-byte accesses, several drain
    elements per thread), one and two reduced axes, sources of the operands' own shapes as autograd passes
    them, and a strided view as the error: all bit-identical to the CPU state machine."""
    rng = np.random.default_rng(23)
    full = [9, 21, 16]
    e = rng.uniform(-1, 1, full).astype(F[dt])
    te = on(device, e)
    for tgt, oth in (([9, 1, 16], full), ([1, 21, 16], full), ([1, 1, 16], full), ([9, 21, 1], full), ([9, 21, 16], full),
                     ([9, 1, 16], [1, 21, 16]), ([1, 21, 16], [9, 1, 16]), ([1, 1, 16], [9, 21, 16]), ([9, 1, 1], [1, 21, 16])):
        for op in ("add", "subtract", "multiply"):
            for d in (0, 1):
                say("broadcast bwd vec", tgt, oth, op, d, dt)
                other = rng.uniform(-1, 1, oth).astype(F[dt])
                tother = on(device, other)
                drn = Tensor._on_device(device, F[dt], tgt)
                device.launch_broadcast(op, d, drn, tother, te)
                assert _lib.last_path() == ("broadcast_backward_vec" if tgt[2] == 16 else "broadcast_backward")
                want = orc.broadcast(op, d, np.zeros(drn.size, dtype=F[dt]), orc.dense_cfg(tgt), other.reshape(-1), orc.dense_cfg(oth), e.reshape(-1), orc.dense_cfg(full))
                assert_bits(drn.getData(), want, f"{tgt} {oth} {op} {d}")
    say("broadcast bwd with a sliced error", dt)
    big = rng.uniform(-1, 1, (18, 21, 33)).astype(F[dt])
    view = on(device, big)[::2, :, 1:33:2]                       # shape [9, 21, 16], strides (2*21*33, 33, 2)
    for tgt in ([9, 1, 16], [1, 1, 16], [1, 21, 1]):
        other = np.zeros(full, dtype=F[dt])
        drn = Tensor._on_device(device, F[dt], tgt)
        device.launch_broadcast("add", 0, drn, on(device, other), view)
        assert _lib.last_path() == "broadcast_backward"
        want = orc.broadcast("add", 0, np.zeros(drn.size, dtype=F[dt]), orc.dense_cfg(tgt), other.reshape(-1), orc.dense_cfg(full), big.reshape(-1), cfg(view))
        assert_bits(drn.getData(), want, f"sliced error {tgt}")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_random_broadcast_gradients_through_every_plan(device, orc, dt):
    """Random ranks, shapes, reduced axes, operators and derivative indices; the other operand in the full shape, in
    its own shape (extent 1 where the drain keeps an axis) or virtual; the error sometimes a slice of a larger
    tensor.  Small integers make every order of the sums exact, so whichever kernel the planner picks -- a thread
    per element, vectors, split sums along or across the rows -- must equal the oracle bit for bit."""
    T = F[dt]
    rng = np.random.default_rng(47)
    seen = set()
    for case in range(120):
        rank = int(rng.integers(1, 5))
        big = case % 3 == 0                                # long sums: the split kernels
        full = [int(rng.choice([1, 2, 3, 5, 8, 16, 31, 64] if not big else [1, 4, 20, 33, 64, 130, 512])) for _ in range(rank)]
        while int(np.prod(full)) > 300000:
            full[int(np.argmax(full))] //= 2
        tgt = [s if rng.random() < 0.5 else 1 for s in full]
        style = str(rng.choice(["full", "own", "virtual"]))
        if style == "own":
            oth = [s if t == 1 else 1 for s, t in zip(full, tgt)]
            if all(o == 1 for o in oth) and int(np.prod(full)) > 1:
                style, oth = "full", list(full)
        else:
            oth = list(full)
        op = str(rng.choice(["add", "subtract", "multiply"]))
        d = int(rng.integers(0, 2))
        sliced = rng.random() < 0.3
        say("random broadcast gradient", case, full, tgt, oth, style, op, d, "sliced error" if sliced else "", dt)
        if sliced:
            parent = rng.integers(-3, 4, [s + 3 for s in full]).astype(T)
            te = on(device, parent)[tuple(slice(2, 2 + s) for s in full)]
            e_data, e_cfg = parent.reshape(-1), cfg(te)
        else:
            e = rng.integers(-3, 4, full).astype(T)
            te, e_data, e_cfg = on(device, e), e.reshape(-1), orc.dense_cfg(full)
        if style == "virtual":
            other = np.full(oth, 2, dtype=T)
            tother = Tensor.of(T, oth, 2.0).to(device)
        else:
            other = rng.integers(-3, 4, oth).astype(T)
            tother = on(device, other)
        drn = Tensor._on_device(device, T, tgt)
        device.launch_broadcast(op, d, drn, tother, te)
        seen.add(_lib.last_path())
        want = orc.broadcast(op, d, np.zeros(drn.size, dtype=T), orc.dense_cfg(tgt), other.reshape(-1), orc.dense_cfg(oth), e_data, e_cfg)
        assert_bits(drn.getData(), want, f"case {case} {full} -> {tgt}, other {oth} ({style}), {op} d={d} on {_lib.last_path()}")
    say("plans seen", sorted(seen))
    assert {"broadcast_backward", "broadcast_backward_vec", "broadcast_backward_split_vec",
            "broadcast_backward_split_rows", "broadcast_backward_split_rows_vec"} <= seen, sorted(seen)


def test_broadcast_autograd_golden(device, golden):
    g = golden["broadcast_autograd"]
    for row in g["rows"]:
        for dt in (np.float64, np.float32):
            say("golden broadcast autograd", row, dt.__name__)
            a = Tensor.of(dt, g["a"]["shape"], g["a"]["data"]).setRqsGradient(row["which_grad"] == "a").to(device)
            b = Tensor.of(dt, row["b_shape"], g["b_range"]).setRqsGradient(row["which_grad"] == "b").to(device)
            c = {"a+b": lambda: a + b, "a*b": lambda: a * b, "a-b": lambda: a - b, "b-a": lambda: b - a}[row["op"]]()
            assert c.items.tolist() == [float(v) for v in row["c"]]
            c.backward(Tensor.of(dt, [2, 2], g["error"]))
            w = a if row["which_grad"] == "a" else b
            assert w.gradient.items.tolist() == [float(v) for v in row["gradient"]], row


# ---- fused expressions -----------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_fused_chain_equals_unfused_and_oracle(device, orc, dt):
    """tanh(sig(a)*b+c): the fused kernel, the four-kernel sequence the reference runs, and the oracle.
    Contiguous operands, a permuted view and a strided slice."""
    rng = np.random.default_rng(31)
    R, Cc = 96, 200
    fn = Function.of("tanh(sig(I[0])*I[1]+I[2])")
    fused = device.optimizedFunctionOf(fn, "chain")
    bases = [rng.standard_normal((R, Cc)).astype(F[dt]) for _ in range(3)]
    tens = [on(device, b) for b in bases]
    for name, view in (("contiguous", lambda t: t), ("permuted", lambda t: t.T()), ("sliced", lambda t: t[::2, 1:101])):
        say("fused chain", name, dt)
        vs = [view(t) for t in tens]
        got_fused = fused(*vs)
        path = _lib.last_path()
        got_unfused = fn(*vs)
        n = vs[0].size
        oc = orc.dense_cfg(list(vs[0].shape))
        s = orc.activation("sig", -1, np.zeros(n, dtype=F[dt]), oc, bases[0].reshape(-1), cfg(vs[0]))
        m = orc.elementwise("multiply", -1, np.zeros(n, dtype=F[dt]), oc, s, oc, bases[1].reshape(-1), cfg(vs[1]))
        p = orc.elementwise("add", -1, np.zeros(n, dtype=F[dt]), oc, m, oc, bases[2].reshape(-1), cfg(vs[2]))
        want = orc.activation("tanh", -1, np.zeros(n, dtype=F[dt]), oc, p, oc)
        # each kernel is within rtol of the reference's kernel; through the chain the rounding of sig(a)*b
        # is amplified where it cancels against c, so the end-to-end bound is norm-wise: rtol * (|sig(a)*b| + |c|)
        cview = bases[2].reshape(-1)[physical_indices(vs[2].ndc)]
        bound = RTOL[np.dtype(F[dt])] * (np.abs(m) + np.abs(cview) + np.abs(want)) + ATOL[np.dtype(F[dt])]
        assert (np.abs(got_fused.items - want) <= bound).all(), f"fused {name}"
        assert (np.abs(got_unfused.items - want) <= bound).all(), f"unfused {name}"
        assert_bits(got_fused.items, got_unfused.items, f"fused vs unfused {name}")   # same roundings, same kernels' maths
        assert path.startswith({"contiguous": "rows", "permuted": "tile_transpose", "sliced": "rows"}[name]), path
    # nested right operands exercise the saved-intermediate stack of the fused program
    say("fused nested", dt)
    f2 = Function.of("(I[0]*I[1]) + (I[1]-I[2]) * (I[2] / (I[0]*I[0] + 2))")
    assert_bits(device.optimizedFunctionOf(f2, "nested")(*tens).items, f2(*tens).items, "nested")
    if dt == "f64":
        x, y, z = bases
        assert_close(f2(*tens).items, ((x * y) + (y - z) * (z / (x * x + 2))).reshape(-1), "nested vs numpy")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_fused_functions_beyond_one_launch(device, dt):
    """Expressions with more than 6 inputs, 32 op-codes, 8 constants or 4 waiting intermediates run as several launches
    through temporaries:
    the same bits as the unfused graph for + - * (every intermediate is rounded to the element type either way), no
    buffer left behind, and derivatives -- far larger trees than the functions themselves -- through the same staging,
    against central differences in f64."""
    T = F[dt]
    rng = np.random.default_rng(34)
    shape = (33, 40)
    exprs = ["relu(I[0]*I[1]+I[2])*quad(I[3]-I[4])+abs(I[5]*I[6])-I[7]*I[8]+I[9]",
             "+".join(f"quad(I[{k % 3}]*{k + 1}.5-I[{(k + 1) % 3}])" for k in range(14)),
             "I[0]" + "".join(f"{'+-'[k % 2]}(I[1]*{k}.25)" for k in range(40)),
             # 27 op-codes, 6 inputs, 8 stack entries, but six products wait for the seventh
             "I[0]*I[1]+(I[1]*I[2]+(I[2]*I[3]+(I[3]*I[4]+(I[4]*I[5]+(I[5]*I[0]+I[0]*I[2])))))"]
    for expr in exprs:
        say("fused beyond one launch", dt, expr[:60])
        fn = Function.of(expr)
        fused = device.optimizedFunctionOf(fn, "big")
        assert len(fused.stages) > 1
        arrays = [rng.uniform(-1.5, 1.5, shape).astype(T) for _ in range(fn.numberOfArgs())]
        ts = [on(device, a) for a in arrays]
        got = None                                                     # (drop the result of the expression before)
        gc.collect()
        before = device.liveBuffers()
        got = fused(*ts)
        gc.collect()
        assert device.liveBuffers() == before + 1                      # the temporaries are gone
        assert_bits(got.items, fn(*ts).items, "fused in stages vs unfused")
    say("derivatives of a large smooth function", dt)
    expr = "tanh(sig(I[0])*I[1]+I[2])*sin(I[3]*I[0])+exp(I[1]*0.25)*cos(I[2]-I[3])+softplus(I[0]*I[2])*gaus(I[1])"
    fn = Function.of(expr)
    fused = device.optimizedFunctionOf(fn, "smooth")
    arrays = [rng.uniform(0.5, 1.5, shape).astype(T) for _ in range(4)]
    ts = [on(device, a) for a in arrays]
    assert any(len(fused.derivative_stages(i)) > 1 for i in range(4))
    e = rng.uniform(-1, 1, shape).astype(T)
    grads = []
    for runner in (fused, fn):
        gs = [on(device, a).setRqsGradient(True) for a in arrays]
        runner(*gs).backward(on(device, e))
        grads.append([t.gradient.items for t in gs])
    for i in range(4):
        scale = np.abs(grads[1][i]) + np.abs(e.reshape(-1))
        assert (np.abs(grads[0][i] - grads[1][i]) <= 50 * RTOL[np.dtype(T)] * scale + ATOL[np.dtype(T)]).all(), i
    if dt == "f64":
        for i in range(4):
            h = 1e-6
            up, dn = [a.copy() for a in arrays], [a.copy() for a in arrays]
            up[i] += h; dn[i] -= h
            numeric = (fused(*[on(device, a) for a in up]).items - fused(*[on(device, a) for a in dn]).items) / (2 * h)
            got = fused.derive(ts, i).items
            assert (np.abs(got - numeric) <= 1e-6 * np.maximum(1.0, np.abs(numeric))).all(), i


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_fused_derivative_kernels_and_autograd(device, orc, dt):
    """A fused function also carries one kernel per input for its derivative (CLFunctionCompiler.java:155-157).
    They must agree with the chain rule applied by the unfused graph, and with central differences in f64."""
    rng = np.random.default_rng(33)
    shape = (37, 24)
    arrays = [rng.uniform(0.5, 1.5, shape).astype(F[dt]) for _ in range(3)]
    for expr in ("tanh(sig(I[0])*I[1]+I[2])", "sin(I[0])/cos(I[1])+I[2]*I[2]", "(I[0]+2)**I[1]-exp(I[2])"):
        say("fused derivative", expr, dt)
        fn = Function.of(expr)
        fused = device.optimizedFunctionOf(fn, "f")
        # autograd through the fused kernel against autograd through the unfused graph
        e = rng.uniform(-1, 1, shape).astype(F[dt])
        grads = []
        for runner in (fused, fn):
            ts = [on(device, a).setRqsGradient(True) for a in arrays]
            runner(*ts).backward(on(device, e))
            grads.append([t.gradient.items for t in ts])
        for i in range(3):
            scale = np.abs(grads[1][i]) + np.abs(e.reshape(-1))
            assert (np.abs(grads[0][i] - grads[1][i]) <= 20 * RTOL[np.dtype(F[dt])] * scale + ATOL[np.dtype(F[dt])]).all(), (expr, i)
        if dt == "f64":                                   # and the derivative kernels themselves against central differences
            ts = [on(device, a) for a in arrays]
            for i in range(3):
                h = 1e-6
                up, dn = [a.copy() for a in arrays], [a.copy() for a in arrays]
                up[i] += h; dn[i] -= h
                numeric = (fused(*[on(device, a) for a in up]).items - fused(*[on(device, a) for a in dn]).items) / (2 * h)
                got = fused.derive(ts, i).items
                assert (np.abs(got - numeric) <= 1e-6 * np.maximum(1.0, np.abs(numeric))).all(), (expr, i)


# ---- convolution ----------------------------------------------------------------------------------------------
def test_convolution_golden_on_device(device, golden):
    for row in golden["convolution_forward"]["rows"]:
        for dt in (np.float32, np.float64):
            say("golden conv", row["x_shape"], row["k_shape"], dt.__name__)
            x = Tensor.of(dt, row["x_shape"], row["x"]).to(device)
            k = Tensor.of(dt, row["k_shape"], row["k"]).to(device)
            y = x.conv(k)
            assert list(y.shape) == row["y_shape"] and y.items.tolist() == [float(v) for v in row["y"]], row
            y2 = Function.of("I[0] x I[1]")(x, k)
            assert y2.items.tolist() == [float(v) for v in row["y"]]


def test_convolution_autograd_golden_graph(device, golden):
    g = golden["convolution_autograd"]
    say("golden conv autograd")
    f8 = np.float64
    i_a = Tensor.of(f8, g["i_a"]["shape"], g["i_a"]["data"]).to(device)
    w_a = Tensor.of(f8, g["w_a"]["shape"], g["w_a"]["data"]).setRqsGradient(True).to(device)
    w_b = Tensor.of(f8, g["w_b"]["shape"], g["w_b"]["data"]).setRqsGradient(True).to(device)
    w_c = Tensor.of(f8, g["w_c"]["shape"], g["w_c"]["data"]).setRqsGradient(True).to(device)
    o_a = i_a.conv(w_a); o_b = o_a.conv(w_b); o_c = o_a.conv(w_c)
    out = o_b * o_c
    assert o_a.items.tolist() == g["o_a"] and o_b.items.tolist() == g["o_b"] and o_c.items.tolist() == g["o_c"]
    assert out.items.tolist() == g["out"]
    out.backward(Tensor.of(f8, g["backward_error"]["shape"], g["backward_error"]["value"]))
    assert w_b.gradient.items.tolist() == g["w_b_gradient"]
    w_a.applyGradient()
    assert w_a.items.tolist() == g["w_a_after_apply"]


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_convolution_literal_kernels_bit_exact(device, orc, dt):
    """Any rank, either operand order, dense and viewed operands: the literal kernels keep the reference's
    summation order and are bit-identical to the oracle's state machines."""
    rng = np.random.default_rng(41)
    cases = [([9], [4]), ([12, 11], [3, 4]), ([3, 4], [12, 11]), ([3, 9, 8], [3, 2, 3]), ([2, 6, 6], [1, 3, 3]),
             ([2, 3, 1], [1, 3, 2]), ([2, 3, 5, 4], [2, 3, 2, 2])]
    for xs, ks in cases:
        say("conv literal", xs, ks, dt)
        ys = [abs(p - q) + 1 for p, q in zip(xs, ks)]
        x = rng.uniform(-1, 1, xs).astype(F[dt]); k = rng.uniform(-1, 1, ks).astype(F[dt]); e = rng.uniform(-1, 1, ys).astype(F[dt])
        tx, tk, te = on(device, x), on(device, k), on(device, e)
        out = Tensor._on_device(device, F[dt], ys)
        device.launch_convolution(-1, out, tx, tk)
        want = orc.convolve(np.zeros(out.size, dtype=F[dt]), orc.dense_cfg(ys), x.reshape(-1), orc.dense_cfg(xs), k.reshape(-1), orc.dense_cfg(ks))
        if _lib.last_path().startswith("literal"):
            assert_bits(out.getData(), want, f"fwd {xs} {ks}")
        elif _lib.last_path() in ("simple2d", "simple2d_window"):        # what the reference hands to SimpleCPUConvolution: its order, bit for bit
            img, tap, ishape, tshape = (x, k, xs, ks) if xs[-1] >= ks[-1] else (k, x, ks, xs)
            assert len(xs) == 2 or tshape[0] == 1
            simple = orc.simple_conv2d(img.reshape(-1), tap.reshape(-1), ishape[-1], ishape[-2], tshape[-1], tshape[-2], batch=ishape[0] if len(xs) == 3 else 1)
            assert_bits(out.getData(), simple, f"fwd simple {xs} {ks}")
            np.testing.assert_allclose(out.getData(), want, rtol=1e-5 if dt == "f32" else 1e-12, atol=1e-5 if dt == "f32" else 1e-12)
        else:       # dense [C,H,W] x [C,kh,kw] takes the channel kernel: same sums in another order
            assert len(xs) == 3
            np.testing.assert_allclose(out.getData(), want, rtol=1e-5 if dt == "f32" else 1e-12, atol=1e-5 if dt == "f32" else 1e-12)
        for tgt, tgt_shape, other, other_arr, other_shape in ((tx, xs, tk, k, ks), (tk, ks, tx, x, xs)):
            drn = Tensor._on_device(device, F[dt], tgt_shape)
            device.launch_convolution(0, drn, other, te)
            want = orc.deconvolve(np.zeros(drn.size, dtype=F[dt]), orc.dense_cfg(tgt_shape), other_arr.reshape(-1), orc.dense_cfg(other_shape), e.reshape(-1), orc.dense_cfg(ys))
            if _lib.last_path().startswith("literal"):
                assert_bits(drn.getData(), want, f"bwd {tgt_shape} {other_shape}")
            else:       # ... and so do its gradients, and those of a batch of images under one set of taps
                assert len(xs) == 3
                np.testing.assert_allclose(drn.getData(), want, rtol=1e-5 if dt == "f32" else 1e-12, atol=1e-5 if dt == "f32" else 1e-12)
    say("conv literal on a transposed operand", dt)
    x = rng.uniform(-1, 1, (8, 10)).astype(F[dt]); k = rng.uniform(-1, 1, (3, 3)).astype(F[dt])
    tx, tk = on(device, x), on(device, k)
    vx = tx.T()
    out = Tensor._on_device(device, F[dt], [8, 6])
    device.launch_convolution(-1, out, vx, tk)
    want = orc.convolve(np.zeros(48, dtype=F[dt]), orc.dense_cfg([8, 6]), x.reshape(-1), cfg(vx), k.reshape(-1), orc.dense_cfg([3, 3]))
    assert_bits(out.getData(), want, "transposed operand")


def _abs_bound(orc, xs, ks, x, k, dt):
    ys = [abs(p - q) + 1 for p, q in zip(xs, ks)]
    return orc.convolve(np.zeros(int(np.prod(ys))), orc.dense_cfg(ys), np.abs(x).astype(np.float64).reshape(-1), orc.dense_cfg(xs),
                        np.abs(k).astype(np.float64).reshape(-1), orc.dense_cfg(ks))


@pytest.mark.parametrize("shape", [([8, 40, 70], [8, 5, 5]), ([6, 33, 65], [6, 3, 3]), ([5, 20, 21], [5, 4, 2]), ([64, 64, 64], [64, 5, 5]),
                                   ([3, 130, 200], [3, 7, 7]), ([9, 17, 300], [9, 2, 2]), ([2, 12, 12], [2, 4, 4]),
                                   ([3, 10, 71], [3, 3, 3]), ([5, 9, 302], [5, 2, 2]), ([70, 30, 261], [70, 5, 5]),
                                   ([16, 520, 1030], [16, 3, 3]), ([16, 300, 1100], [16, 7, 7]),
                                   # planes that give about one (rows x 64 columns) tile per compute unit: every block reduces all
                                   # channels of its tile (4-row and 8-row tiles, ragged edges, channel counts that leave wavefronts idle)
                                   ([20, 130, 520], [20, 3, 3]), ([17, 200, 700], [17, 5, 5]), ([33, 140, 500], [33, 7, 7]),
                                   ([16, 130, 520], [16, 2, 2]), ([19, 131, 517], [19, 4, 4])])
@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_channel_convolution_fast_paths(device, orc, shape, dt):
    """[C,H,W] x [C,kh,kw] forward and both gradients on the register-window kernels: re-ordered sums, compared
    norm-wise: |delta| <= tol * sum|a||b| per output (tol 1e-5 in f32, 1e-12 in f64).  Covers ragged widths, several
    column blocks per row, taps that reach two lanes to the side, and planes large enough for the forward blocks
    that reduce all channels themselves."""
    xs, ks = shape
    T = F[dt]
    tol = RTOL[np.dtype(T)]
    ys = [1, xs[1] - ks[1] + 1, xs[2] - ks[2] + 1]
    rng = np.random.default_rng(43)
    x = (rng.standard_normal(xs) * 0.1).astype(T); k = (rng.standard_normal(ks) * 0.1).astype(T)
    e = rng.standard_normal(ys).astype(T)
    tx, tk, te = on(device, x), on(device, k), on(device, e)
    square = ks[1] == ks[2]          # the register-window kernels exist for square taps of extent 2, 3, 4, 5, 7
    # other tap shapes take the general kernels: one thread per element, or (sums of 128 terms and more into few elements) split sums
    fwd, dxp, dkp = ("chan_fwd", "chan_dx", "chan_dk") if square else ("literal_fwd", "literal_bwd", "split_bwd")
    if xs[2] >= 500 and xs[1] <= 200:
        fwd = "chan_fwd_tiles"
    say("chan_fwd", xs, ks, dt)
    out = Tensor._on_device(device, T, ys)
    device.launch_convolution(-1, out, tx, tk)
    assert _lib.last_path() == fwd
    want = orc.convolve(np.zeros(out.size, dtype=T), orc.dense_cfg(ys), x.reshape(-1), orc.dense_cfg(xs), k.reshape(-1), orc.dense_cfg(ks))
    bound = tol * _abs_bound(orc, xs, ks, x, k, T) + 1e-30
    assert (np.abs(out.getData().astype(np.float64) - want) <= bound).all(), "chan_fwd"
    out2 = Tensor._on_device(device, T, ys)
    device.launch_convolution(-1, out2, tk, tx)                       # kernel first
    assert _lib.last_path() == fwd
    assert_bits(out2.getData(), out.getData(), "operand order")
    say("chan_dx", xs, ks, dt)
    dx = Tensor._on_device(device, T, xs)
    device.launch_convolution(0, dx, tk, te)
    assert _lib.last_path() == dxp
    want = orc.deconvolve(np.zeros(dx.size, dtype=T), orc.dense_cfg(xs), k.reshape(-1), orc.dense_cfg(ks), e.reshape(-1), orc.dense_cfg(ys), fast=True)
    babs = orc.deconvolve(np.zeros(dx.size), orc.dense_cfg(xs), np.abs(k).astype(np.float64).reshape(-1), orc.dense_cfg(ks), np.abs(e).astype(np.float64).reshape(-1), orc.dense_cfg(ys), fast=True)
    assert (np.abs(dx.getData().astype(np.float64) - want) <= tol * babs + 1e-30).all(), "chan_dx"
    say("chan_dk", xs, ks, dt)
    dk = Tensor._on_device(device, T, ks)
    device.launch_convolution(0, dk, tx, te)
    assert _lib.last_path() == dkp
    want = orc.deconvolve(np.zeros(dk.size, dtype=T), orc.dense_cfg(ks), x.reshape(-1), orc.dense_cfg(xs), e.reshape(-1), orc.dense_cfg(ys), fast=True)
    babs = orc.deconvolve(np.zeros(dk.size), orc.dense_cfg(ks), np.abs(x).astype(np.float64).reshape(-1), orc.dense_cfg(xs), np.abs(e).astype(np.float64).reshape(-1), orc.dense_cfg(ys), fast=True)
    assert (np.abs(dk.getData().astype(np.float64) - want) <= tol * babs + 1e-30).all(), "chan_dk"


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("shape", [([48, 40, 44], [48, 5, 5]), ([200, 20, 21], [200, 4, 2]), ([4, 60, 70], [4, 4, 2]),
                                   ([80, 90], [40, 45]), ([30, 1100, 1], [1, 1100, 20]), ([2, 3, 44, 34], [2, 3, 6, 5]),
                                   ([300, 310], [5, 5]), ([3, 8, 20, 20], [1, 8, 5, 5]), ([6, 40, 40], [1, 3, 3])])
def test_convolution_split_sums(device, orc, shape, dt):
    """Few drain elements with sums of 1024 terms or more: a block per element adds the reference's terms in another
    order.  Norm-wise |delta| <= tol * sum|a||b| per output (tol 1e-5 / 1e-12), exact on integer-valued data; every
    rank, both gradient branches, and a transposed operand."""
    xs, ks = shape
    T = F[dt]
    tol = 1e-5 if dt == "f32" else 1e-12
    ys = [abs(p - q) + 1 for p, q in zip(xs, ks)]
    rng = np.random.default_rng(44)
    seen = set()
    for integer in (True, False):
        draw = (lambda sh: rng.integers(-3, 4, sh).astype(T)) if integer else (lambda sh: rng.uniform(-1, 1, sh).astype(T))
        x, k, e = draw(xs), draw(ks), draw(ys)
        tx, tk, te = on(device, x), on(device, k), on(device, e)
        say("conv split fwd", xs, ks, dt, "integer" if integer else "uniform")
        out = Tensor._on_device(device, T, ys)
        device.launch_convolution(-1, out, tx, tk)
        seen.add(_lib.last_path())
        want = orc.convolve(np.zeros(out.size, dtype=T), orc.dense_cfg(ys), x.reshape(-1), orc.dense_cfg(xs), k.reshape(-1), orc.dense_cfg(ks))
        if integer:
            assert_bits(out.getData(), want, "fwd on integers")
        else:
            assert (np.abs(out.getData().astype(np.float64) - want) <= tol * _abs_bound(orc, xs, ks, x, k, T) + 1e-30).all()
        for name, tgt_shape, other, other_arr, other_shape in (("dx", xs, tk, k, ks), ("dk", ks, tx, x, xs)):
            say("conv split", name, xs, ks, dt)
            drn = Tensor._on_device(device, T, tgt_shape)
            device.launch_convolution(0, drn, other, te)
            seen.add(_lib.last_path())
            want = orc.deconvolve(np.zeros(drn.size, dtype=T), orc.dense_cfg(tgt_shape), other_arr.reshape(-1), orc.dense_cfg(other_shape), e.reshape(-1), orc.dense_cfg(ys), fast=True)
            if integer:
                assert_bits(drn.getData(), want, name + " on integers")
            else:
                babs = orc.deconvolve(np.zeros(drn.size), orc.dense_cfg(tgt_shape), np.abs(other_arr).astype(np.float64).reshape(-1), orc.dense_cfg(other_shape),
                                      np.abs(e).astype(np.float64).reshape(-1), orc.dense_cfg(ys), fast=True)
                assert (np.abs(drn.getData().astype(np.float64) - want) <= tol * babs + 1e-30).all(), name
    if ks == [48, 5, 5]:
        assert seen == {"chan_fwd", "chan_dx", "chan_dk"}, seen          # the register-window kernels take dense square taps
    elif ks == [5, 5]:                                                   # ... and a 2-D image as their one-channel case
        assert seen == {"simple2d_window", "chan_dx", "chan_dk"}, seen
    elif ks == [1, 3, 3]:                                                # ... and a batch of images under one set of taps
        assert seen == {"simple2d", "chan_dx", "chan_dk"}, seen
    else:
        assert seen & {"split_fwd", "split_bwd"}, seen
    if len(xs) == 2:
        say("conv split on a transposed operand", dt)
        x = rng.integers(-3, 4, (xs[1], xs[0])).astype(T)
        vx = on(device, x).T()                                         # shape xs, strides (1, xs[0])
        e = rng.integers(-3, 4, ys).astype(T)
        dk = Tensor._on_device(device, T, ks)
        device.launch_convolution(0, dk, vx, on(device, e))
        assert _lib.last_path() == "split_bwd"
        want = orc.deconvolve(np.zeros(dk.size, dtype=T), orc.dense_cfg(ks), x.reshape(-1), cfg(vx), e.reshape(-1), orc.dense_cfg(ys))
        assert_bits(dk.getData(), want, "transposed operand")


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("shape", [([6, 40, 300], [1, 5, 5]), ([3, 33, 65], [1, 3, 3]), ([40, 70, 70], [1, 7, 7]), ([2, 9, 520], [1, 2, 2]),
                                   ([130, 12, 12], [1, 4, 4])])
def test_batched_image_gradients_on_the_channel_kernels(device, orc, shape, dt):
    """[B,H,W] x [1,k,k]: the error has one plane per image.  The input gradient convolves every image's plane with the
    one set of taps, the tap gradient also sums over the images: exact on integer-valued data, norm-wise otherwise."""
    xs, ks = shape
    T = F[dt]
    tol = RTOL[np.dtype(T)]
    ys = [xs[0], xs[1] - ks[1] + 1, xs[2] - ks[2] + 1]
    rng = np.random.default_rng(49)
    for integer in (True, False):
        draw = (lambda sh: rng.integers(-3, 4, sh).astype(T)) if integer else (lambda sh: rng.uniform(-1, 1, sh).astype(T))
        x, k, e = draw(xs), draw(ks), draw(ys)
        tx, tk, te = on(device, x), on(device, k), on(device, e)
        for name, tgt_shape, other, other_arr, other_shape in (("dx", xs, tk, k, ks), ("dk", ks, tx, x, xs)):
            say("batched conv gradient", name, xs, ks, dt, "integer" if integer else "uniform")
            drn = Tensor._on_device(device, T, tgt_shape)
            device.launch_convolution(0, drn, other, te)
            assert _lib.last_path() == "chan_" + name, _lib.last_path()
            want = orc.deconvolve(np.zeros(drn.size, dtype=T), orc.dense_cfg(tgt_shape), other_arr.reshape(-1), orc.dense_cfg(other_shape), e.reshape(-1), orc.dense_cfg(ys), fast=True)
            if integer:
                assert_bits(drn.getData(), want, name + " on integers")
            else:
                babs = orc.deconvolve(np.zeros(drn.size), orc.dense_cfg(tgt_shape), np.abs(other_arr).astype(np.float64).reshape(-1), orc.dense_cfg(other_shape),
                                      np.abs(e).astype(np.float64).reshape(-1), orc.dense_cfg(ys), fast=True)
                assert (np.abs(drn.getData().astype(np.float64) - want) <= tol * babs + 1e-30).all(), name


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_random_convolutions_through_every_plan(device, orc, dt):
    """Random shapes of rank 1 to 4 (every axis either slides, in either operand, or is reduced), biased towards the
    shapes the specialised kernels take and towards their edges (widths around a wavefront's 256 columns, heights
    that are no multiple of a strip, channel counts that are no multiple of a group), sometimes through a transposed
    or sliced operand.  The data are small integers, so every order of the sums is exact: forward and both gradients
    must equal the oracle's state machines bit for bit on whichever kernel the planner picks."""
    T = F[dt]
    rng = np.random.default_rng(46)
    seen = set()

    def operand(shape, view):
        """A device tensor of the given shape and (its parent's data, its descriptor) for the oracle."""
        if view == "transposed" and len(shape) >= 2:
            parent = rng.integers(-3, 4, shape[:-2] + [shape[-1], shape[-2]]).astype(T)
            axes = list(range(len(shape) - 2)) + [len(shape) - 1, len(shape) - 2]
            t = on(device, parent).permute(*axes)
        elif view == "sliced":
            parent = rng.integers(-3, 4, [s + 2 for s in shape]).astype(T)
            t = on(device, parent)[tuple(slice(1, 1 + s) for s in shape)]
        else:
            parent = rng.integers(-3, 4, shape).astype(T)
            t = on(device, parent)
        assert list(t.shape) == list(shape)
        return t, parent.reshape(-1), cfg(t)

    for case in range(70):
        kind = ("channels", "image", "any")[case % 3]
        if kind == "channels":          # [C,H,W] x [C,k,k]
            c = int(rng.choice([2, 3, 5, 8, 13, 16, 33]))
            kk = int(rng.choice([2, 3, 4, 5, 7, 6, 1]))
            h = int(rng.integers(kk, 40)); w = int(rng.choice([kk, 17, 64, 255, 256, 257, 258, 259, 263, 300, 515]))
            w = max(w, kk)
            xs, ks = [c, h, w], [c, kk, kk if rng.random() < 0.85 else max(1, kk - 1)]
        elif kind == "image":           # [H,W] x [k,k] and [B,H,W] x [1,k,k]
            kk = int(rng.choice([2, 3, 4, 5, 7]))
            h = int(rng.choice([kk, 9, 64, 200, 270])); w = int(rng.choice([kk, 33, 257, 300, 520]))
            xs, ks = [h, w], [kk, kk]
            if rng.random() < 0.4:
                xs, ks = [int(rng.integers(1, 4))] + xs, [1] + ks
        else:
            rank = int(rng.integers(1, 5))
            xs, ks = [], []
            for _ in range(rank):
                a, b = int(rng.integers(1, 12)), int(rng.integers(1, 12))
                mode = rng.random()
                if mode < 0.3: b = a                      # reduced axis
                elif mode < 0.7: a, b = max(a, b), min(a, b)
                xs.append(a); ks.append(b)
        ys = [abs(p - q) + 1 for p, q in zip(xs, ks)]
        views = [str(rng.choice(["dense", "dense", "transposed", "sliced"])) for _ in range(3)]
        say("random convolution", case, kind, xs, ks, views, dt)
        (tx, dx_, cx), (tk, dk_, ck), (te, de_, ce) = operand(xs, views[0]), operand(ks, views[1]), operand(ys, views[2])
        out = Tensor._on_device(device, T, ys)
        if rng.random() < 0.5:
            device.launch_convolution(-1, out, tx, tk)
            want = orc.convolve(np.zeros(out.size, dtype=T), orc.dense_cfg(ys), dx_, cx, dk_, ck)
        else:                                             # taps first
            device.launch_convolution(-1, out, tk, tx)
            want = orc.convolve(np.zeros(out.size, dtype=T), orc.dense_cfg(ys), dk_, ck, dx_, cx)
        seen.add(_lib.last_path())
        assert_bits(out.getData(), want, f"case {case} forward {xs} x {ks} {views} on {_lib.last_path()}")
        for name, tgt_shape, other, other_data, other_cfg in (("dx", xs, tk, dk_, ck), ("dk", ks, tx, dx_, cx)):
            drn = Tensor._on_device(device, T, tgt_shape)
            device.launch_convolution(0, drn, other, te)
            seen.add(_lib.last_path())
            want = orc.deconvolve(np.zeros(drn.size, dtype=T), orc.dense_cfg(tgt_shape), other_data, other_cfg, de_, ce, fast=True)
            assert_bits(drn.getData(), want, f"case {case} {name} {xs} x {ks} {views} on {_lib.last_path()}")
    say("plans seen", sorted(seen))
    want_plans = {"literal_fwd", "literal_bwd", "simple2d", "chan_fwd", "chan_dx", "chan_dk", "simple2d_window"}
    assert want_plans <= seen, (sorted(want_plans - seen), sorted(seen))


@pytest.mark.parametrize("shape", [([300, 523], [5, 5]), ([3, 200, 300], [1, 3, 3]), ([130, 700], [7, 7]), ([260, 257], [2, 2]), ([2, 190, 261], [1, 4, 4])])
@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_conv2d_large_images_bit_exact(device, orc, shape, dt):
    """Large images with square taps take the register-window kernel: the same products, rounded and added in
    SimpleCPUConvolution's order (ky outer, kx inner) -- bit for bit, in f32 and f64."""
    xs, ks = shape
    rng = np.random.default_rng(45)
    x = rng.uniform(-1, 1, xs).astype(F[dt]); k = rng.uniform(-1, 1, ks).astype(F[dt])
    say("conv2d window", xs, ks, dt)
    y = on(device, x).conv(on(device, k))
    assert _lib.last_path() == "simple2d_window", _lib.last_path()
    B = xs[0] if len(xs) == 3 else 1
    want = orc.simple_conv2d(x.reshape(-1), k.reshape(-1), xs[-1], xs[-2], ks[-1], ks[-2], batch=B)
    assert_bits(y.items, want, f"{xs} x {ks}")
    y2 = on(device, k).conv(on(device, x))                        # taps first
    assert_bits(y2.items, want, "operand order")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_conv1d_long_vectors_bit_exact(device, orc, dt):
    """Dense vectors with at least 4096 outputs and 2 to 4096 taps take the 1-D kernel (inputs staged in LDS, sums tap
    by tap in the reference's order): bit for bit the oracle's general state machine, either operand order; shorter
    vectors, longer tap sets and views keep the general kernel -- and agree with it too."""
    T = F[dt]
    rng = np.random.default_rng(48)
    for n, k, path in ((5000, 2, "simple1d"), (70001, 64, "simple1d"), (4096 + 4095, 4096, "simple1d"), (100000, 333, "simple1d"),
                       (4000, 64, "literal_fwd"), (9000, 5000, None), (70001, 1, "literal_fwd")):
        say("conv1d", n, k, dt)
        if path is None:        # whichever general kernel takes it (sums may be split): integer data, exact in any order
            x = rng.integers(-3, 4, n).astype(T); w = rng.integers(-3, 4, k).astype(T)
        else:
            x = rng.uniform(-1, 1, n).astype(T); w = rng.uniform(-1, 1, k).astype(T)
        want = orc.convolve(np.zeros(n - k + 1, dtype=T), orc.dense_cfg([n - k + 1]), x, orc.dense_cfg([n]), w, orc.dense_cfg([k]))
        for first, second in ((x, w), (w, x)):
            out = Tensor._on_device(device, T, [n - k + 1])
            device.launch_convolution(-1, out, on(device, first), on(device, second))
            if path is not None:
                assert _lib.last_path() == path, (_lib.last_path(), n, k)
            assert_bits(out.getData(), want, f"conv1d {n} {k}")
    for n, k in ((5000, 2), (70001, 64), (8200, 4096), (100000, 333)):
        say("conv1d gradient by the long operand", n, k, dt)
        w = rng.uniform(-1, 1, k).astype(T); e = rng.uniform(-1, 1, n - k + 1).astype(T)
        w[0] = np.inf if k == 64 else w[0]                       # an infinite tap must not meet entries outside the error
        dx = Tensor._on_device(device, T, [n])
        device.launch_convolution(0, dx, on(device, w), on(device, e))
        assert _lib.last_path() == "simple1d_grad", _lib.last_path()
        with np.errstate(all="ignore"):
            want = orc.deconvolve(np.zeros(n, dtype=T), orc.dense_cfg([n]), w, orc.dense_cfg([k]), e, orc.dense_cfg([n - k + 1]), fast=True)
        assert_bits(dx.getData(), want, f"conv1d dx {n} {k}")
    tol = 1e-5 if dt == "f32" else 1e-12
    for n, k in ((5000, 2), (70001, 64), (8200, 4096), (100000, 333)):
        for integer in (True, False):
            say("conv1d gradient by the taps", n, k, dt, "integer" if integer else "uniform")
            x = (rng.integers(-3, 4, n) if integer else rng.uniform(-1, 1, n)).astype(T)
            e = (rng.integers(-3, 4, n - k + 1) if integer else rng.uniform(-1, 1, n - k + 1)).astype(T)
            dk = Tensor._on_device(device, T, [k])
            device.launch_convolution(0, dk, on(device, x), on(device, e))
            assert _lib.last_path() == "simple1d_grad_taps", _lib.last_path()
            want = orc.deconvolve(np.zeros(k, dtype=T), orc.dense_cfg([k]), x, orc.dense_cfg([n]), e, orc.dense_cfg([n - k + 1]), fast=True)
            if integer:
                assert_bits(dk.getData(), want, f"conv1d dk {n} {k}")
            else:       # the same terms in another order: bounded by the sum of their magnitudes
                mag = orc.deconvolve(np.zeros(k), orc.dense_cfg([k]), np.abs(x).astype(np.float64), orc.dense_cfg([n]),
                                     np.abs(e).astype(np.float64), orc.dense_cfg([n - k + 1]), fast=True)
                assert (np.abs(dk.getData().astype(np.float64) - want) <= tol * mag + 1e-30).all()
    say("conv1d on a strided view stays general", dt)
    big = rng.uniform(-1, 1, 20000).astype(T); w = rng.uniform(-1, 1, 9).astype(T)
    view = on(device, big)[::2]
    out = Tensor._on_device(device, T, [10000 - 8])
    device.launch_convolution(-1, out, view, on(device, w))
    assert _lib.last_path() == "literal_fwd"
    assert_bits(out.getData(), orc.convolve(np.zeros(9992, dtype=T), orc.dense_cfg([9992]), big, cfg(view), w, orc.dense_cfg([9])), "strided view")


def test_conv2d_config1_shape(device, orc):
    """[64,64] x [3,3] -> [62,62] (the reference runs this on SimpleCPUConvolution: ky outer, kx inner)."""
    say("conv2d 64x64 x 3x3")
    rng = np.random.default_rng(1)
    x = rng.uniform(-1, 1, (64, 64)).astype(np.float32); k = rng.uniform(-1, 1, (3, 3)).astype(np.float32)
    y = on(device, x).conv(on(device, k))
    assert y.shape == (62, 62)
    assert _lib.last_path() == "simple2d"
    want = orc.simple_conv2d(x.reshape(-1), k.reshape(-1), 64, 64, 3, 3)
    assert_bits(y.items, want, "SimpleCPUConvolution order")


# ---- integer scalarization ----------------------------------------------------------------------------------------
INT_OPS = ["add", "subtract", "multiply", "divide", "modulo", "power", "idy"]


@pytest.mark.parametrize("dt", [np.int32, np.int64, np.int16, np.int8])
def test_integer_scalarization_bit_exact(device, orc, golden, dt):
    """drain = src op value on int / long / short / byte data: every operator, the function and both derivatives,
    dense data (16-byte path with a ragged tail) and views, against the oracle's Java arithmetic."""
    rng = np.random.default_rng(81)
    info = np.iinfo(dt)
    n = 4099
    edge = np.array([info.min, info.max, 0, 1, -1, 2, -2, 7, -7, info.min + 1], dtype=dt)
    small = rng.integers(-9, 10, n, dtype=dt)                                  # keeps powers in range
    wide = np.concatenate([edge, rng.integers(info.min, info.max, n - edge.size, dtype=dt, endpoint=True)])
    for op in INT_OPS:
        for d in (-1, 0, 1):
            for value in ((3, -2, 0) if op == "power" else (3, -7, 1, -1, 0, int(info.max), int(info.min))):
                data = small if op == "power" else wide
                if value == 0 and d < 0 and op in ("divide", "modulo") and dt in (np.int32, np.int64):
                    say("int scalarization / by zero", dt.__name__, op)
                    with pytest.raises(Exception, match="by zero"):
                        device.launch_scalarization(op, d, Tensor._on_device(device, dt, (n,)), on(device, data), value)
                    with pytest.raises(orc.JavaArithmeticException):
                        orc.scalarization_int(op, d, np.zeros_like(data), orc.dense_cfg([n]), data, orc.dense_cfg([n]), value)
                    continue
                out = Tensor._on_device(device, dt, (n,))
                device.launch_scalarization(op, d, out, on(device, data), value)
                assert _lib.last_path() == "int_flat"
                want = orc.scalarization_int(op, d, np.zeros_like(data), orc.dense_cfg([n]), data, orc.dense_cfg([n]), value)
                got = out.getData()
                assert (got == want).all(), (dt.__name__, op, d, value, data[got != want][:5], got[got != want][:5], want[got != want][:5])
    say("int scalarization on views", dt.__name__)
    parent = on(device, rng.integers(-100, 100, (40, 66), dtype=dt))
    src = parent[1:39:2, 3:63:3].T()                                           # [20,19] -> transposed [20? ...]
    out_parent = on(device, np.zeros((30, 30), dtype=dt))
    drn = out_parent[2:2 + src.shape[0], 5:5 + src.shape[1]]
    before = out_parent.getData().copy()
    for op, value in (("multiply", 5), ("subtract", -3), ("divide", 4)):
        device.launch_scalarization(op, -1, drn, src, value)
        assert _lib.last_path() == "int_indexed"
        want = orc.scalarization_int(op, -1, before.copy(), cfg(drn), parent.getData(), cfg(src), value)
        assert (out_parent.getData() == want).all(), (dt.__name__, op)
    if dt == np.int32:
        say("recorded (unenforced) integer rows of Tensor_Operation_Spec on the device")
        g = golden["int_scalarization"]
        i0 = on(device, np.array(g["tempeh_i0_recovered"], dtype=np.int32), (2, 3))
        times10 = i0 * 10
        assert (np.abs(times10.items) == np.abs(np.array(g["tempeh_i0_recovered"], dtype=np.int32) * np.int32(10))).all()
        assert (on(device, np.abs(times10.items), (2, 3)) % 3).items.tolist() == g["tempeh_abs_i0_times_10_mod_3"]
    if dt in (np.int32, np.int64):
        s = golden["int_scalarization"]["scalar_broadcast_add"]
        a = on(device, np.array(s["a"], dtype=dt), (3, 2))
        b = on(device, np.array([s["b"]], dtype=dt), (1, 1))
        assert (a + b).items.tolist() == s["c"]                                   # 'Scalar broadcasting works across devices'


# ---- matmul ---------------------------------------------------------------------------------------------------
def test_matmul_hash_known_answers_on_device(device, golden):
    g = golden["matmul_hashes"]
    for rows, rm in ((g["row_major"], True), (g["column_major"], False), (g["column_major_large"], False)):
        for M, K, N, want in rows:
            for dt in (np.float32, np.float64):
                say("golden matmul", M, K, N, "RM" if rm else "CM", dt.__name__)
                A, B = on(device, fill_it(M * K, 43, dt)), on(device, fill_it(K * N, 87, dt))
                Cm = on(device, np.zeros(M * N, dtype=dt))
                device.launch_matmul(rm, M, K, N, A, B, Cm)
                assert java_array_hash(Cm.getData()) == want, (M, K, N, rm, dt)


def test_matmul_simple_kernel_bit_exact(device, orc):
    rng = np.random.default_rng(51)
    for M, K, N in ((17, 23, 13), (1, 64, 1), (70, 5, 129)):
        for dt in (np.float32, np.float64):
            for rm in (True, False):
                say("matmul simple", M, K, N, dt.__name__, rm)
                A = rng.uniform(-1, 1, M * K).astype(dt); B = rng.uniform(-1, 1, K * N).astype(dt); C0 = rng.uniform(-1, 1, M * N).astype(dt)
                tc = on(device, C0)
                device.launch_matmul(rm, M, K, N, on(device, A), on(device, B), tc)
                assert _lib.last_path() == "simple"
                assert_bits(tc.getData(), orc.gemm(rm, A, B, M, K, N, C_init=C0.copy()), "simple")


@pytest.mark.parametrize("mkn", [(128, 32, 128), (256, 96, 128), (384, 256, 512), (1024, 256, 256)])
def test_matmul_mfma_path(device, orc, mkn):
    """The MFMA kernel: exact on integer-valued data (any correct GEMM is), norm-wise 1e-5 on uniform
    data, accumulation into C, both layouts."""
    M, K, N = mkn
    rng = np.random.default_rng(52)
    say("matmul mfma integer", mkn)
    A = rng.integers(-5, 6, (M, K)).astype(np.float32); B = rng.integers(-5, 6, (K, N)).astype(np.float32)
    C0 = rng.integers(-9, 10, (M, N)).astype(np.float32)
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path().replace("_split", "") in ("mfma", "mfma_tiles_of_64")       # (small products: 64 x 64 tiles where the estimate prefers them)
    assert (tc.getData().reshape(M, N) == (A.astype(np.float64) @ B.astype(np.float64) + C0)).all()
    say("matmul mfma column major", mkn)
    tc = on(device, np.zeros((M, N), dtype=np.float32))
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)      # CM storage of A, B
    assert (tc.getData().reshape(N, M).T == A.astype(np.float64) @ B.astype(np.float64)).all()
    say("matmul mfma uniform", mkn)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32); B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    tc = on(device, np.zeros((M, N), dtype=np.float32))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=8).reshape(M, N)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(tc.getData().reshape(M, N).astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("mkn", [(300, 257, 270), (129, 1001, 131), (1000, 33, 1000), (127, 4097, 40), (641, 130, 385)])
def test_matmul_mfma_edge_path(device, orc, mkn):
    """Shapes that are not whole tiles, from 2^24 multiply-adds on: the matrix-core kernel with clamped edges and a
    zeroed k tail.  Exact on integer-valued data, norm-wise 1e-5 on uniform data, accumulation into C, both
    layouts; NaNs parked right behind the operands' rows must not leak into the result."""
    M, K, N = mkn
    rng = np.random.default_rng(54)
    say("matmul mfma edge integer", mkn)
    A = rng.integers(-5, 6, (M, K)).astype(np.float32); B = rng.integers(-5, 6, (K, N)).astype(np.float32)
    C0 = rng.integers(-9, 10, (M, N)).astype(np.float32)
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path().replace("_split", "") in ("mfma_edge", "mfma_tiles_of_64_edge")     # (64 x 64 tiles where the estimate prefers them)
    assert (tc.getData().reshape(M, N) == (A.astype(np.float64) @ B.astype(np.float64) + C0)).all()
    say("matmul mfma edge column major", mkn)
    tc = on(device, np.zeros((M, N), dtype=np.float32))
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)
    assert _lib.last_path().replace("_split", "") in ("mfma_edge", "mfma_tiles_of_64_edge")
    assert (tc.getData().reshape(N, M).T == A.astype(np.float64) @ B.astype(np.float64)).all()
    say("matmul mfma edge uniform", mkn)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32); B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    tc = on(device, np.zeros((M, N), dtype=np.float32))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=8).reshape(M, N)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(tc.getData().reshape(M, N).astype(np.float64) - ref) <= bound).all()
    say("matmul mfma edge, operands inside larger buffers full of NaN", mkn)
    # the C ABI takes addresses: place A, B and C in the middle of NaN-filled allocations
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=np.float32)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(np.zeros((M, N), dtype=np.float32))
    _lib.check(device._lib.nk_matmul(device.handle, 0, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + 4 * pad, pb._data.ptr + 4 * pad, pc._data.ptr + 4 * pad))
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
    assert (np.abs(got[pad:pad + M * N].reshape(M, N).astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("mkn,path", [((256, 256, 256), "mfma_f64_tiles_of_64"), ((384, 112, 512), "mfma_f64_tiles_of_64"), ((128, 1024, 128), "mfma_f64_tiles_of_64"),
                                      ((300, 257, 270), "mfma_f64_tiles_of_64_edge"), ((129, 1001, 131), "mfma_f64_tiles_of_64_edge"),
                                      ((1000, 33, 1000), "mfma_f64_tiles_of_64_edge"), ((127, 4097, 40), "mfma_f64_tiles_of_64_edge"),
                                      ((1024, 1024, 1024), "mfma_f64_tiles_of_64"), ((1500, 17, 1500), "mfma_f64_tiles_of_64_edge"),
                                      ((1536, 1024, 1536), "mfma_f64_tiles_of_64_mixed"), ((1111, 1111, 1111), "mfma_f64_tiles_of_64_edge_mixed"),
                                      ((2560, 512, 2560), "mfma_f64_tiles_of_64_mixed"), ((2500, 1030, 2500), "mfma_f64_tiles_of_64_edge_mixed"),
                                      ((2048, 512, 2048), "mfma_f64_tiles_of_64"), ((1152, 2048, 1152), "mfma_f64_tiles_of_64_mixed"),
                                      ((4096, 256, 4096), "mfma_f64"), ((1280, 1280, 1280), "mfma_f64_tiles_of_64"),
                                      ((255, 255, 250), "simple")])
def test_matmul_f64_matrix_core_path(device, orc, mkn, path):
    """f64 products from 2^24 multiply-adds on run on the f64 matrix cores -- on 64 x 64 tiles (whole, as parts of the k
    range, whole rounds plus parts; shapes that are no whole tiles; a single partial k-slice) where that fills the machine
    better, else on 128 x 128 tiles: exact on integer-valued data, within
    1e-12 norm-wise of the reference's order on uniform data, accumulation into C, both layouts, nothing written
    or read outside the operands; below the threshold the reference's order is kept bit for bit."""
    M, K, N = mkn
    rng = np.random.default_rng(55)
    say("matmul f64 integer", mkn)
    A = rng.integers(-5, 6, (M, K)).astype(np.float64); B = rng.integers(-5, 6, (K, N)).astype(np.float64)
    C0 = rng.integers(-9, 10, (M, N)).astype(np.float64)
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path().replace("_split", "") == path
    assert (tc.getData().reshape(M, N) == A @ B + C0).all()
    say("matmul f64 column major", mkn)
    tc = on(device, np.zeros((M, N), dtype=np.float64))
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)
    assert _lib.last_path().replace("_split", "") == path
    assert (tc.getData().reshape(N, M).T == A @ B).all()
    say("matmul f64 uniform, operands inside larger buffers full of NaN", mkn)
    A = rng.uniform(-1, 1, (M, K)); B = rng.uniform(-1, 1, (K, N))
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=8).reshape(M, N)
    bound = 1e-12 * (np.abs(A) @ np.abs(B))
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=np.float64)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(np.zeros((M, N)))
    _lib.check(device._lib.nk_matmul(device.handle, 1, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + 8 * pad, pb._data.ptr + 8 * pad, pc._data.ptr + 8 * pad))
    assert _lib.last_path().replace("_split", "") == path
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()
    if path == "simple":
        assert_bits(got[pad:pad + M * N], ref.reshape(-1), "simple f64")
    else:
        assert (np.abs(got[pad:pad + M * N].reshape(M, N) - ref) <= bound).all()


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("mkn", [(1, 4096, 4096), (4096, 4096, 1), (128, 8192, 128), (384, 2048, 384), (130, 4100, 70)])
def test_matmul_split_k(device, orc, mkn, dt):
    """Products with fewer tiles than compute units (matrix-vector, small squares, long inner dimension): the inner
    dimension is cut into parts that a second launch adds in order.  Exact on integer-valued data, norm-wise
    1e-5 / 1e-12 on uniform data, accumulation into C."""
    M, K, N = mkn
    T = F[dt]
    tol = 1e-5 if dt == "f32" else 1e-12
    rng = np.random.default_rng(56)
    say("matmul split-k integer", mkn, dt)
    A = rng.integers(-4, 5, (M, K)).astype(T); B = rng.integers(-4, 5, (K, N)).astype(T); C0 = rng.integers(-9, 10, (M, N)).astype(T)
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    few_rows = lambda rows, cols: rows <= 32 and cols % (16 // np.dtype(T).itemsize) == 0 and cols >= 1024 // np.dtype(T).itemsize
    vec = 16 // np.dtype(T).itemsize
    few_cols = lambda inner, cols: cols in (1, 2, 4) and inner % vec == 0
    assert (_lib.last_path().endswith("_split") or (few_rows(M, N) and _lib.last_path().startswith("few_rows"))
            or (few_cols(K, N) and _lib.last_path().startswith("few_cols"))), _lib.last_path()
    assert (tc.getData().reshape(M, N) == A.astype(np.float64) @ B.astype(np.float64) + C0).all()
    say("matmul split-k uniform", mkn, dt)
    A = rng.uniform(-1, 1, (M, K)).astype(T); B = rng.uniform(-1, 1, (K, N)).astype(T)
    tc = on(device, np.zeros((M, N), dtype=T))
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)          # column-major operands
    assert (_lib.last_path().endswith("_split") or (few_rows(N, M) and _lib.last_path().startswith("few_rows"))
            or (few_cols(K, M) and _lib.last_path().startswith("few_cols"))), _lib.last_path()
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=8).reshape(M, N)
    bound = tol * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(tc.getData().reshape(N, M).T.astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_random_products_through_every_plan(device, dt):
    """Random extents around the edges of the tilings (1, 2, just below / at / above 128, 256 and the split and
    matrix-core thresholds), both layouts, accumulation into a non-zero C.  Small integers keep every order of the
    sums exact, so each kernel -- the reference's order, matrix-core tiles whole and partial, inner dimension in
    parts -- must equal the integer product."""
    T = F[dt]
    rng = np.random.default_rng(57)
    sizes = [1, 2, 3, 31, 64, 127, 128, 129, 200, 255, 256, 257, 384, 511, 513, 1024]
    seen = set()
    for case in range(60):
        M, K, N = (int(rng.choice(sizes)) for _ in range(3))
        if case % 6 == 0:
            K = int(rng.choice([2048, 4096, 5000, 8192]))       # few tiles, long inner dimension
            M, N = int(rng.choice([64, 128, 130, 256])), int(rng.choice([64, 128, 130, 256]))
        row_major = bool(rng.random() < 0.6)
        say("random product", case, (M, K, N), "row major" if row_major else "column major", dt)
        A = rng.integers(-3, 4, (M, K)).astype(T); B = rng.integers(-3, 4, (K, N)).astype(T); C0 = rng.integers(-9, 10, (M, N)).astype(T)
        want = A.astype(np.float64) @ B.astype(np.float64) + C0
        if row_major:
            tc = on(device, C0)
            device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
            got = tc.getData().reshape(M, N)
        else:
            tc = on(device, C0.T.copy())
            device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)
            got = tc.getData().reshape(N, M).T
        seen.add(_lib.last_path())
        assert (got == want).all(), (case, M, K, N, row_major, _lib.last_path())
    say("plans seen", sorted(seen))
    assert "simple" in seen and any(p.endswith("_split") for p in seen) and any("edge" in p for p in seen), sorted(seen)


@pytest.mark.parametrize("mkn", [(16384, 64, 1024), (8192, 96, 2048), (65536, 32, 256), (4096, 160, 4096), (12288, 256, 1536)])
def test_matmul_blocks_that_walk_the_tiles(device, orc, mkn):
    """Whole-tile f32 products with few k-slices per tile and at least four tiles per compute unit: the blocks stay,
    walk the tiles and keep the k-slice pipeline running across them (an odd and an even number of slices per tile
    alternate the LDS buffers differently; one slice per tile leaves only the hand-over).  Exact on integer-valued
    data with accumulation into a non-zero C, both layouts; within 1e-5 norm-wise on uniform data."""
    M, K, N = mkn
    rng = np.random.default_rng(58)
    say("matmul walking blocks, integers", mkn)
    A = rng.integers(-3, 4, (M, K)).astype(np.float32); B = rng.integers(-3, 4, (K, N)).astype(np.float32)
    C0 = rng.integers(-9, 10, (M, N)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64) + C0
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == "mfma_stream"
    assert (tc.getData().reshape(M, N) == want).all()
    say("matmul walking blocks, column major", mkn)
    tc = on(device, C0.T.copy())
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)
    assert (tc.getData().reshape(N, M).T == want).all()
    say("matmul walking blocks, uniform", mkn)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32); B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    tc = on(device, np.zeros((M, N), dtype=np.float32))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(tc.getData().reshape(M, N).astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("dt,mkn,path", [
    ("f32", (64, 48, 80), "simple"), ("f32", (384, 2048, 384), "mfma_tiles_of_64_split"), ("f32", (1280, 2048, 1280), "mfma_split"), ("f32", (1536, 1024, 1536), "mfma_tiles_of_64_mixed"), ("f32", (512, 512, 512), "mfma_tiles_of_64"), ("f32", (2048, 1024, 2048), "mfma"),
    ("f32", (12288, 256, 1536), "mfma_stream"), ("f32", (130, 4100, 70), "mfma_tiles_of_64_edge_split"), ("f32", (1000, 300, 520), "mfma_tiles_of_64_edge"), ("f32", (2100, 100, 2100), "mfma_tiles_of_64_edge"),
    ("f64", (64, 48, 80), "simple"), ("f64", (512, 512, 512), "mfma_f64_tiles_of_64_split"), ("f64", (2048, 64, 2048), "mfma_f64_tiles_of_64"),
    ("f64", (1000, 300, 520), "mfma_f64_tiles_of_64_edge"), ("f64", (2100, 130, 2100), "mfma_f64_tiles_of_64_edge"),
    ("f64", (4096, 256, 4096), "mfma_f64"), ("f64", (1152, 2048, 1152), "mfma_f64_tiles_of_64_mixed"), ("f64", (1536, 1024, 1536), "mfma_f64_tiles_of_64_mixed"),
    ("f64", (130, 4100, 70), "mfma_f64_tiles_of_64_edge_split"), ("f64", (1500, 1050, 1500), "mfma_f64_tiles_of_64_edge_mixed"),
    ("f32", (3072, 1024, 3072), "mfma_bands"), ("f32", (3000, 1000, 3000), "mfma_edge_bands"), ("f64", (3072, 1024, 3072), "mfma_f64_bands"),
    ("f32", (5, 4096, 4096), "few_rows"), ("f64", (16, 4096, 1024), "few_rows_f64"), ("f32", (8192, 2048, 1), "few_cols"), ("f64", (4099, 2048, 4), "few_cols_f64"),
    ("f32", (4100, 9, 4096), "short_inner"), ("f64", (4096, 16, 2050), "short_inner_f64"),
    ("f32", (32, 2048, 2048), "few_rows"), ("f64", (20, 4096, 512), "few_rows_f64"),
    ("f32", (1024, 1024, 1024), "mfma_tiles_of_64"), ("f32", (1024, 288, 1024), "mfma_tiles_of_64")])
def test_matmul_set_overwrites_and_equals_accumulation_into_zeros(device, dt, mkn, path):
    """nk_matmul_set (C = A @ B, the OpenCL device's `C[n + m*N] = acc`, CLMatMul.java:50) on every kernel plan, both
    layouts: the drain starts as NaN everywhere, so a single old value read would show; the result must equal, bit for
    bit, what nk_matmul (C += A @ B) leaves in a zeroed C."""
    T = F[dt]
    M, K, N = mkn
    rng = np.random.default_rng(59)
    A = rng.uniform(-1, 1, (M, K)).astype(T); B = rng.uniform(-1, 1, (K, N)).astype(T)
    for row_major in (True, False):
        say("matmul set", dt, mkn, "row major" if row_major else "column major")
        ta, tb = (on(device, A), on(device, B)) if row_major else (on(device, A.T.copy()), on(device, B.T.copy()))
        acc = on(device, np.zeros((M, N), dtype=T))
        device.launch_matmul(row_major, M, K, N, ta, tb, acc)
        if row_major: assert _lib.last_path() == path
        got = on(device, np.full((M, N), np.nan, dtype=T))
        device.launch_matmul(row_major, M, K, N, ta, tb, got, accumulate=False)
        if row_major: assert _lib.last_path() == path
        a, g = acc.getData(), got.getData()
        assert not np.isnan(g).any()
        assert (a.view(np.uint32 if dt == "f32" else np.uint64) == g.view(np.uint32 if dt == "f32" else np.uint64)).all()


@pytest.mark.parametrize("mkn,path", [((2304, 608, 2304), "mfma_mixed"), ((2176, 512, 2176), "mfma_mixed"), ((33024, 512, 128), "mfma_mixed"),
                                      ((2048, 1056, 2560), "mfma_mixed"), ((2560, 512, 2560), "mfma_tiles_of_64"), ((4096, 512, 1536), "mfma_tiles_of_64"),
                                      ((3584, 512, 3584), "mfma_mixed"), ((2300, 520, 2300), "mfma_edge_mixed"), ((2090, 515, 2091), "mfma_edge_mixed")])
def test_matmul_a_few_more_tiles_than_compute_units(device, mkn, path):
    """Products with a few more 128 x 128 tiles than whole rounds of one per compute unit run as one launch in which the
    upper tile rows take the whole k range and the lower rows come as parts of it (their sum follows), shapes that are no
    whole tiles included; with more than half a round of tiles in the lower rows this launch is not taken (64 x 64 tiles serve those here).  Integer data are exact against numpy in both layouts and through both entry
    points (the parts' run lengths do not divide the k range in every case); uniform data stay within the norm-wise
    bound; NaN around the operands and in the drain of an overwriting call shows that nothing else is read."""
    M, K, N = mkn
    rng = np.random.default_rng(71)
    say("matmul mixed integer", mkn)
    A = rng.integers(-5, 6, (M, K)).astype(np.float32); B = rng.integers(-5, 6, (K, N)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64)
    ta, tb = on(device, A), on(device, B)
    tc = on(device, np.full((M, N), np.nan, dtype=np.float32))
    device.launch_matmul(True, M, K, N, ta, tb, tc, accumulate=False)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want).all()
    device.launch_matmul(True, M, K, N, ta, tb, tc)                                        # C += A @ B
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == 2 * want).all()
    say("matmul mixed column major", mkn)
    tc = on(device, np.zeros((N, M), dtype=np.float32))
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)
    assert (tc.getData().reshape(N, M).T == want).all()
    say("matmul mixed uniform, operands inside larger buffers full of NaN", mkn)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32); B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=np.float32)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(np.zeros((M, N), dtype=np.float32))
    _lib.check(device._lib.nk_matmul(device.handle, 0, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + 4 * pad, pb._data.ptr + 4 * pad, pc._data.ptr + 4 * pad))
    assert _lib.last_path() == path, _lib.last_path()
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
    assert (np.abs(got[pad:pad + M * N].reshape(M, N).astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("mkn,path", [((1024, 1024, 1024), "mfma_tiles_of_64"), ((1024, 320, 1024), "mfma_tiles_of_64"),
                                      ((512, 4096, 2048), "mfma_tiles_of_64"), ((1024, 128, 1024), "mfma_tiles_of_64"),
                                      ((1024, 288, 1024), "mfma_tiles_of_64"), ((2048, 160, 512), "mfma_tiles_of_64"),
                                      ((1000, 1000, 1000), "mfma_tiles_of_64_edge"), ((777, 333, 1025), "mfma_tiles_of_64_edge"),
                                      ((65, 1001, 4097), "mfma_tiles_of_64_edge"), ((1023, 129, 1025), "mfma_tiles_of_64_edge"),
                                      ((1536, 1024, 1536), "mfma_tiles_of_64_mixed"), ((1792, 1056, 1792), "mfma_tiles_of_64_mixed"),
                                      ((1500, 1050, 1500), "mfma_tiles_of_64_edge_mixed"), ((1111, 1111, 1111), "mfma_tiles_of_64_edge_mixed"),
                                      ((2560, 512, 2560), "mfma_tiles_of_64"), ((2560, 1024, 2560), "mfma_tiles_of_64_mixed"),
                                      ((2500, 520, 2500), "mfma_tiles_of_64_edge"), ((2500, 1030, 2500), "mfma_tiles_of_64_edge_mixed"),
                                      ((384, 2048, 384), "mfma_tiles_of_64_split"), ((4096, 1024, 64), "mfma_tiles_of_64_split"), ((64, 4096, 1024), "mfma_tiles_of_64_split"),
                                      ((300, 4000, 300), "mfma_tiles_of_64_edge_split"), ((1000, 3001, 100), "mfma_tiles_of_64_edge_split"), ((65, 8190, 129), "mfma_tiles_of_64_edge_split"),
                                      ((1024, 64, 1024), "mfma_tiles_of_64"), ((1024, 32, 1024), "mfma_tiles_of_64"), ((512, 96, 512), "mfma_tiles_of_64"),
                                      ((3000, 40, 3000), "mfma_tiles_of_64_edge"), ((1000, 100, 1000), "mfma_tiles_of_64_edge"), ((1500, 17, 1500), "mfma_tiles_of_64_edge")])
def test_matmul_64_tiles_in_one_launch(device, mkn, path):
    """Products with too few 128 x 128 tiles for the machine but a 64 x 64 tile for every compute unit, or with a last
    round of 128 x 128 tiles that would leave most of the machine idle (2560 and 2500 square: 400 tiles on 256 units): one launch of
    the small-tile kernel, from a single k-slice (a partial one: k = 17) up to long k ranges, and its edge variant for shapes that are no whole
    number of tiles or slices (odd row lengths: operands' rows are then not 16-byte aligned); with less than a round of small tiles and a long k range every tile as parts of the k range; with a few tiles more than
    whole rounds, the upper tile rows whole and the rest as parts of the k range in the same launch.  Integer data are exact against numpy in both layouts and
    through both entry points; uniform data stay within the norm-wise bound; operands inside larger buffers full of NaN
    show that nothing outside them is read."""
    M, K, N = mkn
    rng = np.random.default_rng(67)
    say("matmul 64 tiles integer", mkn)
    A = rng.integers(-5, 6, (M, K)).astype(np.float32); B = rng.integers(-5, 6, (K, N)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64)
    tc = on(device, np.full((M, N), np.nan, dtype=np.float32))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc, accumulate=False)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want).all()
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)                  # C += A @ B
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == 2 * want).all()
    say("matmul 64 tiles column major", mkn)
    tc = on(device, np.zeros((N, M), dtype=np.float32))
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)
    assert (tc.getData().reshape(N, M).T == want).all()
    say("matmul 64 tiles uniform", mkn)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32); B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    tc = on(device, np.zeros((M, N), dtype=np.float32))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == path, _lib.last_path()
    ref = A.astype(np.float64) @ B.astype(np.float64)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(tc.getData().reshape(M, N).astype(np.float64) - ref) <= bound).all()
    say("matmul 64 tiles, operands inside larger buffers full of NaN", mkn)
    for pad in (64,) + ((61,) if "_edge" in path else ()):                     # elements: 64 keeps the 16-byte alignment, 61 breaks it
        def parked(x):
            host = np.full(x.size + 2 * pad, np.nan, dtype=np.float32)
            host[pad:pad + x.size] = x.reshape(-1)
            return on(device, host)
        pa, pb, pc = parked(A), parked(B), parked(np.zeros((M, N), dtype=np.float32))
        _lib.check(device._lib.nk_matmul(device.handle, 0, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + 4 * pad, pb._data.ptr + 4 * pad, pc._data.ptr + 4 * pad))
        assert _lib.last_path() == path, _lib.last_path()
        got = pc.getData()
        assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
        assert (np.abs(got[pad:pad + M * N].reshape(M, N).astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_matmul_random_shapes_are_exact_in_whatever_plan_they_take(device, seed):
    """Shapes drawn at random from six families (any shape, whole small tiles, long k over few tiles, short k over many,
    whole large tiles, mid-size) in both element types: whatever plan the estimates choose, small-integer operands give
    the exact product, for C = A B into NaNs and for C += A B into a non-zero C."""
    rng = np.random.default_rng(seed)
    def draw():
        kind = rng.integers(0, 6)
        if kind == 0: return int(rng.integers(33, 3000)), int(rng.integers(17, 3000)), int(rng.integers(17, 3000))
        if kind == 1: return 64 * int(rng.integers(1, 48)), 32 * int(rng.integers(1, 64)), 64 * int(rng.integers(1, 48))
        if kind == 2: return int(rng.integers(33, 400)), int(rng.integers(1000, 12000)), int(rng.integers(17, 400))
        if kind == 3: return int(rng.integers(1000, 6000)), int(rng.integers(17, 200)), int(rng.integers(1000, 6000))
        if kind == 4: return 128 * int(rng.integers(8, 30)), 32 * int(rng.integers(4, 40)), 128 * int(rng.integers(8, 30))
        return int(rng.integers(1500, 4200)), int(rng.integers(200, 1500)), int(rng.integers(1500, 4200))
    plans = set()
    for _ in range(12):
        M, K, N = draw()
        for dt in (np.float32, np.float64):
            say("matmul random shape", (M, K, N), dt.__name__)
            A = rng.integers(-3, 4, (M, K)).astype(dt); B = rng.integers(-3, 4, (K, N)).astype(dt); C0 = rng.integers(-9, 10, (M, N)).astype(dt)
            want = A.astype(np.float64) @ B.astype(np.float64)
            ta, tb = on(device, A), on(device, B)
            tc = on(device, np.full((M, N), np.nan, dtype=dt))
            device.launch_matmul(True, M, K, N, ta, tb, tc, accumulate=False)
            plans.add(_lib.last_path())
            assert (tc.getData().reshape(M, N) == want).all(), ((M, K, N), dt.__name__, _lib.last_path())
            tc = on(device, C0)
            device.launch_matmul(True, M, K, N, ta, tb, tc)
            assert (tc.getData().reshape(M, N) == want + C0).all(), ((M, K, N), dt.__name__, _lib.last_path())
    say("plans seen", sorted(plans))


@pytest.mark.parametrize("mkn", [(4096, 1024, 4096), (2048, 2048, 8192), (4096, 1056, 4096), (8192, 1024, 8192), (4096, 512, 4096)])
def test_matmul_256_tiles_one_wavefront_per_simd(device, mkn):
    """Large f32 products whose 256 x 256 tiles fill the machine take the kernel with one wavefront per SIMD.  It sums
    in the order of the 128 x 128 kernel, which computes the left half of the same product (half as many tiles: not
    enough for the large kernel) -- bit for bit; integer data are exact against numpy; both entry points, both layouts."""
    M, K, N = mkn
    rng = np.random.default_rng(61)
    say("matmul 256 tiles", mkn)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32); B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    ta, tb = on(device, A), on(device, B)
    c = on(device, np.full((M, N), np.nan, dtype=np.float32))
    device.launch_matmul(True, M, K, N, ta, tb, c, accumulate=False)
    assert _lib.last_path() == "mfma_big", _lib.last_path()
    got = c.getData().reshape(M, N)
    assert not np.isnan(got).any()
    if (M // 256) * (N // 512) < device.maxComputeUnits():       # (four rounds of tiles: the half is a large product itself)
        half = np.ascontiguousarray(B[:, :N // 2])
        th = on(device, half)
        ch = on(device, np.zeros((M, N // 2), dtype=np.float32))
        device.launch_matmul(True, M, K, N // 2, ta, th, ch)
        assert _lib.last_path() == "mfma", _lib.last_path()
        assert_bits(got[:, :N // 2], ch.getData().reshape(M, N // 2), "left half against the 128 x 128 kernel")
    rows = rng.choice(M, 32, replace=False)
    ref = A[rows].astype(np.float64) @ B.astype(np.float64)
    bound = 1e-5 * (np.abs(A[rows]).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(got[rows] - ref) <= bound).all()
    # C += A B on top of the result: exactly twice it (the sum is the same, added to itself)
    device.launch_matmul(True, M, K, N, ta, tb, c)
    assert _lib.last_path() == ("mfma_big" if K >= 1024 else "mfma")          # shallow tiles that also read C: two blocks per compute unit
    assert_bits(c.getData().reshape(M, N), 2 * got, "accumulating")
    say("matmul 256 tiles, integer data, column major", mkn)
    Ai = rng.integers(-3, 4, (M, K)).astype(np.float32); Bi = rng.integers(-3, 4, (K, N)).astype(np.float32)
    tai, tbi = on(device, Ai.T.copy()), on(device, Bi.T.copy())
    ci = on(device, np.zeros((N, M), dtype=np.float32))
    device.launch_matmul(False, M, K, N, tai, tbi, ci, accumulate=False)
    assert _lib.last_path() == "mfma_big"
    assert_bits(ci.getData().reshape(N, M), (Ai @ Bi).T.copy(), "column major")


@pytest.mark.parametrize("mkn", [(4000, 1100, 4000), (4090, 1030, 4001), (8100, 1024, 8000), (3841, 1025, 4096)])
def test_matmul_256_tiles_with_edges(device, mkn):
    """Large f32 products that are no whole number of tiles, on the 256 x 256 kernel with clamped edges and a zeroed
    k tail (rows of C that start at odd addresses included): exact on integer data with accumulation into a non-zero
    C, both layouts, both entry points; NaNs parked around the operands neither leak in nor get overwritten."""
    M, K, N = mkn
    rng = np.random.default_rng(62)
    say("matmul 256 tiles with edges, integers", mkn)
    A = rng.integers(-3, 4, (M, K)).astype(np.float32); B = rng.integers(-3, 4, (K, N)).astype(np.float32)
    C0 = rng.integers(-9, 10, (M, N)).astype(np.float32)
    want = A @ B                                             # exact: |sums| < 2^24
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == "mfma_big_edge", _lib.last_path()
    assert_bits(tc.getData().reshape(M, N), want + C0, "C += A B")
    say("matmul 256 tiles with edges, column major, C = A B into NaNs", mkn)
    tc = on(device, np.full((N, M), np.nan, dtype=np.float32))
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc, accumulate=False)
    assert _lib.last_path() == "mfma_big_edge", _lib.last_path()
    assert_bits(tc.getData().reshape(N, M), want.T.copy(), "column major")
    say("matmul 256 tiles with edges, operands inside larger buffers full of NaN", mkn)
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=np.float32)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(C0)
    _lib.check(device._lib.nk_matmul(device.handle, 0, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + 4 * pad, pb._data.ptr + 4 * pad, pc._data.ptr + 4 * pad))
    assert _lib.last_path() == "mfma_big_edge", _lib.last_path()
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
    assert_bits(got[pad:pad + M * N].reshape(M, N), want + C0, "parked operands")


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("mkn", [(1, 4096, 4096), (16, 4096, 4096), (3, 5001, 4100), (8, 2049, 1024), (2, 70000, 256), (5, 33, 131072), (13, 8192, 512),
                                 (32, 4096, 4096), (17, 1000, 2052), (25, 8191, 256)])
def test_matmul_few_rows(device, orc, mkn, dt):
    """A vector or a small batch times a large matrix (at most 32 rows, from 2^24 multiply-adds on) runs as one stream
    over the matrix with the k range in parts: exact on integer data, C += A B into a non-zero C and C = A B into NaNs,
    column major (a large matrix times a few columns), operands parked between NaNs, uniform data against the oracle."""
    M, K, N = mkn
    T = F[dt]
    tol = 1e-5 if dt == "f32" else 1e-12
    path = "few_rows" if dt == "f32" else "few_rows_f64"
    rng = np.random.default_rng(64)
    say("matmul few rows, integers", mkn, dt)
    A = rng.integers(-3, 4, (M, K)).astype(T); B = rng.integers(-3, 4, (K, N)).astype(T); C0 = rng.integers(-9, 10, (M, N)).astype(T)
    want = A.astype(np.float64) @ B.astype(np.float64)
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want + C0).all()
    say("matmul few rows, C = A B into NaNs", mkn, dt)
    tc = on(device, np.full((M, N), np.nan, dtype=T))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc, accumulate=False)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want).all()
    say("matmul few rows, column major: a large matrix times a few columns", mkn, dt)
    # column-major [N,K] @ [K,M]: the row-major data of the transposes
    tc = on(device, C0)
    device.launch_matmul(False, N, K, M, on(device, B), on(device, A), tc)      # B's row-major data = column-major B^T[N,K], likewise A
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want + C0).all()                      # column-major C^T[N,M] = row-major C[M,N]
    say("matmul few rows, operands inside larger buffers full of NaN", mkn, dt)
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=T)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(C0)
    eb = np.dtype(T).itemsize
    _lib.check(device._lib.nk_matmul(device.handle, 0 if dt == "f32" else 1, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + eb * pad, pb._data.ptr + eb * pad, pc._data.ptr + eb * pad))
    assert _lib.last_path() == path, _lib.last_path()
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
    assert (got[pad:pad + M * N].reshape(M, N) == want + C0).all()
    say("matmul few rows, uniform data against the oracle", mkn, dt)
    A = rng.uniform(-1, 1, (M, K)).astype(T); B = rng.uniform(-1, 1, (K, N)).astype(T)
    tc = on(device, np.zeros((M, N), dtype=T))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=8).reshape(M, N)
    bound = tol * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(tc.getData().reshape(M, N).astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("mkn", [(4096, 4096, 1), (4099, 4096, 1), (10000, 1000, 2), (513, 8192, 4), (70001, 64, 4), (17, 1048576, 1), (2, 2097152, 4)])
def test_matmul_few_columns(device, orc, mkn, dt):
    """A large matrix times a vector (1, 2 or 4 columns, from 2^24 multiply-adds on) runs as one stream over the matrix in
    one launch: exact on integer data, C += A B into a non-zero C and C = A B into NaNs, column major (a vector times a
    large matrix), operands parked between NaNs, uniform data against the oracle."""
    M, K, N = mkn
    T = F[dt]
    tol = 1e-5 if dt == "f32" else 1e-12
    few_rows = M <= 32 and N % (16 // np.dtype(T).itemsize) == 0 and N >= 1024 // np.dtype(T).itemsize
    path = ("few_rows" if few_rows else "few_cols") + ("" if dt == "f32" else "_f64")
    rng = np.random.default_rng(65)
    say("matmul few columns, integers", mkn, dt)
    A = rng.integers(-3, 4, (M, K)).astype(T); B = rng.integers(-3, 4, (K, N)).astype(T); C0 = rng.integers(-9, 10, (M, N)).astype(T)
    want = A.astype(np.float64) @ B.astype(np.float64)
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want + C0).all()
    say("matmul few columns, C = A B into NaNs", mkn, dt)
    tc = on(device, np.full((M, N), np.nan, dtype=T))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc, accumulate=False)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want).all()
    say("matmul few columns, column major: a vector times a large matrix", mkn, dt)
    tc = on(device, C0)
    device.launch_matmul(False, N, K, M, on(device, B), on(device, A), tc)      # the row-major data of the transposes
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want + C0).all()
    say("matmul few columns, operands inside larger buffers full of NaN", mkn, dt)
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=T)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(C0)
    eb = np.dtype(T).itemsize
    _lib.check(device._lib.nk_matmul(device.handle, 0 if dt == "f32" else 1, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + eb * pad, pb._data.ptr + eb * pad, pc._data.ptr + eb * pad))
    assert _lib.last_path() == path, _lib.last_path()
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
    assert (got[pad:pad + M * N].reshape(M, N) == want + C0).all()
    say("matmul few columns, uniform data against the oracle", mkn, dt)
    A = rng.uniform(-1, 1, (M, K)).astype(T); B = rng.uniform(-1, 1, (K, N)).astype(T)
    tc = on(device, np.zeros((M, N), dtype=T))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=8).reshape(M, N)
    bound = tol * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(tc.getData().reshape(M, N).astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("mkn", [(4096, 16, 4096), (4096, 1, 4096), (5000, 7, 3332), (33, 13, 40000), (70000, 3, 256), (1025, 16, 1028)])
def test_matmul_short_inner_dimension(device, orc, mkn, dt):
    """A sum of at most 16 outer products (the gradient of a weight matrix from a small batch, from 2^24 multiply-adds
    on) runs as one stream over C: exact on integer data, C += A B into a non-zero C and C = A B into NaNs, column
    major, operands parked between NaNs, uniform data against the oracle."""
    M, K, N = mkn
    T = F[dt]
    tol = 1e-5 if dt == "f32" else 1e-12
    path = "short_inner" if dt == "f32" else "short_inner_f64"
    rng = np.random.default_rng(66)
    say("matmul short inner dimension, integers", mkn, dt)
    A = rng.integers(-3, 4, (M, K)).astype(T); B = rng.integers(-3, 4, (K, N)).astype(T); C0 = rng.integers(-9, 10, (M, N)).astype(T)
    want = A.astype(np.float64) @ B.astype(np.float64)
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want + C0).all()
    say("matmul short inner dimension, C = A B into NaNs", mkn, dt)
    tc = on(device, np.full((M, N), np.nan, dtype=T))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc, accumulate=False)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want).all()
    say("matmul short inner dimension, column major", mkn, dt)
    tc = on(device, C0)
    device.launch_matmul(False, N, K, M, on(device, B), on(device, A), tc)      # the row-major data of the transposes
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want + C0).all()
    say("matmul short inner dimension, operands inside larger buffers full of NaN", mkn, dt)
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=T)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(C0)
    eb = np.dtype(T).itemsize
    _lib.check(device._lib.nk_matmul(device.handle, 0 if dt == "f32" else 1, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + eb * pad, pb._data.ptr + eb * pad, pc._data.ptr + eb * pad))
    assert _lib.last_path() == path, _lib.last_path()
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
    assert (got[pad:pad + M * N].reshape(M, N) == want + C0).all()
    say("matmul short inner dimension, uniform data bit for bit against the oracle", mkn, dt)
    # the kernel keeps the reference's order and rounding (old value, then the rounded products in k order): the bits of
    # GEMM.partial_F32_MxN_RM, into a non-zero C as well, and the same bits when the operands are moved off the
    # 16-byte boundary (another plan takes them then)
    A = rng.uniform(-1, 1, (M, K)).astype(T); B = rng.uniform(-1, 1, (K, N)).astype(T); C1 = rng.uniform(-1, 1, (M, N)).astype(T)
    tc = on(device, C1)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == path, _lib.last_path()
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, C_init=C1.reshape(-1).copy(), workers=8).reshape(M, N)
    assert_bits(tc.getData().reshape(M, N), ref, "C += A B, uniform data")
    pa, pb, pc = (on(device, np.concatenate([np.zeros(1, dtype=T), x.reshape(-1)])) for x in (A, B, C1))
    _lib.check(device._lib.nk_matmul(device.handle, 0 if dt == "f32" else 1, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + eb, pb._data.ptr + eb, pc._data.ptr + eb))
    assert _lib.last_path() != path
    assert_bits(pc.getData()[1:].reshape(M, N), ref, "the same product from operands off a 16-byte boundary")


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("mkn", [(4096, 4096, 16), (4096, 4096, 8), (4099, 2048, 3), (5000, 1000, 5), (1025, 4096, 11), (70001, 64, 16), (2048, 8192, 13)])
def test_matmul_batch_of_columns(device, orc, mkn, dt):
    """A large matrix times a batch of 3 or 5 to 16 columns (at least 1024 rows, from 2^24 multiply-adds on) runs as one
    stream over the matrix with the columns staged in LDS: exact on integer data, C += A B into a non-zero C and C = A B
    into NaNs, column major, operands parked between NaNs, uniform data against the oracle."""
    M, K, N = mkn
    T = F[dt]
    tol = 1e-5 if dt == "f32" else 1e-12
    path = "some_cols" if dt == "f32" else "some_cols_f64"
    rng = np.random.default_rng(67)
    say("matmul batch of columns, integers", mkn, dt)
    A = rng.integers(-3, 4, (M, K)).astype(T); B = rng.integers(-3, 4, (K, N)).astype(T); C0 = rng.integers(-9, 10, (M, N)).astype(T)
    want = A.astype(np.float64) @ B.astype(np.float64)
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want + C0).all()
    say("matmul batch of columns, C = A B into NaNs", mkn, dt)
    tc = on(device, np.full((M, N), np.nan, dtype=T))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc, accumulate=False)
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want).all()
    say("matmul batch of columns, column major", mkn, dt)
    tc = on(device, C0)
    device.launch_matmul(False, N, K, M, on(device, B), on(device, A), tc)      # the row-major data of the transposes
    assert _lib.last_path() == path, _lib.last_path()
    assert (tc.getData().reshape(M, N) == want + C0).all()
    say("matmul batch of columns, operands inside larger buffers full of NaN", mkn, dt)
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=T)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(C0)
    eb = np.dtype(T).itemsize
    _lib.check(device._lib.nk_matmul(device.handle, 0 if dt == "f32" else 1, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + eb * pad, pb._data.ptr + eb * pad, pc._data.ptr + eb * pad))
    assert _lib.last_path() == path, _lib.last_path()
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
    assert (got[pad:pad + M * N].reshape(M, N) == want + C0).all()
    say("matmul batch of columns, uniform data against the oracle", mkn, dt)
    A = rng.uniform(-1, 1, (M, K)).astype(T); B = rng.uniform(-1, 1, (K, N)).astype(T)
    tc = on(device, np.zeros((M, N), dtype=T))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=8).reshape(M, N)
    bound = tol * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(tc.getData().reshape(M, N).astype(np.float64) - ref) <= bound).all()


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("mkn", [(4, 4096, 4096), (4096, 4096, 2), (4096, 8, 4096), (4096, 4096, 12), (4, 4096, 4098), (4096, 4095, 2), (4096, 8, 4097), (4096, 4094, 12)])
def test_matmul_streaming_plans_need_aligned_operands_and_fall_back(device, mkn, dt):
    """The streaming kernels read 16 bytes at a time: operands that start 4 or 8 bytes off such a boundary, or whose rows
    do, take the tile kernels instead.  Whatever the plan, the integer product is exact and nothing outside C is written."""
    M, K, N = mkn
    T = F[dt]
    eb = np.dtype(T).itemsize
    rng = np.random.default_rng(68)
    A = rng.integers(-3, 4, (M, K)).astype(T); B = rng.integers(-3, 4, (K, N)).astype(T); C0 = rng.integers(-9, 10, (M, N)).astype(T)
    want = A.astype(np.float64) @ B.astype(np.float64)
    for pad in (1, 64):                                                    # 1 element: 4 or 8 bytes off a 16-byte boundary
        say("matmul streaming plans, operands", pad, "elements into their buffers", mkn, dt)
        def parked(x):
            host = np.full(x.size + 2 * pad, np.nan, dtype=T)
            host[pad:pad + x.size] = x.reshape(-1)
            return on(device, host)
        pa, pb, pc = parked(A), parked(B), parked(C0)
        _lib.check(device._lib.nk_matmul(device.handle, 0 if dt == "f32" else 1, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + eb * pad, pb._data.ptr + eb * pad, pc._data.ptr + eb * pad))
        print("[path]", _lib.last_path(), flush=True)
        got = pc.getData()
        assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()
        assert (got[pad:pad + M * N].reshape(M, N) == want + C0).all()


@pytest.mark.parametrize("mkn,path", [((16, 4096, 4096), "few_rows"), ((4096, 4096, 16), "some_cols"), ((4096, 4096, 1), "few_cols")])
def test_matmul_streaming_plans_depend_on_alignment_only_within_tolerance(device, orc, mkn, path):
    """few_rows, few_cols and some_cols add their terms with fused multiply-adds in an order of their own and are chosen
    by the operands' 16-byte alignment as well as by shape: the same product from a view one element into its buffer
    takes another plan and may differ in the last bits.  Both stay within the norm-wise 1e-5 of the oracle (from 2^24
    multiply-adds on every plan re-orders the sum), and so within 2e-5 of each other."""
    M, K, N = mkn
    rng = np.random.default_rng(69)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32); B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    ref = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=8).reshape(M, N).astype(np.float64)
    bound = 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64))
    results = []
    for pad in (0, 1):
        say("matmul plan against alignment", mkn, "operands", pad, "elements into their buffers")
        pa, pb, pc = (on(device, np.concatenate([np.zeros(pad, dtype=np.float32), x.reshape(-1)])) for x in (A, B, np.zeros((M, N), dtype=np.float32)))
        _lib.check(device._lib.nk_matmul_set(device.handle, 0, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + 4 * pad, pb._data.ptr + 4 * pad, pc._data.ptr + 4 * pad))
        assert (_lib.last_path() == path) == (pad == 0), _lib.last_path()
        got = pc.getData()[pad:].reshape(M, N).astype(np.float64)
        assert (np.abs(got - ref) <= bound).all(), _lib.last_path()
        results.append(got)
    assert (np.abs(results[0] - results[1]) <= 2 * bound).all()


@pytest.mark.parametrize("mkn", [(3072, 1024, 3072), (3000, 1000, 3000), (1280, 1024, 8192), (2700, 1100, 3400)])
def test_matmul_row_bands(device, mkn):
    """Products whose 128 x 128 tiles are a few more than whole rounds of the machine run as two row bands, the lower
    one with its k range cut into parts: exact on integer data, C += A B into a non-zero C and C = A B into NaNs, both
    layouts, and with the operands parked between NaNs (the bands start inside the buffers)."""
    M, K, N = mkn
    rng = np.random.default_rng(63)
    whole = M % 128 == 0 and N % 128 == 0 and K % 32 == 0
    path = "mfma_bands" if whole else "mfma_edge_bands"
    say("matmul row bands, integers", mkn)
    A = rng.integers(-3, 4, (M, K)).astype(np.float32); B = rng.integers(-3, 4, (K, N)).astype(np.float32)
    C0 = rng.integers(-9, 10, (M, N)).astype(np.float32)
    want = A @ B                                             # exact: |sums| < 2^24
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    assert _lib.last_path() == path, _lib.last_path()
    assert_bits(tc.getData().reshape(M, N), want + C0, "C += A B")
    say("matmul row bands, C = A B into NaNs", mkn)
    tc = on(device, np.full((M, N), np.nan, dtype=np.float32))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc, accumulate=False)
    assert _lib.last_path() == path, _lib.last_path()
    assert_bits(tc.getData().reshape(M, N), want, "C = A B")
    say("matmul row bands, column major", mkn)
    tc = on(device, C0.T.copy())
    device.launch_matmul(False, M, K, N, on(device, A.T.copy()), on(device, B.T.copy()), tc)
    assert_bits(tc.getData().reshape(N, M), (want + C0).T.copy(), "column major")
    say("matmul row bands, operands inside larger buffers full of NaN", mkn)
    pad = 64
    def parked(x):
        host = np.full(x.size + 2 * pad, np.nan, dtype=np.float32)
        host[pad:pad + x.size] = x.reshape(-1)
        return on(device, host)
    pa, pb, pc = parked(A), parked(B), parked(C0)
    _lib.check(device._lib.nk_matmul(device.handle, 0, _lib.ROW_MAJOR, M, K, N, pa._data.ptr + 4 * pad, pb._data.ptr + 4 * pad, pc._data.ptr + 4 * pad))
    assert _lib.last_path() == path, _lib.last_path()
    got = pc.getData()
    assert np.isnan(got[:pad]).all() and np.isnan(got[pad + M * N:]).all()            # nothing written outside C
    assert_bits(got[pad:pad + M * N].reshape(M, N), want + C0, "parked operands")
    say("matmul row bands, uniform data against float64", mkn)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32); B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    tc = on(device, np.zeros((M, N), np.float32))
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    scale = np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)
    assert (np.abs(tc.getData().reshape(M, N) - ref) <= 1e-5 * scale + 1e-30).all()
    say("matmul row bands, float64", mkn)
    A = rng.uniform(-1, 1, (M, K)); B = rng.uniform(-1, 1, (K, N)); C0 = rng.uniform(-1, 1, (M, N))
    tc = on(device, C0)
    device.launch_matmul(True, M, K, N, on(device, A), on(device, B), tc)
    # (f64 takes the bands too, except where 64 x 64 tiles are estimated to finish clearly earlier: the last shape)
    f64_bands = "mfma_f64_bands" if M % 128 == 0 and N % 128 == 0 and K % 16 == 0 else "mfma_f64_edge_bands"
    assert _lib.last_path() == (f64_bands if mkn != (2700, 1100, 3400) else "mfma_f64_tiles_of_64_edge_mixed"), _lib.last_path()
    assert (np.abs(tc.getData().reshape(M, N) - (ref_d := A @ B + C0)) <= 1e-12 * (np.abs(A) @ np.abs(B) + np.abs(C0))).all()


def test_matmul_through_the_tensor_api(device):
    """a.matMul(b) with transposed and sliced operands (auto-clone), and its backward."""
    say("matmul tensor api")
    rng = np.random.default_rng(53)
    a = rng.integers(-4, 5, (6, 9)).astype(np.float64); b = rng.integers(-4, 5, (9, 5)).astype(np.float64)
    ta, tb = on(device, a).setRqsGradient(True), on(device, b).setRqsGradient(True)
    c = ta.matMul(tb)
    assert (c.items.reshape(6, 5) == a @ b).all()
    assert (on(device, a.T.copy()).T().matMul(tb).items.reshape(6, 5) == a @ b).all()        # a CM view of A
    big = on(device, np.pad(a, ((1, 1), (2, 2))))
    assert (big[1:7, 2:11].matMul(tb).items.reshape(6, 5) == a @ b).all()                    # partial slice -> cloned
    e = rng.integers(-3, 4, (6, 5)).astype(np.float64)
    c.backward(on(device, e))
    assert (ta.gradient.items.reshape(6, 9) == e @ b.T).all() and (tb.gradient.items.reshape(9, 5) == a.T @ e).all()


# ---- whole-tensor reductions ------------------------------------------------------------------------------
def test_stats_golden_on_device(device, golden):
    """Tensor_Stats_Spec / Tensor_Dot_Product_Spec with the tensors on the device."""
    from test_oracle_pinned import stats_function_input
    g = golden["stats"]
    for reduce_type, type_name, expected in g["min_max_function"]["rows"]:
        dt = np.float32 if type_name == "Float" else np.float64
        a = on(device, stats_function_input(reduce_type, type_name, dt), (19, 7))
        r = Function.of(reduce_type.lower() + "(I[0])")(a)
        assert r.shape == (1,) and r.items[0] == expected, (reduce_type, type_name)
    a = on(device, np.array([((31 ** (i + 42)) % 301) - 151 for i in range(133)], dtype=np.float32), (19, 7))
    assert a.min().item(0) == g["min_max_methods"]["min"] and a.max().item(0) == g["min_max_methods"]["max"]
    s = on(device, np.array([((7 ** i) % 11) - 5 for i in range(13 * 73 * 11)], dtype=np.float32), (13, 73, 11)).sum()
    assert s.shape == (1,) and s.item(0) == g["sum"]["expected"] and _lib.last_path() == "tile_tree_128"
    for row in g["dot"]:
        r = on(device, np.array(row["a"], dtype=np.float32)).dot(on(device, np.array(row["b"], dtype=np.float32)))
        assert r.shape == (1,) and r.item(0) == row["expected"]


def test_stats_autograd_golden(device, golden):
    g = golden["stats"]
    a = on(device, np.array(g["min_max_autograd"]["a"], dtype=np.float32)).setRqsGradient(True)
    b = a * Tensor.of(np.float32, (1,), 3.0)
    x = b.min() / Tensor.of(np.float32, (1,), 2.0)
    y = b.max() / Tensor.of(np.float32, (1,), 4.0)
    (x + y).backward()
    assert a.gradient.items.tolist() == g["min_max_autograd"]["gradient"]
    a = on(device, np.array(g["sum_autograd"]["a"], dtype=np.float32)).setRqsGradient(True)
    (a * Tensor.of(np.float32, (1,), 3.0)).sum().backward()
    assert a.gradient.items.tolist() == g["sum_autograd"]["gradient"]
    d = g["dot_autograd"]
    a = on(device, np.array(d["a"], dtype=np.float32))
    w = on(device, np.array(d["w"], dtype=np.float32)).setRqsGradient(True)
    r = a.dot(w)
    assert r.items.tolist() == [d["result"]]
    r.backward(Tensor.of(np.float32, (1,), d["backward_error"]))
    assert w.gradient.shape == (3,) and w.gradient.items.tolist() == d["w_gradient"]


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_sum_is_bit_identical_to_the_cpu_tree(device, orc, dt):
    rng = np.random.default_rng(61)
    for n in (1, 2, 31, 127, 128, 129, 8191, 8192, 16385, 32767, 32768, 32769, 100003, (1 << 21) + 77):
        say("sum", dt, n)
        x = rng.standard_normal(n).astype(F[dt])
        got = on(device, x).sum()
        assert_bits(got.items, np.array([orc.sum_tree(x)], dtype=F[dt]), f"sum n={n}")
    x = np.array([-0.0], dtype=F[dt])                              # a single element is returned as it is
    assert np.signbit(on(device, x).sum().items[0])
    # views are summed through a dense copy: a transposed slice
    m = rng.standard_normal((40, 50)).astype(F[dt])
    v = on(device, m)[3:33, 5:45].T()
    assert_bits(v.sum().items, np.array([orc.sum_tree(np.ascontiguousarray(m[3:33, 5:45].T).reshape(-1))], dtype=F[dt]), "sum of a view")


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_min_max_return_the_reference_index(device, orc, dt):
    rng = np.random.default_rng(62)
    for n in (1, 2, 63, 64, 65, 4095, 4096, 4097, 16383, 16384, 16385, 70001, (1 << 20) + 3):
        say("min/max", dt, n)
        x = rng.integers(-40, 40, n).astype(F[dt])                 # many ties: the first one must win
        t = on(device, x)
        for kind in ("min", "max"):
            assert device.reduce_index(kind, t) == orc.reduce_index(kind, x), (kind, n)
    x = rng.standard_normal(5000).astype(F[dt])
    for at in (0, 64, 70, 4096, 4999):                              # NaNs: sticky only where they open a tile
        y = x.copy(); y[at] = np.nan
        t = on(device, y)
        for kind in ("min", "max"):
            assert device.reduce_index(kind, t) == orc.reduce_index(kind, y), (kind, at)
    assert _lib.last_path() == "tile_tree_64"


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_dot_product(device, orc, dt):
    rng = np.random.default_rng(63)
    for n in (1, 5, 128, 129, 32768, 32769, 100003):
        say("dot", dt, n)
        a, b = rng.standard_normal(n).astype(F[dt]), rng.standard_normal(n).astype(F[dt])
        got = on(device, a).dot(on(device, b)).items
        # rounded products summed in the tree of CPUSum: bit for bit
        assert_bits(got, np.array([orc.sum_tree(a * b)], dtype=F[dt]), f"dot as multiply + sum, n={n}")
        # against the CPU device's DOT.unrolled04 (another summation order): norm-wise
        want = orc.dot(a, b)
        assert abs(float(got[0]) - float(want)) <= RTOL[np.dtype(F[dt])] * float(np.abs(a * b).sum()) + 1e-30
        ai, bi = rng.integers(-9, 10, n).astype(F[dt]), rng.integers(-9, 10, n).astype(F[dt])
        assert on(device, ai).dot(on(device, bi)).items[0] == orc.dot(ai, bi)       # exact on small integers
    with pytest.raises(IllegalArgumentException):
        on(device, np.ones(3, dtype=F[dt])).dot(on(device, np.ones(4, dtype=F[dt])))


# ---- randomised views: every plan of the elementwise engine against the oracle walking the same descriptors ------
def _random_view(device, rng, shape, dt):
    """A tensor of the given shape that is a random permutation of a random strided slice of a larger parent.
    Returns (view, parent data)."""
    rank = len(shape)
    perm = list(rng.permutation(rank))
    pre = [0] * rank                      # shape of the slice: permute(*perm) must turn it into `shape`
    for k in range(rank):
        pre[perm[k]] = shape[k]
    starts = [int(rng.integers(0, 3)) for _ in range(rank)]
    steps = [int(rng.integers(1, 4)) for _ in range(rank)]
    parent_shape = [starts[k] + (pre[k] - 1) * steps[k] + 1 + int(rng.integers(0, 2)) for k in range(rank)]
    data = rng.uniform(-2, 2, parent_shape).astype(dt)
    t = on(device, data)
    sl = t[tuple(slice(starts[k], starts[k] + (pre[k] - 1) * steps[k] + 1, steps[k]) for k in range(rank))]
    assert list(sl.shape) == pre
    v = sl.permute(*perm) if rank > 1 else sl
    assert list(v.shape) == list(shape)
    return v, data


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_random_views_through_every_kernel_plan(device, orc, dt):
    T = F[dt]
    rng = np.random.default_rng(77)
    paths = set()
    for case in range(160):
        rank = int(rng.integers(1, 6))
        shape = [int(rng.choice([1, 2, 3, 4, 5, 7, 8, 16, 33])) for _ in range(rank)]
        while int(np.prod(shape)) > 6000:
            shape[int(np.argmax(shape))] = 2
        kind = ("elementwise", "activation", "scalarization", "broadcast")[case % 4]
        say("random view", case, kind, shape, dt)
        n = int(np.prod(shape))
        if kind == "broadcast":
            sa = [s if rng.random() < 0.6 else 1 for s in shape]
            sb = [s if (a == 1 or rng.random() < 0.6) else 1 for s, a in zip(shape, sa)]
            so = [max(a, b) for a, b in zip(sa, sb)]
            (va, da), (vb, db) = _random_view(device, rng, sa, T), _random_view(device, rng, sb, T)
            out = Tensor._on_device(device, T, so)
            op = str(rng.choice(["add", "subtract", "multiply"]))
            device.launch_broadcast(op, -1, out, va, vb)
            want = orc.broadcast(op, -1, np.zeros(out.size, dtype=T), cfg(out), da.reshape(-1), cfg(va), db.reshape(-1), cfg(vb))
            assert_bits(out.getData(), want, f"case {case} broadcast {op} {sa} {sb}")
        else:
            (va, da), (vb, db) = _random_view(device, rng, shape, T), _random_view(device, rng, shape, T)
            drain_is_view = rng.random() < 0.3
            if drain_is_view:
                vo, do = _random_view(device, rng, shape, T)
                host_out = do.reshape(-1).copy()
            else:
                vo = Tensor._on_device(device, T, shape); host_out = np.zeros(n, dtype=T)
            if kind == "elementwise":
                op = str(rng.choice(["add", "subtract", "multiply", "divide"]))
                device.launch_elementwise(op, -1, vo, va, vb)
                want = orc.elementwise(op, -1, host_out, cfg(vo), da.reshape(-1), cfg(va), db.reshape(-1), cfg(vb))
            elif kind == "activation":
                fun = str(rng.choice(["relu", "quad", "abs", "idy", "softsign"]))
                device.launch_activation(fun, -1, vo, va)
                want = orc.activation(fun, -1, host_out, cfg(vo), da.reshape(-1), cfg(va))
            else:
                op = str(rng.choice(["add", "multiply", "divide", "idy"]))
                device.launch_scalarization(op, -1, vo, va, 1.75)
                want = orc.scalarization(op, -1, host_out, cfg(vo), da.reshape(-1), cfg(va), 1.75)
            got = device._read_all(vo._data) if drain_is_view else vo.getData()
            assert_bits(got, want, f"case {case} {kind} {shape}")
        paths.add(_lib.last_path())
    say("plans seen", sorted(paths))
    assert {"rows", "canon"} <= {p.split("_")[0] for p in paths}
