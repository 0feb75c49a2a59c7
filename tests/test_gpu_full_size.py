"""The five benchmark configurations at their full sizes, through the C ABI.  Where the oracle finishes in
seconds the whole result is compared; the 4 GiB broadcast and the 4096^3 matmul are checked through
sampled slabs plus size-independent properties (linearity, exactness on integer data, a checksum)."""
import numpy as np
import pytest

from helpers import RTOL, assert_bits
from neureka_amd import Function, NDConfiguration, Tensor, _lib

pytestmark = pytest.mark.gpu
f32 = np.float32


def say(*a):
    print("[case]", *a, flush=True)


def on(device, array, shape=None):
    array = np.asarray(array)
    return Tensor.of(array.dtype, shape if shape is not None else array.shape, array.reshape(-1)).to(device)


def free(device, *tensors):
    for t in tensors:
        if device.has(t):
            device.free(t)


def test_config1_conv2d_64x64_3x3(device, orc):
    say("C1 conv2d")
    rng = np.random.default_rng(1)
    x = rng.uniform(-1, 1, (64, 64)).astype(f32); k = rng.uniform(-1, 1, (3, 3)).astype(f32)
    y = on(device, x).conv(on(device, k))
    assert y.shape == (62, 62)
    want = orc.simple_conv2d(x.reshape(-1), k.reshape(-1), 64, 64, 3, 3)          # the path the reference takes for this config
    assert _lib.last_path() == "simple2d"
    assert_bits(y.items, want, "SimpleCPUConvolution order")
    # the general nd path (what the reference's OpenCL kernel computes) sums the same products in another order
    general = orc.convolve(np.zeros(62 * 62, dtype=f32), orc.dense_cfg([62, 62]), x.reshape(-1), orc.dense_cfg([64, 64]), k.reshape(-1), orc.dense_cfg([3, 3]))
    bound = 1e-5 * orc.simple_conv2d(np.abs(x).reshape(-1), np.abs(k).reshape(-1), 64, 64, 3, 3)
    assert (np.abs(y.items - general) <= bound).all()


@pytest.mark.parametrize("dt,s1,s2", [("f32", (1024, 1, 512), (1, 2048, 512)), ("f64", (256, 1, 512), (1, 1024, 512))])
def test_config2_broadcast_full_size(device, orc, dt, s1, s2):
    say("C2 broadcast", dt)
    T = np.dtype(dt.replace("f", "float"))
    rng = np.random.default_rng(2)
    a = rng.uniform(-1, 1, s1).astype(T); b = rng.uniform(-1, 1, s2).astype(T)
    ta, tb = on(device, a), on(device, b)
    so = (s1[0], s2[1], 512)
    out = Tensor._on_device(device, T, so)
    for op, f in (("add", np.add), ("multiply", np.multiply)):
        device.launch_broadcast(op, -1, out, ta, tb)
        assert _lib.last_path() == "rows_vec_binary_lean"      # 64 MiB and more with re-used sources: one unit per block
        got = out.getData().reshape(so)
        # slabs against the oracle (bit for bit) ...
        for o0 in (0, 1, so[0] // 2, so[0] - 1):
            want = orc.broadcast(op, -1, np.zeros(so[1] * 512, dtype=T), orc.dense_cfg((1, so[1], 512)), a[o0].reshape(-1).copy(),
                                 orc.dense_cfg((1, 1, 512)), b.reshape(-1), orc.dense_cfg(s2))
            assert_bits(got[o0].reshape(-1), want, f"{op} slab {o0}")
        # ... and the whole 4 GiB / 1 GiB against numpy broadcasting, slab by slab to bound host memory
        for lo in range(0, so[0], 64):
            assert_bits(got[lo:lo + 64], f(a[lo:lo + 64], b), f"{op} rows {lo}")
        del got
    free(device, out, ta, tb)


def test_config2_broadcast_backward_full_size(device, orc):
    """The reducing backward of config 2: error [1024,2048,512] -> gradients of shape [1024,1,512] and [1,2048,512].
    Integer-valued errors make every order of summation exact (numpy is the check); a slab with random
    errors is compared bit for bit with the oracle's state machine."""
    rng = np.random.default_rng(22)
    shape = (1024, 2048, 512)
    say("C2 backward, integer-valued error")
    e = rng.integers(-4, 5, shape).astype(f32)
    te = on(device, e)
    for d, tgt, oth in ((0, (1024, 1, 512), (1, 2048, 512)), (1, (1, 2048, 512), (1024, 1, 512))):
        drn = Tensor._on_device(device, f32, tgt)
        zeros = Tensor._on_device(device, f32, oth)
        device.launch_broadcast("add", d, drn, zeros, te)
        assert _lib.last_path() == "broadcast_backward_vec_pairs"
        assert_bits(drn.getData().reshape(tgt), e.sum(axis=1 - d, keepdims=True, dtype=np.float64).astype(f32), f"gradient {d}")
        free(device, drn, zeros)
    free(device, te)
    del e
    say("C2 backward, random error, slabs against the oracle")
    # enough slabs that the kernel which keeps the reference's order is the one that runs (gradients with few
    # elements and long sums take the kernel that splits the sums, which is compared norm-wise elsewhere)
    for d, sub, tgt, oth in ((0, (128, 2048, 512), (128, 1, 512), (1, 2048, 512)), (1, (8, 2048, 512), (1, 2048, 512), (8, 1, 512))):
        e = rng.standard_normal(sub).astype(f32)
        te = on(device, e)
        drn = Tensor._on_device(device, f32, tgt)
        zeros = Tensor._on_device(device, f32, oth)
        device.launch_broadcast("add", d, drn, zeros, te)
        assert _lib.last_path() in ("broadcast_backward_vec", "broadcast_backward_vec_pairs")
        want = orc.broadcast("add", d, np.zeros(drn.size, dtype=f32), orc.dense_cfg(tgt), np.zeros(int(np.prod(oth)), dtype=f32), orc.dense_cfg(oth),
                             e.reshape(-1), orc.dense_cfg(sub), workers=16)
        assert_bits(drn.getData(), want, f"slab gradient {d}")
        free(device, drn, zeros, te)


def _chain_oracle(orc, bases, cfgs, shape, workers=16):
    n = int(np.prod(shape))
    oc = orc.dense_cfg(list(shape))
    s = orc.activation("sig", -1, np.zeros(n, dtype=f32), oc, bases[0], cfgs[0], workers=workers)
    m = orc.elementwise("multiply", -1, np.zeros(n, dtype=f32), oc, s, oc, bases[1], cfgs[1], workers=workers)
    p = orc.elementwise("add", -1, np.zeros(n, dtype=f32), oc, m, oc, bases[2], cfgs[2], workers=workers)
    want = orc.activation("tanh", -1, np.zeros(n, dtype=f32), oc, p, oc, workers=workers)
    return want, m


def _check_chain(got, want, m, c_view, what=""):
    """Where the sum p = m + c (m = sig(a) * b) does not cancel, |m + c| >= (|m| + |c|) / 2, the fused output is held to
    plain rtol 1e-5 of the oracle's.  Elsewhere the inner sigmoid's own tolerance is no longer small against p: it may differ
    from the reference's by 1e-5 relative, i.e. m by 1e-5 |m|, which enters p absolutely (tanh' <= 1), plus one rounding
    of the sum, 2^-23 (|m| + |c|) -- the propagated bound.  The share of elements under each bound is printed."""
    c_view = c_view.astype(np.float64); m64 = m.astype(np.float64)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    plain = np.abs(m64 + c_view) >= 0.5 * (np.abs(m64) + np.abs(c_view))
    bad = plain & (err > RTOL[np.dtype(f32)] * np.abs(want) + 1e-30)
    assert not bad.any(), f"{what}: {bad.sum()} of {plain.sum()} elements without cancellation outside plain rtol 1e-5; first {np.flatnonzero(bad)[:3]}"
    bound = RTOL[np.dtype(f32)] * (np.abs(m64) + np.abs(want)) + 2.0 ** -23 * (np.abs(m64) + np.abs(c_view)) + 1e-10
    bad = ~plain & (err > bound)
    assert not bad.any(), f"{what}: {bad.sum()} of {(~plain).sum()} cancelling elements outside the propagated bound; first {np.flatnonzero(bad)[:3]}"
    with np.errstate(all="ignore"):
        worst = float(np.max(np.where(plain & (np.abs(want) > 0), err / np.abs(want), 0.0)))
    print(f"[chain] {what}: {plain.mean() * 100:.2f} % of {plain.size} elements under plain rtol 1e-5 (worst relative error {worst:.2e}), "
          f"{(~plain).mean() * 100:.2f} % under the propagated bound", flush=True)


def test_config3_chain_contiguous_permuted_sliced(device, orc):
    """tanh(sig(a)*b+c): 2^26 contiguous elements, the permuted [4096,16384] view of row-major [16384,4096],
    and the slice [::2, 1:8193] of [8192,16384]; fused kernel against the oracle's four-kernel sequence."""
    rng = np.random.default_rng(3)
    fn = Function.of("tanh(sig(I[0])*I[1]+I[2])")
    fused = device.optimizedFunctionOf(fn, "chain")
    n = 1 << 26
    bases = [rng.standard_normal(n).astype(f32) for _ in range(3)]
    tens = [on(device, b, (16384, 4096)) for b in bases]
    say("C3 contiguous")
    flat = [Tensor(f32, NDConfiguration.ofShape((n,)), None) for _ in tens]
    for v, t in zip(flat, tens): v._set_data(t._data, device)
    got = fused(*flat)
    assert _lib.last_path() == "rows_vec"
    cfg1 = orc.dense_cfg([n])
    want, m = _chain_oracle(orc, bases, [cfg1] * 3, (n,))
    _check_chain(got.items, want, m, bases[2], "contiguous")
    free(device, got)
    say("C3 permuted")
    views = [t.T() for t in tens]
    got = fused(*views)
    assert _lib.last_path() == "tile_transpose" and got.shape == (4096, 16384)
    cfgs = [v.ndc.asInlineArray() for v in views]
    want, m = _chain_oracle(orc, bases, cfgs, (4096, 16384))
    _check_chain(got.items, want, m, bases[2].reshape(16384, 4096).T.reshape(-1), "permuted")
    unf = fn(*views)                                                     # the reference's four launches
    assert_bits(unf.items, got.items, "fused vs unfused, permuted")
    free(device, got, unf, *views, *tens)
    say("C3 sliced")
    parents = [rng.standard_normal(8192 * 16384).astype(f32) for _ in range(3)]
    ptens = [on(device, p, (8192, 16384)) for p in parents]
    views = [t[::2, 1:8193] for t in ptens]
    assert views[0].ndc.asInlineArray().tolist() == [4096, 8192, 16384, 1, 8192, 1, 0, 1, 2, 1]
    got = fused(*views)
    assert _lib.last_path() == "rows_vec" and got.shape == (4096, 8192)
    cfgs = [v.ndc.asInlineArray() for v in views]
    want, m = _chain_oracle(orc, parents, cfgs, (4096, 8192))
    _check_chain(got.items, want, m, parents[2].reshape(8192, 16384)[::2, 1:8193].reshape(-1), "sliced")
    free(device, got, *views, *ptens)


@pytest.mark.parametrize("mkn", [(4096, 4096, 4096), (65536, 256, 256)])
def test_config4_matmul_full_size(device, orc, mkn):
    M, K, N = mkn
    rng = np.random.default_rng(4)
    say("C4 matmul integer data (exact)", mkn)
    A = rng.integers(-3, 4, (M, K)).astype(f32); B = rng.integers(-3, 4, (K, N)).astype(f32)
    ta, tb = on(device, A), on(device, B)
    c = ta.matMul(tb)
    assert _lib.last_path() == ("mfma_big" if K == 4096 else "mfma_stream")  # 256 tiles of 256 x 256: one per compute unit; few k-slices per tile: the blocks walk the tiles
    got = c.items.reshape(M, N)
    rows = rng.choice(M, 48, replace=False)
    assert (got[rows] == A[rows].astype(np.float64) @ B.astype(np.float64)).all()
    # checksum of checksums over the whole product: 1^T (A B) 1 = (1^T A)(B 1), exact in float64 for this data
    assert got.sum(dtype=np.float64) == float(A.sum(axis=0, dtype=np.float64) @ B.sum(axis=1, dtype=np.float64))
    free(device, c, ta, tb)
    say("C4 matmul uniform data (norm-wise 1e-5)", mkn)
    A = rng.uniform(-1, 1, (M, K)).astype(f32); B = rng.uniform(-1, 1, (K, N)).astype(f32)
    ta, tb = on(device, A), on(device, B)
    c = ta.matMul(tb)
    got = c.items.reshape(M, N)
    ref = A[rows].astype(np.float64) @ B.astype(np.float64)
    bound = 1e-5 * (np.abs(A[rows]).astype(np.float64) @ np.abs(B).astype(np.float64))
    assert (np.abs(got[rows] - ref) <= bound).all()
    # the whole product against the oracle's GEMM (GEMM.threaded_F32_MxN_RM restated, float sums in k order), every
    # element within 1e-5 sum_k |a_ik| |b_kj| (that sum from a float product: the bound needs two digits, not seven)
    want = orc.gemm(True, A.reshape(-1), B.reshape(-1), M, K, N, workers=16).reshape(M, N)
    whole = 1e-5 * (np.abs(A) @ np.abs(B)).astype(np.float64)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert (err <= whole).all(), f"{(err > whole).sum()} of {M * N} elements outside the norm-wise bound"
    print(f"[matmul] {mkn}: worst |delta| / sum|a||b| over all {M * N} elements {float(np.max(err / whole)) * 1e-5:.2e}", flush=True)
    # linearity: (2A) B == 2 (A B) bit for bit (scaling by a power of two is exact)
    c2 = on(device, 2 * A).matMul(tb)
    assert_bits(c2.items, 2 * c.items, "linearity")
    free(device, c, c2, ta, tb)


def test_config5_conv_forward_and_backward_full_size(device, orc):
    """[64,256,256] x [64,5,5] -> [1,252,252] with autograd: input and kernel gradients."""
    rng = np.random.default_rng(5)
    xs, ks, ys = [64, 256, 256], [64, 5, 5], [1, 252, 252]
    x = (rng.standard_normal(xs) * 0.1).astype(f32); k = (rng.standard_normal(ks) * 0.1).astype(f32)
    e = rng.standard_normal(ys).astype(f32)
    tx = on(device, x).setRqsGradient(True); tk = on(device, k).setRqsGradient(True)
    say("C5 forward")
    y = tx.conv(tk)
    assert _lib.last_path() == "chan_fwd_tiles" and list(y.shape) == ys      # one launch: every block reduces all channels of its tile
    dc = orc.dense_cfg
    want = orc.convolve(np.zeros(252 * 252, dtype=f32), dc(ys), x.reshape(-1), dc(xs), k.reshape(-1), dc(ks), workers=16)
    babs = orc.convolve(np.zeros(252 * 252), dc(ys), np.abs(x).astype(np.float64).reshape(-1), dc(xs), np.abs(k).astype(np.float64).reshape(-1), dc(ks), workers=16)
    assert (np.abs(y.items.astype(np.float64) - want) <= 1e-5 * babs).all()
    say("C5 backward")
    y.backward(on(device, e))
    gx, gk = tx.gradient, tk.gradient
    assert list(gx.shape) == xs and list(gk.shape) == ks
    want = orc.deconvolve(np.zeros(x.size, dtype=f32), dc(xs), k.reshape(-1), dc(ks), e.reshape(-1), dc(ys), fast=True, workers=16)
    babs = orc.deconvolve(np.zeros(x.size), dc(xs), np.abs(k).astype(np.float64).reshape(-1), dc(ks), np.abs(e).astype(np.float64).reshape(-1), dc(ys), fast=True, workers=16)
    assert (np.abs(gx.items.astype(np.float64) - want) <= 1e-5 * babs + 1e-30).all()
    want = orc.deconvolve(np.zeros(k.size, dtype=f32), dc(ks), x.reshape(-1), dc(xs), e.reshape(-1), dc(ys), fast=True, workers=16)
    babs = orc.deconvolve(np.zeros(k.size), dc(ks), np.abs(x).astype(np.float64).reshape(-1), dc(xs), np.abs(e).astype(np.float64).reshape(-1), dc(ys), fast=True, workers=16)
    assert (np.abs(gk.items.astype(np.float64) - want) <= 1e-5 * babs).all()
    # adjoint identity in float64: <e, x (*) k> = <dL/dx, x> = <dL/dk, k>
    lhs = float(np.dot(e.reshape(-1).astype(np.float64), y.items.astype(np.float64)))
    assert abs(float(np.dot(gx.items.astype(np.float64), x.reshape(-1).astype(np.float64))) - lhs) <= 1e-4 * abs(lhs) + 1e-6
    assert abs(float(np.dot(gk.items.astype(np.float64), k.reshape(-1).astype(np.float64))) - lhs) <= 1e-4 * abs(lhs) + 1e-6


def test_reductions_over_2_pow_26_elements(device, orc):
    """sum, min/max index and dot product of the chain's operand size: the CPU device's trees, bit for bit."""
    rng = np.random.default_rng(6)
    n = 1 << 26
    a = rng.standard_normal(n).astype(f32); b = rng.standard_normal(n).astype(f32)
    ta, tb = on(device, a), on(device, b)
    say("sum 2^26")
    assert_bits(ta.sum().items, np.array([orc.sum_tree(a)], dtype=f32), "sum")
    assert abs(float(ta.sum().items[0]) - float(a.sum(dtype=np.float64))) <= 1e-5 * float(np.abs(a).sum(dtype=np.float64))
    say("min / max 2^26")
    assert device.reduce_index("min", ta) == orc.reduce_index("min", a) == int(np.argmin(a))
    assert device.reduce_index("max", ta) == orc.reduce_index("max", a) == int(np.argmax(a))
    say("dot 2^26")
    got = ta.dot(tb).items
    assert_bits(got, np.array([orc.sum_tree(a * b)], dtype=f32), "dot as multiply + sum")
    assert abs(float(got[0]) - float(np.dot(a.astype(np.float64), b.astype(np.float64)))) <= 1e-5 * float(np.abs(a * b).sum(dtype=np.float64))
    free(device, ta, tb)


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_large_broadcast_outputs_one_unit_per_block(device, orc, dt):
    """Outputs of 64 MiB and more whose sources are re-used take the binary kernel's variant with one unit per block and
    non-temporal stores: rows longer than a block (several column chunks), row counts that leave the last block half
    empty, one to three outer axes, a source that is a slice of a larger tensor, all four operators -- every result
    bit for bit the oracle's (numpy's single IEEE operation per element for + - * /)."""
    T = np.dtype(dt.replace("f", "float"))
    scale = 1 if dt == "f32" else 2                      # the same number of bytes in f64
    rng = np.random.default_rng(9)
    cases = [("add", (4096 // scale, 4100), (1, 4100), None),
             ("subtract", (4099 // scale, 1, 512), (1, 9, 512), None),
             ("multiply", (70 // scale, 1, 17, 256), (1, 61, 1, 256), None),
             ("divide", (4096 // scale, 1, 260), (1, 17, 260), None),
             ("add", (4096 // scale, 4100), (1, 4100), "sliced"),
             ("multiply", (1, 4100), (4096 // scale, 4100), None),
             ("multiply", (8192 // scale, 1), (1, 4096), None),              # an outer product: both sources constant along a row or a column
             ("add", ((1 << 20) // scale, 1), (1, 32), None),               # short rows: several rows per wavefront
             ("subtract", ((1 << 19) // scale, 64), (1, 64), None),
             ("divide", (300 // scale, 1, 70, 1), (1, 50, 1, 64), None),
             ("add", (4096 // scale, 4099), (1, 4099), None),                # rows that are no multiple of a vector
             ("subtract", (1, 9, 515), (4099 // scale, 1, 515), None),
             ("add", (33 // scale + 1, 1, 1021, 64), (1, 9, 1, 64), None),   # three outer axes above rows of 64 elements
             ("multiply", (524289 // scale, 32), (524289 // scale, 1), None)]  # an odd number of short rows, a per-row scale
    for op, sa, sb, view in cases:
        so = tuple(max(p, q) for p, q in zip(sa, sb))
        say("large broadcast", op, sa, sb, view or "", dt)
        assert int(np.prod(so)) * T.itemsize >= 64 << 20
        b = rng.uniform(0.5, 1.5, sb).astype(T)
        tb = on(device, b)
        if view == "sliced":                              # rows of a wider parent, starting 16 bytes in
            pad = 16 // T.itemsize
            parent = rng.uniform(-1, 1, (sa[0] + 2, sa[1] + 2 * pad)).astype(T)
            ta = on(device, parent)[1:1 + sa[0], pad:pad + sa[1]]
            a = parent[1:1 + sa[0], pad:pad + sa[1]]
        else:
            a = rng.uniform(-1, 1, sa).astype(T)
            ta = on(device, a)
        out = Tensor._on_device(device, T, so)
        device.launch_broadcast(op, -1, out, ta, tb)
        flat = sa[-1] == 515 and dt == "f32"       # ragged rows of 129 vectors: half the one-unit kernel's lanes would idle
        assert _lib.last_path() == ("rows_vec_binary" if flat else "rows_vec_binary_lean"), _lib.last_path()
        f = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply, "divide": np.divide}[op]
        assert_bits(out.getData().reshape(so), f(a, b).astype(T), f"{op} {sa} {sb}")
        # ... and a slab through the oracle's own state machine
        rows = 3
        first = tuple(slice(0, min(rows, s)) if k == 0 else slice(None) for k, s in enumerate(so))
        ssa = tuple(min(rows, s) if k == 0 else s for k, s in enumerate(sa)); ssb = tuple(min(rows, s) if k == 0 else s for k, s in enumerate(sb))
        sso = tuple(max(p, q) for p, q in zip(ssa, ssb))
        want = orc.broadcast(op, -1, np.zeros(int(np.prod(sso)), dtype=T), orc.dense_cfg(sso), np.ascontiguousarray(a[first[:len(sa)]] if sa[0] > 1 else a).reshape(-1),
                             orc.dense_cfg(ssa), np.ascontiguousarray(b[first[:len(sb)]] if sb[0] > 1 else b).reshape(-1), orc.dense_cfg(ssb))
        assert_bits(out.getData().reshape(so)[first].reshape(-1), want, f"oracle slab {op}")
        free(device, ta, tb, out)


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_large_scalar_fills_one_unit_per_block(device, dt):
    """Fills of 64 MiB and more through the elementwise engine: dense tensors take the variant with one unit per block,
    slices of larger tensors the general rows kernel; every element of the view takes the value, everything around a
    sliced view stays as it was."""
    T = np.dtype(dt.replace("f", "float"))
    scale = 1 if dt == "f32" else 2
    say("large fill, dense", dt)
    t = Tensor._on_device(device, T, (4099 // scale, 4100))
    device.launch_scalar_fill(t, -2.5)
    assert _lib.last_path() == "rows_vec_fill_lean", _lib.last_path()
    assert (t.getData() == T.type(-2.5)).all()
    free(device, t)
    for shape, sl in (((4100 // scale, 4200), (slice(1, 4097 // scale), slice(8, 4108))),
                      ((70 // scale, 61, 17, 272), (slice(None), slice(2, 60), slice(None), slice(8, 264)))):
        say("large fill, sliced", shape, dt)
        parent = Tensor._on_device(device, T, shape)
        device.launch_scalar_fill(parent, 1.0)
        view = parent[sl]
        assert view.size * T.itemsize >= 64 << 20
        device.launch_scalar_fill(view, 7.25)
        assert _lib.last_path() == "rows_vec", _lib.last_path()              # a drain with gaps keeps the kernel with several units per block
        want = np.ones(shape, dtype=T); want[sl] = 7.25
        assert parent.getData().tobytes() == want.tobytes()
        free(device, parent)
