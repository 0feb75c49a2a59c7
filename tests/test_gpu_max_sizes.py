"""Tensors at the largest sizes the boundary accepts: 2^31-1 elements (a Java array's limit, what every entry point
states as its own), i.e. buffers of 8 GiB (f32, int32) and 16 GiB (f64) whose byte offsets no longer fit 32 bits.
Checked in full where one numpy operation is the oracle (+ - * /, fills, integer-valued sums and products), through
the C oracle where it defines the order (the reduction trees; the reference's own tile arithmetic `offset + RTS`
overflows an int beyond 2^31-128 elements, so the reductions stop there) and on slabs at both ends and across the
4 GiB boundary for the transcendental kernels."""
import numpy as np
import pytest

from helpers import assert_bits, assert_close
from neureka_amd import NDConfiguration, Tensor, _lib

pytestmark = pytest.mark.gpu
f32, f64, i32 = np.float32, np.float64, np.int32
NMAX = (1 << 31) - 1
NRED = (1 << 31) - 129          # the largest odd size whose last tile of 128 still ends below 2^31


def say(*a):
    print("[case]", *a, flush=True)


def on(device, array, shape=None):
    array = np.asarray(array)
    return Tensor.of(array.dtype, shape if shape is not None else array.shape, array.reshape(-1)).to(device)


def free(device, *tensors):
    for t in tensors:
        if device.has(t):
            device.free(t)


def big(rng, n, dtype, integers=None):
    """n values without drawing n random numbers: a random block of 2^24 scaled by 128 random factors (or, integers =
    (lo, hi), a block of small integers repeated with a random integer offset per repetition)."""
    block = 1 << 24
    reps = (n + block - 1) // block
    if integers is None:
        base = rng.standard_normal(block).astype(dtype)
        scale = rng.uniform(0.5, 2.0, reps).astype(dtype)
        return (scale[:, None] * base[None, :]).reshape(-1)[:n]
    lo, hi = integers
    base = rng.integers(lo, hi + 1, block).astype(dtype)
    sign = rng.choice(np.array([-1, 1], dtype=dtype), reps)
    return (sign[:, None] * base[None, :]).reshape(-1)[:n]


def same(got, want, what):
    assert got.dtype == want.dtype and got.shape == want.shape, f"{what}: {got.dtype}{got.shape} vs {want.dtype}{want.shape}"
    u = {4: np.uint32, 8: np.uint64}[got.dtype.itemsize]
    if not np.array_equal(got.view(u), want.view(u)):
        bad = np.flatnonzero(got.view(u) != want.view(u))
        raise AssertionError(f"{what}: {bad.size} of {want.size} values differ in bits; first at {bad[0]}: {got[bad[0]]!r} vs {want[bad[0]]!r}")


SLABS = ((0, 1 << 22), ((1 << 30) - (1 << 21), (1 << 30) + (1 << 21)), (NMAX - (1 << 22), NMAX))


def test_elementwise_f32_at_2_pow_31_minus_1(device, orc):
    rng = np.random.default_rng(31)
    a = big(rng, NMAX, f32); b = big(rng, NMAX, f32)
    ta, tb = on(device, a), on(device, b)
    out = Tensor._on_device(device, f32, (NMAX,))
    for op, f in (("add", np.add), ("divide", np.divide)):
        say("max size", op, "f32")
        device.launch_elementwise(op, -1, out, ta, tb)
        print("[path]", _lib.last_path(), flush=True)
        same(out.getData(), f(a, b), op)
    say("max size scalar multiply f32")
    device.launch_scalarization("multiply", -1, out, ta, 3.0)
    print("[path]", _lib.last_path(), flush=True)
    same(out.getData(), a * f32(3.0), "scalar multiply")
    say("max size fill f32")
    device.launch_scalar_fill(out, -2.5)
    print("[path]", _lib.last_path(), flush=True)
    got = out.getData()
    assert got.size == NMAX and (got == f32(-2.5)).all()
    del got
    for fun in ("tanh", "sig"):
        say("max size", fun, "f32")
        device.launch_activation(fun, -1, out, ta)
        print("[path]", _lib.last_path(), flush=True)
        got = out.getData()
        for lo, hi in SLABS:
            cfg = orc.dense_cfg([hi - lo])
            want = orc.activation(fun, -1, np.zeros(hi - lo, dtype=f32), cfg, np.ascontiguousarray(a[lo:hi]), cfg, workers=16)
            assert_close(got[lo:hi], want, f"{fun} [{lo}:{hi}]")
        assert np.isfinite(got).all() and (np.abs(got) <= 1).all()
        del got
    free(device, ta, tb, out)


def test_reductions_f32_at_2_pow_31_minus_129(device, orc):
    rng = np.random.default_rng(32)
    a = big(rng, NRED, f32); b = big(rng, NRED, f32)
    a[NRED - 2] = 1e6; a[(1 << 30) + 5] = -1e6            # the winners sit behind the 4 GiB boundary and at the very end
    ta, tb = on(device, a), on(device, b)
    say("max size sum f32")
    assert_bits(ta.sum().items, np.array([orc.sum_tree(a)], dtype=f32), "sum")
    say("max size min / max index f32")
    assert device.reduce_index("max", ta) == orc.reduce_index("max", a) == NRED - 2
    assert device.reduce_index("min", ta) == orc.reduce_index("min", a) == (1 << 30) + 5
    say("max size dot f32")
    assert_bits(ta.dot(tb).items, np.array([orc.sum_tree(a * b)], dtype=f32), "dot as multiply + sum")
    free(device, ta, tb)


def test_broadcast_forward_and_backward_into_8_gib(device, orc):
    rng = np.random.default_rng(33)
    sa, sb, so = (2047, 1, 512), (1, 2048, 512), (2047, 2048, 512)
    a = rng.integers(-1, 2, sa).astype(f32); b = rng.integers(-1, 2, sb).astype(f32)
    ta, tb = on(device, a), on(device, b)
    out = Tensor._on_device(device, f32, so)
    say("max size broadcast add", sa, sb)
    device.launch_broadcast("add", -1, out, ta, tb)
    print("[path]", _lib.last_path(), flush=True)
    e = a + b
    same(out.getData().reshape(so), e, "broadcast add")
    for d, tgt, oth, axes in ((0, sa, sb, (1,)), (1, sb, sa, (0,)), (0, (1, 1, 512), (2047, 2048, 1), (0, 1)), (0, (2047, 1, 1), sb, (1, 2))):
        say("max size broadcast backward ->", tgt)
        drn = Tensor._on_device(device, f32, tgt)
        zeros = Tensor._on_device(device, f32, oth)
        device.launch_broadcast("add", d, drn, zeros, out)
        print("[path]", _lib.last_path(), flush=True)
        same(drn.getData().reshape(tgt), e.sum(axis=axes, keepdims=True, dtype=np.float64).astype(f32), f"gradient {tgt}")
        free(device, drn, zeros)
    free(device, ta, tb, out)


def test_matmul_into_8_gib(device):
    rng = np.random.default_rng(34)
    for M, K, N, path in ((65408, 64, 32768, "mfma_stream"), (65535, 64, 32768, "mfma_tiles_of_64_edge")):
        say("max size matmul", (M, K, N))
        A = rng.integers(-3, 4, (M, K)).astype(f32); B = rng.integers(-3, 4, (K, N)).astype(f32)
        want = A @ B
        ta, tb = on(device, A), on(device, B)
        c = Tensor._on_device(device, f32, (M, N))
        device.launch_scalar_fill(c, 1.0)
        device.launch_matmul(True, M, K, N, ta, tb, c, accumulate=False)
        assert _lib.last_path() == path, _lib.last_path()
        same(c.getData().reshape(M, N), want, "C = A B")
        device.launch_matmul(True, M, K, N, ta, tb, c, accumulate=True)
        want *= 2
        same(c.getData().reshape(M, N), want, "C += A B")
        free(device, ta, tb, c)
        del want


def test_matmul_streams_over_8_gib(device):
    """The kernels that stream one large operand once, at the largest operand the entry point accepts (2^31 - 4096
    elements): a matrix times a vector, a vector times a matrix, an outer product.  Small integers: every sum is exact."""
    rng = np.random.default_rng(39)
    L, S = 524287, 4096                                     # L * S = 2^31 - 4096
    say("max size matmul: [L,S] @ [S,1]")
    A = big(rng, L * S, f32, integers=(-3, 3)).reshape(L, S); x = rng.integers(-3, 4, (S, 1)).astype(f32)
    ta, tx = on(device, A), on(device, x)
    c = Tensor._on_device(device, f32, (L, 1))
    device.launch_scalar_fill(c, 1.0)
    device.launch_matmul(True, L, S, 1, ta, tx, c, accumulate=False)
    assert _lib.last_path() == "few_cols", _lib.last_path()
    want = A @ x
    same(c.getData().reshape(L, 1), want, "C = A x")
    device.launch_matmul(True, L, S, 1, ta, tx, c, accumulate=True)
    same(c.getData().reshape(L, 1), want * 2, "C += A x")
    free(device, tx, c)
    say("max size matmul: [1,L] @ [L,S] (the same 8 GiB read as a matrix of S columns)")
    y = rng.integers(-3, 4, (1, L)).astype(f32)
    ty = on(device, y)
    c = Tensor._on_device(device, f32, (1, S))
    device.launch_scalar_fill(c, 1.0)
    device.launch_matmul(True, 1, L, S, ty, ta, c, accumulate=False)
    assert _lib.last_path() == "few_rows", _lib.last_path()
    want = (y.astype(np.float64) @ A.astype(np.float64)).astype(f32)     # |sums| < 2^24: exact either way
    same(c.getData().reshape(1, S), want, "C = y A")
    device.launch_matmul(True, 1, L, S, ty, ta, c, accumulate=True)
    same(c.getData().reshape(1, S), want * 2, "C += y A")
    free(device, ta, ty, c)
    del A, want
    say("max size matmul: [L,2] @ [2,S] into 8 GiB")
    u = rng.integers(-3, 4, (L, 2)).astype(f32); v = rng.integers(-3, 4, (2, S)).astype(f32)
    tu, tv = on(device, u), on(device, v)
    c = Tensor._on_device(device, f32, (L, S))
    device.launch_scalar_fill(c, 1.0)
    device.launch_matmul(True, L, 2, S, tu, tv, c, accumulate=False)
    assert _lib.last_path() == "short_inner", _lib.last_path()
    want = u @ v
    same(c.getData().reshape(L, S), want, "C = u v")
    device.launch_matmul(True, L, 2, S, tu, tv, c, accumulate=True)
    want *= 2
    same(c.getData().reshape(L, S), want, "C += u v")
    free(device, tu, tv, c)


def test_int32_scalar_operations_at_2_pow_31_minus_1(device, orc):
    rng = np.random.default_rng(35)
    x = big(rng, NMAX, i32, integers=(0, 1 << 30))
    tx = on(device, x)
    out = Tensor._on_device(device, i32, (NMAX,))
    cfg = orc.dense_cfg([NMAX])
    for op, v in (("multiply", 3), ("divide", 7)):
        say("max size int32", op)
        device.launch_scalarization(op, -1, out, tx, v)
        print("[path]", _lib.last_path(), flush=True)
        want = orc.scalarization_int(op, -1, np.zeros(NMAX, dtype=i32), cfg, x, cfg, v)
        assert np.array_equal(out.getData(), want), op
    free(device, tx, out)


def test_permuted_and_strided_views_of_8_gib(device):
    rng = np.random.default_rng(36)
    R, Cn = 32768, 65535                                   # R * Cn = 2^31 - 32768
    a = big(rng, R * Cn, f32).reshape(R, Cn); b = big(rng, R * Cn, f32).reshape(Cn, R)
    ta, tb = on(device, a), on(device, b)
    say("max size permuted add")
    out = Tensor._on_device(device, f32, (Cn, R))
    device.launch_elementwise("add", -1, out, ta.T(), tb)
    assert _lib.last_path() == "tile_transpose", _lib.last_path()
    same(out.getData().reshape(Cn, R), a.T + b, "a^T + b")
    free(device, out)
    say("max size doubly strided subtract")
    va, vb = ta[1::2, 3::2], tb.T()[1::2, 3::2]
    out = Tensor._on_device(device, f32, va.shape)
    device.launch_elementwise("subtract", -1, out, va, vb)
    print("[path]", _lib.last_path(), flush=True)
    same(out.getData().reshape(va.shape), a[1::2, 3::2] - b.T[1::2, 3::2], "strided views")
    free(device, out, va, vb, ta, tb)


def test_f64_add_and_sum_of_16_gib(device, orc):
    rng = np.random.default_rng(37)
    a = big(rng, NMAX, f64); b = big(rng, NMAX, f64)
    ta, tb = on(device, a), on(device, b)
    out = Tensor._on_device(device, f64, (NMAX,))
    say("max size add f64")
    device.launch_elementwise("add", -1, out, ta, tb)
    print("[path]", _lib.last_path(), flush=True)
    same(out.getData(), a + b, "add f64")
    free(device, out, tb)
    del b
    say("max size sum f64")
    free(device, ta)
    a = a[:NRED]
    ta = on(device, a)
    assert_bits(ta.sum().items, np.array([orc.sum_tree(a)], dtype=f64), "sum f64")
    say("max size max index f64")
    assert device.reduce_index("max", ta) == orc.reduce_index("max", a)
    free(device, ta)


def test_convolution_of_an_8_gib_image(device):
    """[32768, 65535] x [3, 3] as a plain 2-D convolution and as [1, 1, H, W] x [1, 1, 3, 3]: integer data, so every
    order of summation is exact; three bands of rows (the first, those around byte offset 4 GiB, the last) against the
    nine shifted products, and the sum of the whole result against the nine window sums of the image."""
    rng = np.random.default_rng(38)
    H, W = 32768, 65535
    x = big(rng, H * W, f32, integers=(-3, 3)).reshape(H, W)
    k = rng.integers(-2, 3, (3, 3)).astype(f32)
    OH, OW = H - 2, W - 2
    full_rows = x.sum(axis=1, dtype=np.float64)
    total = 0.0
    for kx in range(3):
        rows = full_rows - x[:, :kx].sum(axis=1, dtype=np.float64) - x[:, kx + OW:].sum(axis=1, dtype=np.float64)
        for ky in range(3):
            total += float(k[ky, kx]) * float(rows[ky:ky + OH].sum())
    mid = (1 << 30) // OW
    bands = ((0, 64), (mid - 32, mid + 32), (OH - 64, OH))
    tx = on(device, x)
    for shape_x, shape_k in (((H, W), (3, 3)), ((1, 1, H, W), (1, 1, 3, 3))):
        say("max size convolution", shape_x, shape_k)
        vx = Tensor(f32, NDConfiguration.ofShape(shape_x), None); vx._set_data(tx._data, device)
        y = vx.conv(on(device, k, shape_k))
        print("[path]", _lib.last_path(), flush=True)
        got = y.getData().reshape(OH, OW)
        for lo, hi in bands:
            want = np.zeros((hi - lo, OW), dtype=f32)
            for ky in range(3):
                for kx in range(3):
                    want += x[lo + ky:hi + ky, kx:kx + OW] * k[ky, kx]
            same(got[lo:hi], want, f"rows {lo}:{hi}")
        assert float(got.sum(dtype=np.float64)) == total
        free(device, y)
        del got
    # 2047 images of [1024, 1024] in one launch: the planes behind byte offset 4 GiB
    B, S = 2047, 1024
    say("max size batched convolution", (B, S, S), (1, 3, 3))
    x3 = x.reshape(-1)[:B * S * S].reshape(B, S, S)
    O = S - 2
    full_rows = x3.sum(axis=2, dtype=np.float64)
    total = 0.0
    for kx in range(3):
        rows = full_rows - x3[:, :, :kx].sum(axis=2, dtype=np.float64) - x3[:, :, kx + O:].sum(axis=2, dtype=np.float64)
        for ky in range(3):
            total += float(k[ky, kx]) * float(rows[:, ky:ky + O].sum())
    vx = Tensor(f32, NDConfiguration.ofShape((B, S, S)), None); vx._set_data(tx._data, device)
    y = vx.conv(on(device, k, (1, 3, 3)))
    assert _lib.last_path() == "simple2d_window", _lib.last_path()
    got = y.getData().reshape(B, O, O)
    for lo, hi in ((0, 2), (1023, 1026), (B - 2, B)):
        want = np.zeros((hi - lo, O, O), dtype=f32)
        for ky in range(3):
            for kx in range(3):
                want += x3[lo:hi, ky:ky + O, kx:kx + O] * k[ky, kx]
        same(got[lo:hi], want, f"images {lo}:{hi}")
    assert float(got.sum(dtype=np.float64)) == total
    free(device, y, tx)


def test_channel_convolution_with_autograd_over_8_gib(device):
    """[511, 2048, 2048] x [511, 3, 3] -> [1, 2046, 2046] and both gradients: channels behind byte offset 4 GiB, a
    gradient of 8 GiB.  Small integers keep every sum exact in any order: bands of rows / channels against numpy, and the
    sum of each whole result against its closed form."""
    from scipy.signal import convolve2d
    rng = np.random.default_rng(39)
    Cc, S, O = 511, 2048, 2046
    x = big(rng, Cc * S * S, f32, integers=(-3, 3)).reshape(Cc, S, S)
    k = rng.integers(-2, 3, (Cc, 3, 3)).astype(f32)
    e = rng.integers(-1, 2, (1, O, O)).astype(f32)
    tx = on(device, x).setRqsGradient(True); tk = on(device, k).setRqsGradient(True)
    say("max size channel convolution forward")
    y = tx.conv(tk)
    print("[path]", _lib.last_path(), flush=True)
    assert tuple(y.shape) == (1, O, O)
    got = y.getData().reshape(O, O)
    for lo, hi in ((0, 8), (1019, 1027), (O - 8, O)):
        want = np.zeros((hi - lo, O), dtype=np.float64)
        for ky in range(3):
            for kx in range(3):
                want += np.einsum("cyx,c->yx", x[:, lo + ky:hi + ky, kx:kx + O], k[:, ky, kx], dtype=np.float64)
        same(got[lo:hi], want.astype(f32), f"forward rows {lo}:{hi}")
    full_rows = x.sum(axis=2, dtype=np.float64)                          # [c, y]
    total = 0.0
    for kx in range(3):
        rows = full_rows - x[:, :, :kx].sum(axis=2, dtype=np.float64) - x[:, :, kx + O:].sum(axis=2, dtype=np.float64)
        for ky in range(3):
            total += float(np.dot(k[:, ky, kx].astype(np.float64), rows[:, ky:ky + O].sum(axis=1)))
    assert float(got.sum(dtype=np.float64)) == total
    say("max size channel convolution backward")
    y.backward(on(device, e))
    gx, gk = tx.gradient, tk.gradient
    assert tuple(gx.shape) == (Cc, S, S) and tuple(gk.shape) == (Cc, 3, 3)
    gxh = gx.getData().reshape(Cc, S, S)
    for c in (0, 1, 255, 256, 257, Cc - 1):
        same(gxh[c], convolve2d(e[0].astype(np.float64), k[c].astype(np.float64), mode="full").astype(f32), f"input gradient, channel {c}")
    assert float(gxh.sum(dtype=np.float64)) == float(e.sum(dtype=np.float64)) * float(k.sum(dtype=np.float64))
    del gxh
    gkh = gk.getData().reshape(Cc, 3, 3)
    e64 = e[0].astype(np.float64)
    for c in (0, 1, 255, 256, 257, Cc - 1):
        want = np.array([[float((e64 * x[c, ky:ky + O, kx:kx + O]).sum()) for kx in range(3)] for ky in range(3)])
        same(gkh[c], want.astype(f32), f"kernel gradient, channel {c}")
    planes = x.sum(axis=0, dtype=np.float64)
    assert float(gkh.sum(dtype=np.float64)) == sum(float((e64 * planes[ky:ky + O, kx:kx + O]).sum()) for ky in range(3) for kx in range(3))
    free(device, y, gx, gk, tx, tk)
