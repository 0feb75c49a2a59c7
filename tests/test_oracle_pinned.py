"""Pins the CPU oracle (oracle/neureka_cpu_oracle.c) before anything trusts it: against the literal
known answers of the reference's own tests (tests/golden/reference_vectors.json) and against what the
mathematics fixes (numpy / scipy closed forms, brute force).  No GPU."""
import itertools
import math

import numpy as np
import pytest
import scipy.signal

from helpers import assert_bits, assert_close, fill_it, java_array_hash, rounded_sum

F = {"f32": np.float32, "f64": np.float64}


# ---- index maths ---------------------------------------------------------------------------------
def test_index_of_index_rows_of_ndconfiguration_spec(golden, orc):
    """Every row: the C index function equals the definition evaluated in Python integers."""
    for shape, strides, imap, spread, offset, _ in golden["ndconfiguration_spec"]["rows"]:
        cfg = shape + strides + imap + offset + spread
        size = int(np.prod(shape))
        for i in range(size):
            rest, want = i, 0
            for k in range(len(shape)):
                idx, rest = rest // imap[k], rest % imap[k]
                want += (idx * spread[k] + offset[k]) * strides[k]
            assert orc.index_of_index(cfg, i) == want


def test_index_of_index_matches_numpy_strides(orc):
    """Dense, permuted and sliced views against numpy's own strided addressing."""
    base = np.arange(5 * 6 * 7).reshape(5, 6, 7)
    views = {
        "dense": (base, [5, 6, 7], [42, 7, 1], [1, 1, 1], [0, 0, 0]),
        "permuted": (base.transpose(2, 0, 1), [7, 5, 6], [1, 42, 7], [1, 1, 1], [0, 0, 0]),
        "sliced": (base[1:5:2, 2:6, ::3], [2, 4, 3], [42, 7, 1], [2, 1, 3], [1, 2, 0]),
    }
    for name, (view, shape, strides, spread, offset) in views.items():
        imap = orc.dense_cfg(shape)[len(shape):2 * len(shape)].tolist()
        cfg = shape + strides + imap + offset + spread
        want = view.reshape(-1)
        got = [orc.index_of_index(cfg, i) for i in range(want.size)]
        assert got == want.tolist(), name


# ---- seeded generator + activations -------------------------------------------------------------
def test_long_string_hash(orc):
    h = 1125899906842597
    for ch in "Tempeh":
        h = (31 * h + ord(ch)) & 0xFFFFFFFFFFFFFFFF
    h = h - (1 << 64) if h >= (1 << 63) else h
    assert orc.long_string_hash("Tempeh") == h


def _eval_stress_expression(orc, expr, x):
    """'f(i0)*100 % i0' and 'fast_gaus(i0)+i0' of Calculus_Stress_Test.groovy:207-226, operation by operation."""
    dt = x.dtype
    cfg = orc.dense_cfg([x.size])
    name = expr.split("(")[0]
    y = np.zeros_like(x)
    orc.activation(name, -1, y, cfg, x, cfg)
    if expr.endswith("+i0"):
        out = np.zeros_like(x)
        return orc.elementwise("add", -1, out, cfg, y, cfg, x, cfg)
    z = np.zeros_like(x)
    orc.scalarization("multiply", -1, z, cfg, y, cfg, 100.0)
    out = np.zeros_like(x)
    return orc.elementwise("modulo", -1, out, cfg, z, cfg, x, cfg)


def test_seeded_activation_sums(golden, orc):
    """Generator + activation + scalar multiply + modulo against the enforced sums of the reference."""
    g = golden["activation_sums"]
    for row in g["rows"]:
        x = orc.seeded(F[row["type"]], g["size"], g["seed"])
        out = _eval_stress_expression(orc, row["expression"], x)
        assert str(rounded_sum(out)) == row["sum"], row


def test_seeded_activation_vectors(golden, orc):
    g = golden["activation_vectors"]
    for row in g["rows"]:
        dt = F[row["type"]]
        x = orc.seeded(dt, g["size"], g["seed"])
        cfg = orc.dense_cfg([x.size])
        out = np.zeros_like(x)
        orc.activation(row["fun"], 0 if row["derive"] else -1, out, cfg, x, cfg)
        want = np.array(row["expected"], dtype=dt)
        # Math.exp is not bit-specified: 1 ulp of slack, as the reference's own platform would have
        np.testing.assert_array_max_ulp(out, want, maxulp=2 if row["type"] == "f64" else 1)


def test_activations_against_closed_forms(orc):
    """All 23 functions and derivatives against independent float64 closed forms (numpy)."""
    x = np.linspace(-4.0, 4.0, 161)
    x = x[np.abs(x) > 1e-3]
    sig = lambda v: 1 / (1 + np.exp(-v))
    A, S = 1.6732632423543772848170429916717, 1.0507009873554804934193349852946
    forms = {
        "abs": (np.abs, np.sign), "cos": (np.cos, lambda v: -np.sin(v)), "sin": (np.sin, np.cos),
        "gasu": (lambda v: v**3 / (1 + np.abs(v**3)), lambda v: 3 * v * v / (1 + np.abs(v**3)) ** 2),
        "gatu": (lambda v: np.tanh(v**3), lambda v: 3 * v * v / np.cosh(v**3) ** 2),
        "gaus": (lambda v: np.exp(-v * v), lambda v: -2 * v * np.exp(-v * v)),
        "fast_gaus": (lambda v: 1 / (1 + v * v), lambda v: -2 * v / (1 + v * v) ** 2),
        "gelu": (lambda v: v * sig(1.702 * v), lambda v: sig(1.702 * v) + 1.702 * v * sig(1.702 * v) * (1 - sig(1.702 * v))),
        "idy": (lambda v: v, lambda v: np.ones_like(v)), "quad": (lambda v: v * v, lambda v: 2 * v),
        "relu": (lambda v: np.where(v >= 0, v, 0.01 * v), lambda v: np.where(v >= 0, 1.0, 0.01)),
        "selu": (lambda v: np.where(v > 0, S * v, S * A * np.expm1(v)), lambda v: np.where(v > 0, S, S * A * np.exp(v))),
        "sig": (sig, lambda v: sig(v) * (1 - sig(v))), "silu": (lambda v: v * sig(v), lambda v: sig(v) + v * sig(v) * (1 - sig(v))),
        "softplus": (lambda v: np.log1p(np.exp(v)), sig),
        "softsign": (lambda v: v / (1 + np.abs(v)), lambda v: 1 / (1 + np.abs(v)) ** 2),
        "tanh": (np.tanh, lambda v: 1 / np.cosh(v) ** 2),
        "fast_tanh": (lambda v: v / np.sqrt(1 + v * v), lambda v: (1 + v * v) ** -1.5),
        "exp": (np.exp, np.exp),
    }
    pos = {"ln": (np.log, lambda v: 1 / v), "log10": (np.log10, lambda v: 1 / (v * math.log(10))),
           "sqrt": (np.sqrt, lambda v: 0.5 / np.sqrt(v)), "cbrt": (np.cbrt, lambda v: 1 / (3 * np.cbrt(v) ** 2))}
    for name, (f, df) in {**forms, **pos}.items():
        xs = x[x > 0] if name in pos else x
        for dt, tol in ((np.float64, 1e-9), (np.float32, 3e-5)):
            xi = xs.astype(dt)
            # fast_tanh / sqrt' use the 2- or 4-step bit-trick inverse root: accurate to ~5e-6 (f32) / 1e-10
            slack = 2e-5 if name in ("fast_tanh", "sqrt") and dt == np.float32 else tol
            np.testing.assert_allclose(orc.fun(name, xi), f(xi.astype(np.float64)), rtol=slack, atol=slack, err_msg=name)
            np.testing.assert_allclose(orc.fun(name, xi, derive=True), df(xi.astype(np.float64)), rtol=slack, atol=slack, err_msg=name + "'")


# ---- broadcast -----------------------------------------------------------------------------------
def _cycle(values, n, dt):
    return np.resize(np.array(values, dtype=dt), n)


def _fmt(v):
    if np.isnan(v): return "NaN"
    if np.isinf(v): return "-inf" if v < 0 else "inf"
    r = round(float(v), 5)
    return repr(r) if r != 0 else ("-0.0" if np.signbit(v) else "0.0")


def test_broadcast_forward_golden(golden, orc):
    g = golden["broadcast_stress"]
    for row in g["rows"]:
        for dt in (np.float64, np.float32):
            s1, s2, so = row["shape1"], row["shape2"], row["shape"]
            if len(s1) != len(s2):     # Permute.makeFit pads [2,1] vs [2,2]: same rank here
                continue
            a, b = _cycle(g["t1_range"], int(np.prod(s1)), dt), _cycle(g["t2_range"], int(np.prod(s2)), dt)
            out = np.zeros(int(np.prod(so)), dtype=dt)
            orc.broadcast(row["op"], -1, out, orc.dense_cfg(so), a, orc.dense_cfg(s1), b, orc.dense_cfg(s2))
            assert [_fmt(v) for v in out] == row["expected"], row


def test_broadcast_forward_is_numpy_broadcasting(orc):
    rng = np.random.default_rng(7)
    ops = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply, "divide": np.divide}
    for s1, s2 in [([3, 1, 5], [1, 4, 5]), ([1, 4, 1], [3, 4, 5]), ([2, 3], [2, 3]), ([6, 1], [1, 7])]:
        so = [max(p, q) for p, q in zip(s1, s2)]
        for dt in (np.float32, np.float64):
            a = rng.uniform(-1, 1, s1).astype(dt)
            b = rng.uniform(-1, 1, s2).astype(dt)
            for name, f in ops.items():
                out = np.zeros(int(np.prod(so)), dtype=dt)
                orc.broadcast(name, -1, out, orc.dense_cfg(so), a.reshape(-1), orc.dense_cfg(s1), b.reshape(-1), orc.dense_cfg(s2))
                assert_bits(out.reshape(so), f(a, b).astype(dt), f"{name} {s1} {s2}")


def test_broadcast_backward_golden_and_sums(golden, orc):
    """Tensor_Operation_Spec rows: gradient of a+b / a-b / b-a w.r.t. the broadcast operand, produced by
    the reducing kernel on (zeros like target, zeros like other, error)."""
    g = golden["broadcast_autograd"]
    err = np.array(g["error"], dtype=np.float64)
    for row in g["rows"]:
        if row["which_grad"] != "b" or row["op"] == "a*b":
            continue
        bs = row["b_shape"]
        bs = [1] * (2 - len(bs)) + bs           # makeFit pads in front for a [2,2] partner
        op = "add" if row["op"] == "a+b" else "subtract"
        d = 0 if row["op"] == "b-a" else 1      # position of b in the operation
        drn = np.zeros(int(np.prod(bs)))
        other = np.zeros(4)
        orc.broadcast(op, d, drn, orc.dense_cfg(bs), other, orc.dense_cfg([2, 2]), err, orc.dense_cfg([2, 2]))
        assert drn.tolist() == [float(v) for v in row["gradient"]], row
    # against numpy: the reduction is a sum over the broadcast axes
    rng = np.random.default_rng(3)
    e = rng.standard_normal((4, 5, 6))
    for shape, axes in [([4, 1, 6], (1,)), ([1, 5, 1], (0, 2)), ([1, 1, 1], (0, 1, 2)), ([4, 5, 6], ())]:
        drn = np.zeros(int(np.prod(shape)))
        orc.broadcast("add", 0, drn, orc.dense_cfg(shape), np.zeros(120), orc.dense_cfg([4, 5, 6]), e.reshape(-1), orc.dense_cfg([4, 5, 6]))
        np.testing.assert_allclose(drn.reshape(shape), e.sum(axis=axes, keepdims=True) if axes else e, rtol=1e-13)


# ---- convolution ------------------------------------------------------------------------------------
def _conv(orc, x, xs, k, ks, dt):
    ys = [abs(a - b) + 1 for a, b in zip(xs, ks)]
    out = np.zeros(int(np.prod(ys)), dtype=dt)
    orc.convolve(out, orc.dense_cfg(ys), np.array(x, dtype=dt), orc.dense_cfg(xs), np.array(k, dtype=dt), orc.dense_cfg(ks))
    return out, ys


def test_convolution_forward_golden(golden, orc):
    for row in golden["convolution_forward"]["rows"]:
        for dt in (np.float32, np.float64):
            out, ys = _conv(orc, row["x"], row["x_shape"], row["k"], row["k_shape"], dt)
            assert ys == row["y_shape"] and out.tolist() == [float(v) for v in row["y"]], row


def test_convolution_forward_is_valid_cross_correlation(orc):
    """The state machine against scipy's 'valid' correlation (2-D, 3-D with a full-axis reduction) and
    the 2-D fast path of SimpleCPUConvolution against the general path."""
    rng = np.random.default_rng(11)
    x = rng.uniform(-1, 1, (9, 8))
    k = rng.uniform(-1, 1, (3, 2))
    out, ys = _conv(orc, x.reshape(-1), [9, 8], k.reshape(-1), [3, 2], np.float64)
    np.testing.assert_allclose(out.reshape(ys), scipy.signal.correlate(x, k, mode="valid"), rtol=1e-13)
    simple = orc.simple_conv2d(x.reshape(-1).copy(), k.reshape(-1).copy(), 8, 9, 2, 3)
    np.testing.assert_allclose(simple, out, rtol=1e-13)
    # operands swapped: the smaller one may come first
    out2, _ = _conv(orc, k.reshape(-1), [3, 2], x.reshape(-1), [9, 8], np.float64)
    np.testing.assert_allclose(out2, out, rtol=1e-13)
    x3 = rng.uniform(-1, 1, (4, 7, 6))
    k3 = rng.uniform(-1, 1, (4, 3, 3))
    out3, ys3 = _conv(orc, x3.reshape(-1), [4, 7, 6], k3.reshape(-1), [4, 3, 3], np.float64)
    assert ys3 == [1, 5, 4]
    np.testing.assert_allclose(out3.reshape(ys3), scipy.signal.correlate(x3, k3, mode="valid"), rtol=1e-12)


def test_convolution_summation_order_is_axis0_fastest(orc):
    """f32 sums are order-sensitive: reproduce the reference order (axis 0 fastest, products rounded
    before the add) in numpy scalars and require bit equality."""
    rng = np.random.default_rng(5)
    xs, ks = [3, 6, 5], [3, 2, 3]
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    k = rng.uniform(-1, 1, ks).astype(np.float32)
    out, ys = _conv(orc, x.reshape(-1), xs, k.reshape(-1), ks, np.float32)
    want = np.zeros(ys, dtype=np.float32)
    for oy in range(ys[1]):
        for ox in range(ys[2]):
            acc = np.float32(0)
            for kx in range(ks[2]):            # slowest
                for ky in range(ks[1]):
                    for c in range(ks[0]):     # fastest
                        acc = np.float32(acc + np.float32(x[c, oy + ky, ox + kx] * k[c, ky, kx]))
            want[0, oy, ox] = acc
    assert_bits(out.reshape(ys), want, "order")


def test_convolution_backward_golden_graph(golden, orc):
    """The whole graph of Tensor_Convolution_Spec.groovy:303-366 evaluated with the oracle's kernels."""
    g = golden["convolution_autograd"]
    f8 = np.float64
    conv = lambda a, ash, b, bsh: _conv(orc, a, ash, b, bsh, f8)
    def deconv(target_shape, other, other_shape, err, err_shape):
        drn = np.zeros(int(np.prod(target_shape)))
        orc.deconvolve(drn, orc.dense_cfg(target_shape), np.array(other, dtype=f8), orc.dense_cfg(other_shape), np.array(err, dtype=f8), orc.dense_cfg(err_shape))
        return drn
    i_a, w_a, w_b, w_c = (np.array(g[n]["data"], dtype=f8) for n in ("i_a", "w_a", "w_b", "w_c"))
    o_a, sa = conv(i_a, [2, 1], w_a, [2, 2]); assert o_a.tolist() == g["o_a"] and sa == [1, 2]
    o_b, sb = conv(o_a, sa, w_b, [2, 2]); assert o_b.tolist() == g["o_b"] and sb == [2, 1]
    o_c, sc = conv(o_a, sa, w_c, [2, 2]); assert o_c.tolist() == g["o_c"]
    out = o_b * o_c
    assert out.tolist() == g["out"]
    e = np.ones(2)
    e_b, e_c = e * o_c, e * o_b                                   # d(out)/d(o_b), d(out)/d(o_c)
    g_wb = deconv([2, 2], o_a, sa, e_b, sb)                       # d = 1: derivative = the other operand o_a
    assert g_wb.tolist() == g["w_b_gradient"]
    e_a = deconv(sa, w_b, [2, 2], e_b, sb) + deconv(sa, w_c, [2, 2], e_c, sc)
    g_wa = deconv([2, 2], i_a, [2, 1], e_a, sa)
    assert (w_a + g_wa).tolist() == g["w_a_after_apply"]          # gradients are added on apply


def test_deconvolve_fast_equals_literal_and_autodiff(orc):
    """The range-restricted gradient is bit-identical to the literal loop, and both equal the
    derivative of the forward definition (checked by finite linearity: <dy, conv(x,k)> pairing)."""
    rng = np.random.default_rng(2)
    for xs, ks in [([3, 7, 6], [3, 3, 2]), ([5, 5], [2, 3]), ([2, 4, 4], [1, 2, 2])]:
        ys = [abs(a - b) + 1 for a, b in zip(xs, ks)]
        for dt in (np.float32, np.float64):
            x = rng.uniform(-1, 1, xs).astype(dt).reshape(-1)
            k = rng.uniform(-1, 1, ks).astype(dt).reshape(-1)
            e = rng.uniform(-1, 1, ys).astype(dt).reshape(-1)
            for tgt_shape, other, other_shape in ((xs, k, ks), (ks, x, xs)):
                lit = np.zeros(int(np.prod(tgt_shape)), dtype=dt)
                fast = np.zeros_like(lit)
                orc.deconvolve(lit, orc.dense_cfg(tgt_shape), other, orc.dense_cfg(other_shape), e, orc.dense_cfg(ys))
                orc.deconvolve(fast, orc.dense_cfg(tgt_shape), other, orc.dense_cfg(other_shape), e, orc.dense_cfg(ys), fast=True)
                assert_bits(fast, lit, f"{xs} {ks}")
        # adjoint identity in float64: <e, conv(x, k)> == <dx, x> == <dk, k>
        x = rng.uniform(-1, 1, xs).reshape(-1); k = rng.uniform(-1, 1, ks).reshape(-1); e = rng.uniform(-1, 1, ys).reshape(-1)
        y, _ = _conv(orc, x, xs, k, ks, np.float64)
        dx = np.zeros(x.size); dk = np.zeros(k.size)
        orc.deconvolve(dx, orc.dense_cfg(xs), k, orc.dense_cfg(ks), e, orc.dense_cfg(ys))
        orc.deconvolve(dk, orc.dense_cfg(ks), x, orc.dense_cfg(xs), e, orc.dense_cfg(ys))
        np.testing.assert_allclose(np.dot(dx, x), np.dot(e, y), rtol=1e-12)
        np.testing.assert_allclose(np.dot(dk, k), np.dot(e, y), rtol=1e-12)


# ---- matmul -----------------------------------------------------------------------------------------
def test_matmul_hash_known_answers(golden, orc):
    g = golden["matmul_hashes"]
    for rows, row_major in ((g["row_major"], True), (g["column_major"], False)):
        for M, K, N, want in rows:
            for dt in (np.float32, np.float64):
                A, B = fill_it(M * K, 43, dt), fill_it(K * N, 87, dt)
                Cm = orc.gemm(row_major, A, B, M, K, N)
                assert java_array_hash(Cm) == want, (M, K, N, row_major, dt)


def test_matmul_is_numpy_matmul(orc):
    rng = np.random.default_rng(9)
    M, K, N = 17, 23, 13
    A = rng.integers(-5, 6, (M, K)).astype(np.float32)
    B = rng.integers(-5, 6, (K, N)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64)
    rm = orc.gemm(True, A.reshape(-1).copy(), B.reshape(-1).copy(), M, K, N, workers=4)
    assert (rm.reshape(M, N) == want).all()
    cm = orc.gemm(False, A.T.reshape(-1).copy(), B.T.reshape(-1).copy(), M, K, N, workers=4)     # column-major storage
    assert (cm.reshape(N, M).T == want).all()
    # accumulates into C
    C0 = np.full(M * N, 2.0, dtype=np.float32)
    acc = orc.gemm(True, A.reshape(-1).copy(), B.reshape(-1).copy(), M, K, N, C_init=C0)
    assert (acc.reshape(M, N) == want + 2).all()


# ---- executor split ---------------------------------------------------------------------------------
def test_work_split_covers_range_with_power_of_two_leaves(orc):
    for n, workers in [(1000, 8), (1 << 20, 6), (33, 16), (32, 16), (5, 4), (1 << 16, 1)]:
        leaves = orc.split_leaves(0, n, workers)
        assert leaves[0][0] == 0 and leaves[-1][1] == n
        assert all(leaves[i][1] == leaves[i + 1][0] for i in range(len(leaves) - 1))
        if n > 32 * workers:
            assert len(leaves) == 2 ** int(math.log2(workers))


def test_threaded_equals_sequential(orc):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(10007).astype(np.float32)
    cfg = orc.dense_cfg([x.size])
    a = orc.activation("tanh", -1, np.zeros_like(x), cfg, x, cfg, workers=1)
    b = orc.activation("tanh", -1, np.zeros_like(x), cfg, x, cfg, workers=8)
    assert_bits(a, b)


# ---- whole-tensor reductions: CPUSum, CPUReduce, DOT ------------------------------------------------------
def _java_string_hash(s: str) -> int:
    h = 0
    for ch in s:
        h = (31 * h + ord(ch)) & 0xFFFFFFFF
    return h - (1 << 32) if h >= (1 << 31) else h


def stats_function_input(reduce_type: str, type_name: str, dtype) -> np.ndarray:
    """The tensor of Tensor_Stats_Spec.groovy:33-37: Groovy evaluates 31**(i+13) exactly (BigInteger)."""
    seed = _java_string_hash(type_name) + _java_string_hash(reduce_type)
    return np.array([((seed + 31 ** (i + 13)) % 301) - 151 for i in range(19 * 7)], dtype=dtype)


def test_reduce_index_reproduces_the_stats_spec(golden, orc):
    g = golden["stats"]
    for reduce_type, type_name, expected in g["min_max_function"]["rows"]:
        a = stats_function_input(reduce_type, type_name, np.float32 if type_name == "Float" else np.float64)
        i = orc.reduce_index(reduce_type.lower(), a)
        assert a[i] == expected
        assert i == (np.argmin(a) if reduce_type == "MIN" else np.argmax(a))          # first occurrence
    a = np.array([((31 ** (i + 42)) % 301) - 151 for i in range(133)], dtype=np.float32)
    assert a[orc.reduce_index("min", a)] == g["min_max_methods"]["min"] and a[orc.reduce_index("max", a)] == g["min_max_methods"]["max"]


def test_reduce_index_ties_and_tile_structure(orc):
    """Strict comparison keeps the first of equal values, within a tile of 64 and across the recursion; a NaN
    is only ever selected when it opens a tile (CPUReduce.java:117-127)."""
    rng = np.random.default_rng(5)
    for n in (1, 2, 63, 64, 65, 4095, 4096, 4097, 70001):
        a = rng.integers(-50, 50, n).astype(np.float32)        # many ties
        assert orc.reduce_index("min", a) == int(np.argmin(a)) and orc.reduce_index("max", a) == int(np.argmax(a))
    a = np.arange(200, dtype=np.float64)
    a[70] = np.nan                                             # inside a tile: never beats, never beaten -> ignored
    assert orc.reduce_index("max", a) == 199 and orc.reduce_index("min", a) == 0
    a = np.arange(200, dtype=np.float64)
    a[64] = np.nan                                             # opens the second tile: that tile's value is NaN ...
    assert orc.reduce_index("max", a) == 199                   # ... and loses to nothing, wins nothing, in the next level (it is not first there)
    a[0] = np.nan                                              # opens the first tile of every level: sticks
    assert orc.reduce_index("max", a) == 0 and orc.reduce_index("min", a) == 0


def test_sum_tree_reproduces_the_stats_spec_and_its_own_definition(golden, orc):
    g = golden["stats"]["sum"]
    a = np.array([((7 ** i) % 11) - 5 for i in range(13 * 73 * 11)], dtype=np.float32)
    assert orc.sum_tree(a) == g["expected"]
    # the definition, restated with numpy: tiles of 128 front to back, recursively
    def tree(x):
        while x.size > 1:
            pad = (-x.size) % 128
            tiles = np.concatenate([x, np.zeros(pad, dtype=x.dtype)]).reshape(-1, 128)
            acc = np.zeros(tiles.shape[0], dtype=x.dtype)
            for j in range(128):
                acc = acc + tiles[:, j]
            x = acc
        return x[0]
    rng = np.random.default_rng(6)
    for dt in (np.float32, np.float64):
        for n in (2, 127, 128, 129, 16384, 16385, 100003):
            x = rng.standard_normal(n).astype(dt)
            got = orc.sum_tree(x)
            assert got == tree(x), (dt, n)
            assert abs(float(got) - math.fsum(x.tolist())) <= (1e-5 if dt == np.float32 else 1e-12) * float(np.abs(x).sum())


def test_dot_reproduces_the_dot_product_spec(golden, orc):
    for row in golden["stats"]["dot"]:
        a, b = np.array(row["a"], dtype=np.float32), np.array(row["b"], dtype=np.float32)
        assert orc.dot(a, b) == row["expected"]
    rng = np.random.default_rng(7)
    for n in (1, 3, 4, 5, 1001):
        a, b = rng.integers(-9, 10, n).astype(np.float64), rng.integers(-9, 10, n).astype(np.float64)
        assert orc.dot(a, b) == float(np.dot(a, b))           # exact on small integers, any order
    a, b = rng.standard_normal(1001).astype(np.float32), rng.standard_normal(1001).astype(np.float32)
    s = [np.float32(0)] * 4                                    # four running sums, remainder into the first
    for i in range(1000):
        s[i % 4] = s[i % 4] + a[i] * b[i]
    s[0] = s[0] + a[1000] * b[1000]
    assert orc.dot(a, b) == ((s[0] + s[1]) + s[2]) + s[3]


# ---- integer scalarization (CPUScalarBroadcast on Integer / Long / Short / Byte) ---------------------------------
def _iscal(orc, op, d, data, value, dtype):
    src = np.asarray(data, dtype=dtype)
    cfg = orc.dense_cfg([src.size])
    return orc.scalarization_int(op, d, np.zeros_like(src), cfg, src, cfg, value)


def test_int_scalarization_is_consistent_with_the_recorded_integer_rows_of_the_operation_spec(golden, orc):
    """Tensor_Operation_Spec.groovy:560-636, Integer rows.  The reference does not enforce them (its assertion parses as
    `(a == (expected instanceof Map)) ? .. : expected`, always truthy) and they were recorded with a former generator,
    so they are no known-answer test; they are outputs the reference once produced, and four of them hang together
    only under Java's int arithmetic: relu(i0) and relu(i0)-i0 give the tensor, and 'abs(i0*10)%3', 'relu(-i0-5)+i0*3'
    and 'relu(-i0)+i0' must then follow (wrapping multiply, int remainder, relu as (int) Math.round(relu((double) x))).
    The enforced rows are the Integer / Long ones of 'Scalar broadcasting works across devices' (:484-513)."""
    g = golden["int_scalarization"]
    i0 = np.array(g["tempeh_i0_recovered"], dtype=np.int32)

    def relu(x):
        return np.where(x >= 0, x, np.floor(x.astype(np.float64) * .01 + 0.5).astype(np.int64)).astype(np.int32)
    assert relu(i0).tolist() == g["tempeh_relu_i0"]
    times10 = _iscal(orc, "multiply", -1, i0, 10, np.int32)                      # wraps
    assert _iscal(orc, "modulo", -1, np.abs(times10), 3, np.int32).tolist() == g["tempeh_abs_i0_times_10_mod_3"]
    neg = (-i0.astype(np.int64)).astype(np.int32)
    with np.errstate(over="ignore"):
        got = relu(_iscal(orc, "subtract", -1, neg, 5, np.int32)) + _iscal(orc, "multiply", -1, i0, 3, np.int32)
        assert got.tolist() == g["tempeh_relu_neg_i0_minus_5_plus_i0_times_3"]
        assert (relu(neg) + i0).tolist() == g["tempeh_relu_neg_i0_plus_i0"]
    s = g["scalar_broadcast_add"]
    for dt in (np.int32, np.int64):
        assert _iscal(orc, "add", -1, s["a"], s["b"], dt).tolist() == s["c"]


def test_int_scalarization_follows_the_java_language_rules(orc):
    """Known answers worked out by hand from the Java Language Specification (15.17 integer division and remainder,
    5.1.3 narrowing) and the contract of Math.round (ties towards positive infinity, NaN -> 0, saturation)."""
    i32, i64, i16, i8 = np.int32, np.int64, np.int16, np.int8
    IMIN, IMAX, LMIN, LMAX = -2**31, 2**31 - 1, -2**63, 2**63 - 1
    rows = [
        # int: integer overloads
        (i32, "add", -1, [IMAX, 5], 1, [IMIN, 6]), (i32, "subtract", -1, [IMIN], 1, [IMAX]), (i32, "multiply", -1, [IMAX, -3], 2, [-2, -6]),
        (i32, "divide", -1, [7, -7, IMIN], 2, [3, -3, -2**30]), (i32, "divide", -1, [IMIN, 5], -1, [IMIN, -5]),
        (i32, "modulo", -1, [-7, 7, 6], 3, [-1, 1, 0]), (i32, "modulo", -1, [7, -7], -3, [1, -1]), (i32, "modulo", -1, [IMIN], -1, [0]),
        (i32, "power", -1, [10], 10, [1410065408]), (i32, "power", -1, [-2, 0, 3], 3, [-8, 0, 27]), (i32, "power", -1, [2, -2, 4], -1, [1, 0, 0]),
        (i32, "power", -1, [0, 7], 0, [1, 1]), (i32, "idy", -1, [4, 5], 9, [9, 9]),
        (i32, "add", 0, [3], 4, [1]), (i32, "add", 1, [3], 4, [1]), (i32, "subtract", 0, [3], 4, [1]), (i32, "subtract", 1, [3], 4, [-1]),
        (i32, "multiply", 0, [3], 4, [4]), (i32, "multiply", 1, [3], 4, [3]),
        (i32, "divide", 0, [9], 2, [1]), (i32, "divide", 0, [9], -2, [0]), (i32, "divide", 0, [9], 3, [0]), (i32, "divide", 0, [9], 0, [-1]),
        (i32, "divide", 1, [7, -7, 5, 6], 2, [-2, 2, -1, -1]), (i32, "modulo", 0, [9], 1, [1]), (i32, "modulo", 1, [8], 2, [-2]),
        (i32, "power", 0, [3], 2, [6]), (i32, "power", 0, [2], 0, [0]), (i32, "power", 1, [2], 3, [6]), (i32, "power", 1, [-2, 0], 2, [0, 0]),
        (i32, "power", 1, [0], 0, [0]),
        # long
        (i64, "add", -1, [LMAX], 1, [LMIN]), (i64, "multiply", -1, [2**62], 2, [LMIN]), (i64, "divide", -1, [LMIN, -9], -1, [LMIN, 9]),
        (i64, "divide", -1, [-9, 9], 2, [-4, 4]), (i64, "modulo", -1, [-9, LMIN], -1, [0, 0]), (i64, "power", -1, [3], 40, [LMAX]),
        (i64, "power", -1, [2, 10], 18, [2**18, 10**18]), (i64, "power", -1, [2], 62, [2**62]), (i64, "divide", 0, [1], 0, [LMAX]),
        (i64, "divide", 1, [7], 2, [-2]), (i64, "power", 1, [0], 0, [LMIN]),
        # short: no overloads, everything through double and (short) Math.round
        (i16, "divide", -1, [7, -7, 1, -1, 0], 2, [4, -3, 1, 0, 0]), (i16, "divide", -1, [7, -7, 0], 0, [-1, 0, 0]),
        (i16, "modulo", -1, [-7, 7], 3, [-1, 1]), (i16, "modulo", -1, [7], 0, [0]), (i16, "multiply", -1, [300], 300, [24464]),
        (i16, "add", -1, [32767], 1, [-32768]), (i16, "power", -1, [2], 15, [-32768]), (i16, "power", -1, [2], 16, [0]),
        (i16, "divide", 0, [5], 2, [1]), (i16, "divide", 1, [6], 2, [-1]), (i16, "idy", -1, [1], 70000, [4464]),
        # byte
        (i8, "add", -1, [100], 100, [-56]), (i8, "multiply", -1, [90], 2, [-76]), (i8, "divide", -1, [7], 2, [4]), (i8, "subtract", -1, [-128], 1, [127]),
        (i8, "idy", -1, [0], 300, [44]), (i8, "power", 1, [2], 3, [6]),
    ]
    for dt, op, d, data, value, want in rows:
        assert _iscal(orc, op, d, data, value, dt).tolist() == want, (dt.__name__, op, d, data, value)
    for dt in (i32, i64):
        for op in ("divide", "modulo"):
            with pytest.raises(orc.JavaArithmeticException):
                _iscal(orc, op, -1, [1, 2], 0, dt)


def test_int_scalarization_matches_exact_integer_arithmetic_and_views(orc):
    """Random data against Python's exact integers (wrapped), through a strided source view into a permuted drain."""
    rng = np.random.default_rng(77)
    for dt, bits in ((np.int32, 32), (np.int64, 64)):
        lo, hi = -2**(bits - 1), 2**(bits - 1) - 1
        data = rng.integers(lo, hi, 500, dtype=dt, endpoint=True)
        wrap = lambda v: (v - lo) % 2**bits + lo
        for value in (3, -7, hi, lo + 1):
            for op, f in (("add", lambda a, b: a + b), ("subtract", lambda a, b: a - b), ("multiply", lambda a, b: a * b),
                          ("divide", lambda a, b: abs(a) // abs(b) * (1 if (a < 0) == (b < 0) else -1)),
                          ("modulo", lambda a, b: (abs(a) % abs(b)) * (-1 if a < 0 else 1))):
                want = [wrap(f(int(a), value)) for a in data]
                assert _iscal(orc, op, -1, data, value, dt).tolist() == want, (dt.__name__, op, value)
    base = np.arange(4 * 6, dtype=np.int16)
    src_cfg = [3, 3, 6, 1, 3, 1, 0, 1, 1, 2]                     # shape | strides | indicesMap | offset | spread: rows 0..2, columns 1, 3, 5
    drn_cfg = [3, 3, 1, 3, 3, 1, 0, 0, 1, 1]                     # column-major strides
    out = orc.scalarization_int("multiply", -1, np.zeros(9, dtype=np.int16), drn_cfg, base, src_cfg, 5)
    assert out.reshape(3, 3).T.tolist() == (base.reshape(4, 6)[0:3, 1::2] * 5).tolist()


def test_power_follows_the_special_cases_of_java_math_pow(orc):
    """The operator ** is Math.pow (CPUBiElementWisePower.java:11): its documented special cases, including the two
    where C's pow answers differently (a NaN exponent with base 1; a base of magnitude 1 with an infinite exponent)."""
    inf, nan = np.inf, np.nan
    rows = [  # (base, exponent, Math.pow)
        (3.0, 0.0, 1.0), (nan, 0.0, 1.0), (inf, -0.0, 1.0), (-2.5, 1.0, -2.5), (nan, 1.0, nan),
        (1.0, nan, nan), (0.0, nan, nan), (inf, nan, nan), (nan, 2.5, nan), (nan, -1.0, nan),
        (2.0, inf, inf), (-2.0, inf, inf), (0.5, -inf, inf), (-0.5, -inf, inf),
        (2.0, -inf, 0.0), (-2.0, -inf, 0.0), (0.5, inf, 0.0), (-0.5, inf, 0.0),
        (1.0, inf, nan), (-1.0, inf, nan), (1.0, -inf, nan), (-1.0, -inf, nan),
        (0.0, 2.5, 0.0), (inf, -3.0, 0.0), (0.0, -2.5, inf), (inf, 3.0, inf),
        (-0.0, 2.0, 0.0), (-0.0, 2.5, 0.0), (-inf, -2.0, 0.0), (-inf, -2.5, 0.0),
        (-0.0, 3.0, -0.0), (-inf, -3.0, -0.0),
        (-0.0, -2.0, inf), (-0.0, -2.5, inf), (-inf, 2.0, inf), (-inf, 2.5, inf),
        (-0.0, -3.0, -inf), (-inf, 3.0, -inf),
        (-2.0, 2.0, 4.0), (-2.0, 3.0, -8.0), (-2.0, -2.0, 0.25), (-2.0, 0.5, nan), (-8.0, 1.0 / 3.0, nan),
        (2.0, 10.0, 1024.0), (4.0, 0.5, 2.0), (10.0, -2.0, 0.01), (2.0, 0.5, np.sqrt(2.0)),
    ]
    a = np.array([r[0] for r in rows]); b = np.array([r[1] for r in rows]); want = np.array([r[2] for r in rows])
    c = orc.dense_cfg([a.size])
    for T in (np.float64, np.float32):
        with np.errstate(all="ignore"):
            got = orc.elementwise("power", -1, np.zeros(a.size, dtype=T), c, a.astype(T), c, b.astype(T), c)
            expect = want.astype(T)
            if T is np.float32:      # the float form is (float) Math.pow((double) a, (double) b) on the rounded arguments
                expect[rows.index((-8.0, 1.0 / 3.0, nan))] = nan
        for i, r in enumerate(rows):
            g, w = got[i], expect[i]
            ok = (np.isnan(g) and np.isnan(w)) or (g == w and np.signbit(g) == np.signbit(w)) or \
                 (np.isfinite(w) and w != 0 and abs(g - w) <= 4 * np.finfo(T).eps * abs(w))
            assert ok, (T.__name__, r, float(g))
