"""The f32 activations that go through exp -- the two of the benchmark chain (sig, tanh) and everything built on them --
swept densely against the oracle's evaluation of the reference's formulas ((float) f((double) x), ScalarSigmoid.java:14-38,
ScalarTanh.java:20-38, CPUFun.java:7-9): every binade from 2^-30 to 2^7 on both signs, the neighbourhood of the series
switch of tanh at |x| = 1/8, and the points where the functions saturate or underflow.

Contract: |got - want| <= 1e-5 * |want| + atol for EVERY element.  atol is 1e-30 (it only admits results in the
subnormal range, where the device flushes to zero), except for the two functions whose reference formula cancels in
double at arguments this sweep reaches: gatu = tanh(x^3) evaluates 2/(1+exp(-2y))-1 at y = x^3 down to 1e-27, and selu
evaluates exp(x)-1 at x down to -1e-9; both return multiples of the double rounding quantum there (0, 1.1e-16,
2.2e-16, ...) where the true value is smaller, so those results are pinned only to within that quantum (4e-16).
The worst relative error seen per function is printed."""
import numpy as np
import pytest

from neureka_amd import Tensor, _lib

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-30
QUANTUM = {"gatu": 4e-16, "selu": 4e-16}       # cancellation quantum of the reference's own double formula, see above
SWEPT = ["sig", "tanh", "silu", "gelu", "softplus", "gatu", "gaus", "selu", "exp"]


def sweep_points() -> np.ndarray:
    rng = np.random.default_rng(2026)
    parts = []
    for e in range(-30, 8):                                   # 38 binades x 2 signs x 140 000 points
        mag = np.float32(2.0) ** e * (1 + rng.random(140_000, dtype=np.float32))
        parts += [mag, -mag]
    dense = lambda lo, hi, n: (lo + (hi - lo) * rng.random(n)).astype(np.float32)
    sw = dense(0.12, 0.13, 1 << 20)                           # the series switch of tanh, both signs
    parts += [sw, -sw, np.float32(0.125) + np.arange(-2048, 2048, dtype=np.float32) * np.float32(2.0 ** -27)]
    for lo, hi in ((8.3, 9.2), (16.0, 18.0), (86.0, 90.0), (100.0, 105.0)):   # tanh -> 1, sig -> 1, exp(-x) underflows, leaves the subnormals
        s = dense(lo, hi, 1 << 19)
        parts += [s, -s]
    specials = np.array([0.0, -0.0, 1e-38, -1e-38, 1e-45, 88.72, -88.72, 87.33, -87.33, -103.97, 128.0, -128.0, 255.9, -255.9], dtype=np.float32)
    return np.concatenate(parts + [specials]).astype(np.float32)


def test_f32_exp_based_activations_dense_sweep(device, orc):
    x = sweep_points()
    n = x.size
    assert n >= 1 << 24, n
    cfg = orc.dense_cfg([n])
    tx = Tensor.of(np.float32, (n,), x).to(device)
    out = Tensor._on_device(device, np.float32, (n,))
    report = []
    # ... and the derivatives whose f32 kernels leave the reference's double routine for a float one (sin', cos') or for
    # the logarithm-and-exp2 power (cbrt')
    for name, d in [(name, d) for name in SWEPT for d in (-1, 0)] + [("sin", 0), ("cos", 0), ("cbrt", 0)]:
        if True:
            print(f"[case] sweep {name} d={d} over {n} points", flush=True)
            device.launch_activation(name, d, out, tx)
            assert _lib.last_path() == "rows_vec_single", _lib.last_path()
            got = out.getData().astype(np.float64)
            with np.errstate(all="ignore"):
                want32 = orc.activation(name, d, np.zeros(n, dtype=np.float32), cfg, x, cfg, workers=16)
            want = want32.astype(np.float64)
            finite = np.isfinite(want)
            assert (np.isnan(got) == np.isnan(want)).all(), f"{name} d={d}: NaNs differ"
            inf = np.isinf(want)
            assert (got[inf] == want[inf]).all(), f"{name} d={d}: infinities differ"
            err = np.abs(got[finite] - want[finite])
            atol = QUANTUM.get(name, ATOL) if d < 0 else ATOL
            bound = RTOL * np.abs(want[finite]) + atol
            bad = err > bound
            with np.errstate(all="ignore"):
                rel = np.where(np.abs(want[finite]) > 1e5 * atol, err / np.abs(want[finite]), 0.0)
            worst = int(np.argmax(rel))
            xs = x[finite]
            report.append((name, d, float(rel[worst]), float(xs[worst])))
            print(f"[sweep] {name:9s} d={d:2d} worst relative error {rel[worst]:.3e} at x = {xs[worst]!r}", flush=True)
            assert not bad.any(), (f"{name} d={d}: {int(bad.sum())} of {n} outside rtol {RTOL}; first at x = {xs[np.flatnonzero(bad)[0]]!r}: "
                                   f"got {got[finite][np.flatnonzero(bad)[0]]!r}, want {want[finite][np.flatnonzero(bad)[0]]!r}")
    device.free(tx); device.free(out)
    print("[sweep] summary: " + "; ".join(f"{n_} d={d} {r:.2e}" for n_, d, r, _ in report), flush=True)


def test_f32_power_dense_sweep(device, orc):
    """a ** b in f32 against the oracle's (float) pow((double) a, (double) b) (CPUBiElementWisePower.java:11-31), every
    element within 1e-5 relative: bases over every binade from 2^-40 to 2^40 with exponents in [-12, 12], bases within
    2^-12 of 1 with exponents up to 3e6 (the logarithm's relative accuracy decides), results that overflow, underflow
    or land in the subnormals, negative bases with whole and fractional exponents, zeros and infinities."""
    rng = np.random.default_rng(2027)
    A, B = [], []
    for e in range(-40, 41):
        A.append((np.float32(2.0) ** e * (1 + rng.random(100_000, dtype=np.float32))).astype(np.float32))
        B.append(rng.uniform(-12, 12, 100_000).astype(np.float32))
    near = (1 + rng.uniform(-2.0 ** -12, 2.0 ** -12, 1 << 21)).astype(np.float32)
    A.append(near); B.append((rng.uniform(-3e6, 3e6, near.size)).astype(np.float32))
    big = rng.uniform(0.5, 2.0, 1 << 20).astype(np.float32)
    A.append(big); B.append(rng.uniform(-260, 260, big.size).astype(np.float32))         # results from 2^-260 to 2^260
    neg = -rng.uniform(0.1, 10, 1 << 18).astype(np.float32)
    A.append(neg); B.append(np.rint(rng.uniform(-9, 9, neg.size)).astype(np.float32))
    A.append(neg); B.append(rng.uniform(-3, 3, neg.size).astype(np.float32))
    sp = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, 3.4e38, 0.5, 2.0, 3.0, -2.0, 1e-38], dtype=np.float32)
    A.append(np.repeat(sp, sp.size)); B.append(np.tile(sp, sp.size))
    a, b = np.concatenate(A), np.concatenate(B)
    n = a.size
    assert n >= 11_000_000
    print(f"[case] sweep power over {n} pairs", flush=True)
    cfg = orc.dense_cfg([n])
    ta, tb = Tensor.of(np.float32, (n,), a).to(device), Tensor.of(np.float32, (n,), b).to(device)
    out = Tensor._on_device(device, np.float32, (n,))
    # the operator, then its derivatives by the base (b * a ** (b - 1)) and by the exponent (a ** b * ln a), which the
    # reference forms in double and rounds once (CPUBiElementWisePower.java:13-31)
    for d in (-1, 0, 1):
        print(f"[case] sweep power d={d}", flush=True)
        device.launch_elementwise("power", d, out, ta, tb)
        assert _lib.last_path() == "rows_vec_pair", _lib.last_path()        # one heavy operator: compiled in, not interpreted
        got = out.getData().astype(np.float64)
        with np.errstate(all="ignore"):
            want = orc.elementwise("power", d, np.zeros(n, dtype=np.float32), cfg, a, cfg, b, cfg, workers=16).astype(np.float64)
        assert (np.isnan(got) == np.isnan(want)).all(), f"d={d}: NaNs differ"
        inf = np.isinf(want)
        assert (got[inf] == want[inf]).all(), f"d={d}: infinities differ"
        finite = np.isfinite(want)
        err = np.abs(got[finite] - want[finite])
        # results below the smallest normal float are rounded to a multiple of 2^-149 by both sides: one such step apart at most
        bound = RTOL * np.abs(want[finite]) + 1.5e-45
        bad = err > bound
        with np.errstate(all="ignore"):
            rel = np.where(np.abs(want[finite]) > 1.2e-38, err / np.abs(want[finite]), 0.0)
        w = int(np.argmax(rel))
        print(f"[sweep] power d={d} worst relative error {rel[w]:.3e} at a = {a[finite][w]!r}, b = {b[finite][w]!r}", flush=True)
        assert not bad.any(), (f"d={d}: {int(bad.sum())} of {n} outside rtol {RTOL}; first at a = {a[finite][np.flatnonzero(bad)[0]]!r}, "
                               f"b = {b[finite][np.flatnonzero(bad)[0]]!r}: got {got[finite][np.flatnonzero(bad)[0]]!r}, want {want[finite][np.flatnonzero(bad)[0]]!r}")
    for t in (ta, tb, out):
        device.free(t)


def test_f64_logarithm_softplus_and_cube_root_derivative_dense_sweep(device, orc):
    """The f64 functions that do not go through the device library's routine -- ln, log10 and softplus on a table-free
    double logarithm, the derivative of cbrt on the squared cube root -- against the oracle's libm evaluation of the reference's
    formulas (ScalarLogarithm.java, ScalarLog10.java, ScalarSoftplus.java, ScalarCbrt.java:28-33), every element within 1e-12 relative (what
    Math.log / Math.pow, specified to 1 ulp and not bit for bit, leave room for): every binade of the doubles, subnormals
    included, the neighbourhood of 1 (where ln passes through zero and only a relatively accurate logarithm survives),
    the seam of the range reduction at sqrt(1/2) and sqrt 2, both signs, zeros, infinities, NaN."""
    rng = np.random.default_rng(2028)
    parts = [np.ldexp(1 + rng.random(1500), e) for e in range(-1074, 1024)]              # 3.1 M points over every binade
    parts += [1 + rng.uniform(-1e-3, 1e-3, 1 << 19), 1 + rng.uniform(-1e-9, 1e-9, 1 << 17), np.nextafter(1.0, 2.0) + np.zeros(1),
              np.sqrt(0.5) * (1 + rng.uniform(-1e-6, 1e-6, 1 << 17)), np.sqrt(2.0) * (1 + rng.uniform(-1e-6, 1e-6, 1 << 17)),
              rng.uniform(0.25, 4.0, 1 << 20)]
    pos = np.concatenate(parts)
    sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 5e-324, 2.2250738585072014e-308, 1.7976931348623157e308, 1.0, -1.0])
    x_ln = np.concatenate([pos, -pos[::64], sp])
    x_soft = np.concatenate([rng.uniform(-750, 750, 1 << 21), rng.uniform(-40, 40, 1 << 21), rng.standard_normal(1 << 20), sp])
    tens = np.array([float(10 ** k) for k in range(23)])                                  # the doubles that are powers of ten
    x_log10 = np.concatenate([x_ln, tens, np.nextafter(tens, np.inf), np.nextafter(tens, 0.0)])
    for name, d, x in (("ln", -1, x_ln), ("log10", -1, x_log10), ("softplus", -1, x_soft), ("cbrt", 0, x_ln)):
        n = x.size
        print(f"[case] f64 sweep {name} d={d} over {n} points", flush=True)
        cfg = orc.dense_cfg([n])
        tx = Tensor.of(np.float64, (n,), x).to(device)
        out = Tensor._on_device(device, np.float64, (n,))
        device.launch_activation(name, d, out, tx)
        assert _lib.last_path() == "rows_vec_single", _lib.last_path()
        got = out.getData()
        with np.errstate(all="ignore"):
            want = orc.activation(name, d, np.zeros(n, dtype=np.float64), cfg, x, cfg, workers=16)
        assert (np.isnan(got) == np.isnan(want)).all(), f"{name} d={d}: NaNs differ"
        inf = np.isinf(want)
        assert (got[inf] == want[inf]).all(), f"{name} d={d}: infinities differ"
        finite = np.isfinite(want)
        err = np.abs(got[finite] - want[finite])
        # softplus: the reference's log(1 + e^x) rounds 1 + e^x to a multiple of 2.2e-16 before the logarithm, so a last-place
        # difference between two exponentials can move the result by that quantum whatever its size
        bad = err > 1e-12 * np.abs(want[finite]) + (2.3e-16 if name == "softplus" else 0.0)
        with np.errstate(all="ignore"):
            rel = np.where(want[finite] != 0, err / np.abs(want[finite]), 0.0)
        w = int(np.argmax(rel))
        print(f"[sweep] f64 {name} d={d} worst relative error {rel[w]:.3e} at x = {x[finite][w]!r}", flush=True)
        assert not bad.any(), (f"{name} d={d}: {int(bad.sum())} of {n} outside rtol 1e-12; first at x = {x[finite][np.flatnonzero(bad)[0]]!r}: "
                               f"got {got[finite][np.flatnonzero(bad)[0]]!r}, want {want[finite][np.flatnonzero(bad)[0]]!r}")
        if name == "log10":                                      # Math.log10: the whole number n for an argument equal to 10^n
            at = x_ln.size
            assert (got[at:at + 23] == np.arange(23.0)).all(), got[at:at + 23]
        device.free(tx); device.free(out)


def test_config3_single_kernels_full_size(device, orc):
    """The four kernels the reference runs for tanh(sig(a)*b+c), each alone on 2^26 elements: sig and tanh within 1e-5
    of the oracle element by element, multiply and add bit for bit."""
    n = 1 << 26
    rng = np.random.default_rng(33)
    a = rng.standard_normal(n).astype(np.float32); b = rng.standard_normal(n).astype(np.float32)
    cfg = orc.dense_cfg([n])
    ta = Tensor.of(np.float32, (n,), a).to(device); tb = Tensor.of(np.float32, (n,), b).to(device)
    out = Tensor._on_device(device, np.float32, (n,))
    for name in ("sig", "tanh"):
        print(f"[case] full-size {name}", flush=True)
        device.launch_activation(name, -1, out, ta)
        got = out.getData().astype(np.float64)
        want = orc.activation(name, -1, np.zeros(n, dtype=np.float32), cfg, a, cfg, workers=16).astype(np.float64)
        err = np.abs(got - want)
        assert (err <= RTOL * np.abs(want) + ATOL).all(), f"{name}: worst relative error {np.max(err / np.abs(want)):.3e}"
        print(f"[sweep] {name} over 2^26 N(0,1) values: worst relative error {np.max(err / np.maximum(np.abs(want), 1e-300)):.3e}", flush=True)
    for op in ("multiply", "add"):
        print(f"[case] full-size {op}", flush=True)
        device.launch_elementwise(op, -1, out, ta, tb)
        want = orc.elementwise(op, -1, np.zeros(n, dtype=np.float32), cfg, a, cfg, b, cfg, workers=16)
        assert out.getData().tobytes() == want.tobytes(), op
    for t in (ta, tb, out):
        device.free(t)


def test_backward_and_heavy_kernels_full_size(device, orc):
    """The launches the backward pass and the heavy functions make, each alone on 2^25 elements (128 MiB: the variants
    with non-temporal loads): the derivatives of tanh, sig, relu and of a division, sin, log10, softplus, cbrt, modulo and
    power -- element by element within 1e-5 of the oracle (relu' and modulo bit for bit) -- and the three derivative
    programs of the fused chain against the product of the oracle's single derivatives."""
    from neureka_amd import Function
    n = 1 << 25
    rng = np.random.default_rng(35)
    a = rng.uniform(0.25, 3.0, n).astype(np.float32) * rng.choice(np.array([-1, 1], dtype=np.float32), n)
    b = rng.uniform(0.5, 2.0, n).astype(np.float32)
    c = rng.standard_normal(n).astype(np.float32)
    cfg = orc.dense_cfg([n])
    ta, tb, tc = (Tensor.of(np.float32, (n,), v).to(device) for v in (a, b, c))
    out = Tensor._on_device(device, np.float32, (n,))
    zeros = lambda: np.zeros(n, dtype=np.float32)

    def close(got, want, what):
        err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        assert (err <= RTOL * np.abs(want.astype(np.float64)) + ATOL).all(), f"{what}: worst relative error {np.max(err / np.maximum(np.abs(want), 1e-300)):.3e}"

    for name, d, src, host in (("tanh", 0, ta, a), ("sig", 0, ta, a), ("relu", 0, ta, a), ("sin", -1, ta, a), ("softplus", -1, ta, a),
                               ("log10", -1, tb, b), ("cbrt", -1, tb, b), ("sin", 0, ta, a)):
        print(f"[case] full-size {name} d={d}", flush=True)
        device.launch_activation(name, d, out, src)
        assert _lib.last_path() == "rows_vec_single", _lib.last_path()      # one function: compiled in, not interpreted
        want = orc.activation(name, d, zeros(), cfg, host, cfg, workers=16)
        if name == "relu":
            assert out.getData().tobytes() == want.tobytes()
        else:
            close(out.getData(), want, f"{name} d={d}")
    for op, d in (("divide", 0), ("divide", 1), ("modulo", -1), ("power", -1)):
        print(f"[case] full-size {op} d={d}", flush=True)
        x = tb if op == "power" else ta
        hx = b if op == "power" else a
        device.launch_elementwise(op, d, out, x, tb)
        assert _lib.last_path() == "rows_vec_pair", _lib.last_path()
        want = orc.elementwise(op, d, zeros(), cfg, hx, cfg, b, cfg, workers=16)
        if op == "modulo":
            assert out.getData().tobytes() == want.tobytes()
        else:
            close(out.getData(), want, f"{op} d={d}")
    print("[case] full-size derivatives of the fused chain", flush=True)
    fused = device.optimizedFunctionOf(Function.of("tanh(sig(I[0])*I[1]+I[2])"), "chain")
    # (1 - t^2 is the difference of quantised floats once tanh saturates: it follows the last bit of its argument, so the
    # argument is built from the forward kernel's own sigmoid, checked against the oracle in the test above)
    device.launch_activation("sig", -1, out, ta)
    s = out.getData()
    p = ((s * b).astype(np.float32) + c).astype(np.float32)
    dt = orc.activation("tanh", 0, zeros(), cfg, p, cfg, workers=16).astype(np.float64)
    ds = orc.activation("sig", 0, zeros(), cfg, a, cfg, workers=16).astype(np.float64)
    wants = (dt * (ds * b), dt * s, dt)
    for i, want in enumerate(wants):
        got = fused.derive([ta, tb, tc], i).getData().astype(np.float64)
        # the program multiplies rounded floats where this reference multiplies doubles: a few roundings on top
        assert (np.abs(got - want) <= 4 * RTOL * np.abs(want) + ATOL).all(), i
    for t in (ta, tb, tc, out):
        device.free(t)
