"""Known answers of the reference's own (enforced) test scripts, re-expressed twice: against the CPU oracle
(`-m "not gpu"`: they pin the oracle) and through the device mirror on the GPU (`-m gpu`: the HIP path gives what
the reference's tests expect).  Inputs and expected outputs live in tests/golden/reference_scripts.json."""
import json
import os

import numpy as np
import pytest

from neureka_amd import Tensor, NDConfiguration

F = {"f32": np.float32, "f64": np.float64}
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def scripts():
    with open(os.path.join(ROOT, "tests", "golden", "reference_scripts.json")) as f:
        return json.load(f)


def say(*a):
    print("[case]", *a, flush=True)


def five_decimals(x):
    """How the reference's tensor printer shows these numbers: a value whose text starts with "0." is cut to seven
    characters (view/NdaAsString.java:520-531), the others appear rounded to five decimals."""
    return [repr(float(v))[:7] if repr(float(v)).startswith("0.") else "%.5f" % v for v in np.asarray(x, dtype=np.float64)]


def cyclic(shape, lo, hi, dt):
    return np.resize(np.arange(lo, hi + 1, dtype=dt), int(np.prod(shape)))


def host(dt, shape, values):
    return Tensor.of(dt, shape, np.asarray(values, dtype=dt))


def cfg_of(t):
    return np.array(t.ndc.asInlineArray(), dtype=np.int32)


# ---- oracle ------------------------------------------------------------------------------------------------------
def _orc_bin(orc, op, x, y, data, dt, scalar=None):
    """x op y for two views (host tensors that share `data`), or x op scalar; returns dense items."""
    out = np.zeros(x.size, dtype=dt)
    ocfg = orc.dense_cfg(list(x.shape))
    if scalar is not None:
        return orc.scalarization(op, -1, out, ocfg, data[0], cfg_of(x), scalar)
    return orc.elementwise(op, -1, out, ocfg, data[0], cfg_of(x), data[1], cfg_of(y))


@pytest.mark.parametrize("dt", ["f64", "f32"])
def test_oracle_cross_device_system_test(scripts, orc, dt):
    g = scripts["cross_device_system_test"]
    T = F[dt]
    c = g["conv_same_shape"]
    a = np.array(c["a"], dtype=T)
    out = orc.convolve(np.zeros(1, dtype=T), orc.dense_cfg(c["expected_shape"]), a, orc.dense_cfg(c["shape"]), np.array(c["b"], dtype=T), orc.dense_cfg(c["shape"]))
    assert out.tolist() == c["expected"]
    m = g["elementwise_mul"]
    cf = orc.dense_cfg(m["shape"])
    assert orc.elementwise("multiply", -1, np.zeros(4, dtype=T), cf, np.array(m["a"], dtype=T), cf, np.array(m["b"], dtype=T), cf).tolist() == m["expected"]
    s = g["softplus"]
    cf = orc.dense_cfg(s["shape"])
    got = orc.activation("softplus", -1, np.zeros(15, dtype=T), cf, np.array(s["x"], dtype=T), cf)
    assert five_decimals(got) == s["expected_5_decimals"]
    for key in ("conv_rank3", "conv_with_gradient"):
        c = g[key]
        a, b = np.array(c["a"], dtype=T), np.array(c["b"], dtype=T)
        out = orc.convolve(np.zeros(len(c["expected"]), dtype=T), orc.dense_cfg(c["expected_shape"]), a, orc.dense_cfg(c["a_shape"]), b, orc.dense_cfg(c["b_shape"]))
        assert out.tolist() == c["expected"], key
    c = g["conv_with_gradient"]
    grad = orc.deconvolve(np.zeros(4, dtype=T), orc.dense_cfg(c["a_shape"]), np.array(c["b"], dtype=T), orc.dense_cfg(c["b_shape"]),
                          np.array(c["error"], dtype=T), orc.dense_cfg(c["expected_shape"]))
    assert grad.tolist() == c["gradient_of_a"]
    c = g["conv_large_constant"]
    a = np.full(int(np.prod(c["a_shape"])), c["a_value"], dtype=T); b = np.full(int(np.prod(c["b_shape"])), c["b_value"], dtype=T)
    out = orc.convolve(np.zeros(int(np.prod(c["expected_shape"])), dtype=T), orc.dense_cfg(c["expected_shape"]), a, orc.dense_cfg(c["a_shape"]), b, orc.dense_cfg(c["b_shape"]), workers=8)
    assert (out == c["expected_every_item"]).all()


@pytest.mark.parametrize("dt", ["f64", "f32"])
def test_oracle_matmul_known_answers(scripts, orc, dt):
    T = F[dt]
    for row in scripts["matmul_core"]["rows"]:
        for rm in (True, False):
            A = np.array(row["A"], dtype=T).reshape(row["M"], row["K"]); B = np.array(row["B"], dtype=T).reshape(row["K"], row["N"])
            if rm:
                got = orc.gemm(True, A.reshape(-1), B.reshape(-1), row["M"], row["K"], row["N"])
            else:       # column-major storage of both operands and of the product (Matrix_Multiplication_Spec 'COL' rows)
                got = orc.gemm(False, A.T.copy().reshape(-1), B.T.copy().reshape(-1), row["M"], row["K"], row["N"]).reshape(row["N"], row["M"]).T.reshape(-1)
            assert got.tolist() == row["C"], (row, rm)
    m = scripts["matmul_method"]
    A = np.resize(np.array(m["a_fill"], dtype=T), 7); B = np.resize(np.array(m["b_fill"], dtype=T), 56)
    assert orc.gemm(True, A, B, 1, 7, 8).tolist() == m["expected"]


@pytest.mark.parametrize("dt", ["f64", "f32"])
def test_oracle_slice_scripts(scripts, orc, dt):
    """x + y on two overlapping row slices of one tensor, and the 3x3 stencil built from slices and scalar products."""
    T = F[dt]
    g = scripts["slice_addition"]
    data = cyclic(g["shape"], g["fill_from"], g["fill_to"], T)
    a = host(T, g["shape"], data)
    x, y = a[1:-1, :], a[0:-2, :]
    t = _orc_bin(orc, "add", x, y, (data, data), T)
    assert list(x.shape) == g["result_shape"] and t[:50].tolist() == g["first_items"]
    for key in ("small", "large"):
        m = scripts["manual_convolution"][key]
        data = cyclic(m["shape"], m["fill_from"], m["fill_to"], T)
        a = host(T, m["shape"], data)
        x, y, z, u = a[1:-1, :], a[0:-2, :], a[2:, :], a[1:-1, 1:-1]
        xy = _orc_bin(orc, "add", x, y, (data, data), T)
        rows, cols = x.shape
        xy_t = host(T, (rows, cols), xy)
        rowconvol = orc.elementwise("add", -1, np.zeros(rows * cols, dtype=T), orc.dense_cfg([rows, cols]), xy, cfg_of(xy_t), data, cfg_of(z))
        rc = host(T, (rows, cols), rowconvol)
        k, v, j = rc[:, 1:-1], rc[:, 0:-2], rc[:, 2:]
        kv = _orc_bin(orc, "add", k, v, (rowconvol, rowconvol), T)
        kv_t = host(T, k.shape, kv)
        kvj = orc.elementwise("add", -1, np.zeros(k.size, dtype=T), orc.dense_cfg(list(k.shape)), kv, cfg_of(kv_t), rowconvol, cfg_of(j))
        nine_u = _orc_bin(orc, "multiply", u, None, (data,), T, scalar=9.0)
        dense = orc.dense_cfg(list(k.shape))
        colconvol = orc.elementwise("subtract", -1, np.zeros(k.size, dtype=T), dense, kvj, dense, nine_u, dense)
        got = {"x": x.items, "y": y.items, "z": z.items, "rowconvol": rowconvol, "k": k.items, "v": v.items, "j": j.items, "u": u.items, "colconvol": colconvol}
        for name, want in m.items():
            if name in got:
                assert np.asarray(got[name])[:len(want)].tolist() == want, (key, name)


# ---- device ------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def device():
    from neureka_amd import HipDevice
    return HipDevice.get(0)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["f64", "f32"])
def test_device_cross_device_system_test(scripts, device, dt):
    g = scripts["cross_device_system_test"]
    T = F[dt]
    say("CrossDeviceSystemTest", dt)
    m = g["elementwise_mul"]
    a, b = host(T, m["shape"], m["a"]).to(device), host(T, m["shape"], m["b"]).to(device)
    assert (a * b).items.tolist() == m["expected"]
    c = g["conv_same_shape"]
    out = a.conv(b)
    assert list(out.shape) == c["expected_shape"] and out.items.tolist() == c["expected"]
    s = g["softplus"]
    from neureka_amd.function import Function
    got = Function.of("softplus(I[0])")(host(T, s["shape"], s["x"]).to(device))
    assert five_decimals(got.items) == s["expected_5_decimals"]
    sm = g["scalar_mul"]
    assert (host(T, (2,), sm["a"]).to(device) * host(T, (2,), sm["b"]).to(device)).items.tolist() == sm["expected"]
    c = g["conv_rank3"]
    out = host(T, c["a_shape"], c["a"]).to(device).conv(host(T, c["b_shape"], c["b"]).to(device))
    assert list(out.shape) == c["expected_shape"] and out.items.tolist() == c["expected"]
    c = g["conv_large_constant"]
    out = Tensor.of(T, c["a_shape"], c["a_value"]).to(device).conv(Tensor.of(T, c["b_shape"], c["b_value"]).to(device))
    assert list(out.shape) == c["expected_shape"] and (out.items == c["expected_every_item"]).all()
    c = g["conv_with_gradient"]
    ta = host(T, c["a_shape"], c["a"]).to(device).setRqsGradient(True)
    out = ta.conv(host(T, c["b_shape"], c["b"]).to(device))
    assert out.items.tolist() == c["expected"]
    out.backward(host(T, c["expected_shape"], c["error"]).to(device))
    assert ta.gradient.items.tolist() == c["gradient_of_a"]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["f64", "f32"])
def test_device_matmul_known_answers(scripts, device, dt):
    T = F[dt]
    say("matmul known answers", dt)
    m = scripts["matmul_method"]
    c = host(T, m["a_shape"], np.resize(m["a_fill"], 7)).to(device).matMul(host(T, m["b_shape"], np.resize(m["b_fill"], 56)).to(device))
    assert list(c.shape) == [1, 8] and c.items.tolist() == m["expected"]
    from neureka_amd import Layout
    for row in scripts["matmul_core"]["rows"]:
        for layout in (Layout.ROW_MAJOR, Layout.COLUMN_MAJOR):
            a = host(T, (row["M"], row["K"]), row["A"]).to(device).toLayoutCopy(layout)
            b = host(T, (row["K"], row["N"]), row["B"]).to(device).toLayoutCopy(layout)
            c = a.matMul(b)
            assert list(c.shape) == [row["M"], row["N"]] and c.items.tolist() == row["C"], (row, layout)
    for row in scripts["matmul_transposed"]["rows"]:
        M, K, N = row["M"], row["K"], row["N"]
        a = host(T, (K, M) if row["a_t"] else (M, K), np.resize(np.array(row["A"], dtype=T), M * K)).to(device)
        b = host(T, (N, K) if row["b_t"] else (K, N), np.resize(np.array(row["B"], dtype=T), K * N)).to(device)
        if row["a_t"]: a = a.T()
        if row["b_t"]: b = b.T()
        c = a.matMul(b)
        assert list(c.shape) == [M, N] and c.items.tolist() == row["C"], row


@pytest.mark.gpu
@pytest.mark.parametrize("dt", ["f64", "f32"])
def test_device_slice_scripts(scripts, device, dt):
    T = F[dt]
    say("slice addition and the stencil from slices", dt)
    g = scripts["slice_addition"]
    a = host(T, g["shape"], cyclic(g["shape"], g["fill_from"], g["fill_to"], T)).to(device)
    t = a[1:-1, :] + a[0:-2, :]
    assert list(t.shape) == g["result_shape"] and t.items[:50].tolist() == g["first_items"]
    for key in ("small", "large"):
        m = scripts["manual_convolution"][key]
        a = host(T, m["shape"], cyclic(m["shape"], m["fill_from"], m["fill_to"], T)).to(device)
        x, y, z = a[1:-1, :], a[0:-2, :], a[2:, :]
        rowconvol = x + y + z
        k, v, j = rowconvol[:, 1:-1], rowconvol[:, 0:-2], rowconvol[:, 2:]
        u = a[1:-1, 1:-1]
        colconvol = k + v + j - u * 9
        got = {"x": x, "y": y, "z": z, "rowconvol": rowconvol, "k": k, "v": v, "j": j, "u": u, "colconvol": colconvol}
        for name, want in m.items():
            if name in got:
                assert got[name].items[:len(want)].tolist() == want, (key, name)
