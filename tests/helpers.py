"""Shared helpers of the test-suite (no GPU use at import)."""
import decimal

import numpy as np

# Tolerances of the parity contract.  + - * and copies are compared bit for bit; transcendental
# activations and reductions (convolution, matmul) within RTOL relative, with an absolute floor of four rounding
# quanta of a double near 1: the reference's own formulas 2/(1+e^-2x)-1 and e^x-1 are evaluated in double (also for
# float tensors) and return multiples of 2^-52 near 0, whatever the true value is.
RTOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}
ATOL = {np.dtype(np.float32): 2.0 ** -50, np.dtype(np.float64): 2.0 ** -50}


def assert_close(got, want, what=""):
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    dt = np.dtype(want.dtype)
    both_nan = np.isnan(got) & np.isnan(want)
    both_inf = np.isinf(want) & (got == want)
    with np.errstate(invalid="ignore"):          # inf - inf in the difference of matching infinities
        ok = both_nan | both_inf | (np.abs(got - want) <= RTOL[dt] * np.abs(want) + ATOL[dt])
    if not ok.all():
        bad = np.flatnonzero(~ok.reshape(-1))
        i = bad[0]
        raise AssertionError(f"{what}: {bad.size} of {want.size} values outside rtol={RTOL[dt]} atol={ATOL[dt]}; "
                             f"first at {i}: got {got.reshape(-1)[i]!r}, want {want.reshape(-1)[i]!r}")


def assert_bits(got, want, what=""):
    """Bit-for-bit equality (distinguishes -0.0 from 0.0; NaNs must match as NaN)."""
    got, want = np.ascontiguousarray(got), np.ascontiguousarray(want)
    assert got.dtype == want.dtype and got.shape == want.shape, f"{what}: {got.dtype}{got.shape} vs {want.dtype}{want.shape}"
    u = np.uint32 if got.dtype.itemsize == 4 else np.uint64
    gb, wb = got.view(u), want.view(u)
    same = (gb == wb) | (np.isnan(got) & np.isnan(want))
    if not same.all():
        bad = np.flatnonzero(~same.reshape(-1))
        i = bad[0]
        raise AssertionError(f"{what}: {bad.size} of {want.size} values differ in bits; first at {i}: "
                             f"got {got.reshape(-1)[i]!r}, want {want.reshape(-1)[i]!r}")


def norm_tolerance(a_abs_dot_b_abs, dtype):
    """Reductions: |delta| <= rtol * sum_i |a_i||b_i| per output (the bound a re-ordered sum can meet)."""
    return RTOL[np.dtype(dtype)] * a_abs_dot_b_abs + ATOL[np.dtype(dtype)]


def rounded_sum(values, places=3):
    """sum(BigDecimal(v).round(3)).round(3) of Calculus_Stress_Test.groovy:204-205 (HALF_UP)."""
    q = decimal.Decimal(1).scaleb(-places)
    total = decimal.Decimal(0)
    for v in values:
        total += decimal.Decimal(float(v)).quantize(q, rounding=decimal.ROUND_HALF_UP)
    return total.quantize(q, rounding=decimal.ROUND_HALF_UP)


def java_float_to_string(v, is_double):
    """Float.toString / Double.toString for integral values of moderate size (enough for the matmul hashes)."""
    f = float(v)
    if f == int(f) and abs(f) < 1e7:
        return f"{int(f)}.0" if not (f == 0 and np.signbit(f)) else "-0.0"
    raise ValueError("only integral values below 1e7 are supported")


def java_array_hash(arr):
    """Arrays.toString(float[]/double[]).hashCode()"""
    s = "[" + ", ".join(java_float_to_string(v, arr.dtype == np.float64) for v in arr) + "]"
    h = 0
    for ch in s:
        h = (31 * h + ord(ch)) & 0xFFFFFFFF
    return h - (1 << 32) if h >= (1 << 31) else h


def fill_it(n, seed, dtype):
    """InternalMatMulTest._fillIt32/_fillIt64: data[i] = ((i + (32**seed) % 11) % 11) - 5"""
    h = (32 ** seed) % 11
    return (((np.arange(n, dtype=np.int64) + h) % 11) - 5).astype(dtype)


VIEW_DTYPES = {"f64": np.float64, "f32": np.float32, "i32": np.int32, "i8": np.int8}


def view_row_parent(row):
    """The parent array of a row of tests/golden/reference_views.json: listed values, a Groovy range cycled through the
    shape (Tensor.of(shape, -3d..7d)) or a cycle of given values (andFill)."""
    dt = VIEW_DTYPES[row["dtype"]]
    size = int(np.prod(row["shape"]))
    if "values" in row:
        src = np.asarray(row["values"], dtype=dt)
    elif "range" in row:
        src = np.arange(row["range"][0], row["range"][1] + 1).astype(dt)
    else:
        src = np.asarray(row["cycle"], dtype=dt)
    return np.resize(src, size).astype(dt)


def apply_view_chain(t, chain):
    """Applies the chain of a row of tests/golden/reference_views.json to a Tensor."""
    for step in chain:
        kind = step[0]
        if kind == "slice":
            keys = []
            for r in step[1:]:
                if isinstance(r, int):
                    keys.append(r)
                else:
                    first, last = r[0], r[1]
                    keys.append(slice(first, last + 1, r[2] if len(r) > 2 else 1))
            t = t.getAt(*keys)
        elif kind == "all":
            t = t.getAt(*[slice(None)] * t.rank)
        elif kind == "T":
            t = t.T()
        elif kind == "pad_front":
            t = t.permute(-1, *range(t.rank))
        else:
            raise ValueError(kind)
    return t
