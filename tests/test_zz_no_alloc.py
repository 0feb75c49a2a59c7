"""nk_sum_static, the entry point that allocates nothing: same bits as nk_sum, on two calls in a row (the second on a
smaller input, so that stale partial results of the first would show), and no change in the device's allocations."""
import ctypes as C

import numpy as np
import pytest

from helpers import assert_bits

pytestmark = pytest.mark.gpu


def _sum_through(device, entry, data, out):
    from neureka_amd import _lib
    code = _lib.F32 if data.dtype == np.float32 else _lib.F64
    _lib.check(getattr(device._lib, entry)(device.handle, code, data.ptr, data.size, out.ptr))
    return device._read(out, 0, 1)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_static_sum_matches_nk_sum_on_two_calls_in_a_row(device, orc, dt):
    from neureka_amd import _lib
    rng = np.random.default_rng(71)
    big = rng.standard_normal((1 << 22) + 12345).astype(dt)      # three launches: 2 levels, 2 levels, tail
    small = rng.standard_normal(40961).astype(dt)                # one block finishes it
    bufs = [device.allocateFromAll(x) for x in (big, small)]
    out = device.allocate(dt, 1)
    try:
        want = [_sum_through(device, "nk_sum", b, out) for b in bufs]       # also grows the workspace once
        live_before = device.liveBuffers()
        for x, b, w in zip((big, small), bufs, want):
            print(f"[no-alloc] {np.dtype(dt).name} n={x.size}", flush=True)
            got = _sum_through(device, "nk_sum_static", b, out)
            assert _lib.last_path() == "tile_tree_128_static"
            assert_bits(got, w, f"nk_sum_static vs nk_sum, n={x.size}")
            assert_bits(got, np.array([orc.sum_tree(x)], dtype=dt), f"nk_sum_static vs the CPU tree, n={x.size}")
        assert device.liveBuffers() == live_before
    finally:
        for b in bufs + [out]:
            b.release()


def test_static_sum_rejects_what_it_cannot_hold(device):
    from neureka_amd import _lib
    data = device.allocate(np.float32, 16)
    out = device.allocate(np.float32, 1)
    try:
        rc = device._lib.nk_sum_static(device.handle, _lib.F32, data.ptr, (1 << 30) + 1, out.ptr)
        assert rc != 0
        msg = device._lib.nk_last_error().decode()
        assert "exceeds the maximum" in msg, msg
    finally:
        data.release(); out.release()
