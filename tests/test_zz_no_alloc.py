"""nk_sum_static, the entry point that allocates nothing: the bits of the CPU tree and of nk_sum, on calls in a row (each
on a smaller input than the one before, so that stale partial results would show), from a device handle on which nk_sum
has never run (its grow-on-demand workspace does not exist yet, so a fall-back to it would have to allocate), with the
driver's free memory, the pool's count of driver allocations and the registry of live buffers unchanged across the calls."""
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
def test_static_sum_allocates_nothing_and_matches_the_tree(orc, dt):
    from neureka_amd import HipDevice, _lib
    fresh = HipDevice(0)                 # a handle of its own: no workspace yet, an empty pool
    try:
        rng = np.random.default_rng(71)
        # A tile-level launch covers two levels of the tree (a factor of 16 384).  2^29 + 12345 floats: two tile-level
        # launches -- the second reads the partial results of the first out of the scratch array and writes behind them --
        # and the tail; 2^22 + 12345: one tile-level launch and the tail; 30001: the tail alone.  (f64 leaves the 4 GiB case out.)
        sizes = ((1 << 29) + 12345, (1 << 22) + 12345, 30001) if dt == np.float32 else ((1 << 23) + 4321, (1 << 22) + 12345, 30001)
        inputs = [rng.standard_normal(n, dtype=np.float32).astype(dt) if n > (1 << 28) else rng.standard_normal(n).astype(dt) for n in sizes]
        bufs = [fresh.allocateFromAll(x) for x in inputs]
        out = fresh.allocate(dt, 1)
        fresh._read(out, 0, 1)           # the staging chunks of the transfers exist from here on
        fresh.sync()
        free_before, pool_before, live_before = fresh.freeMemory(), fresh.poolStats(), fresh.liveBuffers()
        got = []
        for x, b in zip(inputs, bufs):
            print(f"[no-alloc] {np.dtype(dt).name} n={x.size}", flush=True)
            got.append(_sum_through(fresh, "nk_sum_static", b, out))
            assert _lib.last_path() == "tile_tree_128_static"
        fresh.sync()
        assert fresh.freeMemory() == free_before, "the driver's free memory changed across nk_sum_static"
        assert fresh.poolStats()["driver_allocations"] == pool_before["driver_allocations"]
        assert fresh.liveBuffers() == live_before
        for x, g in zip(inputs, got):
            assert_bits(g, np.array([orc.sum_tree(x)], dtype=dt), f"nk_sum_static vs the CPU tree, n={x.size}")
        for x, b, g in zip(inputs, bufs, got):      # nk_sum comes last: it allocates the workspace
            assert_bits(_sum_through(fresh, "nk_sum", b, out), g, f"nk_sum vs nk_sum_static, n={x.size}")
        for b in bufs + [out]:
            b.release()
    finally:
        fresh.dispose()


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
