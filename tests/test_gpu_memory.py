"""The buffer pool behind nk_alloc / nk_free and the staged host transfers behind nk_h2d / nk_d2h.

The reference allocates an OpenCL buffer per tensor and releases it when the tensor is collected
(OpenCLDevice.java:465,954-966); what must hold here is what those calls promise -- a buffer nobody else owns, data that
arrives whole -- while blocks change owners without a wait on the device's one in-order stream."""
import ctypes as C
import threading

import numpy as np
import pytest

from helpers import assert_bits
from neureka_amd import Tensor, _lib

pytestmark = pytest.mark.gpu


def say(*a):
    print("[case]", *a, flush=True)


def test_a_freed_block_serves_the_next_allocation_of_its_class(device):
    say("pool reuse")
    device.sync(); device.trimPool()
    s0 = device.poolStats()
    assert s0["resting_blocks"] == 0 and s0["resting_bytes"] == 0
    a = device.allocate(np.float32, 100_000)
    ptr = a.ptr
    a.release()
    s1 = device.poolStats()
    assert s1["resting_blocks"] == 1 and s1["resting_bytes"] >= 400_000 and s1["driver_allocations"] == s0["driver_allocations"] + 1
    b = device.allocate(np.float32, 99_000)             # the same size class: the block at rest, no call to the driver
    s2 = device.poolStats()
    assert b.ptr == ptr and s2["driver_allocations"] == s1["driver_allocations"] and s2["reuses"] == s1["reuses"] + 1
    assert s2["resting_blocks"] == 0
    c = device.allocate(np.float32, 300_000)            # another class: a new block
    assert c.ptr != ptr and device.poolStats()["driver_allocations"] == s1["driver_allocations"] + 1
    # the bound a view is checked against is what the caller asked for, not the block's size
    with pytest.raises(_lib.HipError):
        device._read(b, 99_000, 1)
    b.release(); c.release()
    assert device.poolStats()["resting_blocks"] == 2
    device.trimPool()
    assert device.poolStats()["resting_blocks"] == 0 and device.poolStats()["resting_bytes"] == 0


def test_the_limit_sends_blocks_back_to_the_driver(device):
    say("pool limit")
    device.sync(); device.trimPool()
    try:
        device.configurePool(max_resting_bytes=1 << 20)
        small = [device.allocate(np.uint8, 300 << 10) for _ in range(4)]
        big = device.allocate(np.uint8, 8 << 20)
        for d in small:
            d.release()
        assert device.poolStats()["resting_bytes"] <= 1 << 20          # three blocks of 300 KiB fit, the fourth pushed one out
        big.release()                                                 # larger than the limit: released at once
        assert device.poolStats()["resting_bytes"] <= 1 << 20
    finally:
        device.configurePool(poison=True)                             # the session's setting (conftest)
    device.trimPool()


def test_fresh_blocks_hold_arbitrary_bytes_and_operations_do_not_care(device, orc):
    """With poisoning on, every block arrives filled with 0xFF bytes: a drain that is allocated without the fill must
    be written in full by the kernel it goes to.  (The session runs with poisoning on, so every other test of the
    Tensor API proves the same for its operation.)"""
    say("poisoned drains")
    device.configurePool(poison=True)
    raw = device.allocate(np.float32, 1000)
    assert np.isnan(device._read_all(raw)).all()
    raw.release()
    rng = np.random.default_rng(5)
    a = rng.uniform(-1, 1, (33, 1, 65)).astype(np.float32); b = rng.uniform(-1, 1, (1, 17, 65)).astype(np.float32)
    ta = Tensor.of(np.float32, a.shape, a).to(device); tb = Tensor.of(np.float32, b.shape, b).to(device)
    assert_bits((ta + tb).items.reshape(33, 17, 65), a + b, "broadcast add into a poisoned drain")
    assert_bits((ta * tb).items.reshape(33, 17, 65), a * b, "broadcast multiply into a poisoned drain")
    x = rng.standard_normal((6, 40, 44)).astype(np.float32); k = rng.standard_normal((6, 5, 5)).astype(np.float32)
    tx = Tensor.of(np.float32, x.shape, x).to(device).setRqsGradient(True); tk = Tensor.of(np.float32, k.shape, k).to(device).setRqsGradient(True)
    y = tx.conv(tk)
    assert not np.isnan(y.items).any()
    y.backward(Tensor.of(np.float32, y.shape, rng.standard_normal(y.size).astype(np.float32)))
    assert not np.isnan(tx.gradient.items).any() and not np.isnan(tk.gradient.items).any()
    m = Tensor.of(np.float32, (70, 50), rng.integers(-5, 6, 3500).astype(np.float32)).to(device)
    n = Tensor.of(np.float32, (50, 30), rng.integers(-5, 6, 1500).astype(np.float32)).to(device)
    assert (m.matMul(n).items.reshape(70, 30) == m.items.reshape(70, 50).astype(np.float64) @ n.items.reshape(50, 30).astype(np.float64)).all()
    assert not np.isnan(m.sum().items).any()


def test_ten_thousand_allocations_from_four_threads_between_kernels(device):
    """4 threads x 2500 rounds: three buffers of a mixed size each, two filled with values of the round, their sum
    launched into the third, the sources freed at once (their blocks go to whoever allocates next, while the kernel that
    reads them may still be queued); every result is read back some rounds later and must be exact."""
    say("pool under threads")
    lib, h = device._lib, device.handle
    one = np.array([1, 1, 1, 0, 1], dtype=np.int32)      # descriptor of a dense vector: shape | strides | indicesMap | offset | spread
    errors = []
    s0 = device.poolStats()

    def worker(seed):
        try:
            rng = np.random.default_rng(seed)
            pending = []
            for r in range(2500):
                n = int(rng.choice([1, 3, 64, 1000, 4097, 65_536, 250_001, 1_048_576])) + int(rng.integers(0, 5))
                va, vb = np.float32(rng.uniform(-4, 4)), np.float32(rng.uniform(-4, 4))
                a, b, out = (device.allocate(np.float32, n) for _ in range(3))
                device._fill(a, 0, n, va); device._fill(b, 0, n, vb)
                cfg = one.copy(); cfg[0] = n
                p = _lib.cfg_ptr(cfg)
                _lib.check(lib.nk_elementwise(h, _lib.OP["add"], -1, _lib.F32, 1, out.ptr, p, a.ptr, p, b.ptr, p, n))
                a.release(); b.release()
                pending.append((out, n, va + vb))
                if len(pending) > 6:
                    o, m, want = pending.pop(0)
                    got = device._read_all(o)
                    if not (got.view(np.uint32) == np.float32(want).view(np.uint32)).all():
                        errors.append((seed, r, m, float(want), got[:4].tolist()))
                    o.release()
            for o, m, want in pending:
                got = device._read_all(o)
                if not (got.view(np.uint32) == np.float32(want).view(np.uint32)).all():
                    errors.append((seed, "tail", m, float(want), got[:4].tolist()))
                o.release()
        except Exception as e:       # noqa: BLE001 - reported below, on the main thread
            errors.append((seed, repr(e)))

    live_before = device.liveBuffers()
    threads = [threading.Thread(target=worker, args=(100 + i,)) for i in range(4)]
    for t in threads: t.start()
    for t in threads: t.join()
    assert not errors, errors[:3]
    assert device.liveBuffers() == live_before
    s1 = device.poolStats()
    assert s1["reuses"] - s0["reuses"] > 28_000          # 30 000 allocations, all but the first of each class from blocks at rest
    assert s1["driver_allocations"] - s0["driver_allocations"] < 1000


@pytest.mark.parametrize("nbytes", [1, 3, 4096, 65_537, (256 << 10) + 1, (1 << 20) - 1, 6 << 20, (17 << 20) + 12_345, (64 << 20) + 7])
def test_host_transfers_round_trip_at_odd_sizes_and_offsets(device, nbytes):
    say("staged transfer", nbytes)
    rng = np.random.default_rng(nbytes)
    pad = 13
    buf = device.allocate(np.uint8, nbytes + 2 * pad)
    device._fill(buf, 0, nbytes + 2 * pad, 0xAB)
    host = rng.integers(0, 256, nbytes + 3, dtype=np.uint8)[3:]          # a host pointer off every alignment
    _lib.check(device._lib.nk_h2d(device.handle, buf.ptr, pad, host.ctypes.data_as(C.c_void_p), nbytes))
    back = np.zeros(nbytes + 2 * pad + 1, dtype=np.uint8)[1:]
    _lib.check(device._lib.nk_d2h(device.handle, back.ctypes.data_as(C.c_void_p), buf.ptr, 0, nbytes + 2 * pad))
    assert (back[:pad] == 0xAB).all() and (back[pad + nbytes:] == 0xAB).all(), "bytes around the written range changed"
    assert back[pad:pad + nbytes].tobytes() == host.tobytes()
    part = np.zeros(max(1, nbytes // 3), dtype=np.uint8)                 # a read from the middle
    start = pad + nbytes // 2
    count = min(part.size, nbytes + pad - start)
    _lib.check(device._lib.nk_d2h(device.handle, part.ctypes.data_as(C.c_void_p), buf.ptr, start, count))
    assert part[:count].tobytes() == host[nbytes // 2: nbytes // 2 + count].tobytes()
    buf.release()


def test_transfers_from_several_threads(device):
    say("staged transfers under threads")
    errors = []

    def worker(seed):
        rng = np.random.default_rng(seed)
        for r in range(12):
            n = int(rng.integers(1, 3 << 20))
            host = rng.integers(0, 256, n, dtype=np.uint8)
            d = device.allocate(np.uint8, n)
            device._write(d, 0, host)
            if device._read_all(d).tobytes() != host.tobytes():
                errors.append((seed, r, n))
            d.release()

    threads = [threading.Thread(target=worker, args=(7 + i,)) for i in range(4)]
    for t in threads: t.start()
    for t in threads: t.join()
    assert not errors, errors
