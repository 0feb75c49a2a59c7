#!/usr/bin/env python3
"""Benchmark of the HipDevice hot path on one MI355X.

Workload (the configuration the metric is quoted on): broadcast elementwise add and multiply,
f32 [1024,1,512] o [1,2048,512] -> [1024,2048,512], uniform[-1,1] from a seed.  One step = one add launch
plus one multiply launch through the C ABI of libneureka_hip.so, inputs and output resident in HBM.

Prints ONE JSON line: whole-job throughput in GB/s of algorithmic bytes (`value`), the roofline of the
dominant kernel measured with HIP events on the device's own stream (`roofline`), the CPU oracle timed
on this box's host cores on a bounded sample (`cpu_baseline`), and kernel-level figures for the other
configurations (`others`: GB/s or GFLOP/s with their fraction of the HBM / fp32-matrix peak).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
FP32_PEAK_TFLOPS = 157.3       # MI355X dense fp32 matrix, published
FP64_PEAK_TFLOPS = 78.6        # MI355X dense fp64 matrix, published
# HBM bytes per launch of the headline kernel come from two rocprofv3 --pmc runs (FETCH_SIZE, then WRITE_SIZE, each
# scaled by what the same counter reads for a plain 1 GiB copy); the command that writes the profile summaries writes
# the figure, the kernel it belongs to and a digest of that kernel's sources into this file.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "rows_binary_lean_kernel_broadcast_c2.json")
SETTLE_MS = 60.0               # untimed load before the warm-up steps, so that the timed steps run at the working clock
HOST_CORE_SHARE = 16           # host threads one GPU's box grants a job, whatever the machine's core count


def event_time_ms(dev, launch, reps):
    """Average duration of `launch` over `reps` back-to-back launches, HIP events on the device stream."""
    e0, e1 = dev.event(), dev.event()
    dev.record(e0)
    for _ in range(reps):
        launch()
    dev.record(e1)
    return dev.elapsed_ms(e0, e1) / reps


def event_times_ms(dev, launch, reps):
    """Durations of `reps` single launches, each bracketed by its own pair of HIP events on the device stream."""
    events = [dev.event() for _ in range(reps + 1)]
    dev.record(events[0])
    for i in range(reps):
        launch()
        dev.record(events[i + 1])
    return [dev.elapsed_ms(events[i], events[i + 1]) for i in range(reps)]


def cpu_side_of_the_other_configs(cores):
    """The oracle (the reference's CPU kernels restated in C, split like JVMExecutor over `cores` threads) on bounded
    samples of the configurations besides the headline one; every entry says what was timed."""
    from oracle import cpu_oracle as orc
    f32 = np.float32
    rng = np.random.default_rng(3)
    out = {}

    def timed(fn, reps):
        fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    x = rng.uniform(-1, 1, 4096).astype(f32); k = rng.uniform(-1, 1, 9).astype(f32)
    sec = timed(lambda: orc.simple_conv2d(x, k, 64, 64, 3, 3), 200)
    out["conv2d_64x64_3x3"] = {"ms": round(sec * 1e3, 4), "GFLOP/s": round(69192 / sec / 1e9, 3), "cores": 1,
                               "sample": "the whole configuration (SimpleCPUConvolution.ImplF32, one image)"}
    n = 1 << 24
    a, b, c = [rng.standard_normal(n).astype(f32) for _ in range(3)]
    cf = orc.dense_cfg([n]); tmp = np.zeros(n, f32); o = np.zeros(n, f32)

    def chain():
        orc.activation("sig", -1, tmp, cf, a, cf, workers=cores); orc.elementwise("multiply", -1, o, cf, tmp, cf, b, cf, workers=cores)
        orc.elementwise("add", -1, tmp, cf, o, cf, c, cf, workers=cores); orc.activation("tanh", -1, o, cf, tmp, cf, workers=cores)
    sec = timed(chain, 3)
    out["chain_unfused_4_kernels"] = {"ms": round(sec * 1e3, 2), "GB/s": round(40 * n / sec / 1e9, 2), "cores": cores,
                                      "sample": "2^24 of the 2^26 elements, the four kernels the reference runs (10 arrays, 40 B per element)"}
    del a, b, c, tmp, o
    M, K, N = 512, 4096, 4096
    A = rng.uniform(-1, 1, M * K).astype(f32); B = rng.uniform(-1, 1, K * N).astype(f32)
    sec = timed(lambda: orc.gemm(True, A, B, M, K, N, workers=cores), 1)
    out["matmul_4096"] = {"ms": round(sec * 1e3 * 4096 / M, 1), "GFLOP/s": round(2.0 * M * K * N / sec / 1e9, 2), "cores": cores,
                          "sample": "the first 512 of the 4096 rows of A (GEMM.threaded_F32_MxN_RM splits rows), time scaled by 8"}
    M, K, N = 65536, 256, 256
    A = rng.uniform(-1, 1, M * K).astype(f32); B = rng.uniform(-1, 1, K * N).astype(f32)
    sec = timed(lambda: orc.gemm(True, A, B, M, K, N, workers=cores), 1)
    out["matmul_tall_skinny"] = {"ms": round(sec * 1e3, 1), "GFLOP/s": round(2.0 * M * K * N / sec / 1e9, 2), "cores": cores, "sample": "the whole configuration"}
    del A, B
    xs, ks, ys = [64, 256, 256], [64, 5, 5], [1, 252, 252]
    x5 = (rng.standard_normal(64 * 256 * 256) * 0.1).astype(f32); k5 = (rng.standard_normal(1600) * 0.1).astype(f32)
    e5 = rng.standard_normal(252 * 252).astype(f32)
    y = np.zeros(252 * 252, f32)
    sec = timed(lambda: orc.convolve(y, orc.dense_cfg(ys), x5, orc.dense_cfg(xs), k5, orc.dense_cfg(ks), workers=cores), 3)
    out["conv_c5_forward"] = {"ms": round(sec * 1e3, 2), "GFLOP/s": round(203212800 / sec / 1e9, 3), "cores": cores, "sample": "the whole configuration (_convolve32)"}
    dk = np.zeros(1600, f32)
    sec = timed(lambda: orc.deconvolve(dk, orc.dense_cfg(ks), x5, orc.dense_cfg(xs), e5, orc.dense_cfg(ys), workers=cores), 2)
    out["conv_c5_grad_kernel"] = {"ms": round(sec * 1e3, 2), "GFLOP/s": round(203212800 / sec / 1e9, 3), "cores": cores, "sample": "the whole configuration (_deConvolve32)"}
    dx = np.zeros(64 * 256 * 256, f32)
    part = dx.size // 1024
    sec = timed(lambda: orc.run("deconvolve", 0, 0, dx, orc.dense_cfg(xs), k5, orc.dense_cfg(ks), e5, orc.dense_cfg(ys), workers=cores, first=0, limit=part), 1)
    out["conv_c5_grad_input"] = {"ms": round(sec * 1e3 * 1024, 0), "GFLOP/s": round(203212800 / (sec * 1024) / 1e9, 4), "cores": cores,
                                 "sample": "the first 1/1024 of the drain, time scaled by 1024: _deConvolve32 visits every entry of the error for every drain element"}
    return out


def torch_yardstick():
    """--yardstick: the same workloads through PyTorch's own kernels (vendor BLAS, MIOpen, its elementwise and
    reduction kernels) on this GPU, microseconds per call from torch's events over 50 calls after 20 -- a yardstick
    printed beside the figures of this library, never part of them."""
    import torch
    import torch.nn.functional as F
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    d = "cuda:0"
    res = {"torch": torch.__version__}

    def t(name, fn, n=50, warm=20):
        for _ in range(warm): fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n): fn()
        e1.record(); torch.cuda.synchronize()
        res[name] = round(e0.elapsed_time(e1) / n * 1e3, 1)

    a = torch.randn(1024, 1, 512, device=d); b = torch.randn(1, 2048, 512, device=d); o = torch.empty(1024, 2048, 512, device=d)
    t("broadcast_add_us", lambda: torch.add(a, b, out=o))
    ga = torch.empty(1024, 1, 512, device=d); gb = torch.empty(1, 2048, 512, device=d)
    gbias = torch.empty(1, 1, 512, device=d); gs = torch.empty(1024, 1, 1, device=d)
    t("broadcast_backward_grad0_us", lambda: torch.sum(o, dim=1, keepdim=True, out=ga))
    t("broadcast_backward_grad1_us", lambda: torch.sum(o, dim=0, keepdim=True, out=gb))
    t("broadcast_backward_bias_us", lambda: torch.sum(o, dim=(0, 1), keepdim=True, out=gbias))
    t("broadcast_backward_per_slab_us", lambda: torch.sum(o, dim=(1, 2), keepdim=True, out=gs))
    t("sum_2^30_us", lambda: torch.sum(o))
    t("max_index_2^30_us", lambda: torch.argmax(o))
    del o
    n = 1 << 26
    x, y, z = (torch.randn(n, device=d) for _ in range(3)); out = torch.empty(n, device=d)

    def chain(p, q, r, dst):
        s = torch.sigmoid(p); s.mul_(q); s.add_(r); torch.tanh(s, out=dst)
    t("chain_unfused_4_kernels_us", lambda: chain(x, y, z, out))
    xp, yp, zp = (v.view(16384, 4096).t() for v in (x, y, z))
    t("chain_unfused_permuted_us", lambda: chain(xp, yp, zp, out.view(4096, 16384)))
    t("tanh_us", lambda: torch.tanh(x, out=out))
    t("add_us", lambda: torch.add(x, y, out=out))
    t("sum_2^26_us", lambda: torch.sum(x))
    t("max_index_2^26_us", lambda: torch.argmax(x))
    t("dot_2^26_us", lambda: torch.dot(x, y))
    del x, y, z, out
    for name, (M, K, N), dt in (("matmul_4096_us", (4096, 4096, 4096), torch.float32), ("matmul_4000_us", (4000, 4000, 4000), torch.float32),
                                ("matmul_3072_us", (3072, 3072, 3072), torch.float32), ("matmul_3072_f64_us", (3072, 3072, 3072), torch.float64),
                                ("matmul_2560_us", (2560, 2560, 2560), torch.float32), ("matmul_2048_us", (2048, 2048, 2048), torch.float32),
                                ("matmul_1536_us", (1536, 1536, 1536), torch.float32), ("matmul_1024_us", (1024, 1024, 1024), torch.float32),
                                ("matmul_narrow_result_us", (4096, 4096, 64), torch.float32), ("matmul_short_k_us", (3000, 64, 3000), torch.float32),
                                ("matmul_2048_f64_us", (2048, 2048, 2048), torch.float64), ("matmul_1024_f64_us", (1024, 1024, 1024), torch.float64),
                                ("matmul_narrow_result_f64_us", (4096, 4096, 64), torch.float64),
                                ("matmul_tall_skinny_us", (65536, 256, 256), torch.float32), ("matmul_4096_f64_us", (4096, 4096, 4096), torch.float64),
                                ("matmul_matrix_vector_us", (4096, 4096, 1), torch.float32), ("matmul_batch_of_16_rows_us", (16, 4096, 4096), torch.float32),
                                ("matmul_16_outer_products_us", (4096, 16, 4096), torch.float32), ("matmul_batch_of_16_columns_us", (4096, 4096, 16), torch.float32)):
        A = torch.randn(M, K, device=d, dtype=dt); B = torch.randn(K, N, device=d, dtype=dt); C = torch.empty(M, N, device=d, dtype=dt)
        t(name, lambda: torch.mm(A, B, out=C))
    xi = torch.randn(1, 64, 256, 256, device=d, requires_grad=True); w = torch.randn(1, 64, 5, 5, device=d, requires_grad=True)
    t("conv_c5_forward_us", lambda: F.conv2d(xi, w))
    yv = F.conv2d(xi, w); e = torch.randn_like(yv)
    t("conv_c5_grad_input_us", lambda: torch.autograd.grad(yv, xi, e, retain_graph=True))
    t("conv_c5_grad_kernel_us", lambda: torch.autograd.grad(yv, w, e, retain_graph=True))
    img = torch.randn(1, 1, 4096, 4096, device=d); k3 = torch.randn(1, 1, 3, 3, device=d)
    t("conv2d_4096x4096_3x3_us", lambda: F.conv2d(img, k3))
    return res


def counted_traffic(path):
    """(bytes, note): the counter-measured HBM traffic per launch of the headline kernel, or (None, why not) when the
    record is missing, belongs to another kernel plan, or was taken from other sources than the library was built from."""
    from neureka_amd.profile_summary import kernel_sources_digest
    if not os.path.exists(TRAFFIC_FILE):
        return None, "no counter record beside the profile"
    with open(TRAFFIC_FILE) as f:
        rec = json.load(f)
    if rec.get("path") != path:
        return None, f"the counter record is of plan {rec.get('path')}, this run took {path}"
    if rec.get("sources_sha256") != kernel_sources_digest():
        return None, "the kernel's sources changed since the counters were read"
    return int(rec["traffic_bytes"]), f"FETCH_SIZE x {rec['fetch_scale']} + WRITE_SIZE x {rec['write_scale']}, {rec['dispatches']} dispatches"


def percentiles(xs):
    xs = sorted(xs)
    return {"p10": round(xs[len(xs) // 10], 4), "median": round(xs[len(xs) // 2], 4), "p90": round(xs[(len(xs) * 9) // 10], 4)}


def wall_ms(dev, call, reps, warm=10):
    """Host wall clock per call in steady state: `reps` calls queued back to back, one synchronisation at the end; the
    median of three such batches."""
    for _ in range(warm):
        call()
    dev.sync()
    batches = []
    for _ in range(3):
        t0 = time.perf_counter()
        for _ in range(reps):
            call()
        dev.sync()
        batches.append((time.perf_counter() - t0) * 1e3 / reps)
    return sorted(batches)[1]


def memory_figures(dev, C, _lib):
    """What the memory side of an operation costs (the reference pays an allocation and a zero fill per output:
    Broadcast.java:89-92, OpenCLDevice.java:465,478-486): nk_alloc + nk_free of the headline output from the pool and
    from the driver, the zero fill of that output, and the host transfers."""
    lib, h = dev._lib, C.c_uint64(dev.handle)
    nbytes = 4 << 30
    buf = C.c_uint64(0)
    out = {}
    # host transfers: pageable numpy arrays (touched beforehand), blocking calls as the reference's CL_TRUE transfers.
    # Measured before anything below returns memory to the driver: for 100 to 200 ms after a hipFree of gigabytes the
    # copy engines run at two thirds of their rate (the driver clears the released memory with them).
    for label, n in (("6MiB", 6 << 20), ("256MiB", 256 << 20)):
        host = np.ones(n, np.uint8); back = np.ones(n, np.uint8)
        _lib.check(lib.nk_alloc(h, n, C.byref(buf)))
        up = lambda: lib.nk_h2d(h, buf, 0, host.ctypes.data_as(C.c_void_p), n)
        down = lambda: lib.nk_d2h(h, back.ctypes.data_as(C.c_void_p), buf, 0, n)
        reps = 30 if n < (64 << 20) else 6
        for name, fn in (("h2d", up), ("d2h", down)):
            for _ in range(3): fn()
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter(); fn(); ts.append((time.perf_counter() - t0) * 1e3)
            med = sorted(ts)[len(ts) // 2]
            out[f"{name}_{label}_ms"] = round(med, 4)
            out[f"{name}_{label}_GBs"] = round(n / (med * 1e-3) / 1e9, 2)
        _lib.check(lib.nk_free(h, buf))
    dev.sync(); dev.trimPool()
    t0 = time.perf_counter()
    _lib.check(lib.nk_alloc(h, nbytes, C.byref(buf))); _lib.check(lib.nk_free(h, buf))
    cold = (time.perf_counter() - t0) * 1e3

    def pooled():
        lib.nk_alloc(h, nbytes, C.byref(buf)); lib.nk_free(h, buf)
    pool_us = wall_ms(dev, pooled, 2000) * 1e3
    _lib.check(lib.nk_alloc(h, nbytes, C.byref(buf)))
    zero = np.zeros(1, np.float32)
    fill = lambda: lib.nk_fill(h, buf, 0, zero.ctypes.data_as(C.c_void_p), 4, nbytes // 4)
    for _ in range(10): fill()
    fill_ms = event_time_ms(dev, fill, 50)
    _lib.check(lib.nk_free(h, buf))
    out.update({"alloc_free_4GiB_from_pool_us": round(pool_us, 3), "alloc_free_4GiB_from_driver_ms": round(cold, 3),
           "zero_fill_4GiB_ms": round(fill_ms, 4),
           "note": "an output of an operation comes from the pool and, where the kernel writes every element, is not filled"})
    out["h2d_GBs"], out["d2h_GBs"] = out["h2d_256MiB_GBs"], out["d2h_256MiB_GBs"]
    return out


def operation_figures(dev, rng, C, _lib, Function, Tensor, reps):
    """Whole operations beside their kernels: `ms` = wall clock per call through HipBackend (the Python mirror of the
    reference's call path: algorithm choice, call preparation with the drain's allocation, launch, drop of the result),
    `abi_ms` = the same C-ABI calls without the interpreter between them (nk_alloc, the launch, nk_free -- what a JVM
    binding issues), `kernel_ms` = the launch alone into a drain that exists.  Steady state, calls queued back to back."""
    f32 = np.float32
    lib, h = dev._lib, C.c_uint64(dev.handle)
    out = {}

    def record(name, mirror, abi, kernel, n_mirror=None):
        for _ in range(10): kernel()
        k = event_time_ms(dev, kernel, reps)
        e = {"ms": round(wall_ms(dev, mirror, n_mirror or reps), 4)}
        if abi: e["abi_ms"] = round(wall_ms(dev, abi, reps), 4)
        e["kernel_ms"] = round(k, 4)
        e["mirror_over_kernel"] = round(e["ms"] / k, 3)
        if abi: e["abi_over_kernel"] = round(e["abi_ms"] / k, 3)
        out[name] = e

    def abi_sequence(nbytes, launch_with):
        """nk_alloc(nbytes) -> launch_with(buffer) -> nk_free"""
        buf = C.c_uint64(0)
        launch = launch_with(buf)
        def call():
            lib.nk_alloc(h, nbytes, C.byref(buf)); launch(); lib.nk_free(h, buf)
        return call

    def cfg_of(t):
        inline = t.ndc.asInlineArray()
        return inline, _lib.cfg_ptr(inline)

    # C2: a + b
    s1, s2, so = (1024, 1, 512), (1, 2048, 512), (1024, 2048, 512)
    ta = Tensor.of(f32, s1, rng.uniform(-1, 1, s1).astype(f32)).to(dev); tb = Tensor.of(f32, s2, rng.uniform(-1, 1, s2).astype(f32)).to(dev)
    drn = Tensor._on_device(dev, f32, so, zeroed=False)
    keep = [cfg_of(drn), cfg_of(ta), cfg_of(tb)]
    n = drn.size
    def c2(buf):
        return lambda: lib.nk_broadcast(h, _lib.OP["add"], -1, _lib.F32, 3, buf, keep[0][1], ta._data.ptr, keep[1][1], tb._data.ptr, keep[2][1], n)
    record("op_c2_add", lambda: ta + tb, abi_sequence(4 * n, c2), dev.prepared_launch("broadcast", "add", -1, drn, ta, tb))
    dev.free(drn); dev.free(ta); dev.free(tb)

    # C3: tanh(sig(a)*b+c), operation by operation (four kernels, three temporaries) and as the fused operation
    n = 1 << 26
    srcs = [Tensor.of(f32, (n,), rng.standard_normal(n).astype(f32)).to(dev) for _ in range(3)]
    o = Tensor._on_device(dev, f32, (n,), zeroed=False); tmp = Tensor._on_device(dev, f32, (n,), zeroed=False)
    fn = Function.of("tanh(sig(I[0])*I[1]+I[2])", doAD=False)
    fused = dev.optimizedFunctionOf(fn, "chain")
    four = [dev.prepared_launch("activation", "sig", -1, tmp, srcs[0]), dev.prepared_launch("elementwise", "multiply", -1, o, tmp, srcs[1]),
            dev.prepared_launch("elementwise", "add", -1, tmp, o, srcs[2]), dev.prepared_launch("activation", "tanh", -1, o, tmp)]
    record("op_c3_chain", lambda: fn(*srcs), None, lambda: [k() for k in four])
    record("op_c3_chain_fused", lambda: fused(*srcs), None, dev.prepared_launch("fused", fused.program, fused.consts, o, srcs))
    for t in srcs + [o, tmp]: dev.free(t)

    # C4: A @ B
    M = K = N = 4096
    A = Tensor.of(f32, (M, K), rng.uniform(-1, 1, M * K).astype(f32)).to(dev); B = Tensor.of(f32, (K, N), rng.uniform(-1, 1, K * N).astype(f32)).to(dev)
    Cm = Tensor._on_device(dev, f32, (M, N), zeroed=False)
    def c4(buf):
        return lambda: lib.nk_matmul_set(h, _lib.F32, _lib.ROW_MAJOR, M, K, N, A._data.ptr, B._data.ptr, buf)
    record("op_c4_matmul", lambda: A.matMul(B), abi_sequence(4 * M * N, c4), dev.prepared_launch("matmul_set", True, M, K, N, A, B, Cm))
    for t in (A, B, Cm): dev.free(t)

    # C5: x conv k, and the backward pass (both gradients) of that operation
    x5 = Tensor.of(f32, (64, 256, 256), (rng.standard_normal(64 * 256 * 256) * 0.1).astype(f32)).to(dev)
    k5 = Tensor.of(f32, (64, 5, 5), (rng.standard_normal(1600) * 0.1).astype(f32)).to(dev)
    e5 = Tensor.of(f32, (1, 252, 252), rng.standard_normal(252 * 252).astype(f32)).to(dev)
    y5 = Tensor._on_device(dev, f32, (1, 252, 252), zeroed=False)
    dx5 = Tensor._on_device(dev, f32, (64, 256, 256), zeroed=False); dk5 = Tensor._on_device(dev, f32, (64, 5, 5), zeroed=False)
    kc = [cfg_of(y5), cfg_of(x5), cfg_of(k5), cfg_of(e5), cfg_of(dx5), cfg_of(dk5)]
    def c5(buf):
        return lambda: lib.nk_convolution(h, -1, _lib.F32, 3, buf, kc[0][1], x5._data.ptr, kc[1][1], k5._data.ptr, kc[2][1], y5.size)
    record("op_c5_conv_forward", lambda: x5.conv(k5), abi_sequence(4 * y5.size, c5), dev.prepared_launch("convolution", -1, y5, x5, k5), n_mirror=2000)
    bx, bk = C.c_uint64(0), C.c_uint64(0)
    def c5_backward_abi():
        lib.nk_alloc(h, 4 * dx5.size, C.byref(bx)); lib.nk_alloc(h, 4 * dk5.size, C.byref(bk))
        lib.nk_convolution(h, 0, _lib.F32, 3, bx, kc[4][1], k5._data.ptr, kc[2][1], e5._data.ptr, kc[3][1], dx5.size)
        lib.nk_convolution(h, 0, _lib.F32, 3, bk, kc[5][1], x5._data.ptr, kc[1][1], e5._data.ptr, kc[3][1], dk5.size)
        lib.nk_free(h, bx); lib.nk_free(h, bk)
    gx, gk = dev.prepared_launch("convolution", 0, dx5, k5, e5), dev.prepared_launch("convolution", 0, dk5, x5, e5)
    x5.setRqsGradient(True); k5.setRqsGradient(True)
    y = x5.conv(k5)
    def c5_backward():
        x5.gradient = None; k5.gradient = None
        y.backward(e5)
    record("op_c5_backward", c5_backward, c5_backward_abi, lambda: (gx(), gk()), n_mirror=2000)
    x5.gradient = None; k5.gradient = None
    del y
    for t in (x5, k5, e5, y5, dx5, dk5): dev.free(t)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-others", action="store_true", help="skip the figures of the other configurations")
    ap.add_argument("--no-ops", action="store_true", help="skip the whole-operation and memory figures")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one plain 1 GiB device-to-device copy (a copy kernel of known size), so that a "
                         "rocprofv3 --pmc run of this command holds a reference for FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--yardstick", action="store_true",
                    help="also time the same workloads through PyTorch's own kernels (reported under \"yardstick\")")
    ap.add_argument("--yardstick-only", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.yardstick_only:             # the child process of --yardstick: PyTorch brings its own HIP runtime, which
        print(json.dumps(torch_yardstick()))    # does not find the GPU in a process where the system's is already at work
        return
    if args.gpus != 1:
        print("bench.py measures one MI355X: this build has no multi-GPU path (every kernel shards without "
              "exchange), run it with --gpus 1", file=sys.stderr)
        sys.exit(2)

    from neureka_amd import Function, HipDevice, NDConfiguration, Tensor, _lib

    dev = HipDevice.get(0)
    rng = np.random.default_rng(2)
    f32 = np.float32

    # ---- the headline workload -------------------------------------------------------------------------
    s1, s2, so = (1024, 1, 512), (1, 2048, 512), (1024, 2048, 512)
    a = rng.uniform(-1, 1, s1).astype(f32)
    b = rng.uniform(-1, 1, s2).astype(f32)
    ta = Tensor.of(f32, s1, a).to(dev)
    tb = Tensor.of(f32, s2, b).to(dev)
    out = Tensor._on_device(dev, f32, so)
    n_out = int(np.prod(so))
    bytes_per_launch = 4 * (n_out + a.size + b.size)          # 4 301 258 752: write the output once, read each input once

    # the two launches of a step, with their C-ABI arguments marshalled once (the Python wrapper would
    # otherwise spend tens of microseconds per call building descriptors)
    launch_add = dev.prepared_launch("broadcast", "add", -1, out, ta, tb)
    launch_mul = dev.prepared_launch("broadcast", "multiply", -1, out, ta, tb)

    def step():
        launch_add()
        launch_mul()

    if args.calibrate:
        _lib.check(dev._lib.nk_d2d(dev.handle, out._data.ptr, 0, out._data.ptr, 2 << 30, 1 << 30))
    # The clock of an idle device takes about 30 ms of load to reach its working frequency (the first steps after
    # idleness run at 1.5 ms, the 25th at 1.2 ms), more than a handful of warm-up steps: load the device for
    # SETTLE_MS first, untimed, then run the W warm-up steps, synchronise, and time exactly K steps.
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < SETTLE_MS:
        step()
        dev.sync()
    for _ in range(args.warmup):
        step()
    dev.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    dev.sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = 2 * bytes_per_launch / (ms_per_step * 1e-3) / 1e9
    path = _lib.last_path()

    k_add = event_time_ms(dev, launch_add, args.steps)
    k_mul = event_time_ms(dev, launch_mul, args.steps)
    k_ms = 0.5 * (k_add + k_mul)
    achieved = bytes_per_launch / (k_ms * 1e-3) / 1e9
    singles = sorted(event_times_ms(dev, launch_add, 50) + event_times_ms(dev, launch_mul, 50))
    traffic, traffic_note = counted_traffic(path)
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_note,
                "kernel": f"nk::rows_binary_lean_kernel<float, 4, 2, 0, true> ({path})",
                "launch_ms": round(k_ms, 4), "algorithmic_bytes": bytes_per_launch,
                "single_launch_ms": {"p10": round(singles[len(singles) // 10], 4), "median": round(singles[len(singles) // 2], 4),
                                     "p90": round(singles[(len(singles) * 9) // 10], 4), "launches": len(singles)}}

    # spot check of the timed output against numpy (the full parity tests live in tests/)
    got = dev._read(out._data, 5 * 2048 * 512 + 7 * 512, 512)
    assert got.tobytes() == (a[5, 0] * b[0, 7]).tobytes(), "benchmark output is wrong"

    # ---- CPU baseline: the oracle's restatement of CPUBroadcast, scheduled like JVMExecutor ----------------
    cpu = None
    if not args.no_cpu:
        from oracle import cpu_oracle as orc
        cores = min(HOST_CORE_SHARE, len(os.sched_getaffinity(0)))
        rows = 256                                             # sample: the first 256 of 1024 slabs of the output
        sample_shape = (rows, 2048, 512)
        drn = np.zeros(int(np.prod(sample_shape)), dtype=f32)
        a_s = a[:rows].reshape(-1).copy()
        sample_bytes = 4 * (drn.size + a_s.size + b.size)
        passes, spent = 0, 0.0
        while spent < 10.0 and passes < 64:                    # about 10 s of CPU work, add and multiply alternating
            op = "add" if passes % 2 == 0 else "multiply"
            t0 = time.perf_counter()
            orc.broadcast(op, -1, drn, orc.dense_cfg(sample_shape), a_s, orc.dense_cfg((rows, 1, 512)), b.reshape(-1), orc.dense_cfg(s2), workers=cores)
            spent += time.perf_counter() - t0
            passes += 1
        want = (a[0, 0] + b[0, 7]) if op == "add" else (a[0, 0] * b[0, 7])
        assert drn[7 * 512:8 * 512].tobytes() == want.tobytes()
        cpu = {"value": round(passes * sample_bytes / spent / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"{passes} passes (add, multiply alternating) over the first {rows}/1024 slabs of the output "
                         f"({drn.size} elements per pass, {spent:.1f} s in total): the oracle's restatement of "
                         "CPUBroadcast._broadcastF32 split like JVMExecutor over min(host cores, "
                         f"{HOST_CORE_SHARE}) threads ({len(os.sched_getaffinity(0))} cores visible; {HOST_CORE_SHARE} is "
                         "the CPU share of a one-GPU job on this pool, the reference would take availableProcessors()); "
                         "no JVM exists on this box"}
        del drn
    dev.free(out)

    # ---- the other configurations: kernel figures only ------------------------------------------------------
    others = {}
    if not args.no_others:
        reps = max(50, min(args.steps, 100))                   # after 10 warm-up launches each

        def warm(launch):
            # at least 10 launches and about 5 ms of queued work: the clock needs a few milliseconds of load to settle
            t0, count = time.perf_counter(), 0
            while count < 10 or (time.perf_counter() - t0 < 0.005 and count < 2000):
                launch()
                count += 1
            dev.sync()

        def spread(launch):
            # `ms` is the mean of `reps` launches queued back to back between one pair of events; the spread comes from
            # 30 launches with an event after each (an event between two launches costs them their overlap of tail and
            # start, a microsecond or two: these are upper figures for kernels of a few microseconds)
            return percentiles(event_times_ms(dev, launch, 30))

        def hbm(name, nbytes, launch, note=None):
            warm(launch)
            ms = event_time_ms(dev, launch, reps)
            gbs = nbytes / (ms * 1e-3) / 1e9
            others[name] = {"ms": round(ms, 4), "GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "path": _lib.last_path(),
                            "single_launch_ms": spread(launch)}
            if note: others[name]["note"] = note

        def flops(name, nflop, nbytes, launch, f64=False, note=None):
            warm(launch)
            ms = event_time_ms(dev, launch, reps)
            tf = nflop / (ms * 1e-3) / 1e12
            frac = {"frac_fp64": round(tf / FP64_PEAK_TFLOPS, 4)} if f64 else {"frac_fp32": round(tf / FP32_PEAK_TFLOPS, 4)}
            others[name] = {"ms": round(ms, 4), "GFLOP/s": round(tf * 1e3, 1), **frac,
                            "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1), "path": _lib.last_path(), "single_launch_ms": spread(launch)}
            if note: others[name]["note"] = note

        # C2 f64
        a64 = Tensor.of(np.float64, (256, 1, 512), rng.uniform(-1, 1, 256 * 512)).to(dev)
        b64 = Tensor.of(np.float64, (1, 1024, 512), rng.uniform(-1, 1, 1024 * 512)).to(dev)
        o64 = Tensor._on_device(dev, np.float64, (256, 1024, 512))
        hbm("broadcast_add_f64", 8 * (o64.size + a64.size + b64.size), dev.prepared_launch("broadcast", "add", -1, o64, a64, b64))
        for t in (a64, b64, o64): dev.free(t)
        # the headline operation with an inner extent that is no power of two (rows of 2000 bytes)
        a5 = Tensor.of(f32, (1024, 1, 500), rng.uniform(-1, 1, 1024 * 500).astype(f32)).to(dev)
        b5 = Tensor.of(f32, (1, 2048, 500), rng.uniform(-1, 1, 2048 * 500).astype(f32)).to(dev)
        o5 = Tensor._on_device(dev, f32, (1024, 2048, 500))
        hbm("broadcast_add_rows_of_500", 4 * (o5.size + a5.size + b5.size), dev.prepared_launch("broadcast", "add", -1, o5, a5, b5))
        for t in (a5, b5, o5): dev.free(t)

        # C2 backward: the reducing kernel, error [1024,2048,512] -> gradient [1024,1,512] (axis 1 summed) and [1,2048,512]
        err = Tensor._on_device(dev, f32, (1024, 2048, 512))
        for d, tgt, oth in ((0, (1024, 1, 512), (1, 2048, 512)), (1, (1, 2048, 512), (1024, 1, 512))):
            g_t = Tensor._on_device(dev, f32, tgt); z_t = Tensor._on_device(dev, f32, oth)
            hbm(f"broadcast_backward_grad{d}", 4 * (err.size + g_t.size + z_t.size), dev.prepared_launch("broadcast", "add", d, g_t, z_t, err))
            dev.free(g_t); dev.free(z_t)
        # a bias gradient (few outputs, long sums) and the sum over the innermost axis of the same 4 GiB of error
        for name, tgt in (("broadcast_backward_bias", (1, 1, 512)), ("broadcast_backward_per_slab", (1024, 1, 1))):
            g_t = Tensor._on_device(dev, f32, tgt); z_t = Tensor._on_device(dev, f32, tuple(1 if t > 1 else f for t, f in zip(tgt, (1024, 2048, 512))))
            hbm(name, 4 * (err.size + g_t.size + z_t.size), dev.prepared_launch("broadcast", "add", 0, g_t, z_t, err))
            dev.free(g_t); dev.free(z_t)
        # the same 2^30 elements through the whole-tensor reductions: what the fixed tree streams at when its second,
        # latency-bound launch (about 5 us) no longer weighs (the 2^26 entries below are a tenth tail)
        one30 = Tensor._on_device(dev, f32, (1,)); slot30 = dev.allocate(np.int32, 1)
        hbm("sum_2^30", 4 * err.size, dev.prepared("nk_sum", dev.handle, 0, err._data.ptr, err.size, one30._data.ptr))
        hbm("max_index_2^30", 4 * err.size, dev.prepared("nk_reduce_index", dev.handle, 1, 0, err._data.ptr, err.size, slot30.ptr))
        dev.free(one30); slot30.release()
        dev.free(err)
        # rows shorter than a 16-byte vector: [2^20,1,3] + [1,64,3] -> [2^20,64,3] (one element per thread, index arithmetic bound)
        a3 = Tensor.of(f32, (1 << 20, 1, 3), rng.uniform(-1, 1, 3 << 20).astype(f32)).to(dev)
        b3 = Tensor.of(f32, (1, 64, 3), rng.uniform(-1, 1, 192).astype(f32)).to(dev)
        o3s = Tensor._on_device(dev, f32, (1 << 20, 64, 3))
        hbm("broadcast_add_rows_of_3", 4 * (o3s.size + a3.size + b3.size), dev.prepared_launch("broadcast", "add", -1, o3s, a3, b3))
        for t in (a3, b3, o3s): dev.free(t)

        # C3: tanh(sig(a)*b+c) on 2^26 elements: fused, and the reference's 4-kernel sequence
        n = 1 << 26
        srcs = [Tensor.of(f32, (n,), rng.standard_normal(n).astype(f32)).to(dev) for _ in range(3)]
        o = Tensor._on_device(dev, f32, (n,))
        tmp = Tensor._on_device(dev, f32, (n,))
        fn = Function.of("tanh(sig(I[0])*I[1]+I[2])")
        fused = dev.optimizedFunctionOf(fn, "chain")
        hbm("chain_fused_contiguous", 16 * n, dev.prepared_launch("fused", fused.program, fused.consts, o, srcs))
        four = [dev.prepared_launch("activation", "sig", -1, tmp, srcs[0]), dev.prepared_launch("elementwise", "multiply", -1, o, tmp, srcs[1]),
                dev.prepared_launch("elementwise", "add", -1, tmp, o, srcs[2]), dev.prepared_launch("activation", "tanh", -1, o, tmp)]

        def unfused():
            for k in four:
                k()
        hbm("chain_unfused_4_kernels", 40 * n, unfused)
        hbm("activation_tanh", 8 * n, dev.prepared_launch("activation", "tanh", -1, o, srcs[0]))
        hbm("activation_sig", 8 * n, dev.prepared_launch("activation", "sig", -1, o, srcs[0]))
        hbm("elementwise_add", 12 * n, dev.prepared_launch("elementwise", "add", -1, o, srcs[0], srcs[1]))
        hbm("elementwise_mul", 12 * n, dev.prepared_launch("elementwise", "multiply", -1, o, srcs[0], srcs[1]))
        # what the backward pass launches for an activation and for a division, and a heavy forward function
        hbm("activation_tanh_derivative", 8 * n, dev.prepared_launch("activation", "tanh", 0, o, srcs[0]))
        hbm("activation_sig_derivative", 8 * n, dev.prepared_launch("activation", "sig", 0, o, srcs[0]))
        hbm("activation_relu_derivative", 8 * n, dev.prepared_launch("activation", "relu", 0, o, srcs[0]))
        hbm("divide_derivative", 12 * n, dev.prepared_launch("elementwise", "divide", 1, o, srcs[0], srcs[1]))
        hbm("activation_softplus", 8 * n, dev.prepared_launch("activation", "softplus", -1, o, srcs[0]))
        # the slow tails of the elementwise engine, measured so that they are on record: the derivative kernel of the fused
        # chain (double-precision intermediates), general power (the device library's float pow: arithmetic, not memory,
        # bounds both) and a view no fast path takes (every 16th column of every 2nd row: one element per thread)
        dprog, dconsts = fused.derivative_program(0)
        hbm("chain_derivative_by_input0", 16 * n, dev.prepared_launch("fused", dprog, dconsts, o, srcs))
        pos = Tensor.of(f32, (n,), rng.uniform(0.1, 2.0, n).astype(f32)).to(dev)
        hbm("power_tensor_exponent", 12 * n, dev.prepared_launch("elementwise", "power", -1, o, pos, srcs[1]))
        # its derivative by the exponent, a ** b * ln a, which the reference forms in double and rounds once
        hbm("power_derivative_by_exponent", 12 * n, dev.prepared_launch("elementwise", "power", 1, o, pos, srcs[1]))
        dev.free(pos)
        wide = Tensor(f32, NDConfiguration.ofShape((4096, 16384)), None); wide._set_data(srcs[0]._data, dev)
        strided = wide[::2, ::16]
        small = Tensor(f32, NDConfiguration.ofShape(strided.shape), None); small._set_data(o._data, dev)
        hbm("tanh_of_every_16th_column", 8 * strided.size, dev.prepared_launch("activation", "tanh", -1, small, strided))
        # whole-tensor reductions of the same 2^26 elements (the operations that follow the hot path in training loops)
        one = Tensor._on_device(dev, f32, (1,))
        slot = dev.allocate(np.int32, 1)
        hbm("sum_2^26", 4 * n, dev.prepared("nk_sum", dev.handle, 0, srcs[0]._data.ptr, n, one._data.ptr))
        hbm("max_index_2^26", 4 * n, dev.prepared("nk_reduce_index", dev.handle, 1, 0, srcs[0]._data.ptr, n, slot.ptr))
        hbm("dot_2^26", 8 * n, dev.prepared("nk_dot", dev.handle, 0, srcs[0]._data.ptr, srcs[1]._data.ptr, n, one._data.ptr))
        dev.free(one); slot.release()
        # integer scalarization of 2^26 int32 elements
        i_src = Tensor.of(np.int32, (n,), rng.integers(-2**31, 2**31 - 1, n, dtype=np.int32)).to(dev)
        i_out = Tensor._on_device(dev, np.int32, (n,))
        hbm("scalarization_int32_multiply", 8 * n, dev.prepared_launch("scalarization_int", "multiply", -1, i_out, i_src, 3))
        hbm("scalarization_int32_divide", 8 * n, dev.prepared_launch("scalarization_int", "divide", -1, i_out, i_src, 7))
        dev.free(i_src); dev.free(i_out)
        # permuted [4096,16384] views of row-major [16384,4096]
        pv = []
        for t in srcs:
            v = Tensor(f32, NDConfiguration.ofShape((16384, 4096)).newReshaped((1, 0)), None)
            v._set_data(t._data, dev)
            pv.append(v)
        o2 = Tensor(f32, NDConfiguration.ofShape((4096, 16384)), None); o2._set_data(o._data, dev)
        hbm("chain_fused_permuted", 16 * n, dev.prepared_launch("fused", fused.program, fused.consts, o2, pv))
        # slice [::2, 1:8193] of [8192,16384] (the three 2^26 buffers are too small: use 2^27-element parents)
        for t in srcs + [tmp]: dev.free(t)
        parents = [Tensor.of(f32, (8192, 16384), rng.standard_normal(8192 * 16384).astype(f32)).to(dev) for _ in range(3)]
        sv = [p[::2, 1:8193] for p in parents]
        o3 = Tensor(f32, NDConfiguration.ofShape((4096, 8192)), None); o3._set_data(o._data, dev)
        hbm("chain_fused_sliced", 16 * (1 << 25), dev.prepared_launch("fused", fused.program, fused.consts, o3, sv))
        for p in parents: dev.free(p)
        dev.free(o)

        # C4 matmul
        # (4000^3: a large shape that is no whole number of tiles)
        for name, (M, K, N) in (("matmul_4096", (4096, 4096, 4096)), ("matmul_tall_skinny", (65536, 256, 256)), ("matmul_4000", (4000, 4000, 4000)),
                                ("matmul_3072", (3072, 3072, 3072)),           # 576 tiles of 128 x 128: a round of the machine and an eighth
                                ("matmul_2560", (2560, 2560, 2560)),           # 400 tiles: the last round of large tiles would idle most units
                                ("matmul_2048", (2048, 2048, 2048)), ("matmul_1536", (1536, 1536, 1536)),   # a round of tiles, and less
                                ("matmul_1024", (1024, 1024, 1024)),
                                ("matmul_narrow_result", (4096, 4096, 64)),    # few tiles, a long k range
                                ("matmul_short_k", (3000, 64, 3000))):          # two k-slices, no whole tiles
            A = Tensor.of(f32, (M, K), rng.uniform(-1, 1, M * K).astype(f32)).to(dev)
            B = Tensor.of(f32, (K, N), rng.uniform(-1, 1, K * N).astype(f32)).to(dev)
            Cm = Tensor._on_device(dev, f32, (M, N))
            # what the registered implementation launches: C = A @ B (nk_matmul_set, as CLMatMul's kernel); the accumulating
            # entry point (C += A @ B, the old C read as well) beside it
            flops(name, 2.0 * M * K * N, 4 * (M * K + K * N + M * N), dev.prepared_launch("matmul_set", True, M, K, N, A, B, Cm))
            flops(name + "_accumulating", 2.0 * M * K * N, 4 * (M * K + K * N + 2 * M * N), dev.prepared_launch("matmul", True, M, K, N, A, B, Cm))
            for t in (A, B, Cm): dev.free(t)
        M = K = N = 4096
        A = Tensor.of(np.float64, (M, K), rng.uniform(-1, 1, M * K)).to(dev)
        B = Tensor.of(np.float64, (K, N), rng.uniform(-1, 1, K * N)).to(dev)
        Cm = Tensor._on_device(dev, np.float64, (M, N))
        flops("matmul_4096_f64", 2.0 * M * K * N, 8 * (M * K + K * N + M * N), dev.prepared_launch("matmul_set", True, M, K, N, A, B, Cm), f64=True)
        for t in (A, B, Cm): dev.free(t)
        # the products of a dense layer with a small batch: each streams its large operand once (memory-bound)
        for name, (M, K, N) in (("matmul_matrix_vector", (4096, 4096, 1)), ("matmul_batch_of_16_rows", (16, 4096, 4096)),
                                ("matmul_batch_of_32_rows", (32, 4096, 4096)), ("matmul_batch_of_4_rows", (4, 4096, 4096)),
                                ("matmul_16_outer_products", (4096, 16, 4096)), ("matmul_batch_of_16_columns", (4096, 4096, 16))):
            A = Tensor.of(f32, (M, K), rng.uniform(-1, 1, M * K).astype(f32)).to(dev)
            B = Tensor.of(f32, (K, N), rng.uniform(-1, 1, K * N).astype(f32)).to(dev)
            Cm = Tensor._on_device(dev, f32, (M, N))
            hbm(name, 4 * (M * K + K * N + M * N), dev.prepared_launch("matmul_set", True, M, K, N, A, B, Cm))
            for t in (A, B, Cm): dev.free(t)
        for name, (M, K, N) in (("matmul_3072_f64", (3072, 3072, 3072)), ("matmul_2048_f64", (2048, 2048, 2048)), ("matmul_1024_f64", (1024, 1024, 1024)),
                                ("matmul_narrow_result_f64", (4096, 4096, 64))):
            A = Tensor.of(np.float64, (M, K), rng.uniform(-1, 1, M * K)).to(dev)
            B = Tensor.of(np.float64, (K, N), rng.uniform(-1, 1, K * N)).to(dev)
            Cm = Tensor._on_device(dev, np.float64, (M, N))
            flops(name, 2.0 * M * K * N, 8 * (M * K + K * N + M * N), dev.prepared_launch("matmul_set", True, M, K, N, A, B, Cm), f64=True)
            for t in (A, B, Cm): dev.free(t)

        # C1 and C5 convolutions
        x1 = Tensor.of(f32, (64, 64), rng.uniform(-1, 1, 4096).astype(f32)).to(dev)
        k1 = Tensor.of(f32, (3, 3), rng.uniform(-1, 1, 9).astype(f32)).to(dev)
        y1 = Tensor._on_device(dev, f32, (62, 62))
        flops("conv2d_64x64_3x3", 69192, 31796, dev.prepared_launch("convolution", -1, y1, x1, k1),
              note="what this line times is the ctypes call of the benchmark, one every 7 us: the kernel itself takes 2.4 us in "
                   "the kernel trace, and a C client of the same entry point issues a launch every 2.7 us")
        # the same operation on an image large enough to fill the machine
        xl = Tensor.of(f32, (2048, 2048), rng.uniform(-1, 1, 2048 * 2048).astype(f32)).to(dev)
        kl = Tensor.of(f32, (5, 5), rng.uniform(-1, 1, 25).astype(f32)).to(dev)
        yl = Tensor._on_device(dev, f32, (2044, 2044))
        flops("conv2d_2048x2048_5x5", 2.0 * 2044 * 2044 * 25, 4 * (2048 * 2048 + 25 + 2044 * 2044), dev.prepared_launch("convolution", -1, yl, xl, kl),
              note="a parity decision, not a slow kernel: every tap is a rounded multiply followed by a rounded add, as "
                   "SimpleCPUConvolution computes it, so that the result has the reference's bits; 50 vector "
                   "instructions per output bound the kernel, a fused multiply-add would halve them and change the bits")
        for t in (xl, kl, yl): dev.free(t)
        # 3x3 taps on a 4096^2 image: 18 unfused vector operations per output instead of 50, so memory gets a say
        xl = Tensor.of(f32, (4096, 4096), rng.uniform(-1, 1, 4096 * 4096).astype(f32)).to(dev)
        kl = Tensor.of(f32, (3, 3), rng.uniform(-1, 1, 9).astype(f32)).to(dev)
        yl = Tensor._on_device(dev, f32, (4094, 4094))
        flops("conv2d_4096x4096_3x3", 2.0 * 4094 * 4094 * 9, 4 * (4096 * 4096 + 9 + 4094 * 4094), dev.prepared_launch("convolution", -1, yl, xl, kl))
        for t in (xl, kl, yl): dev.free(t)
        x5 = Tensor.of(f32, (64, 256, 256), (rng.standard_normal(64 * 256 * 256) * 0.1).astype(f32)).to(dev)
        k5 = Tensor.of(f32, (64, 5, 5), (rng.standard_normal(1600) * 0.1).astype(f32)).to(dev)
        y5 = Tensor._on_device(dev, f32, (1, 252, 252))
        e5 = Tensor.of(f32, (1, 252, 252), rng.standard_normal(252 * 252).astype(f32)).to(dev)
        dx5 = Tensor._on_device(dev, f32, (64, 256, 256))
        dk5 = Tensor._on_device(dev, f32, (64, 5, 5))
        flops("conv_c5_forward", 203212800, 17037632, dev.prepared_launch("convolution", -1, y5, x5, k5))
        flops("conv_c5_grad_input", 203212800, 17037632, dev.prepared_launch("convolution", 0, dx5, k5, e5))
        flops("conv_c5_grad_kernel", 203212800, 17037632, dev.prepared_launch("convolution", 0, dk5, x5, e5))
        for t in (x5, k5, y5, e5, dx5, dk5): dev.free(t)
        # the same shapes in f64: the channel kernels instantiated for double
        f64 = np.float64
        x5 = Tensor.of(f64, (64, 256, 256), rng.standard_normal(64 * 256 * 256) * 0.1).to(dev)
        k5 = Tensor.of(f64, (64, 5, 5), rng.standard_normal(1600) * 0.1).to(dev)
        y5 = Tensor._on_device(dev, f64, (1, 252, 252))
        e5 = Tensor.of(f64, (1, 252, 252), rng.standard_normal(252 * 252)).to(dev)
        dx5 = Tensor._on_device(dev, f64, (64, 256, 256))
        dk5 = Tensor._on_device(dev, f64, (64, 5, 5))
        flops("conv_c5_forward_f64", 203212800, 2 * 17037632, dev.prepared_launch("convolution", -1, y5, x5, k5), f64=True)
        flops("conv_c5_grad_input_f64", 203212800, 2 * 17037632, dev.prepared_launch("convolution", 0, dx5, k5, e5), f64=True)
        flops("conv_c5_grad_kernel_f64", 203212800, 2 * 17037632, dev.prepared_launch("convolution", 0, dk5, x5, e5), f64=True)

    # ---- whole operations through the backend, allocation, fill and host transfers ---------------------------------
    operations = memory = None
    if not args.no_ops:
        import ctypes
        operations = operation_figures(dev, rng, ctypes, _lib, Function, Tensor, max(50, min(args.steps, 100)))
        memory = memory_figures(dev, ctypes, _lib)

    # ---- the reference's CPU path beside the other configurations (oracle, bounded samples) -----------------------
    cpu_others = None
    if not args.no_cpu and not args.no_others:
        cpu_others = cpu_side_of_the_other_configs(min(HOST_CORE_SHARE, len(os.sched_getaffinity(0))))

    result = {
        "metric": "GB/s & % HBM peak (broadcast/elementwise)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "broadcast add + multiply, f32 [1024,1,512] o [1,2048,512] -> [1024,2048,512], "
                               "one step = one add launch + one multiply launch, 4 301 258 752 algorithmic bytes each",
                   "device": dev.name(), "compute_units": dev.maxComputeUnits(),
                   "clock_settle": f"{SETTLE_MS:.0f} ms of the same steps, untimed, before the warm-up steps"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "cpu_others": cpu_others,
        "others": others,
        "operations": operations,
        "memory": memory,
        "alloc_ms": None if memory is None else round(memory["alloc_free_4GiB_from_pool_us"] * 1e-3, 6),
        "zero_fill_ms": None if memory is None else memory["zero_fill_4GiB_ms"],
    }
    if args.yardstick:
        import subprocess
        dev.sync()
        child = subprocess.run([sys.executable, os.path.abspath(__file__), "--yardstick-only"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        lines = [ln for ln in child.stdout.splitlines() if ln.startswith("{")]
        result["yardstick"] = json.loads(lines[-1]) if child.returncode == 0 and lines else {"error": child.stderr[-400:]}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
