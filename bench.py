#!/usr/bin/env python3
"""Benchmark of the HIPBackend hot path on one MI355X.

Headline (the one JSON line's `value`): fp16 GEMM, M = N = K = 4096, fp32 accumulate, all four
transA/transB layouts (NN, NT, TN, TT) per step, inputs N(0,1)/sqrt(K) from fixed seeds and
resident in HBM before the timed region. FLOPs = 2*M*N*K per GEMM, the formula of the
reference's HCMatrixBench (Sources/HCMatrixBench/Entrypoint.swift:25).

Also reported in the same line:
  roofline      the slowest layout's GEMM kernel: algorithmic FLOPs / average launch duration
                from HIP events recorded on the backend's own stream inside the timed region
  cpu_baseline  the reference CPUBackend algorithm (oracle/cpu_ref.c restatement, the literal
                single-thread triple loop) timed on this box's host cores on a bounded row slab;
                extra.cpu_reference_path holds the same for configs 1, 3, 4 and 5 (sgemm through OpenBLAS
                with its thread count, the bandwidth-bound ops on one thread)
  extra         the other benchmark configurations: fp32 1024^3, the ragged fp16 sweep, attention-shaped
                batched GEMMs, the bandwidth-bound ops at [8192,4096] with GB/s against the 8 TB/s
                HBM peak (short kernels are timed as graph-replayed batches: device-side duration
                per launch), and the transformer forward pass, eager and as one graph replay

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra] [--no-graph]
                       [--only headline,cfg1,cfg2,cfg3,cfg4,cfg5]
`--only` restricts the run to the named parts (without `headline` the line's `value` is null): what
the per-config rocprofv3 summaries under profiles/ are made with, so that a kernel's launches of
one config are not pooled with another's.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_F16_TFLOPS = 2516.6  # MI355X dense fp16 MFMA
PEAK_F32_TFLOPS = 157.3   # MI355X fp32 MFMA
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E
# HBM bytes per 4096^3 fp16 GEMM launch, from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs of
# this benchmark scaled by a plain copy kernel (not measurable live; the runs that produced it are
# summarised in profiles/gemm_f16_4096_and_cfg4_hbm_traffic_fetch_write_size.md): 196800 KiB read +
# 32768 KiB written.
GEMM_TRAFFIC_BYTES = (196800 + 32768) * 1024
GEMM_TRAFFIC_SOURCE = "constant from profiles/gemm_f16_4096_and_cfg4_hbm_traffic_fetch_write_size.md (rocprofv3 --pmc runs), not measured in this run"


class MfmaProbe:
    """The MFMA-only measurement kernels of bench_probe.hip: bench.py's own code object, loaded
    through the library's raw module entry points (hc_module_load / hc_launch)."""

    class Args(ctypes.Structure):
        _fields_ = [("data", ctypes.c_void_p), ("out", ctypes.c_void_p), ("iters", ctypes.c_uint32),
                    ("chunks", ctypes.c_uint32)]

    def __init__(self, backend):
        self.b, self.lib = backend, backend._lib
        path = os.path.join(ROOT, "bench_probe.hsaco")
        if not os.path.exists(path):
            import subprocess
            subprocess.run(["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "--genco", "-O3", "-std=c++17",
                            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                            "-o", path, os.path.join(ROOT, "bench_probe.hip")], check=True)
        image = open(path, "rb").read()
        self.image = ctypes.create_string_buffer(image, len(image))
        self.module = ctypes.c_void_p()
        backend._check(self.lib.hc_module_load(backend._ctx, self.image, len(image), ctypes.byref(self.module)))
        self.fn = {}
        for shape, name in ((0, b"hc_probe_mfma_f16_32x32x16"), (1, b"hc_probe_mfma_f16_16x16x32")):
            fn = ctypes.c_void_p()
            backend._check(self.lib.hc_module_get_function(self.module, name, ctypes.byref(fn)))
            self.fn[shape] = fn
        marker = ctypes.c_void_p()
        backend._check(self.lib.hc_module_get_function(self.module, b"hc_bench_marker", ctypes.byref(marker)))
        self.marker = marker
        self.cus = backend.deviceInfo()["compute_units"]
        self.out = backend.allocate(self.cus * 256 * 4)

    def launch(self, data, shape, iters=1024):
        """One launch (a workgroup of four waves per compute unit: the occupancy of the large GEMM
        tile); returns its floating-point operations."""
        args = MfmaProbe.Args(data.ptr, self.out.ptr, iters, min(data.byteCount // 16, 0xffffffff))
        grid, block = (ctypes.c_uint32 * 3)(self.cus, 1, 1), (ctypes.c_uint32 * 3)(256, 1, 1)
        self.b._check(self.lib.hc_launch(self.b._ctx, self.fn[shape], grid, block, 0, ctypes.byref(args),
                                         ctypes.sizeof(args)))
        # per iteration and wave: 16 MFMAs of 32 x 32 x 16 (or 32 of 16 x 16 x 32)
        return 2.0 * 32 * 32 * 16 * 16.0 * iters * (self.cus * 256 / 64)

    def mark(self, region):
        """An empty kernel with a grid of `region` workgroups of 64 lanes: in a kernel trace of this
        run, the launches between two markers of the same size are that region's."""
        args = MfmaProbe.Args(None, None, 0, 0)
        grid, block = (ctypes.c_uint32 * 3)(region, 1, 1), (ctypes.c_uint32 * 3)(64, 1, 1)
        self.b._check(self.lib.hc_launch(self.b._ctx, self.marker, grid, block, 0, ctypes.byref(args),
                                         ctypes.sizeof(args)))

    def close(self):
        self.lib.hc_module_unload(self.b._ctx, self.module)


# Regions of a run, by marker size (see MfmaProbe.mark); written into the result as `trace_regions`.
REGIONS = {}
_PROBE = [None]


def mark(backend, name):
    """Launches the marker of the region called `name` (a number is assigned at first use)."""
    if _PROBE[0] is None:
        _PROBE[0] = MfmaProbe(backend)
    region = REGIONS.setdefault(name, len(REGIONS) + 1)
    _PROBE[0].mark(region)


class Events:
    """HIP events on the backend's stream (hc_event_*), for per-launch durations."""

    def __init__(self, backend):
        self.b = backend
        self.lib = backend._lib

    def new(self):
        ev = ctypes.c_void_p()
        self.b._check(self.lib.hc_event_create(self.b._ctx, ctypes.byref(ev)))
        return ev

    def record(self, ev):
        self.b._check(self.lib.hc_event_record(self.b._ctx, ev))

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        self.b._check(self.lib.hc_event_elapsed_ms(a, b, ctypes.byref(ms)))
        return ms.value

    def free(self, ev):
        self.lib.hc_event_destroy(ev)


GRAPH_TIMING = True
SPINUP_MS = 200.0  # untimed load before the warmup steps, see headline()
BATCH_SPINUP_MS = 60.0  # the same for the graph-replayed batches of short kernels


def timed_launches(backend, events, fn, iters, warmup, batched=False, region=None, fusion=False):
    """Average duration (ms) of fn() launches, each bracketed by events on the stream.
    batched=True (short kernels): the host cannot enqueue a microsecond-scale kernel as fast as
    the GPU runs it, so per-launch events would time the host. Instead `iters` launches are
    recorded once into a graph and the replay is bracketed by two events: device-side duration
    per launch, launch gaps included."""
    for _ in range(warmup):
        fn()
    if batched and GRAPH_TIMING:
        # (recorded as issued: the rewrite of a recording would merge the batch's independent launches,
        # e.g. products over the same input into one launch, and the figure would no longer be that of
        # the kernel a single call runs)
        # (every launch of the batch keeps its own output buffer, so that no launch writes into lines
        # the launch before it left in the caches)
        # (fusion=True: a chain of calls that a recording is meant to merge, measured as recorded)
        with backend.switches(**({} if fusion else {"HCHIP_NO_FUSION": "1"})):
            with backend.capture() as cap:
                keep = [fn() for _ in range(iters)]
        # the board's clocks settle only after some tens of milliseconds under load (see headline()):
        # replay untimed for a while first, so that a batch of microsecond kernels is measured at
        # the sustained clocks as well
        t_spin = time.perf_counter()
        while (time.perf_counter() - t_spin) * 1e3 < BATCH_SPINUP_MS:
            for _ in range(10):
                cap.graph.launch()
            backend.sync()
        ms = []
        if region:
            mark(backend, region)
        for _ in range(5):
            a, b = events.new(), events.new()
            events.record(a)
            cap.graph.launch()
            events.record(b)
            backend.sync()
            ms.append(events.elapsed_ms(a, b) / iters)
            events.free(a)
            events.free(b)
        if region:
            mark(backend, region)
        cap.graph.destroy()
        del keep
        return float(np.mean(ms)), float(np.median(ms))
    pairs = []
    if region:
        mark(backend, region)
    for _ in range(iters):
        a, b = events.new(), events.new()
        events.record(a)
        fn()
        events.record(b)
        pairs.append((a, b))
    if region:
        mark(backend, region)
    backend.sync()
    ms = [events.elapsed_ms(a, b) for a, b in pairs]
    for a, b in pairs:
        events.free(a)
        events.free(b)
    return float(np.mean(ms)), float(np.median(ms))


def headline(backend, steps, warmup):
    from honeycrisp_amd.descriptors import DType
    n = 4096
    a = (np.random.default_rng(2).standard_normal((n, n)) / np.sqrt(n)).astype(np.float16)
    b = (np.random.default_rng(3).standard_normal((n, n)) / np.sqrt(n)).astype(np.float16)
    # operands stored pre-transposed so that all four layouts compute the same product
    dev = {
        ("a", False): backend.upload(a), ("a", True): backend.upload(np.ascontiguousarray(a.T)),
        ("b", False): backend.upload(b), ("b", True): backend.upload(np.ascontiguousarray(b.T)),
    }
    layouts = [("NN", False, False), ("NT", False, True), ("TN", True, False), ("TT", True, True)]
    events = Events(backend)

    def gemm(ta, tb):
        return backend.matmul(dev[("a", ta)], ta, dev[("b", tb)], tb, False, n, n, n, DType.float16)

    # The board needs some tens of milliseconds of load before its clocks settle (the first
    # ~50 ms run 10-15 % slower): an untimed spin-up of the same launches precedes the warmup
    # steps, so that a short timed region still measures the sustained rate.
    t_spin = time.perf_counter()
    while (time.perf_counter() - t_spin) * 1e3 < SPINUP_MS:
        for _ in range(10):
            for _, ta, tb in layouts:
                gemm(ta, tb)
        backend.sync()
    for _ in range(warmup):
        for _, ta, tb in layouts:
            gemm(ta, tb)
    backend.sync()
    # Timed region: exactly `steps` steps of four launches, one event per step on the backend's
    # stream (an event after every launch would cost the job 3 %). The average launch duration
    # over the timed region is a step's event-to-event time / 4, gaps between launches included.
    marks = [events.new() for _ in range(steps + 1)]
    mark(backend, "headline_timed_steps")
    backend.sync()
    t0 = time.perf_counter()
    events.record(marks[0])
    for i in range(steps):
        for _, ta, tb in layouts:
            gemm(ta, tb)
        events.record(marks[i + 1])
    backend.sync()
    t1 = time.perf_counter()
    mark(backend, "headline_timed_steps")
    flops = 2.0 * n * n * n
    step_ms = [events.elapsed_ms(marks[i], marks[i + 1]) for i in range(steps)]
    launch_ms = float(np.mean(step_ms)) / 4
    for m in marks:
        events.free(m)
    ms_per_step = (t1 - t0) * 1e3 / steps
    value = 4 * flops / (ms_per_step * 1e-3) / 1e12
    # Per-layout breakdown: a second, untimed pass with one event between consecutive launches.
    per_layout = {name: [] for name, _, _ in layouts}
    reps = min(steps, 50)
    marks = [events.new() for _ in range(4 * reps + 1)]
    events.record(marks[0])
    i = 0
    for _ in range(reps):
        for name, ta, tb in layouts:
            gemm(ta, tb)
            i += 1
            events.record(marks[i])
            per_layout[name].append(i)
    backend.sync()
    layout_ms = {}
    for name, ends in per_layout.items():
        layout_ms[name] = float(np.mean([events.elapsed_ms(marks[j - 1], marks[j]) for j in ends]))
    for m in marks:
        events.free(m)
    achieved = flops / (launch_ms * 1e-3) / 1e12
    roofline = {
        "bound": "mfma", "kernel": "fp16 GEMM 4096^3 (hc_gemm_f16_mi16_256x256_*), mean over the timed region's launches",
        "achieved": round(achieved, 2),
        "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s", "frac": round(achieved / PEAK_F16_TFLOPS, 4),
        "traffic": GEMM_TRAFFIC_BYTES, "traffic_source": GEMM_TRAFFIC_SOURCE, "launch_ms": round(launch_ms, 5),
        "step_ms_min_median_max": [round(float(np.min(step_ms)), 4), round(float(np.median(step_ms)), 4),
                                   round(float(np.max(step_ms)), 4)],
        "step_tflops_min_median_max": [round(4 * flops / (float(np.max(step_ms)) * 1e-3) / 1e12, 1),
                                       round(4 * flops / (float(np.median(step_ms)) * 1e-3) / 1e12, 1),
                                       round(4 * flops / (float(np.min(step_ms)) * 1e-3) / 1e12, 1)],
        "per_layout_tflops": {k: round(flops / (v * 1e-3) / 1e12, 2) for k, v in layout_ms.items()},
        "per_layout_ms": {k: round(v, 4) for k, v in layout_ms.items()},
        "per_layout_note": "separate untimed pass, one event per launch",
    }
    # What the matrix cores alone sustain on these bit patterns: the same MFMA sequence as the
    # GEMM's inner loop with no memory traffic at all. The board lowers the shader clock until
    # power fits, and MFMA power depends on how many operand bits toggle, so this, not the
    # 2.4 GHz figure, is the rate a GEMM on this data could approach.
    probe_in = dev[("a", False)]
    mark(backend, "headline_mfma_only")
    probe = _PROBE[0]
    probe_tflops = {}
    for shape, name in ((1, "16x16x32"), (0, "32x32x16")):
        for _ in range(200):
            probe_flops = probe.launch(probe_in, shape)
        e0, e1 = events.new(), events.new()
        events.record(e0)
        for _ in range(200):
            probe.launch(probe_in, shape)
        events.record(e1)
        backend.sync()
        probe_tflops[name] = 200 * probe_flops / (events.elapsed_ms(e0, e1) * 1e-3) / 1e12
        events.free(e0)
        events.free(e1)
    mark(backend, "headline_mfma_only")
    roofline["mfma_only_same_data"] = {
        "tflops": round(probe_tflops["16x16x32"], 1), "gemm_frac_of_it": round(achieved / probe_tflops["16x16x32"], 4),
        "tflops_32x32x16": round(probe_tflops["32x32x16"], 1),
        "note": "MFMA-only kernels on the GEMM's operand bits, clock as set by power management; the GEMM "
                "uses the 16x16x32 shape"}
    return value, ms_per_step, roofline, (a, b)


def cpu_baseline(a, b, budget_s=20.0):
    """The reference algorithm (single worker thread, scalar i/j/k loop with fp32 accumulate,
    whole-buffer fp16 -> fp32 staging) on a row slab of the same four 4096^3 products."""
    from oracle.oracle_backend import load
    lib = load()
    n = a.shape[0]
    srcs = {False: (a, b), True: (np.ascontiguousarray(a.T), np.ascontiguousarray(b.T))}
    out = np.empty((64, n), dtype=np.float32)

    def run(ta, tb, rows):
        sa, sb = srcs[ta][0], srcs[tb][1]
        t0 = time.perf_counter()
        lib.ref_matmul_rows(2, sa.ctypes.data, int(ta), sb.ctypes.data, int(tb), n, n, n, 0, rows, out.ctypes.data)
        return time.perf_counter() - t0

    probe = run(False, False, 2)            # includes the whole-buffer conversions
    probe8 = run(False, False, 10)
    per_row = max((probe8 - probe) / 8.0, 1e-4)
    rows = int(max(2, min(64, (budget_s / 4.0 - probe) / per_row)))
    total_t, total_flops = 0.0, 0.0
    for ta in (False, True):
        for tb in (False, True):
            total_t += run(ta, tb, rows)
            total_flops += 2.0 * rows * n * n
    return {
        "value": round(total_flops / total_t / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
        "sample": "rows 0..%d of each of the four 4096^3 fp16 products (%.1f s of CPU work), literal "
                  "CPUBackend loop incl. whole-buffer fp16->fp32 staging" % (rows, total_t),
    }


def cpu_reference_ops(budget_s=25.0):
    """Configs 1 and 4 on the host cores the way the reference CPUBackend would run them on Linux:
    the fp32 NN product through cblas_sgemm (the stand-in for vDSP_mmul, BackendCPU.swift:1256;
    here numpy's bundled OpenBLAS, all the threads it takes) and through the literal loop, and the
    bandwidth-bound ops through the CPUBackend restatement on ONE thread (the reference serialises
    its CPU work on one worker thread, BackendCPU.swift:226,235-248). Full-size inputs; an op is
    skipped once the budget is spent."""
    from oracle.oracle_backend import OracleBackend
    from honeycrisp_amd.descriptors import (BroadcastData, BroadcastStrides, DType, ElemwiseOp, NumericBinaryOp,
                                            ReduceDims, ReduceOp, ScatterGatherIndices)
    F32 = DType.float32
    out = {}
    spent = [0.0]

    def timed(name, fn, flops=None, nbytes=None, cores=1, reps=1):
        if spent[0] > budget_s:
            return
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        dt = (time.perf_counter() - t0) / reps
        spent[0] += dt * reps
        r = {"ms": round(dt * 1e3, 2), "cores": cores}
        if flops is not None:
            r["tflops"] = round(flops / dt / 1e12, 5)
        if nbytes is not None:
            r["gbs"] = round(nbytes / dt / 1e9, 3)
        out[name] = r

    rng = np.random.default_rng(1)
    a = rng.standard_normal((1024, 1024)).astype(np.float32)
    b = rng.standard_normal((1024, 1024)).astype(np.float32)
    try:
        import threadpoolctl
        blas_threads = max([i.get("num_threads", 1) for i in threadpoolctl.threadpool_info()
                            if i.get("user_api") == "blas"] or [1])
    except Exception:
        blas_threads = os.cpu_count() or 1
    a @ b
    timed("cfg1_f32_gemm_1024_openblas_sgemm", lambda: a @ b, flops=2.0 * 1024**3, cores=blas_threads, reps=10)
    # The same product the way the reference issues it: vDSP_mmul (BackendCPU.swift:1256) through the
    # Linux stand-in for Accelerate, which forwards to the cblas_sgemm of an OpenBLAS found at run
    # time (here the one bundled with scipy / numpy, if any; else its built-in loop).
    shim_path = os.path.join(ROOT, "swift", "honeycrisp-linux", "Sources", "Accelerate", "libAccelerateShim.so")
    if os.path.exists(shim_path):
        import glob
        libs = []
        for mod in ("scipy", "numpy"):
            try:
                m = __import__(mod)
                libs += sorted(glob.glob(os.path.join(os.path.dirname(os.path.dirname(m.__file__)), mod + ".libs",
                                                      "libscipy_openblas*.so")))
            except ImportError:
                pass
        if libs and not os.environ.get("HC_ACCELERATE_BLAS"):
            os.environ["HC_ACCELERATE_BLAS"] = libs[0]
        shim = ctypes.CDLL(shim_path)
        shim.hc_accelerate_blas_backend.restype = ctypes.c_char_p
        fptr = ctypes.POINTER(ctypes.c_float)
        shim.vDSP_mmul.argtypes = [fptr, ctypes.c_long, fptr, ctypes.c_long, fptr, ctypes.c_long, ctypes.c_ulong,
                                   ctypes.c_ulong, ctypes.c_ulong]
        c = np.empty((1024, 1024), np.float32)
        mmul = lambda: shim.vDSP_mmul(a.ctypes.data_as(fptr), 1, b.ctypes.data_as(fptr), 1, c.ctypes.data_as(fptr), 1,
                                      1024, 1024, 1024)
        mmul()
        threads = shim.hc_accelerate_blas_threads()
        timed("cfg1_f32_gemm_1024_vdsp_mmul_shim", mmul, flops=2.0 * 1024**3, cores=threads or blas_threads, reps=10)
        if "cfg1_f32_gemm_1024_vdsp_mmul_shim" in out:
            out["cfg1_f32_gemm_1024_vdsp_mmul_shim"]["blas"] = os.path.basename(shim.hc_accelerate_blas_backend().decode())
            assert np.allclose(c, a @ b, rtol=1e-3, atol=1e-2)
    ob = OracleBackend(threads=1)
    da, db = ob.upload(a), ob.upload(b)
    timed("cfg1_f32_gemm_1024_literal_loop", lambda: ob.matmul(da, False, db, False, False, 1024, 1024, 1024, F32),
          flops=2.0 * 1024**3)

    R, C = 8192, 4096
    x = ob.upload(np.random.default_rng(7).standard_normal((R, C)).astype(np.float32))
    bias = ob.upload(np.random.default_rng(8).standard_normal((1, C)).astype(np.float32))
    xs, bs = BroadcastStrides([R, C], [C, 1]), BroadcastStrides([R, C], [0, 1])
    nb = R * C * 4
    dims = ReduceDims(R, C, 1)
    timed("cfg4_bias_add", lambda: ob.binaryOp(BroadcastData(xs, x), BroadcastData(bs, bias), NumericBinaryOp.add, F32),
          nbytes=2 * nb + C * 4)
    timed("cfg4_gelu", lambda: ob.elemwise(x, ElemwiseOp.geluApprox, None, R * C, F32), nbytes=2 * nb)
    timed("cfg4_sum_axis1", lambda: ob.reduce(x, ReduceOp.sum, dims, F32), nbytes=nb + R * 4)
    timed("cfg4_argmax_axis1", lambda: ob.reduce(x, ReduceOp.argmax, dims, F32), nbytes=nb + R * 8)
    table = ob.upload(np.random.default_rng(10).standard_normal((32000, 1024)).astype(np.float32))
    ids = ob.upload(np.random.default_rng(9).integers(0, 32000, size=(65536,)))
    emb = ScatterGatherIndices([32000, 1024], 0, BroadcastData(BroadcastStrides([65536, 1024], [1, 0]), ids))
    timed("cfg4_embedding_gather", lambda: ob.gather(table, emb, F32), nbytes=65536 * 8 + 2 * 65536 * 1024 * 4)
    # config 3 on 4 of its 32 heads (the per-head cost does not depend on the head), fp16 through the
    # CPUBackend's whole-buffer conversions: q k^T, the scale, x v
    F16 = DType.float16
    heads = 4
    rng3 = np.random.default_rng(3)
    q, k_, v = (ob.upload(rng3.standard_normal((heads, 512, 64)).astype(np.float16)) for _ in range(3))
    scores = ob.batchedMatmul(heads, q, False, k_, True, False, 512, 64, 512, F16)
    timed("cfg3_qk_t_4_of_32_heads", lambda: ob.batchedMatmul(heads, q, False, k_, True, False, 512, 64, 512, F16),
          flops=2.0 * heads * 512 * 512 * 64)
    timed("cfg3_scale_4_of_32_heads", lambda: ob.binaryOp(scores, 0.125, NumericBinaryOp.mul, F16, count=heads * 512 * 512),
          nbytes=2 * heads * 512 * 512 * 2)
    timed("cfg3_pv_4_of_32_heads", lambda: ob.batchedMatmul(heads, scores, False, v, False, False, 512, 512, 64, F16),
          flops=2.0 * heads * 512 * 512 * 64)
    # config 5 on one of its 8 sequences (256 tokens, 12.6 GFLOP), fp32: the whole forward pass of the
    # front-end mirror over the CPUBackend restatement
    if spent[0] <= budget_s:
        from honeycrisp_amd.nn import Transformer
        from honeycrisp_amd.tensor import Tensor
        with ob.use():
            model = Transformer(dtype=F32)
            ids5 = Tensor(data=np.random.default_rng(5).integers(0, 8192, size=(1, 256)))
            timed("cfg5_transformer_fwd_f32_1_of_8_sequences", lambda: model(ids5).numpy())
        r = out.get("cfg5_transformer_fwd_f32_1_of_8_sequences")
        if r:
            r["tokens_per_s"] = round(256 / (r["ms"] * 1e-3), 1)
            r["tflops"] = round(100.9e9 / 8 / (r["ms"] * 1e-3) / 1e12, 5)
    out["note"] = ("host cores of this box; the fp32 product through numpy's bundled OpenBLAS and through vDSP_mmul of "
                   "the Linux Accelerate stand-in (which forwards to the cblas_sgemm named in `blas`), everything else "
                   "the CPUBackend restatement on one thread; full-size inputs for configs 1 and 4, 4 of 32 heads for "
                   "config 3, one of 8 sequences for config 5")
    return out


def native_eager_transformer(dtype_name, batching=0, idle_after=0):
    """Runs `HCMatrixBench --transformer` and returns its figures, or None if the program is not built."""
    import subprocess
    binary = os.path.join(ROOT, "honeycrisp_amd", "cpp", "HCMatrixBench")
    if not os.path.exists(binary):
        return None
    proc = subprocess.run([binary, "--transformer", "--dtype", dtype_name, "--iters", "20", "--batching", str(batching),
                           "--idle-after", str(idle_after)],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    if proc.returncode != 0:
        return {"error": (proc.stdout + proc.stderr)[-300:]}
    r = dict(kv.split("=", 1) for kv in proc.stdout.strip().splitlines()[-1].split())
    return {"ms": round(float(r["us"]) / 1e3, 3), "tokens_per_s": round(float(r["tokens_per_s"]), 1),
            "tflops": round(100.9e9 / (float(r["us"]) * 1e-6) / 1e12, 2),
            "ms_back_to_back": round(float(r["us_back_to_back"]) / 1e3, 3),
            "tokens_per_s_back_to_back": round(float(r["tokens_per_s_back_to_back"]), 1),
            "host_enqueue_ms": round(float(r["host_enqueue_us"]) / 1e3, 3),
            **({"launches_listed": int(r["launches_listed"]), "launches_enqueued": int(r["launches_enqueued"])} if batching else {}),
            "note": ("the same calls with hc_set_batching(%d, %d): listed, rewritten and enqueued batch by batch; " % (batching, idle_after)
                     if batching else "eager, ") +
                    "one backend call per op from a C++ host (HCMatrixBench --transformer, child process); "
                    "back_to_back: passes issued without a wait in between"}


def extra_workloads(backend, graph=True, only=("cfg1", "cfg2", "cfg3", "cfg4", "cfg5")):
    """The other configs of BASELINE.json: per-op launch durations from HIP events."""
    from honeycrisp_amd.descriptors import (BroadcastData, BroadcastStrides, DType, ElemwiseOp, NumericBinaryOp,
                                            ReduceDims, ReduceOp, ScatterGatherIndices)
    ev = Events(backend)
    out = {}
    F32, F16, I64 = DType.float32, DType.float16, DType.int64

    def report(name, ms, flops=None, nbytes=None, peak_tflops=None):
        r = {"ms": round(ms, 4)}
        if flops is not None:
            r["tflops"] = round(flops / (ms * 1e-3) / 1e12, 3)
            if peak_tflops:
                r["mfma_frac"] = round(r["tflops"] / peak_tflops, 4)
        if nbytes is not None:
            r["gbs"] = round(nbytes / (ms * 1e-3) / 1e9, 1)
            r["hbm_frac"] = round(r["gbs"] / PEAK_HBM_GBS, 4)
        out[name] = r

    def cfg1():
        # config 1: fp32 1024^3 (two input sets alternate so the operands are not L2-resident twice in a row)
        rng = np.random.default_rng(1)
        sets = [(backend.upload(rng.standard_normal((1024, 1024)).astype(np.float32)),
                 backend.upload(rng.standard_normal((1024, 1024)).astype(np.float32))) for _ in range(2)]
        it = [0]

        def gemm32():
            x, y = sets[it[0] & 1]
            it[0] += 1
            return backend.matmul(x, False, y, False, False, 1024, 1024, 1024, F32)
        ms, _ = timed_launches(backend, ev, gemm32, 50, 10, batched=True, region="cfg1_f32_gemm_1024")
        report("cfg1_f32_gemm_1024", ms, flops=2.0 * 1024**3, peak_tflops=PEAK_F32_TFLOPS)

    def cfg2():
        # the metric's fp32 leg: fp32 4096^3, N(0,1)/sqrt(K) entries, NN and NT (B stored transposed)
        n = 4096
        a32 = backend.upload((np.random.default_rng(2).standard_normal((n, n)) / np.sqrt(n)).astype(np.float32))
        b32 = backend.upload((np.random.default_rng(3).standard_normal((n, n)) / np.sqrt(n)).astype(np.float32))
        for name, tb in (("NN", False), ("NT", True)):
            fn = lambda: backend.matmul(a32, False, b32, tb, False, n, n, n, F32)
            for _ in range(30):     # (the clocks settle under load, see headline())
                fn()
            ms, _ = timed_launches(backend, ev, fn, 30, 10, region="cfg2_f32_gemm_4096_" + name)
            report("cfg2_f32_gemm_4096_" + name, ms, flops=2.0 * n**3, peak_tflops=PEAK_F32_TFLOPS)
        del a32, b32
        # the ragged sweep: fp16 NN products with M, N, K in {127, 1000, 4097}; total FLOPs over
        # total time of the 27 shapes, and the three cubes on their own
        sizes = (127, 1000, 4097)
        total_flops, total_ms = 0.0, 0.0
        rng = np.random.default_rng(20)
        big = rng.standard_normal(4097 * 4097).astype(np.float16)
        for m in sizes:
            for kk in sizes:
                a_dev = backend.upload(big[:m * kk])
                for n in sizes:
                    b_dev = backend.upload(big[:kk * n])
                    fn = lambda: backend.matmul(a_dev, False, b_dev, False, False, m, kk, n, F16)
                    ms, _ = timed_launches(backend, ev, fn, 5, 2, batched=True, region="cfg2_ragged_sweep_27_shapes")
                    total_flops += 2.0 * m * kk * n
                    total_ms += ms
                    if m == kk == n:
                        report("cfg2_ragged_%d_cubed" % m, ms, flops=2.0 * m * kk * n)
        report("cfg2_ragged_sweep_27_shapes", total_ms, flops=total_flops)

    def cfg3():
        # config 3: attention-shaped batched GEMMs, fp16, batch 32 (two sets of inputs alternate, so that no
        # launch finds its operands in the caches because the launch before it used the same ones)
        sets = []
        for s0 in (4, 40):
            q, k, v = [backend.upload(np.random.default_rng(s0 + i).standard_normal((32, 512, 64)).astype(np.float16))
                       for i in range(3)]
            sets.append((q, k, v, backend.batchedMatmul(32, q, False, k, True, False, 512, 64, 512, F16)))
        it = [0]

        def pick():
            it[0] += 1
            return sets[it[0] & 1]

        def qk_t():
            q, k, _, _ = pick()
            return backend.batchedMatmul(32, q, False, k, True, False, 512, 64, 512, F16)

        def scale():
            return backend.binaryOp(pick()[3], 0.125, NumericBinaryOp.mul, F16, count=32 * 512 * 512)

        def pv():
            _, _, v, scores = pick()
            return backend.batchedMatmul(32, scores, False, v, False, False, 512, 512, 64, F16)
        ms, _ = timed_launches(backend, ev, qk_t, 50, 10, batched=True, region="cfg3_qk_t")
        report("cfg3_qk_t", ms, flops=32 * 2.0 * 512 * 64 * 512, nbytes=32 * (2 * 512 * 64 + 512 * 512) * 2)
        ms, _ = timed_launches(backend, ev, scale, 50, 10, batched=True, region="cfg3_scale")
        report("cfg3_scale", ms, nbytes=2 * 32 * 512 * 512 * 2)
        ms, _ = timed_launches(backend, ev, pv, 50, 10, batched=True, region="cfg3_pv")
        report("cfg3_pv", ms, flops=32 * 2.0 * 512 * 512 * 64, nbytes=32 * (2 * 512 * 64 + 512 * 512) * 2)

        # The whole chain q k^T -> * 1/8 -> softmax -> x v as a Honeycrisp program writes it (Softmax.swift:64-66:
        # logSoftmax, then exp): call by call (five launches), and as a recording merges it (one attention
        # kernel with the same bits). Algorithmic bytes of the chain: q, k, v in, the context out.
        from honeycrisp_amd.tensor import Tensor

        def chain():
            q, k, v, _ = pick()
            with backend.use():
                tq, tk, tv = (Tensor(dataHandle=d, shape=[32, 512, 64], dtype=F16) for d in (q, k, v))
                p = (Tensor.batchedMatmul(tq, False, tk, True, False) * 0.125).softmax()
                return Tensor.batchedMatmul(p, False, tv, False, False)
        chain_flops, chain_bytes = 2 * 32 * 2.0 * 512 * 64 * 512, 4 * 32 * 512 * 64 * 2
        ms, _ = timed_launches(backend, ev, chain, 20, 5, batched=True, region="cfg3_chain_five_launches")
        report("cfg3_chain_five_launches", ms, flops=chain_flops, nbytes=chain_bytes)
        ms, _ = timed_launches(backend, ev, chain, 20, 5, batched=True, region="cfg3_chain_recorded_one_kernel", fusion=True)
        report("cfg3_chain_recorded_one_kernel", ms, flops=chain_flops, nbytes=chain_bytes)

    def cfg4():
        # config 4: bandwidth-bound ops at [8192, 4096] fp32
        R, C = 8192, 4096
        x = backend.upload(np.random.default_rng(7).standard_normal((R, C)).astype(np.float32))
        bias = backend.upload(np.random.default_rng(8).standard_normal((1, C)).astype(np.float32))
        xs = BroadcastStrides([R, C], [C, 1])
        bs = BroadcastStrides([R, C], [0, 1])
        nb = R * C * 4
        ms, _ = timed_launches(backend, ev, lambda: backend.binaryOp(BroadcastData(xs, x), BroadcastData(bs, bias), NumericBinaryOp.add, F32), 50, 10, batched=True, region="cfg4_bias_add")
        report("cfg4_bias_add", ms, nbytes=2 * nb + C * 4)
        # plain copy of known size (identity broadcast): the calibration kernel for HBM byte counters
        ms, _ = timed_launches(backend, ev, lambda: backend.broadcast(BroadcastData(xs, x), F32), 50, 10, batched=True, region="copy_134MB_calibration")
        report("copy_134MB_calibration", ms, nbytes=2 * nb)
        ms, _ = timed_launches(backend, ev, lambda: backend.elemwise(x, ElemwiseOp.geluApprox, None, R * C, F32), 50, 10, batched=True, region="cfg4_gelu")
        report("cfg4_gelu", ms, nbytes=2 * nb)
        dims = ReduceDims(R, C, 1)
        ms, _ = timed_launches(backend, ev, lambda: backend.reduce(x, ReduceOp.sum, dims, F32), 50, 10, batched=True, region="cfg4_sum_axis1")
        report("cfg4_sum_axis1", ms, nbytes=nb + R * 4)
        ms, _ = timed_launches(backend, ev, lambda: backend.reduce(x, ReduceOp.argmax, dims, F32), 50, 10, batched=True, region="cfg4_argmax_axis1")
        report("cfg4_argmax_axis1", ms, nbytes=nb + R * 8)

        def max_axis1():  # Tensor.max(axis:) = argmax + gather (ReduceRepeat.swift:201-209)
            i = backend.reduce(x, ReduceOp.argmax, dims, F32)
            return backend.gather(x, ScatterGatherIndices([R, C], 1, BroadcastData(BroadcastStrides([R, 1], [1, 0]), i)), F32)
        ms, _ = timed_launches(backend, ev, max_axis1, 50, 10, batched=True, region="cfg4_max_axis1")
        report("cfg4_max_axis1", ms, nbytes=nb + R * 8 + R * 8 + R * 4 + R * 4)
        # ... and as a recording (or a batch) merges the pair: the row kernel that finds the index stores the element
        ms, _ = timed_launches(backend, ev, max_axis1, 50, 10, batched=True, region="cfg4_max_axis1_recorded_one_kernel", fusion=True)
        report("cfg4_max_axis1_recorded_one_kernel", ms, nbytes=nb + R * 4)
        table = backend.upload(np.random.default_rng(10).standard_normal((32000, 1024)).astype(np.float32))
        ids = backend.upload(np.random.default_rng(9).integers(0, 32000, size=(65536,)))
        emb = ScatterGatherIndices([32000, 1024], 0, BroadcastData(BroadcastStrides([65536, 1024], [1, 0]), ids))
        ms, _ = timed_launches(backend, ev, lambda: backend.gather(table, emb, F32), 50, 10, batched=True, region="cfg4_embedding_gather")
        report("cfg4_embedding_gather", ms, nbytes=65536 * 8 + 2 * 65536 * 1024 * 4)

    def cfg5():
        # config 5: decoder-only transformer forward, 8 x 256 tokens; tokens/s = 2048 / wall time of
        # a forward pass ending in wait() on the logits (host-side op dispatch included)
        from honeycrisp_amd.nn import Transformer
        from honeycrisp_amd.tensor import Tensor
        ids = np.random.default_rng(11).integers(0, 8192, size=(8, 256))
        with backend.use():
            for name, dtype in (("cfg5_transformer_fwd_f32", F32), ("cfg5_transformer_fwd_f16", F16)):
                model = Transformer(dtype=dtype)
                tokens = Tensor(data=ids)
                for _ in range(2):
                    model(tokens).wait()
                mark(backend, name + "_5_passes")
                t0 = time.perf_counter()
                for _ in range(5):
                    model(tokens).wait()
                dt = (time.perf_counter() - t0) / 5
                mark(backend, name + "_5_passes")
                out[name] = {"ms": round(dt * 1e3, 3), "tokens_per_s": round(2048 / dt, 1),
                             "tflops": round(100.9e9 / dt / 1e12, 2)}
                # The same pass issued eagerly from native host code (the C++ HCMatrixBench as a child process:
                # same backend calls in the same order through the C++ mirror of the Backend interface), i.e.
                # what a compiled host program pays per call instead of the Python mirror's interpreter time.
                native = native_eager_transformer("f32" if dtype is F32 else "f16")
                if native:
                    out[name + "_native_host"] = native
                    # ... and with the library's batching on: still one call per op and no recording in
                    # the program, the launches listed and rewritten in batches of up to 256 (earlier when
                    # the device has run dry and 16 are listed)
                    out[name + "_native_host_batched"] = native_eager_transformer("f32" if dtype is F32 else "f16", 256, 16)
                if not graph:
                    continue
                # the same forward pass recorded once and replayed as one graph launch: as recorded
                # (one launch per backend call), and with the recording's rewrite, which merges
                # bias / GELU / residual into the products, LayerNorm and softmax chains into one
                # kernel each, the head swaps into the batched products and q, k, v into one launch
                for suffix, env in (("_graph_unmerged", "1"), ("_graph", None)):
                    with backend.switches(**({"HCHIP_NO_FUSION": env} if env else {})):
                        with backend.capture() as cap:
                            logits = model(tokens)
                    for _ in range(5):
                        cap.graph.launch()
                    logits.wait()
                    mark(backend, name + suffix + "_20_passes")
                    t0 = time.perf_counter()
                    for _ in range(20):
                        cap.graph.launch()
                        logits.wait()
                    dt = (time.perf_counter() - t0) / 20
                    mark(backend, name + suffix + "_20_passes")
                    out[name + suffix] = {"ms": round(dt * 1e3, 3), "tokens_per_s": round(2048 / dt, 1),
                                          "tflops": round(100.9e9 / dt / 1e12, 2), "launches": cap.graph.node_count()}
                    cap.graph.destroy()

    for name, fn in (("cfg1", cfg1), ("cfg2", cfg2), ("cfg3", cfg3), ("cfg4", cfg4), ("cfg5", cfg5)):
        if name in only:
            fn()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the other benchmark configurations")
    ap.add_argument("--only", default="", help="comma-separated parts to run: headline,cfg1,...,cfg5 (default: all)")
    ap.add_argument("--no-graph", action="store_true",
                    help="skip the graph-replay variant of the transformer (rocprofv3's tracer crashes "
                         "inside hipGraphLaunch on this ROCm)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the hot path on ONE GPU only (no collectives, no sharding); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    global GRAPH_TIMING
    GRAPH_TIMING = not args.no_graph
    from honeycrisp_amd.backend import HIPBackend
    backend = HIPBackend(0)
    info = backend.deviceInfo()
    _PROBE[0] = MfmaProbe(backend)
    parts = [x for x in args.only.split(",") if x] or ["headline", "cfg1", "cfg2", "cfg3", "cfg4", "cfg5"]
    unknown = [x for x in parts if x not in ("headline", "cfg1", "cfg2", "cfg3", "cfg4", "cfg5")]
    if unknown:
        ap.error("--only: unknown part(s) %s" % ",".join(unknown))
    if "headline" in parts:
        value, ms_per_step, roofline, (a, b) = headline(backend, args.steps, args.warmup)
    else:      # a profiling run restricted to other configs: no headline launches in its trace
        value, ms_per_step, roofline, a, b = None, None, None, None, None
        args.no_cpu = True
    result = {
        "metric": "matmul TFLOP/s (fp16 in, fp32 accumulate, 4096^3, mean over NN/NT/TN/TT)",
        "value": None if value is None else round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None if value is None else round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "configs[1]: fp16 GEMM M=N=K=4096, four transA/transB layouts per step, "
                               "entries N(0,1)/sqrt(K), seeds 2/3",
                   "device": info["name"], "arch": info["arch"], "compute_units": info["compute_units"],
                   "clock_mhz": info["clock_mhz"], "untimed_spinup_ms": SPINUP_MS},
        "frac_of_peak": None if value is None else round(value / PEAK_F16_TFLOPS, 4),
        "roofline": roofline,
    }
    if args.only:
        result["only"] = parts
    if not args.no_extra:
        result["extra"] = extra_workloads(backend, graph=not args.no_graph,
                                          only=[x for x in parts if x != "headline"])
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(a, b)
        if not args.no_extra and "cfg1" in parts and "cfg4" in parts:
            result["extra"]["cpu_reference_path"] = cpu_reference_ops()
    else:
        result["cpu_baseline"] = None
    result["trace_regions"] = {"kernel": "hc_bench_marker", "workgroups_of_marker": dict(REGIONS),
                               "note": "in a kernel trace of this run, a region's launches lie between two launches "
                                       "of the marker kernel with that many workgroups"}
    backend.sync()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
