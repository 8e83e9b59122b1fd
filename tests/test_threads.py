"""Backend methods are called concurrently from arbitrary threads (one task per tensor op,
Tensor.swift:641-656); the C ABI serialises allocator and launches behind one mutex and orders
everything on one stream. Here several host threads drive independent chains of ops through the
same context at the same time (ctypes drops the interpreter lock during the calls); every thread
must see exactly what it gets when it runs alone."""
import threading

import numpy as np
import pytest

from honeycrisp_amd.descriptors import (BroadcastData, BroadcastStrides, DType, ElemwiseOp, NumericBinaryOp,
                                        ReduceDims, ReduceOp, ScatterGatherIndices)

pytestmark = pytest.mark.gpu

F32, F16, I64 = DType.float32, DType.float16, DType.int64


def chain(backend, seed):
    """upload -> ragged fp16 product (padded copies from the library's scratch pool) -> bias add ->
    GELU -> row argmax -> row gather -> fp32 product -> column sum; returns host copies."""
    rng = np.random.default_rng(seed)
    M, K, N = 130 + seed % 7, 263 + seed % 5, 129 + seed % 3
    a = backend.upload((rng.standard_normal((M, K)) / K ** 0.5).astype(np.float16))
    b = backend.upload(rng.standard_normal((K, N)).astype(np.float16))
    bias = backend.upload(rng.standard_normal(N).astype(np.float16))
    c = backend.matmul(a, False, b, False, False, M, K, N, F16)
    c = backend.binaryOp(BroadcastData(BroadcastStrides([M, N], [N, 1]), c),
                         BroadcastData(BroadcastStrides([M, N], [0, 1]), bias), NumericBinaryOp.add, F16)
    g = backend.elemwise(c, ElemwiseOp.geluApprox, None, M * N, F16)
    idx = backend.reduce(g, ReduceOp.argmax, ReduceDims(M, N, 1), F16)
    rows = backend.upload(rng.integers(0, M, size=64))
    picked = backend.gather(g, ScatterGatherIndices([M, N], 0, BroadcastData(BroadcastStrides([64, N], [1, 0]), rows)), F16)
    w = backend.upload(rng.standard_normal((N, 64)).astype(np.float32))
    p32 = backend.cast(picked, 64 * N, F16, F32)
    prod = backend.matmul(p32, False, w, False, False, 64, N, 64, F32)
    total = backend.reduce(prod, ReduceOp.sum, ReduceDims(1, 64, 64), F32)
    return [x.onCPU().copy() for x in (g, idx, picked, prod, total)]


def test_concurrent_op_chains_match_serial_runs(hip_backend):
    threads, rounds = 8, 12
    want = {s: chain(hip_backend, s) for s in range(threads * rounds)}
    failures = []

    def worker(t):
        try:
            for r in range(rounds):
                seed = t * rounds + r
                got = chain(hip_backend, seed)
                for i, (x, y) in enumerate(zip(got, want[seed])):
                    if not np.array_equal(x, y):
                        failures.append("thread %d seed %d: result %d differs from the serial run" % (t, seed, i))
                        return
        except Exception as e:  # surfaced below: an exception in a thread would otherwise be lost
            failures.append("thread %d: %r" % (t, e))

    pool = [threading.Thread(target=worker, args=(t,)) for t in range(threads)]
    for th in pool:
        th.start()
    for th in pool:
        th.join()
    assert not failures, failures[:5]


def test_a_switch_flipped_by_one_thread_while_others_launch(hip_backend):
    """hc_debug_set from one thread while others run products through the same context: a call
    works on the copy of the switches it took when it started, so every product is computed by one
    consistent choice of kernel (forced tile or the host's own pick, all of which agree within the
    fp16 tolerance and with the result the thread gets alone), and nothing crashes or deadlocks."""
    rng = np.random.default_rng(5)
    M, K, N = 512, 320, 384
    a = hip_backend.upload((rng.standard_normal((M, K)) / K ** 0.5).astype(np.float16))
    b = hip_backend.upload(rng.standard_normal((K, N)).astype(np.float16))
    want = hip_backend.matmul(a, False, b, False, False, M, K, N, F16).onCPU().view(np.float16).astype(np.float32)
    stop, failures = threading.Event(), []

    def flipper():
        values = ["64x64", "128x128", None, "general", "256x128", None]
        i = 0
        while not stop.is_set():
            hip_backend.debugSet("HCHIP_GEMM_TILE", values[i % len(values)])
            hip_backend.debugSet("HCHIP_GEMM_KERNEL", ["dma", None, "dma2"][i % 3])
            i += 1
        hip_backend.debugSet("HCHIP_GEMM_TILE", None)
        hip_backend.debugSet("HCHIP_GEMM_KERNEL", None)

    def worker(t):
        try:
            for _ in range(60):
                got = hip_backend.matmul(a, False, b, False, False, M, K, N, F16).onCPU().view(np.float16).astype(np.float32)
                if not np.allclose(got, want, rtol=1e-2, atol=1e-2):
                    failures.append("thread %d: a product differs beyond the fp16 tolerance" % t)
                    return
        except Exception as e:
            failures.append("thread %d: %r" % (t, e))

    flip = threading.Thread(target=flipper)
    pool = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    flip.start()
    for th in pool:
        th.start()
    for th in pool:
        th.join()
    stop.set()
    flip.join()
    assert not failures, failures[:5]
    with pytest.raises(Exception):
        hip_backend.debugSet("HCHIP_NO_SUCH_SWITCH", "1")


def test_concurrent_reductions_through_the_fixed_scratch_array(hip_backend):
    """hc_reduce_noalloc from several threads through one context: a split reduction is two launches
    that meet in the library's one scratch array, and a per-device lock keeps the two together, so
    each thread sees, bit for bit, what hc_reduce gives for its input."""
    from ctypes import c_void_p
    lib, ctx = hip_backend._lib, hip_backend._ctx
    shapes = [(1, 3000, 512), (1, 2048, 1024), (2, 70000, 1), (1, 1500, 256)]
    jobs = []
    for t, (outer, reduce, inner) in enumerate(shapes):
        rng = np.random.default_rng(100 + t)
        x = hip_backend.upload(rng.standard_normal((outer, reduce, inner)).astype(np.float32))
        want = hip_backend.allocate(outer * inner * 4)
        hip_backend._check(lib.hc_reduce(ctx, 0, int(F32), c_void_p(x.ptr), c_void_p(want.ptr), outer, reduce, inner))
        jobs.append((x, want.onCPU().copy(), outer, reduce, inner))
    failures = []

    def worker(t):
        x, want, outer, reduce, inner = jobs[t]
        try:
            for _ in range(40):
                out = hip_backend.allocate(outer * inner * 4)
                hip_backend._check(lib.hc_reduce_noalloc(ctx, 0, int(F32), c_void_p(x.ptr), c_void_p(out.ptr), outer, reduce, inner))
                if not np.array_equal(out.onCPU(), want):
                    failures.append("thread %d: result differs from hc_reduce" % t)
                    return
        except Exception as e:
            failures.append("thread %d: %r" % (t, e))

    pool = [threading.Thread(target=worker, args=(t,)) for t in range(len(jobs))]
    for th in pool:
        th.start()
    for th in pool:
        th.join()
    assert not failures, failures[:5]
