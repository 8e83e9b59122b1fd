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
