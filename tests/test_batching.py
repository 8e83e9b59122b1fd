"""Batching (hc_set_batching): ordinary call-by-call code whose launches the library lists and
enqueues batch by batch, each batch rewritten like a recording. The reference has no notion of a
recording (one backend call per op, Tensor.swift:634-657), so this is how a program written
against it gets the merged kernels. What must hold: every result has the bits of the unbatched
run wherever a batch happens to end; transfers and waits see what program order promises; a
block released inside a batch is not handed out again before the batch has been enqueued."""
import threading
from ctypes import c_void_p

import numpy as np
import pytest

from honeycrisp_amd.descriptors import BroadcastData, BroadcastStrides, DType, ElemwiseOp, NumericBinaryOp
from honeycrisp_amd.nn import Transformer
from honeycrisp_amd.tensor import Tensor
from test_threads import chain

pytestmark = pytest.mark.gpu

F32, F16 = DType.float32, DType.float16


def dense(n, m):
    return BroadcastStrides([n, m], [m, 1])


def layer(backend, x, w, bias, m, k, n):
    """x[m,k] w[k,n] + bias -> GELU, as three backend calls; intermediates released as a Tensor's would be."""
    c = backend.matmul(x, False, w, False, False, m, k, n, F16)
    d = backend.binaryOp(BroadcastData(dense(m, n), c), BroadcastData(BroadcastStrides([m, n], [0, 1]), bias),
                         NumericBinaryOp.add, F16)
    del c
    g = backend.elemwise(d, ElemwiseOp.geluApprox, None, m * n, F16)
    del d
    return g


@pytest.mark.parametrize("limit", [1, 2, 3, 5, 64])
def test_results_do_not_depend_on_where_a_batch_ends(hip_backend, limit):
    rng = np.random.default_rng(3)
    m, k, n = 256, 192, 320
    x = hip_backend.upload((rng.standard_normal((m, k)) / k ** 0.5).astype(np.float16))
    w = hip_backend.upload(rng.standard_normal((k, n)).astype(np.float16))
    w2 = hip_backend.upload((rng.standard_normal((n, k)) / n ** 0.5).astype(np.float16))
    bias, bias2 = (hip_backend.upload(rng.standard_normal(c).astype(np.float16)) for c in (n, k))

    def two_layers():
        h = layer(hip_backend, x, w, bias, m, k, n)
        return layer(hip_backend, h, w2, bias2, m, n, k).onCPU().copy()

    want = two_layers()
    listed, enqueued = hip_backend.batchingStats()
    with hip_backend.batching(limit):
        got = two_layers()
    listed, enqueued = (b - a for a, b in zip((listed, enqueued), hip_backend.batchingStats()))
    assert np.array_equal(got, want)
    assert listed == 6 and enqueued <= listed
    if limit == 1:
        assert enqueued == 6
    if limit == 64:     # a whole layer in one batch becomes one launch
        assert enqueued == 2


def test_an_upload_into_a_buffer_that_listed_launches_read_waits_for_them(hip_backend):
    rng = np.random.default_rng(4)
    n = 1 << 16
    first, second = (rng.standard_normal(n).astype(np.float32) for _ in range(2))
    x = hip_backend.upload(first)
    with hip_backend.batching():
        y = hip_backend.elemwise(x, ElemwiseOp.exp, None, n, F32)   # listed, reads x
        hip_backend._check(hip_backend._lib.hc_memcpy_h2d(hip_backend._ctx, c_void_p(x.ptr),
                                                          second.ctypes.data_as(c_void_p), second.nbytes))
        z = hip_backend.elemwise(x, ElemwiseOp.exp, None, n, F32)   # reads the new contents
        got_y, got_z = y.onCPU().view(np.float32).copy(), z.onCPU().view(np.float32).copy()
    want_y = hip_backend.elemwise(hip_backend.upload(first), ElemwiseOp.exp, None, n, F32).onCPU().view(np.float32)
    want_z = hip_backend.elemwise(hip_backend.upload(second), ElemwiseOp.exp, None, n, F32).onCPU().view(np.float32)
    assert np.array_equal(got_y, want_y) and np.array_equal(got_z, want_z)


def test_an_upload_into_a_fresh_buffer_overtakes_the_list(hip_backend):
    rng = np.random.default_rng(5)
    n = 4096
    x = hip_backend.upload(rng.standard_normal(n).astype(np.float32))
    with hip_backend.batching():
        before = hip_backend.batchingStats()
        y = hip_backend.elemwise(x, ElemwiseOp.exp, None, n, F32)
        c = hip_backend.upload(np.full(n, 2.0, np.float32))        # a constant in the middle of the block
        assert hip_backend.batchingStats() == before               # nothing was enqueued for it
        z = hip_backend.binaryOp(BroadcastData(dense(1, n), y), BroadcastData(dense(1, n), c), NumericBinaryOp.mul, F32)
        got = z.onCPU().view(np.float32).copy()
        assert hip_backend.batchingStats()[0] - before[0] == 2
    want = np.exp(x.onCPU().view(np.float32).astype(np.float64)) * 2
    np.testing.assert_allclose(got, want, rtol=1e-6)


def test_a_released_block_is_not_handed_out_again_inside_its_batch(hip_backend):
    n = 1 << 20
    want = hip_backend.elemwise(hip_backend.upload(np.ones(n, np.float32)), ElemwiseOp.exp, None, n, F32).onCPU().copy()
    with hip_backend.batching():
        a = hip_backend.upload(np.ones(n, np.float32))
        b = hip_backend.elemwise(a, ElemwiseOp.exp, None, n, F32)    # listed, reads a
        ptr = a.ptr
        del a                                                         # released while the launch is listed
        others = [hip_backend.allocate(n * 4) for _ in range(4)]
        assert ptr not in [o.ptr for o in others]
        for o in others:                                              # something writes them, so a reuse would show
            hip_backend._check(hip_backend._lib.hc_fill(hip_backend._ctx, int(F32), 7.0, 0, c_void_p(o.ptr), n))
        got = b.onCPU().copy()
        # ... and comes back to the pool once the batch has been enqueued
        again = [hip_backend.allocate(n * 4) for _ in range(2)]
        assert ptr in [o.ptr for o in again]
    assert np.array_equal(got, want)


def test_capture_and_replay_inside_batching(hip_backend):
    rng = np.random.default_rng(6)
    m, k, n = 128, 64, 192
    x = hip_backend.upload((rng.standard_normal((m, k)) / k ** 0.5).astype(np.float16))
    w = hip_backend.upload(rng.standard_normal((k, n)).astype(np.float16))
    bias = hip_backend.upload(rng.standard_normal(n).astype(np.float16))
    want = layer(hip_backend, x, w, bias, m, k, n).onCPU().copy()
    with hip_backend.batching():
        pre = layer(hip_backend, x, w, bias, m, k, n)                 # listed when the capture begins
        with hip_backend.capture() as cap:
            out = layer(hip_backend, x, w, bias, m, k, n)
        with pytest.raises(Exception):
            with hip_backend.capture():
                hip_backend.setBatching(8)                            # refused during a capture
        post = layer(hip_backend, x, w, bias, m, k, n)                # listed again afterwards
        cap.graph.launch()
        for got in (pre, out, post):
            assert np.array_equal(got.onCPU(), want)
        cap.graph.destroy()
    in_use, _ = hip_backend.memStats()
    del pre, out, post
    assert hip_backend.memStats()[0] < in_use


def test_waits_and_events_enqueue_the_list(hip_backend):
    n = 1 << 18
    x = hip_backend.upload(np.full(n, 0.5, np.float32))
    once = hip_backend.elemwise(x, ElemwiseOp.exp, None, n, F32)
    want = hip_backend.elemwise(once, ElemwiseOp.exp, None, n, F32).onCPU().copy()
    with hip_backend.batching():
        before = hip_backend.batchingStats()
        y = hip_backend.elemwise(x, ElemwiseOp.exp, None, n, F32)
        assert hip_backend.batchingStats() == before
        y.wait()                                                       # hc_sync
        assert hip_backend.batchingStats()[1] - before[1] == 1
        z = hip_backend.elemwise(y, ElemwiseOp.exp, None, n, F32)
        hip_backend.flush()
        assert hip_backend.batchingStats()[1] - before[1] == 2
        hip_backend.sync()
        assert np.array_equal(z.onCPU(), want)


@pytest.mark.parametrize("dtype", [F16, F32], ids=["f16", "f32"])
def test_config5_forward_pass_batch_limits(hip_backend, dtype):
    """The transformer's forward pass under batches of a few to a few thousand launches (batches end
    anywhere inside layers, chains and attention blocks) and with early batches: the logits of the
    call-by-call run, bit for bit, in both precisions."""
    rng = np.random.default_rng(9)
    with hip_backend.use():
        model = Transformer(dtype=dtype)
        ids = Tensor(data=rng.integers(0, 8192, size=(8, 256)))
        want = model(ids).numpy().copy()
        for limit, idle_after in ((50, 0), (4096, 0), (256, 16), (64, 1), (7, 0), (13, 0), (29, 3), (97, 0), (3, 0)):
            with hip_backend.batching(limit, idle_after):
                for _ in range(2):
                    got = model(ids).numpy()
                    assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), "limit %d, %d" % (limit, idle_after)


def test_a_device_that_has_run_dry_gets_the_list_early(hip_backend):
    """idle_after: with nothing left on the stream, a list of at least that many launches is
    enqueued when the caller lets go of its intermediates (hc_free with at most one buffer of the
    batch still held), long before the limit."""
    n = 1 << 16
    x = hip_backend.upload(np.full(n, 0.25, np.float32))
    want = x
    for _ in range(6):
        want = hip_backend.elemwise(want, ElemwiseOp.exp if _ % 2 == 0 else ElemwiseOp.log, None, n, F32)
    want = want.onCPU().copy()
    hip_backend.sync()
    with hip_backend.batching(1000, 2):
        before = hip_backend.batchingStats()
        y = x
        for i in range(6):
            y = hip_backend.elemwise(y, ElemwiseOp.exp if i % 2 == 0 else ElemwiseOp.log, None, n, F32)   # releases the previous y
        early = hip_backend.batchingStats()[1] - before[1]
        assert np.array_equal(y.onCPU(), want)
    assert early >= 2, early


def test_concurrent_op_chains_under_batching(hip_backend):
    threads, rounds = 6, 8
    want = {s: chain(hip_backend, s) for s in range(threads * rounds)}
    failures = []

    def worker(t):
        try:
            for r in range(rounds):
                seed = t * rounds + r
                for i, (x, y) in enumerate(zip(chain(hip_backend, seed), want[seed])):
                    if not np.array_equal(x, y):
                        failures.append("thread %d seed %d: result %d differs from the unbatched run" % (t, seed, i))
                        return
        except Exception as e:
            failures.append("thread %d: %r" % (t, e))

    with hip_backend.batching(32, 4):
        pool = [threading.Thread(target=worker, args=(t,)) for t in range(threads)]
        for th in pool:
            th.start()
        for th in pool:
            th.join()
    assert not failures, failures[:5]


def test_a_batch_that_cannot_be_enqueued_is_reported(hip_backend):
    """A listed launch that the runtime refuses (here a caller's kernel with an empty grid, rejected on
    the host before anything runs) surfaces in the call that enqueues the batch; when that call is
    one whose status the caller may not see (the batch went out because it was full, or from a
    release), the next wait reports it again, once."""
    import ctypes
    import os
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench_probe.hsaco")
    if not os.path.exists(path):
        pytest.skip("bench_probe.hsaco is not built")
    lib, ctx = hip_backend._lib, hip_backend._ctx
    image = open(path, "rb").read()
    buf = ctypes.create_string_buffer(image, len(image))
    module, fn = ctypes.c_void_p(), ctypes.c_void_p()
    hip_backend._check(lib.hc_module_load(ctx, buf, len(image), ctypes.byref(module)))
    hip_backend._check(lib.hc_module_get_function(module, b"hc_bench_marker", ctypes.byref(fn)))
    n = 4096
    x = hip_backend.upload(np.full(n, 0.5, np.float32))
    want = hip_backend.elemwise(x, ElemwiseOp.exp, None, n, F32).onCPU().copy()
    grid, block = (ctypes.c_uint32 * 3)(0, 1, 1), (ctypes.c_uint32 * 3)(64, 1, 1)
    with hip_backend.batching(2):
        hip_backend._check(lib.hc_launch(ctx, fn, grid, block, 0, None, 0))     # listed: nothing is checked yet
        with pytest.raises(Exception):
            hip_backend.elemwise(x, ElemwiseOp.exp, None, n, F32)                # second launch: the batch is full and goes out
        with pytest.raises(Exception):
            hip_backend.sync()                                                   # ... reported once more
        hip_backend.sync()                                                       # and then no more
        y = hip_backend.elemwise(x, ElemwiseOp.exp, None, n, F32)                # the context works on
        assert np.array_equal(y.onCPU(), want)
