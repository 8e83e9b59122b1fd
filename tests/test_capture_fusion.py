"""The rewrite of a recording (hc_capture_end): a product whose result has exactly one reader takes
that reader's work into its own kernel, and the launches of a LayerNorm and of an attention
softmax become one kernel each. A replay must return the bits the same ops return when issued one
by one, the rewrite must actually remove launches where it applies, and it must leave the
recording alone where a merged intermediate would be missed (a second reader, a result the caller
still holds)."""
from ctypes import byref, c_void_p

import numpy as np
import pytest

from backend_cases import assert_close_arrays
from honeycrisp_amd.descriptors import DType
from honeycrisp_amd.nn import LayerNorm, Linear, Transformer
from honeycrisp_amd.tensor import Tensor

pytestmark = pytest.mark.gpu

NP = {DType.float32: np.float32, DType.float16: np.float16}


def record(backend, fn, fusion=True):
    """Records fn() and returns (graph, output tensor, node count)."""
    with backend.switches(**({} if fusion else {"HCHIP_NO_FUSION": "1"})):
        with backend.capture() as cap:
            out = fn()
    return cap.graph, out, cap.graph.node_count()


def check(backend, fn, removed):
    """fn() recorded with and without the rewrite and issued eagerly: same bits from all three;
    the rewrite removes exactly `removed` launches."""
    bits = lambda a: np.atleast_1d(a).view(np.uint8)
    want = fn().numpy().copy()
    plain, plain_out, plain_nodes = record(backend, fn, fusion=False)
    fused, fused_out, fused_nodes = record(backend, fn)
    for replay in range(2):
        plain.launch()
        fused.launch()
        assert np.array_equal(bits(plain_out.numpy()), bits(want))
        got = fused_out.numpy()
        assert np.array_equal(bits(got), bits(want)), \
            "replay %d: %d of %d elements differ" % (replay, int((got != want).sum()), want.size)
    assert plain_nodes - fused_nodes == removed, (plain_nodes, fused_nodes)
    plain.destroy()
    fused.destroy()
    # ... and the same ops issued call by call under batching: listed, rewritten the same way and
    # enqueued when the result is read
    listed, enqueued = backend.batchingStats()
    with backend.batching():
        got = fn().numpy().copy()
    listed, enqueued = (after - before for after, before in zip(backend.batchingStats(), (listed, enqueued)))
    assert np.array_equal(bits(got), bits(want)), \
        "batching: %d of %d elements differ" % (int((got != want).sum()), want.size)
    assert listed - enqueued == removed, (listed, enqueued)


def operands(rng, dtype, m, k, n):
    x = Tensor(data=rng.standard_normal((m, k)).astype(np.float32), dtype=dtype)
    w = Tensor(data=(rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32), dtype=dtype)
    bias = Tensor(data=rng.standard_normal((n,)).astype(np.float32), dtype=dtype)
    res = Tensor(data=rng.standard_normal((m, n)).astype(np.float32), dtype=dtype)
    return x, w, bias, res


SHAPES = [(2048, 512, 2048), (2048, 2048, 512), (2048, 512, 8192), (96, 64, 128), (200, 72, 136)]


@pytest.mark.parametrize("dtype", [DType.float32, DType.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("m,k,n", SHAPES)
def test_bias_and_gelu_join_the_product(hip_backend, dtype, m, k, n):
    rng = np.random.default_rng(m + n)
    with hip_backend.use():
        x, w, bias, _ = operands(rng, dtype, m, k, n)
        check(hip_backend, lambda: (Tensor.matmul(x, False, w, False, False) + bias).gelu(), removed=2)


@pytest.mark.parametrize("dtype", [DType.float32, DType.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("m,k,n", SHAPES)
def test_bias_and_residual_join_the_product(hip_backend, dtype, m, k, n):
    rng = np.random.default_rng(m + n + 1)
    with hip_backend.use():
        x, w, bias, res = operands(rng, dtype, m, k, n)
        check(hip_backend, lambda: res + (Tensor.matmul(x, False, w, False, False) + bias), removed=2)
        check(hip_backend, lambda: (bias + Tensor.matmul(x, False, w, False, False)) + res, removed=2)
        # one matrix operand per merged kernel: the second dense addition stays a kernel of its own
        check(hip_backend, lambda: (Tensor.matmul(x, False, w, False, False) + res) + res, removed=1)
        # three merged operations is the limit: the fourth stays a kernel of its own
        check(hip_backend,
              lambda: (((Tensor.matmul(x, False, w, False, False) + bias) + bias) + res) + bias, removed=3)
        # GELU ends a list, and does not follow a matrix operand
        check(hip_backend,
              lambda: ((Tensor.matmul(x, False, w, False, False) + bias).gelu() + res).gelu(), removed=2)
        check(hip_backend,
              lambda: (res + (Tensor.matmul(x, False, w, False, False) + bias)).gelu(), removed=2)


def test_transposed_operands_and_a_three_axis_input(hip_backend):
    rng = np.random.default_rng(5)
    with hip_backend.use():
        x, w, bias, res = operands(rng, DType.float16, 512, 256, 384)
        wt = Tensor(data=w.numpy().T.copy(), dtype=DType.float16)
        check(hip_backend, lambda: (Tensor.matmul(x, False, wt, True, False) + bias).gelu(), removed=2)
        # `Linear` on [B, T, D]: reshapes around the product do not get in the way
        lin = Linear(256, 384, rng, dtype=DType.float16, castParams=DType.float16)
        x3 = Tensor(data=rng.standard_normal((4, 128, 256)).astype(np.float32), dtype=DType.float16)
        res3 = Tensor(data=rng.standard_normal((4, 128, 384)).astype(np.float32), dtype=DType.float16)
        # (the fp32 bias is cast to fp16 at call time: that cast is merged as well)
        check(hip_backend, lambda: res3 + lin(x3), removed=3)


def test_a_result_with_two_readers_stays(hip_backend):
    rng = np.random.default_rng(6)
    with hip_backend.use():
        x, w, bias, res = operands(rng, DType.float32, 256, 128, 256)

        def two_readers():
            h = Tensor.matmul(x, False, w, False, False)
            return (h + bias) + h.gelu()

        check(hip_backend, two_readers, removed=0)

        def same_operand_twice():
            h = Tensor.matmul(x, False, w, False, False)
            return h + h

        check(hip_backend, same_operand_twice, removed=0)


def test_a_result_the_caller_keeps_is_written(hip_backend):
    rng = np.random.default_rng(7)
    with hip_backend.use():
        x, w, bias, _ = operands(rng, DType.float32, 256, 128, 256)
        want_h = Tensor.matmul(x, False, w, False, False).numpy()
        want = (Tensor.matmul(x, False, w, False, False) + bias).numpy()
        with hip_backend.capture() as cap:
            h = Tensor.matmul(x, False, w, False, False)        # still referenced after the capture
            out = h + bias
        cap.graph.launch()
        assert np.array_equal(h.numpy(), want_h)
        assert np.array_equal(out.numpy(), want)
        cap.graph.destroy()


def test_a_write_into_a_deferred_input_keeps_the_original_order(hip_backend):
    """The fp32 bias is cast, then overwritten in part (a copy into the middle of its buffer), then
    the cast copy is added to a product. Merging the cast into the product would read the bias
    after the overwrite; the rewrite must see the partial write and leave the cast where it was."""
    from ctypes import c_void_p
    rng = np.random.default_rng(12)
    with hip_backend.use():
        x, w, _, _ = operands(rng, DType.float16, 256, 128, 256)
        bias32 = Tensor(data=rng.standard_normal((256,)).astype(np.float32))
        patch = Tensor(data=np.full((16,), 100.0, np.float32))
        old = bias32.numpy().copy()

        def run():
            b16 = bias32.cast(DType.float16)
            hip_backend._check(hip_backend._lib.hc_memcpy_d2d(hip_backend._ctx, c_void_p(bias32.data.ptr + 64),
                                                               c_void_p(patch.data.ptr), 64))
            return Tensor.matmul(x, False, w, False, False) + b16

        want = (Tensor.matmul(x, False, w, False, False) + Tensor(data=old, dtype=DType.float16)).numpy()
        with hip_backend.capture() as cap:
            out = run()
        for _ in range(2):
            bias32.data.mutateOnCPU(lambda host: host.view(np.float32).__setitem__(slice(None), old))
            cap.graph.launch()
            assert np.array_equal(out.numpy(), want)
        cap.graph.destroy()


def test_blocks_of_merged_intermediates_return_to_the_pool(hip_backend):
    """An intermediate that the rewrite merged away is written by no launch of the graph, so its
    block goes back to the general pool when the capture ends: a recording with the rewrite keeps
    less memory reserved, and whoever receives those blocks is not disturbed by replays."""
    from ctypes import byref, c_size_t
    rng = np.random.default_rng(14)

    def reserved():
        used, cached = c_size_t(0), c_size_t(0)
        hip_backend._check(hip_backend._lib.hc_mem_stats(hip_backend._ctx, byref(used), byref(cached)))
        return used.value, cached.value

    with hip_backend.use():
        model = Transformer(dtype=DType.float16, layers=2, d_model=256, heads=4, mlp=512, vocab=512, seq=64, seed=5)
        ids = Tensor(data=rng.integers(0, 512, size=(4, 64)))
        want = model(ids).numpy().copy()
        hip_backend.sync()
        with hip_backend.switches(HCHIP_NO_FUSION="1"):
            with hip_backend.capture() as plain:
                plain_out = model(ids)
        _, cached_plain = reserved()
        with hip_backend.capture() as fused:
            fused_out = model(ids)
        _, cached_fused = reserved()
        # the second recording found blocks in the pool that the first one could not have left there,
        # and left more behind than it took: its merged intermediates
        assert cached_fused > cached_plain
        # blocks of every size the model uses, filled with a pattern: a replay must not touch them
        held = [Tensor(data=np.full(shape, 7.0, np.float32), dtype=dtype)
                for shape in ((4 * 64, 256), (4 * 64, 512), (4, 4, 64, 64), (256,)) for dtype in (DType.float16, DType.float32)
                for _ in range(6)]
        for _ in range(2):
            fused.graph.launch()
            plain.graph.launch()
            assert np.array_equal(fused_out.numpy().view(np.uint8), want.view(np.uint8))
            assert np.array_equal(plain_out.numpy().view(np.uint8), want.view(np.uint8))
            assert all(np.all(t.numpy() == 7.0) for t in held)
        plain.graph.destroy()
        fused.graph.destroy()


def test_a_callers_own_kernel_is_a_barrier(hip_backend):
    """A launch through hc_launch declares no buffers: it may read or write anything, so nothing
    is merged across it (here it sits between a product and the addition of its bias)."""
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
    hip_backend._check(lib.hc_module_get_function(module, b"hc_probe_mfma_f16_16x16x32", ctypes.byref(fn)))

    class Args(ctypes.Structure):
        _fields_ = [("data", ctypes.c_void_p), ("out", ctypes.c_void_p), ("iters", ctypes.c_uint32), ("chunks", ctypes.c_uint32)]

    rng = np.random.default_rng(15)
    with hip_backend.use():
        x, w, bias, _ = operands(rng, DType.float16, 256, 128, 256)
        data = Tensor(data=rng.standard_normal((4096,)).astype(np.float32), dtype=DType.float16)
        sink = Tensor(data=np.zeros((4 * 256,), np.float32))

        def own_kernel():
            args = Args(data.data.ptr, sink.data.ptr, 1, 4096 * 2 // 16)
            grid, block = (ctypes.c_uint32 * 3)(4, 1, 1), (ctypes.c_uint32 * 3)(256, 1, 1)
            hip_backend._check(lib.hc_launch(ctx, fn, grid, block, 0, ctypes.byref(args), ctypes.sizeof(args)))

        def with_barrier():
            h = Tensor.matmul(x, False, w, False, False)
            own_kernel()
            return (h + bias).gelu()

        def without():      # (the product's result is released before the caller's kernel is issued)
            out = (Tensor.matmul(x, False, w, False, False) + bias).gelu()
            own_kernel()
            return out

        def still_held():   # ... and here it is not: the caller's kernel might read it
            h = Tensor.matmul(x, False, w, False, False)
            out = (h + bias).gelu()
            own_kernel()
            return out

        check(hip_backend, with_barrier, removed=0)
        check(hip_backend, without, removed=2)
        check(hip_backend, still_held, removed=0)
    hip_backend.sync()
    hip_backend._check(lib.hc_module_unload(ctx, module))


def test_other_forms_of_add_are_left_alone(hip_backend):
    rng = np.random.default_rng(8)
    with hip_backend.use():
        x, w, _, _ = operands(rng, DType.float32, 256, 128, 256)
        col = Tensor(data=rng.standard_normal((256, 1)).astype(np.float32))
        ints = Tensor(data=rng.integers(-5, 5, size=(256, 128)))
        iw = Tensor(data=rng.integers(-5, 5, size=(128, 256)))
        irow = Tensor(data=rng.integers(-5, 5, size=(256,)))
        check(hip_backend, lambda: Tensor.matmul(x, False, w, False, False) + col, removed=0)
        check(hip_backend, lambda: Tensor.matmul(x, False, w, False, False) * w.sum(axis=0), removed=0)
        check(hip_backend, lambda: Tensor.matmul(ints, False, iw, False, False) + irow, removed=0)


@pytest.mark.parametrize("dtype,removed", [(DType.float32, 2), (DType.float16, 4)], ids=["f32", "f16"])
@pytest.mark.parametrize("rows,width", [(2048, 512), (77, 1024), (300, 132), (5, 256)])
def test_layernorm_becomes_one_kernel(hip_backend, dtype, removed, rows, width):
    """cast -> normalize -> gain + 1 -> mulAdd -> cast (the casts only around fp16 activations)."""
    rng = np.random.default_rng(rows + width)
    with hip_backend.use():
        ln = LayerNorm([width], rng=rng)
        x = Tensor(data=(rng.standard_normal((rows, width)) * 3 + 1).astype(np.float32), dtype=dtype)
        check(hip_backend, lambda: ln(x), removed=removed)
        x3 = Tensor(data=rng.standard_normal((3, 7, width)).astype(np.float32), dtype=dtype)
        check(hip_backend, lambda: ln(x3), removed=removed)


def test_layernorm_variants(hip_backend):
    rng = np.random.default_rng(21)
    with hip_backend.use():
        x = Tensor(data=rng.standard_normal((64, 256)).astype(np.float32))
        plain = LayerNorm([256], affine=False)
        check(hip_backend, lambda: plain(x), removed=0)                 # normalize alone: nothing to merge
        xh = x.cast(DType.float16)
        check(hip_backend, lambda: plain(xh), removed=2)                # cast, normalize, cast
        ln = LayerNorm([256], rng=rng)
        # the coefficient used as it is (no gain + 1), and a normalized tensor that is read twice
        check(hip_backend,
              lambda: x.normalize(axis=1, eps=1e-5).mul(ln.gain, thenAdd=ln.bias), removed=1)

        def read_twice():
            n = x.normalize(axis=1, eps=1e-5)
            return n.mul(ln.gain + 1, thenAdd=ln.bias) + n

        check(hip_backend, read_twice, removed=0)
        # rows of 1028 floats do not fit a wave's registers, rows of 16 take a smaller team: left alone
        for width in (1028, 16):
            wide = LayerNorm([width], rng=rng)
            xw = Tensor(data=rng.standard_normal((32, width)).astype(np.float32))
            check(hip_backend, lambda: wide(xw), removed=0)


@pytest.mark.parametrize("dtype", [DType.float32, DType.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("heads,t", [(32, 256), (6, 40), (3, 512), (2, 1024)])
def test_attention_softmax_becomes_one_kernel(hip_backend, dtype, heads, t):
    """scores * s -> + mask -> logSoftmax -> exp."""
    rng = np.random.default_rng(heads + t)
    with hip_backend.use():
        scores = Tensor(data=(rng.standard_normal((2, heads, t, t)) * 4).astype(np.float32), dtype=dtype)
        mask = Tensor(data=np.where(np.tril(np.ones((t, t))) > 0, 0.0, -1e4).astype(np.float32), dtype=dtype)
        full = Tensor(data=rng.standard_normal((2, heads, t, t)).astype(np.float32), dtype=dtype)
        check(hip_backend, lambda: (scores * 0.125 + mask).softmax(), removed=3)
        check(hip_backend, lambda: (mask + scores * 0.125).softmax(), removed=3)
        check(hip_backend, lambda: (scores * 0.125 + full).softmax(), removed=3)
        check(hip_backend, lambda: (scores * 0.125).softmax(), removed=2)
        check(hip_backend, lambda: (scores + mask).logSoftmax(), removed=1)
        check(hip_backend, lambda: scores.softmax(), removed=1)


def test_softmax_forms_that_are_left_alone(hip_backend):
    rng = np.random.default_rng(33)
    with hip_backend.use():
        x = Tensor(data=rng.standard_normal((64, 100)).astype(np.float32), dtype=DType.float16)   # 100 halfs: no 16-byte rows
        check(hip_backend, lambda: (x * 0.5).softmax(), removed=0)
        y = Tensor(data=rng.standard_normal((64, 4096)).astype(np.float32))                        # a block per row
        check(hip_backend, lambda: (y * 0.5).softmax(), removed=0)
        z = Tensor(data=rng.standard_normal((64, 256)).astype(np.float32))

        def scaled_read_twice():
            s = z * 0.5
            return s.softmax() + s

        check(hip_backend, scaled_read_twice, removed=1)       # only the exp joins
        col = Tensor(data=rng.standard_normal((64, 1)).astype(np.float32))
        check(hip_backend, lambda: (z + col).softmax(), removed=1)  # a column operand is no mask


@pytest.mark.parametrize("dtype", [DType.float32, DType.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("m,k,n", [(2048, 512, 512), (192, 72, 136)])
def test_products_over_the_same_input_share_a_launch(hip_backend, dtype, m, k, n):
    """q, k, v = three Linear layers of one shape applied to the same activations."""
    rng = np.random.default_rng(m + k)
    cast = DType.float16 if dtype == DType.float16 else None
    with hip_backend.use():
        x = Tensor(data=rng.standard_normal((m, k)).astype(np.float32), dtype=dtype)
        lins = [Linear(k, n, rng, dtype=dtype, castParams=cast) for _ in range(5)]
        for lin in lins:
            lin.bias = Tensor(data=rng.standard_normal((n,)).astype(np.float32))
        other = Linear(k, n + 8, rng, dtype=dtype, castParams=cast)
        per_linear = 2 if dtype == DType.float16 else 1      # bias add (and the bias's cast) merged into each product

        def three():
            q, kk, v = (lin(x) for lin in lins[:3])
            return q * kk * v           # (products of results: nothing else to merge into the matmuls)

        check(hip_backend, three, removed=3 * per_linear + 2)

        def five():          # at most four products per launch: the fifth stays alone
            outs = [lin(x) for lin in lins]
            return ((outs[0] * outs[1]) * (outs[2] * outs[3])) * outs[4]

        check(hip_backend, five, removed=5 * per_linear + 3)

        def chained():       # the second product reads the first one's result: no group
            h = lins[0](x)
            return lins[1](h) if k == n else lins[1](x) * h.gelu()

        check(hip_backend, chained, removed=2 * per_linear + (0 if k == n else 1))

        def different_shapes():
            return lins[0](x).sum(axis=1) * other(x).sum(axis=1)

        check(hip_backend, different_shapes, removed=2 * per_linear)


@pytest.mark.parametrize("dtype", [DType.float32, DType.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("B,T,H,hd", [(8, 256, 8, 64), (2, 96, 3, 40), (1, 128, 4, 64)])
def test_head_swaps_fold_into_the_batched_products(hip_backend, dtype, B, T, H, hd):
    """[B, T, H*hd] -> [B, T, H, hd] -> swap(1, 2) around batchedMatmul: the products read q, k, v
    through the strides and write the context back in [B, T, H, hd] order; no copy is left."""
    rng = np.random.default_rng(B + T + H)
    D = H * hd
    with hip_backend.use():
        q, k, v = (Tensor(data=rng.standard_normal((B, T, D)).astype(np.float32), dtype=dtype) for _ in range(3))

        def heads(x):
            return x.reshape([B, T, H, hd]).swap(1, 2)

        def attention():
            scores = Tensor.batchedMatmul(heads(q), False, heads(k), True, False)
            probs = (scores * 0.125).softmax()
            return Tensor.batchedMatmul(probs, False, heads(v), False, False).swap(1, 2).reshape([B, T, D])

        # 4 swaps, and scale + logSoftmax + exp -> 1; with 64-wide heads the two products and that
        # row kernel then become the attention kernel
        check(hip_backend, attention, removed=4 + 2 + (2 if hd == 64 else 0))
        # one operand swapped, the other dense; result kept in [B, H, T, T] order
        kt = Tensor(data=rng.standard_normal((B, H, T, hd)).astype(np.float32), dtype=dtype)
        check(hip_backend, lambda: Tensor.batchedMatmul(heads(q), False, kt, True, False), removed=1)
        check(hip_backend, lambda: Tensor.batchedMatmul(kt, False, heads(q), True, False), removed=1)
        # a swapped tensor with a second reader stays a copy
        def two_readers():
            hq = heads(q)
            return Tensor.batchedMatmul(hq, False, kt, True, False) + hq.sum(axis=3, keepdims=True)

        check(hip_backend, two_readers, removed=0)


@pytest.mark.parametrize("dtype,heads,t", [(DType.float16, h, t) for h, t in
                                           [(64, 256), (32, 512), (5, 64), (3, 128), (2, 192), (3, 320), (2, 448), (12, 128), (19, 192)]] +
                         [(DType.float32, h, t) for h, t in [(64, 256), (5, 64), (3, 128), (2, 192), (12, 128), (19, 256)]],
                         ids=lambda v: v.name if isinstance(v, DType) else str(v))
def test_attention_becomes_one_kernel(hip_backend, dtype, heads, t):
    """q k^T -> [* s] [+ mask] softmax -> x v over heads of 64 (fp16 up to 512 keys, fp32 up to 256): one launch
    per recording, and a replay returns the bits of the five separate launches (same accumulation order in
    both products, scores and probabilities rounded to the tensor type, the row kernel's own reduction)."""
    rng = np.random.default_rng(heads * 1000 + t)
    f16 = dtype
    with hip_backend.use():
        q, k, v = (Tensor(data=rng.standard_normal((heads, t, 64)).astype(np.float32), dtype=f16) for _ in range(3))
        mask = Tensor(data=np.where(np.tril(np.ones((t, t))) > 0, 0.0, -1e4).astype(np.float32), dtype=f16)

        def attention(scale=True, masked=True, log=False):
            s = Tensor.batchedMatmul(q, False, k, True, False)
            if scale:
                s = s * 0.125
            if masked:
                s = s + mask
            p = s.logSoftmax() if log else s.softmax()
            return Tensor.batchedMatmul(p, False, v, False, False)

        check(hip_backend, attention, removed=3 + 2)                                   # scale, mask, logSoftmax, exp -> 1; -> attention
        check(hip_backend, lambda: attention(masked=False), removed=2 + 2)
        check(hip_backend, lambda: attention(scale=False), removed=2 + 2)
        check(hip_backend, lambda: attention(log=True), removed=2 + 2)                # (log-probabilities times v: same machinery)
        # a bare softmax is a row kernel of its own plus exp: the chain of two still merges, and then the three
        check(hip_backend, lambda: attention(scale=False, masked=False), removed=1 + 2)


def test_attention_forms_that_are_left_alone(hip_backend):
    rng = np.random.default_rng(77)
    f16 = DType.float16

    def qkv(heads, t, hd, dtype=f16):
        return (Tensor(data=rng.standard_normal((heads, t, hd)).astype(np.float32), dtype=dtype) for _ in range(3))

    with hip_backend.use():
        def attention(q, k, v):
            s = Tensor.batchedMatmul(q, False, k, True, False) * 0.125
            return Tensor.batchedMatmul(s.softmax(), False, v, False, False)

        q, k, v = qkv(8, 128, 32)                # heads of 32
        check(hip_backend, lambda: attention(q, k, v), removed=2)
        q, k, v = qkv(2, 320, 64, DType.float32)  # fp32 rows longer than the score tile holds
        check(hip_backend, lambda: attention(q, k, v), removed=2)
        q, k, v = qkv(2, 576, 64)                # rows longer than the score tile holds
        check(hip_backend, lambda: attention(q, k, v), removed=2)
        q, k, v = qkv(4, 128, 64)

        def probabilities_read_twice():
            p = (Tensor.batchedMatmul(q, False, k, True, False) * 0.125).softmax()
            return Tensor.batchedMatmul(p, False, v, False, False).sum(axis=2) + p.sum(axis=2)

        check(hip_backend, probabilities_read_twice, removed=2)

        def scores_kept():                        # the caller keeps the scores: they must be written
            s = Tensor.batchedMatmul(q, False, k, True, False)
            return s, Tensor.batchedMatmul((s * 0.125).softmax(), False, v, False, False)

        want_s, want_o = (x.numpy().copy() for x in scores_kept())
        with hip_backend.capture() as cap:
            s, o = scores_kept()
        cap.graph.launch()
        assert np.array_equal(s.numpy(), want_s) and np.array_equal(o.numpy(), want_o)
        cap.graph.destroy()


@pytest.mark.parametrize("dtype", [DType.float32, DType.float16], ids=["f32", "f16"])
def test_config5_forward_recorded_with_the_rewrite(hip_backend, dtype):
    rng = np.random.default_rng(9)
    with hip_backend.use():
        model = Transformer(dtype=dtype)
        ids = Tensor(data=rng.integers(0, 8192, size=(8, 256)))
        want = model(ids).numpy().copy()
        plain, plain_out, plain_nodes = record(hip_backend, lambda: model(ids), fusion=False)
        fused, fused_out, fused_nodes = record(hip_backend, lambda: model(ids))
        print("config 5", dtype.name, "launches per forward pass:", plain_nodes, "->", fused_nodes, flush=True)
        for replay in range(3):
            fused.launch()
            assert np.array_equal(fused_out.numpy().view(np.uint8), want.view(np.uint8)), "replay %d" % replay
        plain.launch()
        assert np.array_equal(plain_out.numpy(), want)
        # per block: q, k, v (+bias), o and fc2 (+bias, +residual), fc1 (+bias, GELU) = 9 launches
        # merged into products, 2 LayerNorms of 3 launches (fp16: 5), a softmax of 4, the 4 swaps of
        # the heads, and q, k, v in one launch; then the last LayerNorm and the unembedding's bias;
        # in fp16 also the 6 + 1 casts of the fp32 biases
        half = dtype == DType.float16
        per_block = 9 + 2 * (4 if half else 2) + 3 + 4 + 2 + (6 if half else 0)
        # ... and (64-wide heads) scores, softmax and context of a block are one attention kernel
        per_block += 2
        assert plain_nodes - fused_nodes == 6 * per_block + (4 if half else 2) + (2 if half else 1)
        assert fused_nodes == 46
        plain.destroy()
        fused.destroy()
        # the same forward pass call by call under batching: one batch, the same launches
        listed, enqueued = hip_backend.batchingStats()
        with hip_backend.batching(1024):
            for _ in range(2):
                assert np.array_equal(model(ids).numpy().view(np.uint8), want.view(np.uint8))
        listed, enqueued = (after - before for after, before in zip(hip_backend.batchingStats(), (listed, enqueued)))
        assert (listed, enqueued) == (2 * plain_nodes, 2 * fused_nodes)


class _Raw:
    """Calls straight into the C ABI with plain addresses, so that operands can be views: pointers
    into the middle of a block that hc_malloc handed out (include/hchip.h allows them)."""

    def __init__(self, backend):
        from honeycrisp_amd import _lib
        self.b, self.lib, self.ctx, self.mk = backend, backend._lib, backend._ctx, _lib.make_strides

    def matmul(self, a, b, out, m, k, n, dtype=DType.float32):
        self.b._check(self.lib.hc_matmul(self.ctx, int(dtype), 1, c_void_p(a), 0, c_void_p(b), 0, 0, m, k, n, c_void_p(out)))

    def add_row(self, x, row, out, m, n, dtype=DType.float32):
        xs, rs = self.mk((m, n), (n, 1)), self.mk((m, n), (0, 1))
        self.b._check(self.lib.hc_binary_op(self.ctx, 0, int(dtype), c_void_p(x), byref(xs), c_void_p(row), byref(rs), c_void_p(out)))

    def fill(self, ptr, count, value, dtype=DType.float32):
        self.b._check(self.lib.hc_fill(self.ctx, int(dtype), float(value), 0, c_void_p(ptr), count))

    def copy(self, dst, src, nbytes):
        self.b._check(self.lib.hc_memcpy_d2d(self.ctx, c_void_p(dst), c_void_p(src), nbytes))

    def malloc(self, nbytes):
        p = c_void_p()
        self.b._check(self.lib.hc_malloc(self.ctx, nbytes, byref(p)))
        return p.value

    def free(self, ptr):
        self.b._check(self.lib.hc_free(self.ctx, c_void_p(ptr)))


def test_a_write_through_a_view_keeps_the_product_in_front_of_it(hip_backend):
    """The product's second operand is a view into a block; between the product and the addition
    that the rewrite would merge into it, a fill writes through another view of the same block,
    over part of that operand. Deferring the product past the fill would make it read the new
    values: the recording must give what the call-by-call order gives."""
    raw = _Raw(hip_backend)
    rng = np.random.default_rng(31)
    m, k, n = 256, 128, 192
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.standard_normal((k, n)).astype(np.float32)
    bias = rng.standard_normal((n,)).astype(np.float32)
    want = (x @ w + bias).astype(np.float32)
    block = hip_backend.allocate(4096 + w.nbytes)            # the operand starts 1 KiB into its block
    xd, bd, out = hip_backend.upload(x), hip_backend.upload(bias), hip_backend.allocate(want.nbytes)
    w_ptr, hole_ptr = block.ptr + 1024, block.ptr + 1024 + 40 * n * 4     # rows 40.. of the operand

    def upload_w():
        hip_backend._check(hip_backend._lib.hc_memcpy_h2d(hip_backend._ctx, c_void_p(w_ptr), w.ctypes.data_as(c_void_p), w.nbytes))

    def issue():
        tmp = raw.malloc(want.nbytes)
        raw.matmul(xd.ptr, w_ptr, tmp, m, k, n)
        raw.fill(hole_ptr, 16 * n, 100.0)
        raw.add_row(tmp, bd.ptr, out.ptr, m, n)
        raw.free(tmp)

    graphs = []
    for fusion in (False, True):
        with hip_backend.switches(**({} if fusion else {"HCHIP_NO_FUSION": "1"})):
            with hip_backend.capture() as cap:
                issue()
        graphs.append(cap.graph)
    for graph in graphs:
        for replay in range(2):
            upload_w()
            raw.fill(out.ptr, m * n, 0.0)
            graph.launch()
            got = out.onCPU().view(np.float32).reshape(m, n)
            assert_close_arrays(got, want, 1e-4, 1e-4)
        graph.destroy()


def test_a_read_through_a_view_keeps_grouped_products_in_front_of_it(hip_backend):
    """Two products over one input that the rewrite would run as one launch where the second one
    stands; in between, a copy reads the first product's result through a pointer into the middle
    of it (the caller keeps that result, so the recording never sees its release). The copy must
    still see the first product's values."""
    raw = _Raw(hip_backend)
    rng = np.random.default_rng(32)
    m, k, n = 512, 256, 256
    x = rng.standard_normal((m, k)).astype(np.float32)
    wq = rng.standard_normal((k, n)).astype(np.float32)
    wk = rng.standard_normal((k, n)).astype(np.float32)
    xd, wqd, wkd = hip_backend.upload(x), hip_backend.upload(wq), hip_backend.upload(wk)
    q, kk = hip_backend.allocate(m * n * 4), hip_backend.allocate(m * n * 4)
    rows = 8
    picked = hip_backend.allocate(rows * n * 4)
    offset = 100 * n * 4                                     # rows 100..107 of q

    def issue():
        raw.matmul(xd.ptr, wqd.ptr, q.ptr, m, k, n)
        raw.copy(picked.ptr, q.ptr + offset, rows * n * 4)
        raw.matmul(xd.ptr, wkd.ptr, kk.ptr, m, k, n)

    want_q, want_k = x @ wq, x @ wk
    for fusion in (False, True):
        with hip_backend.switches(**({} if fusion else {"HCHIP_NO_FUSION": "1"})):
            with hip_backend.capture() as cap:
                issue()
        for replay in range(2):
            raw.fill(q.ptr, m * n, -7.0)
            raw.fill(picked.ptr, rows * n, 0.0)
            cap.graph.launch()
            assert_close_arrays(picked.onCPU().view(np.float32).reshape(rows, n), want_q[100:108], 1e-4, 1e-4)
            assert_close_arrays(q.onCPU().view(np.float32).reshape(m, n), want_q, 1e-4, 1e-4)
            assert_close_arrays(kk.onCPU().view(np.float32).reshape(m, n), want_k, 1e-4, 1e-4)
        cap.graph.destroy()


def test_a_buffer_written_before_the_merged_product_stays_with_the_graph(hip_backend):
    """fill(X), then a product into X whose only reader is merged into it: X is written by no launch
    of the merged chain any more, but the fill in front of it still writes it on every replay, so its
    block must stay reserved for the graph instead of going back to the pool."""
    raw = _Raw(hip_backend)
    rng = np.random.default_rng(33)
    m, k, n = 256, 128, 128
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.standard_normal((k, n)).astype(np.float32)
    bias = rng.standard_normal((n,)).astype(np.float32)
    xd, wd, bd, out = hip_backend.upload(x), hip_backend.upload(w), hip_backend.upload(bias), hip_backend.allocate(m * n * 4)
    with hip_backend.capture() as cap:
        tmp = raw.malloc(m * n * 4)
        raw.fill(tmp, m * n, 3.0)
        raw.matmul(xd.ptr, wd.ptr, tmp, m, k, n)
        raw.add_row(tmp, bd.ptr, out.ptr, m, n)
        raw.free(tmp)
    # whoever allocates a block of that size now must not receive the one the recorded fill writes
    others = [hip_backend.allocate(m * n * 4) for _ in range(8)]
    for o in others:
        raw.fill(o.ptr, m * n, 9.0)
    for replay in range(2):
        cap.graph.launch()
        assert_close_arrays(out.onCPU().view(np.float32).reshape(m, n), (x @ w + bias).astype(np.float32), 1e-4, 1e-4)
        for o in others:
            assert np.all(o.onCPU().view(np.float32) == 9.0)
    cap.graph.destroy()


def extremum_input(rng, dtype, rows, cols):
    """Rows with repeated extrema (the first one's index decides) and, for floats, a few NaNs."""
    if dtype == DType.bool:
        return Tensor(data=(rng.random((rows, cols)) < 0.5).astype(np.float32)).cast(DType.bool)
    if dtype == DType.int64:
        return Tensor(data=rng.integers(-50, 50, (rows, cols)), dtype=DType.int64)
    data = np.round(rng.standard_normal((rows, cols)) * 8).astype(np.float32) / 4
    data[rng.random((rows, cols)) < 0.002] = np.nan
    return Tensor(data=data, dtype=dtype)


@pytest.mark.parametrize("dtype", [DType.float32, DType.float16, DType.int64, DType.bool], ids=["f32", "f16", "i64", "bool"])
@pytest.mark.parametrize("rows,cols", [(1000, 5), (333, 100), (257, 1000), (9, 3001), (2, 30000)])
def test_max_and_min_over_rows_become_one_kernel(hip_backend, dtype, rows, cols):
    """Tensor.max / min are an arg-reduction and a gather of its indices (ReduceRepeat.swift:201-209);
    over the last axis, the row kernel that finds the index leaves the element itself."""
    rng = np.random.default_rng(rows * 7 + cols)
    with hip_backend.use():
        x = extremum_input(rng, dtype, rows, cols)
        check(hip_backend, lambda: x.max(axis=1), removed=1)
        check(hip_backend, lambda: x.min(axis=-1, keepdims=True), removed=1)
        if dtype == DType.bool:
            check(hip_backend, lambda: x.some(axis=1), removed=1)
            check(hip_backend, lambda: x.all(axis=1, keepdims=True), removed=1)
        # three axes, the last one reduced: still rows
        if rows % 3 == 0:
            y = x.reshape([3, rows // 3, cols])
            check(hip_backend, lambda: y.max(axis=2), removed=1)


def test_extrema_that_are_left_alone(hip_backend):
    rng = np.random.default_rng(5)
    with hip_backend.use():
        x = extremum_input(rng, DType.float32, 300, 64)
        other = extremum_input(rng, DType.float32, 300, 64)
        # an axis that is not the last one: a column reduction
        check(hip_backend, lambda: x.max(axis=0), removed=0)
        # the indices pick from another tensor
        check(hip_backend, lambda: other.gather(1, x.argmax(axis=1, keepdims=True)), removed=0)
        # the caller keeps the indices
        held = []

        def both():
            idx = x.argmax(axis=1, keepdims=True)
            held.append(idx)
            return x.gather(1, idx)

        check(hip_backend, both, removed=0)
        # a long row cut into segments: two launches find the index
        long_row = extremum_input(rng, DType.float32, 1, 300000)
        check(hip_backend, lambda: long_row.max(), removed=0)
        # the input changes between the two launches: the gather must see the new values
        first = Tensor(data=rng.standard_normal((64, 32)).astype(np.float32))
        second = Tensor(data=rng.standard_normal((64, 32)).astype(np.float32))

        def rewritten():
            t = first + 0.0
            idx = t.argmax(axis=1, keepdims=True)
            hip_backend._check(hip_backend._lib.hc_memcpy_d2d(hip_backend._ctx, c_void_p(t.data.ptr),
                                                               c_void_p(second.data.ptr), 64 * 32 * 4))
            return t.gather(1, idx)

        check(hip_backend, rewritten, removed=0)
        want = np.take_along_axis(second.numpy(), first.numpy().argmax(axis=1)[:, None], axis=1)
        assert np.array_equal(rewritten().numpy(), want)
