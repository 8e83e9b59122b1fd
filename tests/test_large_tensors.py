"""Maximum sizes: tensors of more than 2^31 elements (more than 4 GiB of fp16) through the
bandwidth-bound kernels, checked against numpy on the whole result. What this pins is the
index arithmetic (32-bit lane ids times vector widths, byte offsets beyond 4 GiB, row counts
times row lengths), not the arithmetic itself, so the ops are chosen to be exact: every
comparison is bit for bit. The data repeat with an odd period, so that an offset that wraps
by any power of two lands on different values."""
import numpy as np
import pytest

from honeycrisp_amd.descriptors import (BroadcastData, BroadcastStrides, DType, ElemwiseOp, NumericBinaryOp,
                                        ReduceDims, ReduceOp, ScatterGatherIndices)

pytestmark = pytest.mark.gpu

F32, F16 = DType.float32, DType.float16
ROWS, COLS = 524300, 4100  # 2 149 630 000 elements > 2^31
N = ROWS * COLS
CHUNK_ROWS = 16384


@pytest.fixture(scope="module")
def big(hip_backend):
    rng = np.random.default_rng(31)
    block = rng.standard_normal(33554467).astype(np.float16)
    x = np.resize(block, N)
    dev = hip_backend.upload(x)
    yield x.reshape(ROWS, COLS), dev
    del dev
    hip_backend.sync()


def chunks():
    for r0 in range(0, ROWS, CHUNK_ROWS):
        yield r0, min(r0 + CHUNK_ROWS, ROWS)


def assert_same_bits(got, want, what):
    bits = {2: np.uint16, 4: np.uint32, 8: np.uint64}[got.dtype.itemsize]
    bad = got.view(bits) != want.view(bits)
    if bad.any():
        i = np.argwhere(bad)[0]
        raise AssertionError("%s: %d elements differ, first at %s: got %r want %r" %
                             (what, int(bad.sum()), tuple(i), got[tuple(i)], want[tuple(i)]))


def test_scalar_and_unary_beyond_2_31_elements(hip_backend, big):
    x, dev = big
    print("scalar mul, %d elements" % N, flush=True)
    out = hip_backend.binaryOp(dev, 0.5, NumericBinaryOp.mul, F16, count=N).onCPU().view(np.float16).reshape(ROWS, COLS)
    for r0, r1 in chunks():
        assert_same_bits(out[r0:r1], (x[r0:r1].astype(np.float32) * np.float32(0.5)).astype(np.float16), "x * 0.5 rows %d.." % r0)
    del out
    print("relu", flush=True)
    out = hip_backend.elemwise(dev, ElemwiseOp.relu, None, N, F16).onCPU().view(np.float16).reshape(ROWS, COLS)
    for r0, r1 in chunks():
        c = x[r0:r1]
        assert_same_bits(out[r0:r1], np.where(c < 0, np.float16(0), c), "relu rows %d.." % r0)


def test_cast_writes_beyond_8_gib(hip_backend, big):
    x, dev = big
    print("cast f16 -> f32, %d elements" % N, flush=True)
    out = hip_backend.cast(dev, N, F16, F32).onCPU().view(np.float32).reshape(ROWS, COLS)
    for r0, r1 in chunks():
        assert_same_bits(out[r0:r1], x[r0:r1].astype(np.float32), "cast rows %d.." % r0)


def test_broadcast_add_beyond_2_31_elements(hip_backend, big):
    x, dev = big
    bias = np.random.default_rng(32).standard_normal(COLS).astype(np.float16)
    print("bias add [%d, %d] + [1, %d]" % (ROWS, COLS, COLS), flush=True)
    out = hip_backend.binaryOp(BroadcastData(BroadcastStrides([ROWS, COLS], [COLS, 1]), dev),
                               BroadcastData(BroadcastStrides([ROWS, COLS], [0, 1]), hip_backend.upload(bias)),
                               NumericBinaryOp.add, F16).onCPU().view(np.float16).reshape(ROWS, COLS)
    b32 = bias.astype(np.float32)
    for r0, r1 in chunks():
        assert_same_bits(out[r0:r1], (x[r0:r1].astype(np.float32) + b32).astype(np.float16), "bias add rows %d.." % r0)


def test_row_argmax_and_gather_beyond_2_31_elements(hip_backend, big):
    x, dev = big
    print("argmax over rows", flush=True)
    idx = hip_backend.reduce(dev, ReduceOp.argmax, ReduceDims(ROWS, COLS, 1), F16).onCPU().view(np.int64)
    for r0, r1 in chunks():
        want = np.argmax(x[r0:r1], axis=1)
        assert np.array_equal(idx[r0:r1], want), "argmax rows %d.." % r0
    print("argmax over columns", flush=True)
    idx = hip_backend.reduce(dev, ReduceOp.argmax, ReduceDims(1, ROWS, COLS), F16).onCPU().view(np.int64)
    best, where = x[0].copy(), np.zeros(COLS, dtype=np.int64)
    for r0, r1 in chunks():  # first occurrence wins
        c = x[r0:r1]
        j = np.argmax(c, axis=0)
        v = c[j, np.arange(COLS)]
        better = v > best
        best[better], where[better] = v[better], j[better] + r0
    assert np.array_equal(idx, where)
    print("row gather from the far end of the table", flush=True)
    ids = np.concatenate([np.arange(ROWS - 300, ROWS), np.arange(0, 300), np.random.default_rng(33).integers(0, ROWS, 1448)])
    s = ScatterGatherIndices([ROWS, COLS], 0, BroadcastData(BroadcastStrides([len(ids), COLS], [1, 0]), hip_backend.upload(ids)))
    out = hip_backend.gather(dev, s, F16).onCPU().view(np.float16).reshape(len(ids), COLS)
    assert_same_bits(out, x[ids], "gather")


def _pattern(shape, seed):
    block = np.random.default_rng(seed).standard_normal(33554467).astype(np.float16)
    block[block == 0] = 0  # no -0: x * 1 + 0 * 0 would turn it into +0
    return np.resize(block, int(np.prod(shape))).reshape(shape)


def test_batched_matmul_operands_beyond_4_gib_in_total(hip_backend):
    """36 products of 8192^2 fp16 matrices (4.8 GB per operand) with the identity on the right:
    every matrix must come back bit for bit, so batch offsets beyond 2^32 bytes are right."""
    batch, n = 36, 8192
    a = _pattern((batch, n, n), 41)
    eye = np.ascontiguousarray(np.broadcast_to(np.eye(n, dtype=np.float16), (batch, n, n)))
    print("batched matmul %d x %d^3" % (batch, n), flush=True)
    da, de = hip_backend.upload(a), hip_backend.upload(eye)
    del eye
    out = hip_backend.batchedMatmul(batch, da, False, de, False, False, n, n, n, F16).onCPU().view(np.float16).reshape(batch, n, n)
    for b in range(batch):
        assert_same_bits(out[b], a[b], "A x I, matrix %d" % b)


@pytest.mark.parametrize("transA", [False, True], ids=["k_contiguous", "m_contiguous"])
def test_matmul_single_operand_beyond_4_gib(hip_backend, transA):
    """One fp16 operand of 4.4 GB (its element offsets no longer fit 32 bits of bytes) times a
    0/1 selection matrix: column j of the product is column sel[j] of A, exactly."""
    M, K, N = 36000, 61440, 64
    a = _pattern((K, M) if transA else (M, K), 42)
    sel = np.random.default_rng(43).integers(0, K, size=N)
    sel[:4] = (0, K - 1, K - 64, 32768)
    b = np.zeros((K, N), dtype=np.float16)
    b[sel, np.arange(N)] = 1
    print("matmul %d x %d x %d, transA=%s" % (M, K, N, transA), flush=True)
    out = hip_backend.matmul(hip_backend.upload(a), transA, hip_backend.upload(b), False, False, M, K, N, F16)
    out = out.onCPU().view(np.float16).reshape(M, N)
    want = np.ascontiguousarray((a[sel, :].T if transA else a[:, sel]))
    assert_same_bits(out, want, "A x selection")
