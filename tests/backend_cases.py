"""Backend-parametric cases, the counterpart of the reference's shared `BackendTests`
(Sources/HCTestUtils/BackendTests.swift): every function runs against whatever backend is
current and checks the reference's own expected vectors / invariants (forward values only).
The drivers run them under the CPU oracle (no GPU needed) and under HIPBackend (GPU).
"""
import json
import os

import numpy as np

from honeycrisp_amd.descriptors import DType
from honeycrisp_amd.tensor import FlipAxis, FullRange, NewAxis, PermuteAxes, Tensor

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "backend_tests.json")))

F32, F16, I64, BOOL = DType.float32, DType.float16, DType.int64, DType.bool


def assertDataEqual(x, y):
    """Assertions.swift:60-90: exact equality of the values as floats."""
    got = x.floats()
    want = y.floats() if isinstance(y, Tensor) else [float(np.float32(v)) for v in y]
    assert got == want, "%s != %s" % (got, want)


def assertClose(x, y, atol=1e-4, rtol=1e-4):
    """Assertions.swift:6-47: NaN pattern equal and |a-b| <= atol or |a/b-1| <= rtol."""
    got = np.asarray(x.floats(), dtype=np.float32)
    want = np.asarray(y.floats() if isinstance(y, Tensor) else y, dtype=np.float32).reshape(-1)
    assert got.shape == want.shape
    assert_close_arrays(got, want, atol, rtol)


def assert_close_arrays(got, want, atol, rtol):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    want = np.asarray(want, dtype=np.float64).reshape(-1)
    assert got.shape == want.shape
    nan_ok = np.isnan(got) == np.isnan(want)
    with np.errstate(divide="ignore", invalid="ignore"):
        bad = (np.abs(got - want) > atol) & ((want == 0) | (np.abs(got / want - 1) > rtol))
    bad = (bad & ~np.isnan(want)) | ~nan_ok
    # equal infinities are fine
    bad &= ~((got == want) & np.isinf(want))
    if bad.any():
        i = int(np.argmax(bad))
        raise AssertionError("%d of %d elements differ; first at %d: got %r want %r" %
                             (int(bad.sum()), got.size, i, got[i], want[i]))


def testCreateFromData():
    """BackendTests.swift:39-68."""
    for dtype in (I64, F16, F32):
        for reverse in (False, True):
            rev = (lambda a: list(reversed(a))) if reverse else (lambda a: a)
            assertDataEqual(Tensor(data=[1, 2, 3], dtype=dtype, reverse=reverse), rev([1.0, 2.0, 3.0]))
            assertDataEqual(Tensor(data=range(1, 4), dtype=dtype, reverse=reverse), rev([1.0, 2.0, 3.0]))
            assertDataEqual(Tensor(data=range(-1, 4), dtype=dtype, reverse=reverse), rev([-1.0, 0.0, 1.0, 2.0, 3.0]))
            assertDataEqual(Tensor(data=range(-4, -2), dtype=dtype, reverse=reverse), rev([-4.0, -3.0]))


def testCast():
    """BackendTests.swift:70-84."""
    x = Tensor(data=[1.0, 2.0, 0.0], shape=[3], dtype=F32)
    assertDataEqual(x, [1.0, 2.0, 0.0])
    y = x.cast(F16)
    assert y.dtype == F16
    assertDataEqual(y, [1.0, 2.0, 0.0])
    assertDataEqual(x.cast(I64), [1.0, 2.0, 0.0])
    assertDataEqual(x.cast(BOOL), [1.0, 1.0, 0.0])
    big = Tensor(data=[1_000_000_000], shape=[1], dtype=F32)
    assert not np.isfinite(big.cast(F16).item())


def testAdd():
    """BackendTests.swift:86-100."""
    x = Tensor(data=[1.0, 2.0, 0.0], shape=[3], dtype=F32)
    y = Tensor(data=[-1.0, 2.0, -3.0], shape=[3], dtype=F32)
    assertDataEqual(x + y, [0.0, 4.0, -3.0])
    assertDataEqual(x.cast(I64) + y.cast(I64), [0.0, 4.0, -3.0])
    assertDataEqual(x.cast(F16) + y.cast(F16), [0.0, 4.0, -3.0])
    assertDataEqual(x + 3, [4.0, 5.0, 3.0])
    assertDataEqual(x.cast(I64) + 3, [4.0, 5.0, 3.0])
    assertDataEqual(x.cast(F16) + 3, [4.0, 5.0, 3.0])
    assertDataEqual(3 + x, [4.0, 5.0, 3.0])
    assertDataEqual(3 + x.cast(I64), [4.0, 5.0, 3.0])
    assertDataEqual(3 + x.cast(F16), [4.0, 5.0, 3.0])
    assertDataEqual(x + 1.5, [2.5, 3.5, 1.5])
    assertDataEqual(1.5 + x, [2.5, 3.5, 1.5])


def testSub():
    """BackendTests.swift:102-116."""
    x = Tensor(data=[1.0, 2.0, 0.0], shape=[3], dtype=F32)
    y = Tensor(data=[-1.0, 2.0, -3.0], shape=[3], dtype=F32)
    assertDataEqual(x - y, [2.0, 0.0, 3.0])
    assertDataEqual(x.cast(I64) - y.cast(I64), [2.0, 0.0, 3.0])
    assertDataEqual(x.cast(F16) - y.cast(F16), [2.0, 0.0, 3.0])
    assertDataEqual(x - (-3), [4.0, 5.0, 3.0])
    assertDataEqual(x.cast(I64) - (-3), [4.0, 5.0, 3.0])
    assertDataEqual(x.cast(F16) - (-3), [4.0, 5.0, 3.0])
    assertDataEqual(3 - x, [2.0, 1.0, 3.0])
    assertDataEqual(3 - x.cast(I64), [2.0, 1.0, 3.0])
    assertDataEqual(3 - x.cast(F16), [2.0, 1.0, 3.0])
    assertDataEqual(x - 1.5, [-0.5, 0.5, -1.5])
    assertDataEqual(1.5 - x, [0.5, -0.5, 1.5])


def testMul():
    """BackendTests.swift:118-130."""
    x = Tensor(data=[1.0, 2.0, 3.0, 0.0], shape=[4], dtype=F32)
    y = Tensor(data=[-1.0, 2.0, 2.0, -3.0], shape=[4], dtype=F32)
    assertDataEqual(x * y, [-1.0, 4.0, 6.0, 0.0])
    assertDataEqual(x.cast(F16) * y.cast(F16), [-1.0, 4.0, 6.0, 0.0])
    assertDataEqual(x.cast(I64) * y.cast(I64), [-1.0, 4.0, 6.0, 0.0])
    for t in (x, x.cast(F16), x.cast(I64)):
        assertDataEqual(t * 2, [2.0, 4.0, 6.0, 0.0])
        assertDataEqual(2 * t, [2.0, 4.0, 6.0, 0.0])


def testDiv():
    """BackendTests.swift:132-152 (forward)."""
    x = Tensor(data=[1.0, 2.0, 6.0, 0.0], shape=[4], dtype=F32)
    y = Tensor(data=[-1.0, 2.0, 2.0, 3.0], shape=[4], dtype=F32)
    assertDataEqual(x / y, [-1.0, 1.0, 3.0, 0.0])
    assertDataEqual(x.cast(F16) / y.cast(F16), [-1.0, 1.0, 3.0, 0.0])
    assertDataEqual(x.cast(I64) / y.cast(I64), [-1.0, 1.0, 3.0, 0.0])
    assertDataEqual(x / 2, [0.5, 1.0, 3.0, 0.0])
    assertDataEqual(x.cast(F16) / 2, [0.5, 1.0, 3.0, 0.0])
    assertDataEqual(x.cast(I64) / 2, [0.0, 1.0, 3.0, 0.0])
    assertDataEqual(6 / y, [-6.0, 3.0, 3.0, 2.0])
    assertDataEqual(6 / y.cast(F16), [-6.0, 3.0, 3.0, 2.0])
    assertDataEqual(6 / y.cast(I64), [-6.0, 3.0, 3.0, 2.0])
    assertDataEqual(2 / y.cast(I64), [-2.0, 1.0, 1.0, 0.0])


def testFusedAddMul():
    """BackendTests.swift:154-191 (forward)."""
    for dtype in (F32, F16, I64):
        x = Tensor(data=[1, 2, 0], shape=[3], dtype=dtype)
        y = Tensor(data=[-2, 3, -4], shape=[3], dtype=dtype)
        z = Tensor(data=[2, 3, 0], shape=[3], dtype=dtype)
        assertDataEqual(x.add(y, thenMul=z), (x + y) * z)
        assertDataEqual(x.mul(y, thenAdd=z), (x * y) + z)


def testFusedNormalize(rng):
    """BackendTests.swift:193-219 (forward)."""
    epsilon = 0.3
    for dtype in (F32, F16):
        tol = 1e-4 if dtype == F32 else 2e-2
        for shape in ([6, 1025], [1, 1025], [6, 8], [256, 4], [256, 256], [1025, 4]):
            for axis in range(len(shape)):
                xData = Tensor(data=rng.standard_normal(shape).astype(np.float32), dtype=dtype)
                x = xData.cast(F32)
                mean = x.mean(axis=axis, keepdims=True)
                variance = (x - mean).pow(2).mean(axis=axis, keepdims=True)
                normed = (x - mean) / (variance + epsilon).sqrt()
                normedFused = xData.normalize(axis=axis, eps=epsilon)
                assertClose(normed, normedFused.cast(dtype), atol=tol, rtol=tol)


def testMod():
    """BackendTests.swift:221-252 (forward)."""
    m = GOLDEN["mod"]
    for a, b, out in m["simple"]:
        for dtype in (F32, F16, I64):
            assertDataEqual(Tensor(data=[a], shape=[1], dtype=dtype) % Tensor(data=[b], shape=[1], dtype=dtype),
                            [float(out)])
    x = Tensor(data=m["x"], shape=[7], dtype=F32)
    y = Tensor(data=m["y"], shape=[7], dtype=F32)
    assertDataEqual(Tensor(data=[3], shape=[1]) % Tensor(data=[2], shape=[1]), [1])
    assertDataEqual(x % y, m["x_mod_y"])
    assertDataEqual(x.cast(F16) % y.cast(F16), m["x_mod_y"])
    assertDataEqual(x.cast(I64) % y.cast(I64), m["xi_mod_yi"])
    assertDataEqual(x % 2, m["x_mod_2"])
    assertDataEqual(x.cast(F16) % 2, m["x_mod_2"])
    assertDataEqual(x.cast(I64) % 2, m["xi_mod_2"])
    assertDataEqual(7.5 % y, m["7.5_mod_y"])
    assertDataEqual(7.5 % y.cast(F16), m["7.5_mod_y"])
    assertDataEqual(7 % y.cast(I64), m["7_mod_yi"])


def testEquals():
    """BackendTests.swift:287-299."""
    x = Tensor(data=[1.0, 2.0, 3.0, -2.0, 3.0], shape=[5])
    y = Tensor(data=[1, 2, 2, -2, -3], shape=[5]).cast(x)
    assertDataEqual(x == y, [1, 1, 0, 1, 0])
    assert (x == y).dtype == BOOL and (x == y).shape == x.shape
    t1 = Tensor(data=[1, 2, 3, 4, 3, 1, 2, 0], shape=[2, 4])
    t2 = Tensor(data=[1, 0, 4, 4, 0, 0, 1, 0], shape=[2, 4])
    assertDataEqual(t1 == 2, [0, 1, 0, 0, 0, 0, 1, 0])
    assertDataEqual(t1 == t2, [1, 0, 0, 1, 0, 0, 0, 1])


def testComparison():
    """BackendTests.swift:301-311."""
    x = Tensor(data=[1.0, 2.0, 3.0, -2.0, 3.0], shape=[5])
    y = Tensor(data=[1.5, 2, 2, -2, -3], shape=[5])
    assertDataEqual(x == y, [0, 1, 0, 1, 0])
    assertDataEqual(x <= y, [1, 1, 0, 1, 0])
    assertDataEqual(x < y, [1, 0, 0, 0, 0])
    assertDataEqual(x >= y, [0, 1, 1, 1, 1])
    assertDataEqual(x > y, [0, 0, 1, 0, 1])
    assert (x >= y).dtype == BOOL and (x >= y).shape == x.shape


def testSum():
    """BackendTests.swift:335-434 (forward)."""
    x = Tensor(data=[1.0, 2.0, 3.0, -2.0, 3.0, 7.0], shape=[1, 2, 3, 1], dtype=F32)
    s = x.sum(axis=2)
    assert s.shape == [1, 2, 1]
    assertDataEqual(s, [6.0, 8.0])
    s = x.sum(axis=2, keepdims=True)
    assert s.shape == [1, 2, 1, 1]
    assertDataEqual(s, [6.0, 8.0])
    s = x.sum(axis=1)
    assert s.shape == [1, 3, 1]
    assertDataEqual(s, [-1.0, 5.0, 10.0])
    s = x.sum(axis=1, keepdims=True)
    assert s.shape == [1, 1, 3, 1]
    assertDataEqual(s, [-1.0, 5.0, 10.0])
    for axis in (0, -1):
        for keepdims in (False, True):
            s = x.sum(axis=axis, keepdims=keepdims)
            if keepdims:
                assert s.shape == [1, 2, 3, 1]
            elif axis == 0:
                assert s.shape == [2, 3, 1]
            else:
                assert s.shape == [1, 2, 3]
            assertDataEqual(s, x)
    s = x.sum()
    assert s.shape == []
    assertDataEqual(s, [14.0])
    s = x.sum(keepdims=True)
    assert s.shape == [1, 1, 1, 1]
    assertDataEqual(s, [14.0])
    nd = Tensor(data=list(range(1, 13)), shape=[2, 2, 3], dtype=F32)
    assertDataEqual(nd.sum(axis=1), [5, 7, 9, 17, 19, 21])
    inp = Tensor(data=list(range(1, 10)), shape=[3, 3], dtype=F32)
    assertDataEqual(inp.sum(axis=1), [6, 15, 24])
    assertDataEqual(inp.sum(axis=0), [12, 15, 18])
    inp1 = Tensor(data=list(range(1, 9)), shape=[2, 2, 2], dtype=F32)
    assertDataEqual(inp1.sum(axis=1), [4, 6, 12, 14])
    assertDataEqual(inp1.sum(), [36])


def testGather():
    """BackendTests.swift:585-682 (forward)."""
    for dtype in (F16, F32):
        x = Tensor(data=[1.0, 2.0, 3.0, -2.0, 3.0, 7.0], shape=[1, 2, 3, 1], dtype=dtype)
        out = x.gather(2, Tensor(data=[2, 0, 1, 2], shape=[1, 2, 2, 1], dtype=I64))
        assert out.shape == [1, 2, 2, 1]
        assertDataEqual(out, [3.0, 1.0, 3.0, 7.0])
        out = x.gather(2, Tensor(data=[2, 0], shape=[2], dtype=I64))
        assert out.shape == [1, 2, 2, 1]
        assertDataEqual(out, [3.0, 1.0, 7.0, -2.0])
        out = x.gather(1, Tensor(data=[0, 1, 0, 1, 0, 0], shape=[1, 2, 3, 1], dtype=I64))
        assert out.shape == [1, 2, 3, 1]
        assertDataEqual(out, [1.0, 3.0, 3.0, -2.0, 2.0, 3.0])
        out = x.gather(1, Tensor(data=[1, 0], shape=[2], dtype=I64))
        assert out.shape == [1, 2, 3, 1]
        assertDataEqual(out, [-2.0, 3.0, 7.0, 1.0, 2.0, 3.0])
    tr = GOLDEN["transpose_2x3x4"]
    for dtype in (F16, F32, I64):
        t = Tensor(data=tr["data"], shape=tr["shape"], dtype=dtype)
        assertDataEqual(t.t(), tr["out"])
        assert t.t().data.byteCount >= t.dtype.byteSize * 24
        assertDataEqual(t.t() == 0, (t == 0).t())  # boolean gather


def testGatherBroadcastOtherAxis(rng):
    """BackendTests.swift:660-681 (forward)."""
    for dtype in (F16, F32):
        y = Tensor(data=rng.random([3, 4, 5]).astype(np.float32), dtype=dtype)
        indices = Tensor(data=[i % 4 for i in range(20)], shape=[1, 4, 5])
        actual = y.gather(1, indices)
        expected = y.gather(1, indices.expand([3, 4, 5]))
        assertDataEqual(actual, expected)


def testMatrixMatrixProduct():
    """BackendTests.swift:684-726 (forward)."""
    g = GOLDEN["matmul_2x3_3x4"]
    for transA in (False, True):
        for transB in (False, True):
            for transOut in (False, True):
                for dtype in (F32, F16):
                    a = Tensor(data=g["x"], shape=g["x_shape"], dtype=dtype)
                    b = Tensor(data=g["y_pre_t"], shape=g["y_pre_t_shape"], dtype=dtype).t()
                    sub = Tensor.matmul(a.t() if transA else a, transA, b.t() if transB else b, transB, transOut)
                    out = sub.t() if transOut else sub
                    assert out.shape == [2, 4]
                    assertDataEqual(out, g["out"])
    x = Tensor.ones([64, 128])
    y = Tensor.ones([128, 32])
    z = Tensor.matmul(x, False, y, False, False)
    assert z.shape == [64, 32]
    assertDataEqual(z, [128.0] * (64 * 32))
    small = x.cast(F16) @ y.cast(F16)
    assert np.isfinite(small.cast(F32).sum().item())
    big = (x.cast(F16) * 1000) @ (y.cast(F16) * 1000)
    assert not np.isfinite(big.cast(F32).sum().item())


def testBatchedMatmul(rng):
    """BackendTests.swift:728-767 (forward): batched == per-matrix for all 8 flag combos."""
    for transA in (False, True):
        for transB in (False, True):
            for transOut in (False, True):
                for dtype in (F32, F16):
                    x = Tensor(data=rng.random([3, 2, 3]).astype(np.float32), dtype=dtype)
                    y = Tensor(data=rng.random([3, 3, 4]).astype(np.float32), dtype=dtype)
                    pre = Tensor.batchedMatmul(x.t() if transA else x, transA, y.t() if transB else y, transB,
                                               transOut)
                    out = pre.t() if transOut else pre
                    assert out.shape == [3, 2, 4]
                    eps = 1e-4 if dtype == F32 else 1e-2
                    for i in range(3):
                        a, b = x[i], y[i]
                        single = Tensor.matmul(a.t() if transA else a, transA, b.t() if transB else b, transB,
                                               transOut)
                        sub = single.t() if transOut else single
                        assert sub.shape == out[i].shape
                        assertClose(sub, out[i], atol=eps, rtol=eps)


def testMatrixVectorProduct():
    """BackendTests.swift:769-783 (forward)."""
    g = GOLDEN["matvec"]
    x = Tensor(data=g["x"], shape=g["x_shape"], dtype=F32)
    y = Tensor(data=g["y"], shape=g["y_shape"], dtype=F32)
    assertDataEqual(x @ y, g["out"])


def testTriangular():
    """BackendTests.swift:785-800 (first cases)."""
    t = Tensor(data=[1, 2, 3, 4, 5, 6], shape=[3, 2])
    assertDataEqual(t.tril(), [1, 0, 3, 4, 5, 6])
    assertDataEqual(t.tril(offset=-4), [0, 0, 0, 0, 0, 0])
    assertDataEqual(t.tril(offset=-3), [0, 0, 0, 0, 0, 0])
    assertDataEqual(t.tril(offset=-2), [0, 0, 0, 0, 5, 0])


def testIndexing():
    """BackendTests.swift:931-1029 (forward)."""
    x = Tensor(data=[1, 2, 3, 4, 5, 6], shape=[3, 2])
    assert x[0].shape == [2]
    assert x[..., 0].shape == [3]
    assertDataEqual(x[1], [3, 4])
    assertDataEqual(x[1:3], [3, 4, 5, 6])
    assertDataEqual(x[1:2], [3, 4])
    assertDataEqual(x[-2:-1], [3, 4])
    assertDataEqual(x[-2:], [3, 4, 5, 6])
    assertDataEqual(x[:-1], [1, 2, 3, 4])
    assertDataEqual(x[:-2], [1, 2])
    assertDataEqual(x[-2], [3, 4])
    assertDataEqual(x[-1], [5, 6])
    y = Tensor(data=list(range(1, 13)), shape=[3, 1, 4], dtype=F32)
    assert y[..., 0].shape == [3, 4]
    assertDataEqual(y[..., 0], y)
    assert y[0, ..., 0].shape == [1]
    assertDataEqual(y[0, ..., 0], [1])
    assert y[..., 0, ...].shape == [3, 4]
    assertDataEqual(y[0, FullRange(2)], [1, 2, 3, 4])
    assert y[0, FullRange(2)].shape == [1, 4]
    assert y[0, 0, 0].shape == []
    assertDataEqual(y[0, 0, 0], [1])
    assertDataEqual(y[0:2, ..., 3], [4, 8])
    assertDataEqual(y[0:3, ..., 3], [4, 8, 12])
    assertDataEqual(y[0:, ..., 3], [4, 8, 12])
    assertDataEqual(y[1:3, ..., 2:4], [7, 8, 11, 12])
    assertDataEqual(y[0:3, ..., 2:4], [3, 4, 7, 8, 11, 12])
    assertDataEqual(y[0:3, 0:1, 2:4], [3, 4, 7, 8, 11, 12])
    assertDataEqual(y[FullRange(3), NewAxis()], y)
    assert y[FullRange(3), NewAxis()].shape == [3, 1, 4, 1]
    assert y[FullRange(2), NewAxis()].shape == [3, 1, 1, 4]
    assert y[NewAxis()].shape == [1, 3, 1, 4]
    assertDataEqual(y[..., ..., FlipAxis()], [4, 3, 2, 1, 8, 7, 6, 5, 12, 11, 10, 9])
    assert y[..., 0, 3].shape == [3]
    g = GOLDEN["permute5d"]
    big = Tensor(data=g["data"], shape=g["shape"], dtype=F32)
    for name in ("perm1", "perm2", "perm3"):
        p = g[name]
        index = ([FullRange(p["full"])] if p["full"] else []) + [PermuteAxes(p["perm"])]
        out = big[tuple(index)]
        assert out.shape == p["shape"]
        assertDataEqual(out, g["data"] if p["out"] == "same_as_input" else p["out"])


def _apply_elemwise(name, t):
    return {
        "pow2": lambda: t.pow(2), "pow-1": lambda: t.pow(-1), "exp": t.exp, "sqrt": t.sqrt,
        "gelu_approx": lambda: t.gelu("approx"), "gelu_exact": lambda: t.gelu("exact"), "erf": t.erf,
        "abs": t.abs, "relu": t.relu, "sigmoid": t.sigmoid, "log": t.log,
        "exp_log": lambda: t.exp().log(), "tan": t.tan, "atan": t.atan, "acos": t.acos, "asin": t.asin,
    }[name]()


def testElemwise():
    """BackendTests.swift:1047-1200 (forward): tol 1e-4 for fp32 (1e-3 for gelu/erf), x100 for fp16."""
    for case in GOLDEN["elemwise"]["cases"]:
        for dtype in (F32, F16):
            t = Tensor(data=case["input"], shape=[len(case["input"])], dtype=dtype)
            tol = case["tol"] * (1.0 if dtype == F32 else 100.0)
            assertClose(_apply_elemwise(case["op"], t), case["output"], atol=tol, rtol=tol)


def testRounding():
    """BackendTests.swift:1214-1232: round/floor/ceil == Float.rounded(), .down, .up."""
    for dtype in (F16, F32):
        x = Tensor(data=GOLDEN["rounding_inputs"]["input"], dtype=dtype)
        vals = np.asarray(x.floats(), dtype=np.float32)
        half_away = np.where(vals >= 0, np.floor(vals + np.float32(0.5)), np.ceil(vals - np.float32(0.5)))
        # vals +- 0.5 is exact for these inputs in fp32, so the expression above is
        # round-half-away-from-zero without double rounding
        assertDataEqual(x.round(), Tensor(data=half_away, dtype=dtype))
        assertDataEqual(x.floor(), Tensor(data=np.floor(vals), dtype=dtype))
        assertDataEqual(x.ceil(), Tensor(data=np.ceil(vals), dtype=dtype))


def testMinMax():
    """BackendTests.swift:1325-1362 (forward)."""
    inp = Tensor(data=[1, 10, 2, 7, 8, 9, 6, 4, 5], shape=[3, 3], dtype=F32)
    assertDataEqual(inp.max(axis=1), [10, 9, 6])
    assertDataEqual(inp.max(axis=0), [7, 10, 9])
    assertDataEqual(inp.min(axis=0), [1, 4, 2])
    m = inp.max()
    assert m.shape == []
    assertDataEqual(m, [10])
    m = inp.min()
    assert m.shape == []
    assertDataEqual(m, [1])
    assert inp.max(keepdims=True).shape == [1, 1]
    assert inp.max(axis=0, keepdims=True).shape == [1, 3]
    assert inp.max(axis=1, keepdims=True).shape == [3, 1]


def testExpandAndRepeat():
    """BackendTests.swift:1427-1459 (forward)."""
    t1Arr = [1.0, 2.0, 3.0, 4.0]
    t2Arr = [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    t1 = Tensor(data=t1Arr, shape=[2, 2])
    assert t1.reshape([1, 2, 1, 2]).expand([3, 7, 2, 5, 2]).shape == [3, 7, 2, 5, 2]
    t2 = Tensor(data=t2Arr, shape=[1, 2, 1, 3, 1])
    assertDataEqual(t2.repeating(0, 2), t2Arr + t2Arr)
    assertDataEqual(t2.repeating(0, 2), t2.expand([2, 2, 1, 3, 1]))
    assertDataEqual(t2.repeating(1, 2), t2Arr + t2Arr)
    assertDataEqual(t2.repeating(2, 2), [1, 2, 3, 1, 2, 3, 4, 5, 6, 4, 5, 6])
    assertDataEqual(t2.expand([1, 2, 2, 3, 1]), [1, 2, 3, 1, 2, 3, 4, 5, 6, 4, 5, 6])
    assertDataEqual(t2.repeating(3, 2), [1, 2, 3, 1, 2, 3, 4, 5, 6, 4, 5, 6])
    assertDataEqual(t2.repeating(4, 2), [1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 6])
    assertDataEqual(t2.expand([1, 2, 1, 3, 2]), [1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 6])
    assert t1.repeating(2, 3).shape == [2, 2, 3]
    assertDataEqual(t1.repeating(2, 3), [1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4])


BROADCAST_SHAPES = [
    ([6], [3, 6]), ([3, 6], [6]), ([3, 1, 6], [1, 2, 6]), ([1, 1, 3], [3, 4, 3]),
    ([1, 3, 1, 3, 1], [3, 1, 3, 1, 3]), ([3, 1, 3, 1, 3, 1], [1, 3, 1, 3, 1, 3]),
]


def testBinaryBroadcast(rng):
    """BackendTests.swift:1461-1502 (forward): implicit broadcast == explicit expand."""
    ops = [
        lambda a, b: a + b, lambda a, b: a * b, lambda a, b: a - b, lambda a, b: a / b, lambda a, b: a % b,
        lambda a, b: a.mul(b, thenAdd=b), lambda a, b: a.add(b, thenMul=b),
        lambda a, b: a.mul(b, thenAdd=a), lambda a, b: a.add(b, thenMul=a),
        lambda a, b: a < b, lambda a, b: a <= b, lambda a, b: a > b, lambda a, b: a >= b, lambda a, b: a == b,
    ]
    for op in ops:
        for leftShape, rightShape in BROADCAST_SHAPES:
            left = Tensor(data=rng.random(leftShape).astype(np.float32))
            right = Tensor(data=rng.random(rightShape).astype(np.float32)) + 1
            bl, br = Tensor.broadcast([left, right])
            outB = op(bl, br)
            outI = op(left, right)
            assert outB.shape == outI.shape
            if outB.dtype == BOOL:
                assertDataEqual(outB, outI)
            else:
                assertClose(outB, outI)


def testFusedBroadcast(rng):
    """BackendTests.swift:1504-1550 (forward)."""
    for op in (lambda a, b, c: a.mul(b, thenAdd=c), lambda a, b, c: a.add(b, thenMul=c)):
        for aS, bS, cS in [
            ([6], [3, 6], [6]), ([6], [3, 6], [3, 3, 6]), ([1, 3, 1, 3, 1], [3, 1, 3, 1, 3], [1, 1]),
            ([1, 3, 1, 3, 1], [3, 1, 3, 1, 3], []), ([1, 1, 3, 3, 1, 1], [3, 3, 1, 1, 3, 3], [1, 3]),
            ([1, 1, 3, 3, 1, 1], [3, 3, 1, 1, 3, 3], [3, 1]), ([3, 1], [1, 1, 3, 3, 1, 1], [3, 3, 1, 1, 3, 3]),
        ]:
            a = Tensor(data=rng.random(aS).astype(np.float32), shape=aS)
            b = Tensor(data=rng.random(bS).astype(np.float32), shape=bS)
            c = Tensor(data=rng.random(cS).astype(np.float32), shape=cS)
            bc = Tensor.broadcast([a, b, c])
            outB = op(bc[0], bc[1], bc[2])
            outI = op(a, b, c)
            assert outB.shape == outI.shape
            assertClose(outB, outI)


def testSoftmax(rng):
    """BackendTests.swift:1552-1626 (forward)."""
    g = GOLDEN["softmax"]
    x = Tensor(data=g["x"], shape=g["shape"])
    assertClose(x.logSoftmax(axis=0), g["axis0"])
    assertClose(x.logSoftmax(axis=1), g["axis1"])
    for dtype in (F16, F32):
        tol = 1e-2 if dtype == F16 else 1e-4
        inp = Tensor(data=rng.random([7, 3, 292]).astype(np.float32), dtype=dtype)
        out1 = inp.logSoftmax(axis=-1)
        out2 = inp.move(-1, 1).logSoftmax(axis=1).move(1, -1)
        assertClose(out1, out2, atol=tol, rtol=tol)


def testCumulativeSum():
    """BackendTests.swift:466-500 (forward values)."""
    for dtype in (F16, F32, I64):
        raw = Tensor(data=[1, 2, 3, -2, 4, 7], shape=[2, 3], dtype=dtype)
        for exclusive, reverse, want in [(False, False, [1, 3, 6, -2, 2, 9]), (True, False, [0, 1, 3, 0, -2, 2]),
                                         (False, True, [6, 5, 3, 9, 11, 7]), (True, True, [5, 3, 0, 11, 7, 0])]:
            assertDataEqual(raw.cumulativeSum(1, exclusive, reverse), want)
            ax0 = raw.t().cumulativeSum(1, exclusive, reverse).t()
            assertDataEqual(ax0, raw.cumulativeSum(0, exclusive, reverse))


def testCumulativeProd():
    """BackendTests.swift:502-524."""
    for dtype in (F16, F32, I64):
        raw = Tensor(data=[1, 2, 3, -2, 4, -2], shape=[2, 3], dtype=dtype)
        for exclusive, reverse, want in [(False, False, [1, 2, 6, -2, -8, 16]), (True, False, [1, 1, 2, 1, -2, -8]),
                                         (False, True, [6, 6, 3, 16, -8, -2]), (True, True, [6, 3, 1, -8, -2, 1])]:
            assertDataEqual(raw.cumulativeProd(1, exclusive, reverse), want)
            ax0 = raw.t().cumulativeProd(1, exclusive, reverse).t()
            assertDataEqual(ax0, raw.cumulativeProd(0, exclusive, reverse))


def testArgsort(rng):
    """BackendTests.swift:526-564: gathering with the sorted indices sorts every axis, and the
    stable order of equal keys."""
    for dtype in (F16, F32, I64):
        values = rng.integers(-30, 31, size=(2, 3, 4))
        unsorted = Tensor(data=values, dtype=I64).cast(dtype)
        for descending in (False, True):
            for stable in (False, True):
                for axis in (0, 1, 2):
                    want = np.sort(values, axis=axis)
                    if descending:
                        want = np.flip(want, axis=axis)
                    idx = unsorted.argsort(axis, descending=descending, stable=stable)
                    assert idx.dtype == I64
                    assertDataEqual(unsorted.gather(axis, idx), want.reshape(-1))
            ties = Tensor(data=[1, 2, 3, 1, 4, 3, 5, 3], shape=[8]).cast(dtype)
            expected = [6, 4, 2, 5, 7, 1, 0, 3] if descending else [0, 3, 1, 2, 5, 7, 4, 6]
            assertDataEqual(ties.argsort(0, descending=descending, stable=True), expected)


def testBitwise():
    """BackendTests.swift:312-333."""
    x = Tensor(data=[0x123456789f, 0xff00ff00, 2, 1], shape=[4], dtype=I64)
    y = Tensor(data=[1, 2, 0x123456789f, 0xff00ff00], shape=[4], dtype=I64)
    ints = lambda t: [int(v) for v in t.numpy().reshape(-1)]
    assert ints(x ^ y) == [0x123456789e, 0xff00ff02, 0x123456789d, 0xff00ff01]
    assert ints(x & y) == [1, 0, 2, 0]
    assert ints(x | y) == [0x123456789f, 0xff00ff02, 0x123456789f, 0xff00ff01]
    assert ints(x ^ 2) == [0x123456789d, 0xff00ff02, 0, 3]
    assert ints(x | 2) == [0x123456789f, 0xff00ff02, 2, 3]
    assert ints(x & 2) == [2, 0, 2, 0]
    assert ints(x & 0x1000000000) == [0x1000000000, 0, 0, 0]
    assert ints(2 ^ x) == [0x123456789d, 0xff00ff02, 0, 3]
    assert ints(2 | x) == [0x123456789f, 0xff00ff02, 2, 3]
    assert ints(2 & x) == [2, 0, 2, 0]
    assert ints(0x1000000000 & x) == [0x1000000000, 0, 0, 0]
    # boolean masks, the everyday use (e.g. BackendTests.swift:1262-1264)
    a = Tensor(data=[1, 0, 1, 0], shape=[4]).cast(BOOL)
    b = Tensor(data=[1, 1, 0, 0], shape=[2, 1, 4][2:]).cast(BOOL)
    assertDataEqual(a & b, [1, 0, 0, 0])
    assertDataEqual(a | b, [1, 1, 1, 0])
    assertDataEqual(a ^ b, [0, 1, 1, 0])


def testSoftmaxGrad(rng):
    """BackendTests.swift:1552-1626, the gradients: logSoftmaxGrad called the way
    Tensor.logSoftmax's backward does (Softmax.swift), golden input gradients for both axes,
    and axis-invariance on random data."""
    from honeycrisp_amd.backend import Backend
    g = GOLDEN["softmax"]
    x = Tensor(data=g["x"], shape=g["shape"])
    og = Tensor(data=g["out_grad"], shape=g["shape"])
    backend = Backend.current()
    for axis, key in ((0, "axis0_grad"), (1, "axis1_grad")):
        data = backend.logSoftmaxGrad(x.data, og.data, x.reduceDims(axis), x.dtype)
        assertClose(Tensor(dataHandle=data, shape=x.shape, dtype=x.dtype), g[key])
    for dtype in (F16, F32):
        tol = 1e-2 if dtype == F16 else 1e-4
        inp = Tensor(data=rng.random([7, 3, 292]).astype(np.float32), dtype=dtype)
        grad = Tensor(data=rng.random([7, 3, 292]).astype(np.float32), dtype=dtype)
        g1 = Tensor(dataHandle=backend.logSoftmaxGrad(inp.data, grad.data, inp.reduceDims(-1), dtype),
                    shape=inp.shape, dtype=dtype)
        moved, movedGrad = inp.move(-1, 1), grad.move(-1, 1)
        g2 = Tensor(dataHandle=backend.logSoftmaxGrad(moved.data, movedGrad.data, moved.reduceDims(1), dtype),
                    shape=moved.shape, dtype=dtype).move(1, -1)
        assertClose(g1, g2, atol=tol, rtol=tol)


def testScatter():
    """BackendTests.swift:585-650: the input gradients of testGather are scatters of the output
    gradient with the gather's indices (ScatterGather.swift:98-108), plus the direct scatter
    permutation (:626-633)."""
    for dtype in (F16, F32):
        def grad_of_gather(axis, indices, outGrad, shape, unique=False):
            og = Tensor(data=outGrad, shape=shape, dtype=dtype)
            return og.scatter(axis, [1, 2, 3, 1][axis], indices, indicesAreUnique=unique)
        for unique in (False, True):
            got = grad_of_gather(2, Tensor(data=[2, 0, 1, 2], shape=[1, 2, 2, 1], dtype=I64),
                                 [1.0, 2.0, 3.0, 4.0], [1, 2, 2, 1], unique)
            assert got.shape == [1, 2, 3, 1]
            assertDataEqual(got, [2.0, 0.0, 1.0, 0.0, 3.0, 4.0])
            got = grad_of_gather(2, Tensor(data=[2, 0], shape=[2], dtype=I64),
                                 [1.0, 2.0, 3.0, 4.0], [1, 2, 2, 1], unique)
            assertDataEqual(got, [2.0, 0.0, 1.0, 4.0, 0.0, 3.0])
        got = grad_of_gather(1, Tensor(data=[0, 1, 0, 1, 0, 0], shape=[1, 2, 3, 1], dtype=I64),
                             [1.0, 2.0, 3.0, 4.0, 5.0, 6.0], [1, 2, 3, 1])
        assertDataEqual(got, [1.0, 5.0, 9.0, 4.0, 2.0, 0.0])
        got = grad_of_gather(1, Tensor(data=[1, 0], shape=[2], dtype=I64),
                             [1.0, 2.0, 3.0, 4.0, 5.0, 6.0], [1, 2, 3, 1])
        assertDataEqual(got, [4.0, 5.0, 6.0, 1.0, 2.0, 3.0])
        permuteMe = Tensor(data=[1.0, 2.0, 3.0, 4.0, 5.0, 6.0], shape=[1, 2, 3, 1], dtype=dtype)
        for unique in (False, True):
            out = permuteMe.scatter(1, 2, Tensor(data=[1, 0], shape=[2]), indicesAreUnique=unique)
            assertDataEqual(out, [4.0, 5.0, 6.0, 1.0, 2.0, 3.0])
    # int64 values accumulate too
    vals = Tensor(data=[5, 6, 7, 8], shape=[4], dtype=I64)
    assertDataEqual(vals.scatter(0, 3, Tensor(data=[2, 0, 2, 2], shape=[4])), [6, 0, 20])


def testScatterIsAdjointOfGather(rng):
    """BackendTests.swift:660-681, the gradient half: scattering with broadcast indices equals
    scattering with the explicitly expanded ones."""
    for dtype in (F16, F32):
        tol = 1e-2 if dtype == F16 else 1e-4
        indices = Tensor(data=[i % 4 for i in range(20)], shape=[1, 4, 5])
        outGrad = Tensor(data=rng.random([3, 4, 5]).astype(np.float32), dtype=dtype)
        actual = outGrad.scatter(1, 4, indices)
        expected = outGrad.scatter(1, 4, indices.expand([3, 4, 5]))
        assert actual.shape == [3, 4, 5]
        assertClose(actual, expected, atol=tol, rtol=tol)


def testClamp():
    """BackendTests.swift:1235-1323 (forward values)."""
    g = GOLDEN["clamp"]
    for dtype in (I64, F16, F32):
        dim1 = Tensor(data=g["dim1"], shape=[5, 1, 1], dtype=dtype)
        dim2 = Tensor(data=g["dim2"], shape=[1, 4, 1], dtype=dtype)
        dim3 = Tensor(data=g["dim3"], shape=[1, 1, 6], dtype=dtype)
        clamped = dim1.clamp(min=dim2, max=dim3)
        assert clamped.shape == [5, 4, 6]
        assertDataEqual(clamped, g["out"])
        a = Tensor(data=[1, 2, 3, 4, 5], shape=[5, 1], dtype=dtype)
        b = Tensor(data=[1, 2, 3], shape=[1, 3], dtype=dtype)
        assertClose(a.clamp(min=b, max=4), g["tensor_scalar_out"])
    x = Tensor(data=[1.0, 2.0, 3.0])
    assertDataEqual(x.clamp(min=10, max=-3), [-3, -3, -3])
    assertDataEqual(x.clamp(min=10, max=Tensor(data=[-3.0, -3.0, -3.0])), [-3, -3, -3])
    assertDataEqual(x.clamp(min=2), [2, 2, 3])
    assertDataEqual(x.clamp(max=2), [1, 2, 2])


def testAdam():
    """BackendTests.swift:1779-1797: three AdamW steps (lr 1, beta1 0.25, beta2 0.5, decay 0.1) on
    a three-element parameter, moments starting at zero and the step counter at 1
    (Optimizer.swift:129-152)."""
    from honeycrisp_amd.backend import Backend
    g = GOLDEN["adam"]
    backend = Backend.current()
    for dtype in (F16, F32):
        tol = 0.01 if dtype == F16 else 0.0001
        param = Tensor(data=g["param"], dtype=dtype)
        m1 = Tensor.zeros([3], dtype=dtype)
        m2 = Tensor.zeros([3], dtype=dtype)
        for t, (grad, want) in enumerate(zip(g["grads"], g["expected"]), start=1):
            gradT = Tensor(data=grad, dtype=dtype)
            p, a, b = backend.adamW(param.data, gradT.data, m1.data, m2.data, g["beta1"], g["beta2"], g["eps"],
                                    g["weightDecay"], g["lr"], float(t), 3, dtype)
            param, m1, m2 = (Tensor(dataHandle=d, shape=[3], dtype=dtype) for d in (p, a, b))
            assertClose(param, want, atol=tol, rtol=tol)


def testNormalizeGrad(rng):
    """Backend.normalizeGrad (Backend.swift:332-455) against central differences of normalize
    in float64 arithmetic (numpy): the analytic gradient of (x - mean) / sqrt(var + eps)."""
    from honeycrisp_amd.backend import Backend
    backend = Backend.current()
    x = rng.standard_normal((5, 7, 3)).astype(np.float32)
    og = rng.standard_normal((5, 7, 3)).astype(np.float32)
    eps = 1e-3
    xt, ogt = Tensor(data=x), Tensor(data=og)
    data = backend.normalizeGrad(xt.data, ogt.data, xt.reduceDims(1), np.float32(eps), F32)
    got = np.asarray(Tensor(dataHandle=data, shape=[5, 7, 3], dtype=F32).floats()).reshape(5, 7, 3)
    x64, og64 = x.astype(np.float64), og.astype(np.float64)
    mean = x64.mean(1, keepdims=True)
    c = x64 - mean
    var = (c * c).mean(1, keepdims=True)
    inv = (var + eps) ** -0.5
    cg = og64 - og64.mean(1, keepdims=True)
    want = cg * inv - c * (c * og64).sum(1, keepdims=True) * (var + eps) ** -1.5 / 7
    assert_close_arrays(got, want, 1e-4, 1e-4)


def testProd(rng):
    """BackendTests.swift:436-465 (forward values): a product over positive inputs equals
    exp(sum(log x)); signs."""
    raw = Tensor(data=(rng.random((3, 4, 5)) + 0.5).astype(np.float32))
    for axis in range(3):
        expected = raw.log().sum(axis=axis).exp()
        for dtype in (F16, F32):
            tol = 1e-4 if dtype == F32 else 1e-2
            assertClose(expected, raw.cast(dtype).prod(axis=axis).cast(F32), atol=tol, rtol=tol)
    x = Tensor(data=[2.0, -3.0, 4.0, 2.0, -3.0, -4.0], shape=[2, 3])
    for dtype in (F16, F32, I64):
        assertDataEqual(x.cast(dtype).prod(axis=0), [4.0, 9.0, -16.0])
        assertDataEqual(x.cast(dtype).prod(axis=1), [-24.0, 24.0])


def testRepeat():
    """BackendTests.swift:566-583: repeating along an axis; its gradient is the sum over the
    copies (flatApplySums of the inverse RepeatDims, ReduceRepeat.swift:283-305)."""
    x = Tensor(data=[1.0, 2.0, 3.0, -2.0, 3.0, 7.0], shape=[1, 2, 3, 1])
    repeated = x.repeating(axis=2, count=2)
    assert repeated.shape == [1, 2, 6, 1]
    assertDataEqual(repeated, [1.0, 2.0, 3.0, 1.0, 2.0, 3.0, -2.0, 3.0, 7.0, -2.0, 3.0, 7.0])
    grad = Tensor(data=[float(i) for i in range(1, 13)], shape=[1, 2, 6, 1])
    assertDataEqual(grad.reshape([2, 2, 3]).sum(axis=1), [5.0, 7.0, 9.0, 17.0, 19.0, 21.0])


def testAllSome():
    """BackendTests.swift:1364-1425."""
    def checkEqual(t1, t2):
        assert t1.shape == t2.shape and t1.dtype == t2.dtype
        assertDataEqual(t1, t2)

    bits = [False, True, False, False, True, True, True, False]
    checkEqual(Tensor(data=bits, shape=[4, 2]).all(axis=1), Tensor(data=[False, False, True, False], shape=[4]))
    checkEqual(Tensor(data=bits, shape=[4, 2]).all(axis=1, keepdims=True),
               Tensor(data=[False, False, True, False], shape=[4, 1]))
    checkEqual(Tensor(data=bits, shape=[4, 2]).some(axis=1), Tensor(data=[True, False, True, True], shape=[4]))
    checkEqual(Tensor(data=bits, shape=[4, 2]).some(axis=1, keepdims=True),
               Tensor(data=[True, False, True, True], shape=[4, 1]))
    empty = lambda: Tensor(data=[], shape=[4, 0], dtype=BOOL)
    none = lambda shape: Tensor(data=[], shape=shape, dtype=BOOL)
    for fn, unit in ((Tensor.all, True), (Tensor.some, False)):
        checkEqual(fn(empty()), Tensor(data=[unit], shape=[]))
        checkEqual(fn(empty(), keepdims=True), Tensor(data=[unit], shape=[1, 1]))
        checkEqual(fn(empty(), axis=1), Tensor(data=[unit] * 4, shape=[4]))
        checkEqual(fn(empty(), axis=1, keepdims=True), Tensor(data=[unit] * 4, shape=[4, 1]))
        checkEqual(fn(empty(), axis=0), none([0]))
        checkEqual(fn(empty(), axis=0, keepdims=True), none([1, 0]))


def testConcatInner():
    """BackendTests.swift:1629-1642; the gradients of a concatenation are the matching slices of
    the output gradient (ConcatSplit.swift)."""
    x = Tensor(data=[1, 2, 3, 4, 5, 6], shape=[2, 3]).cast(F32)
    y = Tensor(data=[7, 8, 9, 10], shape=[2, 2]).cast(F32)
    combined = Tensor.concat([x, y], axis=1)
    assert combined.shape == [2, 5]
    assertDataEqual(combined, [1, 2, 3, 7, 8, 4, 5, 6, 9, 10])
    grad = Tensor(data=[1, 2, 3, 4, 5, 6, 7, 8, 9, 10], shape=[2, 5]).cast(F32)
    assertDataEqual(grad[:, 0:3], [1, 2, 3, 6, 7, 8])
    assertDataEqual(grad[:, 3:5], [4, 5, 9, 10])


def testConcatOuter():
    """BackendTests.swift:1644-1657."""
    x = Tensor(data=[1, 2, 3, 4, 5, 6], shape=[2, 3]).cast(F32)
    y = Tensor(data=[7, 8, 9], shape=[1, 3]).cast(F32)
    combined = Tensor.concat([x, y], axis=0)
    assert combined.shape == [3, 3]
    assertDataEqual(combined, [1, 2, 3, 4, 5, 6, 7, 8, 9])
    grad = Tensor(data=[1, 2, 3, 4, 5, 6, 7, 8, 9], shape=[3, 3]).cast(F32)
    assertDataEqual(grad[0:2], [1, 2, 3, 4, 5, 6])
    assertDataEqual(grad[2:3], [7, 8, 9])


def testConcat():
    """Concatenation along an inner and an outer axis (Tensor(concat:), ConcatSplit.swift:4-75;
    CPU loop BackendCPU.swift:1768-1794); expected values follow from the definition."""
    x = Tensor(data=[1, 2, 3, 4, 5, 6], shape=[2, 3]).cast(F32)
    y = Tensor(data=[-1, -2, -3, -4], shape=[2, 2]).cast(F32)
    assertDataEqual(Tensor.concat([x, y], axis=1), [1, 2, 3, -1, -2, 4, 5, 6, -3, -4])
    z = Tensor(data=[7, 8, 9], shape=[1, 3]).cast(F32)
    assertDataEqual(Tensor.concat([x, z], axis=0), [1, 2, 3, 4, 5, 6, 7, 8, 9])


def testWhen(rng):
    """BackendTests.swift:1659-1755: values, the gradients (mask.when(grad, 0) / mask.when(0, grad),
    When.swift), pure scalar branches, and implicit == explicit broadcasting over every pairing of
    the three shapes with tensor and scalar branches."""
    x = Tensor(data=[1.0, 2.0, 3.0, 4.0], shape=[4])
    y = Tensor(data=[-1.0, -2.0, -3.0, -4.0], shape=[4])
    mask = Tensor(data=[False, True, True, False], shape=[4])
    assertDataEqual(mask.when(x, y), [-1.0, 2.0, 3.0, -4.0])
    grad = Tensor(data=[5.0, 6.0, 7.0, 8.0], shape=[4])
    assertDataEqual(mask.when(grad, 0.0), [0, 6.0, 7.0, 0.0])
    assertDataEqual(mask.when(0.0, grad), [5.0, 0.0, 0.0, 8.0])
    assertDataEqual(mask.when(1.0, -1.0, dtype=F32), [-1, 1, 1, -1])
    shapes = [[1, 6, 1], [3, 6, 2], [3, 1, 2]]
    for maskShape in shapes:
        m = Tensor(data=rng.random(maskShape).astype(np.float32)) < 0.5
        for trueShape in shapes:
            t = Tensor(data=rng.random(trueShape).astype(np.float32))
            for falseShape in shapes:
                f = Tensor(data=rng.random(falseShape).astype(np.float32))
                b = Tensor.broadcast([m, t, f])
                assertDataEqual(m.when(t, f), b[0].when(b[1], b[2]))
                b = Tensor.broadcast([m, t])
                assertDataEqual(m.when(t, 3.1415), b[0].when(b[1], 3.1415))
                b = Tensor.broadcast([m, f])
                assertDataEqual(m.when(3.1415, f), b[0].when(3.1415, b[1]))


def testChunk():
    """BackendTests.swift:1031-1048."""
    for i in range(1, 10):
        for count in range(1, i + 1):
            if i % count != 0:
                continue
            parts = Tensor(data=range(i)).chunk(axis=0, count=count)
            assert len(parts) == count
            assert all(p.shape[0] == parts[0].shape[0] for p in parts)
            assertDataEqual(Tensor.concat(parts, axis=0), [float(v) for v in range(i)])


def testOneHot():
    """BackendTests.swift:1757-1760."""
    assertDataEqual(Tensor.oneHot(3, count=5), [0, 0, 0, 1, 0])
    assertDataEqual(Tensor.oneHot([3, 1], count=5), [0, 0, 0, 1, 0, 0, 1, 0, 0, 0])


def testWhenForms():
    """When.swift semantics: mask ? a : b with tensor / scalar branches, broadcasting."""
    mask = Tensor(data=[1, 0, 1, 0, 0, 1], shape=[2, 3]).cast(BOOL)
    a = Tensor(data=[1.0, 2.0, 3.0], shape=[3])
    b = Tensor(data=[-1.0, -2.0], shape=[2, 1])
    assertDataEqual(mask.when(a, b), [1, -1, 3, -2, -2, 3])
    assertDataEqual(mask.when(a, 0.5), [1, 0.5, 3, 0.5, 0.5, 3])
    assertDataEqual(mask.when(7, b.cast(I64)), [7, -1, 7, -2, -2, 7])
    out = mask.when(0, -1e4, dtype=F16)
    assert out.dtype == F16
    assertDataEqual(out, [0, -1e4, 0, -1e4, -1e4, 0])


ALL_CASES = [
    testCreateFromData, testCast, testAdd, testSub, testMul, testDiv, testFusedAddMul, testFusedNormalize,
    testMod, testEquals, testComparison, testSum, testGather, testGatherBroadcastOtherAxis,
    testMatrixMatrixProduct, testBatchedMatmul, testMatrixVectorProduct, testTriangular, testIndexing,
    testElemwise, testRounding, testMinMax, testExpandAndRepeat, testBinaryBroadcast, testFusedBroadcast,
    testSoftmax, testConcat, testWhen, testCumulativeSum, testCumulativeProd, testArgsort, testBitwise, testSoftmaxGrad, testScatter, testScatterIsAdjointOfGather, testClamp,
    testAdam, testNormalizeGrad, testProd, testRepeat, testAllSome, testConcatInner, testConcatOuter,
    testWhenForms, testChunk, testOneHot,
]
