"""The ragged-shape sweep M, K, N in {127, 1000, 4097} of the fp16 GEMM workload, all 27 shapes, and
the products that the host splits into a multiple-of-256 body plus thin fringes (extents 1..32 over
a multiple of 256, K >= 2048): straight through hc_matmul (the C ABI), every storage layout.

What is compared, per product:
  * row slabs (first / middle / last rows, the last ones being the fringe rows) x all columns and
    all rows x column slabs (first / last columns: the fringe columns) against the CPU oracle
    (BackendCPU.swift:1260-1304 restated), tolerance 1e-2 (fp16) / 1e-4 (fp32);
  * the whole result against the general kernel (HCHIP_GEMM_TILE=general: no tuned tile, no split),
    against the same call with HCHIP_GEMM_NO_PEEL=1 (tuned tiles, no split) and against the same call
    with HCHIP_GEMM_NO_DIRECT=1 (rows that are not 16-byte aligned go through zero-padded copies
    instead of being fetched and stored where they lie);
  * guard elements in front of and behind the output: nothing may be written outside C.
"""
from ctypes import c_void_p

import numpy as np
import pytest

from honeycrisp_amd.descriptors import DType
from honeycrisp_amd.tensor import Tensor
from backend_cases import assert_close_arrays

pytestmark = pytest.mark.gpu

F32, F16 = DType.float32, DType.float16
TOL = {F32: 1e-4, F16: 1e-2}
GUARD = 64  # elements on either side of C (a multiple of 16 bytes: C keeps its natural alignment)


def slabs(n, width=8):
    """First, middle and last `width` indices of range(n), without repeats."""
    idx = np.r_[0:min(width, n), max(n // 2 - width // 2, 0):min(n // 2 + width // 2, n), max(n - width, 0):n]
    return np.unique(idx)


class Product:
    """One product A[batch, M, K] x B[batch, K, N] with its operands on the device in both storage
    orders and oracle values for row and column slabs of C."""

    def __init__(self, hip, oracle, dtype, batch, M, K, N, seed):
        rng = np.random.default_rng(seed)
        self.hip, self.dtype, self.batch, self.M, self.K, self.N = hip, dtype, batch, M, K, N
        np_t = dtype.numpy
        a = (rng.standard_normal((batch, M, K)) / np.sqrt(K)).astype(np_t)
        b = rng.standard_normal((batch, K, N)).astype(np_t)
        self.rows, self.cols = slabs(M), slabs(N)
        with oracle.use():
            self.want_rows = Tensor.batchedMatmul(Tensor(data=np.ascontiguousarray(a[:, self.rows])), False,
                                                  Tensor(data=b), False, False).numpy()
            self.want_cols = Tensor.batchedMatmul(Tensor(data=a), False,
                                                  Tensor(data=np.ascontiguousarray(b[:, :, self.cols])), False,
                                                  False).numpy()
        self.dev = {("a", False): hip.upload(a), ("a", True): hip.upload(np.ascontiguousarray(a.transpose(0, 2, 1))),
                    ("b", False): hip.upload(b), ("b", True): hip.upload(np.ascontiguousarray(b.transpose(0, 2, 1)))}
        self.guard = rng.standard_normal(batch * M * N + 2 * GUARD).astype(np_t)
        self.guard_dev = hip.upload(self.guard)

    def run(self, transA, transB, transOut):
        """C as [batch, M, N] (a transposed output is transposed back on the host)."""
        hip, es = self.hip, np.dtype(self.dtype.numpy).itemsize
        n_out = self.batch * self.M * self.N
        out = hip.allocate(self.guard.nbytes)
        hip._check(hip._lib.hc_memcpy_d2d(hip._ctx, c_void_p(out.ptr), c_void_p(self.guard_dev.ptr), self.guard.nbytes))
        hip._check(hip._lib.hc_matmul(hip._ctx, int(self.dtype), self.batch, c_void_p(self.dev[("a", transA)].ptr),
                                      int(transA), c_void_p(self.dev[("b", transB)].ptr), int(transB), int(transOut),
                                      self.M, self.K, self.N, c_void_p(out.ptr + GUARD * es)))
        host = out.onCPU().view(self.dtype.numpy)
        bits = np.uint16 if self.dtype is F16 else np.uint32
        assert np.array_equal(host[:GUARD].view(bits), self.guard[:GUARD].view(bits)), "wrote in front of C"
        assert np.array_equal(host[GUARD + n_out:].view(bits), self.guard[GUARD + n_out:].view(bits)), "wrote behind C"
        c = host[GUARD:GUARD + n_out]
        if transOut:
            return c.reshape(self.batch, self.N, self.M).transpose(0, 2, 1)
        return c.reshape(self.batch, self.M, self.N)

    def check_against_oracle(self, c):
        tol = TOL[self.dtype]
        assert_close_arrays(np.ascontiguousarray(c[:, self.rows]), self.want_rows, tol, tol)
        assert_close_arrays(np.ascontiguousarray(c[:, :, self.cols]), self.want_cols, tol, tol)
        scale = float(np.max(np.abs(self.want_rows.astype(np.float64))))
        err = float(np.max(np.abs(c[:, self.rows].astype(np.float64) - self.want_rows.astype(np.float64))))
        assert err <= tol * scale

    def check_all(self, layouts, label):
        tol = TOL[self.dtype]
        with self.hip.switches(HCHIP_GEMM_TILE="general"):
            general = self.run(False, False, False)
        self.check_against_oracle(general)
        for (transA, transB, transOut) in layouts:
            print(label, self.dtype.name, self.batch, self.M, self.K, self.N, transA, transB, transOut, flush=True)
            c = self.run(transA, transB, transOut)
            self.check_against_oracle(c)
            assert_close_arrays(np.ascontiguousarray(c), general, tol, tol)
            with self.hip.switches(HCHIP_GEMM_NO_PEEL="1"):
                whole = self.run(transA, transB, transOut)
            assert_close_arrays(np.ascontiguousarray(c), np.ascontiguousarray(whole), tol, tol)
            with self.hip.switches(HCHIP_GEMM_NO_DIRECT="1"):
                padded = self.run(transA, transB, transOut)
            assert_close_arrays(np.ascontiguousarray(c), np.ascontiguousarray(padded), tol, tol)


ALL_LAYOUTS = [(ta, tb, to) for to in (False, True) for ta in (False, True) for tb in (False, True)]
FOUR_LAYOUTS = [(ta, tb, False) for ta in (False, True) for tb in (False, True)]
SWEEP = [(m, k, n) for m in (127, 1000, 4097) for k in (127, 1000, 4097) for n in (127, 1000, 4097)]


@pytest.mark.parametrize("shape", SWEEP, ids=lambda s: "x".join(map(str, s)))
def test_ragged_sweep_fp16(hip_backend, oracle_backend, shape):
    """All 27 shapes of the sweep in the four storage layouts; the cubes and the three shapes that
    are split into body and fringes (4097^3, 4097 x 4097 x 1000, 1000 x 4097 x 4097 as M x K x N)
    also with a transposed output."""
    M, K, N = shape
    peeled = K == 4097 and ((M == 4097 and N >= 1000) or (N == 4097 and M >= 1000))
    layouts = ALL_LAYOUTS if (M == K == N or peeled) else FOUR_LAYOUTS
    Product(hip_backend, oracle_backend, F16, 1, M, K, N, seed=M * 7 + K * 3 + N).check_all(layouts, "sweep")


# (batch, M, K, N): extents 1..32 over a multiple of 256 with K >= 2048. Fringes of 1..4 rows or
# columns run on the skinny kernels, 5..32 on 64 x 64 edge tiles. 16-byte aligned rows need no
# padded copies (sub-blocks of the caller's own buffers); odd extents go through them.
PEEL_SHAPES = [(1, 4104, 4096, 4112), (1, 4128, 2048, 2056), (1, 4097, 2048, 4100), (2, 2050, 2304, 4128),
               (1, 2056, 4100, 2049), (3, 2052, 2048, 2080)]


@pytest.mark.parametrize("dtype", [F16, F32], ids=["f16", "f32"])
@pytest.mark.parametrize("shape", PEEL_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_body_plus_fringes(hip_backend, oracle_backend, dtype, shape):
    batch, M, K, N = shape
    Product(hip_backend, oracle_backend, dtype, batch, M, K, N, seed=batch + M + K + N).check_all(ALL_LAYOUTS, "peel")


# Rows that are not a whole number of 16-byte pieces, fetched where they lie: the piece that
# straddles the end of a row also holds the first elements of the next row. (M, K, N); K or N odd.
LOOSE_SHAPES = [(130, 127, 72), (66, 1001, 257), (300, 71, 129), (64, 8, 127), (257, 3, 1000), (1000, 4097, 135)]


@pytest.mark.parametrize("dtype", [F16, F32], ids=["f16", "f32"])
@pytest.mark.parametrize("shape", LOOSE_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_neighbouring_rows_do_not_leak(hip_backend, dtype, shape):
    """Every other row of A (and of B^T) is infinite. A finite row's last piece reaches into its
    infinite neighbour, so anything that leaks across the end of a row turns finite outputs into
    NaN; they must match a float64 product of the finite rows, and the others must not be finite."""
    M, K, N = shape
    rng = np.random.default_rng(M + K + N)
    np_t = dtype.numpy
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np_t)
    b = rng.standard_normal((K, N)).astype(np_t)
    want = a.astype(np.float64) @ b.astype(np.float64)
    tol = TOL[dtype]
    hip = hip_backend

    def product(a_host, trans_a, b_host, trans_b):
        da = hip.upload(np.ascontiguousarray(a_host.T if trans_a else a_host))
        db = hip.upload(np.ascontiguousarray(b_host.T if trans_b else b_host))
        out = hip.allocate(M * N * np.dtype(np_t).itemsize)
        hip._check(hip._lib.hc_matmul(hip._ctx, int(dtype), 1, c_void_p(da.ptr), int(trans_a), c_void_p(db.ptr),
                                      int(trans_b), 0, M, K, N, c_void_p(out.ptr)))
        return out.onCPU().view(np_t)[:M * N].reshape(M, N).astype(np.float64)

    # infinite rows of A (stored [M, K], K-contiguous): the odd m
    a_inf = a.copy()
    a_inf[1::2] = np.inf
    for trans_b in (False, True):
        print("rows of A", dtype.name, shape, trans_b, flush=True)
        c = product(a_inf, False, b, trans_b)
        assert np.all(np.isfinite(c[0::2])), "an infinite neighbouring row of A leaked into a finite one"
        assert not np.any(np.isfinite(c[1::2]))
        assert_close_arrays(c[0::2], want[0::2], tol, tol)
    # infinite rows of B^T (stored [N, K], K-contiguous): the odd n
    b_inf = b.copy()
    b_inf[:, 1::2] = np.inf
    for trans_a in (False, True):
        print("rows of B^T", dtype.name, shape, trans_a, flush=True)
        c = product(a, trans_a, b_inf, True)
        assert np.all(np.isfinite(c[:, 0::2])), "an infinite neighbouring row of B^T leaked into a finite one"
        assert not np.any(np.isfinite(c[:, 1::2]))
        assert_close_arrays(c[:, 0::2], want[:, 0::2], tol, tol)


@pytest.mark.parametrize("dtype", [F16, F32], ids=["f16", "f32"])
def test_operand_that_fills_its_block(hip_backend, oracle_backend, dtype):
    """Operands whose bytes are exactly a block of the allocator (a power of two) leave no room
    behind the last row for the last piece's 16 bytes: such products go through padded copies."""
    es = np.dtype(dtype.numpy).itemsize
    K = 8 // es          # rows of 8 bytes: half a piece
    M = 4096 // (K * es)  # A = 4096 bytes
    N = 4096 // (K * es)  # B^T = 4096 bytes
    rng = np.random.default_rng(5)
    a = rng.standard_normal((M, K)).astype(dtype.numpy)
    bt = rng.standard_normal((N, K)).astype(dtype.numpy)
    with oracle_backend.use():
        want = Tensor.batchedMatmul(Tensor(data=a[None]), False, Tensor(data=bt[None]), True, False).numpy()[0]
    hip = hip_backend
    da, db = hip.upload(a), hip.upload(bt)
    out = hip.allocate(M * N * es)
    hip._check(hip._lib.hc_matmul(hip._ctx, int(dtype), 1, c_void_p(da.ptr), 0, c_void_p(db.ptr), 1, 0, M, K, N,
                                  c_void_p(out.ptr)))
    got = out.onCPU().view(dtype.numpy)[:M * N].reshape(M, N)
    assert_close_arrays(got, want, TOL[dtype], TOL[dtype])


def test_random_products_with_infinite_surroundings(hip_backend):
    """Seeded random extents (around the piece, wave and tile sizes, a few long K), dtypes, batches
    and flags; operands and output start at random element offsets inside their buffers, the
    elements in front of and behind each operand are infinite, the output's surroundings are
    checked bit for bit. Whatever a kernel fetches beyond an operand's rows (the last 16-byte piece
    of the last row reaches into the infinities) must not reach the result."""
    hip = hip_backend
    rng = np.random.default_rng(31)
    dims = [1, 2, 3, 5, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 100, 127, 129, 191, 200, 255, 257, 264, 320, 383, 500, 513,
            640, 1000, 1023, 1025]
    for case in range(160):
        dtype = F16 if rng.integers(0, 3) else F32
        np_t = dtype.numpy
        es = np.dtype(np_t).itemsize
        bits = np.uint16 if es == 2 else np.uint32
        M, K, N = (int(rng.choice(dims)) for _ in range(3))
        if case % 11 == 0:
            K = int(rng.choice([1500, 2050, 2304, 4097]))
        if case % 13 == 0:
            M, N = int(rng.choice([2049, 2052, 2080])), int(rng.choice([1024, 2049, 1000]))
        batch = int(rng.choice([1, 1, 1, 2, 3]))
        ta, tb, to = (bool(rng.integers(0, 2)) for _ in range(3))
        offa, offb, offc = (int(rng.integers(0, 9)) for _ in range(3))
        a = (rng.standard_normal((batch, M, K)) / np.sqrt(K)).astype(np_t)
        b = rng.standard_normal((batch, K, N)).astype(np_t)
        sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if ta else a
        sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if tb else b
        abuf = np.full(offa + sa.size + 16, np.inf, np_t)
        abuf[offa:offa + sa.size] = sa.reshape(-1)
        bbuf = np.full(offb + sb.size + 16, np.inf, np_t)
        bbuf[offb:offb + sb.size] = sb.reshape(-1)
        cbuf = rng.standard_normal(offc + batch * M * N + 16).astype(np_t)
        da, db, dc = hip.upload(abuf), hip.upload(bbuf), hip.upload(cbuf)
        print("case", case, dtype.name, batch, M, K, N, ta, tb, to, offa, offb, offc, flush=True)
        hip._check(hip._lib.hc_matmul(hip._ctx, int(dtype), batch, c_void_p(da.ptr + offa * es), int(ta),
                                      c_void_p(db.ptr + offb * es), int(tb), int(to), M, K, N, c_void_p(dc.ptr + offc * es)))
        host = dc.onCPU().view(np_t)[:cbuf.size]
        n_out = batch * M * N
        assert np.array_equal(host[:offc].view(bits), cbuf[:offc].view(bits)), "wrote in front of C"
        assert np.array_equal(host[offc + n_out:].view(bits), cbuf[offc + n_out:].view(bits)), "wrote behind C"
        c = host[offc:offc + n_out].astype(np.float64)
        c = c.reshape(batch, N, M).transpose(0, 2, 1) if to else c.reshape(batch, M, N)
        want = a.astype(np.float64) @ b.astype(np.float64)
        assert np.all(np.isfinite(c)), "something outside the operands reached the result"
        tol = TOL[dtype]
        assert float(np.max(np.abs(c - want))) <= 1.5 * tol * max(float(np.max(np.abs(want))), 1e-30)
