"""Parity proper: the HIP path (through the C ABI) against the CPU oracle on the same seeded
inputs. Bit-exact for integer / index / data-movement work and for element-wise fp32
arithmetic that involves no libm call; otherwise the reference's own criterion
(|a-b| <= tol or |a/b-1| <= tol, Assertions.swift:16) with tol 1e-4 for fp32 and 1e-2 for
fp16, plus a norm-wise bound for GEMMs."""
import os

import numpy as np
import pytest

from honeycrisp_amd.descriptors import DType, ElemwiseOp, ReduceDims, ReduceOp
from honeycrisp_amd.tensor import Tensor
from backend_cases import assert_close_arrays

pytestmark = pytest.mark.gpu

F32, F16, I64, BOOL = DType.float32, DType.float16, DType.int64, DType.bool
TOL = {F32: 1e-4, F16: 1e-2}


def both(hip, oracle, fn):
    """Run fn() under each backend; returns (hip result, oracle result) as numpy arrays."""
    with hip.use():
        got = fn().numpy()
    with oracle.use():
        want = fn().numpy()
    return got, want


def check_exact(hip, oracle, fn):
    got, want = both(hip, oracle, fn)
    assert got.dtype == want.dtype and got.shape == want.shape
    if got.dtype.kind == "f":
        # same bits, except that any NaN matches any NaN
        bits = {2: np.uint16, 4: np.uint32}[got.dtype.itemsize]
        differ = (got.view(bits) != want.view(bits)) & ~(np.isnan(got) & np.isnan(want))
    else:
        differ = got != want
    if differ.any():
        i = np.argwhere(differ)[0]
        raise AssertionError("%d of %d elements differ; first at %s: got %r want %r" %
                             (int(differ.sum()), got.size, tuple(i), got[tuple(i)], want[tuple(i)]))


def check_close(hip, oracle, fn, tol):
    got, want = both(hip, oracle, fn)
    assert got.dtype == want.dtype and got.shape == want.shape
    assert_close_arrays(got, want, tol, tol)
    return got, want


def rand(rng, shape, dtype, scale=1.0):
    if dtype == I64:
        return rng.integers(-50, 50, size=shape)
    return (rng.standard_normal(shape) * scale).astype(dtype.numpy)


# ---------------------------------------------------------------- matmul

GEMM_SHAPES = [(128, 128, 128), (256, 64, 384), (127, 1000, 65), (1, 33, 1), (5, 4097, 3), (200, 8, 136),
               (64, 0, 16), (129, 257, 131), (512, 192, 384), (1024, 64, 2048), (256, 320, 128),
               # 16-byte aligned rows but ragged against every tile and K-slice: the edge kernels
               (264, 72, 520), (1000, 1000, 1000), (8, 64, 8), (2040, 520, 1000),
               # odd extents, large enough to be re-pitched into aligned copies first
               (1001, 515, 999), (4097, 127, 1000), (333, 4097, 129)]


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape", GEMM_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_matmul_all_flag_combinations(hip_backend, oracle_backend, dtype, shape):
    M, K, N = shape
    rng = np.random.default_rng(100 + M + K + N)
    a = rand(rng, (M, K), dtype, 1.0 / max(K, 1) ** 0.5)
    b = rand(rng, (K, N), dtype)
    for transA in (False, True):
        for transB in (False, True):
            for transOut in (False, True):
                print("matmul", dtype.name, shape, transA, transB, transOut, flush=True)
                sa = np.ascontiguousarray(a.T) if transA else a
                sb = np.ascontiguousarray(b.T) if transB else b
                fn = lambda: Tensor.matmul(Tensor(data=sa), transA, Tensor(data=sb), transB, transOut)
                got, want = check_close(hip_backend, oracle_backend, fn, TOL[dtype])
                scale = float(np.max(np.abs(want.astype(np.float64)))) if want.size else 0.0
                if scale > 0:
                    err = float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))))
                    assert err / scale <= TOL[dtype]


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_batched_matmul_attention_shapes(hip_backend, oracle_backend, dtype):
    """Config 3: batch 32, Q[512,64] x K^T -> [512,512], scale 1/8, then scores x V[512,64]."""
    rng = np.random.default_rng(4)
    q = rand(rng, (32, 512, 64), dtype)
    k = rand(rng, (32, 512, 64), dtype)
    v = rand(rng, (32, 512, 64), dtype)

    def fn():
        scores = Tensor.batchedMatmul(Tensor(data=q), False, Tensor(data=k), True, False) * 0.125
        return Tensor.batchedMatmul(scores.softmax(), False, Tensor(data=v), False, False)

    def scores_fn():
        return Tensor.batchedMatmul(Tensor(data=q), False, Tensor(data=k), True, False) * 0.125

    check_close(hip_backend, oracle_backend, scores_fn, TOL[dtype])
    check_close(hip_backend, oracle_backend, fn, TOL[dtype])


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
@pytest.mark.parametrize("batch", [8, 12, 20, 33])
def test_batched_matmul_slices_in_groups_of_eight(hip_backend, oracle_backend, dtype, batch):
    """Small batched products (at most 8 blocks per slice, 8 slices or more) hand the blocks of a slice to
    workgroups 8 apart so that a slice runs on one XCD; slices beyond the last whole group of 8 keep the
    launch order. Every slice must still get its own operands, whatever the batch count leaves over."""
    rng = np.random.default_rng(batch)
    # every slice scaled differently: a block that took another slice's operands cannot pass
    scale = (1.0 + np.arange(batch, dtype=np.float32))[:, None, None]
    for m, k, n in ((128, 64, 64), (256, 192, 64), (64, 64, 128), (130, 72, 60)):
        a = (rand(rng, (batch, m, k), F32) * scale / np.sqrt(k)).astype(dtype.numpy)
        b = rand(rng, (batch, k, n), dtype)
        fn = lambda: Tensor.batchedMatmul(Tensor(data=a), False, Tensor(data=b), False, False)
        check_close(hip_backend, oracle_backend, fn, TOL[dtype])
        bt = np.ascontiguousarray(np.swapaxes(b, 1, 2))
        fn = lambda: Tensor.batchedMatmul(Tensor(data=a), False, Tensor(data=bt), True, False)
        check_close(hip_backend, oracle_backend, fn, TOL[dtype])


def test_batched_matmul_all_flags_small(hip_backend, oracle_backend):
    rng = np.random.default_rng(5)
    for dtype in (F32, F16):
        a = rand(rng, (7, 24, 40), dtype)
        b = rand(rng, (7, 40, 56), dtype)
        for transA in (False, True):
            for transB in (False, True):
                for transOut in (False, True):
                    sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if transA else a
                    sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if transB else b
                    fn = lambda: Tensor.batchedMatmul(Tensor(data=sa), transA, Tensor(data=sb), transB, transOut)
                    check_close(hip_backend, oracle_backend, fn, TOL[dtype])


@pytest.mark.parametrize("pipeline", ["dma", "dma2", "mi16"])
@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_matmul_both_pipelines_every_tile(hip_backend, oracle_backend, switch, pipeline, dtype):
    """The host picks a direct-to-LDS pipeline and a tile by problem size; here every tile of both
    pipelines is forced in turn (the library reads the two variables at every call) on whole-tile,
    ragged (edge kernels: clamped rows, zero-filled K tail) and batched problems, all four layouts."""
    rng = np.random.default_rng(77)
    switch.setenv("HCHIP_GEMM_KERNEL", pipeline)
    tiles = ("256x256", "256x128", "128x128", "256x64", "128x64", "64x64")
    if (pipeline == "mi16" and dtype is F16) or (pipeline == "dma2" and dtype is F32):
        tiles += ("256x192", "192x256", "192x192")  # (extents that are not powers of two: these pipelines only)
    for tile in tiles:
        switch.setenv("HCHIP_GEMM_TILE", tile)
        shapes = [(1, 256, 192, 256), (2, 264, 200, 136), (3, 128, 1024, 64)]
        if "192" in tile:
            shapes.append((1, 768, 320, 768))  # whole tiles of every 192-extent shape
        for (batch, M, K, N) in shapes:
            a = rand(rng, (batch, M, K), dtype, 1.0 / K ** 0.5)
            b = rand(rng, (batch, K, N), dtype)
            for transA in (False, True):
                for transB in (False, True):
                    sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if transA else a
                    sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if transB else b
                    print("matmul", pipeline, tile, dtype.name, batch, M, K, N, transA, transB, flush=True)
                    fn = lambda: Tensor.batchedMatmul(Tensor(data=sa), transA, Tensor(data=sb), transB, False)
                    got, want = check_close(hip_backend, oracle_backend, fn, TOL[dtype])
                    scale = float(np.max(np.abs(want.astype(np.float64))))
                    assert float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) <= TOL[dtype] * scale


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_matmul_single_slice_variant(hip_backend, oracle_backend, switch, dtype):
    """Products whose whole K is one 128-byte slice (attention scores over 64-wide heads) run a
    variant of the two-stage kernels that fetches once and uses one stage of LDS. Every tile that
    has it, the layouts with a K-contiguous operand, whole and ragged extents, short and odd K,
    batches: against the oracle, and bit for bit against the general loop (HCHIP_GEMM_ONE=0)."""
    rng = np.random.default_rng(123)
    slice_k = 64 if dtype is F16 else 32
    bits = np.uint16 if dtype is F16 else np.uint32
    for tile in ("256x128", "128x128", "128x64", "64x64"):
        switch.setenv("HCHIP_GEMM_TILE", tile)
        for K in (slice_k, slice_k - 24, slice_k // 2 + 1, 8, 1):
            for (batch, M, N) in ((1, 256, 128), (3, 512, 512), (2, 200, 72), (1, 67, 129)):
                a = rand(rng, (batch, M, K), dtype, 1.0 / K ** 0.5)
                b = rand(rng, (batch, K, N), dtype)
                for transA, transB in ((False, False), (False, True), (True, True)):
                    sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if transA else a
                    sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if transB else b
                    print("single slice", tile, dtype.name, batch, M, K, N, transA, transB, flush=True)
                    fn = lambda: Tensor.batchedMatmul(Tensor(data=sa), transA, Tensor(data=sb), transB, False)
                    got, want = check_close(hip_backend, oracle_backend, fn, TOL[dtype])
                    switch.setenv("HCHIP_GEMM_ONE", "0")
                    with hip_backend.use():
                        loop = fn().numpy()
                    switch.delenv("HCHIP_GEMM_ONE")
                    assert np.array_equal(np.ascontiguousarray(got).view(bits), np.ascontiguousarray(loop).view(bits))


def test_matmul_ring_of_four(hip_backend, oracle_backend, switch):
    """The 128-byte-slice pipeline's two smallest fp16 tiles also exist with a ring of four stages
    (picked when a workgroup has a compute unit, or half of one, to itself). Forced here on products
    whose K is shorter than the ring, as long as it, a multiple of it and ragged, whole tiles and
    edges, odd leading dimensions, batches: against the oracle, and bit for bit against the
    two-stage kernels (same instructions on the same accumulators in the same order)."""
    rng = np.random.default_rng(98)
    dtype, bits = F16, np.uint16
    for tile in ("64x64", "128x64"):
        switch.setenv("HCHIP_GEMM_TILE", tile)
        for K in (192, 200, 256, 320, 512 + 5, 1024, 1001, 64 * 11 - 7):
            for (batch, M, N) in ((1, 128, 128), (2, 200, 72), (1, 67, 129)):
                a = rand(rng, (batch, M, K), dtype, 1.0 / K ** 0.5)
                b = rand(rng, (batch, K, N), dtype)
                for transA, transB in ((False, False), (True, True), (False, True), (True, False)):
                    sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if transA else a
                    sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if transB else b
                    print("ring of four", tile, batch, M, K, N, transA, transB, flush=True)
                    fn = lambda: Tensor.batchedMatmul(Tensor(data=sa), transA, Tensor(data=sb), transB, False)
                    switch.setenv("HCHIP_GEMM_RING", "4")
                    got, want = check_close(hip_backend, oracle_backend, fn, TOL[dtype])
                    switch.setenv("HCHIP_GEMM_RING", "2")
                    switch.setenv("HCHIP_GEMM_KERNEL", "dma2")
                    with hip_backend.use():
                        two = fn().numpy()
                    switch.delenv("HCHIP_GEMM_RING")
                    switch.delenv("HCHIP_GEMM_KERNEL")
                    assert np.array_equal(np.ascontiguousarray(got).view(bits), np.ascontiguousarray(two).view(bits))


@pytest.mark.parametrize("pipeline", ["auto", "dma", "dma2", "mi16"])
def test_matmul_random_shapes(hip_backend, oracle_backend, switch, pipeline):
    """Seeded random extents (aligned and odd), batches and flags through each pipeline: row and
    K raggedness against every tile edge, re-pitched operands, transposed outputs."""
    rng = np.random.default_rng(2024)
    if pipeline != "auto":
        switch.setenv("HCHIP_GEMM_KERNEL", pipeline)
    for case in range(24):
        dtype = F16 if (pipeline == "mi16" or case % 2 == 0) else F32
        align = [1, 8, 8, 64][case % 4]
        M, K, N = (int(rng.integers(1, 90 if align < 64 else 24)) * align for _ in range(3))
        batch = int(rng.integers(1, 4))
        transA, transB, transOut = (bool(rng.integers(0, 2)) for _ in range(3))
        a = rand(rng, (batch, M, K), dtype, 1.0 / K ** 0.5)
        b = rand(rng, (batch, K, N), dtype)
        sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if transA else a
        sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if transB else b
        print("matmul", pipeline, dtype.name, batch, M, K, N, transA, transB, transOut, flush=True)
        fn = lambda: Tensor.batchedMatmul(Tensor(data=sa), transA, Tensor(data=sb), transB, transOut)
        got, want = check_close(hip_backend, oracle_backend, fn, TOL[dtype])
        scale = float(np.max(np.abs(want.astype(np.float64))))
        assert float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) <= TOL[dtype] * max(scale, 1e-30)


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_matmul_repitched_operands_every_residue(hip_backend, oracle_backend, dtype):
    """Operands and outputs whose rows are not 16-byte aligned are copied into padded buffers and
    back. Every residue of the row length modulo a 16-byte piece, batches of odd-sized matrices
    (so matrices start on odd element addresses) and buffers that end exactly with the last
    element; `A x I` must come back bit for bit, which checks the copies on their own."""
    rng = np.random.default_rng(808)
    for r in range(9):
        batch, M, K, N = 3, 129 + (r % 3), 263 + r, 257 + r  # >= 2^24 multiply-adds: the copies are used
        a = rand(rng, (batch, M, K), dtype, 1.0 / K ** 0.5)
        b = rand(rng, (batch, K, N), dtype)
        for transA, transB, transOut in ((False, False, False), (True, True, False), (False, True, True), (True, False, True)):
            sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if transA else a
            sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if transB else b
            print("repitch", dtype.name, batch, M, K, N, transA, transB, transOut, flush=True)
            fn = lambda: Tensor.batchedMatmul(Tensor(data=sa), transA, Tensor(data=sb), transB, transOut)
            got, want = check_close(hip_backend, oracle_backend, fn, TOL[dtype])
            scale = float(np.max(np.abs(want.astype(np.float64))))
            assert float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) <= TOL[dtype] * scale
        # identity on the right: the product is A itself, exactly (but for -0, which x*1 + 0*0 turns into +0)
        a[a == 0] = 0
        eye = np.broadcast_to(np.eye(K, dtype=a.dtype), (batch, K, K)).copy()
        with hip_backend.use():
            out = Tensor.batchedMatmul(Tensor(data=a), False, Tensor(data=eye), False, False).numpy()
        np.testing.assert_array_equal(out.view(np.uint16 if dtype is F16 else np.uint32),
                                      a.view(np.uint16 if dtype is F16 else np.uint32))


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_matmul_skinny_products(hip_backend, oracle_backend, dtype):
    """One extent of C at most 32 (matrix-vector products, fringes of ragged GEMMs): the
    wave-per-row and the lane-per-row / split-K kernels, every layout, a batch, odd strides."""
    rng = np.random.default_rng(55)
    for (batch, M, K, N) in [(1, 4097, 1032, 1), (1, 1, 1000, 5000), (2, 3000, 777, 7), (1, 20, 2048, 1024),
                             (3, 1, 512, 2048), (1, 600, 64, 32), (1, 5, 4099, 515)]:
        a = rand(rng, (batch, M, K), dtype, 1.0 / K ** 0.5)
        b = rand(rng, (batch, K, N), dtype)
        for transA in (False, True):
            for transB in (False, True):
                for transOut in (False, True):
                    sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if transA else a
                    sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if transB else b
                    print("skinny", dtype.name, batch, M, K, N, transA, transB, transOut, flush=True)
                    fn = lambda: Tensor.batchedMatmul(Tensor(data=sa), transA, Tensor(data=sb), transB, transOut)
                    got, want = check_close(hip_backend, oracle_backend, fn, TOL[dtype])
                    scale = float(np.max(np.abs(want.astype(np.float64))))
                    assert float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) <= TOL[dtype] * scale


def test_matmul_fp16_4096_against_oracle_slab_and_identity(hip_backend, oracle_backend):
    """Config 2 at full size: every layout; a 96-row slab of each product is checked against
    the oracle, and A x I == A exactly."""
    rng = np.random.default_rng(2)
    n = 4096
    a = (rng.standard_normal((n, n)) / np.sqrt(n)).astype(np.float16)
    b = rng.standard_normal((n, n)).astype(np.float16)
    rows = np.r_[0:32, 2000:2032, n - 32:n]
    with oracle_backend.use():
        want = Tensor.matmul(Tensor(data=a[rows]), False, Tensor(data=b), False, False).numpy()
    with hip_backend.use():
        ta, tb = Tensor(data=a), Tensor(data=b)
        tat, tbt = Tensor(data=np.ascontiguousarray(a.T)), Tensor(data=np.ascontiguousarray(b.T))
        for transA, transB in [(False, False), (False, True), (True, False), (True, True)]:
            print("4096^3 layout", transA, transB, flush=True)
            out = Tensor.matmul(tat if transA else ta, transA, tbt if transB else tb, transB, False).numpy()
            assert_close_arrays(out[rows], want, 1e-2, 1e-2)
        eye = Tensor(data=np.eye(n, dtype=np.float16))
        assert np.array_equal(Tensor.matmul(ta, False, eye, False, False).numpy(), a)
        assert np.array_equal(Tensor.matmul(eye, False, tb, False, False).numpy(), b)


def test_matmul_fp32_4096_against_oracle_slab_and_identity(hip_backend, oracle_backend):
    """The fp32 leg of the headline metric at full size (BackendCPU.swift:1245-1304), the two layouts
    the bench reports (NN, NT) and the other two: a 96-row slab of each product against the oracle at
    1e-4 (absolute or relative) and 1e-4 of the largest element, and A x I == A, I x B == B exactly."""
    rng = np.random.default_rng(3)
    n = 4096
    a = (rng.standard_normal((n, n)) / np.sqrt(n)).astype(np.float32)
    b = rng.standard_normal((n, n)).astype(np.float32)
    rows = np.r_[0:32, 2000:2032, n - 32:n]
    with oracle_backend.use():
        want = Tensor.matmul(Tensor(data=a[rows]), False, Tensor(data=b), False, False).numpy()
    scale = float(np.max(np.abs(want)))
    with hip_backend.use():
        ta, tb = Tensor(data=a), Tensor(data=b)
        tat, tbt = Tensor(data=np.ascontiguousarray(a.T)), Tensor(data=np.ascontiguousarray(b.T))
        for transA, transB in [(False, False), (False, True), (True, False), (True, True)]:
            print("fp32 4096^3 layout", transA, transB, flush=True)
            out = Tensor.matmul(tat if transA else ta, transA, tbt if transB else tb, transB, False).numpy()
            assert_close_arrays(out[rows], want, 1e-4, 1e-4)
            assert float(np.max(np.abs(out[rows].astype(np.float64) - want.astype(np.float64)))) <= 1e-4 * scale
        eye = Tensor(data=np.eye(n, dtype=np.float32))
        assert np.array_equal(Tensor.matmul(ta, False, eye, False, False).numpy(), a)
        assert np.array_equal(Tensor.matmul(eye, False, tb, False, False).numpy(), b)
        assert np.array_equal(Tensor.matmul(ta, False, eye, True, False).numpy(), a)


@pytest.mark.parametrize("shape", [(4100, 1032, 4104), (3000, 1096, 3016)], ids=lambda s: "x".join(map(str, s)))
def test_matmul_fp16_large_ragged_against_oracle_slab(hip_backend, oracle_backend, shape):
    """Products large enough for the host to pick the full-device fp16 kernels (the second one
    with 192 x 192 tiles), but ragged in M, N and K (edge variants: clamped rows, zero-filled K
    tail, predicated stores): row slabs against the oracle, the whole result against the general
    kernel, and nothing written past the edges."""
    rng = np.random.default_rng(12)
    M, K, N = shape
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float16)
    b = rng.standard_normal((K, N)).astype(np.float16)
    rows = np.r_[0:24, M // 2 - 10:M // 2 + 14, M - 24:M]
    with oracle_backend.use():
        want = Tensor.matmul(Tensor(data=a[rows]), False, Tensor(data=b), False, False).numpy()
    with hip_backend.use():
        ta, tb = Tensor(data=a), Tensor(data=b)
        tat, tbt = Tensor(data=np.ascontiguousarray(a.T)), Tensor(data=np.ascontiguousarray(b.T))
        with hip_backend.switches(HCHIP_GEMM_TILE="general"):
            general = Tensor.matmul(ta, False, tb, False, False).numpy()
        assert_close_arrays(general[rows], want, 1e-2, 1e-2)
        for transA, transB in [(False, False), (False, True), (True, False), (True, True)]:
            print(shape, "layout", transA, transB, flush=True)
            out = Tensor.matmul(tat if transA else ta, transA, tbt if transB else tb, transB, False).numpy()
            assert out.shape == (M, N)
            assert_close_arrays(out[rows], want, 1e-2, 1e-2)
            assert_close_arrays(out, general, 1e-2, 1e-2)


def test_matmul_fp32_192_tiles_against_oracle_slab(hip_backend, oracle_backend):
    """An fp32 product whose output the host covers with 192 x 192 tiles (ragged in M, N and K:
    edge variant): row slabs against the oracle, the whole result against the general kernel."""
    rng = np.random.default_rng(13)
    M, K, N = 3000, 520, 3016
    a = (rng.standard_normal((M, K)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal((K, N)).astype(np.float32)
    rows = np.r_[0:16, M // 2 - 8:M // 2 + 8, M - 16:M]
    with oracle_backend.use():
        want = Tensor.matmul(Tensor(data=a[rows]), False, Tensor(data=b), False, False).numpy()
    with hip_backend.use():
        ta, tb = Tensor(data=a), Tensor(data=b)
        tat, tbt = Tensor(data=np.ascontiguousarray(a.T)), Tensor(data=np.ascontiguousarray(b.T))
        with hip_backend.switches(HCHIP_GEMM_TILE="general"):
            general = Tensor.matmul(ta, False, tb, False, False).numpy()
        assert_close_arrays(general[rows], want, 1e-4, 1e-4)
        for transA, transB in [(False, False), (False, True), (True, False), (True, True)]:
            print("3000x520x3016 fp32 layout", transA, transB, flush=True)
            out = Tensor.matmul(tat if transA else ta, transA, tbt if transB else tb, transB, False).numpy()
            assert out.shape == (M, N)
            assert_close_arrays(out[rows], want, 1e-4, 1e-4)
            assert_close_arrays(out, general, 1e-4, 1e-4)


def test_matmul_int64(hip_backend, oracle_backend):
    """int64 products (BackendCPU.swift:1307): all flag combinations, ragged extents, a batch."""
    rng = np.random.default_rng(8)
    for (m, k, n) in [(17, 33, 9), (64, 16, 48), (1, 5, 1), (40, 0, 3)]:
        a = rng.integers(-1000, 1000, size=(m, k))
        b = rng.integers(-1000, 1000, size=(k, n))
        for ta in (False, True):
            for tb in (False, True):
                for to in (False, True):
                    an = np.ascontiguousarray(a.T) if ta else a
                    bn = np.ascontiguousarray(b.T) if tb else b
                    fn = lambda: Tensor.matmul(Tensor(data=an), ta, Tensor(data=bn), tb, to)
                    check_exact(hip_backend, oracle_backend, fn)
                    with hip_backend.use():
                        assert np.array_equal(fn().numpy(), (a @ b).T if to else a @ b)
    a = rng.integers(-(2 ** 40), 2 ** 40, size=(3, 6, 7))        # sums that wrap around 2^64
    b = rng.integers(-(2 ** 40), 2 ** 40, size=(3, 7, 5))
    check_exact(hip_backend, oracle_backend, lambda: Tensor.batchedMatmul(Tensor(data=a), False, Tensor(data=b), False, False))


def test_matmul_fp32_1024(hip_backend, oracle_backend):
    """Config 1: fp32 [1024,1024] x [1024,1024], N(0,1) entries, no transposes."""
    rng = np.random.default_rng(1)
    a = rng.standard_normal((1024, 1024)).astype(np.float32)
    b = rng.standard_normal((1024, 1024)).astype(np.float32)
    got, want = check_close(hip_backend, oracle_backend,
                            lambda: Tensor.matmul(Tensor(data=a), False, Tensor(data=b), False, False), 1e-4)
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) <= 1e-4


# ---------------------------------------------------------------- element-wise

BCAST_PAIRS = [([512, 1024], [1, 1024]), ([512, 1024], [512, 1]), ([33, 1025], [33, 1025]), ([6], [3, 6]),
               ([3, 1, 6], [1, 2, 6]), ([1, 3, 1, 3, 1], [3, 1, 3, 1, 3]), ([3, 1, 3, 1, 3, 1], [1, 3, 1, 3, 1, 3]),
               ([8, 8, 64, 64], [64, 64]), ([2, 3, 4, 5, 6, 7, 8], [1, 3, 1, 5, 1, 7, 1]), ([], [4, 4]), ([0, 5], [0, 5])]


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_binary_broadcast_ops(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(11)
    for sa, sb in BCAST_PAIRS:
        a = np.asarray(rand(rng, sa, dtype, 3.0))
        b = np.asarray(rand(rng, sb, dtype, 3.0))
        if dtype == I64:
            b = np.where(b == 0, 7, b)
        print("binary", dtype.name, sa, sb, flush=True)
        for op in (lambda x, y: x + y, lambda x, y: x - y, lambda x, y: x * y, lambda x, y: x / y,
                   lambda x, y: x % y):
            check_exact(hip_backend, oracle_backend,
                        lambda: op(Tensor(data=a, shape=sa, dtype=dtype), Tensor(data=b, shape=sb, dtype=dtype)))
        for op in (lambda x, y: x.mul(y, thenAdd=x), lambda x, y: x.add(y, thenMul=y)):
            check_exact(hip_backend, oracle_backend,
                        lambda: op(Tensor(data=a, shape=sa, dtype=dtype), Tensor(data=b, shape=sb, dtype=dtype)))
        for op in (lambda x, y: x < y, lambda x, y: x == y, lambda x, y: x >= y, lambda x, y: x != y):
            check_exact(hip_backend, oracle_backend,
                        lambda: op(Tensor(data=a, shape=sa, dtype=dtype), Tensor(data=b, shape=sb, dtype=dtype)))


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_scalar_ops(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(12)
    for n in (1, 7, 4096, 100003):
        x = rand(rng, (n,), dtype, 4.0)
        if dtype == I64:
            x = np.where(x == 0, 3, x)
        for s in ([3, -7] if dtype == I64 else [3, 0.125, -2.5]):
            for op in (lambda t: t + s, lambda t: t - s, lambda t: t * s, lambda t: t / s, lambda t: t % s,
                       lambda t: s + t, lambda t: s - t, lambda t: s * t, lambda t: s / t, lambda t: s % t,
                       lambda t: t < s, lambda t: s >= t, lambda t: t == s):
                check_exact(hip_backend, oracle_backend, lambda: op(Tensor(data=x, dtype=dtype)))


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_elemwise_all_ops(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(13)
    x = np.concatenate([rng.standard_normal(20000) * 2.5, np.linspace(-6, 6, 1203), [0.0, -0.0, 25.0, -25.0]])
    x = x.astype(dtype.numpy)
    unit = np.clip(x.astype(np.float32) / 7.0, -0.98, 0.98).astype(dtype.numpy)
    scales = rng.standard_normal(x.size).astype(dtype.numpy)
    # fp16 keeps the reference's x100 widening (BackendTests.swift:1065)
    tol = 1e-4 if dtype == F32 else 1e-2
    for op in ElemwiseOp:
        src = unit if op in (ElemwiseOp.acos, ElemwiseOp.asin, ElemwiseOp.acosGrad, ElemwiseOp.asinGrad) else x
        if op == ElemwiseOp.log:
            src = np.abs(x) + dtype.numpy(0.01)
        print("elemwise", op.name, dtype.name, flush=True)
        for sc in (None, scales):
            def fn():
                from honeycrisp_amd.backend import Backend
                be = Backend.current()
                t = Tensor(data=src)
                s = Tensor(data=sc).data if sc is not None else None
                return Tensor(dataHandle=be.elemwise(t.data, op, s, src.size, dtype), shape=[src.size], dtype=dtype)
            if op in (ElemwiseOp.relu, ElemwiseOp.reluGrad, ElemwiseOp.abs, ElemwiseOp.absGrad, ElemwiseOp.floor,
                      ElemwiseOp.ceil, ElemwiseOp.round, ElemwiseOp.recip):
                check_exact(hip_backend, oracle_backend, fn)
            else:
                check_close(hip_backend, oracle_backend, fn, tol)


def test_gelu_tail_is_judged_abs_or_rel(hip_backend, oracle_backend):
    """For x << 0 the (1 + tanh) term of the approximate GELU cancels to about one bit, so a
    1-ulp expf difference doubles the value at magnitude 1e-7: abs <= 1e-4 is what holds."""
    x = np.linspace(-12, -3, 4001).astype(np.float32)
    got, want = check_close(hip_backend, oracle_backend, lambda: Tensor(data=x).gelu(), 1e-4)
    assert np.max(np.abs(got - want)) < 1e-6


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_pow(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(14)
    x = np.abs(rand(rng, (5003,), dtype, 2.0)) + (1 if dtype == I64 else dtype.numpy(0.05))
    sc = rand(rng, (5003,), dtype)
    from honeycrisp_amd.backend import Backend
    for b, scale in ([(2, 1), (3, 2)] if dtype == I64 else [(2.0, 1.0), (2.0, 3.0), (-1.0, 0.5), (1.0, 4.0), (0.5, 1.0),
                                                          (-0.5, 1.0), (3.0, 2.0), (-1.5, 0.25)]):
        for scales in (None, sc):
            def fn():
                be = Backend.current()
                s = Tensor(data=scales, dtype=dtype).data if scales is not None else None
                data = be.pow(Tensor(data=x, dtype=dtype).data, b, scale, s, x.size, dtype)
                return Tensor(dataHandle=data, shape=[x.size], dtype=dtype)
            if dtype == F32 and b in (2.0, -1.0, 1.0) or dtype == I64:
                check_exact(hip_backend, oracle_backend, fn)
            else:
                check_close(hip_backend, oracle_backend, fn, 1e-4 if dtype == F32 else 1e-2)


def test_cast_all_pairs(hip_backend, oracle_backend):
    rng = np.random.default_rng(15)
    f = np.concatenate([rng.standard_normal(3001) * 100, [0.0, -0.0, 0.4, -0.6, 65519.0, 65520.0, 1e9, -1e9, 5e-8]])
    srcs = {F32: f.astype(np.float32), F16: rng.standard_normal(3001).astype(np.float16) * np.float16(50),
            I64: rng.integers(-2**40, 2**40, size=3001), BOOL: rng.integers(0, 2, size=3001).astype(np.bool_)}
    for it, src in srcs.items():
        for ot in DType:
            if it == F32 and ot == I64:
                src_ = src[np.abs(src) < 1e6]
            else:
                src_ = src
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=src_, dtype=it).cast(ot))


def test_when_fill_triangular_concat_broadcast(hip_backend, oracle_backend):
    rng = np.random.default_rng(16)
    mask = rng.integers(0, 2, size=(6, 1, 40)).astype(np.bool_)
    for dtype in (F32, F16, I64, BOOL):
        a = rand(rng, (5, 40), dtype) if dtype != BOOL else rng.integers(0, 2, size=(5, 40)).astype(np.bool_)
        b = rand(rng, (40,), dtype) if dtype != BOOL else rng.integers(0, 2, size=(40,)).astype(np.bool_)
        check_exact(hip_backend, oracle_backend,
                    lambda: Tensor(data=mask).when(Tensor(data=a, dtype=dtype), Tensor(data=b, dtype=dtype)))
        if dtype != BOOL:
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=mask).when(Tensor(data=a, dtype=dtype), 2))
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=mask).when(0, -1e4 if dtype != I64 else -7, dtype=dtype))
        m = rand(rng, (3, 17, 23), dtype) if dtype != BOOL else rng.integers(0, 2, size=(3, 17, 23)).astype(np.bool_)
        for off in (-20, -3, 0, 2, 30):
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=m, dtype=dtype).tril(off))
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=m, dtype=dtype).triu(off))
        check_exact(hip_backend, oracle_backend,
                    lambda: Tensor.concat([Tensor(data=m, dtype=dtype), Tensor(data=m[:, :5], dtype=dtype)], axis=1))
        check_exact(hip_backend, oracle_backend,
                    lambda: Tensor.concat([Tensor(data=m, dtype=dtype), Tensor(data=m[:, :, :9], dtype=dtype)], axis=2))
        wide = rand(rng, (2, 70, 64), dtype) if dtype != BOOL else rng.integers(0, 2, size=(2, 70, 64)).astype(np.bool_)
        for off in (-65, -7, 0, 1, 33, 80):       # rows that are whole 16-byte vectors
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=wide, dtype=dtype).tril(off))
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=wide, dtype=dtype).triu(off))
        # pieces whose widths allow 16-, 8-, 4- and 2-byte copy units, three inputs, axis 0
        w = rand(rng, (9, 64), dtype) if dtype != BOOL else rng.integers(0, 2, size=(9, 64)).astype(np.bool_)
        for widths in [(64, 32), (8, 64, 24), (4, 60), (2, 6, 64), (1, 63), (64, 64, 64)]:
            check_exact(hip_backend, oracle_backend,
                        lambda: Tensor.concat([Tensor(data=w[:, :c], dtype=dtype) for c in widths], axis=1))
        check_exact(hip_backend, oracle_backend,
                    lambda: Tensor.concat([Tensor(data=w, dtype=dtype), Tensor(data=w[:4], dtype=dtype), Tensor(data=w[:1], dtype=dtype)], axis=0))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=b, dtype=dtype).expand([7, 3, 40]))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=a, dtype=dtype).reshape([5, 1, 40]).expand([5, 6, 40]))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=a, dtype=dtype).repeating(1, 3))
        check_exact(hip_backend, oracle_backend, lambda: Tensor.constant(1 if dtype == BOOL else 3, [1001], dtype))


# ---------------------------------------------------------------- reductions

REDUCE_SHAPES = [(8, 4096, 1), (37, 513, 1), (5, 1, 1), (3, 7, 1), (1, 100000, 1), (64, 1024, 1), (4, 33, 65),
                 (1, 300, 4096), (17, 2, 3), (9, 8192, 2),
                 # tall and narrow: the reduce axis is split over blocks and combined in a second pass
                 (2, 5000, 96), (1, 4097, 260), (1, 70000, 8),
                 # rows of a few elements (a lane or 8 lanes per row) and few long rows (cut into
                 # segments that leave partials; 300001 is odd, so its segments are read element-wise)
                 (70000, 3, 1), (5000, 8, 1), (4097, 100, 1), (1, 400000, 1), (3, 300001, 1), (2, 65536, 1),
                 # inner narrower than a wave: the wave's other lanes take further rows
                 (1, 100000, 3), (2, 30000, 64), (3, 1000, 20), (5, 77, 1), (1, 9000, 5)]


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_reduce_all_ops(hip_backend, oracle_backend, dtype):
    from honeycrisp_amd.backend import Backend
    rng = np.random.default_rng(17)
    for outer, red, inner in REDUCE_SHAPES:
        x = rand(rng, (outer, red, inner), dtype)
        if dtype != I64:
            # plant ties so that first-occurrence matters
            x = np.round(x * 4) / dtype.numpy(4)
        dims = ReduceDims(outer, red, inner)
        print("reduce", dtype.name, (outer, red, inner), flush=True)
        for op in ReduceOp:
            if op == ReduceOp.prod:
                src = (x % 3 + 1) if dtype == I64 else (np.sign(x) + (x == 0)) * (1 + np.abs(x) / dtype.numpy(64))
                src = src[:, :min(red, 60)].astype(dtype.numpy)
                d = ReduceDims(outer, src.shape[1], inner)
            else:
                src, d = x, dims
            def fn():
                be = Backend.current()
                data = be.reduce(Tensor(data=src, dtype=dtype).data, op, d, dtype)
                return Tensor(dataHandle=data, shape=[d.outCount], dtype=I64 if op.isIntOut else dtype)
            if op.isIntOut or dtype == I64:
                check_exact(hip_backend, oracle_backend, fn)
            else:
                # summation order differs from the sequential CPU loop; fp16 sums of up to 1e5
                # unit-scale terms are judged relative to the magnitude a sequential fp32 sum has
                got, want = both(hip_backend, oracle_backend, fn)
                atol = TOL[dtype] * max(1.0, float(np.sqrt(d.reduceCount)))
                assert_close_arrays(got, want, atol, TOL[dtype])


def test_argmax_nan_and_tie_rules(hip_backend, oracle_backend):
    """Bit-exact first-extremum semantics, including NaN placement (BackendCPU.swift:848-877)."""
    rng = np.random.default_rng(18)
    nan, inf = np.nan, np.inf
    base = np.array([[1, nan, 3, 3], [nan, 5, 9, 1], [-inf, nan, -inf, -inf], [2, 2, nan, 2], [inf, nan, inf, 0],
                     [nan, nan, nan, nan], [nan, inf, -inf, 0]], dtype=np.float32)
    for dtype in (F32, F16):
        for op in (ReduceOp.argmax, ReduceOp.argmin):
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=base, dtype=dtype).reduce(op, axis=1))
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=base, dtype=dtype).reduce(op, axis=0))
    # long rows with few distinct values and NaNs sprinkled in, rows and columns
    x = rng.integers(-2, 3, size=(64, 5000)).astype(np.float32)
    x[rng.random(x.shape) < 0.01] = nan
    x[::7, 0] = nan
    for op in (ReduceOp.argmax, ReduceOp.argmin):
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x).reduce(op, axis=1))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x).reduce(op, axis=0))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x[:, :777]).reduce(op, axis=1))
    # max / min = arg-reduction + gather
    y = rng.standard_normal((33, 4096)).astype(np.float32)
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=y).max(axis=1))
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=y).min(axis=0))
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=y).max())
    # one long row in segments: ties and NaNs across segment boundaries, NaN at element 0
    z = rng.integers(-3, 4, size=(2, 200000)).astype(np.float32)
    z[rng.random(z.shape) < 0.001] = nan
    z[1, 0] = nan
    for op in (ReduceOp.argmax, ReduceOp.argmin):
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=z).reduce(op, axis=1))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=z[0]).reduce(op, axis=0))
    # rows of 3 and of 100 elements with ties and NaNs
    for width in (3, 100):
        w = rng.integers(-1, 2, size=(3000, width)).astype(np.float32)
        w[rng.random(w.shape) < 0.05] = nan
        for op in (ReduceOp.argmax, ReduceOp.argmin):
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=w).reduce(op, axis=1))


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_log_softmax_and_normalize(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(19)
    for shape, axis in [((64, 256), 1), ((16, 8, 32, 32), 3), ((5, 1000), 1), ((7, 33, 9), 1), ((300, 4), 0),
                        ((2, 1), 1), ((3, 10000), 1), ((4096, 96), 0), ((2, 3000, 40), 1), ((3, 129, 7), 1),
                        # short rows: a lane or 8 lanes per row
                        ((7000, 3), 1), ((3001, 8), 1), ((1000, 100), 1), ((999, 128), 1), ((500, 16), 1),
                        ((30000, 3), 0), ((5000, 64), 0), ((2, 900, 20), 1),
                        # few long rows: cut over many blocks (column path / op-by-op composition)
                        ((2, 70000), 1), ((1, 40001), 1)]:
        x = rand(rng, shape, dtype, 3.0)
        print("logsoftmax/normalize", dtype.name, shape, axis, flush=True)
        check_close(hip_backend, oracle_backend, lambda: Tensor(data=x).logSoftmax(axis=axis), TOL[dtype])
        tol = 1e-4 if dtype == F32 else 2e-2   # the reference's own normalize tolerance (BackendTests.swift:196-197)
        check_close(hip_backend, oracle_backend, lambda: Tensor(data=x).normalize(axis=axis, eps=1e-5), tol)
        check_close(hip_backend, oracle_backend, lambda: Tensor(data=x).normalize(axis=axis, eps=0.3), tol)
    neg = np.full((4, 50), -np.inf, dtype=dtype.numpy)
    neg[1, 3] = 0
    neg[2, 7] = np.nan
    check_close(hip_backend, oracle_backend, lambda: Tensor(data=neg).logSoftmax(), TOL[dtype])


# ---------------------------------------------------------------- gather / permute

def test_gather_forms(hip_backend, oracle_backend):
    rng = np.random.default_rng(20)
    for dtype in (F32, F16, I64, BOOL):
        table = rand(rng, (1000, 64), dtype) if dtype != BOOL else rng.integers(0, 2, size=(1000, 64)).astype(np.bool_)
        ids = rng.integers(0, 1000, size=(4099,))
        print("gather", dtype.name, flush=True)
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=table, dtype=dtype).gather(0, Tensor(data=ids)))
        x = table.reshape(10, 100, 64)
        idx3 = rng.integers(0, 100, size=(10, 7, 64))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x, dtype=dtype).gather(1, Tensor(data=idx3)))
        idx_last = rng.integers(0, 64, size=(10, 100, 5))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x, dtype=dtype).gather(2, Tensor(data=idx_last)))
        idx_b = rng.integers(0, 100, size=(1, 9, 1))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x, dtype=dtype).gather(1, Tensor(data=idx_b)))
        odd = table[:, :37]
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=odd, dtype=dtype).gather(0, Tensor(data=ids[:300])))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x, dtype=dtype).t())
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x, dtype=dtype).swap(0, 1))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x, dtype=dtype).move(2, 0))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x, dtype=dtype)[2:9, ..., 5])


def test_axis_permutation(hip_backend, oracle_backend):
    from honeycrisp_amd.backend import Backend
    for perm, shape in [([1, 0], [256, 8]), ([2, 0, 1], [3, 4, 5]), ([0], [7]), ([3, 1, 0, 2], [2, 3, 4, 5]),
                        ([1, 0], [1, 1]), ([4, 3, 2, 1, 0], [2, 3, 4, 5, 6])]:
        def fn():
            data = Backend.current().axisPermutation(perm, shape)
            return Tensor(dataHandle=data, shape=[int(np.prod(shape))], dtype=I64)
        check_exact(hip_backend, oracle_backend, fn)


@pytest.mark.parametrize("dtype", [F32, F16, I64, BOOL], ids=["f32", "f16", "i64", "bool"])
def test_permuted_views_take_the_direct_copy(hip_backend, oracle_backend, dtype):
    """t / swap / move / PermuteAxes: the gather whose indices come from axisPermutation runs as
    one direct copy (rows as vectors, a moved innermost axis through LDS tiles). Same result as the
    oracle's gather and as numpy's transpose, bit for bit, for every element size, ragged tiles,
    batch prefixes, odd row lengths, and the index vector itself stays readable."""
    rng = np.random.default_rng(61)
    cases = [((100, 70), (1, 0)), ((64, 64), (1, 0)), ((1, 300), (1, 0)), ((129, 1), (1, 0)),
             ((6, 33, 65), (0, 2, 1)), ((5, 8, 16, 32), (0, 2, 1, 3)), ((5, 8, 16, 6), (2, 0, 1, 3)),
             ((3, 4, 5, 6), (3, 2, 1, 0)), ((7, 9, 11), (2, 0, 1)), ((4, 40, 24), (1, 0, 2)),
             ((2, 3, 130, 67), (0, 1, 3, 2)), ((2050, 3), (1, 0)), ((8, 256, 8, 64), (0, 2, 1, 3)),
             # one of the two transposed axes short: long narrow tiles
             ((5000, 2), (1, 0)), ((2, 5000), (1, 0)), ((3, 1500, 5), (0, 2, 1)), ((7, 3000), (1, 0)), ((1100, 20), (1, 0)),
             # both axes long, ragged against the tiles
             ((256, 384), (1, 0)), ((3, 130, 258), (0, 2, 1)), ((200, 128), (1, 0)), ((2, 128, 3, 128), (3, 1, 2, 0))]
    for shape, perm in cases:
        x = rng.integers(0, 2, size=shape) if dtype == BOOL else rand(rng, shape, dtype)
        print("permute", dtype.name, shape, perm, flush=True)
        n = len(perm)
        lead = 0
        while lead < n and perm[lead] == lead:
            lead += 1
        from honeycrisp_amd.tensor import FullRange, PermuteAxes
        def fn():
            t = Tensor(data=x, dtype=dtype)
            return t[PermuteAxes(*perm)]
        check_exact(hip_backend, oracle_backend, fn)
        with hip_backend.use():
            got = fn().numpy()
        assert np.array_equal(got, np.ascontiguousarray(np.transpose(np.asarray(x).astype(got.dtype), perm)))
    # eight permuted axes, and eight behind a leading axis (one more than the direct copy takes)
    z8 = rand(rng, (2, 3, 2, 2, 3, 2, 2, 3), F32)
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=z8)[PermuteAxes(7, 6, 5, 4, 3, 2, 1, 0)])
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=z8)[PermuteAxes(0, 7, 1, 6, 2, 5, 3, 4)])
    # the 2-D helpers, with a batch prefix
    y = rand(rng, (3, 50, 70), F32)
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=y).t())
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=y).swap(0, 2))
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=y).move(2, 0))
    # the index vector is still a tensor like any other
    from honeycrisp_amd.backend import Backend
    def indices():
        data = Backend.current().axisPermutation([1, 0], [50, 70])
        return Tensor(dataHandle=data, shape=[3500], dtype=I64) + 1
    check_exact(hip_backend, oracle_backend, indices)


@pytest.mark.parametrize("seed", list(range(6)))
def test_random_broadcasts_against_oracle(hip_backend, oracle_backend, seed):
    """Seeded random broadcast patterns (each operand drops a random subset of the axes) through the
    broadcasting kernels, which pick a load form per operand from its innermost stride: binary
    arithmetic, comparison, when, mulAdd / addMul. All bit-exact (fp32 arithmetic without library
    calls, halfs computed in fp32 and rounded once on both sides)."""
    rng = np.random.default_rng(2000 + seed)
    extents = [1, 2, 3, 7, 8, 9, 16, 17, 33, 64, 65, 128, 257, 1000]
    for case in range(40):
        nd = int(rng.integers(1, 5))
        shape = [int(rng.choice(extents)) for _ in range(nd)]
        while int(np.prod(shape)) > 1 << 19:
            shape[int(np.argmax(shape))] = max(1, max(shape) // 4)
        dtype = [F32, F16, I64][int(rng.integers(0, 3))]
        def operand():
            keep = [bool(rng.integers(0, 2)) for _ in range(nd)]
            lead = int(rng.integers(0, nd + 1))        # also drop leading axes altogether
            shp = [s if k else 1 for s, k in zip(shape, keep)][lead:]
            v = rand(rng, shp if shp else [1], dtype)
            if dtype != I64:
                v = (np.round(v * 8) / 8).astype(dtype.numpy)
            return v
        a, b, c = operand(), operand(), operand()
        full = rand(rng, shape, dtype)                 # one operand of the full shape fixes the output shape
        op = ["add", "mul", "sub", "lt", "eq", "when", "mulAdd", "addMul"][int(rng.integers(0, 8))]
        print("broadcast case", seed, case, op, dtype.name, shape, a.shape, b.shape, c.shape, flush=True)
        T_ = lambda v: Tensor(data=v, dtype=dtype)
        if op == "add":
            fn = lambda: T_(full) + T_(a) + T_(b)
        elif op == "mul":
            fn = lambda: T_(a) * T_(full) * T_(b)
        elif op == "sub":
            fn = lambda: T_(a) - T_(full)
        elif op == "lt":
            fn = lambda: (T_(a) + T_(full) * 0) < T_(b)
        elif op == "eq":
            fn = lambda: T_(full) == T_(a)
        elif op == "when":
            fn = lambda: (T_(full) < T_(a)).when(T_(b), T_(c))
        elif op == "mulAdd":
            fn = lambda: T_(full).mul(T_(a), thenAdd=T_(b))
        else:
            fn = lambda: T_(full).add(T_(a), thenMul=T_(b))
        check_exact(hip_backend, oracle_backend, fn)


@pytest.mark.parametrize("seed", list(range(6)))
def test_random_gathers_and_scatters_against_oracle(hip_backend, oracle_backend, seed):
    """Seeded random gathers and scatters: value shapes with awkward extents, any axis, index tensors
    that are 1-D (one index per position of the axis), full-shaped, or broadcast along some of the other
    axes; scatters with unique and with repeated indices. Gathers and int64 / unique scatters are
    bit-exact; float scatters with repeated indices add in hardware-atomic order (tolerance), except
    the long-row form, which follows the CPU's order."""
    rng = np.random.default_rng(3000 + seed)
    extents = [1, 2, 3, 5, 8, 16, 17, 33, 64, 65, 127, 128, 256, 300, 1024]
    for case in range(30):
        nd = int(rng.integers(1, 5))
        shape = [int(rng.choice(extents)) for _ in range(nd)]
        while int(np.prod(shape)) > 1 << 19:
            shape[int(np.argmax(shape))] = max(1, max(shape) // 4)
        axis = int(rng.integers(0, nd))
        dtype = [F32, F16, I64, BOOL][int(rng.integers(0, 4))]
        count = int(rng.choice([1, 2, 7, 64, 300]))           # gathered positions along the axis
        form = int(rng.integers(0, 3))
        if form == 0:
            idx_shape = [count]
        else:
            idx_shape = list(shape)
            idx_shape[axis] = count
            if form == 2:                                      # broadcast along a random subset of the other axes
                for a in range(nd):
                    if a != axis and rng.random() < 0.5:
                        idx_shape[a] = 1
        x = rng.integers(0, 2, size=shape).astype(np.bool_) if dtype == BOOL else rand(rng, shape, dtype)
        idx = rng.integers(0, shape[axis], size=idx_shape)
        print("gather case", seed, case, dtype.name, shape, "axis", axis, "indices", idx_shape, flush=True)
        gather = lambda: Tensor(data=x, dtype=dtype).gather(axis, Tensor(data=idx))
        check_exact(hip_backend, oracle_backend, gather)
        if dtype == BOOL:
            continue
        # scatter the gathered values back into an axis of `target` positions
        with oracle_backend.use():
            g = gather().numpy()
        target = int(rng.choice([shape[axis], shape[axis] + 3, 2 * count + 1]))
        sidx = rng.integers(0, target, size=idx_shape)
        unique = False
        if rng.random() < 0.4 and count <= target:              # distinct indices along the axis
            perm = np.stack([rng.permutation(target)[:count] for _ in range(int(np.prod(idx_shape)) // count)])
            sidx = np.moveaxis(perm.reshape([s for a, s in enumerate(idx_shape) if a != (axis if form else 0)] + [count]),
                               -1, axis if form else 0)
            unique = True
        scatter = lambda: Tensor(data=g, dtype=dtype).scatter(axis, target, Tensor(data=np.ascontiguousarray(sidx)),
                                                              indicesAreUnique=unique)
        if dtype == I64 or unique:
            check_exact(hip_backend, oracle_backend, scatter)
        else:
            got, want = both(hip_backend, oracle_backend, scatter)
            assert_close_arrays(got, want, TOL[dtype] * 8, TOL[dtype])


@pytest.mark.parametrize("seed", list(range(12)))
def test_random_shapes_against_oracle(hip_backend, oracle_backend, seed):
    """Seeded random shapes with awkward extents (around vector, wave and tile sizes, extent 1, a
    few long axes) through the ops whose kernels choose a form by shape: reductions, arg-reductions,
    logSoftmax, normalize, cumulative sums, permuted views, concat, triangular."""
    from honeycrisp_amd.tensor import PermuteAxes
    rng = np.random.default_rng(1000 + seed)
    extents = [1, 2, 3, 5, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 100, 127, 128, 129, 255, 257, 1000, 1023, 4099]
    long_extents = [20000, 40001, 70000]
    for case in range(40):
        nd = int(rng.integers(1, 5))
        shape = [int(rng.choice(extents)) for _ in range(nd)]
        if rng.random() < 0.3:
            shape[int(rng.integers(0, nd))] = int(rng.choice(long_extents))
        while int(np.prod(shape)) > 1 << 20:
            shape[int(np.argmax(shape))] = max(1, max(shape) // 8)
        dtype = [F32, F16, I64][int(rng.integers(0, 3))]
        axis = int(rng.integers(0, nd))
        x = rand(rng, shape, dtype)
        if dtype != I64:
            x = (np.round(x * 4) / 4).astype(dtype.numpy)      # ties for the arg-reductions, exact partial sums
        op = ["sum", "argmax", "argmin", "logSoftmax", "normalize", "cumsum", "permute", "concat", "tril"][int(rng.integers(0, 9))]
        print("random case", seed, case, op, dtype.name, shape, "axis", axis, flush=True)
        t = lambda: Tensor(data=x, dtype=dtype)
        if op == "sum":
            fn = lambda: t().sum(axis=axis)
            if dtype == I64:
                check_exact(hip_backend, oracle_backend, fn)
            else:
                got, want = both(hip_backend, oracle_backend, fn)
                assert_close_arrays(got, want, TOL[dtype] * max(1.0, float(np.sqrt(shape[axis]))), TOL[dtype])
        elif op in ("argmax", "argmin"):
            check_exact(hip_backend, oracle_backend, lambda: getattr(t(), op)(axis=axis))
        elif op in ("logSoftmax", "normalize"):
            if dtype == I64:
                continue
            tol = TOL[dtype] if op == "logSoftmax" or dtype == F32 else 2e-2
            if op == "logSoftmax":
                check_close(hip_backend, oracle_backend, lambda: t().logSoftmax(axis=axis), tol)
            elif shape[axis] > 1:
                check_close(hip_backend, oracle_backend, lambda: t().normalize(axis=axis, eps=1e-3), tol)
        elif op == "cumsum":
            if dtype == F16 and shape[axis] > 500:
                continue    # running sums leave the range in which halfs are exact
            excl, rev = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
            small = t if dtype == I64 else (lambda: Tensor(data=np.sign(x).astype(dtype.numpy), dtype=dtype))
            check_exact(hip_backend, oracle_backend, lambda: small().cumulativeSum(axis, exclusive=excl, reverse=rev))
        elif op == "permute":
            perm = [int(p) for p in rng.permutation(nd)]
            check_exact(hip_backend, oracle_backend, lambda: t()[PermuteAxes(*perm)])
        elif op == "concat":
            other = rand(rng, [s if a != axis else int(rng.choice([1, 2, 8, 17])) for a, s in enumerate(shape)], dtype)
            check_exact(hip_backend, oracle_backend, lambda: Tensor.concat([t(), Tensor(data=other, dtype=dtype), t()], axis=axis))
        elif op == "tril" and nd >= 2:
            off = int(rng.integers(-3, 4))
            check_exact(hip_backend, oracle_backend, lambda: t().tril(off))


# ---------------------------------------------------------------- config 4 at full size

def test_bandwidth_ops_full_size(hip_backend, oracle_backend):
    """Config 4: X[8192,4096] + bias[1,4096], GELU, sum / max / argmax over axis 1, and an
    int64 gather of 65536 ids from a [32000,1024] table, all at the benchmark's sizes."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((8192, 4096)).astype(np.float32)
    bias = np.random.default_rng(8).standard_normal((1, 4096)).astype(np.float32)
    with hip_backend.use():
        tx = Tensor(data=x)
        h = tx + Tensor(data=bias)
        g = h.gelu()
        s = h.sum(axis=1)
        am = h.argmax(axis=1)
        mx = h.max(axis=1)
        h_np, g_np, s_np, am_np, mx_np = h.numpy(), g.numpy(), s.numpy(), am.numpy(), mx.numpy()
    want_h = x + bias
    assert np.array_equal(h_np, want_h)                        # IEEE add: bit-exact
    assert np.array_equal(am_np, want_h.argmax(axis=1))        # first maximum
    assert np.array_equal(mx_np, want_h.max(axis=1))
    # fp32 row sums: the order of a sum is not fixed (vDSP_sve, BackendCPU.swift:792-806), so the bound is
    # the one that holds for any order: 1e-4 of the row's sum of magnitudes
    exact = want_h.astype(np.float64).sum(axis=1)
    assert np.all(np.abs(s_np.astype(np.float64) - exact) <= 1e-4 * np.abs(want_h.astype(np.float64)).sum(axis=1))
    assert_close_arrays(s_np, exact, 1e-3, 1e-4)
    with oracle_backend.use():
        g_want = Tensor(data=want_h).gelu().numpy()
    assert_close_arrays(g_np, g_want, 1e-4, 1e-4)
    table = np.random.default_rng(10).standard_normal((32000, 1024)).astype(np.float32)
    ids = np.random.default_rng(9).integers(0, 32000, size=(65536,))
    with hip_backend.use():
        out = Tensor(data=table).gather(0, Tensor(data=ids)).numpy()
    assert np.array_equal(out, table[ids])


# ---------------------------------------------------------------- backward primitives

@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_scatter_forms(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(31)
    # small integers: every partial sum is exact, so the order of the atomic adds cannot matter
    vals = rng.integers(-8, 9, size=(6, 37, 20))
    vals = vals if dtype == I64 else vals.astype(dtype.numpy)
    idx = rng.integers(0, 11, size=(6, 37, 20))
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=vals).scatter(1, 11, Tensor(data=idx)))
    # broadcast indices (one index per row), the embedding-gradient shape
    rows = rng.integers(0, 50, size=(300,))
    emb = rng.integers(-8, 9, size=(300, 64))
    emb = emb if dtype == I64 else emb.astype(dtype.numpy)
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=emb).scatter(0, 50, Tensor(data=rows)))
    # unique indices: plain stores
    perm = rng.permutation(300)
    check_exact(hip_backend, oracle_backend,
                lambda: Tensor(data=emb).scatter(0, 300, Tensor(data=perm), indicesAreUnique=True))
    # empty input still zero-fills the output
    empty = np.zeros((0, 4), dtype=np.int64 if dtype == I64 else dtype.numpy)
    check_exact(hip_backend, oracle_backend,
                lambda: Tensor(data=empty, shape=[0, 4], dtype=dtype).scatter(0, 3, Tensor(data=[], shape=[0], dtype=I64)))


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_scatter_long_rows_bit_exact(hip_backend, oracle_backend, dtype):
    """Rows of 1 KiB and more whose index does not depend on the position in the row are added in
    source order, like the CPU loop: random floats match bit for bit."""
    rng = np.random.default_rng(33)
    width = {F32: 256, F16: 512, I64: 128}[dtype]
    cases = [
        (rng.integers(0, 300, size=(2000,)), 300, 1),          # a few sources per destination, some empty rows
        (rng.integers(0, 3, size=(700,)), 5, 1),               # hundreds per destination: sorted in LDS
        (np.zeros(4500, dtype=np.int64), 2, 1),                # more than the LDS holds: sorted in place
        (rng.integers(0, 40, size=(3, 90)), 40, 3),            # an outer axis in front
    ]
    for rows, count, outer in cases:
        shape = (rows.shape[0], width) if outer == 1 else (outer, rows.shape[1], width)
        vals = rand(rng, shape, dtype)
        axis = 0 if outer == 1 else 1
        index = rows if outer == 1 else rows[:, :, None]
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=vals).scatter(axis, count, Tensor(data=index)))
    # twice the same call: no run-to-run differences
    vals = rand(rng, (3000, width), dtype)
    rows = rng.integers(0, 17, size=(3000,))
    with hip_backend.use():
        first = Tensor(data=vals).scatter(0, 17, Tensor(data=rows)).numpy()
        second = Tensor(data=vals).scatter(0, 17, Tensor(data=rows)).numpy()
    assert first.tobytes() == second.tobytes()


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_scatter_random_floats_within_tolerance(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(32)
    vals = rng.standard_normal((4096, 96)).astype(dtype.numpy)
    rows = rng.integers(0, 257, size=(4096,))
    check_close(hip_backend, oracle_backend, lambda: Tensor(data=vals).scatter(0, 257, Tensor(data=rows)),
                TOL[dtype])


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_log_softmax_grad(hip_backend, oracle_backend, dtype):
    from honeycrisp_amd.backend import Backend
    rng = np.random.default_rng(33)
    for shape, axis in [((64, 300), 1), ((7, 33, 40), 1), ((5, 1, 9), 2), ((3, 1000), 0), ((2048, 256), 1),
                        ((4096, 96), 0), ((2, 3000, 40), 1), ((16, 5000), 1), ((9, 33000), 1),
                        ((7000, 3), 1), ((3001, 8), 1), ((1000, 100), 1), ((999, 128), 1), ((2, 70000), 1)]:
        x, g = rand(rng, shape, dtype, 2.0), rand(rng, shape, dtype)
        def run():
            xt, gt = Tensor(data=x), Tensor(data=g)
            data = Backend.current().logSoftmaxGrad(xt.data, gt.data, xt.reduceDims(axis), dtype)
            return Tensor(dataHandle=data, shape=list(shape), dtype=dtype)
        check_close(hip_backend, oracle_backend, run, TOL[dtype])


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_clamp(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(34)
    x, lo = rand(rng, (33, 1, 40), dtype), rand(rng, (1, 17, 40), dtype)
    hi = rand(rng, (33, 17, 1), dtype)
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x).clamp(min=Tensor(data=lo), max=Tensor(data=hi)))
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x).clamp(min=Tensor(data=lo)))
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x).clamp(max=Tensor(data=hi)))
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x).clamp(min=-1, max=2))
    flat = rand(rng, (100003,), dtype)
    check_exact(hip_backend, oracle_backend, lambda: Tensor(data=flat).clamp(min=-1))
    if dtype != I64:
        special = np.array([np.nan, -np.inf, np.inf, -0.0, 0.0, 1.5], dtype=dtype.numpy)
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=special).clamp(min=-1, max=1))


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_adamw_fused_equals_composition(hip_backend, oracle_backend, dtype):
    """The fused kernel against the base class's op-by-op composition run on the same device
    (bit for bit), and against the oracle's composition (tolerance: libm vs device powf)."""
    from honeycrisp_amd.backend import Backend
    rng = np.random.default_rng(35)
    n = 100003
    p, g = rand(rng, (n,), dtype), rand(rng, (n,), dtype)
    m, v = rand(rng, (n,), dtype, 0.1), np.abs(rand(rng, (n,), dtype, 0.1))
    for hyper in [(0.9, 0.999, 1e-8, 0.01, 3e-3, 7.0), (0.25, 0.5, 1e-8, 0.1, 1.0, 1.0), (0.9, 0.0, 1e-6, 0.0, 1e-2, 2.0)]:
        def run(backend, composed):
            with backend.use():
                args = [Tensor(data=a).data for a in (p, g, m, v)]
                fn = (lambda *a: Backend.adamW(backend, *a)) if composed else backend.adamW
                outs = fn(*args, *hyper, n, dtype)
                return [Tensor(dataHandle=d, shape=[n], dtype=dtype).numpy() for d in outs]
        fused, composed, want = run(hip_backend, False), run(hip_backend, True), run(oracle_backend, True)
        bits = {2: np.uint16, 4: np.uint32}[dtype.byteSize]
        for a, b, c in zip(fused, composed, want):
            same = (a.view(bits) == b.view(bits)) | (np.isnan(a) & np.isnan(b))
            assert same.all(), "%d elements differ from the composition" % int((~same).sum())
            assert_close_arrays(a, c, TOL[dtype], TOL[dtype])


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_normalize_grad(hip_backend, oracle_backend, dtype):
    from honeycrisp_amd.backend import Backend
    rng = np.random.default_rng(36)
    tol = 2e-2 if dtype == F16 else 1e-4
    for shape, axis in [((64, 512), 1), ((6, 33, 5), 1)]:
        x, g = rand(rng, shape, dtype), rand(rng, shape, dtype)
        def run():
            xt, gt = Tensor(data=x), Tensor(data=g)
            data = Backend.current().normalizeGrad(xt.data, gt.data, xt.reduceDims(axis), np.float32(1e-3), dtype)
            return Tensor(dataHandle=data, shape=list(shape), dtype=dtype)
        check_close(hip_backend, oracle_backend, run, tol)


def test_bitwise_ops(hip_backend, oracle_backend):
    rng = np.random.default_rng(37)
    a64, b64 = rng.integers(-2**62, 2**62, size=(33, 1, 40)), rng.integers(-2**62, 2**62, size=(1, 17, 40))
    ah, bh = rng.standard_normal((1000, 24)).astype(np.float16), rng.standard_normal((1, 24)).astype(np.float16)
    af = rng.standard_normal((100003,)).astype(np.float32)
    m1, m2 = rng.random((64, 1, 33)) < 0.5, rng.random((1, 9, 33)) < 0.5
    for op in ("__and__", "__or__", "__xor__"):
        check_exact(hip_backend, oracle_backend, lambda: getattr(Tensor(data=a64), op)(Tensor(data=b64)))
        check_exact(hip_backend, oracle_backend, lambda: getattr(Tensor(data=ah), op)(Tensor(data=bh)))
        check_exact(hip_backend, oracle_backend, lambda: getattr(Tensor(data=m1), op)(Tensor(data=m2)))
        check_exact(hip_backend, oracle_backend, lambda: getattr(Tensor(data=a64), op)(0x00ff00ff00ff00ff))
        check_exact(hip_backend, oracle_backend, lambda: getattr(Tensor(data=af), op)(0x7fffffff))


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_cumulative_ops(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(38)
    for shape, axis in [((7, 1000), 1), ((3, 257, 5), 1), ((5000, 3), 0), ((4, 1), 1), ((2, 64), 1), ((1, 70000), 1),
                        ((300, 512), 0), ((4, 200, 256), 1),      # 16-byte column vectors, with / without segments
                        # a lane per row; thousands of segments per line (the carry scan works in waves)
                        ((5000, 3), 1), ((777, 16), 1), ((40000, 3), 0), ((30000, 64), 0)]:
        # small integers: every partial sum is exact, so the scan order cannot matter
        x = rng.integers(-3, 4, size=shape)
        x = x if dtype == I64 else x.astype(dtype.numpy)
        for exclusive in (False, True):
            for reverse in (False, True):
                if dtype == F16 and shape[axis] > 2000:
                    continue        # running sums leave the range in which halfs are exact integers
                check_exact(hip_backend, oracle_backend,
                            lambda: Tensor(data=x).cumulativeSum(axis, exclusive=exclusive, reverse=reverse))
        signs = rng.choice([-1, 1], size=shape) * rng.choice([1, 1, 1, 2], size=shape)
        short = tuple(slice(0, 12) if a == axis else slice(None) for a in range(len(shape)))
        y = signs[short] if dtype == I64 else signs[short].astype(dtype.numpy)
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=y).cumulativeProd(axis))
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=y).cumulativeProd(axis, exclusive=True, reverse=True))
    if dtype != I64:
        # general floats: the device combines in tree / segment order, the CPU sequentially
        for shape, axis in [((16, 3000), 1), ((2, 20000), 1), ((6000, 4), 0), ((3000, 256), 0)]:
            r = rand(rng, shape, dtype)
            for reverse in (False, True):
                got, want = both(hip_backend, oracle_backend, lambda: Tensor(data=r).cumulativeSum(axis, reverse=reverse))
                assert_close_arrays(got, want, TOL[dtype] * 60, TOL[dtype])


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_argsort(hip_backend, oracle_backend, dtype):
    rng = np.random.default_rng(39)
    for shape, axis in [((9, 100), 1), ((3, 4096), 1), ((5, 77, 6), 1), ((300, 2), 0), ((4, 1), 1), ((2, 1025), 1)]:
        x = rng.integers(-20, 21, size=shape)           # many ties: the stable order is pinned
        x = x if dtype == I64 else x.astype(dtype.numpy)
        for descending in (False, True):
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x).argsort(axis, descending=descending, stable=True))
    if dtype != I64:
        f = rand(rng, (6, 999), dtype)
        f[0, :5] = [0.0, -0.0, np.inf, -np.inf, 0.0]
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=f).argsort(1))


@pytest.mark.parametrize("dtype", [F32, F16, I64], ids=["f32", "f16", "i64"])
def test_argsort_long_axes(hip_backend, oracle_backend, dtype):
    """Axes beyond one in-LDS sort: runs of 4096 merged pairwise (1, 2, 3 and 4 merge passes, ragged last
    runs, a strided inner axis)."""
    rng = np.random.default_rng(40)
    for shape, axis in [((2, 4097), 1), ((3, 8192), 1), ((2, 10000), 1), ((1, 50257), 1), ((12289, 3), 0),
                        ((2, 5000, 2), 1)]:
        x = rng.integers(-300, 301, size=shape)         # many ties across runs
        x = x if dtype == I64 else x.astype(dtype.numpy)
        for descending in (False, True):
            check_exact(hip_backend, oracle_backend, lambda: Tensor(data=x).argsort(axis, descending=descending, stable=True))
    if dtype != I64:
        f = rand(rng, (2, 20000), dtype)
        check_exact(hip_backend, oracle_backend, lambda: Tensor(data=f).argsort(1))
        got, _ = both(hip_backend, oracle_backend, lambda: Tensor(data=f).gather(1, Tensor(data=f).argsort(1)))
        assert np.all(np.diff(got.astype(np.float32), axis=1) >= 0)


@pytest.mark.parametrize("dtype", [F32, F16], ids=["f32", "f16"])
def test_matmul_pointers_at_odd_element_offsets(hip_backend, oracle_backend, dtype):
    """Straight through the C ABI: operands and output that start 1, 3 and 5 elements into their
    allocations (a view into a larger buffer), so that no pointer is 16-byte aligned and, for
    fp16, some are not even 4-byte aligned. Aligned and odd extents, large enough for the padded
    copies; the elements around the output must stay untouched."""
    from ctypes import c_void_p
    lib, ctx = hip_backend._lib, hip_backend._ctx
    es = np.dtype(dtype.numpy).itemsize
    rng = np.random.default_rng(909)
    for (M, K, N) in [(256, 512, 256), (255, 513, 259), (130, 1000, 131)]:
        a = rand(rng, (M, K), dtype, 1.0 / K ** 0.5)
        b = rand(rng, (K, N), dtype)
        with oracle_backend.use():
            want = Tensor.matmul(Tensor(data=a), False, Tensor(data=b), False, False).numpy()
        offs = (1, 3, 5)
        host_a = np.zeros(M * K + 16, dtype=a.dtype)
        host_a[offs[0]:offs[0] + M * K] = a.reshape(-1)
        host_b = np.zeros(K * N + 16, dtype=a.dtype)
        host_b[offs[1]:offs[1] + K * N] = b.reshape(-1)
        guard = rand(rng, (M * N + 16,), dtype)
        da, db, dc = hip_backend.upload(host_a), hip_backend.upload(host_b), hip_backend.upload(guard)
        print("matmul at odd offsets", dtype.name, M, K, N, flush=True)
        hip_backend._check(lib.hc_matmul(ctx, int(dtype), 1, c_void_p(da.ptr + offs[0] * es), 0,
                                         c_void_p(db.ptr + offs[1] * es), 0, 0, M, K, N, c_void_p(dc.ptr + offs[2] * es)))
        out = dc.onCPU().view(a.dtype)
        got = out[offs[2]:offs[2] + M * N].reshape(M, N)
        assert_close_arrays(got, want, TOL[dtype], TOL[dtype])
        bits = np.uint16 if dtype is F16 else np.uint32
        assert np.array_equal(out[:offs[2]].view(bits), guard[:offs[2]].view(bits))
        assert np.array_equal(out[offs[2] + M * N:].view(bits), guard[offs[2] + M * N:].view(bits))
