"""hc_reduce_noalloc (the entry point for callers that cannot allocate device memory) against
hc_reduce, straight through the C ABI: same kernels, partial results in the library's fixed
device array instead of pool blocks. Results must agree bit for bit, on two calls in a row
(the second with a smaller input, so that it finds the first call's partials in the array), and
the context's pool must not move."""
from ctypes import byref, c_size_t, c_void_p

import numpy as np
import pytest

from honeycrisp_amd import _lib
from honeycrisp_amd.descriptors import DType

pytestmark = pytest.mark.gpu

F32, F16, I64 = DType.float32, DType.float16, DType.int64
SUM, PROD, ARGMAX, ARGMIN = 0, 1, 2, 3


def pool(hip):
    in_use, cached = c_size_t(0), c_size_t(0)
    hip._check(hip._lib.hc_mem_stats(hip._ctx, byref(in_use), byref(cached)))
    return in_use.value, cached.value


def reduce_both(hip, op, dtype, x, outer, reduce, inner):
    """(hc_reduce result, hc_reduce_noalloc result) as raw bytes, plus the pool before / after the
    no-allocation call."""
    lib, ctx = hip._lib, hip._ctx
    out_bytes = outer * inner * (8 if op in (ARGMAX, ARGMIN) or dtype is I64 else np.dtype(dtype.numpy).itemsize)
    src = hip.upload(x)
    # outputs start out different, so a call that writes nothing cannot pass
    ref_out, out = hip.upload(np.full(out_bytes, 0x5A, np.uint8)), hip.upload(np.full(out_bytes, 0xA5, np.uint8))
    hip._check(lib.hc_reduce(ctx, op, int(dtype), c_void_p(src.ptr), c_void_p(ref_out.ptr), outer, reduce, inner))
    before = pool(hip)
    hip._check(lib.hc_reduce_noalloc(ctx, op, int(dtype), c_void_p(src.ptr), c_void_p(out.ptr), outer, reduce, inner))
    after = pool(hip)
    return ref_out.onCPU(), out.onCPU(), before, after


def make(rng, dtype, shape):
    if dtype is I64:
        return rng.integers(-1000, 1000, size=shape)
    x = rng.standard_normal(shape).astype(dtype.numpy)
    return x


# (op, dtype, [outer, reduce, inner] of the first call, of the second, smaller call)
CASES = [
    (SUM, F32, (1, 4096, 2048), (1, 1000, 333)),       # column reduction cut into ranges
    (ARGMAX, F32, (2, 3000, 1024), (1, 700, 40)),      # the same with (value, index) partials
    (ARGMIN, F16, (1, 8192, 4096), (3, 513, 24)),
    (SUM, I64, (1, 5000, 512), (1, 300, 64)),
    (SUM, F32, (3, 500000, 1), (2, 70000, 1)),         # long rows cut into segments
    (ARGMAX, F16, (4, 300001, 1), (1, 40000, 1)),
    (PROD, F32, (1, 2048, 256), (1, 128, 256)),
    (SUM, F32, (8192, 4096, 1), (100, 37, 1)),         # forms without partials pass through unchanged
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "%d-%s-%s" % (c[0], c[1].name, "x".join(map(str, c[2]))))
def test_two_calls_in_a_row_match_hc_reduce(hip_backend, case):
    op, dtype, first, second = case
    rng = np.random.default_rng(sum(first) + op)
    for (outer, reduce, inner) in (first, second):
        x = make(rng, dtype, (outer, reduce, inner))
        if op == PROD:
            x = (1.0 + 0.001 * x).astype(dtype.numpy)
        if op in (ARGMAX, ARGMIN):  # ties across ranges / segments: the first one must win
            x[:, reduce // 7] = x[:, reduce - 1] = (50 if op == ARGMAX else -50)
        print("hc_reduce_noalloc", op, dtype.name, outer, reduce, inner, flush=True)
        want, got, before, after = reduce_both(hip_backend, op, dtype, x, outer, reduce, inner)
        assert np.array_equal(got, want)
        assert before == after, "the call moved the context's pool: %r -> %r" % (before, after)


def test_partials_beyond_the_fixed_array_are_refused(hip_backend):
    """fp16 argmax over [192, 523776] along axis 0: 3 ranges x 523776 columns x (4 + 4) bytes of
    partials = 12.6 MB, more than the array holds."""
    lib, ctx = hip_backend._lib, hip_backend._ctx
    outer, reduce, inner = 1, 192, 1023 * 512
    src = hip_backend.allocate(outer * reduce * inner * 2)
    hip_backend._check(lib.hc_fill(ctx, int(F16), 1.0, 0, c_void_p(src.ptr), outer * reduce * inner))
    out = hip_backend.allocate(outer * inner * 8)
    status = lib.hc_reduce_noalloc(ctx, ARGMAX, int(F16), c_void_p(src.ptr), c_void_p(out.ptr), outer, reduce, inner)
    assert status == _lib.HC_ERR_TOO_LARGE
    message = lib.hc_last_error_string().decode()
    assert "scratch" in message and str(8 << 20) in message
    # the allocating entry point takes the same call
    hip_backend._check(lib.hc_reduce(ctx, ARGMAX, int(F16), c_void_p(src.ptr), c_void_p(out.ptr), outer, reduce, inner))
    assert not out.onCPU().view(np.int64).any()
