"""Error behaviour of the C ABI on a live context: status codes and messages instead of
crashes, mapped to the reference's BackendError cases (Backend.swift:6-16). Every call here
is rejected on the host before anything is enqueued."""
import ctypes
from ctypes import byref, c_float, c_int64, c_size_t, c_void_p

import numpy as np
import pytest

from honeycrisp_amd import _lib
from honeycrisp_amd.descriptors import BackendError, DType
from honeycrisp_amd.tensor import Tensor

pytestmark = pytest.mark.gpu


def status_and_message(backend, status):
    return status, backend._lib.hc_last_error_string().decode()


def test_status_codes_for_bad_arguments(hip_backend):
    lib, ctx = hip_backend._lib, hip_backend._ctx
    buf = hip_backend.allocate(4096)
    p = c_void_p(buf.ptr)
    # a dtype matmul has no arithmetic for
    s, msg = status_and_message(hip_backend, lib.hc_matmul(ctx, int(DType.bool), 1, p, 0, p, 0, 0, 2, 2, 2, p))
    assert s == _lib.HC_ERR_UNSUPPORTED and "not numeric" in msg
    # negative dimension, null pointers
    assert lib.hc_matmul(ctx, int(DType.float32), 1, p, 0, p, 0, 0, -1, 2, 2, p) == _lib.HC_ERR_INVALID
    assert lib.hc_matmul(ctx, int(DType.float32), 1, None, 0, p, 0, 0, 2, 2, 2, p) == _lib.HC_ERR_INVALID
    assert lib.hc_reduce(ctx, 99, int(DType.float32), p, p, 1, 4, 1) == _lib.HC_ERR_INVALID
    # arg-reduction over an empty axis is refused, a sum over it is fine
    assert lib.hc_reduce(ctx, 2, int(DType.float32), p, p, 4, 0, 1) == _lib.HC_ERR_INVALID
    assert lib.hc_reduce(ctx, 0, int(DType.float32), p, p, 4, 0, 1) == _lib.HC_OK
    # logSoftmax of a non-float dtype
    assert lib.hc_log_softmax(ctx, int(DType.int64), p, p, 1, 4, 1) == _lib.HC_ERR_UNSUPPORTED
    # more than 8 dimensions in a stride descriptor
    bad = _lib.hc_strides()
    bad.ndim = 9
    assert lib.hc_broadcast(ctx, int(DType.float32), p, byref(bad), p) == _lib.HC_ERR_INVALID
    # a permutation that repeats an axis, too many axes, an empty tensor
    two = (c_int64 * 2)
    assert lib.hc_permute(ctx, int(DType.float32), p, two(0, 0), two(4, 4), 2, 1, p) == _lib.HC_ERR_INVALID
    assert lib.hc_permute(ctx, int(DType.float32), p, two(1, 0), two(4, 4), 9, 1, p) == _lib.HC_ERR_INVALID
    assert lib.hc_permute(ctx, int(DType.float32), None, two(1, 0), two(4, 0), 2, 1, None) == _lib.HC_OK
    # freeing something the context never handed out, or twice
    assert lib.hc_free(ctx, c_void_p(buf.ptr + 64)) == _lib.HC_ERR_INVALID
    q = c_void_p()
    assert lib.hc_malloc(ctx, c_size_t(1024), byref(q)) == _lib.HC_OK
    assert lib.hc_free(ctx, q) == _lib.HC_OK
    assert lib.hc_free(ctx, q) == _lib.HC_ERR_INVALID
    # an allocation nobody can satisfy
    s, msg = status_and_message(hip_backend, lib.hc_malloc(ctx, c_size_t(1 << 50), byref(q)))
    assert s == _lib.HC_ERR_ALLOC and "bytes" in msg
    # zero-sized work is a no-op, not an error
    assert lib.hc_matmul(ctx, int(DType.float16), 0, None, 0, None, 0, 0, 8, 8, 8, None) == _lib.HC_OK
    assert lib.hc_elemwise(ctx, 0, int(DType.float32), None, None, None, c_size_t(0)) == _lib.HC_OK
    hip_backend.sync()


def test_alignment_contract(hip_backend):
    """Views that start in the middle of an allocation: the contiguous maps and row kernels ask
    for 16-byte aligned buffers (HC_ERR_INVALID with a message that says so), the broadcasting
    and data-movement entry points take any element-aligned pointer and compute the same values."""
    lib, ctx = hip_backend._lib, hip_backend._ctx
    F32 = int(DType.float32)
    x = np.arange(64, dtype=np.float32)
    buf, out = hip_backend.upload(np.concatenate([[0.0], x]).astype(np.float32)), hip_backend.allocate(4 * 80)
    view, dst = c_void_p(buf.ptr + 4), c_void_p(out.ptr + 4)        # 4-byte aligned only
    whole = c_void_p(out.ptr)
    for status in (lib.hc_elemwise(ctx, 11, F32, view, None, whole, c_size_t(64)),
                   lib.hc_elemwise(ctx, 11, F32, c_void_p(buf.ptr), None, dst, c_size_t(64)),
                   lib.hc_cast(ctx, view, F32, whole, int(DType.float16), c_size_t(64)),
                   lib.hc_pow(ctx, F32, view, c_float(2.0), c_float(1.0), 0, 0, None, whole, c_size_t(64)),
                   lib.hc_binary_op_scalar(ctx, 0, F32, view, c_float(1.0), 0, 0, whole, c_size_t(64)),
                   lib.hc_fill(ctx, F32, c_float(1.0), 0, dst, c_size_t(64)),
                   lib.hc_log_softmax(ctx, F32, view, whole, 4, 16, 1),
                   lib.hc_normalize(ctx, F32, view, whole, 4, 16, 1, c_float(1e-5)),
                   lib.hc_reduce(ctx, 0, F32, view, whole, 4, 16, 1)):
        assert status == _lib.HC_ERR_INVALID
        assert "16-byte aligned" in lib.hc_last_error_string().decode()
    # element-aligned views are fine here
    s = _lib.make_strides([64], [1])
    hip_backend._check(lib.hc_binary_op(ctx, 0, F32, view, byref(s), view, byref(s), dst))
    got = out.onCPU().view(np.float32)[1:65]
    assert np.array_equal(got, x + x)
    hip_backend._check(lib.hc_reduce(ctx, 0, F32, view, dst, 1, 8, 8))       # column sums, inner > 1
    assert np.array_equal(out.onCPU().view(np.float32)[1:9], x.reshape(8, 8).sum(0))
    idx = hip_backend.upload(np.array([3, 0, 5], dtype=np.int64))
    si = _lib.make_strides([3, 8], [1, 0])
    hip_backend._check(lib.hc_gather(ctx, F32, view, c_void_p(idx.ptr), byref(si), dst, 1, 8, 3, 8))
    assert np.array_equal(out.onCPU().view(np.float32)[1:25].reshape(3, 8), x.reshape(8, 8)[[3, 0, 5]])


def test_errors_surface_as_backend_errors(hip_backend):
    with hip_backend.use():
        x = Tensor(data=np.arange(6, dtype=np.int64).reshape(2, 3))
        with pytest.raises(BackendError) as e:
            x.logSoftmax(axis=1)                                  # no integer logSoftmax on any backend
        assert e.value.kind == "notImplemented"
        with pytest.raises(BackendError) as e:
            hip_backend.allocate(1 << 50)
        assert e.value.kind == "allocationFailed"
        # the context keeps working afterwards
        assert np.array_equal((x + 1).numpy(), np.arange(6).reshape(2, 3) + 1)


def test_replay_api_misuse_is_reported(hip_backend):
    lib, ctx = hip_backend._lib, hip_backend._ctx
    g = c_void_p()
    assert lib.hc_capture_end(ctx, byref(g)) == _lib.HC_ERR_INVALID       # nothing being recorded
    assert lib.hc_capture_begin(ctx) == _lib.HC_OK
    assert lib.hc_capture_begin(ctx) == _lib.HC_ERR_INVALID               # one recording at a time
    assert lib.hc_sync(ctx) == _lib.HC_ERR_INVALID
    assert lib.hc_capture_abort(ctx) == _lib.HC_OK
    assert lib.hc_sync(ctx) == _lib.HC_OK
