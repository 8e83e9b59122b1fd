"""Host-side mirror of Honeycrisp's `Backend` op interface and its MI355X implementation.

`Backend` restates the open class of Sources/Honeycrisp/Backend.swift:28-890 (same method
names, argument meaning and error behaviour: every op of the bare base class raises
`BackendError.notImplemented`, `normalize` and `repeated` have the base-class compositions).
`HIPBackend` is the drop-in for the ops on the hot path: each method enqueues one call of
the C ABI (include/hchip.h) on the context's in-order stream and returns a device buffer
(`HIPData`, the `Tensor.Data` of this backend) immediately.

There is no CPU fallback here: an op or dtype the kernels do not cover raises
`BackendError.notImplemented`, and a missing libhchip.so is an ImportError.
"""
import contextlib
import ctypes
import os
import threading
from ctypes import byref, c_float, c_int64, c_size_t, c_void_p
from typing import List, Optional, Sequence, Union

import numpy as np

from . import _lib
from .descriptors import (BackendError, BitwiseOp, BroadcastData, BroadcastStrides, ComparisonOp, DType,
                          ElemwiseOp, NumericBinaryOp, ReduceDims, ReduceOp, RepeatDims,
                          ScatterGatherIndices, product)


class Backend:
    """Abstract op set (Backend.swift:170-815)."""

    _default: Optional["Backend"] = None
    _tls = threading.local()

    # -- Backend.defaultBackend / current / use (Backend.swift:44-88)
    @classmethod
    def setDefault(cls, backend: "Backend"):
        Backend._default = backend

    @classmethod
    def current(cls) -> "Backend":
        stack = getattr(Backend._tls, "stack", None)
        if stack:
            return stack[-1]
        if Backend._default is None:
            raise RuntimeError("no default backend installed (Backend.setDefault)")
        return Backend._default

    class _Use:
        def __init__(self, backend):
            self.backend = backend

        def __enter__(self):
            if not hasattr(Backend._tls, "stack"):
                Backend._tls.stack = []
            Backend._tls.stack.append(self.backend)
            return self.backend

        def __exit__(self, *exc):
            Backend._tls.stack.pop()
            return False

    def use(self):
        return Backend._Use(self)

    def _ni(self, name):
        raise BackendError.notImplemented(name)

    def allocate(self, byteCount):
        self._ni("allocate")

    def broadcast(self, a, dtype):
        self._ni("broadcast")

    def binaryOp(self, a, b, op, dtype, count=None):
        self._ni("binaryOp")

    def mulAdd(self, input, coeff, bias, dtype):
        self._ni("mulAdd")

    def addMul(self, input, bias, coeff, dtype):
        self._ni("addMul")

    def compare(self, a, b, op, dtype, count=None):
        self._ni("compare")

    def cast(self, a, count, inType, outType):
        self._ni("cast")

    def pow(self, a, b, scale, scales, count, dtype):
        self._ni("pow")

    def reduce(self, a, op, dims, dtype):
        self._ni("reduce")

    def logSoftmax(self, a, dims, dtype):
        self._ni("logSoftmax")

    def gather(self, a, s, dtype):
        self._ni("gather")

    def scatter(self, a, s, dtype):
        self._ni("scatter")

    def bitwiseOp(self, a, b, op, dtype, count=None):
        """a, b: BroadcastData, or one of them an integer bit pattern of the element's size
        (Backend.swift:215-237)."""
        self._ni("bitwiseOp")

    @staticmethod
    def scalarBits(value: int, dtype: DType) -> np.ndarray:
        """The bytes of an element-sized bit pattern (TensorElementBitPattern.bitsForBitwiseOp)."""
        size = dtype.byteSize
        return np.frombuffer((int(value) & ((1 << (8 * size)) - 1)).to_bytes(size, "little"), dtype=np.uint8).copy()

    def logSoftmaxGrad(self, a, outGrad, dims, dtype):
        self._ni("logSoftmaxGrad")

    def cumulativeSum(self, a, dims, exclusive, reverse, dtype):
        self._ni("cumulativeSum")

    def cumulativeProd(self, a, dims, exclusive, reverse, dtype):
        self._ni("cumulativeProd")

    def argsort(self, a, dims, descending, stable, dtype):
        self._ni("argsort")

    def clamp(self, a, min, max, dtype):
        self._ni("clamp")

    def when(self, mask, a, b, dtype):
        self._ni("when")

    def matmul(self, a, transA, b, transB, transOut, rows, inner, cols, dtype):
        self._ni("matmul")

    def batchedMatmul(self, matrixCount, a, transA, b, transB, transOut, rows, inner, cols, dtype):
        self._ni("batchedMatmul")

    def triangular(self, a, batch, rows, cols, upper, offset, dtype):
        self._ni("triangular")

    def elemwise(self, a, op, scales, count, dtype):
        self._ni("elemwise")

    def concat(self, inputs, outerCount, innerCounts, dtype):
        self._ni("concat")

    def constant(self, value, count, dtype):
        self._ni("constant")

    def collection(self, collection, reverse, dtype):
        self._ni("collection")

    def axisPermutation(self, permutation, shape):
        self._ni("axisPermutation")

    # -- base-class compositions

    def repeated(self, a, dims: RepeatDims, dtype):
        """Backend.swift:590-606."""
        return self.broadcast(
            BroadcastData(
                BroadcastStrides([dims.outerCount, dims.repeatCount, dims.innerCount],
                                 [dims.innerCount, 0, 1]), a), dtype)

    def normalize(self, input, dims: ReduceDims, eps, dtype):
        """Backend.swift:265-327: two-pass mean / biased variance, op by op."""
        full = BroadcastStrides.contiguousForShape([dims.outerCount, dims.reduceCount, dims.innerCount])
        reduced = BroadcastStrides(full.shape, [dims.innerCount, 0, 1])
        inv_n = np.float32(1.0) / np.float32(dims.reduceCount)
        mean = self.binaryOp(self.reduce(input, ReduceOp.sum, dims, dtype), inv_n, NumericBinaryOp.mul,
                             dtype, count=reduced.dataCount)
        centered = self.binaryOp(BroadcastData(full, input), BroadcastData(reduced, mean),
                                 NumericBinaryOp.sub, dtype)
        variance = self.binaryOp(
            self.reduce(self.pow(centered, 2.0, 1.0, None, full.dataCount, dtype), ReduceOp.sum, dims, dtype),
            inv_n, NumericBinaryOp.mul, dtype, count=reduced.dataCount)
        normalizer = self.pow(
            self.binaryOp(variance, eps, NumericBinaryOp.add, dtype, count=reduced.dataCount),
            -0.5, 1.0, None, reduced.dataCount, dtype)
        return self.binaryOp(BroadcastData(full, centered), BroadcastData(reduced, normalizer),
                             NumericBinaryOp.mul, dtype)


    def normalizeGrad(self, input, outGrad, dims: ReduceDims, eps, dtype):
        """Backend.swift:332-455, op by op."""
        f32 = np.float32
        full = BroadcastStrides.contiguousForShape([dims.outerCount, dims.reduceCount, dims.innerCount])
        reduced = BroadcastStrides(full.shape, [dims.innerCount, 0, 1])
        inv_n = f32(1.0) / f32(dims.reduceCount)
        n_red = reduced.dataCount
        bd_full = lambda d: BroadcastData(full, d)
        bd_red = lambda d: BroadcastData(reduced, d)
        mean = self.binaryOp(self.reduce(input, ReduceOp.sum, dims, dtype), inv_n, NumericBinaryOp.mul,
                             dtype, count=n_red)
        centered = self.binaryOp(bd_full(input), bd_red(mean), NumericBinaryOp.sub, dtype)
        variance = self.binaryOp(
            self.reduce(self.pow(centered, 2.0, 1.0, None, full.dataCount, dtype), ReduceOp.sum, dims, dtype),
            inv_n, NumericBinaryOp.mul, dtype, count=n_red)
        stable = self.binaryOp(variance, eps, NumericBinaryOp.add, dtype, count=n_red)
        normalizer1 = self.pow(stable, -0.5, 1.0, None, n_red, dtype)
        normalizer2 = self.pow(stable, -1.5, f32(1) / f32(dims.reduceCount), None, n_red, dtype)
        meanGrad = self.binaryOp(self.reduce(outGrad, ReduceOp.sum, dims, dtype), f32(1) / f32(dims.reduceCount),
                                 NumericBinaryOp.mul, dtype, count=n_red)
        centeredGrad = self.binaryOp(bd_full(outGrad), bd_red(meanGrad), NumericBinaryOp.sub, dtype)
        covTerm = self.reduce(self.binaryOp(bd_full(centered), bd_full(outGrad), NumericBinaryOp.mul, dtype),
                              ReduceOp.sum, dims, dtype)
        term1 = self.binaryOp(bd_full(centeredGrad), bd_red(normalizer1), NumericBinaryOp.mul, dtype)
        covTimesCentered = self.binaryOp(bd_full(centered), bd_red(covTerm), NumericBinaryOp.mul, dtype)
        term2 = self.binaryOp(bd_full(covTimesCentered), bd_red(normalizer2), NumericBinaryOp.mul, dtype)
        return self.binaryOp(bd_full(term1), bd_full(term2), NumericBinaryOp.sub, dtype)

    def adamW(self, param, grad, moment1, moment2, beta1, beta2, eps, weightDecay, lr, step, count, dtype):
        """Backend.swift:818-892, op by op; returns (param, moment1, moment2). All scalar
        arithmetic is in Float as there."""
        f32 = np.float32
        beta1, beta2, eps, weightDecay, lr, step = (f32(v) for v in (beta1, beta2, eps, weightDecay, lr, step))
        bd = lambda d: BroadcastData(BroadcastStrides.contiguousForShape([count]), d)
        mul, add, sub, div = NumericBinaryOp.mul, NumericBinaryOp.add, NumericBinaryOp.sub, NumericBinaryOp.div
        newMt = self.binaryOp(bd(self.binaryOp(beta1, moment1, mul, dtype, count=count)),
                              bd(self.binaryOp(f32(1) - beta1, grad, mul, dtype, count=count)), add, dtype)
        gradSq = self.pow(grad, 2.0, f32(1) - beta2, None, count, dtype)
        newVt = self.binaryOp(bd(self.binaryOp(beta2, moment2, mul, dtype, count=count)), bd(gradSq), add, dtype)
        scaledMt = self.binaryOp(newMt, f32(1.0) / (f32(1) - powf(beta1, step)), mul, dtype, count=count)
        scaledVt = self.binaryOp(newVt, f32(1.0) / (f32(1) - powf(beta2, step)), mul, dtype, count=count)
        denom = self.binaryOp(self.pow(scaledVt, 0.5, 1.0, None, count, dtype), eps, add, dtype, count=count)
        stepDir = self.binaryOp(self.binaryOp(bd(scaledMt), bd(denom), div, dtype), lr, mul, dtype, count=count)
        decayed = self.binaryOp(param, f32(1) - lr * weightDecay, mul, dtype, count=count)
        newParam = self.binaryOp(bd(decayed), bd(stepDir), sub, dtype)
        return newParam, newMt, newVt


_libm = ctypes.CDLL("libm.so.6")
_libm.powf.restype = ctypes.c_float
_libm.powf.argtypes = [ctypes.c_float, ctypes.c_float]


def powf(x, y) -> np.float32:
    """C powf (Foundation.pow on Float)."""
    return np.float32(_libm.powf(float(x), float(y)))


class HIPData:
    """Device buffer backing a tensor: this backend's `Tensor.Data` (Tensor.swift:69-85)."""

    def __init__(self, backend: "HIPBackend", ptr: int, byteCount: int):
        self.backend = backend
        self.ptr = ptr
        self.byteCount = byteCount

    def wait(self):
        self.backend.sync()

    def onCPU(self) -> np.ndarray:
        """Host copy of the bytes (blocking, ordered after all enqueued work)."""
        host = np.empty(self.byteCount, dtype=np.uint8)
        if self.byteCount:
            self.backend._check(self.backend._lib.hc_memcpy_d2h(
                self.backend._ctx, host.ctypes.data_as(c_void_p), c_void_p(self.ptr), self.byteCount))
        return host

    def mutateOnCPU(self, fn):
        """`fn(host_bytes)` edits a host copy in place; the result is written back
        (Tensor.Data.mutateOnCPU, Tensor.swift:69-85). Blocking."""
        host = self.onCPU()
        fn(host)
        if self.byteCount:
            self.backend._check(self.backend._lib.hc_memcpy_h2d(
                self.backend._ctx, c_void_p(self.ptr), host.ctypes.data_as(c_void_p), self.byteCount))

    def __del__(self):
        backend, ptr = self.backend, self.ptr
        self.ptr = None
        if ptr and backend is not None and backend._ctx:
            backend._lib.hc_free(backend._ctx, c_void_p(ptr))


class PermutationData(HIPData):
    """The int64 index vector of axisPermutation(permutation, shape), produced on first use of its
    pointer: the usual consumer is the gather of t / swap / move, which HIPBackend.gather runs as a
    direct copy from (permutation, shape) alone, so most vectors are never written."""

    def __init__(self, backend: "HIPBackend", permutation, shape):
        self.backend = backend
        self.permutation = (tuple(permutation), tuple(shape))
        self.byteCount = product(shape) * 8
        self._ptr = None

    @property
    def ptr(self):
        if self._ptr is None and self.backend is not None:
            backend = self.backend
            perm, shape = self.permutation
            n = len(shape)
            block = backend.allocate(self.byteCount)
            self._ptr, block.ptr = block.ptr, None      # this object owns the block now
            backend._check(backend._lib.hc_axis_permutation(
                backend._ctx, (c_int64 * max(n, 1))(*perm), (c_int64 * max(n, 1))(*shape), n, c_void_p(self._ptr)))
            if backend._capturing:
                # written by a recorded kernel, i.e. not before the graph runs: stop sharing it
                backend._perm_cache.pop(self.permutation, None)
        return self._ptr

    @ptr.setter
    def ptr(self, value):
        self._ptr = value

    def __del__(self):
        backend, ptr = self.backend, self._ptr
        self._ptr = None
        if ptr and backend is not None and backend._ctx:
            backend._lib.hc_free(backend._ctx, c_void_p(ptr))


Scalar = Union[int, float, np.floating, np.integer]


class Graph:
    """A recorded sequence of backend ops (see HIPBackend.capture)."""

    def __init__(self, backend: "HIPBackend", handle: int):
        self.backend, self._handle = backend, handle

    def launch(self):
        self.backend._check(self.backend._lib.hc_graph_launch(self.backend._ctx, c_void_p(self._handle)))

    def node_count(self) -> int:
        """Kernel launches and copies one replay issues (after the recording's rewrite)."""
        n = c_size_t(0)
        self.backend._check(self.backend._lib.hc_graph_node_count(c_void_p(self._handle), byref(n)))
        return int(n.value)

    def destroy(self):
        if self._handle and self.backend._ctx:
            self.backend._check(self.backend._lib.hc_graph_destroy(self.backend._ctx, c_void_p(self._handle)))
        self._handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class Capture:
    def __init__(self, backend: "HIPBackend"):
        self.backend, self.graph = backend, None

    def __enter__(self):
        self.backend._check(self.backend._lib.hc_capture_begin(self.backend._ctx))
        self.backend._capturing = True
        return self

    def __exit__(self, exc_type, exc, tb):
        self.backend._capturing = False
        if exc_type is not None:
            self.backend._lib.hc_capture_abort(self.backend._ctx)
            return False
        handle = c_void_p()
        self.backend._check(self.backend._lib.hc_capture_end(self.backend._ctx, byref(handle)))
        self.graph = Graph(self.backend, handle.value)
        return False


class HIPBackend(Backend):
    """MI355X backend: one device, one in-order stream, kernels from libhchip.so."""

    def __init__(self, device: int = 0):
        self._ctx = None
        self._capturing = False
        self._perm_cache, self._perm_cache_bytes = {}, 0
        self._lib = _lib.load()
        ctx = c_void_p()
        status = self._lib.hc_init(device, byref(ctx))
        if status != _lib.HC_OK:
            self._raise(status)
        self._ctx = ctx
        # hc_set_batching's current values (HCHIP_BATCHING in the environment gives a context its first)
        env = (os.environ.get("HCHIP_BATCHING") or "0").split(",")
        self._batching = (int(env[0]), int(env[1]) if len(env) > 1 else 0)

    def close(self):
        if self._ctx:
            self._perm_cache.clear()
            self._lib.hc_shutdown(self._ctx)
            self._ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- errors (mapping of Backend.swift:6-16)

    def _raise(self, status):
        msg = self._lib.hc_last_error_string().decode("utf-8", "replace")
        if status == _lib.HC_ERR_ALLOC:
            raise BackendError.allocationFailed(msg)
        if status in (_lib.HC_ERR_LOAD, _lib.HC_ERR_NO_DEVICE):
            raise BackendError.failedToLoadKernels(msg)
        if status == _lib.HC_ERR_UNSUPPORTED:
            raise BackendError.notImplemented(msg)
        raise BackendError.kernelFailed(msg)

    def _check(self, status):
        if status != _lib.HC_OK:
            self._raise(status)

    # -- device / stream

    def deviceInfo(self) -> dict:
        info = _lib.hc_device_info()
        self._check(self._lib.hc_get_device_info(self._ctx, byref(info)))
        return {
            "name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units,
            "clock_mhz": info.clock_mhz, "wavefront_size": info.wavefront_size,
            "lds_bytes_per_block": info.lds_bytes_per_block, "total_mem": info.total_mem,
        }

    def debugSet(self, name: str, value=None):
        """Sets one of the library's measurement / test switches on this context (hc_debug_set);
        `value` None restores the default."""
        self._check(self._lib.hc_debug_set(self._ctx, name.encode(), None if value is None else str(value).encode()))

    @contextlib.contextmanager
    def switches(self, **kv):
        """`with backend.switches(HCHIP_GEMM_TILE="256x256"):` sets the named switches for the
        block and restores their defaults afterwards."""
        for k, v in kv.items():
            self.debugSet(k, v)
        try:
            yield self
        finally:
            for k in kv:
                self.debugSet(k, None)

    def sync(self):
        self._check(self._lib.hc_sync(self._ctx))

    def memStats(self):
        """(bytes in blocks handed out, bytes in the pool's free blocks) of this context (hc_mem_stats)."""
        used, cached = c_size_t(0), c_size_t(0)
        self._check(self._lib.hc_mem_stats(self._ctx, byref(used), byref(cached)))
        return used.value, cached.value

    def setBatching(self, max_launches: int, idle_after: int = 0):
        """hc_set_batching: with max_launches > 0 the ops of ordinary, call-by-call code are listed
        and enqueued batch by batch, each batch rewritten like a recording (same bits, fewer
        launches); 0 goes back to one launch per call. idle_after > 0: a list of at least that
        many launches is also enqueued as soon as the device has run out of work."""
        self._check(self._lib.hc_set_batching(self._ctx, int(max_launches), int(idle_after)))
        self._batching = (int(max_launches), int(idle_after))

    @contextlib.contextmanager
    def batching(self, max_launches: int = 512, idle_after: int = 0):
        """`with backend.batching():` batches the ops of the block (see setBatching) and restores
        the setting of before afterwards."""
        before = self._batching
        self.setBatching(max_launches, idle_after)
        try:
            yield self
        finally:
            self.setBatching(*before)

    def flush(self):
        """Enqueues what batching has listed so far (hc_flush)."""
        self._check(self._lib.hc_flush(self._ctx))

    def batchingStats(self):
        """(launches listed by batches, launches enqueued in their place) since the context was created."""
        listed, enqueued = ctypes.c_uint64(0), ctypes.c_uint64(0)
        self._check(self._lib.hc_batching_stats(self._ctx, ctypes.byref(listed), ctypes.byref(enqueued)))
        return listed.value, enqueued.value

    def capture(self) -> "Capture":
        """`with backend.capture() as cap: out = model(x)` records every op issued inside the
        block instead of running it; `cap.graph.launch()` then replays the whole recording with
        one call and `out` holds the results of the latest replay. Inputs must be on the device
        before the block (no host transfers inside) and must stay alive while the graph is used.
        Honeycrisp has no counterpart: it pays one backend call per op (Tensor.swift:634-657)."""
        return Capture(self)

    # -- storage (DataAllocator, Backend.swift:894-896)

    def allocate(self, byteCount: int) -> HIPData:
        ptr = c_void_p()
        self._check(self._lib.hc_malloc(self._ctx, c_size_t(max(int(byteCount), 0)), byref(ptr)))
        return HIPData(self, ptr.value, int(byteCount))

    def upload(self, host: np.ndarray) -> HIPData:
        host = np.ascontiguousarray(host)
        data = self.allocate(host.nbytes)
        if host.nbytes:
            self._check(self._lib.hc_memcpy_h2d(self._ctx, c_void_p(data.ptr),
                                                host.ctypes.data_as(c_void_p), host.nbytes))
        return data

    def _dev(self, data) -> HIPData:
        """Device buffer for `data`; foreign data is uploaded (cf. BackendMPS.swift:585-620)."""
        if isinstance(data, HIPData) and data.backend is self:
            return data
        if isinstance(data, np.ndarray):
            return self.upload(data)
        if hasattr(data, "onCPU"):
            return self.upload(data.onCPU())
        raise TypeError("cannot use %r as tensor data" % type(data))

    @staticmethod
    def _s(strides: BroadcastStrides):
        return _lib.make_strides(strides.shape, strides.strides)

    @staticmethod
    def _scalar(value, dtype: DType):
        """(float32 value, int64 value) the way T.toFloat() / T.toInt64() would give them."""
        if dtype == DType.int64:
            return c_float(0.0), c_int64(int(value))
        return c_float(float(np.float32(value))), c_int64(0)

    # -- ops

    def collection(self, collection, reverse: bool, dtype: DType) -> HIPData:
        """Backend.swift:794-800: host values -> buffer of `dtype` (arrayToPointer conversion)."""
        arr = np.asarray(list(collection) if not isinstance(collection, np.ndarray) else collection)
        if reverse:
            arr = arr[::-1]
        return self.upload(convert_host_array(arr.reshape(-1), dtype))

    def constant(self, value, count: int, dtype: DType) -> HIPData:
        out = self.allocate(count * dtype.byteSize)
        vf, vi = self._scalar(value, dtype)
        if dtype != DType.int64:
            vf = c_float(float(np.float32(value)))
        self._check(self._lib.hc_fill(self._ctx, int(dtype), vf, vi, c_void_p(out.ptr), count))
        return out

    def broadcast(self, a: BroadcastData, dtype: DType) -> HIPData:
        out = self.allocate(product(a.strides.shape) * dtype.byteSize)
        ad = self._dev(a.data)
        s = self._s(a.strides)
        self._check(self._lib.hc_broadcast(self._ctx, int(dtype), c_void_p(ad.ptr), byref(s), c_void_p(out.ptr)))
        return out

    def binaryOp(self, a, b, op: NumericBinaryOp, dtype: DType, count: Optional[int] = None) -> HIPData:
        if isinstance(a, BroadcastData) and isinstance(b, BroadcastData):
            out = self.allocate(product(a.strides.shape) * dtype.byteSize)
            ad, bd = self._dev(a.data), self._dev(b.data)
            sa, sb = self._s(a.strides), self._s(b.strides)
            self._check(self._lib.hc_binary_op(self._ctx, int(op), int(dtype), c_void_p(ad.ptr), byref(sa),
                                               c_void_p(bd.ptr), byref(sb), c_void_p(out.ptr)))
            return out
        if count is None:
            raise TypeError("binaryOp with a scalar needs count")
        scalar_first = isinstance(a, (int, float, np.floating, np.integer))
        tensor, scalar = (b, a) if scalar_first else (a, b)
        out = self.allocate(count * dtype.byteSize)
        td = self._dev(tensor)
        sf, si = self._scalar(scalar, dtype)
        self._check(self._lib.hc_binary_op_scalar(self._ctx, int(op), int(dtype), c_void_p(td.ptr), sf, si,
                                                  int(scalar_first), c_void_p(out.ptr), count))
        return out

    def _fused(self, fn, x, y, z, dtype):
        out = self.allocate(product(x.strides.shape) * dtype.byteSize)
        xd, yd, zd = self._dev(x.data), self._dev(y.data), self._dev(z.data)
        sx, sy, sz = self._s(x.strides), self._s(y.strides), self._s(z.strides)
        self._check(fn(self._ctx, int(dtype), c_void_p(xd.ptr), byref(sx), c_void_p(yd.ptr), byref(sy),
                       c_void_p(zd.ptr), byref(sz), c_void_p(out.ptr)))
        return out

    def mulAdd(self, input: BroadcastData, coeff: BroadcastData, bias: BroadcastData, dtype: DType):
        return self._fused(self._lib.hc_mul_add, input, coeff, bias, dtype)

    def addMul(self, input: BroadcastData, bias: BroadcastData, coeff: BroadcastData, dtype: DType):
        return self._fused(self._lib.hc_add_mul, input, bias, coeff, dtype)

    def when(self, mask: BroadcastData, a, b, dtype: DType):
        """a / b: BroadcastData, or ("scalar", value, shape) like Backend.TensorOrScalar
        (Backend.swift:30-42); scalars become 1-element constants with all-zero strides
        (BackendCPU.swift:1860-1868)."""
        def branch(x):
            if isinstance(x, BroadcastData):
                return x
            _, value, shape = x
            return BroadcastData(BroadcastStrides(shape, [0] * len(shape)), self.constant(value, 1, dtype))
        return self._fused(self._lib.hc_when, mask, branch(a), branch(b), dtype)

    def compare(self, a, b, op: ComparisonOp, dtype: DType, count: Optional[int] = None) -> HIPData:
        if isinstance(a, BroadcastData) and isinstance(b, BroadcastData):
            out = self.allocate(product(a.strides.shape))
            ad, bd = self._dev(a.data), self._dev(b.data)
            sa, sb = self._s(a.strides), self._s(b.strides)
            self._check(self._lib.hc_compare(self._ctx, int(op), int(dtype), c_void_p(ad.ptr), byref(sa),
                                             c_void_p(bd.ptr), byref(sb), c_void_p(out.ptr)))
            return out
        if count is None:
            raise TypeError("compare with a scalar needs count")
        scalar_first = isinstance(a, (int, float, bool, np.floating, np.integer, np.bool_))
        tensor, scalar = (b, a) if scalar_first else (a, b)
        out = self.allocate(count)
        td = self._dev(tensor)
        sf, si = self._scalar(scalar, dtype)
        self._check(self._lib.hc_compare_scalar(self._ctx, int(op), int(dtype), c_void_p(td.ptr), sf, si,
                                                int(scalar_first), c_void_p(out.ptr), count))
        return out

    def cast(self, a, count: int, inType: DType, outType: DType) -> HIPData:
        out = self.allocate(count * outType.byteSize)
        ad = self._dev(a)
        self._check(self._lib.hc_cast(self._ctx, c_void_p(ad.ptr), int(inType), c_void_p(out.ptr),
                                      int(outType), count))
        return out

    def pow(self, a, b: Scalar, scale: Scalar, scales, count: int, dtype: DType) -> HIPData:
        out = self.allocate(count * dtype.byteSize)
        ad = self._dev(a)
        sd = self._dev(scales) if scales is not None else None
        bf, bi = self._scalar(b, dtype)
        scf, sci = self._scalar(scale, dtype)
        self._check(self._lib.hc_pow(self._ctx, int(dtype), c_void_p(ad.ptr), bf, scf, bi, sci,
                                     c_void_p(sd.ptr) if sd else None, c_void_p(out.ptr), count))
        return out

    def elemwise(self, a, op: ElemwiseOp, scales, count: int, dtype: DType) -> HIPData:
        out = self.allocate(count * dtype.byteSize)
        ad = self._dev(a)
        sd = self._dev(scales) if scales is not None else None
        self._check(self._lib.hc_elemwise(self._ctx, int(op), int(dtype), c_void_p(ad.ptr),
                                          c_void_p(sd.ptr) if sd else None, c_void_p(out.ptr), count))
        return out

    def reduce(self, a, op: ReduceOp, dims: ReduceDims, dtype: DType) -> HIPData:
        outType = DType.int64 if op.isIntOut else dtype
        out = self.allocate(dims.outCount * outType.byteSize)
        ad = self._dev(a)
        self._check(self._lib.hc_reduce(self._ctx, int(op), int(dtype), c_void_p(ad.ptr), c_void_p(out.ptr),
                                        dims.outerCount, dims.reduceCount, dims.innerCount))
        return out

    def logSoftmax(self, a, dims: ReduceDims, dtype: DType) -> HIPData:
        out = self.allocate(dims.inCount * dtype.byteSize)
        ad = self._dev(a)
        self._check(self._lib.hc_log_softmax(self._ctx, int(dtype), c_void_p(ad.ptr), c_void_p(out.ptr),
                                             dims.outerCount, dims.reduceCount, dims.innerCount))
        return out

    def normalize(self, input, dims: ReduceDims, eps: Scalar, dtype: DType) -> HIPData:
        """Fused override of the base-class composition (same arithmetic, one kernel for
        innerCount == 1)."""
        out = self.allocate(dims.inCount * dtype.byteSize)
        ad = self._dev(input)
        self._check(self._lib.hc_normalize(self._ctx, int(dtype), c_void_p(ad.ptr), c_void_p(out.ptr),
                                           dims.outerCount, dims.reduceCount, dims.innerCount,
                                           c_float(float(np.float32(eps)))))
        return out

    def gather(self, a, s: ScatterGatherIndices, dtype: DType) -> HIPData:
        out = self.allocate(s.gatherOutCount * dtype.byteSize)
        # The gather of t / swap / move / PermuteAxes: its index vector came from axisPermutation
        # and runs along the gathered axis only. One direct copy moves the same bytes without
        # reading 8 bytes of index per element.
        meta = getattr(s.indices.data, "permutation", None)
        st_ = s.indices.strides
        if (meta is not None and st_.shape[s.axis] == s.middleCount == product(meta[1])
                and all(stride == (1 if ax == s.axis else 0) or size == 1
                        for ax, (stride, size) in enumerate(zip(st_.strides, st_.shape)))):
            perm, shape = list(meta[0]), list(meta[1])
            if s.outerCount > 1:
                perm, shape = [0] + [p + 1 for p in perm], [s.outerCount] + shape
            n = len(shape)
            if n <= 8:      # (hc_permute takes up to 8 axes; more fall through to the index gather)
                self._check(self._lib.hc_permute(self._ctx, int(dtype), c_void_p(self._dev(a).ptr),
                                                 (c_int64 * max(n, 1))(*perm), (c_int64 * max(n, 1))(*shape), n,
                                                 s.innerCount, c_void_p(out.ptr)))
                return out
        ad, idx = self._dev(a), self._dev(s.indices.data)
        st = self._s(s.indices.strides)
        self._check(self._lib.hc_gather(self._ctx, int(dtype), c_void_p(ad.ptr), c_void_p(idx.ptr), byref(st),
                                        c_void_p(out.ptr), s.outerCount, s.middleCount, s.outCount,
                                        s.innerCount))
        return out

    def bitwiseOp(self, a, b, op: BitwiseOp, dtype: DType, count: Optional[int] = None) -> HIPData:
        def operand(x, other):
            if isinstance(x, BroadcastData):
                return x
            shape = other.strides.shape
            return BroadcastData(BroadcastStrides(shape, [0] * len(shape)), self.upload(self.scalarBits(x, dtype)))
        if not isinstance(a, BroadcastData) or not isinstance(b, BroadcastData):
            # tensor (op) scalar: the tensor side arrives as plain data of `count` elements
            wrap = lambda x: x if isinstance(x, (BroadcastData, int, np.integer)) else BroadcastData(
                BroadcastStrides.contiguousForShape([count]), x)
            a, b = wrap(a), wrap(b)
        if not isinstance(a, BroadcastData) and not isinstance(b, BroadcastData):
            raise TypeError("bitwiseOp needs at least one tensor operand")
        a, b = operand(a, b), operand(b, a)
        out = self.allocate(product(a.strides.shape) * dtype.byteSize)
        ad, bd = self._dev(a.data), self._dev(b.data)
        sa, sb = self._s(a.strides), self._s(b.strides)
        self._check(self._lib.hc_bitwise_op(self._ctx, int(op), int(dtype), c_void_p(ad.ptr), byref(sa),
                                            c_void_p(bd.ptr), byref(sb), c_void_p(out.ptr)))
        return out

    def scatter(self, a, s: ScatterGatherIndices, dtype: DType) -> HIPData:
        out = self.allocate(s.gatherInCount * dtype.byteSize)
        ad, idx = self._dev(a), self._dev(s.indices.data)
        st = self._s(s.indices.strides)
        self._check(self._lib.hc_scatter(self._ctx, int(dtype), c_void_p(ad.ptr), c_void_p(idx.ptr), byref(st),
                                         c_void_p(out.ptr), s.outerCount, s.middleCount, s.outCount,
                                         s.innerCount, int(bool(s.indicesAreUnique))))
        return out

    def logSoftmaxGrad(self, a, outGrad, dims: ReduceDims, dtype: DType) -> HIPData:
        out = self.allocate(dims.inCount * dtype.byteSize)
        ad, gd = self._dev(a), self._dev(outGrad)
        self._check(self._lib.hc_log_softmax_grad(self._ctx, int(dtype), c_void_p(ad.ptr), c_void_p(gd.ptr),
                                                  c_void_p(out.ptr), dims.outerCount, dims.reduceCount,
                                                  dims.innerCount))
        return out

    def _cumulative(self, op: int, a, dims: ReduceDims, exclusive: bool, reverse: bool, dtype: DType) -> HIPData:
        out = self.allocate(dims.inCount * dtype.byteSize)
        ad = self._dev(a)
        self._check(self._lib.hc_cumulative(self._ctx, op, int(dtype), c_void_p(ad.ptr), c_void_p(out.ptr),
                                            dims.outerCount, dims.reduceCount, dims.innerCount, int(bool(exclusive)),
                                            int(bool(reverse))))
        return out

    def cumulativeSum(self, a, dims: ReduceDims, exclusive: bool, reverse: bool, dtype: DType) -> HIPData:
        return self._cumulative(0, a, dims, exclusive, reverse, dtype)

    def cumulativeProd(self, a, dims: ReduceDims, exclusive: bool, reverse: bool, dtype: DType) -> HIPData:
        return self._cumulative(1, a, dims, exclusive, reverse, dtype)

    def argsort(self, a, dims: ReduceDims, descending: bool, stable: bool, dtype: DType) -> HIPData:
        """Always stable, which `stable=False` permits (Backend.swift:535-545)."""
        out = self.allocate(dims.inCount * 8)
        ad = self._dev(a)
        self._check(self._lib.hc_argsort(self._ctx, int(dtype), c_void_p(ad.ptr), c_void_p(out.ptr), dims.outerCount,
                                         dims.reduceCount, dims.innerCount, int(bool(descending))))
        return out

    def clamp(self, a: BroadcastData, min, max, dtype: DType) -> HIPData:
        """min / max: None, BroadcastData, or ("scalar", value, shape) (Backend.TensorOrScalar)."""
        if min is None and max is None:
            raise ValueError("cannot use clamp() without bounds")
        def bound(x):
            if x is None or isinstance(x, BroadcastData):
                return x
            _, value, shape = x
            return BroadcastData(BroadcastStrides(shape, [0] * len(shape)), self.constant(value, 1, dtype))
        lo, hi = bound(min), bound(max)
        out = self.allocate(product(a.strides.shape) * dtype.byteSize)
        ad, sa = self._dev(a.data), self._s(a.strides)
        lod, hid = (self._dev(lo.data) if lo else None), (self._dev(hi.data) if hi else None)
        sl, sh = (self._s(lo.strides) if lo else None), (self._s(hi.strides) if hi else None)
        self._check(self._lib.hc_clamp(
            self._ctx, int(dtype), c_void_p(ad.ptr), byref(sa),
            c_void_p(lod.ptr) if lo else None, byref(sl) if lo else None,
            c_void_p(hid.ptr) if hi else None, byref(sh) if hi else None, c_void_p(out.ptr)))
        return out

    def adamW(self, param, grad, moment1, moment2, beta1, beta2, eps, weightDecay, lr, step, count,
              dtype: DType):
        """One fused kernel, bit-identical to the base-class composition (Backend.adamW)."""
        outs = [self.allocate(count * dtype.byteSize) for _ in range(3)]
        ins = [self._dev(x) for x in (param, grad, moment1, moment2)]
        self._check(self._lib.hc_adamw(
            self._ctx, int(dtype), *[c_void_p(x.ptr) for x in ins], c_float(beta1), c_float(beta2), c_float(eps),
            c_float(weightDecay), c_float(lr), c_float(step), c_size_t(count), *[c_void_p(o.ptr) for o in outs]))
        return tuple(outs)

    def matmul(self, a, transA: bool, b, transB: bool, transOut: bool, rows: int, inner: int, cols: int,
               dtype: DType) -> HIPData:
        return self.batchedMatmul(1, a, transA, b, transB, transOut, rows, inner, cols, dtype)

    def batchedMatmul(self, matrixCount: int, a, transA: bool, b, transB: bool, transOut: bool, rows: int,
                      inner: int, cols: int, dtype: DType) -> HIPData:
        out = self.allocate(matrixCount * rows * cols * dtype.byteSize)
        ad, bd = self._dev(a), self._dev(b)
        self._check(self._lib.hc_matmul(self._ctx, int(dtype), matrixCount, c_void_p(ad.ptr), int(transA),
                                        c_void_p(bd.ptr), int(transB), int(transOut), rows, inner, cols,
                                        c_void_p(out.ptr)))
        return out

    def triangular(self, a, batch: int, rows: int, cols: int, upper: bool, offset: int, dtype: DType):
        out = self.allocate(batch * rows * cols * dtype.byteSize)
        ad = self._dev(a)
        self._check(self._lib.hc_triangular(self._ctx, int(dtype), c_void_p(ad.ptr), c_void_p(out.ptr), batch,
                                            rows, cols, int(upper), offset))
        return out

    def concat(self, inputs: Sequence, outerCount: int, innerCounts: Sequence[int], dtype: DType):
        assert len(inputs) == len(innerCounts)
        devs = [self._dev(x) for x in inputs]
        out = self.allocate(outerCount * sum(innerCounts) * dtype.byteSize)
        n = len(devs)
        ptrs = (c_void_p * max(n, 1))(*[d.ptr for d in devs])
        counts = (c_int64 * max(n, 1))(*innerCounts)
        self._check(self._lib.hc_concat(self._ctx, int(dtype), ptrs, counts, n, outerCount, c_void_p(out.ptr)))
        return out

    # bytes of permutation index vectors kept for reuse
    PERMUTATION_CACHE_BYTES = 256 << 20

    def axisPermutation(self, permutation: List[int], shape: List[int]) -> HIPData:
        """The index vector depends on (permutation, shape) only and every permuted view of that
        shape asks for it again (Index.swift:238-266). It is handed out as a PermutationData, which
        writes the vector only if somebody reads its pointer, and shared: buffers are never
        modified after creation. Entries are never evicted (a recorded graph may read them),
        except that a vector first written while recording stops being shared."""
        key = (tuple(permutation), tuple(shape))
        hit = self._perm_cache.get(key)
        if hit is not None:
            return hit
        out = PermutationData(self, permutation, shape)
        if self._perm_cache_bytes + out.byteCount <= self.PERMUTATION_CACHE_BYTES:
            self._perm_cache[key] = out
            self._perm_cache_bytes += out.byteCount
        return out


def convert_host_array(arr: np.ndarray, dtype: DType) -> np.ndarray:
    """Host array -> bytes of `dtype` with the conversions of arrayToPointer
    (TensorElement.swift:225-260): float sources truncate toward zero into int64, anything
    becomes bool by `!= 0`, floats round to nearest even into float16."""
    arr = np.asarray(arr)
    if dtype == DType.bool:
        return np.ascontiguousarray(arr != 0)
    if dtype == DType.int64:
        if arr.dtype.kind == "f":
            return np.trunc(arr).astype(np.int64)
        return arr.astype(np.int64)
    if dtype == DType.float32:
        return arr.astype(np.float32)
    return arr.astype(np.float32).astype(np.float16)
