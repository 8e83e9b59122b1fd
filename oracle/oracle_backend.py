"""TEST INFRASTRUCTURE ONLY: the reference CPUBackend arithmetic behind the same `Backend`
interface as the product, so a test can run one piece of front-end code under both and
compare. Data are host byte buffers; the arithmetic is liboracle.so (oracle/cpu_ref.c), a C
restatement of Sources/Honeycrisp/BackendCPU.swift.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_float, c_int, c_int64, c_size_t, c_uint8, c_void_p

import numpy as np

from honeycrisp_amd._lib import hc_strides, make_strides  # same struct layout as ref_strides
from honeycrisp_amd.backend import Backend, convert_host_array
from honeycrisp_amd.descriptors import (BroadcastData, BroadcastStrides, DType, ReduceDims,
                                        ScatterGatherIndices, product)

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")

_S = POINTER(hc_strides)
_P = c_void_p

_PROTOS = {
    "ref_set_threads": (None, [c_int]),
    "ref_f32_to_f16_n": (None, [_P, _P, c_size_t]),
    "ref_f16_to_f32_n": (None, [_P, _P, c_size_t]),
    "ref_strides_index": (c_int64, [_S, c_int64]),
    "ref_broadcast": (None, [c_int, _P, _S, _P]),
    "ref_binary_op": (None, [c_int, c_int, _P, _S, _P, _S, _P]),
    "ref_binary_op_scalar": (None, [c_int, c_int, _P, c_float, c_int64, c_int, _P, c_size_t]),
    "ref_mul_add": (None, [c_int, _P, _S, _P, _S, _P, _S, _P]),
    "ref_add_mul": (None, [c_int, _P, _S, _P, _S, _P, _S, _P]),
    "ref_compare": (None, [c_int, c_int, _P, _S, _P, _S, _P]),
    "ref_compare_scalar": (None, [c_int, c_int, _P, c_float, c_int64, c_int, _P, c_size_t]),
    "ref_cast": (None, [_P, c_int, _P, c_int, c_size_t]),
    "ref_pow": (None, [c_int, _P, c_float, c_float, c_int64, c_int64, _P, _P, c_size_t]),
    "ref_elemwise": (None, [c_int, c_int, _P, _P, _P, c_size_t]),
    "ref_reduce": (None, [c_int, c_int, _P, _P, c_int64, c_int64, c_int64]),
    "ref_log_softmax": (None, [c_int, _P, _P, c_int64, c_int64, c_int64]),
    "ref_gather": (None, [c_int, _P, _P, _S, _P, c_int64, c_int64, c_int64, c_int64]),
    "ref_cumulative": (None, [c_int, c_int, _P, _P, c_int64, c_int64, c_int64, c_int, c_int]),
    "ref_argsort": (None, [c_int, _P, _P, c_int64, c_int64, c_int64, c_int]),
    "ref_bitwise_op": (None, [c_int, c_int, _P, _S, _P, _S, _P]),
    "ref_scatter": (None, [c_int, _P, _P, _S, _P, c_int64, c_int64, c_int64, c_int64]),
    "ref_log_softmax_grad": (None, [c_int, _P, _P, _P, c_int64, c_int64, c_int64]),
    "ref_clamp": (None, [c_int, _P, _S, _P, _S, _P, _S, _P]),
    "ref_when": (None, [c_int, _P, _S, _P, _S, _P, _S, _P]),
    "ref_matmul": (None, [c_int, c_int64, _P, c_int, _P, c_int, c_int, c_int64, c_int64, c_int64, _P]),
    "ref_matmul_rows": (None, [c_int, _P, c_int, _P, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, _P]),
    "ref_triangular": (None, [c_int, _P, _P, c_int64, c_int64, c_int64, c_int, c_int64]),
    "ref_fill": (None, [c_int, c_float, c_int64, _P, c_size_t]),
    "ref_axis_permutation": (None, [POINTER(c_int64), POINTER(c_int64), c_int, _P]),
    "ref_normalize": (None, [c_int, _P, _P, c_int64, c_int64, c_int64, c_float]),
    "ref_concat": (None, [c_int, POINTER(c_void_p), POINTER(c_int64), c_int, c_int64, _P]),
}


def build():
    subprocess.run(["make", "-C", HERE, "liboracle.so"], check=True, stdout=subprocess.PIPE,
                   stderr=subprocess.STDOUT)


def load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        build()
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in _PROTOS.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


class CPUData:
    """Host byte buffer (CPUData, BackendCPU.swift:11-48)."""

    def __init__(self, nbytes: int):
        self.buf = np.zeros(max(int(nbytes), 1), dtype=np.uint8)
        self.byteCount = int(nbytes)

    @property
    def ptr(self):
        return self.buf.ctypes.data_as(c_void_p)

    def onCPU(self) -> np.ndarray:
        return self.buf[:self.byteCount]

    def wait(self):
        pass


class OracleBackend(Backend):
    def __init__(self, threads: int = 0):
        self.lib = load()
        self.lib.ref_set_threads(threads)

    def _host(self, data) -> CPUData:
        if isinstance(data, CPUData):
            return data
        raw = data if isinstance(data, np.ndarray) else data.onCPU()
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        out = CPUData(raw.nbytes)
        out.buf[:raw.nbytes] = raw
        return out

    @staticmethod
    def _s(strides: BroadcastStrides):
        return make_strides(strides.shape, strides.strides)

    @staticmethod
    def _scalar(value, dtype):
        if dtype == DType.int64:
            return c_float(0.0), c_int64(int(value))
        return c_float(float(np.float32(value))), c_int64(0)

    def allocate(self, byteCount):
        return CPUData(byteCount)

    def upload(self, host: np.ndarray) -> CPUData:
        return self._host(np.ascontiguousarray(host))

    def sync(self):
        pass

    def collection(self, collection, reverse, dtype):
        arr = np.asarray(list(collection) if not isinstance(collection, np.ndarray) else collection)
        if reverse:
            arr = arr[::-1]
        return self._host(convert_host_array(arr.reshape(-1), dtype))

    def constant(self, value, count, dtype):
        out = CPUData(count * dtype.byteSize)
        vf, vi = self._scalar(value, dtype)
        if dtype != DType.int64:
            vf = c_float(float(np.float32(value)))
        self.lib.ref_fill(int(dtype), vf, vi, out.ptr, count)
        return out

    def broadcast(self, a, dtype):
        out = CPUData(product(a.strides.shape) * dtype.byteSize)
        self.lib.ref_broadcast(int(dtype), self._host(a.data).ptr, self._s(a.strides), out.ptr)
        return out

    def binaryOp(self, a, b, op, dtype, count=None):
        if isinstance(a, BroadcastData) and isinstance(b, BroadcastData):
            out = CPUData(product(a.strides.shape) * dtype.byteSize)
            self.lib.ref_binary_op(int(op), int(dtype), self._host(a.data).ptr, self._s(a.strides),
                                   self._host(b.data).ptr, self._s(b.strides), out.ptr)
            return out
        scalar_first = isinstance(a, (int, float, np.floating, np.integer))
        tensor, scalar = (b, a) if scalar_first else (a, b)
        out = CPUData(count * dtype.byteSize)
        sf, si = self._scalar(scalar, dtype)
        self.lib.ref_binary_op_scalar(int(op), int(dtype), self._host(tensor).ptr, sf, si, int(scalar_first),
                                      out.ptr, count)
        return out

    def mulAdd(self, input, coeff, bias, dtype):
        out = CPUData(product(input.strides.shape) * dtype.byteSize)
        self.lib.ref_mul_add(int(dtype), self._host(input.data).ptr, self._s(input.strides),
                             self._host(coeff.data).ptr, self._s(coeff.strides),
                             self._host(bias.data).ptr, self._s(bias.strides), out.ptr)
        return out

    def addMul(self, input, bias, coeff, dtype):
        out = CPUData(product(input.strides.shape) * dtype.byteSize)
        self.lib.ref_add_mul(int(dtype), self._host(input.data).ptr, self._s(input.strides),
                             self._host(bias.data).ptr, self._s(bias.strides),
                             self._host(coeff.data).ptr, self._s(coeff.strides), out.ptr)
        return out

    def when(self, mask, a, b, dtype):
        def branch(x):
            if isinstance(x, BroadcastData):
                return x
            _, value, shape = x
            return BroadcastData(BroadcastStrides(shape, [0] * len(shape)), self.constant(value, 1, dtype))
        a, b = branch(a), branch(b)
        out = CPUData(product(mask.strides.shape) * dtype.byteSize)
        self.lib.ref_when(int(dtype), self._host(mask.data).ptr, self._s(mask.strides),
                          self._host(a.data).ptr, self._s(a.strides), self._host(b.data).ptr,
                          self._s(b.strides), out.ptr)
        return out

    def compare(self, a, b, op, dtype, count=None):
        if isinstance(a, BroadcastData) and isinstance(b, BroadcastData):
            out = CPUData(product(a.strides.shape))
            self.lib.ref_compare(int(op), int(dtype), self._host(a.data).ptr, self._s(a.strides),
                                 self._host(b.data).ptr, self._s(b.strides), out.ptr)
            return out
        scalar_first = isinstance(a, (int, float, bool, np.floating, np.integer, np.bool_))
        tensor, scalar = (b, a) if scalar_first else (a, b)
        out = CPUData(count)
        sf, si = self._scalar(scalar, dtype)
        self.lib.ref_compare_scalar(int(op), int(dtype), self._host(tensor).ptr, sf, si, int(scalar_first),
                                    out.ptr, count)
        return out

    def cast(self, a, count, inType, outType):
        out = CPUData(count * outType.byteSize)
        self.lib.ref_cast(self._host(a).ptr, int(inType), out.ptr, int(outType), count)
        return out

    def pow(self, a, b, scale, scales, count, dtype):
        out = CPUData(count * dtype.byteSize)
        bf, bi = self._scalar(b, dtype)
        scf, sci = self._scalar(scale, dtype)
        self.lib.ref_pow(int(dtype), self._host(a).ptr, bf, scf, bi, sci,
                         self._host(scales).ptr if scales is not None else None, out.ptr, count)
        return out

    def elemwise(self, a, op, scales, count, dtype):
        out = CPUData(count * dtype.byteSize)
        self.lib.ref_elemwise(int(op), int(dtype), self._host(a).ptr,
                              self._host(scales).ptr if scales is not None else None, out.ptr, count)
        return out

    def reduce(self, a, op, dims: ReduceDims, dtype):
        outType = DType.int64 if op.isIntOut else dtype
        out = CPUData(dims.outCount * outType.byteSize)
        self.lib.ref_reduce(int(op), int(dtype), self._host(a).ptr, out.ptr, dims.outerCount,
                            dims.reduceCount, dims.innerCount)
        return out

    def logSoftmax(self, a, dims, dtype):
        out = CPUData(dims.inCount * dtype.byteSize)
        self.lib.ref_log_softmax(int(dtype), self._host(a).ptr, out.ptr, dims.outerCount, dims.reduceCount,
                                 dims.innerCount)
        return out

    # normalize: inherited base-class composition (the CPU backend does not override it);
    # ref_normalize in C is the same composition and is cross-checked against it in tests.

    def gather(self, a, s: ScatterGatherIndices, dtype):
        out = CPUData(s.gatherOutCount * dtype.byteSize)
        self.lib.ref_gather(int(dtype), self._host(a).ptr, self._host(s.indices.data).ptr,
                            self._s(s.indices.strides), out.ptr, s.outerCount, s.middleCount, s.outCount,
                            s.innerCount)
        return out

    def cumulativeSum(self, a, dims, exclusive, reverse, dtype):
        return self._cumulative(0, a, dims, exclusive, reverse, dtype)

    def cumulativeProd(self, a, dims, exclusive, reverse, dtype):
        return self._cumulative(1, a, dims, exclusive, reverse, dtype)

    def _cumulative(self, op, a, dims, exclusive, reverse, dtype):
        out = CPUData(dims.inCount * dtype.byteSize)
        self.lib.ref_cumulative(op, int(dtype), self._host(a).ptr, out.ptr, dims.outerCount, dims.reduceCount,
                                dims.innerCount, int(exclusive), int(reverse))
        return out

    def argsort(self, a, dims, descending, stable, dtype):
        out = CPUData(dims.inCount * 8)
        self.lib.ref_argsort(int(dtype), self._host(a).ptr, out.ptr, dims.outerCount, dims.reduceCount,
                             dims.innerCount, int(descending))
        return out

    def bitwiseOp(self, a, b, op, dtype, count=None):
        def operand(x, other):
            if isinstance(x, BroadcastData):
                return x
            shape = other.strides.shape
            return BroadcastData(BroadcastStrides(shape, [0] * len(shape)), self._host(self.scalarBits(x, dtype)))
        if not isinstance(a, BroadcastData) or not isinstance(b, BroadcastData):
            wrap = lambda x: BroadcastData(BroadcastStrides.contiguousForShape([count]), x) \
                if isinstance(x, (CPUData, np.ndarray)) or hasattr(x, "onCPU") else x
            a, b = wrap(a), wrap(b)
        a, b = operand(a, b), operand(b, a)
        out = CPUData(product(a.strides.shape) * dtype.byteSize)
        self.lib.ref_bitwise_op(int(op), int(dtype), self._host(a.data).ptr, self._s(a.strides),
                                self._host(b.data).ptr, self._s(b.strides), out.ptr)
        return out

    def scatter(self, a, s: ScatterGatherIndices, dtype):
        out = CPUData(s.gatherInCount * dtype.byteSize)
        self.lib.ref_scatter(int(dtype), self._host(a).ptr, self._host(s.indices.data).ptr,
                             self._s(s.indices.strides), out.ptr, s.outerCount, s.middleCount, s.outCount,
                             s.innerCount)
        return out

    def logSoftmaxGrad(self, a, outGrad, dims, dtype):
        out = CPUData(dims.inCount * dtype.byteSize)
        self.lib.ref_log_softmax_grad(int(dtype), self._host(a).ptr, self._host(outGrad).ptr, out.ptr,
                                      dims.outerCount, dims.reduceCount, dims.innerCount)
        return out

    def clamp(self, a, min, max, dtype):
        assert min is not None or max is not None, "cannot use clamp() without bounds"
        def bound(x):
            if x is None or isinstance(x, BroadcastData):
                return x
            _, value, shape = x
            return BroadcastData(BroadcastStrides(shape, [0] * len(shape)), self.constant(value, 1, dtype))
        lo, hi = bound(min), bound(max)
        out = CPUData(product(a.strides.shape) * dtype.byteSize)
        self.lib.ref_clamp(int(dtype), self._host(a.data).ptr, self._s(a.strides),
                           self._host(lo.data).ptr if lo else None, self._s(lo.strides) if lo else None,
                           self._host(hi.data).ptr if hi else None, self._s(hi.strides) if hi else None, out.ptr)
        return out

    def matmul(self, a, transA, b, transB, transOut, rows, inner, cols, dtype):
        return self.batchedMatmul(1, a, transA, b, transB, transOut, rows, inner, cols, dtype)

    def batchedMatmul(self, matrixCount, a, transA, b, transB, transOut, rows, inner, cols, dtype):
        out = CPUData(matrixCount * rows * cols * dtype.byteSize)
        self.lib.ref_matmul(int(dtype), matrixCount, self._host(a).ptr, int(transA), self._host(b).ptr,
                            int(transB), int(transOut), rows, inner, cols, out.ptr)
        return out

    def triangular(self, a, batch, rows, cols, upper, offset, dtype):
        out = CPUData(batch * rows * cols * dtype.byteSize)
        self.lib.ref_triangular(int(dtype), self._host(a).ptr, out.ptr, batch, rows, cols, int(upper), offset)
        return out

    def concat(self, inputs, outerCount, innerCounts, dtype):
        hosts = [self._host(x) for x in inputs]
        out = CPUData(outerCount * sum(innerCounts) * dtype.byteSize)
        n = len(hosts)
        ptrs = (c_void_p * max(n, 1))(*[h.buf.ctypes.data for h in hosts])
        counts = (c_int64 * max(n, 1))(*innerCounts)
        self.lib.ref_concat(int(dtype), ptrs, counts, n, outerCount, out.ptr)
        return out

    def axisPermutation(self, permutation, shape):
        n = len(shape)
        out = CPUData(product(shape) * 8)
        perm = (c_int64 * max(n, 1))(*permutation)
        shp = (c_int64 * max(n, 1))(*shape)
        self.lib.ref_axis_permutation(perm, shp, n, out.ptr)
        return out
