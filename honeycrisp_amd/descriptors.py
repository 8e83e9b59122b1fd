"""Descriptor types of the Honeycrisp backend interface, mirrored one for one.

Reference: Tensor.DType (Sources/Honeycrisp/Tensor.swift:24-67), BroadcastStrides /
BroadcastData (Broadcast.swift:9-113), ReduceDims / RepeatDims / ReduceOp
(ReduceRepeat.swift:12-63), ScatterGatherIndices (ScatterGather.swift:4-46),
NumericBinaryOp (BinaryOps.swift:2-23), ElemwiseOp (Elemwise.swift:13-43),
ComparisonOp (Comparison.swift:4-28), BackendError (Backend.swift:6-16).
"""
import enum
from dataclasses import dataclass
from typing import Any, List, Sequence

import numpy as np


class DType(enum.IntEnum):
    int64 = 0
    bool = 1
    float16 = 2
    float32 = 3

    @property
    def byteSize(self) -> int:
        return (8, 1, 2, 4)[int(self)]

    @property
    def isNumeric(self) -> bool:
        return self != DType.bool

    @property
    def isFloat(self) -> bool:
        return self in (DType.float16, DType.float32)

    @property
    def numpy(self):
        return (np.int64, np.bool_, np.float16, np.float32)[int(self)]

    @staticmethod
    def of(arr: np.ndarray) -> "DType":
        for d in DType:
            if np.dtype(d.numpy) == arr.dtype:
                return d
        raise TypeError("no tensor dtype for numpy dtype %s" % arr.dtype)


class NumericBinaryOp(enum.IntEnum):
    add = 0
    mul = 1
    sub = 2
    div = 3
    mod = 4


class ReduceOp(enum.IntEnum):
    sum = 0
    prod = 1
    argmax = 2
    argmin = 3

    @property
    def isIntOut(self) -> bool:
        return self in (ReduceOp.argmax, ReduceOp.argmin)


class BitwiseOp(enum.IntEnum):
    """BitwiseOps.swift:38-41 (order of include/hchip.h)."""
    or_ = 0
    and_ = 1
    xor = 2


class ComparisonOp(enum.IntEnum):
    equal = 0
    notEqual = 1
    less = 2
    lessEqual = 3
    greater = 4
    greaterEqual = 5


class ElemwiseOp(enum.IntEnum):
    sin = 0
    cos = 1
    minusSin = 2
    tan = 3
    tanGrad = 4
    atan = 5
    atanGrad = 6
    acos = 7
    acosGrad = 8
    asin = 9
    asinGrad = 10
    exp = 11
    log = 12
    recip = 13
    sigmoid = 14
    sigmoidGrad = 15
    relu = 16
    reluGrad = 17
    abs = 18
    absGrad = 19
    geluApprox = 20
    geluApproxGrad = 21
    geluExact = 22
    geluExactGrad = 23
    erf = 24
    erfGrad = 25
    floor = 26
    ceil = 27
    round = 28


class BackendError(Exception):
    """Mirrors the cases of BackendError a backend throws (Backend.swift:6-16)."""

    def __init__(self, kind: str, detail: Any = None):
        super().__init__("%s(%s)" % (kind, detail))
        self.kind = kind
        self.detail = detail

    @staticmethod
    def notImplemented(name):
        return BackendError("notImplemented", name)

    @staticmethod
    def allocationFailed(nbytes):
        return BackendError("allocationFailed", nbytes)

    @staticmethod
    def kernelFailed(msg):
        return BackendError("kernelFailed", msg)

    @staticmethod
    def failedToLoadKernels(msg):
        return BackendError("failedToLoadKernels", msg)


def product(xs: Sequence[int]) -> int:
    n = 1
    for x in xs:
        n *= int(x)
    return n


def stridesForShape(shape: Sequence[int]) -> List[int]:
    """Row-major strides (Broadcast.swift:238-244)."""
    return [product(shape[i + 1:]) for i in range(len(shape))]


class BroadcastStrides:
    """Virtual shape plus per-axis data strides, 0 on broadcast axes (Broadcast.swift:9-30)."""

    def __init__(self, shape: Sequence[int], strides: Sequence[int]):
        assert len(shape) == len(strides)
        self.shape = [int(s) for s in shape]
        self.strides = [int(s) for s in strides]
        self.dataCount = product([size for stride, size in zip(self.strides, self.shape) if stride != 0])
        self.isNoOp = all(stride != 0 or size == 1 for stride, size in zip(self.strides, self.shape))

    @staticmethod
    def contiguousForShape(shape: Sequence[int]) -> "BroadcastStrides":
        return BroadcastStrides(shape, stridesForShape(shape))

    def __call__(self, i: int) -> int:
        """Virtual index -> data index (Broadcast.swift:72-90)."""
        if self.isNoOp:
            return i
        cur, result = i, 0
        for stride, size in zip(reversed(self.strides), reversed(self.shape)):
            result += stride * (cur % size)
            cur //= size
        return result

    def __repr__(self):
        return "BroadcastStrides(shape=%s, strides=%s)" % (self.shape, self.strides)


@dataclass
class BroadcastData:
    strides: BroadcastStrides
    data: Any

    @property
    def dataCount(self) -> int:
        return self.strides.dataCount

    @property
    def isSimple(self) -> bool:
        return self.strides.isNoOp

    @staticmethod
    def simple(data, shape) -> "BroadcastData":
        return BroadcastData(BroadcastStrides.contiguousForShape(shape), data)


@dataclass(frozen=True)
class ReduceDims:
    outerCount: int
    reduceCount: int
    innerCount: int

    @property
    def inCount(self):
        return self.outerCount * self.reduceCount * self.innerCount

    @property
    def outCount(self):
        return self.outerCount * self.innerCount

    def inverse(self):
        return RepeatDims(self.outerCount, self.reduceCount, self.innerCount)


@dataclass(frozen=True)
class RepeatDims:
    outerCount: int
    repeatCount: int
    innerCount: int

    @property
    def inCount(self):
        return self.outerCount * self.innerCount

    @property
    def outCount(self):
        return self.outerCount * self.repeatCount * self.innerCount

    def inverse(self):
        return ReduceDims(self.outerCount, self.repeatCount, self.innerCount)


@dataclass
class ScatterGatherIndices:
    """Low-level gather description (ScatterGather.swift:4-46)."""
    valueShape: List[int]
    axis: int
    indices: BroadcastData
    indicesAreUnique: bool = False

    @property
    def outerCount(self):
        return product(self.valueShape[:self.axis])

    @property
    def middleCount(self):
        return self.valueShape[self.axis]

    @property
    def innerCount(self):
        return product(self.valueShape[self.axis + 1:])

    @property
    def outCount(self):
        return self.indices.strides.shape[self.axis]

    @property
    def gatherInCount(self):
        return product(self.valueShape)

    @property
    def gatherOutCount(self):
        return product(self.indices.strides.shape)
