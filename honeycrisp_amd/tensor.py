"""Forward-only mirror of the Honeycrisp `Tensor` front-ends that sit on the hot path.

Each method does the shape / stride bookkeeping its Swift counterpart does and then emits
the same backend call(s) with the same arguments, so a `Backend` implementation sees exactly
the traffic the reference front-end would send it. No autodiff, no laziness: calls go to
`Backend.current()` immediately (the reference captures `Backend.current` when the op is
created, Tensor.swift:634-657, and runs it in a Task).

Reference: Tensor.swift:802-1177 (cast, arithmetic, pow), Linalg.swift:46-137,
ReduceRepeat.swift:67-331, ScatterGather.swift:51-110, Index.swift:36-410,
Broadcast.swift:115-245, Elemwise.swift:187-322, Softmax.swift, FusedOps.swift,
Comparison.swift, When.swift, ConcatSplit.swift.
"""
from typing import List, Optional, Sequence

import numpy as np

from .backend import Backend, convert_host_array
from .descriptors import (BitwiseOp, BroadcastData, BroadcastStrides, ComparisonOp, DType, ElemwiseOp,
                          NumericBinaryOp, ReduceDims, ReduceOp, RepeatDims, ScatterGatherIndices,
                          product, stridesForShape)

_SCALARS = (int, float, np.floating, np.integer)


# ---------------------------------------------------------------- index helpers (Index.swift)

class TensorIndexResult:
    def __init__(self, reshape, indices, indicesAreUnique, gatherAxis, gatherReshape):
        self.reshape = list(reshape)
        self.indices = indices
        self.indicesAreUnique = indicesAreUnique
        self.gatherAxis = gatherAxis
        self.gatherReshape = None if gatherReshape is None else list(gatherReshape)


class FullRange:
    """Index.swift:118-135."""

    def __init__(self, count=1):
        self.count = count

    minTensorIndexDims = property(lambda self: self.count)

    def tensorIndex(self, inShape):
        assert len(inShape) >= self.count
        return TensorIndexResult(inShape, None, True, self.count - 1, None)


class NewAxis:
    """Index.swift:137-154."""

    def __init__(self, count=1):
        self.count = count

    minTensorIndexDims = 0

    def tensorIndex(self, inShape):
        return TensorIndexResult([1] * self.count + list(inShape), None, True, self.count - 1, None)


class FlipAxis:
    """Index.swift:203-217."""
    minTensorIndexDims = 1

    def tensorIndex(self, inShape):
        idx = Tensor(data=range(inShape[0]), dtype=DType.int64, reverse=True)
        return TensorIndexResult(inShape, idx, True, 0, None)


class PermuteAxes:
    """Index.swift:219-267."""

    def __init__(self, *perm):
        if len(perm) == 1 and isinstance(perm[0], (list, tuple)):
            perm = tuple(perm[0])
        assert all(0 <= x < len(perm) for x in perm), "invalid permutation indices %s" % (perm,)
        assert len(set(perm)) == len(perm), "permutation has repeated axis %s" % (perm,)
        self.perm = list(perm)

    minTensorIndexDims = property(lambda self: len(self.perm))

    def tensorIndex(self, inShape):
        newPerm = list(self.perm)
        removed = 0
        while newPerm and newPerm[0] == 0:
            newPerm = [x - 1 for x in newPerm[1:]]
            removed += 1
        if removed > 0:
            return _index_list([FullRange(removed), PermuteAxes(newPerm)], inShape)
        n = len(self.perm)
        assert n <= len(inShape), "incompatible permutation %s for shape %s" % (self.perm, inShape)
        reshape = [product(inShape[:n])] + list(inShape[n:])
        outShape = [inShape[p] for p in self.perm]
        backend = Backend.current()
        data = backend.axisPermutation(self.perm, list(inShape[:n]))
        indices = Tensor(dataHandle=data, shape=[reshape[0]], dtype=DType.int64)
        return TensorIndexResult(reshape, indices, True, 0, outShape)


def _as_index(x):
    if isinstance(x, (FullRange, NewAxis, FlipAxis, PermuteAxes)):
        return x
    if x is Ellipsis:
        return FullRange(1)  # the reference's `...` is one full axis (UnboundedRange)
    if isinstance(x, (int, np.integer)):
        return _IntIndex(int(x))
    if isinstance(x, slice):
        return _RangeIndex(x)
    raise TypeError("unsupported tensor index %r" % (x,))


class _IntIndex:
    """Index.swift:42-57."""
    minTensorIndexDims = 1

    def __init__(self, i):
        self.i = i

    def tensorIndex(self, inShape):
        idx = inShape[0] + self.i if self.i < 0 else self.i
        assert 0 <= idx < inShape[0], "index %d out of range for size %d" % (self.i, inShape[0])
        return TensorIndexResult(inShape, Tensor(data=[idx], shape=[1], dtype=DType.int64), True, 0, [])


class _RangeIndex:
    """Range / ClosedRange / partial ranges (Index.swift:59-198), written as Python slices
    with unit step (the upper bound is exclusive)."""
    minTensorIndexDims = 1

    def __init__(self, s: slice):
        assert s.step in (None, 1)
        self.s = s

    def tensorIndex(self, inShape):
        n = inShape[0]
        start = 0 if self.s.start is None else (n + self.s.start if self.s.start < 0 else self.s.start)
        end = n if self.s.stop is None else (n + self.s.stop if self.s.stop < 0 else self.s.stop)
        assert end >= start and 0 <= start <= n and 0 <= end <= n
        if start == 0 and end == n:
            return FullRange().tensorIndex(inShape)
        return TensorIndexResult(inShape, Tensor(data=np.arange(start, end, dtype=np.int64), dtype=DType.int64),
                                 True, 0, None)


def _index_list(items, inShape) -> TensorIndexResult:
    """Array<TensorIndex>.tensorIndex (Index.swift:269-357)."""
    if len(items) == 0:
        return TensorIndexResult(inShape, None, True, -1, None)
    if len(items) == 1:
        return items[0].tensorIndex(inShape)
    outerShape: List[int] = []
    gatherInSize = 1
    gatherShape: List[int] = []
    indices: Optional[Tensor] = None
    unique = True
    innerShape = list(inShape)

    def addFullAxes(axesShape):
        nonlocal indices, gatherInSize, outerShape, gatherShape
        if indices is None:
            outerShape += list(axesShape)
        else:
            innerCount = product(axesShape)
            if innerCount != 0 and indices.shape[0] != 0:
                indices = innerCount * indices.unsqueeze(1)
                indices = (indices + Tensor(data=range(innerCount))).flatten()
            else:
                indices = Tensor.zeros([0], dtype=indices.dtype)
            gatherShape += list(axesShape)
            gatherInSize *= innerCount

    for x in items:
        result = x.tensorIndex(innerShape)
        if not result.indicesAreUnique:
            unique = False
        assert product(result.reshape) == product(innerShape)
        if result.gatherAxis > 0:
            addFullAxes(result.reshape[:result.gatherAxis])
        if result.indices is not None:
            newIndices = result.indices
            if indices is None:
                indices = newIndices
            else:
                if newIndices.shape[0] != 0 and indices.shape[0] != 0:
                    axisSize = result.reshape[result.gatherAxis]
                    indices = axisSize * indices.unsqueeze(1)
                    indices = (indices + newIndices).flatten()
                else:
                    indices = Tensor.zeros([0], dtype=indices.dtype)
            gatherShape += result.gatherReshape if result.gatherReshape is not None else [newIndices.shape[0]]
            gatherInSize *= result.reshape[result.gatherAxis]
        elif result.gatherAxis >= 0:
            axisSize = result.reshape[result.gatherAxis]
            addFullAxes(result.gatherReshape if result.gatherReshape is not None else [axisSize])
        innerShape = list(result.reshape[result.gatherAxis + 1:])
    reshape = outerShape + [gatherInSize] + innerShape
    if indices is not None:
        assert product(gatherShape) == indices.shape[0]
    assert product(reshape) == product(inShape)
    return TensorIndexResult(reshape, indices, unique, len(outerShape), gatherShape)


# ---------------------------------------------------------------- Tensor

class Tensor:
    def __init__(self, data=None, shape=None, dtype=None, reverse=False, dataHandle=None):
        """Tensor(data:shape:dtype:) uploads host values through `Backend.collection`
        (Tensor.swift:433-515); `dataHandle` wraps existing backend data."""
        if dataHandle is not None:
            self.data = dataHandle
            self.shape = list(shape)
            self.dtype = DType(dtype)
            return
        if isinstance(data, np.ndarray):
            arr = data
            if dtype is None:
                dtype = DType.of(arr) if arr.dtype != np.float64 else DType.float32
            if shape is None:
                shape = list(arr.shape)
            arr = arr.reshape(-1)
        else:
            values = list(data)
            is_bool = len(values) > 0 and all(isinstance(v, (bool, np.bool_)) for v in values)
            is_int = all(isinstance(v, (int, np.integer)) and not isinstance(v, bool) for v in values)
            if dtype is None:
                # T.dtype of the element type: Bool collections make bool tensors, Int collections
                # int64 tensors, Float / Double collections float32
                dtype = DType.bool if is_bool else DType.int64 if is_int else DType.float32
            arr = np.asarray(values, dtype=np.bool_ if is_bool else np.int64 if is_int else np.float64)
            if shape is None:
                shape = [len(values)]
        self.dtype = DType(dtype)
        self.shape = list(shape)
        assert product(self.shape) == arr.size, "data count %d does not match shape %s" % (arr.size, self.shape)
        self.data = Backend.current().collection(arr, reverse, self.dtype)

    # -- constructors (Tensor.swift:517-560)

    @staticmethod
    def constant(value, shape, dtype=DType.float32) -> "Tensor":
        data = Backend.current().constant(value, product(shape), DType(dtype))
        return Tensor(dataHandle=data, shape=shape, dtype=dtype)

    @staticmethod
    def zeros(shape, dtype=DType.float32) -> "Tensor":
        return Tensor.constant(0, shape, dtype)

    @staticmethod
    def ones(shape, dtype=DType.float32) -> "Tensor":
        return Tensor.constant(1, shape, dtype)

    # -- host access (Tensor.swift:577-621)

    def numpy(self) -> np.ndarray:
        raw = self.data.onCPU()
        n = product(self.shape)
        return np.frombuffer(raw.tobytes(), dtype=self.dtype.numpy, count=n).reshape(self.shape).copy()

    def floats(self) -> List[float]:
        return [float(x) for x in self.numpy().astype(np.float32).reshape(-1)]

    def int64s(self) -> List[int]:
        return [int(x) for x in self.numpy().astype(np.int64).reshape(-1)]

    def item(self):
        assert product(self.shape) == 1
        return self.floats()[0]

    def wait(self):
        self.data.wait()

    def _new(self, data, shape=None, dtype=None) -> "Tensor":
        return Tensor(dataHandle=data, shape=self.shape if shape is None else shape,
                      dtype=self.dtype if dtype is None else dtype)

    def positiveAxis(self, axis):
        if axis is None:
            return None
        return axis + len(self.shape) if axis < 0 else axis

    # -- shape-only ops (Tensor.swift:724-800)

    def reshape(self, newShape: Sequence[int]) -> "Tensor":
        newShape = list(newShape)
        if -1 in newShape:
            i = newShape.index(-1)
            rest = product(newShape[:i] + newShape[i + 1:])
            newShape[i] = product(self.shape) // rest if rest else 0
        assert product(newShape) == product(self.shape), "cannot reshape %s to %s" % (self.shape, newShape)
        return self._new(self.data, shape=newShape)

    def flatten(self) -> "Tensor":
        return self.reshape([product(self.shape)])

    def squeeze(self, axis: int) -> "Tensor":
        axis = self.positiveAxis(axis)
        assert self.shape[axis] == 1
        return self.reshape(self.shape[:axis] + self.shape[axis + 1:])

    def unsqueeze(self, axis: int) -> "Tensor":
        axis = axis + len(self.shape) + 1 if axis < 0 else axis
        return self.reshape(self.shape[:axis] + [1] + self.shape[axis:])

    def cast(self, newType) -> "Tensor":
        """Tensor.swift:802-819."""
        newType = newType.dtype if isinstance(newType, Tensor) else DType(newType)
        if newType == self.dtype:
            return self
        data = Backend.current().cast(self.data, product(self.shape), self.dtype, newType)
        return self._new(data, dtype=newType)

    # -- broadcasting (Broadcast.swift:115-236)

    def expandStrides(self, newShape) -> BroadcastStrides:
        newShape = list(newShape)
        assert len(newShape) >= len(self.shape), "cannot broadcast %s to shorter shape %s" % (self.shape, newShape)
        extra = len(newShape) - len(self.shape)
        strides = [0] * extra
        for i, (oldSize, oldStride) in enumerate(zip(self.shape, stridesForShape(self.shape))):
            newSize = newShape[i + extra]
            if newSize != oldSize:
                assert oldSize == 1, "axis %d cannot expand from size %d to %d" % (i, oldSize, newSize)
                strides.append(0)
            else:
                strides.append(oldStride)
        return BroadcastStrides(newShape, strides)

    @staticmethod
    def broadcastShape(shapes) -> List[int]:
        shapes = [list(s) for s in shapes]
        if len(shapes) == 1:
            return shapes[0]
        if len(shapes) == 2:
            s0, s1 = shapes
            while len(s0) < len(s1):
                s0 = [1] + s0
            while len(s1) < len(s0):
                s1 = [1] + s1
            out = []
            for x, y in zip(s0, s1):
                if x == y:
                    out.append(x)
                elif x == 0 or y == 0:
                    raise ValueError("shapes %s and %s do not support broadcasting" % tuple(shapes))
                elif x == 1:
                    out.append(y)
                elif y == 1:
                    out.append(x)
                else:
                    raise ValueError("shapes %s and %s do not support broadcasting" % tuple(shapes))
            return out
        return Tensor.broadcastShape([Tensor.broadcastShape(shapes[:2])] + shapes[2:])

    @staticmethod
    def lazyBroadcast(ts: Sequence["Tensor"]):
        newShape = Tensor.broadcastShape([t.shape for t in ts])
        return newShape, [t.expandStrides(newShape) for t in ts]

    def expand(self, shape) -> "Tensor":
        shape = shape.shape if isinstance(shape, Tensor) else list(shape)
        if self.shape == shape:
            return self
        strides = self.expandStrides(shape)
        data = Backend.current().broadcast(BroadcastData(strides, self.data), self.dtype)
        return self._new(data, shape=shape)

    @staticmethod
    def broadcast(ts: Sequence["Tensor"]) -> List["Tensor"]:
        shape = Tensor.broadcastShape([t.shape for t in ts])
        return [t.expand(shape) for t in ts]

    def repeating(self, axis: int, count: int) -> "Tensor":
        """ReduceRepeat.swift:249-264."""
        axis = self.positiveAxis(axis)
        assert 0 <= axis <= len(self.shape)
        outerCount = product(self.shape[:axis])
        innerCount = product(self.shape[axis:])
        if axis == len(self.shape):
            newShape = self.shape + [count]
        else:
            newShape = self.shape[:axis] + [self.shape[axis] * count] + self.shape[axis + 1:]
        data = Backend.current().repeated(self.data, RepeatDims(outerCount, count, innerCount), self.dtype)
        return self._new(data, shape=newShape)

    # -- arithmetic (Tensor.swift:821-1138)

    def _binary(self, other, op: NumericBinaryOp, reverse=False) -> "Tensor":
        backend = Backend.current()
        assert self.dtype.isNumeric, "dtype %s cannot be used with arithmetic operators" % self.dtype.name
        if isinstance(other, _SCALARS):
            n = product(self.shape)
            if reverse:
                # scalar + tensor and scalar * tensor are rewritten as tensor (op) scalar
                if op in (NumericBinaryOp.add, NumericBinaryOp.mul):
                    data = backend.binaryOp(self.data, other, op, self.dtype, count=n)
                else:
                    data = backend.binaryOp(other, self.data, op, self.dtype, count=n)
            else:
                data = backend.binaryOp(self.data, other, op, self.dtype, count=n)
            return self._new(data)
        lhs, rhs = (other, self) if reverse else (self, other)
        assert lhs.dtype == rhs.dtype, "dtypes do not match: %s and %s" % (lhs.dtype.name, rhs.dtype.name)
        shape, (ls, rs) = Tensor.lazyBroadcast([lhs, rhs])
        data = backend.binaryOp(BroadcastData(ls, lhs.data), BroadcastData(rs, rhs.data), op, lhs.dtype)
        return Tensor(dataHandle=data, shape=shape, dtype=lhs.dtype)

    def __add__(self, o): return self._binary(o, NumericBinaryOp.add)
    def __radd__(self, o): return self._binary(o, NumericBinaryOp.add, True)
    def __sub__(self, o): return self._binary(o, NumericBinaryOp.sub)
    def __rsub__(self, o): return self._binary(o, NumericBinaryOp.sub, True)
    def __mul__(self, o): return self._binary(o, NumericBinaryOp.mul)
    def __rmul__(self, o): return self._binary(o, NumericBinaryOp.mul, True)
    def __truediv__(self, o): return self._binary(o, NumericBinaryOp.div)
    def __rtruediv__(self, o): return self._binary(o, NumericBinaryOp.div, True)
    def __mod__(self, o): return self._binary(o, NumericBinaryOp.mod)
    def __rmod__(self, o): return self._binary(o, NumericBinaryOp.mod, True)
    def __neg__(self): return self * -1

    def pow(self, exponent) -> "Tensor":
        """Tensor.swift:1141-1159."""
        data = Backend.current().pow(self.data, exponent, 1.0, None, product(self.shape), self.dtype)
        return self._new(data)

    def sqrt(self): return self.pow(0.5)
    def rsqrt(self): return self.pow(-0.5)

    def mul(self, coeff: "Tensor", thenAdd: "Tensor") -> "Tensor":
        """FusedOps.swift:5-39."""
        bias = thenAdd
        assert self.dtype == coeff.dtype == bias.dtype
        shape, (ts, cs, bs) = Tensor.lazyBroadcast([self, coeff, bias])
        data = Backend.current().mulAdd(BroadcastData(ts, self.data), BroadcastData(cs, coeff.data),
                                        BroadcastData(bs, bias.data), self.dtype)
        return Tensor(dataHandle=data, shape=shape, dtype=self.dtype)

    def add(self, bias: "Tensor", thenMul: "Tensor") -> "Tensor":
        """FusedOps.swift:41-79."""
        coeff = thenMul
        assert self.dtype == coeff.dtype == bias.dtype
        shape, (ts, cs, bs) = Tensor.lazyBroadcast([self, coeff, bias])
        data = Backend.current().addMul(BroadcastData(ts, self.data), BroadcastData(bs, bias.data),
                                        BroadcastData(cs, coeff.data), self.dtype)
        return Tensor(dataHandle=data, shape=shape, dtype=self.dtype)

    def normalize(self, axis: int, eps) -> "Tensor":
        """FusedOps.swift:81-103."""
        assert self.dtype.isFloat
        data = Backend.current().normalize(self.data, self.reduceDims(axis), eps, self.dtype)
        return self._new(data)

    # -- elementwise (Elemwise.swift:187-322)

    def elemwise(self, op: ElemwiseOp) -> "Tensor":
        assert self.dtype.isFloat, "dtype %s not supported for elemwise" % self.dtype.name
        data = Backend.current().elemwise(self.data, op, None, product(self.shape), self.dtype)
        return self._new(data)

    def sin(self): return self.elemwise(ElemwiseOp.sin)
    def cos(self): return self.elemwise(ElemwiseOp.cos)
    def tan(self): return self.elemwise(ElemwiseOp.tan)
    def atan(self): return self.elemwise(ElemwiseOp.atan)
    def acos(self): return self.elemwise(ElemwiseOp.acos)
    def asin(self): return self.elemwise(ElemwiseOp.asin)
    def exp(self): return self.elemwise(ElemwiseOp.exp)
    def log(self): return self.elemwise(ElemwiseOp.log)
    def recip(self): return self.elemwise(ElemwiseOp.recip)
    def sigmoid(self): return self.elemwise(ElemwiseOp.sigmoid)
    def relu(self): return self.elemwise(ElemwiseOp.relu)
    def abs(self): return self.elemwise(ElemwiseOp.abs)
    def erf(self): return self.elemwise(ElemwiseOp.erf)
    def floor(self): return self.elemwise(ElemwiseOp.floor)
    def ceil(self): return self.elemwise(ElemwiseOp.ceil)
    def round(self): return self.elemwise(ElemwiseOp.round)

    def gelu(self, mode="approx"):
        return self.elemwise(ElemwiseOp.geluApprox if mode == "approx" else ElemwiseOp.geluExact)

    def tanh(self):
        return 2 * (2 * self).sigmoid() - 1

    def silu(self):
        return self * self.sigmoid()

    # -- comparison / when (Comparison.swift, When.swift)

    def _compare(self, other, op: ComparisonOp, reverse=False) -> "Tensor":
        backend = Backend.current()
        if isinstance(other, Tensor):
            lhs, rhs = (other, self) if reverse else (self, other)
            assert lhs.dtype == rhs.dtype
            shape, (ls, rs) = Tensor.lazyBroadcast([lhs, rhs])
            data = backend.compare(BroadcastData(ls, lhs.data), BroadcastData(rs, rhs.data), op, lhs.dtype)
            return Tensor(dataHandle=data, shape=shape, dtype=DType.bool)
        n = product(self.shape)
        if reverse:
            data = backend.compare(other, self.data, op, self.dtype, count=n)
        else:
            data = backend.compare(self.data, other, op, self.dtype, count=n)
        return self._new(data, dtype=DType.bool)

    def __eq__(self, o): return self._compare(o, ComparisonOp.equal)
    def __ne__(self, o): return self._compare(o, ComparisonOp.notEqual)
    def __lt__(self, o): return self._compare(o, ComparisonOp.less)
    def __le__(self, o): return self._compare(o, ComparisonOp.lessEqual)
    def __gt__(self, o): return self._compare(o, ComparisonOp.greater)
    def __ge__(self, o): return self._compare(o, ComparisonOp.greaterEqual)
    __hash__ = object.__hash__

    # -- bitwise operators (BitwiseOps.swift:58-110): same dtype on both sides, or an integer bit
    # pattern of the element's size

    def _bitwise(self, other, op: BitwiseOp) -> "Tensor":
        backend = Backend.current()
        if isinstance(other, Tensor):
            assert self.dtype == other.dtype, "dtypes for bitwise operator do not match"
            shape, (ls, rs) = Tensor.lazyBroadcast([self, other])
            data = backend.bitwiseOp(BroadcastData(ls, self.data), BroadcastData(rs, other.data), op, self.dtype)
            return Tensor(dataHandle=data, shape=shape, dtype=self.dtype)
        data = backend.bitwiseOp(self.data, int(other), op, self.dtype, count=product(self.shape))
        return self._new(data)

    def __and__(self, o): return self._bitwise(o, BitwiseOp.and_)
    def __rand__(self, o): return self._bitwise(o, BitwiseOp.and_)
    def __or__(self, o): return self._bitwise(o, BitwiseOp.or_)
    def __ror__(self, o): return self._bitwise(o, BitwiseOp.or_)
    def __xor__(self, o): return self._bitwise(o, BitwiseOp.xor)
    def __rxor__(self, o): return self._bitwise(o, BitwiseOp.xor)

    def when(self, isTrue, isFalse, dtype=None) -> "Tensor":
        """When.swift:5-109."""
        assert self.dtype == DType.bool, "can only call when() on boolean Tensor"
        backend = Backend.current()
        tensors = [self] + [x for x in (isTrue, isFalse) if isinstance(x, Tensor)]
        shape, strides = Tensor.lazyBroadcast(tensors)
        it = iter(strides[1:])
        outType = None
        branches = []
        for x in (isTrue, isFalse):
            if isinstance(x, Tensor):
                outType = x.dtype
                branches.append(BroadcastData(next(it), x.data))
            else:
                branches.append(("scalar", x, shape))
        if outType is None:
            assert dtype is not None, "when() with two scalars needs dtype"
            outType = DType(dtype)
        data = backend.when(BroadcastData(strides[0], self.data), branches[0], branches[1], outType)
        return Tensor(dataHandle=data, shape=shape, dtype=outType)

    # -- reductions (ReduceRepeat.swift:67-247)

    def reduceDims(self, axis=None) -> ReduceDims:
        if axis is None:
            return ReduceDims(1, product(self.shape), 1)
        axis = self.positiveAxis(axis)
        assert 0 <= axis < len(self.shape), "axis %d out of bounds for shape %s" % (axis, self.shape)
        return ReduceDims(product(self.shape[:axis]), self.shape[axis], product(self.shape[axis + 1:]))

    def reduce(self, op: ReduceOp, axis=None, keepdims=False) -> "Tensor":
        axis = self.positiveAxis(axis)
        if axis is None:
            outShape = [1] * len(self.shape) if keepdims else []
            return self.reshape([product(self.shape)]).reduce(op, axis=0).reshape(outShape)
        assert 0 <= axis < len(self.shape)
        data = Backend.current().reduce(self.data, op, self.reduceDims(axis), self.dtype)
        newShape = self.shape[:axis] + ([1] if keepdims else []) + self.shape[axis + 1:]
        return Tensor(dataHandle=data, shape=newShape, dtype=DType.int64 if op.isIntOut else self.dtype)

    def sum(self, axis=None, keepdims=False): return self.reduce(ReduceOp.sum, axis, keepdims)
    def prod(self, axis=None, keepdims=False): return self.reduce(ReduceOp.prod, axis, keepdims)
    def argmax(self, axis=None, keepdims=False): return self.reduce(ReduceOp.argmax, axis, keepdims)
    def argmin(self, axis=None, keepdims=False): return self.reduce(ReduceOp.argmin, axis, keepdims)

    def gatherFromReduce(self, op: ReduceOp, axis, keepdims) -> "Tensor":
        """ReduceRepeat.swift:201-209: max/min = arg-reduction + gather."""
        axis = self.positiveAxis(axis)
        if axis is None:
            result = self.flatten().gatherFromReduce(op, 0, False)
            return result.reshape([1] * len(self.shape)) if keepdims else result
        indices = self.reduce(op, axis=axis, keepdims=True)
        selection = self.gather(axis, indices)
        return selection if keepdims else selection.squeeze(axis)

    def max(self, axis=None, keepdims=False): return self.gatherFromReduce(ReduceOp.argmax, axis, keepdims)
    def min(self, axis=None, keepdims=False): return self.gatherFromReduce(ReduceOp.argmin, axis, keepdims)

    def _allSome(self, axis, keepdims, isAll: bool) -> "Tensor":
        """ReduceRepeat.swift:103-162: min (all) / max (some) of a bool tensor; an empty axis yields
        the constant true (all) / false (some)."""
        assert self.dtype == DType.bool, "can only apply all() / some() to boolean tensors"
        axis = self.positiveAxis(axis)
        if axis is not None:
            if self.shape[axis] == 0:
                outShape = self.shape[:axis] + ([1] if keepdims else []) + self.shape[axis + 1:]
                return Tensor.constant(isAll, outShape, DType.bool)
        elif product(self.shape) == 0:
            return Tensor.constant(isAll, [1] * len(self.shape) if keepdims else [], DType.bool)
        return self.min(axis, keepdims) if isAll else self.max(axis, keepdims)

    def all(self, axis=None, keepdims=False): return self._allSome(axis, keepdims, True)
    def some(self, axis=None, keepdims=False): return self._allSome(axis, keepdims, False)

    def cumulativeSum(self, axis: int, exclusive=False, reverse=False) -> "Tensor":
        """ReduceRepeat.swift: running sum along `axis`."""
        data = Backend.current().cumulativeSum(self.data, self.reduceDims(axis), exclusive, reverse, self.dtype)
        return self._new(data)

    def cumulativeProd(self, axis: int, exclusive=False, reverse=False) -> "Tensor":
        data = Backend.current().cumulativeProd(self.data, self.reduceDims(axis), exclusive, reverse, self.dtype)
        return self._new(data)

    def argsort(self, axis: int, descending=False, stable=False) -> "Tensor":
        """Indices (int64) that sort the tensor along `axis`."""
        data = Backend.current().argsort(self.data, self.reduceDims(axis), descending, stable, self.dtype)
        return self._new(data, dtype=DType.int64)

    def mean(self, axis=None, keepdims=False):
        axis = self.positiveAxis(axis)
        n = self.shape[axis] if axis is not None else product(self.shape)
        return self.sum(axis, keepdims) / float(n)

    # -- gather / indexing (ScatterGather.swift:51-110, Index.swift:359-410)

    def expandIndices(self, axis: int, indices: "Tensor"):
        if len(indices.shape) == 1:
            bcastShape = [1] * len(self.shape)
            bcastShape[axis] = indices.shape[0]
            indices = indices.reshape(bcastShape)
        expandShape = list(self.shape)
        expandShape[axis] = indices.shape[axis]
        return indices, indices.expandStrides(expandShape)

    def gather(self, axis: int, indices: "Tensor", indicesAreUnique=False) -> "Tensor":
        assert len(self.shape) > 0, "cannot gather() on a zero-dimensional tensor"
        assert indices.dtype == DType.int64, "can only gather with indices of dtype int64"
        axis = self.positiveAxis(axis)
        indices, indicesStrides = self.expandIndices(axis, indices)
        data = Backend.current().gather(
            self.data,
            ScatterGatherIndices(list(self.shape), axis, BroadcastData(indicesStrides, indices.data),
                                 indicesAreUnique), self.dtype)
        return self._new(data, shape=indicesStrides.shape)

    def scatter(self, axis: int, count: int, indices: "Tensor", indicesAreUnique=False) -> "Tensor":
        """ScatterGather.swift:113-154: the adjoint of gather (values with equal index add up)."""
        assert len(self.shape) > 0, "cannot scatter() on a zero-dimensional tensor"
        assert indices.dtype == DType.int64, "can only scatter with indices of dtype int64"
        axis = self.positiveAxis(axis)
        indices, indicesStrides = self.expandIndices(axis, indices)
        assert indices.shape[axis] == self.shape[axis], \
            "shape %s is not compatible with indices shape %s for scatter along axis %d" % (
                self.shape, indices.shape, axis)
        newShape = list(self.shape)
        newShape[axis] = count
        data = Backend.current().scatter(
            self.data,
            ScatterGatherIndices(newShape, axis, BroadcastData(indicesStrides, indices.data), indicesAreUnique),
            self.dtype)
        return self._new(data, shape=newShape)

    def clamp(self, min=None, max=None) -> "Tensor":
        """Clamp.swift: element-wise min(max, max(min, x)); bounds are tensors or scalars."""
        assert min is not None or max is not None, "cannot use clamp() without bounds"
        tensors = [self] + [x for x in (min, max) if isinstance(x, Tensor)]
        shape, strides = Tensor.lazyBroadcast(tensors)
        it = iter(strides[1:])
        bounds = []
        for x in (min, max):
            if x is None:
                bounds.append(None)
            elif isinstance(x, Tensor):
                assert x.dtype == self.dtype, "clamp bounds must have the tensor's dtype"
                bounds.append(BroadcastData(next(it), x.data))
            else:
                bounds.append(("scalar", x, shape))
        data = Backend.current().clamp(BroadcastData(strides[0], self.data), bounds[0], bounds[1], self.dtype)
        return Tensor(dataHandle=data, shape=shape, dtype=self.dtype)

    def __getitem__(self, index) -> "Tensor":
        if not isinstance(index, tuple):
            index = (index,)
        result = _index_list([_as_index(x) for x in index], self.shape)
        out = self.reshape(result.reshape)
        if result.indices is not None:
            out = out.gather(result.gatherAxis, result.indices, result.indicesAreUnique)
        if result.gatherReshape is not None:
            out = out.reshape(result.reshape[:result.gatherAxis] + result.gatherReshape +
                              result.reshape[result.gatherAxis + 1:])
        return out

    def t(self) -> "Tensor":
        return self[FullRange(len(self.shape) - 2), PermuteAxes(1, 0)]

    def swap(self, axis: int, with_: int) -> "Tensor":
        axis, with_ = self.positiveAxis(axis), self.positiveAxis(with_)
        if axis == with_:
            return self
        perm = list(range(max(axis, with_) + 1))
        perm[axis], perm[with_] = with_, axis
        return self[PermuteAxes(perm)]

    def move(self, axis: int, to: int) -> "Tensor":
        axis, to = self.positiveAxis(axis), self.positiveAxis(to)
        if axis == to:
            return self
        perm = list(range(max(axis, to) + 1))
        perm.remove(axis)
        perm.insert(to, axis)
        return self[PermuteAxes(perm)]

    # -- softmax (Softmax.swift)

    def logSoftmax(self, axis=-1) -> "Tensor":
        posAxis = self.positiveAxis(axis)
        assert 0 <= posAxis < len(self.shape)
        dims = ReduceDims(product(self.shape[:posAxis]), self.shape[posAxis], product(self.shape[posAxis + 1:]))
        return self._new(Backend.current().logSoftmax(self.data, dims, self.dtype))

    def softmax(self, axis=-1) -> "Tensor":
        # Softmax.swift:64-66 ignores `axis` and always normalises the last axis.
        return self.logSoftmax().exp()

    # -- linear algebra (Linalg.swift:46-172)

    @staticmethod
    def matmul(a: "Tensor", transA: bool, b: "Tensor", transB: bool, transOut: bool) -> "Tensor":
        assert len(a.shape) == 2 and len(b.shape) == 2, "invalid shapes for matmul: %s, %s" % (a.shape, b.shape)
        assert a.dtype == b.dtype
        aShape = [a.shape[1], a.shape[0]] if transA else a.shape
        bShape = [b.shape[1], b.shape[0]] if transB else b.shape
        assert aShape[1] == bShape[0], "shape mismatch for matmul (with transposes): %s, %s" % (aShape, bShape)
        outShape = [bShape[1], aShape[0]] if transOut else [aShape[0], bShape[1]]
        data = Backend.current().matmul(a.data, transA, b.data, transB, transOut, aShape[0], aShape[1],
                                        bShape[1], a.dtype)
        return Tensor(dataHandle=data, shape=outShape, dtype=a.dtype)

    @staticmethod
    def batchedMatmul(a: "Tensor", transA: bool, b: "Tensor", transB: bool, transOut: bool) -> "Tensor":
        assert len(a.shape) > 2 and len(b.shape) > 2 and a.shape[:-2] == b.shape[:-2]
        assert a.dtype == b.dtype
        batchShape = a.shape[:-2]
        aShape = [a.shape[-1], a.shape[-2]] if transA else a.shape[-2:]
        bShape = [b.shape[-1], b.shape[-2]] if transB else b.shape[-2:]
        assert aShape[1] == bShape[0]
        outShape = batchShape + ([bShape[1], aShape[0]] if transOut else [aShape[0], bShape[1]])
        data = Backend.current().batchedMatmul(product(batchShape), a.data, transA, b.data, transB, transOut,
                                               aShape[0], aShape[1], bShape[1], a.dtype)
        return Tensor(dataHandle=data, shape=outShape, dtype=a.dtype)

    def __matmul__(self, rhs: "Tensor") -> "Tensor":
        """The reference's `&*` operator (Linalg.swift:131-137)."""
        if len(self.shape) <= 2:
            return Tensor.matmul(self, False, rhs, False, False)
        return Tensor.batchedMatmul(self, False, rhs, False, False)

    def _triangular(self, upper: bool, offset: int) -> "Tensor":
        assert len(self.shape) >= 2
        data = Backend.current().triangular(self.data, product(self.shape[:-2]), self.shape[-2], self.shape[-1],
                                            upper, offset, self.dtype)
        return self._new(data)

    def tril(self, offset=0): return self._triangular(False, offset)
    def triu(self, offset=0): return self._triangular(True, offset)

    # -- split / chunk (ConcatSplit.swift:87-115), one-hot rows (OneHot.swift)

    def split(self, axis: int, counts: Sequence[int]) -> List["Tensor"]:
        axis = self.positiveAxis(axis)
        assert 0 <= axis < len(self.shape), "axis %d out of bounds for shape %s" % (axis, self.shape)
        assert self.shape[axis] == sum(counts), "split counts %s do not sum to axis %d of shape %s" % (counts, axis, self.shape)
        results, start = [], 0
        for count in counts:
            results.append(self[(FullRange(axis), slice(start, start + count))] if axis else self[start:start + count])
            start += count
        return results

    def chunk(self, axis: int, count: int) -> List["Tensor"]:
        axis = self.positiveAxis(axis)
        assert self.shape[axis] >= count and self.shape[axis] % count == 0, \
            "shape %s incompatible with chunk of count %d on axis %d" % (self.shape, count, axis)
        return self.split(axis, [self.shape[axis] // count] * count)

    @staticmethod
    def oneHot(indices, count: int, dtype=DType.float32) -> "Tensor":
        """Tensor(oneHot:count:): a host-built vector (one index) or matrix of rows (a list)."""
        single = isinstance(indices, (int, np.integer))
        rows = [indices] if single else list(indices)
        data = np.zeros((len(rows), count), dtype=np.float32)
        for i, idx in enumerate(rows):
            assert 0 <= idx < count, "oneHot index %d out of range [0, %d)" % (idx, count)
            data[i, idx] = 1
        return Tensor(data=data.reshape(-1), shape=[count] if single else [len(rows), count], dtype=dtype)

    # -- concat (ConcatSplit.swift:4-75)

    @staticmethod
    def concat(tensors: Sequence["Tensor"], axis=0) -> "Tensor":
        assert len(tensors) > 0, "cannot concatenate zero tensors"
        axis = tensors[0].positiveAxis(axis)
        for t in tensors:
            assert t.dtype == tensors[0].dtype
            assert t.shape[:axis] == tensors[0].shape[:axis] and t.shape[axis + 1:] == tensors[0].shape[axis + 1:]
        innerCounts = [product(t.shape[axis:]) for t in tensors]
        outerCount = product(tensors[0].shape[:axis])
        data = Backend.current().concat([t.data for t in tensors], outerCount, innerCounts, tensors[0].dtype)
        newShape = list(tensors[0].shape)
        newShape[axis] = sum(t.shape[axis] for t in tensors)
        return Tensor(dataHandle=data, shape=newShape, dtype=tensors[0].dtype)
