"""The raw-tensor side of the backend contract, for the broadcast / reduction path.

`AbstractRawTensor` mirrors the reference's
kten-api/src/main/kotlin/eu/redbean/kten/api/tensor/store/AbstractRawTensor.kt: the same
member names, argument meaning and error behaviour, with the concrete helpers of the
base class (axis normalisation, keep-dims handling, reshape / squeeze / unsqueeze,
common-shape calculation) restated once here so that every backend shares them, as in
the reference. Kotlin's overloads on (tensor | Float) become one Python method that
dispatches on the argument type; Kotlin operators are also exposed as Python operators.

Members of the contract that lie outside the accelerated path (BLAS level 2 and 3, nn other
than batch normalisation) are not part of this mirror.
"""
from enum import Enum
from typing import List, Sequence

from . import shape_functions as sf


class AggregatingOperation(Enum):
    """kten-api/.../tensor/store/AggregatingOperation.kt:3-5"""
    SUM = "SUM"
    MEAN = "MEAN"
    MAX = "MAX"
    MIN = "MIN"
    ARG_MAX = "ARG_MAX"
    ARG_MIN = "ARG_MIN"


def _is_number(x) -> bool:
    return isinstance(x, (int, float)) and not isinstance(x, bool)


class AbstractRawTensor:
    """AbstractRawTensor.kt:5-23 — a shape plus a backend-owned store."""

    def __init__(self, shape: Sequence[int]):
        self._shape = list(shape)

    # --- shape -------------------------------------------------------------------------
    @property
    def shape(self) -> List[int]:
        return self._shape

    @shape.setter
    def shape(self, value: Sequence[int]):
        self._shape = list(value)

    @property
    def dimensions(self) -> int:
        return len(self._shape)

    # --- abstract: what a backend supplies (AbstractRawTensor.kt:25-75,121-122,164-246) ---
    def broadcastTo(self, shape): raise NotImplementedError
    def _binary(self, op: str, other): raise NotImplementedError             # tensor (op) tensor, broadcasting
    def _binary_assign(self, op: str, other): raise NotImplementedError      # in place, equal shapes
    def _scalar(self, op: str, constant: float, reverse=False): raise NotImplementedError
    def _scalar_assign(self, op: str, constant: float): raise NotImplementedError
    def _compare(self, op: str, other): raise NotImplementedError            # tensor or float
    def _unary(self, op: str): raise NotImplementedError
    def clamp(self, min: float, max: float): raise NotImplementedError
    def aggregateOverAxis(self, axis: int, resShape, aggregatingOperation): raise NotImplementedError
    def _sum_all(self): raise NotImplementedError
    def _mean_all(self): raise NotImplementedError
    def view(self, shape): raise NotImplementedError
    def copy(self, shallow: bool = False): raise NotImplementedError
    def getSingleValue(self, indexes) -> float: raise NotImplementedError
    def containsNan(self) -> bool: raise NotImplementedError
    def inplaceFill(self, value: float): raise NotImplementedError
    def inplaceResize(self, *shape): raise NotImplementedError               # new store: leading values kept, zeros beyond
    def toList(self): raise NotImplementedError                              # flat host copy (serializable data)

    # --- arithmetic (AbstractRawTensor.kt:39-73) ---------------------------------------
    def plus(self, other):
        return self._scalar("plus", float(other)) if _is_number(other) else self._binary("plus", other)

    def plusAssign(self, other):
        if _is_number(other): self._scalar_assign("plus", float(other))
        else: self._binary_assign("plus", other)

    def minus(self, other):
        return self._scalar("minus", float(other)) if _is_number(other) else self._binary("minus", other)

    def unaryMinus(self):
        return self._unary("neg")

    def times(self, other):
        return self._scalar("times", float(other)) if _is_number(other) else self._binary("times", other)

    def timesAssign(self, other):
        if _is_number(other): self._scalar_assign("times", float(other))
        else: self._binary_assign("times", other)

    def div(self, other):
        return self._scalar("div", float(other)) if _is_number(other) else self._binary("div", other)

    def divAssign(self, constant):
        self._scalar_assign("div", float(constant))

    def pow(self, other):
        return self._scalar("pow", float(other)) if _is_number(other) else self._binary("pow", other)

    def reciprocal(self): return self._unary("reciprocal")
    def log(self): return self._unary("log")

    __add__ = plus
    __sub__ = minus
    __mul__ = times
    __truediv__ = div
    __pow__ = pow
    __neg__ = unaryMinus

    def __iadd__(self, other):
        self.plusAssign(other)
        return self

    def __imul__(self, other):
        self.timesAssign(other)
        return self

    def __itruediv__(self, other):
        self.divAssign(other)
        return self

    # --- comparisons (AbstractRawTensor.kt:194-206) ------------------------------------
    def lt(self, other): return self._compare("lt", other)
    def lte(self, other): return self._compare("lte", other)
    def gt(self, other): return self._compare("gt", other)
    def gte(self, other): return self._compare("gte", other)
    def eq(self, other): return self._compare("eq", other)
    def neq(self, other): return self._compare("neq", other)

    # --- pointwise maths (AbstractRawTensor.kt:208-227) --------------------------------
    def exp(self): return self._unary("exp")
    def tanh(self): return self._unary("tanh")
    def sigmoid(self): return self._unary("sigmoid")
    def sinh(self): return self._unary("sinh")
    def cosh(self): return self._unary("cosh")
    def abs(self): return self._unary("abs")
    def sign(self): return self._unary("sign")
    def sqrt(self): return self._unary("sqrt")
    def sin(self): return self._unary("sin")
    def cos(self): return self._unary("cos")
    def tan(self): return self._unary("tan")
    def asin(self): return self._unary("asin")
    def acos(self): return self._unary("acos")
    def atan(self): return self._unary("atan")
    def floor(self): return self._unary("floor")
    def ceil(self): return self._unary("ceil")
    def round(self): return self._unary("round")
    def trunc(self): return self._unary("trunc")
    def rsqrt(self): return self._unary("rsqrt")

    # --- reshaping helpers (AbstractRawTensor.kt:77-88,124-144) ------------------------
    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (list, tuple)):
            shape = shape[0]
        new_shape = sf.reshape(self.shape, shape)
        res = self.copy()
        res.shape = new_shape
        return res

    def inplaceReshape(self, shape):
        self.shape = sf.reshape(self.shape, shape)

    def inplaceSqueeze(self, axis: int):
        new_shape = list(self.shape)
        del new_shape[sf.normalize_axis(self.shape, axis)]
        self.shape = new_shape

    def squeeze(self, axis: int):
        res = self.copy()
        res.inplaceSqueeze(axis)
        return res

    def inplaceUnsqueeze(self, axis: int):
        self.shape = sf.unsqueeze(self.shape, axis)

    def unsqueeze(self, axis: int):
        res = self.copy()
        res.inplaceUnsqueeze(axis)
        return res

    # --- reductions (AbstractRawTensor.kt:92-122) --------------------------------------
    def _aggregatingOpOverAxis(self, axis: int, keepDims: bool, op: AggregatingOperation):
        """AbstractRawTensor.kt:92-108: normalise the axis, reduce to the keep-dims shape,
        then drop the dim unless kept or the result would become 0-D."""
        normalized = sf.normalize_axis(self.shape, axis)
        res_shape = sf.aggregate_over(self.shape, normalized, True)
        res = self.aggregateOverAxis(normalized, res_shape, op)
        if not keepDims and len(res_shape) > 1:
            without = list(res_shape)
            del without[normalized]
            res.shape = without
        return res

    def sum(self, axis=None, keepDimensions: bool = False):
        if axis is None:
            return self._sum_all()
        return self._aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation.SUM)

    def mean(self, axis=None, keepDimensions: bool = False):
        if axis is None:
            return self._mean_all()
        return self._aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation.MEAN)

    def max(self, axis: int, keepDimensions: bool = False):
        return self._aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation.MAX)

    def min(self, axis: int, keepDimensions: bool = False):
        return self._aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation.MIN)

    def argMax(self, axis: int = 0, keepDimensions: bool = False):
        return self._aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation.ARG_MAX)

    def argMin(self, axis: int = 0, keepDimensions: bool = False):
        return self._aggregatingOpOverAxis(axis, keepDimensions, AggregatingOperation.ARG_MIN)

    # --- indexed moves along an axis (AbstractRawTensor.kt:146-164) --------------------
    def gather(self, axis: int, index): raise NotImplementedError
    def _scatter(self, axis: int, index, src, add: bool): raise NotImplementedError   # src: tensor or float

    def inplaceScatter(self, axis: int, index, src):
        self._scatter(axis, index, src, False)

    def inplaceScatterAdd(self, axis: int, index, src):
        self._scatter(axis, index, src, True)

    def scatter(self, axis: int, index, src):
        """AbstractRawTensor.kt:152-162: copy, then scatter into the copy."""
        res = self.copy()
        res.inplaceScatter(axis, index, src)
        return res

    # --- get / set by index (AbstractRawTensor.kt:27-37) --------------------------------
    # An index is a sequence of ints (Kotlin IntArray: leading dims, negative values wrap)
    # or a sequence of shape_functions.IntRange / (first, last) pairs / ALL (Kotlin
    # Array<IntRange>, both ends inclusive). Backends supply moves of one contiguous store
    # range and of a box of ranges.
    def _get_store_range(self, offset: int, length: int, resShape): raise NotImplementedError
    def _set_store_range(self, offset: int, length: int, value): raise NotImplementedError     # value: tensor or float
    def _get_ranges(self, first, last, resShape): raise NotImplementedError
    def _set_ranges(self, first, last, value): raise NotImplementedError                       # value: tensor or float
    def _permute(self, axes, resShape): raise NotImplementedError
    def _transpose(self, axis1: int, axis2: int, resShape): raise NotImplementedError
    def maskedFill(self, mask, value: float): raise NotImplementedError

    def get(self, index):
        index = list(index)
        if sf.is_range_index(index):                                   # JVMRawTensor.kt:276-280
            norm, res_shape = sf.normalized_range_indexed_shape(self.shape, index)
            first, last = sf.full_ranges(self.shape, norm)
            return self._get_ranges(first, last, res_shape)
        norm, res_shape = sf.normalized_indexed_shape(self.shape, index)   # JVMRawTensor.kt:270-274
        offset, length = sf.store_range(self.shape, norm)
        return self._get_store_range(offset, length, res_shape)

    def set(self, index, value):
        index = list(index)
        if sf.is_range_index(index):                                   # JVMRawTensor.kt:291-304,311-315
            norm = sf.normalize_range_index(self.shape, index)
            first, last = sf.full_ranges(self.shape, norm)
            if not _is_number(value):
                size = sf.to_store_size([l - f + 1 for f, l in zip(first, last)])
                if size != sf.to_store_size(value.shape):
                    raise ValueError(f"Cannot set tensor with shape {value.shape} to tensor with shape: {self.shape} "
                                     f"at index: {[tuple(sf.as_range(r)) for r in index]}")
            self._set_ranges(first, last, value)
            return
        norm = sf.normalize_index(self.shape, index)                   # JVMRawTensor.kt:282-289,306-309
        offset, length = sf.store_range(self.shape, norm)
        if not _is_number(value) and sf.to_store_size(value.shape) != length:
            raise ValueError(f"Cannot set tensor with shape: {value.shape} to tensor with shape: {self.shape} "
                             f"at index: {index}")
        self._set_store_range(offset, length, value)

    def __getitem__(self, index):
        return self.get(index if isinstance(index, (tuple, list)) and not isinstance(index, sf.IntRange) else [index])

    def __setitem__(self, index, value):
        self.set(index if isinstance(index, (tuple, list)) and not isinstance(index, sf.IntRange) else [index], value)

    # --- transpose / permute / narrow (AbstractRawTensor.kt:228-232) --------------------
    def transpose(self, axis1: int, axis2: int):
        new_shape, a1, a2 = sf.transpose_normalize_axes(self.shape, axis1, axis2)
        return self._transpose(a1, a2, new_shape)

    def permute(self, axes):
        axes = list(axes)
        return self._permute(axes, sf.permute(self.shape, axes))

    def narrow(self, axis: int, start: int, length: int):
        """JVMRawTensor.kt:468-473: the range start until start + length at the axis, every
        other dim in full, through the range get (which also validates the range)."""
        a = sf.normalize_axis(self.shape, axis)
        ranges = sf.to_index_ranges(self.shape)
        ranges[a] = sf.IntRange(start, start + length - 1)
        return self.get(ranges)

    # --- indexSelect / indexAdd (AbstractRawTensor.kt:236-238) ---------------------------
    def _index_select(self, axis: int, index, resShape): raise NotImplementedError
    def _index_add(self, axis: int, index, src, alpha: float): raise NotImplementedError

    def indexSelect(self, axis: int, index):
        a, res_shape = sf.index_select_norm_axis_shape(self.shape, axis, index.shape)
        return self._index_select(a, index, res_shape)

    def indexAdd(self, axis: int, index, src, alpha: float = 1.0):
        a = sf.index_add_check_shapes_norm_axis(self.shape, axis, index.shape, src.shape)
        self._index_add(a, index, src, float(alpha))

    # --- dot (AbstractRawTensor.kt:234) ---------------------------------------------------
    def dot(self, vector):
        """JVMRawTensor.kt:475-482: elementwise products rounded to float, then their sum. A
        backend may override it; this composition is two operations of the path (times, sum)."""
        sf.dot_shape(self.shape, vector.shape)
        products = self.times(vector)
        res = products._sum_all()
        self.ops.release(products)
        return res

    # --- broadcasting (AbstractRawTensor.kt:170-192) -----------------------------------
    def calculateCommonShapeWith(self, other) -> List[int]:
        """Right-align, keep the longer operand's extra leading dims, per-dim max.
        Validity is only checked later, by broadcastTo's rule."""
        if self.shape == other.shape:
            return list(self.shape)
        a, b = list(self.shape), list(other.shape)
        res: List[int] = []
        diff = len(a) - len(b)
        if diff > 0:
            res.extend(a[:diff]); a = a[diff:]
        elif diff < 0:
            res.extend(b[:-diff]); b = b[-diff:]
        res.extend(max(x, y) for x, y in zip(a, b))
        return res


def concat(ops, axis: int, inputs):
    """TensorOperations.concat (TensorOperations.kt:41) as the JVM backend builds it
    (AbstractJVMTensorOperations.kt:106-120): a new tensor of the concatenated shape, then one
    range set per input at its offset along the axis."""
    inputs = list(inputs)
    shapes = [t.shape for t in inputs]
    res_shape = sf.concat_shapes(shapes, axis)
    a = sf.normalize_axis(shapes[0], axis)
    target = sf.to_index_ranges(res_shape)
    res = ops.createRaw(res_shape)
    last = 0
    for t in inputs:
        target[a] = sf.IntRange(last, last + t.shape[a] - 1)
        res.set(target, t)
        last += t.shape[a]
    return res
