"""Python face of the CPU checker (test infrastructure; never imported by the library).

`lib()` loads oracle/libkten_jvm_oracle.so (the C restatement of kten-jvm's arithmetic,
kten_jvm_oracle.c) and `JvmOracleRawTensor` / `JvmOracleOperations` wrap it behind the
same raw-tensor contract the HIP backend implements, so one graph written against the
`Tensor` API can run on both and be compared. Only tests, the smoke check and the
benchmark's CPU-baseline leg may import this module.
"""
import ctypes
import os
import subprocess
from contextlib import contextmanager
from ctypes import POINTER, c_double, c_float, c_int, c_int32, c_int64, c_void_p

import numpy as np

from kten_amd.host_mirror import shape_functions as sf
from kten_amd.host_mirror.raw_tensor import AbstractRawTensor, AggregatingOperation, _is_number, concat as raw_concat

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libkten_jvm_oracle.so")
_lib = None

OPS = {"plus": 0, "minus": 1, "times": 2, "div": 3, "pow": 4, "reciprocal": 5, "log": 6,
       "sum": 7, "mean": 8, "max": 9, "min": 10, "arg_max": 11, "arg_min": 12,
       "lt": 13, "lte": 14, "gt": 15, "gte": 16, "eq": 17, "neq": 18,
       "exp": 19, "tanh": 20, "sigmoid": 21, "sinh": 22, "cosh": 23, "abs": 24, "sign": 25, "sqrt": 26,
       "sin": 27, "cos": 28, "tan": 29, "asin": 30, "acos": 31, "atan": 32, "floor": 33, "ceil": 34,
       "round": 35, "trunc": 36, "rsqrt": 37, "neg": 40}
_AGG = {AggregatingOperation.SUM: 7, AggregatingOperation.MEAN: 8, AggregatingOperation.MAX: 9,
        AggregatingOperation.MIN: 10, AggregatingOperation.ARG_MAX: 11, AggregatingOperation.ARG_MIN: 12}


def build():
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        build()
    L = ctypes.CDLL(_SO)
    fp, ip = c_void_p, POINTER(c_int32)
    L.kjo_set_threads.argtypes = [c_int]
    L.kjo_get_threads.restype = c_int
    L.kjo_common_shape.argtypes = [ip, c_int, ip, c_int, ip]
    L.kjo_common_shape.restype = c_int
    L.kjo_broadcast_to.argtypes = [fp, ip, c_int, fp, ip, c_int]
    L.kjo_broadcast_to.restype = c_int
    L.kjo_binary_same.argtypes = [c_int, fp, fp, fp, c_int64, c_float]
    L.kjo_binary.argtypes = [c_int, fp, ip, c_int, fp, ip, c_int, fp, ip, c_float]
    L.kjo_binary.restype = c_int
    L.kjo_binary_inplace.argtypes = [c_int, fp, fp, c_int64, c_float]
    L.kjo_scalar.argtypes = [c_int, fp, c_float, c_int, fp, c_int64, c_float]
    L.kjo_scalar_inplace.argtypes = [c_int, fp, c_float, c_int64]
    L.kjo_unary.argtypes = [c_int, fp, fp, c_int64]
    L.kjo_clamp.argtypes = [fp, fp, c_int64, c_float, c_float]
    L.kjo_fill.argtypes = [fp, c_int64, c_float]
    L.kjo_contains_nan.argtypes = [fp, c_int64]
    L.kjo_contains_nan.restype = c_int
    L.kjo_sum_all.argtypes = [fp, c_int64]
    L.kjo_sum_all.restype = c_float
    L.kjo_mean_all.argtypes = [fp, c_int64]
    L.kjo_mean_all.restype = c_float
    L.kjo_aggregate_over_axis.argtypes = [c_int, fp, fp, c_int64, c_int64, c_int64]
    L.kjo_sum_all_f64.argtypes = [fp, c_int64]
    L.kjo_sum_all_f64.restype = c_double
    L.kjo_axis_sum_f64.argtypes = [fp, fp, fp, c_int64, c_int64, c_int64]
    L.kjo_gather.argtypes = [fp, ip, fp, ip, c_int, c_int, fp]
    L.kjo_gather.restype = c_int
    L.kjo_scatter.argtypes = [c_int, fp, ip, fp, ip, fp, ip, c_int, c_int]
    L.kjo_scatter.restype = c_int
    L.kjo_scatter_fill.argtypes = [fp, ip, fp, ip, c_int, c_int, c_float]
    L.kjo_scatter_fill.restype = c_int
    L.kjo_index_select.argtypes = [fp, ip, c_int, c_int, fp, c_int64, fp]
    L.kjo_index_select.restype = c_int
    L.kjo_index_add.argtypes = [fp, ip, c_int, c_int, fp, c_int64, fp, c_float]
    L.kjo_index_add.restype = c_int
    L.kjo_range_size.argtypes = [ip, c_int, ip, ip]
    L.kjo_range_size.restype = c_int64
    L.kjo_get_range.argtypes = [fp, ip, c_int, ip, ip, fp]
    L.kjo_set_range.argtypes = [fp, ip, c_int, ip, ip, fp, c_int64]
    L.kjo_set_range.restype = c_int
    L.kjo_fill_range.argtypes = [fp, ip, c_int, ip, ip, c_float]
    L.kjo_transpose_jvm.argtypes = [fp, ip, c_int, c_int, c_int, fp, fp]
    L.kjo_permute.argtypes = [fp, ip, c_int, ip, fp]
    L.kjo_masked_fill.argtypes = [fp, fp, c_float, fp, c_int64]
    L.kjo_batch_norm_apply.argtypes = [fp, ip, c_int, c_int, fp, fp, fp, fp, fp]
    L.kjo_batch_norm_output.argtypes = [fp, ip, c_int, c_int, c_int, c_float, c_float, fp, fp, fp, fp, fp, fp, fp]
    L.kjo_batch_norm_grad_in.argtypes = [fp, ip, c_int, c_int, c_int, fp, fp, fp, fp, fp, fp, fp]
    L.kjo_batch_norm_grads.argtypes = [fp, ip, c_int, c_int, c_int, c_float, fp, fp, fp, fp, fp, fp, fp, fp, fp]
    L.kjo_unary_f64.argtypes = [c_int, c_float]
    L.kjo_unary_f64.restype = c_double
    _lib = L
    return L


def _p(a: np.ndarray):
    return a.ctypes.data_as(c_void_p)


def _sh(shape):
    return (c_int32 * max(len(shape), 1))(*shape)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


# ---------------------------------------------------------------- array-level helpers

def set_threads(n: int):
    lib().kjo_set_threads(int(n))


def unary(op: str, a) -> np.ndarray:
    a = _f32(a); out = np.empty_like(a)
    lib().kjo_unary(OPS[op], _p(a), _p(out), a.size)
    return out


def scalar(op: str, a, c: float, reverse=False, eps=1e-7) -> np.ndarray:
    a = _f32(a); out = np.empty_like(a)
    lib().kjo_scalar(OPS[op], _p(a), c, 1 if reverse else 0, _p(out), a.size, eps)
    return out


def clamp(a, lo: float, hi: float) -> np.ndarray:
    a = _f32(a); out = np.empty_like(a)
    lib().kjo_clamp(_p(a), _p(out), a.size, lo, hi)
    return out


def binary(op: str, a, b, eps=1e-7) -> np.ndarray:
    """Broadcasting binary op; raises ValueError where the reference throws."""
    a, b = _f32(a), _f32(b)
    oshape = (c_int32 * 10)()
    odims = lib().kjo_common_shape(_sh(a.shape), a.ndim, _sh(b.shape), b.ndim, oshape)
    shape = [oshape[i] for i in range(odims)]
    out = np.empty(shape, dtype=np.float32)
    rc = lib().kjo_binary(OPS[op], _p(a), _sh(a.shape), a.ndim, _p(b), _sh(b.shape), b.ndim, _p(out), oshape, eps)
    if rc < 0:
        raise ValueError(f"Shapes {list(a.shape)} and {list(b.shape)} do not broadcast")
    return out


def broadcast_to(a, shape) -> np.ndarray:
    a = _f32(a); out = np.empty(list(shape), dtype=np.float32)
    if lib().kjo_broadcast_to(_p(a), _sh(a.shape), a.ndim, _p(out), _sh(shape), len(shape)) != 0:
        raise ValueError(f"Tensor with shape: {list(a.shape)} cannot be broadcasted to shape: {list(shape)}")
    return out


def aggregate(op: str, a, axis: int) -> np.ndarray:
    """aggregateOverAxis with keep-dims result shape."""
    a = _f32(a)
    outer, length, inner = sf.outer_axis_inner(list(a.shape), axis)
    res_shape = list(a.shape); res_shape[axis] = 1
    out = np.empty(res_shape, dtype=np.float32)
    lib().kjo_aggregate_over_axis(OPS[op], _p(a), _p(out), outer, length, inner)
    return out


def sum_all(a) -> np.float32:
    a = _f32(a)
    return np.float32(lib().kjo_sum_all(_p(a), a.size))


def mean_all(a) -> np.float32:
    a = _f32(a)
    return np.float32(lib().kjo_mean_all(_p(a), a.size))


def sum_all_f64(a) -> float:
    a = _f32(a)
    return lib().kjo_sum_all_f64(_p(a), a.size)


def axis_sum_f64(a, axis: int):
    """(sum, sum of |x|) per lane in extended precision, keep-dims shape."""
    a = _f32(a)
    outer, length, inner = sf.outer_axis_inner(list(a.shape), axis)
    res_shape = list(a.shape); res_shape[axis] = 1
    out = np.empty(res_shape, dtype=np.float64); ab = np.empty(res_shape, dtype=np.float64)
    lib().kjo_axis_sum_f64(_p(a), _p(out), _p(ab), outer, length, inner)
    return out, ab


def get_range(a, first, last) -> np.ndarray:
    """get(Array<IntRange>) with one normalised inclusive range per dim; keeps the dims."""
    a = _f32(a)
    shape = [l - f + 1 for f, l in zip(first, last)]
    out = np.empty(shape, dtype=np.float32)
    lib().kjo_get_range(_p(a), _sh(a.shape), a.ndim, _sh(first), _sh(last), _p(out))
    return out


def set_range(target, first, last, value) -> np.ndarray:
    """set(Array<IntRange>, tensor | Float) on a copy of `target`."""
    t = _f32(target).copy()
    if isinstance(value, (int, float)):
        lib().kjo_fill_range(_p(t), _sh(t.shape), t.ndim, _sh(first), _sh(last), float(value))
        return t
    v = _f32(value)
    if lib().kjo_set_range(_p(t), _sh(t.shape), t.ndim, _sh(first), _sh(last), _p(v), v.size) != 0:
        raise ValueError(f"Cannot set tensor with shape {list(v.shape)} to tensor with shape: {list(t.shape)}")
    return t


def transpose_jvm(a, axis1: int, axis2: int) -> np.ndarray:
    """kten-jvm's slab-copy transpose, literally (equals the axis swap for adjacent axes)."""
    a = _f32(a)
    shape = list(a.shape); shape[axis1], shape[axis2] = shape[axis2], shape[axis1]
    out = np.empty(shape, dtype=np.float32)
    scratch = np.empty(max(a.size // max(a.shape[axis1], 1), 1), dtype=np.float32)
    lib().kjo_transpose_jvm(_p(a), _sh(a.shape), a.ndim, axis1, axis2, _p(out), _p(scratch))
    return out


def permute(a, axes) -> np.ndarray:
    a = _f32(a)
    out = np.empty([a.shape[x] for x in axes], dtype=np.float32)
    lib().kjo_permute(_p(a), _sh(a.shape), a.ndim, _sh(axes), _p(out))
    return out


def masked_fill(a, mask, value: float) -> np.ndarray:
    a, mask = _f32(a), _f32(mask)
    if mask.shape != a.shape:
        mask = broadcast_to(mask, a.shape)
    out = np.empty_like(a)
    lib().kjo_masked_fill(_p(a), _p(mask), value, _p(out), a.size)
    return out


def _po(a):
    return None if a is None else _p(a)


def batch_norm_apply(x, axis, mean, stdev, gamma=None, beta=None) -> np.ndarray:
    """The elementwise half of calculateOutput from given per-channel statistics."""
    x = _f32(x); out = np.empty_like(x)
    mean, stdev = _f32(mean), _f32(stdev)
    gamma = None if gamma is None else _f32(gamma); beta = None if beta is None else _f32(beta)
    lib().kjo_batch_norm_apply(_p(x), _sh(x.shape), x.ndim, axis, _p(mean), _p(stdev), _po(gamma), _po(beta), _p(out))
    return out


def batch_norm_grad_in(x, axis, training, mean, stdev, gamma, grad_out, sums, dots) -> np.ndarray:
    """The elementwise half of calculateGrads from given per-channel scalars."""
    x, grad_out = _f32(x), _f32(grad_out); out = np.empty_like(x)
    mean, stdev, sums, dots = _f32(mean), _f32(stdev), _f32(sums), _f32(dots)
    gamma = None if gamma is None else _f32(gamma)
    lib().kjo_batch_norm_grad_in(_p(x), _sh(x.shape), x.ndim, axis, 1 if training else 0, _p(mean), _p(stdev), _po(gamma),
                                 _p(grad_out), _p(sums), _p(dots), _p(out))
    return out


def unary_f64(op: str, x: float) -> float:
    return lib().kjo_unary_f64(OPS[op], x)


# ---------------------------------------------------------------- the contract on the CPU

class JvmOracleRawTensor(AbstractRawTensor):
    """A FloatArray-backed raw tensor computing through the C restatement."""

    def __init__(self, shape, store: np.ndarray, ops):
        super().__init__(shape)
        self.storeReference = store           # flat float32 array
        self.ops = ops

    def _wrap(self, arr: np.ndarray, shape=None):
        return JvmOracleRawTensor(list(arr.shape) if shape is None else shape, arr.reshape(-1), self.ops)

    def _nd(self) -> np.ndarray:
        return self.storeReference.reshape(self.shape)

    def broadcastTo(self, shape):
        shape = list(shape)
        if self.shape == shape:
            return self
        return self._wrap(broadcast_to(self._nd(), shape))

    def _binary(self, op, other):
        return self._wrap(binary(op, self._nd(), other._nd(), self.ops.epsilon))

    def _binary_assign(self, op, other):
        if self.shape != other.shape:
            raise ValueError(
                f"Shapes does not match for inplace operation on tensors with shapes: {self.shape} and {other.shape}.")
        lib().kjo_binary_inplace(OPS[op], _p(self.storeReference), _p(other.storeReference),
                                 self.storeReference.size, self.ops.epsilon)

    def _scalar(self, op, constant, reverse=False):
        return self._wrap(scalar(op, self.storeReference, constant, reverse, self.ops.epsilon), list(self.shape))

    def _scalar_assign(self, op, constant):
        lib().kjo_scalar_inplace(OPS[op], _p(self.storeReference), constant, self.storeReference.size)

    def _compare(self, op, other):
        if _is_number(other):
            return self._scalar(op, float(other))
        if self.storeReference.size != other.storeReference.size:
            raise ValueError("Comparison needs equally sized tensors")
        out = np.empty_like(self.storeReference)
        lib().kjo_binary_same(OPS[op], _p(self.storeReference), _p(other.storeReference), _p(out), out.size,
                              self.ops.epsilon)
        return self._wrap(out, list(self.shape))

    def _unary(self, op):
        return self._wrap(unary(op, self.storeReference), list(self.shape))

    def clamp(self, min, max):
        return self._wrap(clamp(self.storeReference, min, max), list(self.shape))

    def aggregateOverAxis(self, axis, resShape, aggregatingOperation):
        outer, length, inner = sf.outer_axis_inner(self.shape, axis)
        out = np.empty(sf.to_store_size(resShape), dtype=np.float32)
        lib().kjo_aggregate_over_axis(_AGG[aggregatingOperation], _p(self.storeReference), _p(out), outer, length, inner)
        return self._wrap(out, list(resShape))

    def _sum_all(self):
        return self._wrap(np.array([sum_all(self.storeReference)], dtype=np.float32))

    def _mean_all(self):
        return self._wrap(np.array([mean_all(self.storeReference)], dtype=np.float32))

    def gather(self, axis, index):
        a = sf.normalize_axis(self.shape, axis)
        if index.dimensions != self.dimensions:
            raise ValueError(f"Gather expects index with {self.dimensions} dimensions, got shape {index.shape}")
        out = np.zeros(sf.to_store_size(index.shape), dtype=np.float32)
        if lib().kjo_gather(_p(self.storeReference), _sh(self.shape), _p(index.storeReference), _sh(index.shape),
                            self.dimensions, a, _p(out)) != 0:
            raise ValueError("Gather got invalid index, an index value is out of bounds at the axis")
        return self._wrap(out, list(index.shape))

    def _scatter(self, axis, index, src, add):
        if _is_number(src):
            a = sf.normalize_axis(self.shape, axis)
            rc = lib().kjo_scatter_fill(_p(self.storeReference), _sh(self.shape), _p(index.storeReference),
                                        _sh(index.shape), self.dimensions, a, float(src))
        else:
            a = sf.normalized_axis_scatter(self.shape, axis, index.shape, src.shape)
            rc = lib().kjo_scatter(1 if add else 0, _p(self.storeReference), _sh(self.shape), _p(index.storeReference),
                                   _sh(index.shape), _p(src.storeReference), _sh(src.shape), self.dimensions, a)
        if rc != 0:
            raise ValueError("Scatter got invalid index, an index value is out of bounds at the axis")

    def _index_select(self, axis, index, resShape):
        out = np.zeros(sf.to_store_size(resShape), dtype=np.float32)
        if lib().kjo_index_select(_p(self.storeReference), _sh(self.shape), self.dimensions, axis, _p(index.storeReference),
                                  index.storeReference.size, _p(out)) != 0:
            raise ValueError("Index select got invalid index, an index value is out of bounds at the axis")
        return JvmOracleRawTensor(list(resShape), out, self.ops)

    def _index_add(self, axis, index, src, alpha):
        if lib().kjo_index_add(_p(self.storeReference), _sh(self.shape), self.dimensions, axis, _p(index.storeReference),
                               index.storeReference.size, _p(src.storeReference), alpha) != 0:
            raise ValueError("Index Add got invalid index, an index value is out of bounds at the axis")

    def _get_store_range(self, offset, length, resShape):                      # JVM:270-274 sliceArray
        return JvmOracleRawTensor(list(resShape), self.storeReference[offset:offset + length].copy(), self.ops)

    def _set_store_range(self, offset, length, value):                         # JVM:282-289,306-309
        if _is_number(value):
            self.storeReference[offset:offset + length] = np.float32(value)
        else:
            self.storeReference[offset:offset + length] = value.storeReference[:length]

    def _get_ranges(self, first, last, resShape):
        out = np.empty(sf.to_store_size(resShape), dtype=np.float32)
        lib().kjo_get_range(_p(self.storeReference), _sh(self.shape), self.dimensions, _sh(first), _sh(last), _p(out))
        return JvmOracleRawTensor(list(resShape), out, self.ops)

    def _set_ranges(self, first, last, value):
        if _is_number(value):
            lib().kjo_fill_range(_p(self.storeReference), _sh(self.shape), self.dimensions, _sh(first), _sh(last), float(value))
        elif lib().kjo_set_range(_p(self.storeReference), _sh(self.shape), self.dimensions, _sh(first), _sh(last),
                                 _p(value.storeReference), value.storeReference.size) != 0:
            raise ValueError(f"Cannot set tensor with shape {value.shape} to tensor with shape: {self.shape}")

    def _transpose(self, axis1, axis2, resShape):
        return self._wrap(transpose_jvm(self._nd(), axis1, axis2))

    def _permute(self, axes, resShape):
        return self._wrap(permute(self._nd(), axes))

    def maskedFill(self, mask, value):
        if mask.shape != self.shape:
            sf.infer_explicit_broadcast_shape(mask.shape, self.shape)
        return self._wrap(masked_fill(self._nd(), mask._nd(), float(value)))

    def copy(self, shallow=False):
        if shallow:
            return JvmOracleRawTensor(list(self.shape), self.storeReference, self.ops)
        return JvmOracleRawTensor(list(self.shape), self.storeReference.copy(), self.ops)

    def view(self, shape):
        return JvmOracleRawTensor(sf.reshape(self.shape, shape), self.storeReference, self.ops)

    def getSingleValue(self, indexes):
        return float(self.storeReference[sf.store_index(self.shape, list(indexes))])

    def containsNan(self):
        return bool(lib().kjo_contains_nan(_p(self.storeReference), self.storeReference.size))

    def inplaceFill(self, value):
        lib().kjo_fill(_p(self.storeReference), self.storeReference.size, value)

    def inplaceResize(self, *shape):
        """JVMRawTensor.kt:524-531: storeReference.copyOf(new size) keeps the leading values and
        pads with zeros."""
        new_shape = list(shape[0]) if len(shape) == 1 and not isinstance(shape[0], int) else list(shape)
        n = sf.to_store_size(new_shape)
        store = np.zeros(n, dtype=np.float32)
        kept = min(n, self.storeReference.size)
        store[:kept] = self.storeReference[:kept]
        self.storeReference = store
        self.shape = new_shape

    def toArray(self):
        return self.storeReference.reshape(self.shape).copy()

    def toList(self):
        return self.storeReference.tolist()


class JvmOracleBatchNorm:
    """JVMBatchNorm (backend/kten-jvm/.../operations/nn/JVMBatchNorm.kt) through the C restatement."""

    def __init__(self, axis, momentum, epsilon, training, ops):
        self.axis, self.momentum, self.epsilon, self.training, self.ops = axis, float(momentum), float(epsilon), bool(training), ops

    @staticmethod
    def _s(t):
        return None if t is None else _p(t.storeReference)

    def calculateOutput(self, input, runningMean, runningVar, gamma, beta):
        channels = input.shape[self.axis]
        output = self.ops.createRaw(input.shape)
        currentMean, currentStd = self.ops.createRaw([channels]), self.ops.createRaw([channels])
        lib().kjo_batch_norm_output(_p(input.storeReference), _sh(input.shape), input.dimensions, self.axis,
                                    1 if self.training else 0, self.momentum, self.epsilon, self._s(runningMean),
                                    self._s(runningVar), self._s(gamma), self._s(beta), _p(output.storeReference),
                                    _p(currentMean.storeReference), _p(currentStd.storeReference))
        return output, currentMean, currentStd

    def calculateGrads(self, input, runningMean, runningVar, currentMean, currentStd, gamma, gradOut,
                       inRequiresGrad, gammaRequiresGrad, betaRequiresGrad):
        if not (inRequiresGrad or gammaRequiresGrad or betaRequiresGrad):
            return None, None, None
        channels = input.shape[self.axis]
        gradIn = self.ops.createRaw(input.shape) if inRequiresGrad else None
        gradGamma = self.ops.createRaw([channels]) if gammaRequiresGrad else None
        gradBeta = self.ops.createRaw([channels]) if betaRequiresGrad else None
        lib().kjo_batch_norm_grads(_p(input.storeReference), _sh(input.shape), input.dimensions, self.axis,
                                   1 if self.training else 0, self.epsilon, self._s(runningMean), self._s(runningVar),
                                   self._s(currentMean), self._s(currentStd), self._s(gamma), _p(gradOut.storeReference),
                                   self._s(gradIn), self._s(gradGamma), self._s(gradBeta))
        return gradIn, gradGamma, gradBeta


class JvmOracleOperations:
    """The operations object of the CPU checker. Lifetime calls are no-ops, as on the
    JVM backend (AbstractJVMTensorOperations.kt:73-79,90-92)."""

    platformKey = "JVM-oracle"

    def __init__(self):
        lib()
        self.epsilon = 1e-7

    @contextmanager
    def garbageCollector(self):
        yield

    def release(self, *rawTensors): pass
    def incrementRef(self, rawTensor): pass
    def markSurviveGC(self, rawTensor): pass
    def markReleasableInGC(self, rawTensor): pass

    def createRaw(self, shape, init=None):
        shape = list(shape)
        n = sf.to_store_size(shape)
        if init is None:
            store = np.zeros(n, dtype=np.float32)
        elif callable(init):
            store = np.fromiter((init(i) for i in range(n)), dtype=np.float32, count=n)
        else:
            store = np.array(init, dtype=np.float32).reshape(-1)
            if store.size != n:
                raise ValueError(f"init holds {store.size} values, shape {shape} needs {n}")
        return JvmOracleRawTensor(shape, store, self)

    def createRawFill(self, shape, constant):
        return JvmOracleRawTensor(list(shape), np.full(sf.to_store_size(shape), constant, dtype=np.float32), self)

    def zerosLike(self, rawTensor):
        return self.createRawFill(rawTensor.shape, 0.0)

    def zeroOut(self, rawTensor):
        rawTensor.inplaceFill(0.0)

    def pow(self, constant, rawTensor):
        return rawTensor._scalar("pow", float(constant), reverse=True)

    def concat(self, axis, inputs):
        return raw_concat(self, axis, inputs)

    def batchNorm(self, axis, momentum, epsilon, training):
        return JvmOracleBatchNorm(axis, momentum, epsilon, training, self)

    def create(self, shape, requiresGrad=False, init=None):
        from kten_amd.host_mirror.autograd import NoGradVariable, Variable
        raw = self.createRaw(shape, init)
        return Variable(self, raw) if requiresGrad else NoGradVariable(self, raw)

    def createFillConst(self, shape, requiresGrad=False, constant=0.0):
        from kten_amd.host_mirror.autograd import NoGradVariable, Variable
        raw = self.createRawFill(shape, constant)
        return Variable(self, raw) if requiresGrad else NoGradVariable(self, raw)

    def setEpsilon(self, eps):
        self.epsilon = float(eps)

    def sync(self): pass
