"""The HIP backend behind the raw-tensor contract: `HipRawTensor` + `HipTensorOperations`.

Host-side mirror of what the reference's backends provide
(backend/kten-jvm/.../store/JVMRawTensor.kt, backend/kten-opencl/.../store/OCLRawTensor.kt,
backend/kten-opencl/.../operations/OCLTensorOperations.kt): a raw tensor is a shape plus
a handle to a device-resident fp32 store owned by libkten_hip.so; every operation
validates shapes on the host (raising where the reference throws), allocates the result
store from the library's pool and enqueues one kernel through the C ABI. Nothing here
computes on the CPU; without the shared library the import of `abi.load()` fails.
"""
import contextlib
import ctypes
from contextlib import contextmanager
from typing import Callable, List, Optional, Sequence

import numpy as np

from . import abi
from .host_mirror import shape_functions as sf
from .abi import Op, check
from .host_mirror.raw_tensor import AbstractRawTensor, AggregatingOperation, _is_number, concat as raw_concat

_BINARY = {"plus": Op.PLUS, "minus": Op.MINUS, "times": Op.TIMES, "div": Op.DIV, "pow": Op.POW,
           "lt": Op.LT, "lte": Op.LTE, "gt": Op.GT, "gte": Op.GTE, "eq": Op.EQ, "neq": Op.NEQ}
_UNARY = {"neg": Op.NEG, "reciprocal": Op.RECIPROCAL, "log": Op.LOG, "exp": Op.EXP, "tanh": Op.TANH,
          "sigmoid": Op.SIGMOID, "sinh": Op.SINH, "cosh": Op.COSH, "abs": Op.ABS, "sign": Op.SIGN,
          "sqrt": Op.SQRT, "sin": Op.SIN, "cos": Op.COS, "tan": Op.TAN, "asin": Op.ASIN, "acos": Op.ACOS,
          "atan": Op.ATAN, "floor": Op.FLOOR, "ceil": Op.CEIL, "round": Op.ROUND, "trunc": Op.TRUNC,
          "rsqrt": Op.RSQRT}
_AGG = {AggregatingOperation.SUM: Op.SUM, AggregatingOperation.MEAN: Op.MEAN, AggregatingOperation.MAX: Op.MAX,
        AggregatingOperation.MIN: Op.MIN, AggregatingOperation.ARG_MAX: Op.ARG_MAX,
        AggregatingOperation.ARG_MIN: Op.ARG_MIN}


class HipRawTensor(AbstractRawTensor):
    """Shape + store handle. Reference counting follows OCLRawTensor.kt:21-48: the count
    starts at 1, `release` at 0 hands the store back to the device pool; shallow copies
    and views share the store and hold their own reference on it (OCLRawTensor.kt:252-263)."""

    def __init__(self, shape: Sequence[int], handle: int, ops: "HipTensorOperations"):
        super().__init__(shape)
        self.storeReference = handle
        self.ops = ops
        self._refCount = 1
        self.mustSurviveGC = False
        ops._instanceCollector(self)

    # --- lifetime ----------------------------------------------------------------------
    def incrementRef(self):
        if self._refCount <= 0:
            raise RuntimeError(f"Store reference is already released. (Tensor shape: {self.shape})")
        self._refCount += 1

    def referenced(self) -> bool:
        return self._refCount > 0

    def release(self) -> bool:
        if self._refCount <= 0:
            return False
        if not self.mustSurviveGC:
            self._refCount -= 1
        if self._refCount == 0:
            check(self.ops.lib.kth_release(self.storeReference))
            return True
        return False

    def __del__(self):
        # Safety net the JVM does not have: a wrapper dropped by Python while it still
        # owns its store gives the store back.
        try:
            if self._refCount > 0 and self.ops.alive:
                self._refCount = 0
                self.ops.lib.kth_release(self.storeReference)
        except Exception:
            pass

    # --- helpers -----------------------------------------------------------------------
    @property
    def size(self) -> int:
        return sf.to_store_size(self.shape)

    def _new(self, shape) -> "HipRawTensor":
        return self.ops.createRaw(shape)

    def _require_live(self):
        if self._refCount <= 0:
            raise RuntimeError(f"Raw tensor with shape {self.shape} was released")

    # --- contract ----------------------------------------------------------------------
    def broadcastTo(self, shape):
        """JVMRawTensor.kt:51-73: equal shape returns `this`; otherwise validate by
        ShapeFunctions.kt:187-201 and materialise."""
        shape = list(shape)
        if self.shape == shape:
            return self
        self._require_live()
        sf.infer_explicit_broadcast_shape(self.shape, shape)
        res = self._new(shape)
        check(self.ops.lib.kth_broadcast_to(self.storeReference, abi.shape_array(self.shape), len(self.shape),
                                            res.storeReference, abi.shape_array(shape), len(shape)))
        return res

    def _binary(self, op, other):
        """JVMRawTensor.kt:81-87: common shape, both operands broadcast (fused into the
        kernel instead of materialised), one elementwise pass."""
        self._require_live(); other._require_live()
        common = self.calculateCommonShapeWith(other)
        if self.shape != common:
            sf.infer_explicit_broadcast_shape(self.shape, common)
        if other.shape != common:
            sf.infer_explicit_broadcast_shape(other.shape, common)
        res = self._new(common)
        check(self.ops.lib.kth_binary(_BINARY[op],
                                      self.storeReference, abi.shape_array(self.shape), len(self.shape),
                                      other.storeReference, abi.shape_array(other.shape), len(other.shape),
                                      res.storeReference, abi.shape_array(common), len(common)))
        return res

    def _binary_assign(self, op, other):
        """JVMRawTensor.kt:89-97: shapes must be equal."""
        self._require_live(); other._require_live()
        if self.shape != other.shape:
            raise ValueError(
                f"Shapes does not match for inplace operation on tensors with shapes: {self.shape} and {other.shape}.")
        check(self.ops.lib.kth_binary_inplace(_BINARY[op], self.storeReference, other.storeReference, self.size))

    def _scalar(self, op, constant, reverse=False):
        """JVMRawTensor.kt:99-103 with a constant operand."""
        self._require_live()
        res = self._new(self.shape)
        check(self.ops.lib.kth_scalar(_BINARY[op], self.storeReference, constant, 1 if reverse else 0,
                                      res.storeReference, self.size))
        return res

    def _scalar_assign(self, op, constant):
        """JVMRawTensor.kt:105-108."""
        self._require_live()
        check(self.ops.lib.kth_scalar(_BINARY[op], self.storeReference, constant, 0, self.storeReference, self.size))

    def _compare(self, op, other):
        """JVMRawTensor.kt:355-393. Tensor operands are compared store-to-store without
        broadcasting, as on the JVM; unequal sizes are rejected here."""
        if _is_number(other):
            return self._scalar(op, float(other))
        self._require_live(); other._require_live()
        if self.size != other.size:
            raise ValueError(f"Comparison needs equally sized tensors, got shapes {self.shape} and {other.shape}")
        res = self._new(self.shape)
        sh = abi.shape_array([self.size])
        check(self.ops.lib.kth_binary(_BINARY[op], self.storeReference, sh, 1, other.storeReference, sh, 1,
                                      res.storeReference, sh, 1))
        return res

    def _unary(self, op):
        self._require_live()
        res = self._new(self.shape)
        check(self.ops.lib.kth_unary(_UNARY[op], self.storeReference, res.storeReference, self.size))
        return res

    def clamp(self, min, max):
        self._require_live()
        res = self._new(self.shape)
        check(self.ops.lib.kth_clamp(self.storeReference, res.storeReference, self.size, float(min), float(max)))
        return res

    def aggregateOverAxis(self, axis, resShape, aggregatingOperation):
        """JVMRawTensor.kt:211-225; the device sees the tensor as [outer, axis, inner]."""
        self._require_live()
        outer, length, inner = sf.outer_axis_inner(self.shape, axis)
        res = self._new(resShape)
        check(self.ops.lib.kth_reduce_axis(_AGG[aggregatingOperation], self.storeReference, res.storeReference,
                                           outer, length, inner))
        return res

    def _sum_all(self):
        """JVMRawTensor.kt:146-148 -> shape [1]."""
        self._require_live()
        res = self._new([1])
        check(self.ops.lib.kth_reduce_all(Op.SUM, self.storeReference, self.size, res.storeReference))
        return res

    def _mean_all(self):
        """JVMRawTensor.kt:150-152 -> shape [1]."""
        self._require_live()
        res = self._new([1])
        check(self.ops.lib.kth_reduce_all(Op.MEAN, self.storeReference, self.size, res.storeReference))
        return res

    def gather(self, axis, index):
        """JVMRawTensor.kt:334-353: the result has index's shape."""
        self._require_live(); index._require_live()
        a = sf.normalize_axis(self.shape, axis)
        if index.dimensions != self.dimensions:
            raise ValueError(f"Gather expects index with {self.dimensions} dimensions, got shape {index.shape}")
        res = self._new(index.shape)
        check(self.ops.lib.kth_gather(self.storeReference, abi.shape_array(self.shape), index.storeReference,
                                      abi.shape_array(index.shape), self.dimensions, a, res.storeReference))
        return res

    def _scatter(self, axis, index, src, add):
        """JVMRawTensor.kt:227-255 (tensor source) and 317-332 (constant)."""
        self._require_live(); index._require_live()
        if _is_number(src):
            a = sf.normalize_axis(self.shape, axis)
            if index.dimensions != self.dimensions:
                raise ValueError(f"Scatter expects index with {self.dimensions} dimensions, got shape {index.shape}")
            check(self.ops.lib.kth_scatter_fill(self.storeReference, abi.shape_array(self.shape), index.storeReference,
                                                abi.shape_array(index.shape), self.dimensions, a, float(src)))
            return
        src._require_live()
        a = sf.normalized_axis_scatter(self.shape, axis, index.shape, src.shape)
        check(self.ops.lib.kth_scatter(1 if add else 0, self.storeReference, abi.shape_array(self.shape),
                                       index.storeReference, abi.shape_array(index.shape), src.storeReference,
                                       abi.shape_array(src.shape), self.dimensions, a))

    def _index_select(self, axis, index, resShape):
        """JVMRawTensor.kt:484-501."""
        self._require_live(); index._require_live()
        res = self._new(resShape)
        check(self.ops.lib.kth_index_select(self.storeReference, abi.shape_array(self.shape), self.dimensions, axis,
                                            index.storeReference, index.shape[0], res.storeReference))
        return res

    def _index_add(self, axis, index, src, alpha):
        """JVMRawTensor.kt:503-516."""
        self._require_live(); index._require_live(); src._require_live()
        check(self.ops.lib.kth_index_add(self.storeReference, abi.shape_array(self.shape), self.dimensions, axis,
                                         index.storeReference, index.shape[0], src.storeReference, alpha))

    # --- layout movers -------------------------------------------------------------------
    def _get_store_range(self, offset, length, resShape):
        """JVMRawTensor.kt:270-274: one contiguous store range."""
        self._require_live()
        res = self._new(resShape)
        check(self.ops.lib.kth_copy(res.storeReference, 0, self.storeReference, offset, length))
        return res

    def _set_store_range(self, offset, length, value):
        """JVMRawTensor.kt:282-289 (tensor) and 306-309 (constant)."""
        self._require_live()
        if _is_number(value):
            check(self.ops.lib.kth_fill(self.storeReference, offset, length, float(value)))
            return
        value._require_live()
        check(self.ops.lib.kth_copy(self.storeReference, offset, value.storeReference, 0, length))

    def _get_ranges(self, first, last, resShape):
        """JVMRawTensor.kt:276-280."""
        self._require_live()
        res = self._new(resShape)
        check(self.ops.lib.kth_get_range(self.storeReference, abi.shape_array(self.shape), self.dimensions,
                                         abi.shape_array(first), abi.shape_array(last), res.storeReference))
        return res

    def _set_ranges(self, first, last, value):
        """JVMRawTensor.kt:291-304 (tensor) and 311-315 (constant)."""
        self._require_live()
        if _is_number(value):
            check(self.ops.lib.kth_fill_range(self.storeReference, abi.shape_array(self.shape), self.dimensions,
                                              abi.shape_array(first), abi.shape_array(last), float(value)))
            return
        value._require_live()
        check(self.ops.lib.kth_set_range(self.storeReference, abi.shape_array(self.shape), self.dimensions,
                                         abi.shape_array(first), abi.shape_array(last), value.storeReference, value.size))

    def _transpose(self, axis1, axis2, resShape):
        """JVMRawTensor.kt:437-451; the axis swap of Tensor.kt:1028-1058."""
        self._require_live()
        res = self._new(resShape)
        check(self.ops.lib.kth_transpose(self.storeReference, abi.shape_array(self.shape), self.dimensions, axis1, axis2,
                                         res.storeReference))
        return res

    def _permute(self, axes, resShape):
        """JVMRawTensor.kt:453-466."""
        self._require_live()
        res = self._new(resShape)
        check(self.ops.lib.kth_permute(self.storeReference, abi.shape_array(self.shape), self.dimensions,
                                       abi.shape_array(axes), res.storeReference))
        return res

    def maskedFill(self, mask, value):
        """JVMRawTensor.kt:537-540: the mask broadcasts to this tensor's shape."""
        self._require_live(); mask._require_live()
        if mask.shape != self.shape:
            sf.infer_explicit_broadcast_shape(mask.shape, self.shape)
        res = self._new(self.shape)
        check(self.ops.lib.kth_masked_fill(self.storeReference, abi.shape_array(self.shape), self.dimensions,
                                           mask.storeReference, abi.shape_array(mask.shape), mask.dimensions,
                                           float(value), res.storeReference))
        return res

    def copy(self, shallow: bool = False):
        """JVMRawTensor.kt:257-262; a shallow copy shares the store (OCLRawTensor.kt:252-258)."""
        self._require_live()
        if shallow:
            check(self.ops.lib.kth_retain(self.storeReference))
            return HipRawTensor(self.shape, self.storeReference, self.ops)
        res = self._new(self.shape)
        check(self.ops.lib.kth_copy(res.storeReference, 0, self.storeReference, 0, self.size))
        return res

    def view(self, shape):
        """JVMRawTensor.kt:264-268: same store, reshaped."""
        self._require_live()
        new_shape = sf.reshape(self.shape, shape)
        check(self.ops.lib.kth_retain(self.storeReference))
        return HipRawTensor(new_shape, self.storeReference, self.ops)

    def getSingleValue(self, indexes) -> float:
        """JVMRawTensor.kt:47-49. Blocks until the stream has produced the value."""
        self._require_live()
        out = ctypes.c_float()
        check(self.ops.lib.kth_read_scalar(self.storeReference, sf.store_index(self.shape, list(indexes)),
                                           ctypes.byref(out)))
        return out.value

    def containsNan(self) -> bool:
        self._require_live()
        flag = ctypes.c_int()
        check(self.ops.lib.kth_contains_nan(self.storeReference, self.size, ctypes.byref(flag)))
        return bool(flag.value)

    def inplaceFill(self, value):
        self._require_live()
        check(self.ops.lib.kth_fill(self.storeReference, 0, self.size, float(value)))

    def inplaceResize(self, *shape):
        """inplaceResize (AbstractRawTensor.kt:242): a new store of the new size that keeps the
        leading values and holds zeros beyond them (FloatArray.copyOf, JVMRawTensor.kt:524-531);
        this wrapper's reference on the old store is given back (OCLRawTensor.kt:383-390)."""
        self._require_live()
        new_shape = list(shape[0]) if len(shape) == 1 and not isinstance(shape[0], int) else list(shape)
        n_new, n_old = sf.to_store_size(new_shape), self.size
        handle = ctypes.c_uint64()
        lib = self.ops.lib
        check(lib.kth_alloc(n_new, ctypes.byref(handle)))
        kept = min(n_new, n_old)
        check(lib.kth_copy(handle, 0, self.storeReference, 0, kept))
        if n_new > kept:
            check(lib.kth_fill(handle, kept, n_new - kept, 0.0))
        check(lib.kth_release(self.storeReference))
        self.storeReference = handle.value
        self.shape = new_shape

    def toArray(self) -> np.ndarray:
        """Device -> host copy shaped like the tensor (the backend's toSerializableData)."""
        self._require_live()
        host = np.empty(self.size, dtype=np.float32)
        check(self.ops.lib.kth_download(host.ctypes.data_as(ctypes.c_void_p), self.storeReference, 0, self.size))
        return host.reshape(self.shape)

    def toList(self):
        return self.toArray().reshape(-1).tolist()


class HipBatchNorm:
    """BatchNormOperation (kten-api/.../tensor/operations/nn/BatchNormOperation.kt:5-41) on the
    device: calculateOutput / calculateGrads return the reference's data classes as tuples."""

    def __init__(self, axis, momentum, epsilon, training, ops):
        self.axis, self.momentum, self.epsilon, self.training, self.ops = axis, float(momentum), float(epsilon), bool(training), ops

    @staticmethod
    def _h(t):
        if t is None:
            return 0
        t._require_live()
        return t.storeReference

    def calculateOutput(self, input, runningMean, runningVar, gamma, beta):
        input._require_live()
        channels = input.shape[sf.normalize_axis(input.shape, self.axis)]
        output = self.ops.createRaw(input.shape)
        currentMean = self.ops.createRaw([channels])
        currentStd = self.ops.createRaw([channels])
        check(self.ops.lib.kth_batch_norm_forward(
            input.storeReference, abi.shape_array(input.shape), input.dimensions, self.axis, 1 if self.training else 0,
            self.momentum, self.epsilon, self._h(runningMean), self._h(runningVar), self._h(gamma), self._h(beta),
            output.storeReference, currentMean.storeReference, currentStd.storeReference))
        return output, currentMean, currentStd

    def calculateGrads(self, input, runningMean, runningVar, currentMean, currentStd, gamma, gradOut,
                       inRequiresGrad, gammaRequiresGrad, betaRequiresGrad):
        if not (inRequiresGrad or gammaRequiresGrad or betaRequiresGrad):
            return None, None, None
        input._require_live(); gradOut._require_live()
        channels = input.shape[self.axis]
        gradIn = self.ops.createRaw(input.shape) if inRequiresGrad else None
        gradGamma = self.ops.createRaw([channels]) if gammaRequiresGrad else None
        gradBeta = self.ops.createRaw([channels]) if betaRequiresGrad else None
        check(self.ops.lib.kth_batch_norm_backward(
            input.storeReference, abi.shape_array(input.shape), input.dimensions, self.axis, 1 if self.training else 0,
            self.epsilon, self._h(runningMean), self._h(runningVar), self._h(currentMean), self._h(currentStd), self._h(gamma),
            gradOut.storeReference, self._h(gradIn), self._h(gradGamma), self._h(gradBeta)))
        return gradIn, gradGamma, gradBeta


class HipTensorOperations:
    """TensorOperations for the HIP platform (kten-api/.../operations/TensorOperations.kt:9-135),
    restricted to the members the broadcast / reduction path uses. Lifetime management
    follows OCLTensorOperations.kt:72-130: `garbageCollector()` opens a scope that records
    every raw tensor constructed while it is open and releases them at close; tensors
    that still hold references survive into the next scope."""

    def __init__(self, device: int = 0):
        self.lib = abi.load()
        check(self.lib.kth_init(device))
        self.alive = True
        name = ctypes.create_string_buffer(256)
        mem, cus, wave = ctypes.c_uint64(), ctypes.c_int(), ctypes.c_int()
        check(self.lib.kth_device_info(name, 256, ctypes.byref(mem), ctypes.byref(cus), ctypes.byref(wave)))
        self.deviceName = name.value.decode()
        self.availableMemory = mem.value
        self.computeUnits = cus.value
        self.waveSize = wave.value
        self.platformKey = f"HIP - {device} - {self.deviceName}"
        self._collector: Optional[List[HipRawTensor]] = None
        self._gcSurvivors: List[HipRawTensor] = []

    # --- instance collection / GC scope --------------------------------------------------
    def _instanceCollector(self, raw: HipRawTensor):
        if self._collector is not None:
            self._collector.append(raw)

    @contextmanager
    def garbageCollector(self):
        if self._collector is not None:       # overlapping scopes: the outer one owns everything
            yield
            return
        instances = list(self._gcSurvivors)
        self._collector = instances
        try:
            yield
        finally:
            self._collector = None
            for raw in instances:
                raw.release()
            self._gcSurvivors = [r for r in instances if r.referenced()]

    def release(self, *rawTensors):
        for r in rawTensors:
            r.release()

    def incrementRef(self, rawTensor):
        rawTensor.incrementRef()

    def markSurviveGC(self, rawTensor):
        rawTensor.mustSurviveGC = True

    def markReleasableInGC(self, rawTensor):
        rawTensor.mustSurviveGC = False

    # --- factories -----------------------------------------------------------------------
    def createRaw(self, shape: Sequence[int], init=None) -> HipRawTensor:
        """createRaw(shape, init) / createRaw(shape) (TensorOperations.kt:11-16). `init` is a
        function of the flat index, or a host array of the right size (uploaded as is)."""
        shape = list(shape)
        n = sf.to_store_size(shape)
        handle = ctypes.c_uint64()
        check(self.lib.kth_alloc(n, ctypes.byref(handle)))
        raw = HipRawTensor(shape, handle.value, self)
        if init is not None:
            if callable(init):
                host = np.fromiter((init(i) for i in range(n)), dtype=np.float32, count=n)
            else:
                host = np.ascontiguousarray(np.asarray(init, dtype=np.float32).reshape(-1))
                if host.size != n:
                    raise ValueError(f"init holds {host.size} values, shape {shape} needs {n}")
            check(self.lib.kth_upload(raw.storeReference, 0, host.ctypes.data_as(ctypes.c_void_p), n))
        return raw

    def createRawFill(self, shape, constant: float) -> HipRawTensor:
        raw = self.createRaw(shape)
        raw.inplaceFill(constant)
        return raw

    def zerosLike(self, rawTensor: HipRawTensor) -> HipRawTensor:
        return self.createRawFill(rawTensor.shape, 0.0)

    def zeroOut(self, rawTensor: HipRawTensor):
        rawTensor.inplaceFill(0.0)

    def pow(self, constant: float, rawTensor: HipRawTensor) -> HipRawTensor:
        """TensorOperations.pow(constant, raw): constant ^ x elementwise
        (AbstractJVMTensorOperations.kt:94-96)."""
        return rawTensor._scalar("pow", float(constant), reverse=True)

    def concat(self, axis: int, inputs) -> HipRawTensor:
        """TensorOperations.kt:41. The reference's backends set one range of a new tensor per input
        (AbstractJVMTensorOperations.kt:106-120, OCLTensorOperations.kt:138-152); here one launch writes every
        element of the result once. Shape errors as ShapeFunctions.kt:85-104 raises them."""
        inputs = list(inputs)
        shapes = [t.shape for t in inputs]
        res_shape = sf.concat_shapes(shapes, axis)
        a = sf.normalize_axis(shapes[0], axis)
        if any(t.size == 0 for t in inputs):
            # an empty input is an empty range to the reference's range set, which rejects it: the same construction
            # here, for the same error (the entry point itself takes inputs of length 0)
            return raw_concat(self, axis, inputs)
        res = self.createRaw(res_shape)
        handles = (ctypes.c_uint64 * len(inputs))(*[t.storeReference for t in inputs])
        lens = (ctypes.c_int32 * len(inputs))(*[t.shape[a] for t in inputs])
        check(self.lib.kth_concat(handles, lens, len(inputs), abi.shape_array(res_shape), len(res_shape), a, res.storeReference))
        return res

    def batchNorm(self, axis: int, momentum: float, epsilon: float, training: bool) -> "HipBatchNorm":
        """TensorOperations.kt:129."""
        return HipBatchNorm(axis, momentum, epsilon, training, self)

    # --- Tensor-level factories (BasicTensorOperations.kt:10-12) ----------------------------
    def create(self, shape, requiresGrad: bool = False, init=None):
        from .host_mirror.autograd import NoGradVariable, Variable
        raw = self.createRaw(shape, init) if init is not None else self.createRawFill(shape, 0.0)
        return Variable(self, raw) if requiresGrad else NoGradVariable(self, raw)

    def createFillConst(self, shape, requiresGrad: bool = False, constant: float = 0.0):
        from .host_mirror.autograd import NoGradVariable, Variable
        raw = self.createRawFill(shape, constant)
        return Variable(self, raw) if requiresGrad else NoGradVariable(self, raw)

    # --- serialisation hooks, config, metrics ------------------------------------------------
    def toSerializableData(self, rawTensor: HipRawTensor):
        return list(rawTensor.shape), rawTensor.toArray().reshape(-1)

    def fromCommonSerializable(self, shape, data) -> HipRawTensor:
        return self.createRaw(shape, data)

    def setEpsilon(self, eps: float):
        """PlatformProvider.epsilon (PlatformProvider.kt:12)."""
        check(self.lib.kth_set_epsilon(float(eps)))

    def setMathMode(self, mode: str):
        """How the transcendental maps are evaluated: "exact" (the float kotlin.math returns, bit for bit, by f64
        routines) or "within_2_ulp" (fp32 routines at the time of a copy; the default). No counterpart in the
        reference, whose two backends each have one way."""
        from .abi import KTH_MATH_EXACT, KTH_MATH_WITHIN_2_ULP
        codes = {"exact": KTH_MATH_EXACT, "within_2_ulp": KTH_MATH_WITHIN_2_ULP}
        if mode not in codes:
            raise ValueError(f"math mode {mode!r} is neither 'exact' nor 'within_2_ulp'")
        check(self.lib.kth_set_math_mode(codes[mode]))

    def getMathMode(self) -> str:
        m = ctypes.c_int()
        check(self.lib.kth_get_math_mode(ctypes.byref(m)))
        return "exact" if m.value == 0 else "within_2_ulp"

    @contextlib.contextmanager
    def mathMode(self, mode: str):
        """The math mode for the calls made inside the block; the previous one afterwards."""
        before = self.getMathMode()
        self.setMathMode(mode)
        try:
            yield self
        finally:
            self.setMathMode(before)

    def setMemoryUsageScaleHint(self, fraction: float):
        """PlatformProvider.memoryUsageScaleHint (PlatformProvider.kt:23-29)."""
        check(self.lib.kth_set_memory_scale_hint(float(fraction)))

    def getMetrics(self):
        """PlatformMetricsProvider.getMetrics (PlatformMetricsProvider.kt:3-6)."""
        v = [ctypes.c_uint64() for _ in range(4)]
        check(self.lib.kth_metrics(*[ctypes.byref(x) for x in v]))
        return {"liveBytes": float(v[0].value), "poolBytes": float(v[1].value),
                "launches": float(v[2].value), "bytesMoved": float(v[3].value)}

    def sync(self):
        check(self.lib.kth_sync())

    def timerBegin(self):
        check(self.lib.kth_timer_begin())

    def timerEnd(self) -> float:
        ms = ctypes.c_float()
        check(self.lib.kth_timer_end(ctypes.byref(ms)))
        return ms.value

    def timerLap(self):
        check(self.lib.kth_timer_lap())

    def timerLaps(self):
        """(milliseconds between consecutive laps, milliseconds from the first lap to the last); forgets the laps."""
        cap = 1 << 16
        buf = (ctypes.c_float * cap)()
        n, total = ctypes.c_int(), ctypes.c_float()
        check(self.lib.kth_timer_laps(buf, cap, ctypes.byref(n), ctypes.byref(total)))
        return [buf[i] for i in range(min(n.value, cap))], total.value

    def measureCopy(self, n_floats: int, reps: int = 10):
        """(GB/s of hipMemcpyAsync device to device, GB/s of the library's copy kernel) for n_floats values,
        read + written bytes counted."""
        a, b = ctypes.c_float(), ctypes.c_float()
        check(self.lib.kth_measure_copy(n_floats, reps, ctypes.byref(a), ctypes.byref(b)))
        return 8.0 * n_floats / a.value / 1e6, 8.0 * n_floats / b.value / 1e6

    def profileBegin(self):
        check(self.lib.kth_profile_begin())

    def profileEnd(self):
        """Stops recording and returns {kernel name: (launches, algorithmic bytes, total ms)}."""
        check(self.lib.kth_profile_end())
        n = ctypes.c_int()
        check(self.lib.kth_profile_count(ctypes.byref(n)))
        out = {}
        for i in range(n.value):
            name = ctypes.create_string_buffer(128)
            launches, nbytes, ms = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_double()
            check(self.lib.kth_profile_entry(i, name, 128, ctypes.byref(launches), ctypes.byref(nbytes), ctypes.byref(ms)))
            out[name.value.decode()] = (launches.value, nbytes.value, ms.value)
        return out

    def shutdown(self):
        if self.alive:
            self.alive = False
            self.lib.kth_shutdown()
