"""The caller of the hot path: `Tensor` and the reverse-mode autograd graph.

In a kten deployment this layer is the reference's own Kotlin code and stays unchanged;
the backend only ever sees the sequence of raw-tensor calls it emits. This module
restates that layer for the operations on the broadcast / reduction path so that the
same sequences can be driven from Python against any backend implementing
`AbstractRawTensor` + the operations object (the HIP backend, or a test's CPU checker).
It computes nothing itself: every number comes from the backend's raw ops.

Reference (paths under kten-api/src/main/kotlin/eu/redbean/kten/api/):
  tensor/Tensor.kt                         public surface, companion factories
  autograd/tensor/AGTensor.kt:85-289       graph routing
  autograd/tensor/NoGradVariable.kt:66-190 eager routing when no operand needs grad
  autograd/tensor/Variable.kt:15-46        leaf with an accumulated gradient
  autograd/functions/Function.kt:47-171    forward / backward life cycle, reference counts
  autograd/functions/BasicFunctions.kt, PointwiseFunctions.kt, AggregatingFunctions.kt,
  TensorFunctions.kt:200-283 (Reshape, Expand), Utils.kt:14-41 (mayUnexpand)
"""
import math
from typing import List, Optional, Sequence

from . import shape_functions as sf

_NO_AXIS = None     # the reference marks "no axis" with Int.MIN_VALUE


def _is_number(x) -> bool:
    return isinstance(x, (int, float)) and not isinstance(x, bool)


def _safe(t):
    """AGTensor.kt:26-30."""
    return t.inplaceSafe() if isinstance(t, AGTensor) else t


def _as_list(args):
    return list(args[0]) if len(args) == 1 and isinstance(args[0], (list, tuple)) else list(args)


def _as_index(index):
    """`t[1, 1]` -> [1, 1]; `t[(1, 1), ALL, (1, -1)]` -> three ranges; `t[2]` -> [2];
    `t[ALL]` -> one range."""
    if isinstance(index, sf.IntRange) or not isinstance(index, (tuple, list)):
        return [index]
    return list(index)


def mayUnexpand(rawTensor, oldShape: Sequence[int], ops):
    """Reduce a gradient back to the shape an operand had before broadcasting
    (functions/Utils.kt:14-41): sum(0) without keepDims once per extra leading dim, then
    sum(d, keepDims) for every remaining dim whose size differs, in ascending order."""
    oldShape = list(oldShape)
    unsqueezed = rawTensor.dimensions - len(oldShape)
    expanded = [i for i, (e, o) in enumerate(zip(rawTensor.shape[unsqueezed:], oldShape)) if e != o]
    res = rawTensor
    for i in range(unsqueezed):
        to_release = res
        res = res.sum(0, keepDimensions=False)
        if i > 0:
            ops.release(to_release)
    for i, d in enumerate(expanded):
        to_release = res
        res = res.sum(d, keepDimensions=True)
        if i > 0:
            ops.release(to_release)
    return res


class Tensor:
    """tensor/Tensor.kt:118 — the user-facing API (the subset on the accelerated path)."""

    def __init__(self, ops):
        self.ops = ops

    # subclasses provide: shape, requiresGrad, getRawValue(), forward(), backward(), grad()
    @property
    def dimensions(self) -> int:
        return len(self.shape)

    @property
    def platform(self) -> str:
        return self.ops.platformKey

    # --- Python operators -> the Kotlin operator functions -------------------------------
    def __add__(self, o): return self.plus(o)
    def __radd__(self, o): return self.rplus(float(o))
    def __sub__(self, o): return self.minus(o)
    def __rsub__(self, o): return self.rminus(float(o))
    def __mul__(self, o): return self.times(o)
    def __rmul__(self, o): return self.rtimes(float(o))
    def __truediv__(self, o): return self.div(o)
    def __rtruediv__(self, o): return self.rdiv(float(o))
    def __pow__(self, o): return self.pow(o)
    def __rpow__(self, o): return self.rpow(float(o))

    def __neg__(self):
        """Tensor.kt:553-555: unaryMinus is `0.0f - this`."""
        return self.rminus(0.0)

    def expand(self, *newShape):
        if len(newShape) == 1 and isinstance(newShape[0], (list, tuple)):
            newShape = newShape[0]
        return self._expand(list(newShape))

    def reshape(self, *newShape):
        if len(newShape) == 1 and isinstance(newShape[0], (list, tuple)):
            newShape = newShape[0]
        return self._reshape(list(newShape))

    def toArray(self):
        """Host copy of the values (forwards a pending graph first)."""
        t = self.inplaceSafe() if isinstance(self, AGTensor) else self
        if t.requiresGrad:
            t.forward()
        return t.getRawValue().toArray()


class AGTensor(Tensor):
    """autograd/tensor/AGTensor.kt — every method builds a graph node."""

    requiresGrad = True
    inplaceSafeThis = None

    def inplaceSafe(self):
        """AGTensor.kt:24-34: after an indexed set the tensor stands for the function that
        performed it, so later uses see the modified value in the graph."""
        return self.inplaceSafeThis if self.inplaceSafeThis is not None else self

    def _forwarded(self):
        """AGTensor.kt:52-59 inplaceSafeForwarded."""
        t = self.inplaceSafe()
        if isinstance(t, Function) and not t.hasValue():
            t.forward()
        return t

    # AGTensor.kt:61-83. An index is all ints (Kotlin `t[1, 1]`) or all ranges: IntRange,
    # (first, last) pairs with both ends inclusive, or ALL (Kotlin `t[1..1, all, 1..-1]`).
    def __getitem__(self, index):
        return Index(self.ops)(_safe(self), _as_index(index))

    def __setitem__(self, index, value):
        index = _as_index(index)
        if _is_number(value):
            self.inplaceSafeThis = IndexSetConstant(self.ops)(_safe(self), index, float(value))
        else:
            self.inplaceSafeThis = IndexSetTensor(self.ops)(_safe(self), index, _safe(value))

    def transpose(self, axis1, axis2): return Transpose(self.ops)(self, axis1, axis2)          # AGTensor.kt:265-267
    def permute(self, *axes): return Permute(self.ops)(self, _as_list(axes))                  # AGTensor.kt:277-279
    def concat(self, axis, tensors): return Concat(self.ops)(axis, [_safe(t) for t in tensors])   # AGTensor.kt:281-283
    def maskedFill(self, mask, value): return MaskedFill(self.ops)(self, mask, float(value))  # AGTensor.kt:525-527
    def copy(self): return Copy(self.ops)(self)
    def squeeze(self, axis): return Squeeze(self.ops)(self, axis)
    def unsqueeze(self, axis): return Unsqueeze(self.ops)(self, axis)

    def item(self) -> float:
        """AGTensor.kt:36-46."""
        t = self._forwarded()
        if t.dimensions != 1 or t.shape[0] != 1:
            raise RuntimeError("Item can only be accessed from singleton tensors (1D tensors with 1 element in them), "
                               f"but tensor shape is {t.shape}")
        return t.getRawValue().getSingleValue([0])

    def getValue(self, index) -> float:
        return self._forwarded().getRawValue().getSingleValue(list(index))

    # AGTensor.kt:85-167
    def plus(self, o): return PlusConstant(self.ops)(self, float(o)) if _is_number(o) else Plus(self.ops)(self, o)
    def rplus(self, c): return PlusConstant(self.ops)(c, self, constant_first=True)
    def minus(self, o): return MinusConstant(self.ops)(self, float(o)) if _is_number(o) else Minus(self.ops)(self, o)
    def rminus(self, c): return MinusConstant(self.ops)(c, self, constant_first=True)
    def times(self, o): return TimesConstant(self.ops)(self, float(o)) if _is_number(o) else Times(self.ops)(self, o)
    def rtimes(self, c): return TimesConstant(self.ops)(c, self, constant_first=True)
    def div(self, o): return DivConstant(self.ops)(self, float(o)) if _is_number(o) else Div(self.ops)(self, o)
    def rdiv(self, c): return DivConstant(self.ops)(c, self, constant_first=True)
    def pow(self, o): return PowConstant(self.ops)(self, float(o)) if _is_number(o) else Pow(self.ops)(self, o)
    def rpow(self, c): return PowConstant(self.ops)(c, self, constant_first=True)

    def sum(self, axis=_NO_AXIS, keepDimensions=False): return Sum(self.ops)(self, axis, keepDimensions)
    def mean(self, axis=_NO_AXIS, keepDimensions=False): return Mean(self.ops)(self, axis, keepDimensions)

    def max(self, axis, keepDimensions=False): return Max(self.ops)(self, axis, keepDimensions)
    def min(self, axis, keepDimensions=False): return Min(self.ops)(self, axis, keepDimensions)
    def gather(self, axis, index): return Gather(self.ops)(self, axis, index)
    def indexSelect(self, axis, index): return IndexSelect(self.ops)(self, index, axis)           # AGTensor.kt:305-307
    def dot(self, vector): return Dot(self.ops)(self, vector)
    def scatter(self, axis, index, source): return Scatter(self.ops)(self, axis, index, source)

    def batchNorm(self, axis, runningMean, runningVar, training, momentum=0.1, epsilon=1e-5, gamma=None, beta=None):
        """functions/nn/TensorExtensions.kt: Tensor.batchNorm."""
        return BatchNormalizationFunction(axis, momentum, epsilon, training, self.ops)(self, runningMean, runningVar, gamma, beta)

    def meanVariance(self, axis, keepDimensions=False, unbiased=True):
        """AGTensor.kt:454-461."""
        tensor = _safe(self)
        mean = tensor.mean(axis, True)
        elements = tensor.shape[sf.normalize_axis(tensor.shape, axis)] - (1 if unbiased else 0)
        zeroCentered = tensor - mean
        variance = (zeroCentered ** 2.0).sum(axis, keepDimensions) / float(elements)
        return mean, variance

    def softmaxCrossEntropy(self, targets):
        """functions/nn/TensorExtensions.kt: logits.softmaxCrossEntropy(targets)."""
        return SoftmaxCrossEntropy(self.ops)(self, targets)

    def argMax(self, axis=0, keepDimensions=False):
        return NoGradVariable(self.ops, self._forwarded().getRawValue().argMax(axis, keepDimensions))

    def argMin(self, axis=0, keepDimensions=False):
        return NoGradVariable(self.ops, self._forwarded().getRawValue().argMin(axis, keepDimensions))

    def exp(self): return Exp(self.ops)(self)
    def log(self): return Log(self.ops)(self)
    def tanh(self): return Tanh(self.ops)(self)
    def sigmoid(self): return Sigmoid(self.ops)(self)
    def sinh(self): return Sinh(self.ops)(self)
    def cosh(self): return Cosh(self.ops)(self)
    def abs(self): return Abs(self.ops)(self)
    def clamp(self, min, max): return Clamp(self.ops)(self, float(min), float(max))
    def sqrt(self): return Sqrt(self.ops)(self)
    def sin(self): return Sin(self.ops)(self)
    def cos(self): return Cos(self.ops)(self)
    def tan(self): return Tan(self.ops)(self)
    def asin(self): return Asin(self.ops)(self)
    def acos(self): return Acos(self.ops)(self)
    def atan(self): return Atan(self.ops)(self)
    def reciprocal(self): return Reciprocal(self.ops)(self)
    def floor(self): return Floor(self.ops)(self)
    def ceil(self): return Ceil(self.ops)(self)
    def round(self): return Round(self.ops)(self)
    def sign(self): return Sign(self.ops)(self)
    def trunc(self): return Trunc(self.ops)(self)
    def rsqrt(self): return Rsqrt(self.ops)(self)
    def _reshape(self, newShape): return Reshape(self.ops)(self, newShape)
    def _expand(self, newShape): return Expand(self.ops)(self, newShape)
    def view(self, *newShape): return Reshape(self.ops, viewMode=True)(self, _as_list(newShape))   # AGTensor.kt:473-475

    def noGrad(self):
        """AGTensor.kt:531-535."""
        self.forward()
        return NoGradVariable(self.ops, self.getRawValue())

    def asVariable(self, requiresGrad=False):
        """AGTensor.kt:541-552."""
        t = self._forwarded()
        if requiresGrad:
            return Variable(self.ops, t.getRawValue())
        return NoGradVariable(self.ops, t.getRawValue())


class NoGradVariable(AGTensor):
    """autograd/tensor/NoGradVariable.kt — no graph while no operand needs grad: the raw
    ops are called directly (NoGradVariable.kt:66-190)."""

    requiresGrad = False

    def __init__(self, ops, rawValue):
        super().__init__(ops)
        self.rawValue = rawValue

    @property
    def shape(self): return self.rawValue.shape

    def getRawValue(self): return self.rawValue
    def forward(self): pass
    def backward(self, gradients=None): raise RuntimeError("Tensor does not require gradients")
    def backwardWithGrad(self, gradient): raise RuntimeError("Tensor does not require gradients")
    def grad(self): raise RuntimeError("Tensor has no gradient")
    def noGrad(self): return self

    def asVariable(self, requiresGrad=False):
        return Variable(self.ops, self.rawValue) if requiresGrad else NoGradVariable(self.ops, self.rawValue)

    def _new(self, raw): return NoGradVariable(self.ops, raw)

    def _eager_binary(self, o, name):
        if _is_number(o):
            return self._new(getattr(self.rawValue, name)(float(o)))
        if o.requiresGrad:
            return getattr(AGTensor, name)(self, o)
        return self._new(getattr(self.rawValue, name)(o.getRawValue()))

    def plus(self, o): return self._eager_binary(o, "plus")
    def minus(self, o): return self._eager_binary(o, "minus")
    def times(self, o): return self._eager_binary(o, "times")
    def div(self, o): return self._eager_binary(o, "div")
    def pow(self, o): return self._eager_binary(o, "pow")
    def rplus(self, c): return self._new(self.rawValue.plus(c))                      # :72
    def rminus(self, c): return self._new(self.rawValue.unaryMinus().plus(c))        # :84  (-t) + c, two ops
    def rtimes(self, c): return self._new(self.rawValue.times(c))                    # :92
    def rdiv(self, c): return self._new(self.rawValue.reciprocal().times(c))         # :104 (1/t) * c, two ops
    def rpow(self, c): return self._new(self.ops.pow(c, self.rawValue))              # :114

    def sum(self, axis=_NO_AXIS, keepDimensions=False):
        return self._new(self.rawValue.sum() if axis is None else self.rawValue.sum(axis, keepDimensions))

    def mean(self, axis=_NO_AXIS, keepDimensions=False):
        return self._new(self.rawValue.mean() if axis is None else self.rawValue.mean(axis, keepDimensions))

    def max(self, axis, keepDimensions=False): return self._new(self.rawValue.max(axis, keepDimensions))
    def min(self, axis, keepDimensions=False): return self._new(self.rawValue.min(axis, keepDimensions))
    def gather(self, axis, index): return self._new(self.rawValue.gather(axis, index.getRawValue()))          # :196
    def indexSelect(self, axis, index): return self._new(self.rawValue.indexSelect(axis, index.getRawValue()))   # :202

    def dot(self, vector):
        if vector.requiresGrad:
            return super().dot(vector)
        return self._new(self.rawValue.dot(vector.getRawValue()))

    def scatter(self, axis, index, source):                                                                   # :198-202
        if source.requiresGrad:
            return AGTensor.scatter(self, axis, index, source)
        return self._new(self.rawValue.scatter(axis, index.getRawValue(), source.getRawValue()))

    def clamp(self, min, max): return self._new(self.rawValue.clamp(float(min), float(max)))
    def _reshape(self, newShape): return self._new(self.rawValue.reshape(newShape))
    def _expand(self, newShape): return self._new(self.rawValue.broadcastTo(newShape))
    def view(self, *newShape): return self._new(self.rawValue.view(_as_list(newShape)))
    def copy(self): return self._new(self.rawValue.copy())

    def __getitem__(self, index): return self._new(self.rawValue.get(_as_index(index)))       # :42-44

    def __setitem__(self, index, value):                                                      # :46-64
        if _is_number(value):
            self.rawValue.set(_as_index(index), float(value))
            return
        if value.requiresGrad:
            value.forward()
        self.rawValue.set(_as_index(index), _safe(value).getRawValue())

    def transpose(self, axis1, axis2): return self._new(self.rawValue.transpose(axis1, axis2))    # :172
    def permute(self, *axes): return self._new(self.rawValue.permute(_as_list(axes)))         # :180

    def concat(self, axis, tensors):                                                          # :182-186
        if any(t.requiresGrad for t in tensors):
            return super().concat(axis, tensors)
        return self._new(self.ops.concat(axis, [t.getRawValue() for t in tensors]))

    def maskedFill(self, mask, value):                                                        # :282
        return self._new(self.rawValue.maskedFill(mask.getRawValue(), float(value)))
    def squeeze(self, axis): return self._new(self.rawValue.squeeze(axis))
    def unsqueeze(self, axis): return self._new(self.rawValue.unsqueeze(axis))
    def lt(self, o): return self._new(self.rawValue.lt(o if _is_number(o) else o.getRawValue()))
    def lte(self, o): return self._new(self.rawValue.lte(o if _is_number(o) else o.getRawValue()))
    def gt(self, o): return self._new(self.rawValue.gt(o if _is_number(o) else o.getRawValue()))
    def gte(self, o): return self._new(self.rawValue.gte(o if _is_number(o) else o.getRawValue()))
    def eq(self, o): return self._new(self.rawValue.eq(o if _is_number(o) else o.getRawValue()))
    def neq(self, o): return self._new(self.rawValue.neq(o if _is_number(o) else o.getRawValue()))

    def release(self): self.ops.release(self.rawValue)
    def incrementRef(self): self.ops.incrementRef(self.rawValue)


for _name in ("exp", "log", "tanh", "sigmoid", "sinh", "cosh", "abs", "sqrt", "sin", "cos", "tan", "asin", "acos",
              "atan", "reciprocal", "floor", "ceil", "round", "sign", "trunc", "rsqrt"):
    def _make(name):
        def method(self):
            return self._new(getattr(self.rawValue, name)())                         # :126-170
        method.__name__ = name
        return method
    setattr(NoGradVariable, _name, _make(_name))


class Variable(AGTensor):
    """autograd/tensor/Variable.kt:15-46 — a leaf; its gradient buffer starts as zeros and
    every backward pass adds into it with plusAssign."""

    def __init__(self, ops, value, gradient=None):
        super().__init__(ops)
        self.value = value
        self.gradient = gradient if gradient is not None else ops.zerosLike(value)

    @property
    def shape(self): return self.value.shape

    def getRawValue(self): return self.value
    def forward(self): pass
    def backward(self, gradients=None):
        if gradients is None:
            return
        if self.shape != gradients.shape:
            raise ValueError(f"Variable with shape: {self.shape} cannot have gradients with shape: {gradients.shape}")
        gradients._forwarded()
        self.backwardWithGrad(gradients.getRawValue())

    def backwardWithGrad(self, gradient):
        self.gradient += gradient                                                     # :44-46

    def zeroGrad(self): self.ops.zeroOut(self.gradient)
    def grad(self): return NoGradVariable(self.ops, self.gradient)

    def asVariable(self, requiresGrad=False):
        return self if requiresGrad else NoGradVariable(self.ops, self.value)

    def release(self): self.ops.release(self.value, self.gradient)

    def incrementRef(self):
        self.ops.incrementRef(self.value)
        self.ops.incrementRef(self.gradient)


class Function(AGTensor):
    """autograd/functions/Function.kt — a graph node. forward runs inputs first, backward
    walks the graph from a [1]-shaped result inside one garbage-collector scope."""

    def __init__(self, ops):
        super().__init__(ops)
        self.keepOutput = False
        self.valuesSaved: List = []
        self._output = None
        self.freeOutput = False
        self.cachedShape: Optional[List[int]] = None
        self.registeredAsInputIn: List["Function"] = []
        self.gradCache = None
        self.backwardRan = False

    # output setter takes a reference (Function.kt:16-21)
    @property
    def output(self): return self._output

    @output.setter
    def output(self, value):
        if value is not None:
            self.ops.incrementRef(value)
        self._output = value

    @property
    def shape(self):
        if self.cachedShape is None:
            if self._output is None:
                self.internalForward()
            self.cachedShape = list(self._output.shape)
        return self.cachedShape

    def hasValue(self) -> bool: return self._output is not None
    def getRawValue(self): return self._output

    def forward(self):                                                                # :47-52
        self.keepOutput = True
        with self.ops.garbageCollector():
            self.internalForward()

    def backward(self, gradients=None):                                               # :54-89
        if gradients is None:
            if len(self.shape) != 1 or self.shape[0] != 1:
                raise RuntimeError("Backward is only allowed on singleton calculation results (tensors with shape [1])")
        elif self.shape != gradients.shape:
            raise ValueError("Backward with gradients require same shape for gradients as the calculation result "
                             f"shape. Result shape: {self.shape} provided gradients shape: {gradients.shape}")
        self._registerInputUsages(self.getInputsAsList())
        with self.ops.garbageCollector():
            if not self.hasValue():
                self.internalForward()
            if gradients is None:
                self.backwardWithGrad(self.ops.createRaw([1], lambda _: 1.0))
            else:
                if isinstance(gradients, Function) and not gradients.hasValue():
                    gradients.forward()
                self.backwardWithGrad(gradients.getRawValue())
            self.releaseUnusedInGraph()

    def _registerInputUsages(self, inputs):                                           # :91-97
        for t in inputs:
            if isinstance(t, Function):
                t.registeredAsInputIn.append(self)
                t._registerInputUsages(t.getInputsAsList())

    def backwardWithGrad(self, gradient):                                             # :108-141
        if len(self.registeredAsInputIn) > 1:
            if self.gradCache is None:
                self.gradCache = gradient.copy()
            else:
                self.gradCache.plusAssign(gradient)
            if not all(f.backwardRan for f in self.registeredAsInputIn):
                return
        gradients = self.doBackward(self.gradCache if self.gradCache is not None else gradient)
        self.backwardRan = True
        self.backwardToInputs(gradients)
        self.ops.release(gradient)
        if self.gradCache is not None:
            self.ops.release(self.gradCache)

    def releaseUnusedInGraph(self):                                                   # :143-152
        if self.freeOutput and self._output is not None:
            self.ops.release(self._output)
            self._output = None
            self.freeOutput = False
        for v in self.valuesSaved:
            self.ops.release(v)
        self.valuesSaved.clear()
        for t in self.getInputsAsList():
            if isinstance(t, Function):
                t.releaseUnusedInGraph()

    def backwardToInputs(self, gradients):                                            # :156-161
        for t, g in zip(self.getInputsAsList(), gradients):
            if isinstance(t, AGTensor) and t.requiresGrad:
                t.backwardWithGrad(g)

    def internalForward(self):                                                        # :163-166
        self.gradCache = None
        self.backwardRan = False

    def saveForBackward(self, *rawValues):                                            # :168-171
        if not self.hasValue() or not self.valuesSaved:
            for r in rawValues:
                self.ops.incrementRef(r)
            self.valuesSaved.extend(rawValues)

    def mayFreeOutput(self):
        if not self.keepOutput:
            self.freeOutput = True

    def grad(self):
        raise RuntimeError("Gradients are only available on variables (graph edges).")

    def release(self):
        if self.keepOutput and self.hasValue():
            self.releaseUnusedInGraph()

    def incrementRef(self):
        if self.hasValue():
            self.ops.incrementRef(self._output)

    def getInputsAsList(self): raise NotImplementedError
    def doBackward(self, gradient): raise NotImplementedError


class BiTensorFunction(Function):
    """functions/BiTensorFunction.kt:10-52."""
    broadcastingOperation = True

    def __call__(self, a, b):
        a, b = _safe(a), _safe(b)
        if self.broadcastingOperation:
            self.cachedShape = sf.infer_implicit_broadcast_shape(a.shape, b.shape)
        self.inputs = (a, b)
        return self

    def getInputsAsList(self): return list(self.inputs)

    def internalForward(self):
        super().internalForward()
        if self.hasValue():
            return
        fns = [t for t in self.inputs if isinstance(t, Function)]
        for f in fns:
            f.internalForward()
        if not self.hasValue():
            a, b = (t.getRawValue() for t in self.inputs)
            self.aShape, self.bShape = list(a.shape), list(b.shape)
            self.doForward(a, b)
        for f in fns:
            f.mayFreeOutput()


class UnaryTensorFunction(Function):
    """functions/UnaryTensorFunction.kt:7-45."""
    modifiesShape = False

    def __call__(self, tensor):
        tensor = _safe(tensor)
        if not self.modifiesShape:
            self.cachedShape = list(tensor.shape)
        self.tensor = tensor
        return self

    def getInputsAsList(self): return [self.tensor]

    def internalForward(self):
        super().internalForward()
        if self.hasValue():
            return
        fn = self.tensor if isinstance(self.tensor, Function) else None
        if fn is not None:
            fn.internalForward()
        if not self.hasValue():
            self.doForward(self.tensor.getRawValue())
        if fn is not None:
            fn.mayFreeOutput()


class TensorConstantFunction(UnaryTensorFunction):
    """functions/TensorConstantFunction.kt:8-28."""

    def __call__(self, x, y=None, constant_first=False):
        if constant_first:
            constant, tensor = x, y
            self.tensorFirst = False
        else:
            tensor, constant = x, y
            self.tensorFirst = True
        super().__call__(tensor)
        self.constant = float(constant)
        return self


# ------------------------------------------------------------------ BasicFunctions.kt

class Plus(BiTensorFunction):                                                         # :7-18
    def doForward(self, a, b): self.output = a + b

    def doBackward(self, gradient):
        return [mayUnexpand(gradient.copy(shallow=True), self.aShape, self.ops),
                mayUnexpand(gradient.copy(shallow=True), self.bShape, self.ops)]


class Minus(BiTensorFunction):                                                        # :20-31
    def doForward(self, a, b): self.output = a - b

    def doBackward(self, gradient):
        return [mayUnexpand(gradient.copy(shallow=True), self.aShape, self.ops),
                mayUnexpand(-gradient, self.bShape, self.ops)]


class Times(BiTensorFunction):                                                        # :33-46
    def doForward(self, a, b):
        self.saveForBackward(a, b)
        self.output = a * b

    def doBackward(self, gradient):
        a, b = self.valuesSaved
        return [mayUnexpand(gradient * b, self.aShape, self.ops), mayUnexpand(gradient * a, self.bShape, self.ops)]


class Div(BiTensorFunction):                                                          # :48-76
    def doForward(self, a, b):
        self.saveForBackward(a, b)
        self.output = a / b

    def doBackward(self, gradient):
        a, b = self.valuesSaved
        bRec = b.reciprocal()
        aGrad = gradient * bRec
        bGrad = -gradient
        if a.shape == b.shape:
            bGrad *= a
            bGrad *= bRec
            bGrad *= bRec
        else:
            bGrad *= a * bRec * bRec
        self.ops.release(bRec)
        return [mayUnexpand(aGrad, self.aShape, self.ops), mayUnexpand(bGrad, self.bShape, self.ops)]


class Pow(BiTensorFunction):                                                          # :78-101
    def doForward(self, a, b):
        self.saveForBackward(a, b)
        self.output = a.pow(b)

    def doBackward(self, gradient):
        a, b = self.valuesSaved
        aGrad = gradient * b
        aGrad *= a.pow(b - 1.0)
        bGrad = gradient * a.pow(b)
        bGrad *= a.log()
        return [mayUnexpand(aGrad, self.aShape, self.ops), mayUnexpand(bGrad, self.bShape, self.ops)]


class PlusConstant(TensorConstantFunction):                                           # :103-114
    def doForward(self, input): self.output = input + self.constant
    def doBackward(self, gradient): return [gradient.copy(shallow=True)]


class MinusConstant(TensorConstantFunction):                                          # :116-137
    def doForward(self, input):
        if self.tensorFirst:
            self.output = input - self.constant
        else:
            self.output = -input
            if self.constant != 0.0:
                self._output += self.constant

    def doBackward(self, gradient):
        return [gradient.copy(shallow=True)] if self.tensorFirst else [-gradient]


class TimesConstant(TensorConstantFunction):                                          # :139-150
    def doForward(self, input): self.output = input * self.constant
    def doBackward(self, gradient): return [gradient * self.constant]


class DivConstant(TensorConstantFunction):                                            # :152-176
    def doForward(self, input):
        if self.tensorFirst:
            self.output = input / self.constant
        else:
            self.saveForBackward(input)
            self.output = input.reciprocal()
            self._output *= self.constant

    def doBackward(self, gradient):
        if self.tensorFirst:
            return [gradient / self.constant]
        res = self.valuesSaved[0].reciprocal()
        res *= res
        res *= gradient
        res *= -self.constant
        return [res]


class PowConstant(TensorConstantFunction):                                            # :178-206
    def doForward(self, input):
        if self.tensorFirst:
            self.saveForBackward(input)
            self.output = input.pow(self.constant)
        else:
            res = self.ops.pow(self.constant, input)
            self.saveForBackward(res)
            self.output = res

    def doBackward(self, gradient):
        if self.tensorFirst:
            (input,) = self.valuesSaved
            inputGrad = gradient * self.constant
            # Kotlin parses `input pow constant - 1f` as input pow (constant - 1f).
            inputGrad *= input.pow(_f32(self.constant - 1.0))
            return [inputGrad]
        (res,) = self.valuesSaved
        inputGrad = gradient * res
        inputGrad *= _f32(math.log(self.constant))     # kotlin.math.ln(Float)
        return [inputGrad]


def _f32(x: float) -> float:
    """Round a Python float to the nearest fp32, as Kotlin Float arithmetic would."""
    import struct
    return struct.unpack("f", struct.pack("f", x))[0]


# ------------------------------------------------------------------ PointwiseFunctions.kt

class Exp(UnaryTensorFunction):                                                       # :8-22
    def doForward(self, input):
        res = input.exp()
        self.saveForBackward(res)
        self.output = res

    def doBackward(self, gradient):
        (res,) = self.valuesSaved
        return [gradient * res]


class Log(UnaryTensorFunction):                                                       # :24-37
    def doForward(self, input):
        self.saveForBackward(input)
        self.output = input.log()

    def doBackward(self, gradient):
        (input,) = self.valuesSaved
        return [gradient / input]


class Tanh(UnaryTensorFunction):                                                      # :39-60
    def doForward(self, input):
        res = input.tanh()
        self.saveForBackward(res)
        self.output = res

    def doBackward(self, gradient):
        (res,) = self.valuesSaved
        g = res * res
        g *= -1.0
        g += 1.0
        g *= gradient
        return [g]


class Sigmoid(UnaryTensorFunction):                                                   # :62-82
    def doForward(self, input):
        res = input.sigmoid()
        self.saveForBackward(res)
        self.output = res

    def doBackward(self, gradient):
        (res,) = self.valuesSaved
        g = -res
        g += 1.0
        g *= res
        g *= gradient
        return [g]


def _saved_input_function(forward_name, backward):
    class _F(UnaryTensorFunction):
        def doForward(self, input):
            self.saveForBackward(input)
            self.output = getattr(input, forward_name)()

        def doBackward(self, gradient):
            (input,) = self.valuesSaved
            return [backward(self, input, gradient)]
    return _F


def _times_assign(t, g):
    t *= g
    return t


def _sqrt_backward(self, input, gradient):                                            # :171-178
    g = input.pow(-0.5)
    g *= gradient
    g /= 2.0
    return g


def _cos_backward(self, input, gradient):                                             # :204-210
    g = input.sin()
    g *= gradient
    g *= -1.0
    return g


def _tan_backward(self, input, gradient):                                             # :222-229
    c = input.cos()
    c2 = c.pow(2.0)
    g = gradient / c2
    self.ops.release(c, c2)
    return g


Sinh = _saved_input_function("sinh", lambda self, x, g: _times_assign(x.cosh(), g))   # :84-98
Cosh = _saved_input_function("cosh", lambda self, x, g: _times_assign(x.sinh(), g))   # :100-114
Abs = _saved_input_function("abs", lambda self, x, g: _times_assign(x.sign(), g))     # :116-130
Sqrt = _saved_input_function("sqrt", _sqrt_backward)                                  # :165-180
Sin = _saved_input_function("sin", lambda self, x, g: _times_assign(x.cos(), g))      # :182-196
Cos = _saved_input_function("cos", _cos_backward)                                     # :198-213
Tan = _saved_input_function("tan", _tan_backward)                                     # :215-231
Asin = _saved_input_function("asin", lambda self, x, g: g * (-(x * x) + 1.0).sqrt().reciprocal())      # :233-245
Acos = _saved_input_function("acos", lambda self, x, g: g * -((-(x * x) + 1.0).sqrt().reciprocal()))   # :247-259
Atan = _saved_input_function("atan", lambda self, x, g: g * (x * x + 1.0).reciprocal())                # :261-273


class Clamp(UnaryTensorFunction):                                                     # :132-163
    def __call__(self, tensor, min, max):
        super().__call__(tensor)
        self.min, self.max = min, max
        return self

    def doForward(self, input):
        self.saveForBackward(input)
        self.output = input.clamp(self.min, self.max)

    def doBackward(self, gradient):
        (input,) = self.valuesSaved
        mask = input.gte(self.min)
        maxMask = input.lte(self.max)
        mask *= maxMask
        gradIn = gradient * mask
        self.ops.release(mask, maxMask)
        return [gradIn]


class Reciprocal(UnaryTensorFunction):                                                # :275-293
    def doForward(self, input):
        res = input.reciprocal()
        self.saveForBackward(res)
        self.output = res

    def doBackward(self, gradient):
        (res,) = self.valuesSaved
        resSqr = res * res
        gradReciprocal = -resSqr
        gradInput = gradient * gradReciprocal
        self.ops.release(resSqr, gradReciprocal)
        return [gradInput]


def _constant_grad(name, gradientValue=0.0):                                          # :295-334
    class _F(UnaryTensorFunction):
        def doForward(self, input):
            self.inputShape = list(input.shape)
            self.output = getattr(input, name)()

        def doBackward(self, gradient):
            return [mayUnexpand(gradient * gradientValue, self.inputShape, self.ops)]
    return _F


Floor, Ceil, Round, Sign, Trunc = (_constant_grad(n) for n in ("floor", "ceil", "round", "sign", "trunc"))


class Rsqrt(UnaryTensorFunction):                                                     # :338-359
    def doForward(self, input):
        res = input.rsqrt()
        self.saveForBackward(res)
        self.output = res

    def doBackward(self, gradient):
        (res,) = self.valuesSaved
        g = res.pow(3.0)
        g /= -2.0
        gradInput = gradient * g
        self.ops.release(g)
        return [gradInput]


# ------------------------------------------------------------------ AggregatingFunctions.kt

class AggregatorFunction(UnaryTensorFunction):
    """functions/AggregatorFunction.kt:9-32."""
    modifiesShape = True

    def __call__(self, tensor, axis, keepDimensions):
        self.cachedShape = [1] if axis is None else sf.aggregate_over(tensor.shape, axis, keepDimensions)
        super().__call__(tensor)
        self.axis = None if axis is None else sf.normalize_axis(tensor.shape, axis)
        self.keepDimensions = keepDimensions
        return self


class Sum(AggregatorFunction):                                                        # :7-26
    def doForward(self, input):
        self.inputShape = list(input.shape)
        self.output = input.sum() if self.axis is None else input.sum(self.axis, self.keepDimensions)

    def doBackward(self, gradient):
        if not self.keepDimensions and len(self.inputShape) != 1 and self.axis is not None:
            gradient.inplaceUnsqueeze(self.axis)
        return [gradient.broadcastTo(self.inputShape)]


class Mean(AggregatorFunction):                                                       # :28-54
    def doForward(self, input):
        self.inputShape = list(input.shape)
        self.output = input.mean() if self.axis is None else input.mean(self.axis, self.keepDimensions)

    def doBackward(self, gradient):
        if self.axis is None:
            gradInput = gradient / float(sf.to_store_size(self.inputShape))
            return [gradInput.broadcastTo(self.inputShape)]
        if not self.keepDimensions and len(self.inputShape) != 1:
            gradient.inplaceUnsqueeze(self.axis)
        gradInput = gradient.broadcastTo(self.inputShape)
        gradInput /= float(self.inputShape[self.axis])
        return [gradInput]


class SelectionFunction(AggregatorFunction):                                          # :56-81
    """Max / Min: the forward keeps the arg indices; the backward scatters the gradient
    into zeros at those indices."""
    def select(self, tensor, axis, keepDimensions): raise NotImplementedError

    def doForward(self, input):
        self.inputShape = list(input.shape)
        res, indices = self.select(input, self.axis, self.keepDimensions)
        self.saveForBackward(input, indices)
        self.output = res

    def doBackward(self, gradient):
        input, indices = self.valuesSaved
        gradInput = self.ops.zerosLike(input)
        if not self.keepDimensions and len(self.inputShape) != 1:
            gradient.inplaceUnsqueeze(self.axis)
            indices.inplaceUnsqueeze(self.axis)
        gradInput.inplaceScatter(self.axis, indices, gradient)
        return [gradInput]


class Max(SelectionFunction):                                                         # :83-87
    def select(self, t, axis, keep): return t.max(axis, keep), t.argMax(axis, keep)


class Min(SelectionFunction):                                                         # :89-93
    def select(self, t, axis, keep): return t.min(axis, keep), t.argMin(axis, keep)


# ------------------------------------------------------------------ TensorFunctions.kt

class Reshape(UnaryTensorFunction):                                                   # :200-231
    modifiesShape = True

    def __init__(self, ops, viewMode=False):
        super().__init__(ops)
        self.viewMode = viewMode

    def __call__(self, tensor, newShape):
        self.cachedShape = sf.reshape(tensor.shape, newShape)
        super().__call__(tensor)
        self.newShape = list(newShape)
        return self

    def doForward(self, input):
        self.oldShape = list(input.shape)
        self.output = input.view(self.newShape) if self.viewMode else input.reshape(self.newShape)

    def doBackward(self, gradient):
        return [gradient.view(self.oldShape) if self.viewMode else gradient.reshape(self.oldShape)]


class Expand(UnaryTensorFunction):                                                    # :233-284
    modifiesShape = True

    def __call__(self, tensor, newShape):
        self.cachedShape = sf.infer_explicit_broadcast_shape(tensor.shape, newShape)
        super().__call__(tensor)
        self.newShape = list(newShape)
        return self

    def doForward(self, input):
        self.output = input.broadcastTo(self.newShape)
        self.unsqueezedDims = len(self.newShape) - input.dimensions
        self.expandedDims = [i for i, (e, o) in enumerate(zip(self.newShape[self.unsqueezedDims:], input.shape))
                             if e != o]

    def doBackward(self, gradient):
        g = gradient
        for i in range(self.unsqueezedDims):
            to_release = g
            g = g.sum(0)
            if i > 0:
                self.ops.release(to_release)
        for i, d in enumerate(self.expandedDims):
            to_release = g
            g = g.sum(d, True)
            if i > 0:
                self.ops.release(to_release)
        return [g]


class Gather(UnaryTensorFunction):                                                    # :444-479
    modifiesShape = True

    def __call__(self, tensor, axis, index):
        if index.requiresGrad:
            raise ValueError("Gather cannot differentiate the index. The index tensor passed to gather should never "
                             "require gradients.")
        super().__call__(tensor)
        self.axis, self.index = axis, index
        return self

    def doForward(self, input):
        self.inputShape = list(input.shape)
        indexRaw = self.index.getRawValue()
        self.saveForBackward(indexRaw)
        self.output = input.gather(self.axis, indexRaw)

    def doBackward(self, gradient):
        gradInput = self.ops.createRawFill(self.inputShape, 0.0)
        (index,) = self.valuesSaved
        gradInput.inplaceScatterAdd(self.axis, index, gradient)
        return [gradInput]


class Scatter(BiTensorFunction):                                                      # :481-527
    broadcastingOperation = False

    def __call__(self, tensor, axis, index, source):
        if index.requiresGrad:
            raise ValueError("Scatter cannot differentiate the index. The index tensor passed to scatter should never "
                             "require gradients.")
        super().__call__(tensor, source)
        self.cachedShape = list(tensor.shape)
        self.axis, self.index = axis, index
        return self

    def doForward(self, tensor, source):
        indexRaw = self.index.getRawValue()
        self.saveForBackward(indexRaw)
        self.output = tensor.scatter(self.axis, indexRaw, source)

    def doBackward(self, gradient):
        (index,) = self.valuesSaved
        if index.shape != self.bShape:
            raise ValueError(f"Index shape: {index.shape} is not compatible with source shape: {self.bShape}")
        first, second = self.inputs
        gradInput = gradient.scatter(self.axis, index, 0.0) if first.requiresGrad else None
        gradSource = gradient.gather(self.axis, index) if second.requiresGrad else None
        return [gradInput, gradSource]


class AnyTensorFunction(Function):
    """functions/AnyTensorFunction.kt — a node over a list of inputs."""

    def getInputsAsList(self): return list(self.inputTensors)

    def internalForward(self):
        super().internalForward()
        if self.hasValue():
            return
        fns = [t for t in self.inputTensors if isinstance(t, Function)]
        for f in fns:
            f.internalForward()
        if not self.hasValue():
            self.doForward([t.getRawValue() for t in self.inputTensors])
        for f in fns:
            f.mayFreeOutput()


class AbstractIndexingFunction(UnaryTensorFunction):                                  # TensorFunctions.kt:33-61
    def __call__(self, tensor, index):
        ranged = sf.is_range_index(index)
        if ranged:
            self.index, indexedShape = sf.normalized_range_indexed_shape(tensor.shape, index)
        else:
            self.index, indexedShape = sf.normalized_indexed_shape(tensor.shape, index)
        super().__call__(tensor)
        if ranged or self.modifiesShape:
            self.cachedShape = indexedShape
        return self

    def doForward(self, input):
        self.inputShape = list(input.shape)


class Index(AbstractIndexingFunction):                                                # :63-82
    modifiesShape = True

    def doForward(self, input):
        super().doForward(input)
        self.output = input.get(self.index)

    def doBackward(self, gradient):
        gradInput = self.ops.createRawFill(self.inputShape, 0.0)
        gradInput.set(self.index, gradient)
        return [gradInput]


class IndexSetTensor(BiTensorFunction):                                               # :84-131
    broadcastingOperation = False

    def __call__(self, tensor, index, value):
        if sf.is_range_index(index):
            normalized, indexedShape = sf.normalized_range_indexed_shape(tensor.shape, index)
        else:
            normalized, indexedShape = sf.normalized_indexed_shape(tensor.shape, index)
        self.valueShape = list(value.shape)
        if self.valueShape != indexedShape:
            raise ValueError(f"Cannot set value with shape: {self.valueShape} at index: {list(index)} on tensor with "
                             f"shape: {tensor.shape}")
        super().__call__(tensor, value)
        self.cachedShape = list(tensor.shape)
        self.index = normalized
        return self

    def doForward(self, a, b):
        self.ops.incrementRef(a)        # not to be freed after forward
        a.set(self.index, b)
        self.output = a

    def doBackward(self, gradient):
        gradInput = gradient.copy()
        gradInput.set(self.index, 0.0)
        gradValue = gradient.get(self.index).view(self.valueShape)
        return [gradInput, gradValue]


class IndexSetConstant(AbstractIndexingFunction):                                     # :133-177
    def __call__(self, tensor, index, value):
        super().__call__(tensor, index)
        self.cachedShape = list(tensor.shape)
        if len(index) != len(tensor.shape):
            raise ValueError(f"Cannot set value at index: {list(index)} on tensor with shape: {tensor.shape} "
                             "(All tensor dimensions must be indexed to set a constant value)")
        self.value = float(value)
        return self

    def doForward(self, input):
        super().doForward(input)
        self.ops.incrementRef(input)
        input.set(self.index, self.value)
        self.output = input

    def doBackward(self, gradient):
        gradInput = gradient.copy()
        gradInput.set(self.index, 0.0)
        return [gradInput]


class Transpose(UnaryTensorFunction):                                                 # :179-198
    modifiesShape = True

    def __call__(self, tensor, axis1, axis2):
        super().__call__(tensor)
        self.cachedShape = sf.transpose_normalize_axes(tensor.shape, axis1, axis2)[0]
        self.axis1, self.axis2 = axis1, axis2
        return self

    def doForward(self, input):
        self.output = input.transpose(self.axis1, self.axis2)

    def doBackward(self, gradient):
        return [gradient.transpose(self.axis1, self.axis2)]


class Permute(UnaryTensorFunction):                                                   # :286-312
    modifiesShape = True

    def __call__(self, tensor, axes):
        super().__call__(tensor)
        self.cachedShape = sf.permute(tensor.shape, axes)
        self.axes = list(axes)
        return self

    def doForward(self, input):
        self.reverseShapeIndices = [self.axes.index(d) for d in range(len(self.axes))]
        self.output = input.permute(self.axes)

    def doBackward(self, gradient):
        return [gradient.permute(self.reverseShapeIndices)]


class Dot(BiTensorFunction):                                                          # functions/BlasFunctions.kt:102-127
    broadcastingOperation = False

    def __call__(self, a, b):
        self.cachedShape = sf.dot_shape(a.shape, b.shape)
        return super().__call__(a, b)

    def doForward(self, a, b):
        self.saveForBackward(a, b)
        self.output = a.dot(b)

    def doBackward(self, gradient):
        vector1, vector2 = self.valuesSaved
        first, second = self.inputs
        return [vector2 * gradient.broadcastTo(self.bShape) if first.requiresGrad else None,
                vector1 * gradient.broadcastTo(self.aShape) if second.requiresGrad else None]


class IndexSelect(UnaryTensorFunction):                                               # :314-347
    modifiesShape = True

    def __call__(self, tensor, index, axis):
        if index.requiresGrad:
            raise ValueError("Index select cannot differentiate the index. The index tensor passed to index select should "
                             "never require gradients.")
        normAxis, outputShape = sf.index_select_norm_axis_shape(tensor.shape, axis, index.shape)
        super().__call__(tensor)
        self.cachedShape = outputShape
        self.originalTensorShape = list(tensor.shape)
        self.axis, self.index = normAxis, index
        return self

    def doForward(self, input):
        self.output = input.indexSelect(self.axis, self.index.getRawValue())

    def doBackward(self, gradient):
        gradInput = self.ops.createRawFill(self.originalTensorShape, 0.0)
        gradInput.indexAdd(self.axis, self.index.getRawValue(), gradient)
        return [gradInput]


class Concat(AnyTensorFunction):                                                      # :349-378
    def __call__(self, axis, inputTensors):
        self.cachedShape = sf.concat_shapes([t.shape for t in inputTensors], axis)
        self.inputTensors = list(inputTensors)
        self.axis = sf.normalize_axis(self.cachedShape, axis)
        return self

    def doForward(self, inputs):
        self.inputSizes = [t.shape[self.axis] for t in inputs]
        self.output = self.ops.concat(self.axis, inputs)

    def doBackward(self, gradient):
        grads, end = [], 0
        for size in self.inputSizes:
            end += size
            grads.append(gradient.narrow(self.axis, end - size, size))
        return grads


class Copy(UnaryTensorFunction):                                                      # :380-392
    def doForward(self, input): self.output = input.copy()
    def doBackward(self, gradient): return [gradient.copy(shallow=True)]


class Squeeze(UnaryTensorFunction):                                                   # :394-420
    modifiesShape = True

    def __call__(self, tensor, axis):
        super().__call__(tensor)
        self.cachedShape = sf.squeeze(tensor.shape, axis)
        self.axis = axis
        return self

    def doForward(self, input):
        self.inputShape = list(input.shape)
        self.output = input.squeeze(self.axis)

    def doBackward(self, gradient):
        return [gradient.reshape(self.inputShape)]


class Unsqueeze(UnaryTensorFunction):                                                 # :422-442
    modifiesShape = True

    def __call__(self, tensor, axis):
        super().__call__(tensor)
        self.cachedShape = sf.unsqueeze(tensor.shape, axis)
        self.axis = axis
        return self

    def doForward(self, input): self.output = input.unsqueeze(self.axis)
    def doBackward(self, gradient): return [gradient.squeeze(self.axis)]


class MaskedFill(UnaryTensorFunction):                                                # :561-584
    def __call__(self, tensor, mask, value):
        super().__call__(tensor)
        if mask.requiresGrad:
            raise ValueError("Masked fill only accepts mask that doesn't require gradients")
        self.mask = mask.getRawValue()
        self.value = float(value)
        return self

    def doForward(self, input):
        self.output = input.maskedFill(self.mask, self.value)

    def doBackward(self, gradient):
        return [gradient.maskedFill(self.mask, 0.0)]


class BatchNormalizationFunction(Function):
    """functions/nn/BatchNormalizationFunction.kt:12-150 — one raw call forward
    (calculateOutput) and one backward (calculateGrads); running statistics are updated in
    place by the forward call in training mode."""

    def __init__(self, axis, momentum, epsilon, training, ops):
        super().__init__(ops)
        self.axis, self.momentum, self.epsilon, self.training = axis, float(momentum), float(epsilon), bool(training)
        self.runningMean = self.runningVar = self.gamma = self.beta = None

    def __call__(self, input, runningMean, runningVar, gamma, beta):
        self.input = _safe(input)
        if runningMean is not None and runningVar is None:
            raise ValueError("Running mean and running var must be both set to non-null or both has to be null")
        if runningMean is None and runningVar is None and not self.training:
            raise ValueError("Running mean and running var must be non-null for inference mode")
        if runningMean is not None:
            if not isinstance(runningMean, NoGradVariable) or not isinstance(runningVar, NoGradVariable):
                raise ValueError("Running mean and running var parameters for batch normalization must be variables "
                                 "requiring no gradients")
            self.runningMean, self.runningVar = runningMean, runningVar
            runningMean.incrementRef(); runningVar.incrementRef()
        self.gamma = _safe(gamma) if gamma is not None else None
        self.beta = _safe(beta) if beta is not None else None
        normAxis = sf.normalize_axis(input.shape, self.axis)
        self.keepOutput = True
        size = self.input.shape[normAxis]
        if runningMean is not None and runningVar is not None:
            if (runningMean.dimensions != 1 or runningVar.dimensions != 1
                    or (self.gamma.dimensions if self.gamma is not None else 1) != 1
                    or (self.beta.dimensions if self.beta is not None else 1) != 1
                    or runningMean.shape[0] != size or runningVar.shape[0] != size):
                raise ValueError("Running mean and running var parameters for batch normalization all must have "
                                 f"shape: [{size}], but got tensors with shapes: running mean: {runningMean.shape} "
                                 f"running var: {runningVar.shape} ")
        if ((self.gamma.shape[0] if self.gamma is not None else size) != size
                or (self.beta.shape[0] if self.beta is not None else size) != size):
            raise ValueError(f"Gamma and beta parameters for batch normalization all must have shape: [{size}]")
        self.batchNormOp = self.ops.batchNorm(normAxis, self.momentum, self.epsilon, self.training)
        self.cachedShape = list(input.shape)
        return self

    def getInputsAsList(self):
        return [t for t in (self.input, self.gamma, self.beta) if t is not None]

    def internalForward(self):
        super().internalForward()
        if self.hasValue():
            return
        fns = [t for t in (self.input, self.runningMean, self.runningVar, self.gamma, self.beta) if isinstance(t, Function)]
        for f in fns:
            f.internalForward()
        if not self.hasValue():
            raw = lambda t: None if t is None else t.getRawValue()
            output, currentMean, currentStd = self.batchNormOp.calculateOutput(
                raw(self.input), raw(self.runningMean), raw(self.runningVar), raw(self.gamma), raw(self.beta))
            self._saved = (raw(self.input), currentMean, currentStd, raw(self.runningMean), raw(self.runningVar), raw(self.gamma))
            self.saveForBackward(*[v for v in self._saved if v is not None])
            self.output = output
        for f in fns:
            f.mayFreeOutput()

    def doBackward(self, gradient):
        input, currentMean, currentStd, runningMean, runningVar, gamma = self._saved
        if gradient.shape != input.shape:
            raise RuntimeError(f"Gradient shape mismatch, output grad shape: {gradient.shape} input shape: {input.shape}")
        return list(self.batchNormOp.calculateGrads(
            input, runningMean, runningVar, currentMean, currentStd, gamma, gradient,
            self.input.requiresGrad, self.gamma.requiresGrad if self.gamma is not None else False,
            self.beta.requiresGrad if self.beta is not None else False))


class SoftmaxCrossEntropy(UnaryTensorFunction):
    """functions/nn/SoftmaxCrossEntropy.kt:10-69 — composed entirely of raw ops on the
    path: max, minus, exp, sum, div, clamp, log, gather, neg, mean; the backward is
    zerosLike, scatter of -1, plusAssign, divAssign (and, as in the reference, does not
    use the incoming gradient)."""
    modifiesShape = True
    epsilon = 1e-7          # PlatformProvider.epsilon

    def __call__(self, logits, targets):
        super().__call__(logits)
        self.cachedShape = [1]
        if targets.requiresGrad:
            raise ValueError("SoftmaxCrossEntropy only accept targets that don't require gradients")
        if logits.dimensions != 2:
            raise ValueError(f"SoftmaxCrossEntropy requires 2D logits, but got tensor with shape {logits.shape}")
        if targets.dimensions != 1:
            raise ValueError(f"SoftmaxCrossEntropy requires 1D targets, but got tensor with shape {targets.shape}")
        if logits.shape[0] != targets.shape[0]:
            raise ValueError("Logits must have the same size at the first dimension as targets, but got tensors with "
                             f"shape: logits: {logits.shape}, targets: {targets.shape}")
        self.targets = targets.unsqueeze(-1)
        return self

    def doForward(self, input):
        maxVal = input.max(-1, keepDimensions=True)
        inputMinusMax = input - maxVal
        expVal = inputMinusMax.exp()
        expValSum = expVal.sum(-1, keepDimensions=True)
        softmaxRes = expVal / expValSum
        self.saveForBackward(softmaxRes)
        softmaxSum = softmaxRes.sum(-1, keepDimensions=True)
        softmaxNorm = softmaxRes / softmaxSum
        softmaxNormClip = softmaxNorm.clamp(_f32(self.epsilon), _f32(1.0 - _f32(self.epsilon)))
        logSoftmax = softmaxNormClip.log()
        logSoftmaxAtTargets = logSoftmax.gather(-1, self.targets.getRawValue())
        negativeLogLikelihood = -logSoftmaxAtTargets
        self.output = negativeLogLikelihood.mean()
        self.ops.release(maxVal, inputMinusMax, expVal, expValSum, softmaxSum, softmaxNorm, softmaxNormClip, logSoftmax,
                         logSoftmaxAtTargets, negativeLogLikelihood)

    def doBackward(self, gradient):
        gradIn = self.ops.zerosLike(self.valuesSaved[0])
        gradIn.inplaceScatter(-1, self.targets.getRawValue(), -1.0)
        gradIn += self.valuesSaved[0]
        gradIn /= float(self.targets.shape[0])
        return [gradIn]


# ------------------------------------------------------------------ companion factories

def tensorOf(ops, *values, requiresGrad=False):
    """Tensor.tensorOf (Tensor.kt:1645-1655): a 1-D tensor of the given values."""
    vals = [float(v) for v in values]
    return ops.create([len(vals)], requiresGrad, vals)


def concat(*tensors, axis=0):
    """Tensor.concat (Tensor.kt:1774-1784)."""
    tensors = _as_list(tensors)
    if len(tensors) == 0:
        raise ValueError("No tensors were passed to concat")
    if len(tensors) == 1:
        return tensors[0]
    owner = next((t for t in tensors if t.requiresGrad), tensors[0])
    return owner.concat(axis, tensors)


def ones(ops, *shape, requiresGrad=False):
    return ops.createFillConst(list(shape), requiresGrad, 1.0)


def zeros(ops, *shape, requiresGrad=False):
    return ops.createFillConst(list(shape), requiresGrad, 0.0)
