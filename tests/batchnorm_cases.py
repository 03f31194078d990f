"""The reference's four batch-norm tests (kten-testing/.../tests/TensorTestsBase.kt:2015-2150),
written once against the `Tensor` API and run on any backend: the fused op must agree with
the same computation composed from elementwise ops and reductions, forward, running
statistics and gradients. Inputs are seeded Gaussians (the reference draws unseeded
Gaussians, AbstractJVMTensorOperations.kt:41-44). Tolerances are the reference's, except for
the gamma gradient: there both sides are sums of ~200 zero-centred values, i.e. rounding
noise of a few 1e-6 around 0, and the reference's 1e-6 holds or fails by chance; 2e-5 is
used instead."""
import numpy as np

from kten_amd.host_mirror.inputs import SplitMix64
from known_answer_cases import assertTensorEquals


def _random(ops, gen, shape, requiresGrad=False):
    return ops.create(list(shape), requiresGrad, gen.normal(list(shape)))


def case_train_mode(ops, with_affine=True, seed=21):                       # :2015-2062 and :2086-2127
    gen = SplitMix64(seed)
    tensor = _random(ops, gen, [10, 3, 4, 5], True)
    axis, momentum, epsilon = 1, 0.1, 1e-3
    gamma = _random(ops, gen, [1, 3, 1, 1], True) if with_affine else None
    beta = _random(ops, gen, [1, 3, 1, 1], True) if with_affine else None
    runningMeanBase = _random(ops, gen, [1, 3, 1, 1])
    runningVarBase = _random(ops, gen, [1, 3, 1, 1])

    t = tensor.permute(1, 0, 2, 3).view(3, -1)
    m, v = t.meanVariance(1)
    mean, variance = m.view(1, 3, 1, 1), v.view(1, 3, 1, 1)
    runningMean = (mean.noGrad() * momentum) + runningMeanBase * (1.0 - momentum)
    runningVar = (variance.noGrad() * momentum) + runningVarBase * (1.0 - momentum)
    result = (tensor - mean) / (variance + epsilon).sqrt()
    if with_affine:
        result = result * gamma + beta
    result.sum().backward()
    grads = [p.grad().toArray().copy() for p in (tensor, gamma, beta) if p is not None]
    for p in (tensor, gamma, beta):
        if p is not None:
            p.zeroGrad()

    runningMean2, runningVar2 = runningMeanBase.reshape(3), runningVarBase.reshape(3)
    result2 = tensor.batchNorm(axis, runningMean2, runningVar2, True, momentum, epsilon,
                               gamma.view(3) if with_affine else None, beta.view(3) if with_affine else None)
    result2.sum().backward()

    assertTensorEquals(result.toArray(), result2, 0.02 if with_affine else 0.01)
    assertTensorEquals(runningMean.view(3).toArray(), runningMean2)
    assertTensorEquals(runningVar.view(3).toArray(), runningVar2)
    assertTensorEquals(grads[0], tensor.grad())
    if with_affine:
        assertTensorEquals(grads[1], gamma.grad(), 2e-5)
        assertTensorEquals(grads[2], beta.grad())


def case_inference_mode(ops, with_affine=True, seed=22):                   # :2064-2084 and :2129-2150
    gen = SplitMix64(seed)
    tensor = _random(ops, gen, [10, 3, 4, 5])
    axis, momentum, epsilon = 2, 0.1, 1e-3
    gamma = _random(ops, gen, [1, 1, 4, 1]) if with_affine else None
    beta = _random(ops, gen, [1, 1, 4, 1]) if with_affine else None
    runningMean = _random(ops, gen, [1, 1, 4, 1])
    runningVar = ops.create([1, 1, 4, 1], False, np.abs(gen.normal([1, 1, 4, 1])))     # a variance: kept non-negative
    result = (tensor - runningMean) / (runningVar + epsilon).sqrt()
    if with_affine:
        result = result * gamma + beta
    result2 = tensor.batchNorm(axis, runningMean.reshape(4), runningVar.reshape(4), False, momentum, epsilon,
                               gamma.view(4) if with_affine else None, beta.view(4) if with_affine else None)
    assertTensorEquals(result.toArray(), result2, 2e-6)


CASES = [("train_mode", lambda ops: case_train_mode(ops, True)),
         ("inference_mode", lambda ops: case_inference_mode(ops, True)),
         ("train_mode_without_gamma_and_beta", lambda ops: case_train_mode(ops, False)),
         ("inference_mode_without_gamma_and_beta", lambda ops: case_inference_mode(ops, False))]
