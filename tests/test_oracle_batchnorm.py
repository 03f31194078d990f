"""Pins the CPU checker's fused batch normalisation: the reference's own four tests (fused op
against the same computation composed from elementwise ops, on the checker backend), float64
closed forms for the forward statistics and an independently derived float64 gradient, and
the literal float order of the running-statistics update."""
import numpy as np
import pytest

import batchnorm_cases as bnc
from kten_amd.host_mirror.inputs import SplitMix64
from oracle import jvm_oracle as jo


@pytest.mark.parametrize("name,case", bnc.CASES, ids=[n for n, _ in bnc.CASES])
def test_reference_batch_norm_tests(name, case, oracle_ops):
    case(oracle_ops)


def _setup(ops, shape, axis, seed, affine=True, running=True):
    gen = SplitMix64(seed)
    c = shape[axis]
    x = gen.normal(shape) * np.float32(1.7) + np.float32(0.3)
    raw = lambda a: ops.createRaw(list(a.shape), a.reshape(-1))
    t = {"x": x, "gamma": gen.normal([c]) if affine else None, "beta": gen.normal([c]) if affine else None,
         "rm": gen.normal([c]) if running else None, "rv": np.abs(gen.normal([c])) if running else None, "go": gen.normal(shape)}
    return t, {k: (None if v is None else raw(v)) for k, v in t.items()}


def f64_batch_norm(x, axis, eps, gamma, beta, go):
    """Textbook batch normalisation and its gradient in float64 (independent of the checker:
    gradIn = gamma * s * (go - mean(go) - xhat * mean(go * xhat)), s = 1/sqrt(var + eps))."""
    red = tuple(d for d in range(x.ndim) if d != axis)
    bshape = [1] * x.ndim; bshape[axis] = x.shape[axis]
    x = x.astype(np.float64); go = go.astype(np.float64)
    g = np.ones(bshape) if gamma is None else gamma.astype(np.float64).reshape(bshape)
    b = np.zeros(bshape) if beta is None else beta.astype(np.float64).reshape(bshape)
    mean = x.mean(red, keepdims=True)
    var = ((x - mean) ** 2).mean(red, keepdims=True)
    s = 1.0 / np.sqrt(var + eps)
    xhat = (x - mean) * s
    out = xhat * g + b
    grad_in = g * s * (go - go.mean(red, keepdims=True) - xhat * (go * xhat).mean(red, keepdims=True))
    return {"out": out, "mean": mean.reshape(-1), "std": s.reshape(-1), "ssd": ((x - mean) ** 2).sum(red),
            "grad_in": grad_in, "grad_gamma": (go * xhat).sum(red), "grad_beta": go.sum(red)}


@pytest.mark.parametrize("shape,axis", [([10, 3, 4, 5], 1), ([6, 5], 1), ([6, 5], 0), ([4, 3, 70], 1), ([2, 3, 4, 5], 3), ([7, 2, 3], 0)])
def test_training_mode_against_float64(shape, axis, oracle_ops):
    eps, momentum = 1e-3, 0.1
    t, r = _setup(oracle_ops, shape, axis, seed=sum(shape) + axis)
    op = oracle_ops.batchNorm(axis, momentum, eps, True)
    rm0, rv0 = t["rm"].copy(), t["rv"].copy()
    out, mean, std = op.calculateOutput(r["x"], r["rm"], r["rv"], r["gamma"], r["beta"])
    ref = f64_batch_norm(t["x"], axis, eps, t["gamma"], t["beta"], t["go"])
    n = t["x"].size // shape[axis]
    assert np.allclose(mean.toArray(), ref["mean"], rtol=0, atol=2e-6)
    assert np.allclose(std.toArray(), ref["std"], rtol=2e-6)
    assert np.allclose(out.toArray(), ref["out"], rtol=1e-5, atol=1e-5)
    # running statistics: momentum * stat + (1 - momentum) * old, with the UNBIASED variance (JVMBatchNorm.kt:72-76)
    assert np.allclose(r["rm"].toArray(), momentum * ref["mean"] + (1 - momentum) * rm0, rtol=1e-6, atol=1e-6)
    assert np.allclose(r["rv"].toArray(), momentum * ref["ssd"] / (n - 1) + (1 - momentum) * rv0, rtol=1e-5, atol=1e-6)
    gin, ggamma, gbeta = op.calculateGrads(r["x"], r["rm"], r["rv"], mean, std, r["gamma"], r["go"], True, True, True)
    scale = np.abs(ref["grad_in"]).max()
    assert np.abs(gin.toArray() - ref["grad_in"]).max() <= 2e-5 * scale
    assert np.allclose(ggamma.toArray(), ref["grad_gamma"], rtol=1e-4, atol=1e-4)
    assert np.allclose(gbeta.toArray(), ref["grad_beta"], rtol=1e-5, atol=1e-4)


def test_inference_mode_against_float64(oracle_ops):
    shape, axis, eps = [5, 4, 6], 1, 1e-3
    t, r = _setup(oracle_ops, shape, axis, seed=9)
    op = oracle_ops.batchNorm(axis, 0.1, eps, False)
    out, mean, std = op.calculateOutput(r["x"], r["rm"], r["rv"], r["gamma"], r["beta"])
    b = [1, 4, 1]
    s = 1.0 / np.sqrt(t["rv"].astype(np.float64).reshape(b) + eps)
    want = (t["x"].astype(np.float64) - t["rm"].reshape(b)) * s * t["gamma"].reshape(b) + t["beta"].reshape(b)
    assert np.allclose(out.toArray(), want, rtol=1e-5, atol=1e-5)
    assert not mean.toArray().any() and not std.toArray().any()            # left as allocated (JVMBatchNorm.kt:41-42,78-81)
    assert np.array_equal(r["rm"].toArray(), t["rm"]) and np.array_equal(r["rv"].toArray(), t["rv"])
    gin, ggamma, gbeta = op.calculateGrads(r["x"], r["rm"], r["rv"], mean, std, r["gamma"], r["go"], True, True, True)
    go = t["go"].astype(np.float64)
    assert np.allclose(gin.toArray(), go * s * t["gamma"].reshape(b), rtol=1e-5, atol=1e-6)
    assert np.allclose(gbeta.toArray(), go.sum((0, 2)), rtol=1e-5, atol=1e-4)
    assert np.allclose(ggamma.toArray(), (go * (t["x"] - t["rm"].reshape(b)) * s).sum((0, 2)), rtol=1e-4, atol=1e-4)


def test_literal_float_order_of_one_channel(oracle_ops):
    """One channel by hand in float32, in the reference's order (JVMBatchNorm.kt:52-91)."""
    f = np.float32
    x = np.array([[0.5, 2.0], [1.25, -3.0], [4.0, 0.75]], dtype=f)        # [3, 2], axis 1: channel 0 = column 0
    col = x[:, 0]
    s = f(0)
    for v in col: s = f(s + v)
    mean = f(s / f(3))
    q = f(0)
    for v in col:
        d = f(v - mean); q = f(q + f(d * d))
    std = f(f(1) / np.sqrt(f(f(q / f(3)) + f(1e-3))))
    out = [f(f(f(f(v - mean) * std) * f(2.0)) + f(0.5)) for v in col]
    r = lambda a: oracle_ops.createRaw(list(np.shape(a)), np.asarray(a, dtype=f).reshape(-1))
    rm, rv = r([1.0, 1.0]), r([2.0, 2.0])
    o, m, sd = oracle_ops.batchNorm(1, 0.1, 1e-3, True).calculateOutput(r(x), rm, rv, r([2.0, 1.0]), r([0.5, 0.0]))
    assert m.toArray()[0] == mean and sd.toArray()[0] == std
    assert o.toArray()[:, 0].tolist() == out
    assert rm.toArray()[0] == f(f(f(0.1) * mean) + f(f(f(1) - f(0.1)) * f(1.0)))
    assert rv.toArray()[0] == f(f(f(0.1) * f(q / f(2))) + f(f(f(1) - f(0.1)) * f(2.0)))


def test_zero_variance_channel_with_zero_epsilon(oracle_ops):
    # JVMBatchNorm.kt:66-68: the reciprocal standard deviation stays 0 when both the sum and epsilon are 0
    r = oracle_ops.createRaw([4, 2], np.array([3, 1, 3, 2, 3, 3, 3, 4], dtype=np.float32))
    out, mean, std = oracle_ops.batchNorm(1, 0.1, 0.0, True).calculateOutput(r, None, None, None, None)
    assert std.toArray()[0] == 0.0 and mean.toArray()[0] == 3.0
    assert not out.toArray()[:, 0].any()
