"""Fused batch normalisation on the device: the reference's own tests, parity with the CPU
checker (statistics to the reduction bar against float64; the elementwise halves bit-exact
from the device's own statistics), every data layout the kernels distinguish, determinism
and error behaviour."""
import numpy as np
import pytest

import batchnorm_cases as bnc
from kten_amd.host_mirror.inputs import SplitMix64
from oracle import jvm_oracle as jo
from parity import assert_bits_equal, assert_reduction_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,case", bnc.CASES, ids=[n for n, _ in bnc.CASES])
def test_reference_batch_norm_tests(name, case, gc):
    case(gc)


def make(ops, arrays):
    return {k: (None if v is None else ops.createRaw(list(v.shape), v.reshape(-1) if ops.platformKey.startswith("JVM") else v))
            for k, v in arrays.items()}


def inputs_for(shape, axis, seed, affine, running):
    gen = SplitMix64(seed)
    c = shape[axis]
    return {"x": gen.normal(shape) * np.float32(1.7) + np.float32(0.3), "go": gen.normal(shape),
            "gamma": gen.normal([c]) if affine else None, "beta": gen.normal([c]) if affine else None,
            "rm": gen.normal([c]) if running else None, "rv": np.abs(gen.normal([c])) if running else None}


def channel_sums64(a, axis):
    red = tuple(d for d in range(a.ndim) if d != axis)
    return a.astype(np.float64).sum(red)


# (shape, axis): long runs with float4 loads, long runs with scalar loads, short runs, channel-last, one channel,
# more channels than workgroup columns, a single row
LAYOUTS = [([10, 3, 4, 5], 1), ([8, 16, 32, 32], 1), ([4, 6, 67], 1), ([4, 5, 257], 1), ([64, 33, 7], 1), ([512, 40], 1),
           ([300, 129], 1), ([40, 512], 0), ([3, 2000], 0), ([2, 3, 4, 5], 3), ([6, 1, 300], 1), ([1, 8, 4096], 1),
           ([9, 4, 1024], 1), ([10, 3, 4, 5], 2),
           # runs whose length is 1, 2, 3 past a multiple of 4 (the last unit overlaps its neighbour), channels innermost
           # with a multiple of 4 channels (parameters read four channels at a time)
           ([20, 12, 13, 13], 1), ([7, 8, 65], 1), ([5, 4, 66], 1), ([3, 5, 71], 1), ([1000, 256], 1), ([33, 4, 7, 12], 3),
           # a matrix of 16, 6, 48 and 3 columns under many rows (the workgroup's threads over several rows at a time), and
           # 20 000 channels of 3 and 12 items (a thread per channel folds them)
           ([30000, 16], 1), ([5000, 2, 3], 1), ([7000, 48], 1), ([9001, 3], 1), ([3, 20000], 1), ([20000, 12], 0),
           # at most 32 items per channel and 16 384 channels or more: no statistics launch, the finalize sums the items
           # (32 items: the last such shape; 33: the statistics launch again; items of an inner dim under an outer one)
           ([32, 16384], 1), ([33, 16384], 1), ([2, 17000, 3], 1), ([5, 16390], 1), ([16385, 2], 0),
           # long runs, where the apply kernels do the finalize step themselves: the shortest run that qualifies (171
           # float4s: a workgroup's tile touches up to four runs, and tiles cross from one outer index to the next), the
           # longest that does not, one channel, and so few channels that their partials are too many to fold per workgroup
           ([5, 7, 684], 1), ([3, 5, 680], 1), ([6, 1, 2048], 1), ([256, 2, 64, 64], 1), ([64, 3, 56, 56], 1)]


@pytest.mark.parametrize("affine,running", [(True, True), (False, False)])
@pytest.mark.parametrize("shape,axis", LAYOUTS, ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else f"axis{v}")
def test_training_mode_parity(shape, axis, affine, running, gc):
    check_training_mode(shape, axis, affine, running, sum(shape) * 7 + axis, gc)


def check_training_mode(shape, axis, affine, running, seed, gc):
    eps, momentum = 1e-3, 0.1
    arrays = inputs_for(shape, axis, seed, affine, running)
    cpu = jo.JvmOracleOperations()
    g, c = make(gc, arrays), make(cpu, arrays)
    gop, cop = gc.batchNorm(axis, momentum, eps, True), cpu.batchNorm(axis, momentum, eps, True)
    gout, gmean, gstd = gop.calculateOutput(g["x"], g["rm"], g["rv"], g["gamma"], g["beta"])
    cout, cmean, cstd = cop.calculateOutput(c["x"], c["rm"], c["rv"], c["gamma"], c["beta"])
    x64 = arrays["x"].astype(np.float64)
    n = arrays["x"].size // shape[axis]
    bshape = [1] * len(shape); bshape[axis] = shape[axis]
    mean64 = channel_sums64(arrays["x"], axis) / n
    assert_reduction_close(gmean.toArray(), mean64, cmean.toArray(), "currentMean")
    # the reciprocal standard deviation, against float64 from the device's own rounded mean
    dev_mean = gmean.toArray().astype(np.float64).reshape(bshape)
    ssd64 = channel_sums64((x64 - dev_mean) ** 2, axis)
    std64 = 1.0 / np.sqrt(ssd64 / n + eps)
    jvm_mean = cmean.toArray().astype(np.float64).reshape(bshape)
    jvm_std64 = 1.0 / np.sqrt(channel_sums64((x64 - jvm_mean) ** 2, axis) / n + eps)
    err = np.abs(gstd.toArray() - std64)
    assert np.all((err <= 1e-5 * std64) | (err <= np.abs(cstd.toArray() - jvm_std64))), "currentStd"
    # the elementwise half, bit for bit from the device's own statistics
    assert_bits_equal(gout.toArray(), jo.batch_norm_apply(arrays["x"], axis, gmean.toArray(), gstd.toArray(),
                                                          arrays["gamma"], arrays["beta"]), "output")
    if running:
        # against float64, or no further from it than the checker's serial float sums are (a quarter of a million items
        # per channel and more leave those beyond 1e-5)
        for key, stat64 in (("rm", mean64), ("rv", ssd64 / (n - 1))):
            want64 = momentum * stat64 + (1.0 - momentum) * arrays[key].astype(np.float64)
            err = np.abs(g[key].toArray() - want64)
            assert np.all((err <= 1e-5 * np.abs(want64) + 1e-6) | (err <= np.abs(c[key].toArray() - want64))), key
        f = np.float32
        want_rm = (f(momentum) * gmean.toArray() + (f(1) - f(momentum)) * arrays["rm"]).astype(f)
        assert_bits_equal(g["rm"].toArray(), want_rm, "running mean from the device's mean, in the reference's float order")

    ggin, ggg, ggb = gop.calculateGrads(g["x"], g["rm"], g["rv"], gmean, gstd, g["gamma"], g["go"], True, affine, affine)
    cgin, cgg, cgb = cop.calculateGrads(c["x"], c["rm"], c["rv"], cmean, cstd, c["gamma"], c["go"], True, affine, affine)
    go64 = arrays["go"].astype(np.float64)
    sum64 = channel_sums64(arrays["go"], axis)
    dot64 = channel_sums64((x64 - dev_mean) * go64, axis)
    if affine:
        assert_reduction_close(ggb.toArray(), sum64, cgb.toArray(), "gradBeta")
        jvm_dot64 = channel_sums64((x64 - jvm_mean) * go64, axis)
        err = np.abs(ggg.toArray() - dot64 * gstd.toArray())
        jerr = np.abs(cgg.toArray() - jvm_dot64 * cstd.toArray())
        assert np.all((err <= 1e-5 * np.abs(dot64 * gstd.toArray())) | (err <= jerr) | (err <= 1e-6)), "gradGamma"
    want_gin = jo.batch_norm_grad_in(arrays["x"], axis, True, gmean.toArray(), gstd.toArray(), arrays["gamma"], arrays["go"],
                                     sum64.astype(np.float32), dot64.astype(np.float32))
    assert_bits_equal(ggin.toArray(), want_gin, "gradIn from the device's statistics and the correctly rounded sums")
    # end to end: against the checker, or no further from a float64 evaluation than the checker is (its serial float sums
    # over a quarter of a million items per channel and more are the less accurate ones)
    scale = np.abs(cgin.toArray()).max()
    mean_b = mean64.reshape(bshape)
    std_b = (1.0 / np.sqrt(channel_sums64((x64 - mean_b) ** 2, axis) / n + eps)).reshape(bshape)
    gamma_b = arrays["gamma"].astype(np.float64).reshape(bshape) if affine else 1.0
    dot_b = channel_sums64((x64 - mean_b) * go64, axis).reshape(bshape)
    gin64 = (go64 - sum64.reshape(bshape) / n - (x64 - mean_b) * dot_b * std_b * std_b / n) * std_b * gamma_b
    err = np.abs(ggin.toArray() - cgin.toArray()).max()
    assert err <= 2e-5 * scale or np.abs(ggin.toArray() - gin64).max() <= np.abs(cgin.toArray() - gin64).max(), \
        "gradIn against the checker end to end"


def long_run_layout(seed):
    """A random layout whose runs are long enough for the apply kernels to do the finalize step themselves (a multiple
    of 4 floats, 684 or more), or just not (every fourth seed): one or two dims inside the axis, up to two outside."""
    rng = np.random.default_rng(9000 + seed)
    run = int(rng.integers(171, 1200)) * 4
    if seed % 4 == 3:
        run = int(rng.integers(100, 171)) * 4 + int(rng.integers(0, 2)) * int(rng.integers(1, 4))
    channels = int(rng.choice([1, 2, 3, 7, 16, 33, 130]))
    outer = [int(rng.integers(1, 7)) for _ in range(int(rng.integers(0, 3)))]
    inner = [run]
    if run % 8 == 0 and rng.random() < 0.5:
        inner = [2, run // 2] if rng.random() < 0.5 else [run // 4, 4]
    while int(np.prod(outer + [channels] + inner)) > 3_000_000 and outer:
        outer.pop()
    if int(np.prod(outer, dtype=np.int64)) * run < 2:
        outer = [2] + outer
    return outer + [channels] + inner, len(outer)


@pytest.mark.parametrize("seed", range(16))
def test_random_layouts_with_long_runs(seed, gc):
    shape, axis = long_run_layout(seed)
    check_training_mode(shape, axis, seed % 2 == 0, seed % 3 != 0, 31 * seed + 5, gc)
    check_inference_mode(shape, axis, 77 * seed + 1, gc)


@pytest.mark.parametrize("shape,axis", [([10, 3, 4, 5], 2), ([8, 16, 32, 32], 1), ([512, 40], 1), ([4, 6, 67], 1), ([3, 20000], 1), ([17000, 2, 2], 0)],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else f"axis{v}")
def test_inference_mode_is_bit_exact(shape, axis, gc):
    check_inference_mode(shape, axis, sum(shape) + 100 * axis, gc)


def check_inference_mode(shape, axis, seed, gc):
    """No reduction feeds the inference output or input gradient, so they match the checker
    bit for bit; gradGamma / gradBeta are sums and go through the reduction bar."""
    eps = 1e-3
    arrays = inputs_for(shape, axis, seed, True, True)
    cpu = jo.JvmOracleOperations()
    g, c = make(gc, arrays), make(cpu, arrays)
    gop, cop = gc.batchNorm(axis, 0.1, eps, False), cpu.batchNorm(axis, 0.1, eps, False)
    gout, gmean, gstd = gop.calculateOutput(g["x"], g["rm"], g["rv"], g["gamma"], g["beta"])
    cout, cmean, cstd = cop.calculateOutput(c["x"], c["rm"], c["rv"], c["gamma"], c["beta"])
    assert_bits_equal(gout.toArray(), cout.toArray(), "output")
    assert_bits_equal(gmean.toArray(), cmean.toArray(), "currentMean stays zero")
    assert_bits_equal(gstd.toArray(), cstd.toArray(), "currentStd stays zero")
    assert_bits_equal(g["rm"].toArray(), arrays["rm"], "running mean untouched")
    assert_bits_equal(g["rv"].toArray(), arrays["rv"], "running var untouched")
    ggin, ggg, ggb = gop.calculateGrads(g["x"], g["rm"], g["rv"], gmean, gstd, g["gamma"], g["go"], True, True, True)
    cgin, cgg, cgb = cop.calculateGrads(c["x"], c["rm"], c["rv"], cmean, cstd, c["gamma"], c["go"], True, True, True)
    assert_bits_equal(ggin.toArray(), cgin.toArray(), "gradIn")
    assert_reduction_close(ggb.toArray(), channel_sums64(arrays["go"], axis), cgb.toArray(), "gradBeta")
    bshape = [1] * len(shape); bshape[axis] = shape[axis]
    std = (1.0 / np.sqrt((arrays["rv"] + np.float32(eps)).astype(np.float64))).astype(np.float32)
    dot64 = channel_sums64((arrays["x"].astype(np.float64) - arrays["rm"].reshape(bshape)) * arrays["go"], axis)
    assert_reduction_close(ggg.toArray(), dot64 * std, cgg.toArray(), "gradGamma")
    only_in, none_g, none_b = gop.calculateGrads(g["x"], g["rm"], g["rv"], gmean, gstd, g["gamma"], g["go"], True, False, False)
    assert none_g is None and none_b is None
    assert_bits_equal(only_in.toArray(), cgin.toArray(), "gradIn alone (no statistics pass)")


@pytest.mark.parametrize("shape,folded", [([8, 16, 32, 32], True), ([5, 7, 684], True), ([3, 5, 680], False), ([256, 2, 64, 64], False),
                                          ([512, 40], False)], ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_long_runs_take_two_launches_per_pass(shape, folded, gc):
    """Which launches a forward and a backward pass make: statistics + apply where the apply kernel can do the
    per-channel arithmetic itself, statistics + finalize + apply otherwise (the parity of both forms is held by the
    tests above, whose layouts cover both)."""
    arrays = inputs_for(shape, 1, 11, True, True)
    g = make(gc, arrays)
    op = gc.batchNorm(1, 0.1, 1e-3, True)
    gc.profileBegin()
    out, mean, std = op.calculateOutput(g["x"], g["rm"], g["rv"], g["gamma"], g["beta"])
    op.calculateGrads(g["x"], g["rm"], g["rv"], mean, std, g["gamma"], g["go"], True, True, True)
    launched = gc.profileEnd()
    names = " ".join(launched)
    assert sum(v[0] for k, v in launched.items() if k.startswith("bn_")) == (4 if folded else 6), names
    assert ("bn_apply_folded_kernel" in names) == folded and ("bn_finalize" in names) != folded, names
    # only gradGamma and gradBeta wanted: no apply kernel to ride in, the finalize launch stays
    gc.profileBegin()
    op.calculateGrads(g["x"], g["rm"], g["rv"], mean, std, g["gamma"], g["go"], False, True, True)
    names = " ".join(gc.profileEnd())
    assert "bn_finalize_backward_kernel" in names and "bn_apply" not in names, names


def test_batch_norm_is_deterministic_and_handles_degenerate_channels(gc):
    arrays = inputs_for([32, 24, 28, 28], 1, 5, True, False)
    arrays["x"][:, 3] = 2.5                                   # a constant channel
    g = make(gc, arrays)
    op = gc.batchNorm(1, 0.1, 0.0, True)                      # epsilon 0: the constant channel's 1/std stays 0
    first = [t.toArray() for t in op.calculateOutput(g["x"], None, None, g["gamma"], g["beta"])]
    again = [t.toArray() for t in op.calculateOutput(g["x"], None, None, g["gamma"], g["beta"])]
    for a, b, name in zip(first, again, ("output", "currentMean", "currentStd")):
        assert_bits_equal(a, b, f"{name} on a second run")
    assert first[1][3] == np.float32(2.5) and first[2][3] == 0.0
    assert_bits_equal(first[0][:, 3], np.full([32, 28, 28], arrays["beta"][3], dtype=np.float32), "constant channel -> beta")


def test_batch_norm_argument_errors(gc):
    x = gc.createRaw([4, 3, 8], np.zeros(96, dtype=np.float32))
    three, two = gc.createRaw([3], [1.0, 1.0, 1.0]), gc.createRaw([2], [1.0, 1.0])
    with pytest.raises(ValueError):
        gc.batchNorm(1, 0.1, 1e-3, False).calculateOutput(x, None, None, None, None)          # inference needs running statistics
    with pytest.raises(ValueError):
        gc.batchNorm(1, 0.1, 1e-3, True).calculateOutput(x, three, None, None, None)          # both or neither
    with pytest.raises(ValueError):
        gc.batchNorm(1, 0.1, 1e-3, True).calculateOutput(x, None, None, two, None)            # gamma too short
    with pytest.raises(ValueError):
        gc.batchNorm(3, 0.1, 1e-3, True).calculateOutput(x, None, None, None, None)           # axis out of range
    t = gc.create([4, 3, 8], True, np.zeros([4, 3, 8], dtype=np.float32))
    with pytest.raises(ValueError):
        t.batchNorm(1, None, None, False)
    with pytest.raises(ValueError):
        t.batchNorm(1, gc.create([3], True, np.zeros(3, dtype=np.float32)), gc.create([3], False, np.ones(3, dtype=np.float32)), True)


def test_batch_norm_workload_at_benchmark_size(gc):
    """NCHW [64,128,56,56], training forward + backward: statistics against float64, the two
    elementwise halves bit for bit from the device's statistics, and what batch normalisation
    guarantees of its own output (per-channel mean beta, variance gamma^2 var / (var + eps))."""
    from kten_amd.host_mirror.workloads import WORKLOADS
    wl = WORKLOADS["batch_norm"]
    inp = wl.make_inputs(wl.full_dims)
    out = {k: v.toArray() for k, v in wl.run(gc, inp).items()}
    x64 = inp["x"].astype(np.float64)
    n = inp["x"].size // 128
    mean64 = x64.sum((0, 2, 3)) / n
    assert np.abs(out["mean"] - mean64).max() <= 1e-5 * np.abs(mean64).max()
    dev_mean = out["mean"].astype(np.float64).reshape(1, 128, 1, 1)
    var64 = ((x64 - dev_mean) ** 2).sum((0, 2, 3)) / n
    std64 = 1.0 / np.sqrt(var64 + 1e-5)
    assert np.abs(out["std"] - std64).max() <= 1e-5 * std64.max()
    assert_bits_equal(out["out"], jo.batch_norm_apply(inp["x"], 1, out["mean"], out["std"], inp["gamma"], inp["beta"]), "output")
    o64 = out["out"].astype(np.float64)
    assert np.abs(o64.mean((0, 2, 3)) - inp["beta"]).max() <= 1e-5
    assert np.allclose(o64.var((0, 2, 3)), inp["gamma"].astype(np.float64) ** 2 * var64 / (var64 + 1e-5), rtol=1e-5)
    go64 = inp["grad_out"].astype(np.float64)
    sum64, dot64 = go64.sum((0, 2, 3)), ((x64 - dev_mean) * go64).sum((0, 2, 3))
    assert np.abs(out["grad_beta"] - sum64).max() <= 1e-5 * np.abs(sum64).max()
    assert np.abs(out["grad_gamma"] - dot64 * out["std"]).max() <= 1e-5 * np.abs(dot64 * out["std"]).max()
    want = jo.batch_norm_grad_in(inp["x"], 1, True, out["mean"], out["std"], inp["gamma"], inp["grad_out"],
                                 sum64.astype(np.float32), dot64.astype(np.float32))
    assert_bits_equal(out["grad_in"], want, "gradIn")
    # the input gradient of batch normalisation sums to zero per channel and is orthogonal to x - mean
    gi64 = out["grad_in"].astype(np.float64)
    # (to float rounding of the 200 704 terms of a channel: a few 1e-7 of their absolute sum)
    assert np.all(np.abs(gi64.sum((0, 2, 3))) <= 1e-6 * np.abs(gi64).sum((0, 2, 3)))
    assert np.all(np.abs((gi64 * (x64 - dev_mean)).sum((0, 2, 3))) <= 1e-6 * np.abs(gi64 * (x64 - dev_mean)).sum((0, 2, 3)))
