"""Property tests over random shapes: broadcast binary ops and axis reductions on the
device against the CPU checker (hypothesis, derandomised so every run sees the same
cases). Elementwise results bit-exact; MAX/MIN/ARG bit-exact; SUM/MEAN by the two-clause
tolerance of parity.py."""
import numpy as np
import pytest
from hypothesis import HealthCheck, given, settings, strategies as st

from oracle import jvm_oracle as jo
from parity import assert_bits_equal, assert_reduction_close

pytestmark = pytest.mark.gpu

SETTINGS = dict(max_examples=80, deadline=None, derandomize=True,
                suppress_health_check=[HealthCheck.function_scoped_fixture, HealthCheck.too_slow])

dim = st.sampled_from([1, 2, 3, 4, 5, 7, 8, 12, 16, 33, 64, 100])


@st.composite
def broadcast_pair(draw):
    """A common shape of 1..6 dims and two operand shapes that broadcast to it."""
    common = draw(st.lists(dim, min_size=1, max_size=6).filter(lambda s: int(np.prod(s)) <= 1 << 17))
    def operand():
        keep = draw(st.integers(0, len(common)))             # drop leading dims
        shape = common[len(common) - keep:] if keep else [1]
        return [d if draw(st.booleans()) else 1 for d in shape] or [1]
    a, b = operand(), operand()
    # make sure the pair really produces `common` for the dims it keeps (numpy decides)
    return a, b


@settings(**SETTINGS)
@given(pair=broadcast_pair(), op=st.sampled_from(["plus", "minus", "times", "div"]), seed=st.integers(0, 2 ** 16))
def test_broadcast_binary_matches_checker(pair, op, seed, hip):
    sa, sb = pair
    rng = np.random.default_rng(seed)
    a = rng.standard_normal(sa).astype(np.float32); b = rng.uniform(0.5, 2.0, sb).astype(np.float32)
    with hip.garbageCollector():
        got = hip.createRaw(sa, a)._binary(op, hip.createRaw(sb, b)).toArray()
    want = jo.binary(op, a, b)
    assert_bits_equal(got, want, f"{op} {sa} {sb}")
    assert list(got.shape) == list(np.broadcast_shapes(tuple(sa), tuple(sb)))


@st.composite
def shape_and_axis(draw):
    shape = draw(st.lists(st.sampled_from([1, 2, 3, 5, 8, 17, 64, 65, 100, 256, 1000]), min_size=1, max_size=4)
                 .filter(lambda s: int(np.prod(s)) <= 1 << 18))
    return shape, draw(st.integers(-len(shape), len(shape) - 1))


@settings(**SETTINGS)
@given(sa=shape_and_axis(), op=st.sampled_from(["sum", "mean", "max", "min", "argMax", "argMin"]),
       keep=st.booleans(), seed=st.integers(0, 2 ** 16))
def test_axis_reduction_matches_checker(sa, op, keep, seed, hip):
    shape, axis = sa
    rng = np.random.default_rng(seed)
    x = np.round(rng.standard_normal(shape) * 4).astype(np.float32) / 4          # quarter steps: many ties
    code = {"sum": "sum", "mean": "mean", "max": "max", "min": "min", "argMax": "arg_max", "argMin": "arg_min"}[op]
    a = axis % len(shape)
    with hip.garbageCollector():
        res = getattr(hip.createRaw(shape, x), op)(axis, keep)
        got_shape, got = res.shape, res.toArray().reshape(-1)
    want_shape = list(shape); want_shape[a] = 1
    if not keep and len(shape) > 1:
        del want_shape[a]
    assert got_shape == want_shape
    want = jo.aggregate(code, x, a).reshape(-1)
    if op in ("sum", "mean"):
        ref, _ = jo.axis_sum_f64(x, a)
        assert_reduction_close(got, ref.reshape(-1) / (shape[a] if op == "mean" else 1), want, f"{op} {shape} {axis}")
    else:
        assert_bits_equal(got, want, f"{op} {shape} axis {axis}")


@st.composite
def shape_and_box(draw):
    shape = draw(st.lists(st.sampled_from([1, 2, 3, 4, 5, 8, 12, 17, 64, 100]), min_size=1, max_size=5)
                 .filter(lambda s: int(np.prod(s)) <= 1 << 16))
    k = draw(st.integers(1, len(shape)))
    box = []
    for d in range(k):
        first = draw(st.integers(0, shape[d] - 1))
        box.append((first, draw(st.integers(first, shape[d] - 1))))
    return shape, box


@settings(**SETTINGS)
@given(sb=shape_and_box(), seed=st.integers(0, 2 ** 16))
def test_range_get_set_fill_match_checker(sb, seed, hip):
    shape, box = sb
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(shape).astype(np.float32)
    cpu = jo.JvmOracleOperations()
    with hip.garbageCollector():
        g, c = hip.createRaw(shape, x), cpu.createRaw(shape, x.reshape(-1))
        got, want = g.get(box), c.get(box)
        assert got.shape == want.shape
        assert_bits_equal(got.toArray(), want.toArray(), f"get {shape} {box}")
        v = rng.standard_normal(want.shape).astype(np.float32)
        g.set(box, hip.createRaw(list(v.shape), v)); c.set(box, cpu.createRaw(list(v.shape), v.reshape(-1)))
        assert_bits_equal(g.toArray(), c.toArray(), f"set {shape} {box}")
        g.set(box, 0.25); c.set(box, 0.25)
        assert_bits_equal(g.toArray(), c.toArray(), f"fill {shape} {box}")


@st.composite
def shape_and_permutation(draw):
    shape = draw(st.lists(st.sampled_from([1, 2, 3, 4, 5, 7, 16, 33, 64, 70]), min_size=1, max_size=5)
                 .filter(lambda s: int(np.prod(s)) <= 1 << 17))
    return shape, draw(st.permutations(list(range(len(shape)))))


@settings(**SETTINGS)
@given(sp=shape_and_permutation(), seed=st.integers(0, 2 ** 16))
def test_permute_matches_checker(sp, seed, hip):
    shape, axes = sp
    x = np.random.default_rng(seed).standard_normal(shape).astype(np.float32)
    with hip.garbageCollector():
        got = hip.createRaw(shape, x).permute(list(axes))
        assert got.shape == [shape[a] for a in axes]
        assert_bits_equal(got.toArray(), jo.permute(x, list(axes)), f"permute {shape} {axes}")


@st.composite
def concat_case(draw):
    """A shape of 1..4 dims, an axis, and 1..10 lengths along it (empty inputs among them, at least one value in all)."""
    shape = draw(st.lists(st.sampled_from([1, 2, 3, 4, 5, 7, 8, 16, 33, 64, 257]), min_size=1, max_size=4)
                 .filter(lambda s: int(np.prod(s)) <= 1 << 14))
    axis = draw(st.integers(0, len(shape) - 1))
    lengths = draw(st.lists(st.sampled_from([0, 1, 1, 2, 3, 4, 5, 8, 9, 31]), min_size=1, max_size=10).filter(lambda v: sum(v) > 0))
    return shape, axis, lengths


@settings(**SETTINGS)
@given(case=concat_case(), seed=st.integers(0, 2 ** 16))
def test_concat_matches_numpy_and_the_checker(case, seed, hip):
    """TensorOperations.concat (TensorOperations.kt:41): one launch on the device, a range set per input in the checker
    (AbstractJVMTensorOperations.kt:106-120), numpy's concatenate as the third opinion."""
    shape, axis, lengths = case
    rng = np.random.default_rng(seed)
    parts = []
    for length in lengths:
        sh = list(shape); sh[axis] = length
        parts.append(rng.standard_normal(sh).astype(np.float32))
    want = np.concatenate(parts, axis=axis)
    cpu = jo.JvmOracleOperations()
    if any(p.size == 0 for p in parts):
        # an empty input is an empty range to the reference's range set, which it rejects: the same error on both sides
        with pytest.raises(ValueError) as on_checker:
            cpu.concat(axis, [cpu.createRaw(list(p.shape), p.reshape(-1)) for p in parts])
        with hip.garbageCollector(), pytest.raises(ValueError) as on_device:
            hip.concat(axis, [hip.createRaw(list(p.shape), p) for p in parts])
        assert str(on_device.value) == str(on_checker.value)
        return
    checker = cpu.concat(axis, [cpu.createRaw(list(p.shape), p.reshape(-1)) for p in parts])
    with hip.garbageCollector():
        got = hip.concat(axis - len(shape) if seed % 2 else axis, [hip.createRaw(list(p.shape), p) for p in parts])
        assert got.shape == list(want.shape) == checker.shape
        assert_bits_equal(got.toArray(), want, f"concat {shape} axis {axis} lengths {lengths}")
        assert_bits_equal(checker.toArray(), want, f"checker's concat {shape} axis {axis} lengths {lengths}")


@st.composite
def batch_norm_case(draw):
    shape = draw(st.lists(st.sampled_from([1, 2, 3, 4, 5, 8, 17, 64, 70, 130]), min_size=2, max_size=4)
                 .filter(lambda s: 2 <= int(np.prod(s)) <= 1 << 16))
    axis = draw(st.integers(0, len(shape) - 1))
    if int(np.prod(shape)) // shape[axis] < 2:          # the unbiased variance needs two values per channel
        axis = int(np.argmin(shape))
    return shape, axis, draw(st.booleans()), draw(st.booleans())


@settings(**SETTINGS)
@given(case=batch_norm_case(), seed=st.integers(0, 2 ** 16))
def test_batch_norm_elementwise_halves_match_checker(case, seed, hip):
    """Output and input gradient bit for bit from the device's own per-channel statistics;
    the statistics themselves close to float64."""
    shape, axis, affine, training = case
    if int(np.prod(shape)) // shape[axis] < 2:
        return
    rng = np.random.default_rng(seed)
    c = shape[axis]
    x = rng.standard_normal(shape).astype(np.float32) * np.float32(2) + np.float32(0.5)
    go = rng.standard_normal(shape).astype(np.float32)
    gamma = rng.standard_normal(c).astype(np.float32) if affine else None
    beta = rng.standard_normal(c).astype(np.float32) if affine else None
    rm, rv = rng.standard_normal(c).astype(np.float32), np.abs(rng.standard_normal(c)).astype(np.float32) + np.float32(0.1)
    raw = lambda a: None if a is None else hip.createRaw(list(a.shape), a)
    red = tuple(d for d in range(len(shape)) if d != axis)
    bshape = [1] * len(shape); bshape[axis] = c
    with hip.garbageCollector():
        op = hip.batchNorm(axis, 0.1, 1e-3, training)
        gx, ggo, gg, gb, grm, grv = raw(x), raw(go), raw(gamma), raw(beta), raw(rm), raw(rv)
        out, mean, std = op.calculateOutput(gx, grm, grv, gg, gb)
        if training:
            m, s = mean.toArray(), std.toArray()
            x64 = x.astype(np.float64)
            assert np.abs(m - x64.mean(red)).max() <= 1e-5 * max(np.abs(x64.mean(red)).max(), 1.0)
            var = ((x64 - m.astype(np.float64).reshape(bshape)) ** 2).mean(red)
            assert np.allclose(s, 1.0 / np.sqrt(var + 1e-3), rtol=1e-5)
        else:
            m, s = rm, (np.float32(1.0) / np.sqrt(rv + np.float32(1e-3))).astype(np.float32)
        assert_bits_equal(out.toArray(), jo.batch_norm_apply(x, axis, m, s, gamma, beta), f"output {shape} axis {axis}")
        gin, ggam, gbet = op.calculateGrads(gx, grm, grv, mean, std, gg, ggo, True, affine, affine)
        if not training:
            s = (1.0 / np.sqrt((rv + np.float32(1e-3)).astype(np.float64))).astype(np.float32)     # JVMBatchNorm.kt:136
        sums = go.astype(np.float64).sum(red).astype(np.float32)
        dots = ((x.astype(np.float64) - m.astype(np.float64).reshape(bshape)) * go).sum(red).astype(np.float32)
        assert_bits_equal(gin.toArray(), jo.batch_norm_grad_in(x, axis, training, m, s, gamma, go, sums, dots),
                          f"gradIn {shape} axis {axis}")
