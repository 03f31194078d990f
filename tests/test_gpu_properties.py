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
