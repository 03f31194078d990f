"""Pins the CPU checker where the reference's own tests leave it open: against what the
mathematics fixes (IEEE-754 single rounding, numpy broadcasting, exact rational
arithmetic, brute force on tiny inputs) and against the documented java.lang.Math /
kotlin.math special cases. Chosen so that a plausible slip (wrong sign, wrong index,
transposed operand, fused multiply-add, wrong tie rule) fails at least one check.
No GPU involved.
"""
import itertools
import math
from fractions import Fraction

import numpy as np
import pytest

from oracle import jvm_oracle as jo

RNG = np.random.default_rng(1234)


def bits(a):
    return np.asarray(a, dtype=np.float32).view(np.uint32)


def ulp_distance(a, b):
    """Distance in units of fp32 spacing; NaN vs NaN counts as 0."""
    a = np.asarray(a, dtype=np.float32); b = np.asarray(b, dtype=np.float32)
    ia = a.view(np.int32).astype(np.int64); ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7fffffff), ia); ib = np.where(ib < 0, -(ib & 0x7fffffff), ib)
    d = np.abs(ia - ib)
    return np.where(np.isnan(a) & np.isnan(b), 0, d)


def assert_bits_equal(got, want):
    got = np.asarray(got, dtype=np.float32); want = np.asarray(want, dtype=np.float32)
    same = (bits(got) == bits(want)) | (np.isnan(got) & np.isnan(want))
    assert same.all(), f"{np.count_nonzero(~same)} mismatches, first at {np.argwhere(~same)[0]}"


def sample_floats(n):
    """Normals, wide-exponent values, denormals and specials."""
    a = RNG.standard_normal(n).astype(np.float32)
    b = (RNG.standard_normal(n) * np.exp(RNG.uniform(-40, 40, n))).astype(np.float32)
    c = RNG.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32)   # any bit pattern
    special = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.17549435e-38,
                        3.4028235e38, -3.4028235e38, 0.5, -0.5, 2.5, -2.5, 8388607.5, 8388608.0], dtype=np.float32)
    return np.concatenate([a, b, c, special])


# ------------------------------------------------------------------ broadcast index map

SHAPE_PAIRS = [
    ([2, 4], [2, 1]), ([3, 3], [3]), ([3, 3], [1]), ([3, 1], [1, 3]), ([1, 3], [3, 3]), ([2, 3, 4], [3, 1]),
    ([2, 1, 4], [3, 1]), ([5], [2, 3, 5]), ([2, 3, 4, 5], [1, 3, 1, 1]), ([1], [1]), ([4, 1, 2, 1], [1, 3, 1, 5]),
    ([2, 3], [2, 3]), ([1, 1, 1], [2, 3, 4]), ([7], [1]),
]


@pytest.mark.parametrize("sa,sb", SHAPE_PAIRS)
def test_binary_broadcast_matches_numpy(sa, sb):
    a = RNG.standard_normal(sa).astype(np.float32)
    b = RNG.standard_normal(sb).astype(np.float32)
    for op, f in (("plus", np.add), ("minus", np.subtract), ("times", np.multiply), ("div", np.divide)):
        got = jo.binary(op, a, b)
        want = f(a, b)
        assert list(got.shape) == list(want.shape)
        assert_bits_equal(got, want)


def test_broadcast_to_brute_force():
    # Nested loops over the target index with size-1 source dims pinned to 0.
    for src_shape, dst_shape in [([3, 1], [2, 3, 4]), ([1], [2, 2]), ([1, 4], [3, 4]), ([2, 1, 1], [2, 3, 2]), ([4], [4])]:
        src = RNG.standard_normal(src_shape).astype(np.float32)
        got = jo.broadcast_to(src, dst_shape)
        padded = [1] * (len(dst_shape) - len(src_shape)) + src_shape
        srcp = src.reshape(padded)
        for idx in itertools.product(*[range(d) for d in dst_shape]):
            sidx = tuple(0 if padded[k] == 1 else idx[k] for k in range(len(idx)))
            assert got[idx] == srcp[sidx]


@pytest.mark.parametrize("sa,sb", [([3], [4]), ([2, 3], [3, 2]), ([2, 3], [4, 1, 2])])
def test_invalid_broadcast_raises(sa, sb):
    with pytest.raises(ValueError):
        jo.binary("plus", np.zeros(sa, np.float32), np.zeros(sb, np.float32))


def test_broadcast_to_rejects_shrinking():
    with pytest.raises(ValueError):
        jo.broadcast_to(np.zeros([2, 3], np.float32), [3])
    with pytest.raises(ValueError):
        jo.broadcast_to(np.zeros([2, 3], np.float32), [2, 1])


# ------------------------------------------------------------------ single-rounding IEEE ops

def test_ieee_binary_ops_bit_exact_including_specials():
    x = sample_floats(20000); y = RNG.permutation(sample_floats(20000))
    with np.errstate(all="ignore"):
        assert_bits_equal(jo.binary("plus", x, y), x + y)
        assert_bits_equal(jo.binary("minus", x, y), x - y)
        assert_bits_equal(jo.binary("times", x, y), x * y)
        assert_bits_equal(jo.binary("div", x, y), x / y)


def test_no_fused_multiply_add():
    # a*b = 1 + 2^-11 + 2^-24 is not representable: times rounds it, then plus adds c.
    # A fused a*b+c keeps the 2^-24 and gives a different float.
    a = np.float32(1.0 + 2 ** -12); b = np.float32(1.0 + 2 ** -12); c = np.float32(-1.0)
    prod = jo.binary("times", [a], [b])
    two_roundings = jo.binary("plus", prod, [c])
    assert two_roundings[0] == np.float32(np.float32(a * b) + c)
    fused = np.float32(float(a) * float(b) + float(c))
    assert two_roundings[0] != fused           # the case really does discriminate


def test_scalar_ops_and_reverse_pow():
    x = sample_floats(5000)
    with np.errstate(all="ignore"):
        for c in (2.0, -0.75, 1e-3, 0.0):
            cf = np.float32(c)
            assert_bits_equal(jo.scalar("plus", x, c), x + cf)
            assert_bits_equal(jo.scalar("minus", x, c), x - cf)
            assert_bits_equal(jo.scalar("times", x, c), x * cf)
            assert_bits_equal(jo.scalar("div", x, c), x / cf)
    small = RNG.uniform(-4, 4, 2000).astype(np.float32)
    want = np.power(np.float64(2.0), small.astype(np.float64)).astype(np.float32)
    assert ulp_distance(jo.scalar("pow", small, 2.0, reverse=True), want).max() <= 1


def test_exact_unary_ops():
    x = sample_floats(20000)
    with np.errstate(all="ignore"):
        assert_bits_equal(jo.unary("neg", x), -x)
        assert_bits_equal(jo.unary("abs", x), np.abs(x))
        assert_bits_equal(jo.unary("reciprocal", x), np.float32(1.0) / x)
        assert_bits_equal(jo.unary("sqrt", x), np.sqrt(x))
        assert_bits_equal(jo.unary("rsqrt", x), np.float32(1.0) / np.sqrt(x))      # two roundings
        assert_bits_equal(jo.unary("floor", x), np.floor(x))
        assert_bits_equal(jo.unary("ceil", x), np.ceil(x))
        assert_bits_equal(jo.unary("trunc", x), np.trunc(x))
        assert_bits_equal(jo.unary("sign", x), np.where(np.isnan(x), x, np.where(x == 0, x, np.sign(x))))


def test_trunc_and_sign_signed_zero():
    got = jo.unary("trunc", [-0.3, 0.3, -0.0, 0.0, -1.7])
    assert list(bits(got)) == list(bits(np.array([-0.0, 0.0, -0.0, 0.0, -1.0], np.float32)))
    got = jo.unary("sign", [-0.0, 0.0, -0.4, 7.0])
    assert list(bits(got)) == list(bits(np.array([-0.0, 0.0, -1.0, 1.0], np.float32)))
    assert np.isnan(jo.unary("sign", [np.nan])[0])


def test_round_is_floor_of_x_plus_half_exactly():
    # Exact rational arithmetic: Math.round(float) = floor(x + 1/2), saturating at the int range.
    xs = np.concatenate([RNG.uniform(-1000, 1000, 3000), RNG.uniform(-3, 3, 3000),
                         np.arange(-6, 6, 0.5), [0.49999997, -0.49999997, 8388607.5, -8388607.5,
                                                  2147483520.0, 3e9, -3e9, 1e20, -1e20]]).astype(np.float32)
    got = jo.unary("round", xs)
    for x, g in zip(xs.tolist(), got.tolist()):
        want = math.floor(Fraction(x) + Fraction(1, 2))
        want = max(-2 ** 31, min(2 ** 31 - 1, want))
        assert g == float(np.float32(want)), (x, g, want)
    specials = jo.unary("round", [np.nan, np.inf, -np.inf, -0.5, -0.0, 2.5, -2.5])
    assert list(bits(specials)) == list(bits(np.array([0.0, 2147483648.0, -2147483648.0, 0.0, 0.0, 3.0, -2.0], np.float32)))


def test_sigmoid_is_the_reference_composition():
    x = RNG.uniform(-30, 30, 5000).astype(np.float32)
    e = np.exp((np.float32(-1.0) * x).astype(np.float64)).astype(np.float32)
    want = np.float32(1.0) / (np.float32(1.0) + e)
    assert ulp_distance(jo.unary("sigmoid", x), want).max() <= 1     # libm exp last-bit only
    assert jo.unary("sigmoid", [0.0])[0] == 0.5


def test_clamp_java_min_max_rules():
    got = jo.clamp([np.nan, -5.0, 0.3, 9.0, -0.0, 0.0], -1.0, 1.0)
    assert np.isnan(got[0]) and list(got[1:4]) == [-1.0, np.float32(0.3), 1.0]
    z = jo.clamp([-0.0, 0.0], 0.0, 5.0)          # max(-0, +0) = +0
    assert list(bits(z)) == [0, 0]
    z = jo.clamp([0.0, -0.0], -5.0, -0.0)        # min(+0, -0) = -0
    assert list(bits(z)) == [0x80000000, 0x80000000]


# ------------------------------------------------------------------ f64-libm-then-round ops

F64 = {"exp": np.exp, "log": np.log, "tanh": np.tanh, "sinh": np.sinh, "cosh": np.cosh, "sin": np.sin,
       "cos": np.cos, "tan": np.tan, "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan}


@pytest.mark.parametrize("op", sorted(F64))
def test_transcendental_is_f64_libm_rounded_once(op):
    x = np.concatenate([RNG.standard_normal(20000) * 3, RNG.uniform(-1, 1, 5000), RNG.uniform(-90, 90, 5000),
                        [0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 89.0, -104.0, 1e-40]]).astype(np.float32)
    with np.errstate(all="ignore"):
        want = F64[op](x.astype(np.float64)).astype(np.float32)
    got = jo.unary(op, x)
    # numpy's f64 routines and glibc's may differ in the last f64 bit, which survives the
    # rounding to fp32 only on rare ties: allow 1 ulp, demand exactness almost everywhere.
    d = ulp_distance(got, want)
    assert d.max() <= 1
    assert np.count_nonzero(d) <= len(x) // 1000


def test_transcendental_specials():
    assert jo.unary("log", [0.0])[0] == -np.inf and np.isnan(jo.unary("log", [-1.0])[0])
    assert jo.unary("exp", [89.0])[0] == np.inf and jo.unary("exp", [-np.inf])[0] == 0.0
    assert jo.unary("exp", [0.0])[0] == 1.0 and jo.unary("log", [1.0])[0] == 0.0
    assert jo.unary("log", [np.float32(math.e)])[0] == np.float32(math.log(float(np.float32(math.e))))


def test_pow_special_cases_follow_java_not_c99():
    nan, inf = np.nan, np.inf
    a = np.array([1.0, -1.0, 1.0, nan, 5.0, -8.0, 2.0, 0.0, -0.0, 2.0, -2.0], np.float32)
    b = np.array([nan, inf, -inf, 0.0, 0.0, 1 / 3, 10.0, -1.0, -1.0, -inf, 3.0], np.float32)
    got = jo.binary("pow", a, b)
    assert np.isnan(got[0]) and np.isnan(got[1]) and np.isnan(got[2])       # Java: NaN (C99 says 1)
    assert got[3] == 1.0 and got[4] == 1.0                                   # anything ** 0 = 1
    assert np.isnan(got[5])                                                  # negative base, fractional exponent
    assert got[6] == 1024.0 and got[7] == inf and got[8] == -inf and got[9] == 0.0 and got[10] == -8.0


def test_pow_exact_exponents():
    x = sample_floats(20000)
    with np.errstate(all="ignore"):
        assert_bits_equal(jo.scalar("pow", x, 2.0), x * x)      # exact product fits f64, so pow(x,2) rounds like x*x
        assert_bits_equal(jo.scalar("pow", x, 1.0), x)
        ones = jo.scalar("pow", x, 0.0)
    assert (ones == 1.0).all()
    y = RNG.uniform(0.01, 50, 5000).astype(np.float32)
    want = np.power(y.astype(np.float64), np.float64(np.float32(-0.5))).astype(np.float32)
    assert ulp_distance(jo.scalar("pow", y, -0.5), want).max() <= 1


# ------------------------------------------------------------------ comparisons

def test_comparisons_and_epsilon():
    a = np.array([1.0, 2.0, 3.0, np.nan, 1.0, 1.0], np.float32)
    b = np.array([2.0, 2.0, 1.0, 1.0, np.float32(1.0 + 5e-8), np.float32(1.0 + 2.4e-7)], np.float32)
    assert list(jo.binary("lt", a, b)) == [1, 0, 0, 0, 0, 1]
    assert list(jo.binary("lte", a, b)) == [1, 1, 0, 0, 1, 1]
    assert list(jo.binary("gt", a, b)) == [0, 0, 1, 0, 0, 0]
    assert list(jo.binary("gte", a, b)) == [0, 1, 1, 0, 1, 0]
    # |a-b| < 1e-7: the 5e-8 case rounds to an equal float; NaN is never equal
    assert list(jo.binary("eq", a, b)) == [0, 1, 0, 0, 1, 0]
    assert list(jo.binary("neq", a, b)) == [1, 0, 1, 1, 0, 1]
    assert list(jo.scalar("gte", a, 2.0)) == [0, 1, 1, 0, 0, 0]
    assert list(jo.scalar("eq", a, 1.0, eps=0.5)) == [1, 0, 0, 0, 1, 1]


# ------------------------------------------------------------------ reductions

def test_full_sum_is_serial_float_in_index_order():
    assert jo.sum_all([1e8, 1.0, -1e8]) == 0.0           # the 1 is absorbed; any tree order would give 1 or 0
    assert jo.sum_all([1.0, -1e8, 1e8]) == 0.0
    assert jo.sum_all([1e8, -1e8, 1.0]) == 1.0
    x = RNG.standard_normal(5000).astype(np.float32)
    acc = np.float32(0.0)
    for v in x:
        acc = np.float32(acc + v)
    assert jo.sum_all(x) == acc
    assert jo.sum_all([3.5]) == 3.5


def test_full_mean_accumulates_in_double_and_rounds_once():
    x = (RNG.standard_normal(5000) * 1000).astype(np.float32)
    acc = 0.0
    for v in x.tolist():
        acc += v
    assert jo.mean_all(x) == np.float32(acc / len(x))
    # float accumulation would lose the small terms here
    y = np.array([16777216.0] + [1.0] * 64, np.float32)
    assert jo.mean_all(y) == np.float32((16777216.0 + 64.0) / 65.0)


def py_lane(op, lane):
    """Independent statement of the per-lane rules (java.lang.Math semantics spelled out)."""
    f32 = np.float32
    if op in ("sum", "mean"):
        acc = f32(0.0)
        with np.errstate(invalid="ignore"):             # inf + -inf is part of the cases
            for v in lane:
                acc = f32(acc + f32(v))
        return acc if op == "sum" else f32(acc / f32(len(lane)))
    if op in ("max", "min"):
        acc = f32(-np.inf) if op == "max" else f32(np.inf)
        for v in lane:
            v = f32(v)
            if np.isnan(acc) or np.isnan(v):
                acc = f32(np.nan)
            elif acc == 0 and v == 0:
                neg = np.signbit(acc) or np.signbit(v) if op == "min" else np.signbit(acc) and np.signbit(v)
                acc = f32(-0.0) if neg else f32(0.0)
            else:
                acc = max(acc, v) if op == "max" else min(acc, v)
        return acc
    best, idx = (-np.inf, 0.0) if op == "arg_max" else (np.inf, 0.0)
    for j, v in enumerate(lane):
        if (op == "arg_max" and v > best) or (op == "arg_min" and v < best):
            best, idx = v, float(j)
    return f32(idx)


@pytest.mark.parametrize("op", ["sum", "mean", "max", "min", "arg_max", "arg_min"])
def test_axis_aggregation_brute_force(op):
    nan, inf = np.nan, np.inf
    x = RNG.integers(-3, 4, size=(3, 5, 4)).astype(np.float32)       # many ties
    x[0, :, 0] = -inf                                                 # lane with nothing > -inf
    x[1, 2, 1] = nan                                                  # NaN inside a lane
    x[2, 0, 2] = nan                                                  # NaN first in a lane
    x[2, :, 3] = [0.0, -0.0, 0.0, -0.0, -0.0]                         # signed zeros only
    x[1, :, 3] = [inf, 1.0, inf, -inf, 0.0]
    for axis in range(3):
        got = jo.aggregate(op, x, axis)
        moved = np.moveaxis(x, axis, -1)
        want = np.empty(moved.shape[:-1], np.float32)
        for idx in np.ndindex(*moved.shape[:-1]):
            want[idx] = py_lane(op, moved[idx].tolist())
        assert_bits_equal(np.squeeze(got, axis), want)


def test_argmax_rules_by_closed_form():
    x = RNG.standard_normal((40, 37)).astype(np.float32)
    x[:, 5] = x[:, 9]                                                  # duplicate column -> ties across axis 1
    assert (jo.aggregate("arg_max", x, 1).reshape(-1) == np.argmax(x, 1)).all()   # numpy: first occurrence
    assert (jo.aggregate("arg_min", x, 0).reshape(-1) == np.argmin(x, 0)).all()
    assert_bits_equal(jo.aggregate("max", x, 0).reshape(-1), x.max(0))
    assert jo.aggregate("arg_max", [[np.nan, np.nan]], 1)[0, 0] == 0.0
    assert jo.aggregate("arg_max", [[np.nan, -np.inf, 3.0, np.nan, 3.0]], 1)[0, 0] == 2.0
    assert np.isnan(jo.aggregate("max", [[1.0, np.nan, 3.0]], 1)[0, 0])


def test_axis_mean_divides_the_float_sum():
    x = np.full((3, 7), 0.1, np.float32)
    acc = np.float32(0)
    for _ in range(7):
        acc = np.float32(acc + np.float32(0.1))
    assert (jo.aggregate("mean", x, 1).reshape(-1) == np.float32(acc / np.float32(7))).all()


def test_f64_yardsticks():
    x = RNG.standard_normal((50, 60)).astype(np.float32)
    s, a = jo.axis_sum_f64(x, 0)
    np.testing.assert_allclose(s.reshape(-1), x.astype(np.float64).sum(0), rtol=1e-14, atol=1e-13)
    np.testing.assert_allclose(a.reshape(-1), np.abs(x.astype(np.float64)).sum(0), rtol=1e-14)
    assert abs(jo.sum_all_f64(x) - math.fsum(x.reshape(-1).tolist())) < 1e-10


def test_contains_nan_and_fill(oracle_ops):
    t = oracle_ops.createRaw([2, 3], [1, 2, 3, 4, 5, 6])
    assert not t.containsNan()
    t.inplaceFill(float("nan"))
    assert t.containsNan()


# ------------------------------------------------------------------ gather / scatter

INDEX_CASES = [([4, 5], [4, 3], 1), ([4, 5], [2, 5], 0), ([3, 4, 5], [3, 2, 5], 1), ([3, 4, 5], [2, 4, 2], 2),
               ([6], [9], 0), ([2, 3, 4, 5], [2, 3, 7, 5], 2)]


@pytest.mark.parametrize("shape,ishape,axis", INDEX_CASES)
def test_gather_matches_numpy_take_along_axis(shape, ishape, axis, oracle_ops):
    x = RNG.standard_normal(shape).astype(np.float32)
    idx = RNG.integers(0, shape[axis], size=ishape)
    got = oracle_ops.createRaw(shape, x).gather(axis, oracle_ops.createRaw(ishape, idx.astype(np.float32))).toArray()
    # numpy needs equal non-axis dims: compare on the corner of x that index addresses
    corner = x[tuple(slice(0, ishape[d]) if d != axis else slice(None) for d in range(len(shape)))]
    assert_bits_equal(got, np.take_along_axis(corner, idx, axis))


@pytest.mark.parametrize("shape,ishape,axis", INDEX_CASES)
def test_scatter_and_scatter_add_brute_force(shape, ishape, axis, oracle_ops):
    idx = RNG.integers(0, shape[axis], size=ishape)                      # duplicates along the axis are likely
    src = RNG.standard_normal(ishape).astype(np.float32)
    base = RNG.standard_normal(shape).astype(np.float32)
    want_set, want_add, want_fill = base.copy(), base.copy(), base.copy()
    for pos in np.ndindex(*ishape):                                      # store order: last write wins, adds in order
        to = list(pos); to[axis] = idx[pos]
        want_set[tuple(to)] = src[pos]
        want_add[tuple(to)] = np.float32(want_add[tuple(to)] + src[pos])
        want_fill[tuple(to)] = 7.5
    ri = oracle_ops.createRaw(ishape, idx.astype(np.float32))
    t = oracle_ops.createRaw(shape, base); t.inplaceScatter(axis, ri, oracle_ops.createRaw(ishape, src))
    assert_bits_equal(t.toArray(), want_set)
    t = oracle_ops.createRaw(shape, base); t.inplaceScatterAdd(axis, ri, oracle_ops.createRaw(ishape, src))
    assert_bits_equal(t.toArray(), want_add)
    t = oracle_ops.createRaw(shape, base); t.inplaceScatter(axis, ri, 7.5)
    assert_bits_equal(t.toArray(), want_fill)
    copy = oracle_ops.createRaw(shape, base).scatter(axis, ri, oracle_ops.createRaw(ishape, src))
    assert_bits_equal(copy.toArray(), want_set)


def test_gather_scatter_reject_bad_indices_and_shapes(oracle_ops):
    x = oracle_ops.createRaw([2, 3], np.arange(6, dtype=np.float32))
    for bad in (3.0, -1.0):
        with pytest.raises(ValueError):
            x.gather(1, oracle_ops.createRaw([2, 1], [0.0, bad]))
        with pytest.raises(ValueError):
            x.inplaceScatter(1, oracle_ops.createRaw([2, 1], [0.0, bad]), oracle_ops.createRaw([2, 1], [1.0, 1.0]))
    assert x.gather(1, oracle_ops.createRaw([2, 1], [2.9, float("nan")])).toArray().tolist() == [[2.0], [3.0]]   # toInt(): 2, 0
    with pytest.raises(ValueError):      # index wider than the source
        x.inplaceScatter(1, oracle_ops.createRaw([2, 2], [0, 1, 0, 1]), oracle_ops.createRaw([2, 1], [1.0, 1.0]))
    with pytest.raises(ValueError):      # dim count mismatch
        x.inplaceScatter(1, oracle_ops.createRaw([2], [0, 1]), oracle_ops.createRaw([2], [1.0, 1.0]))
