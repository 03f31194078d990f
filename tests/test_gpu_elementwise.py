"""Parity of the elementwise HIP kernels with the CPU checker, through the C ABI.
Bars: bit-exact for everything that is a composition of single IEEE roundings or an
index map; at most 2 ulp for the f64-libm-then-round functions (parity.py)."""
import ctypes

import numpy as np
import pytest

from kten_amd import abi
from oracle import jvm_oracle as jo
from parity import assert_bits_equal, assert_ulp_close, sample_floats

pytestmark = pytest.mark.gpu

EXACT_UNARY = ["neg", "reciprocal", "abs", "sign", "sqrt", "floor", "ceil", "round", "trunc", "rsqrt"]
LIBM_UNARY = ["log", "exp", "tanh", "sigmoid", "sinh", "cosh", "sin", "cos", "tan", "asin", "acos", "atan"]


def raw(gc, a):
    a = np.asarray(a, dtype=np.float32)
    return gc.createRaw(list(a.shape) if a.ndim else [1], a)


@pytest.fixture(scope="module")
def samples():
    rng = np.random.default_rng(42)
    return np.concatenate([sample_floats(rng, 200000), rng.uniform(-1, 1, 100003).astype(np.float32)])


@pytest.mark.parametrize("op", EXACT_UNARY)
def test_exact_unary(op, gc, samples):
    assert_bits_equal(raw(gc, samples)._unary(op).toArray(), jo.unary(op, samples), op)


@pytest.mark.parametrize("op", LIBM_UNARY)
def test_libm_unary_within_2ulp(op, gc, samples):
    worst = assert_ulp_close(raw(gc, samples)._unary(op).toArray(), jo.unary(op, samples), what=op)
    print(f"{op}: max ulp distance {worst}")


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 1023, 1024, 1025, 4099, 262147])
def test_unary_sizes_and_tails(n, gc):
    x = np.random.default_rng(n).standard_normal(n).astype(np.float32)
    assert_bits_equal(raw(gc, x)._unary("neg").toArray(), -x)
    assert_bits_equal(raw(gc, x).plus(1.5).toArray(), x + np.float32(1.5))
    assert_bits_equal((raw(gc, x) * raw(gc, x)).toArray(), x * x)


def test_clamp(gc, samples):
    for lo, hi in ((-1.0, 1.0), (0.15, 0.55), (0.0, 5.0), (-5.0, -0.0)):
        assert_bits_equal(raw(gc, samples).clamp(lo, hi).toArray(), jo.clamp(samples, lo, hi), f"clamp {lo} {hi}")


@pytest.mark.parametrize("op", ["plus", "minus", "times", "div", "pow", "lt", "lte", "gt", "gte", "eq", "neq"])
def test_scalar_ops(op, gc, samples):
    x = samples[:50000]
    for c in (2.0, -0.75, 1e-3, 0.0, 3.0, -0.5, 1.0, 4.0, -1.0, -2.0, 0.5):
        got = raw(gc, x)._scalar(op, c).toArray()
        want = jo.scalar(op, x, c)
        if op == "pow":
            assert_ulp_close(got, want, what=f"pow {c}")
            if c in (0.0, 1.0, 2.0, 3.0, 4.0, -1.0, -2.0, 0.5):     # exponents computed without the transcendental routine
                assert_bits_equal(got, want, f"pow {c}")
        else:
            assert_bits_equal(got, want, f"{op} {c}")


def test_reverse_pow(gc, samples):
    x = samples[:50000]
    for c in (2.0, 0.5, 10.0, -2.0, 1.0, 0.0):
        assert_ulp_close(gc.pow(c, raw(gc, x)).toArray(), jo.scalar("pow", x, c, reverse=True), what=f"{c} pow x")


def test_scalar_inplace(gc, samples):
    x = samples[:50000]
    t = raw(gc, x)
    t += 0.25
    t *= -3.0
    t /= 7.0
    want = ((x + np.float32(0.25)) * np.float32(-3.0)) / np.float32(7.0)
    with np.errstate(all="ignore"):
        assert_bits_equal(t.toArray(), want)


SHAPE_PAIRS = [
    ([2, 4], [2, 1]), ([3, 3], [3]), ([3, 3], [1]), ([3, 1], [1, 3]), ([1, 3], [3, 3]), ([2, 3, 4], [3, 1]),
    ([5], [2, 3, 5]), ([2, 3, 4, 5], [1, 3, 1, 1]), ([1], [1]), ([4, 1, 2, 1], [1, 3, 1, 5]), ([7], [1]),
    ([64, 128], [128]), ([64, 128], [64, 1]), ([64, 1], [1, 128]), ([8, 16, 12, 20], [1, 16, 1, 1]),
    ([8, 16, 12, 20], [8, 1, 12, 1]), ([33, 1027], [1027]), ([33, 1027], [33, 1]), ([1, 1], [300, 500]),
    ([6, 1, 8, 1, 4], [1, 5, 1, 3, 4]), ([2, 1, 2, 1, 2, 1, 2, 1, 2, 4], [1, 3, 1, 3, 1, 3, 1, 3, 1, 4]),
    ([1000, 1000], [1000, 1000]), ([4, 250, 1000], [1000]), ([1], [1000003]),
]


@pytest.mark.parametrize("sa,sb", SHAPE_PAIRS, ids=lambda s: "x".join(map(str, s)))
def test_binary_broadcast_index_map_bit_exact(sa, sb, gc):
    rng = np.random.default_rng(sum(sa) * 31 + sum(sb))
    a = rng.standard_normal(sa).astype(np.float32); b = rng.standard_normal(sb).astype(np.float32)
    for op, f in (("plus", np.add), ("times", np.multiply), ("div", np.divide), ("minus", np.subtract)):
        for x, y in ((a, b), (b, a)):
            got = raw(gc, x)._binary(op, raw(gc, y)).toArray()
            assert_bits_equal(got, f(x, y), f"{op} {list(x.shape)} {list(y.shape)}")


# Two operands that are both smaller than the output, innermost dim not a multiple of 4: the outer-product kernel
# that stages both in LDS. Column counts shorter and longer than a workgroup's span of 4096 outputs (the window of
# columns wraps, or the whole operand is staged), runs of 1, 2, 3 and 5 floats that both operands keep, outputs that
# do not end on a group of four, and the two shapes of the measured gap at full size.
OUTER_PAIRS = [
    ([3000, 1], [1, 111]), ([70001, 1], [1, 5]), ([300, 1], [1, 5001]), ([40, 1], [1, 4099]), ([9, 1], [1, 100003]),
    ([20011, 1], [1, 3]), ([56, 1, 2], [3001, 2]), ([700, 1, 3], [37, 3]), ([5, 1, 5], [4001, 5]), ([2, 1, 1023], [17, 1023]),
    ([33, 1, 7], [1, 1250, 7]), ([302683, 1], [1, 111]), ([56, 1, 2], [277788, 2]),
    # a column operand longer than a workgroup's tile: blocks of 8 row indexes by 1024 column offsets, ragged on both sides
    ([13, 1, 3], [100001, 3]), ([17, 1], [1, 8193]), ([8, 1], [1, 8192 + 1025]), ([1000, 1, 2], [4097, 2]),
    # the column operand without the innermost run, [N,1,V] o [1,M,1]: windows of column indexes that wrap, whole operands,
    # two columns, column operands longer than a tile
    ([4225, 1, 5], [1, 158, 1]), ([197, 1, 2], [1, 57497, 1]), ([48, 1, 1, 111], [1, 6259, 1, 1]), ([219, 1, 1, 70], [1, 1, 2188, 1]),
    ([3, 1, 78], [1, 143395, 1]), ([33000, 1, 3], [1, 2, 1]), ([8, 1, 2, 3], [1, 69905, 1, 1]), ([15497, 1, 3, 3], [1, 189, 1, 1]),
    ([7, 1, 1023], [1, 9, 1]), ([600, 1, 7], [1, 1171, 1]), ([2, 1, 5], [1, 4099, 1]),
]


@pytest.mark.parametrize("sa,sb", OUTER_PAIRS, ids=lambda s: "x".join(map(str, s)))
def test_broadcast_of_two_small_operands_bit_exact(sa, sb, gc):
    rng = np.random.default_rng(sum(sa) * 7 + sum(sb))
    a = rng.standard_normal(sa).astype(np.float32); b = rng.standard_normal(sb).astype(np.float32)
    gc.profileBegin()
    results = []
    for op, f in (("minus", np.subtract), ("div", np.divide)):
        for x, y in ((a, b), (b, a)):
            results.append((raw(gc, x)._binary(op, raw(gc, y)).toArray(), f(x, y), f"{op} {list(x.shape)} {list(y.shape)}"))
    kernels = gc.profileEnd()
    assert any(k.startswith("binary_outer_") for k in kernels), f"expected the outer-product kernel, saw {sorted(kernels)}"
    for got, want, what in results:
        assert_bits_equal(got, want, what)


# Two operands that are both smaller than the output in the arrangements the outer-product kernels do not take: an
# operand that keeps the outermost and the innermost dim but not the one between, a batch dim both keep, four to six
# dims, an operand of one value per batch, innermost dims that are no multiple of 4.
MANY_DIM_PAIRS = [
    ([4225, 1, 5], [1, 158, 1]), ([1, 5833, 1], [115, 1, 5]), ([111, 549, 1], [111, 1, 55]), ([248, 4, 1, 21], [1, 4, 161, 1]),
    ([3, 1, 7, 1, 9, 1], [1, 11, 1, 5, 1, 13]), ([2, 90001, 1], [2, 1, 3]), ([7, 1, 1, 3], [7, 6000, 1, 1]), ([50, 1, 3], [50, 401, 1]),
    ([2, 3, 1, 5, 1], [2, 1, 300, 1, 7]), ([1, 3, 1, 3], [40001, 1, 1, 1]), ([9, 1, 1201], [1, 5, 1]), ([1201, 1, 9], [1, 5, 1]),
    ([33000, 1, 3], [1, 2, 1]),
]


@pytest.mark.parametrize("sa,sb", MANY_DIM_PAIRS, ids=lambda s: "x".join(map(str, s)))
def test_broadcast_of_two_small_operands_in_many_dims_bit_exact(sa, sb, gc):
    rng = np.random.default_rng(sum(sa) * 11 + sum(sb))
    a = rng.standard_normal(sa).astype(np.float32); b = rng.standard_normal(sb).astype(np.float32)
    for op, f in (("minus", np.subtract), ("div", np.divide)):
        for x, y in ((a, b), (b, a)):
            assert_bits_equal(raw(gc, x)._binary(op, raw(gc, y)).toArray(), f(x, y), f"{op} {list(x.shape)} {list(y.shape)}")


# The same arrangements where the outermost one or two dims become batch dims of the grid and what is left inside them
# is an outer product or a broadcast with one operand as large as the item: which kernel takes which, and items that
# are no multiple of 4 floats (the outer-product kernel stores at dword addresses; the mixed kernel is not batched then).
BATCHED_PAIRS = [
    (([1, 19, 1, 2], [4, 1, 2045, 1]), "binary_outer_rows_kernel"),           # [N,1,V] o [1,M,1] under a batch dim of 4
    (([46, 1, 4, 1], [1, 26, 4, 165]), "binary_bcast_mixed_kernel_batched"),  # b is as large as the item [26,4,165]
    (([111, 549, 1], [111, 1, 55]), "binary_outer_kernel"),                   # a dim of 111 both keep, over [N,1] o [1,M]
    (([248, 4, 1, 21], [1, 4, 161, 1]), "binary_outer_kernel"),               # two batch dims, items of 3381 floats
    (([37, 3, 1, 7], [1, 3, 211, 1]), "binary_outer_kernel"),                 # items of 1477 floats
    (([3, 70001, 1], [3, 1, 5]), "binary_outer_kernel"),
    (([5, 1, 3, 1], [1, 900, 3, 17]), "binary_bcast_mixed_kernel_batched"),   # items of 45900 floats
    # two batch dims: the full operand has the outer one too, the small one the dim inside it
    (([1, 40, 24, 1], [150, 1, 24, 171]), "binary_bcast_mixed_kernel_batched"),
    (([5, 1, 3, 1], [1, 901, 3, 17]), "binary_bcast_mixed_kernel"),           # items of 45951 floats: not batched
]


@pytest.mark.parametrize("pair,kernel", BATCHED_PAIRS,
                         ids=lambda v: "x".join(map(str, v[0])) + "_" + "x".join(map(str, v[1])) if isinstance(v, tuple) else v)
def test_broadcast_with_outer_dims_as_batch_dims_bit_exact(pair, kernel, gc):
    sa, sb = pair
    rng = np.random.default_rng(sum(sa) * 17 + sum(sb))
    a = rng.standard_normal(sa).astype(np.float32); b = rng.standard_normal(sb).astype(np.float32)
    gc.profileBegin()
    results = []
    for op, f in (("minus", np.subtract), ("div", np.divide)):
        for x, y in ((a, b), (b, a)):
            results.append((raw(gc, x)._binary(op, raw(gc, y)).toArray(), f(x, y), f"{op} {list(x.shape)} {list(y.shape)}"))
    kernels = gc.profileEnd()
    assert any(k.startswith(kernel + "<") for k in kernels), f"expected {kernel}, saw {sorted(kernels)}"
    for got, want, what in results:
        assert_bits_equal(got, want, what)


# An operand that repeats along a dim and holds megabytes inside it: the tiles of the output are taken chunk by chunk
# across the repeats so that the operand's chunk stays in L2. Slices that end inside a tile and inside a chunk, repeats
# over two dims, both operands repeating, a scalar innermost dim of the repeating operand.
CHUNKED_PAIRS = [
    ([6, 511, 1020], [1, 511, 1020]), ([2, 3, 130001, 4], [1, 1, 130001, 4]), ([1, 3, 4, 56860], [5, 1, 4, 56860]),
    ([3, 1, 3, 131076], [1, 2, 3, 131076]), ([6, 400003, 4], [400003, 1]), ([2, 5, 1, 50021, 8], [1, 1, 3, 50021, 8]),
    ([6, 4194304], [4194304]), ([6, 2, 1572864], [1, 2, 1572864]),
]


@pytest.mark.parametrize("sa,sb", CHUNKED_PAIRS, ids=lambda s: "x".join(map(str, s)))
def test_broadcast_with_tiles_ordered_for_reuse_bit_exact(sa, sb, gc):
    rng = np.random.default_rng(sum(sa) * 13 + sum(sb))
    a = rng.standard_normal(sa).astype(np.float32); b = rng.standard_normal(sb).astype(np.float32)
    gc.profileBegin()
    results = []
    for op, f in (("minus", np.subtract), ("div", np.divide)):
        for x, y in ((a, b), (b, a)):
            results.append((raw(gc, x)._binary(op, raw(gc, y)).toArray(), f(x, y), f"{op} {list(x.shape)} {list(y.shape)}"))
    kernels = gc.profileEnd()
    assert any("_chunked" in k for k in kernels), f"expected the chunked tile order, saw {sorted(kernels)}"
    for got, want, what in results:
        assert_bits_equal(got, want, what)


def test_binary_matches_checker_on_small_broadcasts(gc):
    rng = np.random.default_rng(5)
    for sa, sb in SHAPE_PAIRS[:12]:
        a = rng.uniform(0.5, 3, sa).astype(np.float32); b = rng.uniform(-2, 2, sb).astype(np.float32)
        for op in ("plus", "minus", "times", "div", "lt", "gte"):
            if op in ("lt", "gte"):
                continue          # comparisons do not broadcast on the JVM backend
            assert_bits_equal(raw(gc, a)._binary(op, raw(gc, b)).toArray(), jo.binary(op, a, b), op)
        assert_ulp_close(raw(gc, a)._binary("pow", raw(gc, b)).toArray(), jo.binary("pow", a, b), what="pow")


def test_binary_pow_special_cases(gc):
    nan, inf = np.nan, np.inf
    a = np.array([1.0, -1.0, 1.0, nan, 5.0, -8.0, 2.0, 0.0, -0.0, 2.0, -2.0, 0.0, inf], np.float32)
    b = np.array([nan, inf, -inf, 0.0, 0.0, 1 / 3, 10.0, -1.0, -1.0, -inf, 3.0, 0.0, -1.0], np.float32)
    assert_bits_equal(raw(gc, a).pow(raw(gc, b)).toArray(), jo.binary("pow", a, b))


def test_binary_same_shape_specials_and_inplace(gc, samples):
    x = samples[:100000]; y = np.random.default_rng(3).permutation(x)
    with np.errstate(all="ignore"):
        for op, f in (("plus", np.add), ("minus", np.subtract), ("times", np.multiply), ("div", np.divide)):
            assert_bits_equal(raw(gc, x)._binary(op, raw(gc, y)).toArray(), f(x, y), op)
        t = raw(gc, x); t += raw(gc, y); assert_bits_equal(t.toArray(), x + y)
        t = raw(gc, x); t *= raw(gc, y); assert_bits_equal(t.toArray(), x * y)


def test_comparisons(gc, samples):
    x = samples[:100000]; y = np.random.default_rng(4).permutation(x)
    y[:1000] = x[:1000]
    y[1000:2000] = x[1000:2000] + np.float32(5e-8)
    cpu = jo.JvmOracleOperations()
    for op in ("lt", "lte", "gt", "gte", "eq", "neq"):
        got = raw(gc, x)._compare(op, raw(gc, y)).toArray()
        want = cpu.createRaw([x.size], x)._compare(op, cpu.createRaw([y.size], y)).toArray()
        assert_bits_equal(got, want, op)
    gc.setEpsilon(0.5)
    try:
        assert_bits_equal(raw(gc, x).eq(1.0).toArray(), jo.scalar("eq", x, 1.0, eps=0.5))
    finally:
        gc.setEpsilon(1e-7)


def test_no_fused_multiply_add_across_ops(gc):
    a = np.float32(1.0 + 2 ** -12)
    t = raw(gc, [a]) * raw(gc, [a])
    r = (t + (-1.0)).toArray()[0]
    assert r == np.float32(np.float32(a * a) + np.float32(-1.0))


def test_broadcast_to(gc):
    rng = np.random.default_rng(9)
    for src, dst in [([3, 1], [2, 3, 4]), ([1], [5, 5]), ([1, 128], [64, 128]), ([64, 1], [64, 128]), ([1], [1000, 1000]),
                     ([1, 16, 1, 1], [8, 16, 12, 20]), ([7], [3, 7])]:
        a = rng.standard_normal(src).astype(np.float32)
        assert_bits_equal(raw(gc, a).broadcastTo(dst).toArray(), np.broadcast_to(a, dst), f"{src}->{dst}")
    t = raw(gc, rng.standard_normal([4, 5]))
    assert t.broadcastTo([4, 5]) is t


def test_shape_errors_are_raised_before_any_launch(gc):
    a = raw(gc, np.zeros([2, 3])); b = raw(gc, np.zeros([3, 2]))
    launches = gc.getMetrics()["launches"]
    with pytest.raises(ValueError):
        a + b
    with pytest.raises(ValueError):
        a.plusAssign(b)
    with pytest.raises(ValueError):
        a.broadcastTo([3])
    with pytest.raises(ValueError):
        a.sum(5)
    assert gc.getMetrics()["launches"] == launches


def test_empty_tensors_give_empty_results_without_a_launch(gc):
    """A dim of 0 (e.g. the result of indexSelect with no index) reaches the plan builders: the JVM returns empty
    tensors there (JVMRawTensor.kt:75-87 over an empty FloatArray); nothing may be launched or divided by."""
    a = gc.createRaw([0, 3]); b = gc.createRaw([0, 3]); c = raw(gc, np.ones([3])); d = raw(gc, np.ones([1, 3]))
    mask = raw(gc, np.ones([3]))
    launches = gc.getMetrics()["launches"]
    for res in (a + b, a * c, c - a, a.pow(b), a.maskedFill(mask, 2.0), d.broadcastTo([0, 3]), c.broadcastTo([2, 0, 3]),
                a + 1.0, a.exp(), a.clamp(0.0, 1.0), a.copy()):
        assert res.shape[-1] == 3 and res.size == 0 and res.toArray().size == 0
    a.plusAssign(b); a.timesAssign(2.0)
    # straight through the ABI with numpy's rule for a dim of 1 against a dim of 0 as well
    out = gc.createRaw([0, 3])
    abi.check(gc.lib.kth_binary(abi.Op.DIV, a.storeReference, abi.shape_array([0, 3]), 2, d.storeReference, abi.shape_array([1, 3]), 2,
                                out.storeReference, abi.shape_array([0, 3]), 2))
    assert gc.getMetrics()["launches"] == launches
    with pytest.raises(ValueError):
        a + raw(gc, np.ones([2]))
    with pytest.raises(ValueError):
        a / d           # the common shape of [0, 3] and [1, 3] is the per-dim maximum [1, 3] (AbstractRawTensor.kt:170-192): no broadcast


def test_abi_rejects_bad_arguments(hip):
    L = hip.lib
    sh = abi.shape_array([2, 3])
    h = ctypes.c_uint64()
    abi.check(L.kth_alloc(6, ctypes.byref(h)))
    try:
        assert L.kth_unary(abi.Op.EXP, 0xdeadbeef, h.value, 6) == abi.KTH_E_HANDLE
        assert "handle" in abi.last_error()
        assert L.kth_unary(abi.Op.PLUS, h.value, h.value, 6) == abi.KTH_E_ARGUMENT
        assert L.kth_unary(abi.Op.EXP, h.value, h.value, 7) == abi.KTH_E_ARGUMENT
        assert L.kth_binary(abi.Op.PLUS, h.value, sh, 11, h.value, sh, 2, h.value, sh, 2) == abi.KTH_E_ARGUMENT
        assert L.kth_binary(abi.Op.PLUS, h.value, sh, 2, h.value, abi.shape_array([3, 2]), 2, h.value, sh, 2) == abi.KTH_E_SHAPE
        assert L.kth_binary(abi.Op.PLUS, h.value, sh, 2, h.value, abi.shape_array([3]), 1, h.value, sh, 2) == abi.KTH_E_ARGUMENT  # aliases a broadcast operand
        assert L.kth_reduce_axis(abi.Op.SUM, h.value, h.value, 2, 3, 1) == abi.KTH_E_ARGUMENT
        assert L.kth_reduce_axis(abi.Op.EXP, h.value, h.value, 2, 3, 1) == abi.KTH_E_ARGUMENT
        assert L.kth_fill(h.value, 4, 3, 1.0) == abi.KTH_E_ARGUMENT
    finally:
        abi.check(L.kth_release(h.value))
    assert L.kth_release(h.value) == abi.KTH_E_HANDLE          # stale handle detected


def test_store_housekeeping(gc):
    x = np.arange(1000, dtype=np.float32)
    t = raw(gc, x)
    assert t.getSingleValue([999]) == 999.0 and t.getSingleValue([-1000]) == 0.0
    c = t.copy()
    c.inplaceFill(7.0)
    assert t.getSingleValue([5]) == 5.0 and c.getSingleValue([5]) == 7.0
    v = t.view([10, 100])
    assert v.shape == [10, 100] and v.getSingleValue([9, 99]) == 999.0
    s = t.copy(shallow=True)
    s.inplaceFill(1.0)                                      # shares the store
    assert t.getSingleValue([3]) == 1.0
    assert not t.containsNan()
    n = raw(gc, np.where(np.arange(100003) == 77777, np.nan, 1.0))
    assert n.containsNan()
    z = gc.zerosLike(t)
    assert z.shape == [1000] and not z.toArray().any()
    r = t.reshape(4, 250)
    assert r.shape == [4, 250]
    u = t.unsqueeze(0)
    assert u.shape == [1, 1000] and u.squeeze(0).shape == [1000]
    # partial fill through the ABI with unaligned offsets
    for off, cnt in ((1, 5), (3, 64), (0, 1), (7, 990)):
        w = raw(gc, x)
        abi.check(gc.lib.kth_fill(w.storeReference, off, cnt, -1.0))
        want = x.copy(); want[off:off + cnt] = -1.0
        assert_bits_equal(w.toArray(), want, f"fill {off}+{cnt}")


def test_pool_reuses_released_stores(hip):
    with hip.garbageCollector():
        a = hip.createRaw([1 << 20])
        live = hip.getMetrics()["liveBytes"]
    m = hip.getMetrics()
    assert m["liveBytes"] < live and m["poolBytes"] >= (1 << 22)
    with hip.garbageCollector():
        b = hip.createRaw([1 << 20])
        assert hip.getMetrics()["poolBytes"] <= m["poolBytes"] - (1 << 22)


def test_gc_scope_keeps_referenced_tensors(hip):
    with hip.garbageCollector():
        keep = hip.createRaw([16], np.arange(16, dtype=np.float32))
        hip.incrementRef(keep)
        drop = hip.createRaw([16])
    assert keep.referenced() and not drop.referenced()
    assert keep.getSingleValue([15]) == 15.0
    with pytest.raises(RuntimeError):
        drop.getSingleValue([0])
    keep.release()
    assert not keep.referenced()


@pytest.mark.parametrize("c", [3.0, 4.0, -1.0, -2.0, 0.5])
def test_pow_with_exact_exponents_over_the_float_space(c, gc):
    """Every 509th bit pattern (all exponents, signs and specials): the products, the quotient and the square root
    that stand in for pow at these exponents give the checker's pow bit for bit, -0, infinities and NaN included."""
    x = np.arange(0, 1 << 32, 509, dtype=np.uint64).astype(np.uint32).view(np.float32)
    assert_bits_equal(raw(gc, x)._scalar("pow", c).toArray(), jo.scalar("pow", x, c), f"pow {c}")


@pytest.mark.parametrize("n", [1, 2, 3, 5, 1023, 1027, 262147, 3000001])
def test_contains_nan_at_every_kind_of_position(n, gc):
    """A single NaN in the float4 body, in the tail of n mod 4 elements, at either end; infinities are not NaN."""
    x = np.random.default_rng(n).standard_normal(n).astype(np.float32)
    x[n // 3] = np.inf
    assert not raw(gc, x).containsNan()
    for pos in sorted({0, n // 2, max(0, n - 4), max(0, n - 3), max(0, n - 2), n - 1}):
        y = x.copy()
        y[pos] = np.nan
        assert raw(gc, y).containsNan(), f"NaN at {pos} of {n}"
