"""A fill of a store's head (zerosLike, createRawFill, inplaceFill, the upload of one value) is only
noted by the library and launched when somebody reads the store as memory; binary ops take the
constant as a scalar operand, a broadcast passes it on, a scatter starts its rows from it. Every
way in and out of that state must give the bits of the plain sequence (fill, then the op), which
numpy and the CPU checker compute here; the launch counter shows that the folded paths are taken."""
import numpy as np
import pytest

from oracle import jvm_oracle as jo
from parity import assert_bits_equal

pytestmark = pytest.mark.gpu

OPS = [("plus", np.add), ("minus", np.subtract), ("times", np.multiply), ("div", np.divide)]


def launches(gc):
    return gc.getMetrics()["launches"]


def test_a_filled_store_reads_back_whole_or_in_part(gc):
    t = gc.createRawFill([37, 53], 2.5)
    assert_bits_equal(t.toArray(), np.full([37, 53], 2.5, np.float32), "fill then download")
    u = gc.createRawFill([1000], -0.0)
    assert u.getSingleValue([999]) == 0.0 and np.signbit(u.toArray()).all()
    # refilled before anybody looked: the last fill is what the store holds
    v = gc.createRawFill([64, 64], 1.0)
    v.inplaceFill(3.0)
    v.inplaceFill(7.0)
    assert_bits_equal(v.toArray(), np.full([64, 64], 7.0, np.float32), "three fills")
    # a filled store that nobody reads is released without a launch
    before = launches(gc)
    w = gc.createRawFill([1 << 20], 4.0)
    w.release()
    assert launches(gc) == before


def test_partial_writes_into_a_filled_store(gc):
    rng = np.random.default_rng(1)
    t = gc.createRawFill([10, 100], 9.0)
    piece = rng.standard_normal([3, 100]).astype(np.float32)
    t._set_ranges([2, 0], [4, 99], gc.createRaw([3, 100], piece))          # first and last index of the box, inclusive
    want = np.full([10, 100], 9.0, np.float32); want[2:5] = piece
    assert_bits_equal(t.toArray(), want, "range set into a filled store")
    t2 = gc.createRawFill([10, 100], 9.0)
    t2._set_ranges([0, 10], [9, 19], 4.0)
    want = np.full([10, 100], 9.0, np.float32); want[:, 10:20] = 4.0
    assert_bits_equal(t2.toArray(), want, "range fill into a filled store")
    u = gc.createRawFill([10, 100], 9.0)
    u._set_store_range(150, 200, 1.5)
    want = np.full([1000], 9.0, np.float32); want[150:350] = 1.5
    assert_bits_equal(u.toArray().reshape(-1), want, "store-range fill into a filled store")
    # a shorter fill over the head of a longer one keeps the tail
    v = gc.createRawFill([1000], 2.0)
    v._set_store_range(0, 10, 5.0)
    want = np.full([1000], 2.0, np.float32); want[:10] = 5.0
    assert_bits_equal(v.toArray(), want, "short fill over a long one")


@pytest.mark.parametrize("name,ref", OPS, ids=[o[0] for o in OPS])
def test_binary_ops_take_a_filled_operand_as_a_scalar(name, ref, gc):
    rng = np.random.default_rng(2)
    x = rng.standard_normal([129, 67]).astype(np.float32)
    x[0, :6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45]
    for c in (0.0, -0.0, 1.0, -2.75, np.inf, 3.4028235e38):
        gx = gc.createRaw([129, 67], x)
        full = np.full([129, 67], c, np.float32)
        with np.errstate(all="ignore"):
            # the constant on the right, on the left, as a broadcast [1] and a broadcast row
            before = launches(gc)
            got = getattr(gx, name)(gc.createRawFill([129, 67], c))
            assert launches(gc) == before + 1, "fill folded: one launch"
            assert_bits_equal(got.toArray(), ref(x, full), f"x {name} fill({c})")
            assert_bits_equal(getattr(gc.createRawFill([129, 67], c), name)(gx).toArray(), ref(full, x), f"fill({c}) {name} x")
            assert_bits_equal(getattr(gx, name)(gc.createRaw([1], [c])).toArray(), ref(x, full), f"x {name} [1]")
            assert_bits_equal(getattr(gc.createRawFill([67], c), name)(gx).toArray(), ref(full, x), f"row fill {name} x")
            # a constant operand that is the larger one cannot ride as a scalar
            small = gc.createRaw([67], x[1])
            assert_bits_equal(getattr(small, name)(gc.createRawFill([129, 67], c)).toArray(), ref(x[1][None, :], full),
                              f"row {name} fill({c})")
            # both constant
            assert_bits_equal(getattr(gc.createRawFill([5, 7], c), name)(gc.createRawFill([5, 7], 0.5)).toArray(),
                              ref(np.full([5, 7], c, np.float32), np.float32(0.5)), "both filled")


@pytest.mark.parametrize("name,ref", OPS, ids=[o[0] for o in OPS])
def test_inplace_ops_on_and_with_filled_stores(name, ref, gc):
    rng = np.random.default_rng(3)
    x = rng.standard_normal([300, 41]).astype(np.float32)
    assign = name
    with np.errstate(all="ignore"):
        for c in (0.0, -0.0, 2.0):
            acc = gc.createRawFill([300, 41], c)                 # a gradient buffer fresh from zerosLike
            before = launches(gc)
            acc._binary_assign(assign, gc.createRaw([300, 41], x))
            assert launches(gc) == before + 1
            assert_bits_equal(acc.toArray(), ref(np.full([300, 41], c, np.float32), x), f"fill({c}) {assign}= x")
            acc._binary_assign(assign, gc.createRaw([300, 41], x))     # and again, now on real contents
            assert_bits_equal(acc.toArray(), ref(ref(np.full([300, 41], c, np.float32), x), x), f"second {assign}=")
            gx = gc.createRaw([300, 41], x)
            gx._binary_assign(assign, gc.createRawFill([300, 41], c))
            assert_bits_equal(gx.toArray(), ref(x, np.float32(c)), f"x {assign}= fill({c})")
        same = gc.createRawFill([64], 3.0)
        same._binary_assign(assign, same)
        assert_bits_equal(same.toArray(), ref(np.full([64], 3.0, np.float32), np.float32(3.0)), f"fill {assign}= itself")


def test_other_ops_see_the_filled_values(gc):
    t = gc.createRawFill([50, 60], 0.25)
    assert_bits_equal(t.pow(gc.createRawFill([50, 60], 2.0)).toArray(), np.full([50, 60], 0.0625, np.float32), "pow of two fills")
    assert_bits_equal(t.sqrt().toArray(), np.full([50, 60], 0.5, np.float32), "unary of a fill")
    assert_bits_equal(gc.createRawFill([50, 60], 0.25).sum(0).toArray(), np.full([60], 12.5, np.float32), "axis sum of a fill")
    assert gc.createRawFill([10], np.nan).containsNan() and not gc.createRawFill([10], 1.0).containsNan()
    lt = gc.createRawFill([7, 3], 1.0).lt(gc.createRawFill([7, 3], 2.0))
    assert_bits_equal(lt.toArray(), np.ones([7, 3], np.float32), "comparison of two fills")
    c = gc.createRawFill([300, 300], 6.0).copy()
    assert_bits_equal(c.toArray(), np.full([300, 300], 6.0, np.float32), "copy of a fill")
    v = gc.createRawFill([4, 5], 1.5).view([20])
    assert_bits_equal(v.toArray(), np.full([20], 1.5, np.float32), "view of a fill")
    tr = gc.createRawFill([33, 65], 8.0).transpose(0, 1)
    assert_bits_equal(tr.toArray(), np.full([65, 33], 8.0, np.float32), "transpose of a fill")


def test_broadcast_of_one_uploaded_value_stays_a_constant(gc):
    rng = np.random.default_rng(4)
    x = rng.standard_normal([257, 33]).astype(np.float32)
    seed = gc.createRaw([1], [1.0])                              # the seed gradient of backward()
    before = launches(gc)
    wide = seed.broadcastTo([257, 33])
    assert launches(gc) == before, "a broadcast constant is not written out"
    prod = wide.times(gc.createRaw([257, 33], x))
    assert launches(gc) == before + 1
    assert_bits_equal(prod.toArray(), x, "1 * x")
    assert_bits_equal(wide.toArray(), np.ones([257, 33], np.float32), "the broadcast itself, once read")
    assert seed.getSingleValue([0]) == 1.0
    # overwritten by an upload before anybody read it
    s2 = gc.createRaw([1], [5.0])
    s2._set_store_range(0, 1, 6.0)
    assert s2.getSingleValue([0]) == 6.0
    assert_bits_equal(s2.broadcastTo([3, 2]).toArray(), np.full([3, 2], 6.0, np.float32), "refilled scalar, broadcast")


SCATTER_CASES = [([64, 2048], [64, 2048], 1), ([300, 400], [300, 400], 1), ([4096, 96], [4096, 96], 0), ([3, 16384], [3, 5000], 1),
                 ([2, 32769], [2, 5000], 1), ([2, 3000, 40], [2, 2500, 40], 1),
                 # the index does not cover the target off the axis, or the serial form runs: the fill is launched first
                 ([10, 6, 300], [7, 4, 100], 2), ([8192, 3, 5], [8000, 2, 5], 0), ([1000, 300], [1000, 1], 1), ([4, 5], [2, 5], 0)]


@pytest.mark.parametrize("shape,ishape,axis", SCATTER_CASES, ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_scatter_into_a_filled_target(shape, ishape, axis, gc):
    rng = np.random.default_rng(sum(shape) + 7 * axis)
    idx = rng.integers(0, shape[axis], size=ishape).astype(np.float32)
    src = rng.standard_normal(ishape).astype(np.float32)
    cpu = jo.JvmOracleOperations()
    gi, ci = gc.createRaw(ishape, idx), cpu.createRaw(ishape, idx)
    gs, cs = gc.createRaw(ishape, src), cpu.createRaw(ishape, src)
    for c in (0.0, -0.0, 1.25):
        for name in ("inplaceScatter", "inplaceScatterAdd"):
            gt, ct = gc.createRawFill(shape, c), cpu.createRawFill(shape, c)
            getattr(gt, name)(axis, gi, gs); getattr(ct, name)(axis, ci, cs)
            assert_bits_equal(gt.toArray(), ct.toArray(), f"{name} into fill({c})")
            getattr(gt, name)(axis, gi, gs); getattr(ct, name)(axis, ci, cs)          # again, on real contents
            assert_bits_equal(gt.toArray(), ct.toArray(), f"second {name}")
        gt, ct = gc.createRawFill(shape, c), cpu.createRawFill(shape, c)
        gt.inplaceScatter(axis, gi, -1.0); ct.inplaceScatter(axis, ci, -1.0)
        assert_bits_equal(gt.toArray(), ct.toArray(), f"inplaceScatter(Float) into fill({c})")


def test_a_bad_index_into_a_filled_target_still_leaves_the_fill(gc):
    t = gc.createRawFill([4, 300], 2.0)
    idx = np.zeros([4, 300], np.float32); idx[2, 17] = 300.0
    with pytest.raises(ValueError):
        t.inplaceScatter(1, gc.createRaw([4, 300], idx), gc.createRaw([4, 300], np.ones([4, 300], np.float32)))
    got = t.toArray()
    assert (got[:, 1:] == 2.0).all() and (got[:, 0] == 1.0).all()


@pytest.mark.parametrize("name,ref", OPS, ids=[o[0] for o in OPS])
def test_scalar_ops_on_a_filled_store(name, ref, gc):
    """constant (op) constant is folded on the host where host and device arithmetic cannot differ,
    and computed by the kernel otherwise (subnormal operands or results, NaN): numpy's float32
    result either way."""
    consts = [0.0, -0.0, 1.0, -2.75, 3.0, 1e-30, 1e-10, 1e-45, 1.1754944e-38, 3.4028235e38, np.inf, -np.inf, np.nan, 1 / 3]
    rng = np.random.default_rng(5)
    x = rng.standard_normal([40, 25]).astype(np.float32)
    with np.errstate(all="ignore"):
        for c in consts:
            for k in consts:
                want = ref(np.float32(c), np.float32(k))
                t = gc.createRawFill([40, 25], c)
                got = t._scalar(name, float(np.float32(k)))
                assert_bits_equal(got.toArray(), np.full([40, 25], want, np.float32), f"fill({c}) {name} {k}")
                rev = t._scalar(name, float(np.float32(k)), reverse=True)
                assert_bits_equal(rev.toArray(), np.full([40, 25], ref(np.float32(k), np.float32(c)), np.float32), f"{k} {name} fill({c})")
        # the chain of a backward pass: a broadcast seed, times a constant, times a tensor in place
        seed = gc.createRaw([1], [1.0])
        before = launches(gc)
        g = seed.broadcastTo([40, 25])._scalar("times", 2.0)
        assert launches(gc) == before, "constant times constant: nothing to launch"
        g._binary_assign(name, gc.createRaw([40, 25], x))
        assert launches(gc) == before + 1
        assert_bits_equal(g.toArray(), ref(np.float32(2.0), x), f"2 {name}= x")
        # in place on the filled store itself, then read
        h = gc.createRawFill([40, 25], 3.0)
        h._scalar_assign(name, 0.5)
        h._scalar_assign(name, 0.25)
        assert_bits_equal(h.toArray(), np.full([40, 25], ref(ref(np.float32(3.0), np.float32(0.5)), np.float32(0.25)), np.float32),
                          f"fill {name}= 0.5 {name}= 0.25")


INDEX_ADD_CASES = [([500, 64], 0, 700), ([500, 63], 0, 700), ([6, 300, 8], 1, 1000), ([4, 5000], 1, 4000), ([300, 1], 0, 900),
                   ([2, 40, 3, 4], 1, 64), ([100, 16], 0, 63), ([7, 20000], 1, 30000)]


@pytest.mark.parametrize("shape,axis,k", INDEX_ADD_CASES, ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_index_add_into_a_filled_target(shape, axis, k, gc):
    rng = np.random.default_rng(sum(shape) + k)
    idx = rng.integers(0, shape[axis], size=[k]).astype(np.float32)
    idx[: k // 3] = idx[0]                                            # a long run on one row
    sshape = list(shape); sshape[axis] = k
    src = rng.standard_normal(sshape).astype(np.float32)
    cpu = jo.JvmOracleOperations()
    gi, ci = gc.createRaw([k], idx), cpu.createRaw([k], idx)
    gs, cs = gc.createRaw(sshape, src), cpu.createRaw(sshape, src)
    for c, alpha in ((0.0, 1.0), (-0.0, 1.0), (1.5, -0.75)):
        gt, ct = gc.createRawFill(shape, c), cpu.createRawFill(shape, c)
        gt.indexAdd(axis, gi, gs, alpha); ct.indexAdd(axis, ci, cs, alpha)
        assert_bits_equal(gt.toArray(), ct.toArray(), f"indexAdd into fill({c}), alpha {alpha}")
        gt.indexAdd(axis, gi, gs, alpha); ct.indexAdd(axis, ci, cs, alpha)
        assert_bits_equal(gt.toArray(), ct.toArray(), "second indexAdd")
    bad = idx.copy(); bad[k // 2] = shape[axis]
    gt = gc.createRawFill(shape, 2.0)
    with pytest.raises(ValueError):
        gt.indexAdd(axis, gc.createRaw([k], bad), gs, 1.0)
    assert np.isfinite(gt.toArray()).all()
