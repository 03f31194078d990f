"""Seeded random cases at sizes of one to four million elements, where the tiled, streamed and
LDS-staged kernels take over from the small-tensor forms that the property tests reach: axis
reductions, permutes, broadcasts and the indexed moves, against the CPU checker (or numpy where
the checker is pinned to numpy for that op). Bit-exact except SUM, by the two-clause tolerance."""
import numpy as np
import pytest

from oracle import jvm_oracle as jo
from parity import assert_bits_equal, assert_reduction_close

pytestmark = pytest.mark.gpu


def factor(rng, total, k):
    """k dims whose product is about `total`."""
    logs = rng.dirichlet(np.ones(k)) * np.log(total)
    return [max(1, int(round(np.exp(v)))) for v in logs]


@pytest.mark.parametrize("seed", range(6))
def test_random_reductions(seed, gc):
    rng = np.random.default_rng(1000 + seed)
    for _ in range(10):
        k = int(rng.integers(2, 5))
        shape = factor(rng, int(rng.integers(1 << 20, 1 << 22)), k)
        axis = int(rng.integers(0, k))
        if shape[axis] > (1 << 20):
            continue
        x = (np.round(rng.standard_normal(shape) * 8) / 8).astype(np.float32)      # eighths: many ties
        flat = x.reshape(-1)
        flat[rng.integers(0, flat.size, 5)] = np.nan
        flat[rng.integers(0, flat.size, 5)] = -0.0
        t = gc.createRaw(shape, x)
        for op, code in (("max", "max"), ("argMin", "arg_min"), ("argMax", "arg_max")):
            assert_bits_equal(getattr(t, op)(axis).toArray().reshape(-1), jo.aggregate(code, x, axis).reshape(-1),
                              f"{op} {shape} axis {axis}")
        clean = np.nan_to_num(x, nan=1.0)
        tc = gc.createRaw(shape, clean)
        ref64, _ = jo.axis_sum_f64(clean, axis)
        assert_reduction_close(tc.sum(axis).toArray().reshape(-1), ref64, jo.aggregate("sum", clean, axis).reshape(-1),
                               f"sum {shape} axis {axis}")
        gc.release(t); gc.release(tc)


@pytest.mark.parametrize("seed", range(4))
def test_random_permutes(seed, gc):
    rng = np.random.default_rng(2000 + seed)
    for _ in range(10):
        k = int(rng.integers(2, 6))
        shape = factor(rng, int(rng.integers(1 << 19, 1 << 21)), k)
        perm = [int(v) for v in rng.permutation(k)]
        x = rng.standard_normal(shape).astype(np.float32)
        t = gc.createRaw(shape, x)
        got = t.permute(perm)
        assert_bits_equal(got.toArray(), np.transpose(x, perm), f"permute {shape} {perm}")
        gc.release(t); gc.release(got)


@pytest.mark.parametrize("seed", range(4))
def test_random_broadcasts(seed, gc):
    rng = np.random.default_rng(3000 + seed)
    for _ in range(12):
        k = int(rng.integers(2, 5))
        shape = factor(rng, int(rng.integers(1 << 19, 1 << 21)), k)
        a_shape = [d if rng.random() < 0.6 else 1 for d in shape]
        b_shape = [d if rng.random() < 0.6 else 1 for d in shape]
        for i in range(k):
            if a_shape[i] == 1 and b_shape[i] == 1:
                (a_shape if rng.random() < 0.5 else b_shape)[i] = shape[i]
        drop = int(rng.integers(0, k))
        if all(d == 1 for d in b_shape[:drop]):
            b_shape = b_shape[drop:] or [1]
        a = rng.standard_normal(a_shape).astype(np.float32)
        b = rng.uniform(0.5, 2.0, b_shape).astype(np.float32)
        ta, tb = gc.createRaw(a_shape, a), gc.createRaw(b_shape, b)
        for op, fn in (("plus", np.add), ("times", np.multiply), ("div", np.divide), ("minus", np.subtract)):
            got = ta._binary(op, tb)
            assert_bits_equal(got.toArray(), fn(a, b), f"{op} {a_shape} {b_shape}")
            gc.release(got)
        gc.release(ta); gc.release(tb)


@pytest.mark.parametrize("seed", range(4))
def test_random_indexed_moves(seed, gc):
    rng = np.random.default_rng(4000 + seed)
    cpu = jo.JvmOracleOperations()
    for _ in range(6):
        k = int(rng.integers(2, 4))
        shape = factor(rng, int(rng.integers(1 << 18, 1 << 20)), k)
        axis = int(rng.integers(0, k))
        if shape[axis] > 40000:
            continue
        ishape = list(shape)
        ishape[axis] = max(1, int(shape[axis] * rng.uniform(0.2, 1.5)))
        for d in range(k):
            if d != axis and rng.random() < 0.3:
                ishape[d] = max(1, ishape[d] // 2)
        x = rng.standard_normal(shape).astype(np.float32)
        idx = rng.integers(0, shape[axis], size=ishape).astype(np.float32)
        src = rng.standard_normal(ishape).astype(np.float32)
        gx, cx = gc.createRaw(shape, x), cpu.createRaw(shape, x)
        gi, ci = gc.createRaw(ishape, idx), cpu.createRaw(ishape, idx)
        gs, cs = gc.createRaw(ishape, src), cpu.createRaw(ishape, src)
        assert_bits_equal(gx.gather(axis, gi).toArray(), cx.gather(axis, ci).toArray(), f"gather {shape} {ishape} axis {axis}")
        for name in ("inplaceScatter", "inplaceScatterAdd"):
            gt, ct = gc.createRaw(shape, x), cpu.createRaw(shape, x)
            getattr(gt, name)(axis, gi, gs); getattr(ct, name)(axis, ci, cs)
            assert_bits_equal(gt.toArray(), ct.toArray(), f"{name} {shape} {ishape} axis {axis}")
        # row lists
        n_rows = max(1, int(shape[axis] * rng.uniform(0.3, 3.0)))
        rows = rng.integers(0, shape[axis], size=[n_rows]).astype(np.float32)
        gr, cr = gc.createRaw([n_rows], rows), cpu.createRaw([n_rows], rows)
        got, want = gx.indexSelect(axis, gr), cx.indexSelect(axis, cr)
        assert_bits_equal(got.toArray(), want.toArray(), f"indexSelect {shape} axis {axis} k {n_rows}")
        add = rng.standard_normal(want.shape).astype(np.float32)
        ga, ca = gc.createRaw(want.shape, add), cpu.createRaw(want.shape, add)
        gt, ct = gc.createRaw(shape, x), cpu.createRaw(shape, x)
        gt.indexAdd(axis, gr, ga, 0.7); ct.indexAdd(axis, cr, ca, 0.7)
        assert_bits_equal(gt.toArray(), ct.toArray(), f"indexAdd {shape} axis {axis} k {n_rows}")


def tiny_and_large(rng, total, k):
    """k dims: one large, the others drawn from 1..12, in random order; product about `total`."""
    small = [int(rng.integers(1, 13)) for _ in range(k - 1)]
    big = max(1, total // int(np.prod(small)))
    dims = small + [big]
    return [dims[i] for i in rng.permutation(k)]


@pytest.mark.parametrize("seed", range(4))
def test_random_tiny_dims(seed, gc):
    """Tiny dims around one large dim: the smallest slabs, rows and runs of the tiled kernels, whose tile
    paddings and ragged last units differ from those of the mid-sized cases."""
    rng = np.random.default_rng(5000 + seed)
    cpu = jo.JvmOracleOperations()
    for _ in range(8):
        k = int(rng.integers(2, 5))
        shape = tiny_and_large(rng, int(rng.integers(1 << 19, 1 << 21)), k)
        x = (np.round(rng.standard_normal(shape) * 8) / 8).astype(np.float32)
        t = gc.createRaw(shape, x)
        ref = cpu.createRaw(shape, x)
        for axis in range(k):
            for op, code in (("max", "max"), ("argMax", "arg_max"), ("min", "min")):
                assert_bits_equal(getattr(t, op)(axis).toArray().reshape(-1), jo.aggregate(code, x, axis).reshape(-1),
                                  f"{op} {shape} axis {axis}")
            ref64, _ = jo.axis_sum_f64(x, axis)
            assert_reduction_close(t.sum(axis).toArray().reshape(-1), ref64, jo.aggregate("sum", x, axis).reshape(-1),
                                   f"sum {shape} axis {axis}")
        perm = [int(v) for v in rng.permutation(k)]
        assert_bits_equal(t.permute(perm).toArray(), np.transpose(x, perm), f"permute {shape} {perm}")
        # a broadcast partner that keeps a random subset of the dims
        b_shape = [d if rng.random() < 0.5 else 1 for d in shape]
        b = rng.uniform(0.5, 2.0, b_shape).astype(np.float32)
        tb = gc.createRaw(b_shape, b)
        assert_bits_equal(t._binary("times", tb).toArray(), x * b, f"times {shape} {b_shape}")
        assert_bits_equal(tb._binary("minus", t).toArray(), b - x, f"minus {b_shape} {shape}")
        # a box with ragged ends in every dim
        ranges = []
        for d in shape:
            lo = int(rng.integers(0, d)); hi = int(rng.integers(lo, d))
            ranges.append((lo, hi))
        want = x[tuple(slice(lo, hi + 1) for lo, hi in ranges)]
        assert_bits_equal(t.get(ranges).toArray().reshape(-1), want.reshape(-1), f"get {shape} {ranges}")
        assert_bits_equal(ref.get(ranges).toArray().reshape(-1), want.reshape(-1), f"checker get {shape} {ranges}")
