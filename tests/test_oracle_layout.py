"""Pins the CPU checker's layout movers (range get / set / fill, transpose, permute,
maskedFill, concat, narrow) to independent implementations: numpy's slicing, transpose,
where and concatenate on random shapes, and the index normalisation rules to the cases the
reference's tests use. The known answers of the reference's own tests for these members run
in test_oracle_known_answers.py."""
import itertools

import numpy as np
import pytest

from kten_amd.host_mirror import shape_functions as sf
from kten_amd.host_mirror.shape_functions import ALL, IntRange
from oracle import jvm_oracle as jo


def random_box(rng, shape):
    k = int(rng.integers(1, len(shape) + 1))
    ranges = []
    for d in range(k):
        f = int(rng.integers(0, shape[d])); l = int(rng.integers(f, shape[d]))
        ranges.append((f, l))
    return ranges


def test_range_get_set_fill_equal_numpy_slicing(oracle_ops):
    rng = np.random.default_rng(11)
    for _ in range(400):
        shape = [int(rng.integers(1, 7)) for _ in range(int(rng.integers(1, 6)))]
        a = rng.standard_normal(shape).astype(np.float32)
        ranges = random_box(rng, shape)
        sl = tuple(slice(f, l + 1) for f, l in ranges)
        t = oracle_ops.createRaw(shape, a.reshape(-1))
        got = t.get(ranges)
        assert got.shape == list(a[sl].shape)
        assert np.array_equal(got.toArray(), a[sl])
        v = rng.standard_normal(a[sl].shape).astype(np.float32)
        expect = a.copy(); expect[sl] = v
        t.set(ranges, oracle_ops.createRaw(list(v.shape), v.reshape(-1)))
        assert np.array_equal(t.toArray(), expect)
        expect[sl] = 7.0
        t.set(ranges, 7.0)
        assert np.array_equal(t.toArray(), expect)


def test_int_index_selects_the_leading_sub_tensor(oracle_ops):
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    t = oracle_ops.createRaw([2, 3, 4], a.reshape(-1))
    assert np.array_equal(t.get([1]).toArray(), a[1]) and t.get([1]).shape == [3, 4]
    assert np.array_equal(t.get([1, -1]).toArray(), a[1, 2]) and t.get([1, -1]).shape == [4]
    assert t.get([1, 2, 3]).shape == [1] and t.get([1, 2, 3]).toArray()[0] == a[1, 2, 3]      # ShapeFunctions.kt:236
    t.set([0, 1], oracle_ops.createRaw([2, 2], [9.0, 8.0, 7.0, 6.0]))      # only the element count is compared (JVM:284)
    assert t.toArray()[0, 1].tolist() == [9.0, 8.0, 7.0, 6.0]
    t.set([-1], -1.0)
    assert np.all(t.toArray()[1] == -1.0) and np.all(t.toArray()[0, 0] == a[0, 0])
    with pytest.raises(ValueError):
        t.set([0, 1], oracle_ops.createRaw([3], [1.0, 2.0, 3.0]))
    with pytest.raises(ValueError):
        t.get([2])
    with pytest.raises(ValueError):
        t.get([0, 0, 0, 0])


def test_range_normalisation_rules():
    # ShapeFunctions.kt:240-259 with the ranges the reference's tests use (TensorTestsBase.kt:157,217,1880)
    assert sf.normalize_range_index([3, 3, 3], [(1, 1), ALL, (1, -1)]) == [IntRange(1, 1), IntRange(0, 2), IntRange(1, 2)]
    assert sf.normalize_range_index([2, 4], [(-1, -1), (1, 2)]) == [IntRange(1, 1), IntRange(1, 2)]
    assert sf.normalized_range_indexed_shape([3, 3], [ALL, (1, -1)])[1] == [3, 2]
    assert sf.normalized_range_indexed_shape([4, 5, 6], [(1, 2)])[1] == [2, 5, 6]
    for bad in ([(2, 1)], [(0, 3)], [(-4, 0)], [(0, 0), (0, 0), (0, 0)]):
        with pytest.raises(ValueError):
            sf.normalize_range_index([3, 3], bad)
    assert sf.is_range_index([(0, 1)]) and sf.is_range_index([ALL]) and not sf.is_range_index([0, 1])


def test_sparse_store_ranges_drop_trailing_full_dims(oracle_ops):
    # AbstractIndexing.kt:67-73: [1..2, all, all] of [4, 3, 2] is ONE store range of 12 elements
    a = np.arange(24, dtype=np.float32)
    t = oracle_ops.createRaw([4, 3, 2], a)
    assert np.array_equal(t.get([(1, 2), ALL, ALL]).toArray().reshape(-1), a[6:18])
    assert jo.lib().kjo_range_size(jo._sh([4, 3, 2]), 3, jo._sh([1, 0, 0]), jo._sh([2, 2, 1])) == 12


def test_permute_equals_numpy_transpose():
    rng = np.random.default_rng(5)
    for nd in range(1, 6):
        shape = [int(rng.integers(1, 6)) for _ in range(nd)]
        a = rng.standard_normal(shape).astype(np.float32)
        for axes in itertools.islice(itertools.permutations(range(nd)), 30):
            assert np.array_equal(jo.permute(a, list(axes)), np.transpose(a, axes))


def test_jvm_transpose_is_the_axis_swap_exactly_when_the_slab_orders_agree():
    rng = np.random.default_rng(6)
    for shape in ([2, 3], [2, 3, 4], [3, 1, 4], [2, 3, 4, 5], [2, 1, 1, 5]):
        a = rng.standard_normal(shape).astype(np.float32)
        for a1, a2 in itertools.permutations(range(len(shape)), 2):
            lo, hi = min(a1, a2), max(a1, a2)
            between_is_one = all(s == 1 for s in shape[lo + 1:hi])
            same = np.array_equal(jo.transpose_jvm(a, a1, a2), np.swapaxes(a, a1, a2))
            if between_is_one:
                assert same, (shape, a1, a2)
    # the case where kten-jvm departs from the documented axis swap (and from its OpenCL backend)
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    assert not np.array_equal(jo.transpose_jvm(a, 0, 2), np.swapaxes(a, 0, 2))
    assert sorted(jo.transpose_jvm(a, 0, 2).reshape(-1).tolist()) == a.reshape(-1).tolist()


def test_masked_fill_selects_on_exactly_one(oracle_ops):
    a = np.array([[1.0, np.nan, 3.0], [4.0, 5.0, 6.0]], dtype=np.float32)
    mask = np.array([1.0, 0.0, 0.99999994], dtype=np.float32)
    got = jo.masked_fill(a, mask, -7.0)
    assert np.array_equal(got, np.where(np.broadcast_to(mask, a.shape) == 1.0, np.float32(-7.0), a), equal_nan=True)
    rng = np.random.default_rng(7)
    for shape, mshape in (([4, 5, 6], [5, 1]), ([4, 5, 6], [1]), ([4, 5, 6], [4, 5, 6]), ([3, 8], [3, 1])):
        x = rng.standard_normal(shape).astype(np.float32)
        m = (rng.random(mshape) < 0.4).astype(np.float32)
        t, mt = oracle_ops.createRaw(shape, x.reshape(-1)), oracle_ops.createRaw(mshape, m.reshape(-1))
        assert np.array_equal(t.maskedFill(mt, 2.5).toArray(), np.where(np.broadcast_to(m, shape) == 1.0, np.float32(2.5), x))
    with pytest.raises(ValueError):
        oracle_ops.createRaw([2, 3]).maskedFill(oracle_ops.createRaw([2, 2, 3]), 0.0)


def test_concat_and_narrow_equal_numpy(oracle_ops):
    rng = np.random.default_rng(8)
    for shape, axis, sizes in (([3, 4], 0, [1, 2, 3]), ([3, 4], 1, [4, 1]), ([2, 3, 4], -2, [2, 5]), ([5], 0, [1, 1, 7])):
        parts = []
        for s in sizes:
            sh = list(shape); sh[axis] = s
            parts.append(rng.standard_normal(sh).astype(np.float32))
        raws = [oracle_ops.createRaw(list(p.shape), p.reshape(-1)) for p in parts]
        got = oracle_ops.concat(axis, raws)
        want = np.concatenate(parts, axis=axis)
        assert got.shape == list(want.shape) and np.array_equal(got.toArray(), want)
        end = 0
        for p, s in zip(parts, sizes):
            assert np.array_equal(got.narrow(axis, end, s).toArray(), p)
            end += s
    with pytest.raises(ValueError):
        oracle_ops.concat(0, [oracle_ops.createRaw([2, 3]), oracle_ops.createRaw([2, 4])])
    with pytest.raises(ValueError):
        oracle_ops.concat(0, [oracle_ops.createRaw([2, 3]), oracle_ops.createRaw([3])])
    with pytest.raises(ValueError):
        oracle_ops.createRaw([2, 3]).narrow(1, 2, 2)


def test_index_select_and_index_add_equal_numpy(oracle_ops):
    rng = np.random.default_rng(12)
    for shape, axis, k in (([3, 3, 3], 1, 3), ([5, 7], 0, 9), ([5, 7], -1, 4), ([2, 3, 4, 5], 2, 6), ([6], 0, 10)):
        a = rng.standard_normal(shape).astype(np.float32)
        ax = axis % len(shape)
        idx = rng.integers(0, shape[ax], k)
        t, it = oracle_ops.createRaw(shape, a.reshape(-1)), oracle_ops.createRaw([k], idx.astype(np.float32))
        got = t.indexSelect(axis, it)
        want = np.take(a, idx, axis=ax)
        assert got.shape == list(want.shape) and np.array_equal(got.toArray(), want)
        # indexAdd with alpha 1 against np.add.at; repeated indices accumulate (small integers: exact in any order)
        src = rng.integers(-8, 8, want.shape).astype(np.float32)
        base = rng.integers(-8, 8, shape).astype(np.float32)
        t2 = oracle_ops.createRaw(shape, base.reshape(-1))
        t2.indexAdd(axis, it, oracle_ops.createRaw(list(src.shape), src.reshape(-1)), 2.0)
        want2 = base.copy()
        sl = [slice(None)] * len(shape)
        for i, sel in enumerate(idx):
            sl_t = list(sl); sl_t[ax] = sel
            sl_s = list(sl); sl_s[ax] = i
            want2[tuple(sl_t)] += src[tuple(sl_s)] * np.float32(2.0)
        assert np.array_equal(t2.toArray(), want2)
    t = oracle_ops.createRaw([2, 3], np.zeros(6, dtype=np.float32))
    with pytest.raises(ValueError):
        t.indexSelect(1, oracle_ops.createRaw([2], [0.0, 3.0]))                    # JVM:494-496
    with pytest.raises(ValueError):
        t.indexSelect(1, oracle_ops.createRaw([1, 2], [0.0, 1.0]))                 # the index must be 1-D
    with pytest.raises(ValueError):
        t.indexAdd(1, oracle_ops.createRaw([2], [0.0, 1.0]), oracle_ops.createRaw([2, 3], np.zeros(6, dtype=np.float32)))


def test_index_add_accumulates_in_index_order(oracle_ops):
    # 1e8 + 1 - 1e8 in float: the order of the three additions decides between 0 and 1 (JVM:511-513)
    t = oracle_ops.createRaw([1], [0.0])
    t.indexAdd(0, oracle_ops.createRaw([3], [0.0, 0.0, 0.0]), oracle_ops.createRaw([3], [1e8, 1.0, -1e8]))
    assert t.toArray()[0] == 0.0
    t = oracle_ops.createRaw([1], [0.0])
    t.indexAdd(0, oracle_ops.createRaw([3], [0.0, 0.0, 0.0]), oracle_ops.createRaw([3], [1e8, -1e8, 1.0]))
    assert t.toArray()[0] == 1.0


def test_inplace_resize_keeps_the_leading_values_and_pads_with_zeros(oracle_ops):
    """FloatArray.copyOf (JVMRawTensor.kt:528-531): the ones-buffer of the convolution code is
    resized this way (JVMSpatialConvolutionBase.kt:66)."""
    t = oracle_ops.createRaw([2, 3], np.arange(1, 7, dtype=np.float32))
    t.inplaceResize(3, 3)
    assert t.shape == [3, 3] and t.toList() == [1, 2, 3, 4, 5, 6, 0, 0, 0]
    t.inplaceResize([2, 2])
    assert t.shape == [2, 2] and t.toList() == [1, 2, 3, 4]
