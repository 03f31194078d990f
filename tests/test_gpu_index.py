"""gather / inplaceScatter / inplaceScatterAdd / inplaceScatter(Float) on the device against
the CPU checker: bit-exact, including duplicate indices inside a position (assignment:
last write wins; add: summed in ascending order) and the error behaviour."""
import numpy as np
import pytest

from kten_amd import abi

from oracle import jvm_oracle as jo
from parity import assert_bits_equal

pytestmark = pytest.mark.gpu

CASES = [([4, 5], [4, 3], 1), ([4, 5], [2, 5], 0), ([3, 4, 5], [3, 2, 5], 1), ([3, 4, 5], [2, 4, 2], 2), ([6], [9], 0),
         ([2, 3, 4, 5], [2, 3, 7, 5], 2), ([1000, 300], [1000, 1], 1), ([1000, 300], [1, 300], 0), ([64, 2048], [64, 1], 1),
         ([70000, 7], [70000, 3], 1), ([5, 3, 2, 2, 3, 2, 2, 2, 3, 4], [5, 3, 2, 2, 6, 2, 2, 2, 3, 4], 4),
         # long axes with many repeated indices (the last entry of a position wins)
         ([300, 400], [300, 400], 1), ([300, 400], [300, 400], 0), ([64, 2048], [64, 2048], 1), ([2048, 64], [2048, 40], 0),
         ([8, 100, 128], [8, 90, 128], 1), ([50, 33, 70], [50, 33, 64], 2), ([40, 10], [40, 2000], 1),
         # rows along the innermost axis that are scattered inside LDS: the size limits of the assign and add forms
         # and one past them, index dims smaller than the target's, one index value for a whole row
         ([3, 16384], [3, 5000], 1), ([3, 8192], [3, 3000], 1), ([2, 8193], [2, 2000], 1), ([2, 16385], [2, 4000], 1),
         ([2, 32768], [2, 5000], 1), ([2, 32769], [2, 5000], 1), ([3, 100001], [3, 40000], 1), ([70001, 6], [30000, 5], 0),
         ([10, 6, 300], [7, 4, 100], 2), ([5, 1], [5, 700], 1), ([1, 4096], [1, 4096], 1),
         # a long axis that is not the innermost: scattered as rows between two permutes
         ([4096, 96], [4096, 96], 0), ([2, 3000, 40], [2, 2500, 33], 1), ([8192, 3, 5], [8000, 2, 5], 0), ([5000, 7], [700, 7], 0),
         # gathered as rows between permutes too: a long outer or middle axis and an index about as large as the input
         ([3, 3000, 40], [3, 2600, 37], 1), ([9000, 33], [8000, 33], 0), ([2, 300, 5, 101], [2, 300, 5, 101], 1)]


def both(gc, shape, array):
    cpu = jo.JvmOracleOperations()
    return gc.createRaw(shape, array), cpu.createRaw(shape, array)


@pytest.mark.parametrize("shape,ishape,axis", CASES, ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_gather_scatter_parity(shape, ishape, axis, gc):
    rng = np.random.default_rng(sum(shape) + axis)
    x = rng.standard_normal(shape).astype(np.float32)
    idx = rng.integers(0, shape[axis], size=ishape).astype(np.float32)
    src = rng.standard_normal(ishape).astype(np.float32)
    gx, cx = both(gc, shape, x); gi, ci = both(gc, ishape, idx); gs, cs = both(gc, ishape, src)
    assert_bits_equal(gx.gather(axis, gi).toArray(), cx.gather(axis, ci).toArray(), "gather")
    for name in ("inplaceScatter", "inplaceScatterAdd"):
        gt, ct = both(gc, shape, x)
        getattr(gt, name)(axis, gi, gs); getattr(ct, name)(axis, ci, cs)
        assert_bits_equal(gt.toArray(), ct.toArray(), name)
    gt, ct = both(gc, shape, x)
    gt.inplaceScatter(axis, gi, -1.0); ct.inplaceScatter(axis, ci, -1.0)
    assert_bits_equal(gt.toArray(), ct.toArray(), "inplaceScatter(Float)")
    assert_bits_equal(gx.scatter(axis, gi, gs).toArray(), cx.scatter(axis, ci, cs).toArray(), "scatter (copy)")
    assert_bits_equal(gx.toArray(), x, "scatter must not touch its receiver")


def test_gather_along_an_outer_axis_goes_through_rows(gc):
    rng = np.random.default_rng(77)
    x = rng.standard_normal([5000, 70]).astype(np.float32)
    idx = rng.integers(0, 5000, size=[4500, 70]).astype(np.float32)
    gc.profileBegin()
    got = gc.createRaw([5000, 70], x).gather(0, gc.createRaw([4500, 70], idx)).toArray()
    kernels = gc.profileEnd()
    assert any(k.startswith("gather_rows_lds_kernel") for k in kernels) and any(k.startswith("permute") for k in kernels), sorted(kernels)
    assert_bits_equal(got, np.take_along_axis(x, idx.astype(np.int64), axis=0), "gather along axis 0")
    bad = idx.copy(); bad[17, 3] = 5000.0
    with pytest.raises(ValueError):
        gc.createRaw([5000, 70], x).gather(0, gc.createRaw([4500, 70], bad))


def test_copies_of_an_index_share_what_is_known_of_it_until_one_side_changes(gc):
    """A copy that the library has put off reads its source's memory: a check that passed on either side holds for both
    (a targets tensor that is unsqueezed every step is checked once, not once per step); a change to either side after
    the copy concerns that side alone."""
    rng = np.random.default_rng(8)
    x = rng.standard_normal([50, 40]).astype(np.float32)
    gx = gc.createRaw([50, 40], x)
    idx = rng.integers(0, 40, size=[50, 12]).astype(np.float32)
    want = np.take_along_axis(x, idx.astype(np.int64), axis=1)
    src = gc.createRaw([50, 12], idx)
    first = src.copy()
    assert_bits_equal(gx.gather(1, first).toArray(), want, "gather by a copy")            # checked here, for both
    assert_bits_equal(gx.gather(1, src).toArray(), want, "gather by the source")
    second = src.copy()                                                                    # inherits the record
    assert_bits_equal(gx.gather(1, second).toArray(), want, "gather by a later copy")
    # the source changes: the copies keep the old, valid values; the source is checked again and fails
    src._scalar_assign("plus", 30.0)
    assert_bits_equal(gx.gather(1, first).toArray(), want, "first copy after the source changed")
    assert_bits_equal(gx.gather(1, second).toArray(), want, "second copy after the source changed")
    with pytest.raises(ValueError):
        gx.gather(1, src)
    # a copy changes: it is checked again and fails; source and sibling are untouched
    src2 = gc.createRaw([50, 12], idx)
    assert_bits_equal(gx.gather(1, src2).toArray(), want, "gather by a second source")
    c1, c2 = src2.copy(), src2.copy()
    c1._set_store_range(7, 1, 40.0)
    with pytest.raises(ValueError):
        gx.gather(1, c1)
    assert_bits_equal(gx.gather(1, c2).toArray(), want, "sibling copy")
    assert_bits_equal(gx.gather(1, src2).toArray(), want, "second source")
    # a copy of invalid values is found invalid, and leaves no record on its source
    bad = idx.copy(); bad[3, 3] = 40.0
    sb = gc.createRaw([50, 12], bad)
    with pytest.raises(ValueError):
        gx.gather(1, sb.copy())
    with pytest.raises(ValueError):
        gx.gather(1, sb)


def test_an_index_checked_once_is_checked_again_after_any_change(gc):
    """An index tensor that an indexed move found valid is not checked again while nothing touches it; every
    way of changing it (a range fill, an upload, an in-place op, a copy into it, a kernel writing it as its result)
    and a shorter axis must bring the check back."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal([50, 40]).astype(np.float32)
    gx = gc.createRaw([50, 40], x)
    idx = rng.integers(0, 40, size=[50, 12]).astype(np.float32)
    want = np.take_along_axis(x, idx.astype(np.int64), axis=1)

    def fresh():
        gi = gc.createRaw([50, 12], idx)
        assert_bits_equal(gx.gather(1, gi).toArray(), want, "gather")          # checked here
        assert_bits_equal(gx.gather(1, gi).toArray(), want, "gather again")    # known to be valid
        return gi

    gi = fresh(); gi._set_store_range(7, 1, 40.0)
    with pytest.raises(ValueError):
        gx.gather(1, gi)
    gi = fresh(); gi._set_ranges([3, 2], [3, 2], -1.0)
    with pytest.raises(ValueError):
        gx.gather(1, gi)
    gi = fresh(); gi._scalar_assign("plus", 30.0)
    with pytest.raises(ValueError):
        gx.gather(1, gi)
    gi = fresh(); gi._binary_assign("times", gc.createRawFill([50, 12], 2.0))
    with pytest.raises(ValueError):
        gx.gather(1, gi)
    gi = fresh(); gi._set_store_range(0, 600, gc.createRawFill([600], 41.0))     # a copy into it
    with pytest.raises(ValueError):
        gx.gather(1, gi)
    gi = fresh(); gi.inplaceScatter(1, gc.createRaw([50, 1], np.zeros([50, 1], np.float32)), 99.0)   # written as a target
    with pytest.raises(ValueError):
        gx.gather(1, gi)
    # valid for an axis of 40, not for one of 30
    gi = fresh()
    with pytest.raises(ValueError):
        gc.createRaw([50, 30], x[:, :30].copy()).gather(1, gi)
    # and valid again for a longer one, for every kind of indexed move
    wide = gc.createRaw([50, 64], np.zeros([50, 64], np.float32))
    wide.inplaceScatterAdd(1, gi, gc.createRawFill([50, 12], 1.0))
    assert wide.toArray().sum() == 600.0
    # the positions ARG_MAX wrote are valid for the axis they came from; changed afterwards, they are checked again
    am = gx.argMax(1, True)
    t = gc.createRawFill([50, 40], 0.0)
    t.inplaceScatter(1, am, 1.0)
    assert_bits_equal(t.toArray().sum(1), np.ones([50], np.float32), "one-hot of the row maxima")
    am._scalar_assign("plus", 40.0)
    with pytest.raises(ValueError):
        t.inplaceScatter(1, am, 1.0)
    rows = gc.createRaw([20], rng.integers(0, 50, size=[20]).astype(np.float32))
    sel = gx.indexSelect(0, rows)
    acc = gc.createRawFill([50, 40], 0.0)
    acc.indexAdd(0, rows, sel, 1.0)                                           # the list was checked by indexSelect
    rows._set_store_range(19, 1, 50.0)
    with pytest.raises(ValueError):
        acc.indexAdd(0, rows, sel, 1.0)
    with pytest.raises(ValueError):
        gx.indexSelect(0, rows)


def test_bad_indices_raise_like_the_reference(gc):
    x = gc.createRaw([2, 3], np.arange(6, dtype=np.float32))
    for bad in (3.0, -1.0, 1e10):
        with pytest.raises(ValueError):
            x.gather(1, gc.createRaw([2, 1], [0.0, bad]))
        with pytest.raises(ValueError):
            x.inplaceScatter(1, gc.createRaw([2, 1], [0.0, bad]), gc.createRaw([2, 1], [1.0, 1.0]))
        with pytest.raises(ValueError):
            x.inplaceScatter(1, gc.createRaw([2, 1], [0.0, bad]), 5.0)
    got = x.gather(1, gc.createRaw([2, 1], [2.9, float("nan")])).toArray()         # Float.toInt(): 2 and 0
    assert got.tolist() == [[2.0], [3.0]]
    with pytest.raises(ValueError):
        x.inplaceScatter(1, gc.createRaw([2, 2], [0, 1, 0, 1]), gc.createRaw([2, 1], [1.0, 1.0]))
    with pytest.raises(ValueError):
        x.inplaceScatter(1, gc.createRaw([2], [0, 1]), gc.createRaw([2], [1.0, 1.0]))
    with pytest.raises(ValueError):
        x.gather(2, gc.createRaw([2, 1], [0.0, 0.0]))


def test_max_backward_at_scale_matches_checker(gc):
    """Max over the last axis with its scatter backward, and a softmax-cross-entropy step,
    on [512, 1000]: device against the checker running the same graph."""
    from kten_amd.host_mirror.inputs import SplitMix64
    g = SplitMix64(5)
    x = g.normal([512, 1000])
    labels = (g.uniform([512], 0.0, 1.0) * 1000).astype(np.int64).clip(0, 999).astype(np.float32)
    out = []
    for ops in (gc, jo.JvmOracleOperations()):
        t = ops.create([512, 1000], True, x)
        t.max(-1).sum().backward()
        g_max = t.grad().toArray().copy()
        t2 = ops.create([512, 1000], True, x)
        loss = t2.softmaxCrossEntropy(ops.create([512], False, labels))
        loss.backward()
        out.append((g_max, loss.toArray(), t2.grad().toArray()))
    assert_bits_equal(out[0][0], out[1][0], "grad of max")
    assert abs(float(out[0][1][0]) - float(out[1][1][0])) <= 1e-6 * abs(float(out[1][1][0]))
    np.testing.assert_allclose(out[0][2], out[1][2], rtol=0, atol=1e-9)


ROW_CASES = [([3, 3, 3], 1, 3), ([5, 7], 0, 9), ([5, 7], -1, 4), ([2, 3, 4, 5], 2, 6), ([6], 0, 10), ([1000, 64], 0, 5000),
             ([50, 300, 8], 1, 700), ([4096, 33], 0, 100), ([7, 9, 130], 0, 20), ([64, 1000], 1, 256),
             # lists of 64 entries or more are sorted on the device: the threshold, long runs of one target row,
             # a flat tensor, a short middle axis, columns that are not a multiple of 4
             ([9, 7], 0, 63), ([9, 7], 0, 64), ([3, 40], 0, 5000), ([2, 5, 3], 1, 1000), ([100000], 0, 300000),
             ([20, 4100], 1, 9000), ([1, 2, 1], 1, 4097),
             # the device's own radix sort: one, two and three 8-bit passes (axes of up to 256, 65 536 and more rows),
             # lists of less than a tile of 4096 pairs, of many tiles, and of more than 65 536 histogram entries
             # (the scan in three kernels), values whose sums depend on the order of the adds
             ([200], 0, 100000), ([256, 2], 0, 70001), ([257], 0, 4095), ([60000], 0, 4097), ([65536], 0, 200000),
             ([65537, 1], 0, 1200000), ([1000003], 0, 1100000), ([3, 70000], 1, 300001)]


@pytest.mark.parametrize("shape,axis,k", ROW_CASES, ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_index_select_and_index_add_parity(shape, axis, k, gc):
    rng = np.random.default_rng(sum(shape) + k)
    ax = axis % len(shape)
    x = rng.standard_normal(shape).astype(np.float32)
    idx = rng.integers(0, shape[ax], [k]).astype(np.float32)
    gx, cx = both(gc, shape, x); gi, ci = both(gc, [k], idx)
    got, want = gx.indexSelect(axis, gi), cx.indexSelect(axis, ci)
    assert got.shape == want.shape
    assert_bits_equal(got.toArray(), want.toArray(), "indexSelect")
    src = rng.standard_normal(want.shape).astype(np.float32)
    src *= np.exp(rng.uniform(-12, 12, src.shape)).astype(np.float32)      # sums that depend on the order of the adds
    gs, cs = both(gc, want.shape, src)
    for alpha in (1.0, -0.3):
        gt, ct = both(gc, shape, x)
        gt.indexAdd(axis, gi, gs, alpha); ct.indexAdd(axis, ci, cs, alpha)
        assert_bits_equal(gt.toArray(), ct.toArray(), f"indexAdd alpha {alpha} (repeated indices accumulate in index order)")


@pytest.mark.parametrize("shape,i_len,spread", [([300, 5000], 200, 5000), ([300, 5000], 200, 8), ([300, 5000], 200, 1), ([40, 70000], 100, 70000),
                                                ([40, 70000], 333, 3), ([7, 3, 900], 65, 40), ([1000, 600], 32, 600), ([5, 100000], 1000, 2)],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_scatter_by_a_wave_per_row_with_repeated_elements(shape, i_len, spread, gc):
    """Index rows of 32 entries or more along the innermost axis that are too short (or whose target rows are too long)
    for the rows-through-LDS kernel: a wave per row, 64 entries a step. `spread` is how many different elements a row's
    entries name: with few, most lanes of a step share their element and the order of the adds and the last entry
    of an assignment are decided inside the wave."""
    rng = np.random.default_rng(sum(shape) + i_len + spread)
    cpu = jo.JvmOracleOperations()
    ishape = list(shape); ishape[-1] = i_len
    x = rng.standard_normal(shape).astype(np.float32)
    idx = (rng.integers(0, spread, ishape) * (shape[-1] // spread)).astype(np.float32)
    src = rng.standard_normal(ishape).astype(np.float32)
    src *= np.exp(rng.uniform(-12, 12, src.shape)).astype(np.float32)      # sums that depend on the order of the adds
    gi, ci = gc.createRaw(ishape, idx), cpu.createRaw(ishape, idx)
    gs, cs = gc.createRaw(ishape, src), cpu.createRaw(ishape, src)
    gc.profileBegin()
    for name, source in (("inplaceScatter", (gs, cs)), ("inplaceScatterAdd", (gs, cs)), ("inplaceScatter", (2.5, 2.5))):
        gt, ct = gc.createRaw(shape, x), cpu.createRaw(shape, x)
        getattr(gt, name)(-1, gi, source[0]); getattr(ct, name)(-1, ci, source[1])
        assert_bits_equal(gt.toArray(), ct.toArray(), f"{name} {'constant' if source[0] == 2.5 else 'tensor'}")
    names = set(gc.profileEnd())
    assert {"scatter_wave_kernel<set>", "scatter_wave_kernel<add>", "scatter_wave_kernel<fill>"} <= names, names


@pytest.mark.parametrize("shape,axis,i_len,spread,sorted_form", [
    ([100000], 0, 300000, 100000, True), ([100000], 0, 300000, 3, True), ([1 << 20], 0, 70001, 1 << 20, True),
    ([50000, 7], 0, 400000, 50000, None), ([6, 1, 90000], 2, 300000, 17, None), ([3, 40000, 2], 1, 100000, 40000, None),
    ([2, 300000], 1, 500000, 300000, True), ([400], 0, 100000, 400, False)],
    ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_scatter_of_long_rows_at_few_positions_goes_through_a_sort(shape, axis, i_len, spread, sorted_form, gc):
    """A handful of positions with index rows of 70 000 to 500 000 entries: the entries are sorted by the element they
    fall on, an assignment takes the last entry of each run, an add all of them in order. `spread` different elements
    are named per row: with few, the runs are long (hundreds of thousands of entries on one element)."""
    rng = np.random.default_rng(sum(shape) + i_len + spread)
    cpu = jo.JvmOracleOperations()
    ishape = list(shape); ishape[axis] = i_len
    x = rng.standard_normal(shape).astype(np.float32)
    idx = (rng.integers(0, spread, ishape) * (shape[axis] // spread)).astype(np.float32)
    src = rng.standard_normal(ishape).astype(np.float32)
    src *= np.exp(rng.uniform(-12, 12, src.shape)).astype(np.float32)      # sums that depend on the order of the adds
    gi, ci = gc.createRaw(ishape, idx), cpu.createRaw(ishape, idx)
    gs, cs = gc.createRaw(ishape, src), cpu.createRaw(ishape, src)
    gc.profileBegin()
    for name, source in (("inplaceScatter", (gs, cs)), ("inplaceScatterAdd", (gs, cs)), ("inplaceScatter", (2.5, 2.5))):
        gt, ct = gc.createRaw(shape, x), cpu.createRaw(shape, x)
        getattr(gt, name)(axis, gi, source[0]); getattr(ct, name)(axis, ci, source[1])
        assert_bits_equal(gt.toArray(), ct.toArray(), f"{name} {'constant' if source[0] == 2.5 else 'tensor'}")
        # a target that is a constant not yet written out
        gz, cz = gc.createRawFill(shape, -0.0), cpu.createRawFill(shape, -0.0)
        getattr(gz, name)(axis, gi, source[0]); getattr(cz, name)(axis, ci, source[1])
        assert_bits_equal(gz.toArray(), cz.toArray(), f"{name} into a fill")
    names = set(gc.profileEnd())
    if sorted_form is not None:           # (None: whichever the cost estimate picks; a short target row is cheaper walked)
        assert ("scatter_sort" in names) == sorted_form, names
    # a value out of range is refused, the tensor stays usable
    bad = idx.copy(); bad.reshape(-1)[i_len // 2] = float(shape[axis])
    t = gc.createRaw(shape, x)
    with pytest.raises(ValueError):
        t.inplaceScatterAdd(axis, gc.createRaw(ishape, bad), gs)
    t.inplaceFill(1.0)
    assert t.getSingleValue([0] * len(shape)) == 1.0


@pytest.mark.parametrize("shape,i_len,hot", [([40, 3000], 3000, 0.3), ([40, 3000], 9000, 0.9), ([300, 8192], 4096, 0.25), ([12, 16384], 20000, 0.5),
                                             ([6, 40000], 30000, 0.2), ([3, 5, 9000], 5000, 1.0), ([50, 700], 700, 0.05)],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_scatter_add_through_lds_rows_with_a_hot_element(shape, i_len, hot, gc):
    """The add form of the rows-through-LDS scatter retires one entry per element and round; with an element that a
    large share of a row's entries name (a histogram with a full bin) it hands over, after a few rounds, to the waves
    taking turns over what is left. `hot` is the share of the entries that name element 7 (the rest are uniform);
    rows of 256-thread and of 1024-thread workgroups, one band and several, indexAdd along the innermost axis too."""
    rng = np.random.default_rng(sum(shape) + i_len)
    cpu = jo.JvmOracleOperations()
    ishape = list(shape); ishape[-1] = i_len
    x = rng.standard_normal(shape).astype(np.float32)
    idx = rng.integers(0, shape[-1], ishape)
    idx[rng.random(ishape) < hot] = 7
    idx = idx.astype(np.float32)
    src = rng.standard_normal(ishape).astype(np.float32)
    src *= np.exp(rng.uniform(-12, 12, src.shape)).astype(np.float32)      # sums that depend on the order of the adds
    gi, ci = gc.createRaw(ishape, idx), cpu.createRaw(ishape, idx)
    gs, cs = gc.createRaw(ishape, src), cpu.createRaw(ishape, src)
    gc.profileBegin()
    gt, ct = gc.createRaw(shape, x), cpu.createRaw(shape, x)
    gt.inplaceScatterAdd(-1, gi, gs); ct.inplaceScatterAdd(-1, ci, cs)
    assert_bits_equal(gt.toArray(), ct.toArray(), "scatterAdd")
    gz, cz = gc.createRawFill(shape, -0.0), cpu.createRawFill(shape, -0.0)
    gz.inplaceScatterAdd(-1, gi, gs); cz.inplaceScatterAdd(-1, ci, cs)
    assert_bits_equal(gz.toArray(), cz.toArray(), "scatterAdd into a fill")
    assert "scatter_rows_lds_kernel<add>" in set(gc.profileEnd())
    # indexAdd along the innermost axis: one list for every row
    rows = idx.reshape(-1, i_len)[0]
    sshape = list(shape); sshape[-1] = i_len
    gr, cr = gc.createRaw([i_len], rows), cpu.createRaw([i_len], rows)
    gt, ct = gc.createRaw(shape, x), cpu.createRaw(shape, x)
    gt.indexAdd(-1, gr, gs, 0.7); ct.indexAdd(-1, cr, cs, 0.7)
    assert_bits_equal(gt.toArray(), ct.toArray(), "indexAdd along the innermost axis")


def skewed_rows(rng, n_rows, k, hot):
    """k row numbers below n_rows of which the share `hot` names row 3 % n_rows, the others uniform."""
    idx = rng.integers(0, n_rows, [k])
    idx[rng.random(k) < hot] = 3 % n_rows
    return idx.astype(np.float32)


# target shape, axis, list length, share of the list that names one hot row. Runs of 256 entries or more of one target row are
# added by a workgroup whose sixteen waves take turns over 32 entries each (512 a round): run lengths around the
# threshold, around one round and several, rows of 1, 3, 64, 65, 256 and 1023 floats, an outer index, rows that
# only the hot run touches, and lists in which every run is long.
LONG_RUN_CASES = [([7], 0, 300, 0.9), ([40], 0, 20000, 0.5), ([5, 64], 0, 2000, 0.3), ([5, 65], 0, 2600, 0.6), ([300, 256], 0, 9000, 0.2),
                  ([3, 1023], 0, 1500, 0.0), ([2, 6, 3], 1, 4000, 0.4), ([3, 50, 8], 1, 30000, 0.7), ([64, 1], 0, 100000, 0.25),
                  ([1, 100], 0, 255, 0.0), ([1, 100], 0, 256, 0.0), ([1, 100], 0, 257, 0.0), ([1, 100], 0, 511, 0.0), ([1, 100], 0, 512, 0.0),
                  ([1, 100], 0, 513, 0.0), ([1, 100], 0, 1024, 0.0), ([1, 100], 0, 1025, 0.0), ([1, 100], 0, 1056, 0.0), ([2, 4], 0, 1537, 0.0),
                  ([1000, 128], 0, 60000, 0.5), ([12, 2048], 0, 12000, 0.1),
                  # few positions beside the axis: a wave per (run, position), 64 entries at a time; run lengths around the multiples of 64
                  ([1, 2], 0, 256, 0.0), ([1, 2], 0, 257, 0.0), ([1, 2], 0, 319, 0.0), ([1, 2], 0, 320, 0.0), ([1, 2], 0, 321, 0.0), ([1], 0, 1025, 0.0),
                  ([2, 1, 16], 1, 700, 0.0), ([3, 16], 0, 50000, 0.6), ([3, 17], 0, 50000, 0.6), ([9], 0, 300000, 0.8), ([2, 5, 2], 1, 70000, 0.5)]


@pytest.mark.parametrize("shape,axis,k,hot", LONG_RUN_CASES, ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_index_add_with_long_runs(shape, axis, k, hot, gc):
    rng = np.random.default_rng(sum(shape) * 7 + k)
    cpu = jo.JvmOracleOperations()
    x = rng.standard_normal(shape).astype(np.float32)
    idx = skewed_rows(rng, shape[axis], k, hot)
    sshape = list(shape); sshape[axis] = k
    src = rng.standard_normal(sshape).astype(np.float32)
    src *= np.exp(rng.uniform(-12, 12, src.shape)).astype(np.float32)      # sums that depend on the order of the adds
    src[rng.random(src.shape) < 0.01] = -0.0
    gi, ci = gc.createRaw([k], idx), cpu.createRaw([k], idx)
    gs, cs = gc.createRaw(sshape, src), cpu.createRaw(sshape, src)
    for alpha in (1.0, -0.3):
        gt, ct = gc.createRaw(shape, x), cpu.createRaw(shape, x)
        gt.indexAdd(axis, gi, gs, alpha); ct.indexAdd(axis, ci, cs, alpha)
        assert_bits_equal(gt.toArray(), ct.toArray(), f"indexAdd alpha {alpha}")
        # into a target that is a constant nobody has written out (-0.0: 0 + s would lose the sign of a -0 sum)
        for constant in (0.0, -0.0, 1.5):
            gz, cz = gc.createRawFill(shape, constant), cpu.createRawFill(shape, constant)
            gz.indexAdd(axis, gi, gs, alpha); cz.indexAdd(axis, ci, cs, alpha)
            assert_bits_equal(gz.toArray(), cz.toArray(), f"indexAdd into a fill of {constant}, alpha {alpha}")


def test_index_add_long_run_with_a_bad_entry(gc):
    """A list whose runs are long and that holds values out of range: the call is refused, and the valid entries that
    were added before the refusal leave a tensor that still works."""
    idx = np.zeros(5000, dtype=np.float32); idx[1000:3000] = 1.0; idx[4000] = 9.0; idx[4500] = -2.0
    t = gc.createRaw([2, 16], np.zeros(32, dtype=np.float32))
    with pytest.raises(ValueError):
        t.indexAdd(0, gc.createRaw([5000], idx), gc.createRaw([5000, 16], np.ones(80000, dtype=np.float32)))
    t.inplaceFill(1.0)
    assert t.toList() == [1.0] * 32


def test_index_select_errors(gc):
    x = gc.createRaw([2, 3], np.arange(6, dtype=np.float32))
    for bad in (3.0, -1.0):
        with pytest.raises(ValueError):
            x.indexSelect(1, gc.createRaw([2], [0.0, bad]))
        with pytest.raises(ValueError):
            x.indexAdd(1, gc.createRaw([2], [0.0, bad]), gc.createRaw([2, 2], np.ones(4, dtype=np.float32)))
    with pytest.raises(ValueError):
        x.indexSelect(1, gc.createRaw([1, 2], [0.0, 1.0]))
    with pytest.raises(ValueError):
        x.indexAdd(1, gc.createRaw([2], [0.0, 1.0]), gc.createRaw([2, 3], np.ones(6, dtype=np.float32)))
    t = gc.createRaw([1], [0.0])
    t.indexAdd(0, gc.createRaw([3], [0.0, 0.0, 0.0]), gc.createRaw([3], [1e8, 1.0, -1e8]))
    assert t.toArray()[0] == 0.0
    # the same on a list long enough to be sorted: the order of the adds still decides the result
    idx = np.zeros(300, dtype=np.float32)
    vals = np.tile(np.array([1e8, 1.0, -1e8], dtype=np.float32), 100)
    t = gc.createRaw([2], [0.0, 5.0])
    t.indexAdd(0, gc.createRaw([300], idx), gc.createRaw([300], vals))
    assert t.toList() == [0.0, 5.0]
    # a bad value in a long list is reported, and the tensor stays usable
    idx[150] = 2.0
    with pytest.raises(ValueError):
        t.indexAdd(0, gc.createRaw([300], idx), gc.createRaw([300], vals))
    idx[150] = np.nan                                           # toInt() of NaN is 0
    t2 = gc.createRaw([2], [0.0, 5.0])
    t2.indexAdd(0, gc.createRaw([300], idx), gc.createRaw([300], vals))
    assert t2.toList() == [0.0, 5.0]


def test_index_add_full_size_round_trip(gc):
    """At the benchmark's [16384, 4096]: adding the rows of src into a zero tensor at a permutation
    of the rows, then selecting by the same permutation, gives src back bit for bit (0 + s * 1 = s
    for every s that is not -0); with every row sent to one target row the result is the serial
    float sum of the rows in order."""
    rows, cols = 16384, 4096
    rng = np.random.default_rng(5)
    src = rng.standard_normal((rows, cols)).astype(np.float32)
    src[src == 0] = 1.0
    perm = rng.permutation(rows).astype(np.float32)
    s = gc.createRaw([rows, cols], src)
    p = gc.createRaw([rows], perm)
    t = gc.createRawFill([rows, cols], 0.0)
    t.indexAdd(0, p, s)
    back = t.indexSelect(0, p)
    assert_bits_equal(back.toArray(), src, "indexSelect(indexAdd(0, perm, src), perm)")
    # along the last axis, the same with a permutation of the columns
    pc = gc.createRaw([cols], rng.permutation(cols).astype(np.float32))
    t2 = gc.createRawFill([rows, cols], 0.0)
    t2.indexAdd(1, pc, s)
    assert_bits_equal(t2.indexSelect(1, pc).toArray(), src, "the same along the last axis")
    # 4096 rows into one: the adds happen in list order
    few = 4096
    one = gc.createRawFill([2, cols], 0.0)
    one.indexAdd(0, gc.createRawFill([few], 1.0), gc.createRaw([few, cols], src[:few]))
    want = np.zeros(cols, dtype=np.float32)
    for r in range(few):
        want = want + src[r]
    got = one.toArray()
    assert_bits_equal(got[1], want, "serial float sum of the rows, in order")
    assert not got[0].any()


def test_scatter_rows_with_a_larger_source_and_bad_values(gc):
    """The source may be larger than the index in every dim (only the index's extent is read), and
    an index value outside the axis is reported from the LDS form as from the serial one, with the
    valid entries applied."""
    rng = np.random.default_rng(11)
    shape, ishape, sshape = [6, 500], [4, 300], [5, 450]
    x = rng.standard_normal(shape).astype(np.float32)
    idx = rng.integers(0, 500, size=ishape).astype(np.float32)
    src = rng.standard_normal(sshape).astype(np.float32)
    for name in ("inplaceScatter", "inplaceScatterAdd"):
        gt, ct = both(gc, shape, x)
        gi, ci = both(gc, ishape, idx); gs, cs = both(gc, sshape, src)
        getattr(gt, name)(1, gi, gs); getattr(ct, name)(1, ci, cs)
        assert_bits_equal(gt.toArray(), ct.toArray(), name + " with a larger source")
    bad = idx.copy(); bad[2, 17] = 500.0; bad[0, 299] = -3.0
    for name in ("inplaceScatter", "inplaceScatterAdd"):
        gt = gc.createRaw(shape, x)
        with pytest.raises(ValueError):
            getattr(gt, name)(1, gc.createRaw(ishape, bad), gc.createRaw(sshape, src))
    gt = gc.createRaw(shape, x)
    with pytest.raises(ValueError):
        gt.inplaceScatter(1, gc.createRaw(ishape, bad), 2.0)
    with pytest.raises(ValueError):
        gc.createRaw(shape, x).gather(1, gc.createRaw(ishape, bad))
    assert_bits_equal(gc.createRaw(shape, x).gather(1, gc.createRaw(ishape, idx)).toArray(),
                      np.take_along_axis(x[:4], idx.astype(np.int64), 1), "gather of long rows after a reported error")
    ok = gc.createRaw(shape, x)
    ok.inplaceScatter(1, gc.createRaw(ishape, idx), 2.0)          # the library is still usable
    want = x.copy()
    for r in range(4):
        want[r, idx[r].astype(int)] = 2.0
    assert_bits_equal(ok.toArray(), want, "fill after a reported error")


@pytest.mark.parametrize("shape,ishape", [([4, 4096], [4, 6000]), ([2, 12000], [2, 9000]), ([1, 12000], [1, 3000]), ([3, 40000], [3, 20000])],
                         ids=lambda v: "x".join(map(str, v)))
def test_scatter_add_with_hot_elements(shape, ishape, gc):
    """Index rows in which a few elements take most of the entries (and one row that names a single element):
    the adds of one element happen one per round in index order, over hundreds of rounds per chunk, in the
    256- and the 1024-thread form and in bands. Bit-exact against the serial order of the checker."""
    rng = np.random.default_rng(shape[1])
    x = rng.standard_normal(shape).astype(np.float32)
    hot = rng.integers(0, shape[1], size=4)
    idx = np.where(rng.random(ishape) < 0.7, hot[rng.integers(0, 4, size=ishape)], rng.integers(0, shape[1], size=ishape)).astype(np.float32)
    idx[0, :] = float(hot[0]) if shape[0] > 1 else idx[0, :]
    if shape[0] == 1:
        idx[0, : ishape[1] // 2] = 7.0
    src = (rng.standard_normal(ishape) * 100).astype(np.float32)          # large spread: the order of the adds shows in the last bits
    for name in ("inplaceScatterAdd", "inplaceScatter"):
        gt, ct = both(gc, shape, x)
        gi, ci = both(gc, ishape, idx); gs, cs = both(gc, ishape, src)
        getattr(gt, name)(1, gi, gs); getattr(ct, name)(1, ci, cs)
        assert_bits_equal(gt.toArray(), ct.toArray(), name)
    # the same list of hot rows through indexAdd on a vector (inner size 1: the same rounds, with a factor)
    rows = idx[0]
    add = src[0]
    gt, ct = both(gc, [shape[1]], x[0]); gr, cr = both(gc, [ishape[1]], rows); ga, ca = both(gc, [ishape[1]], add)
    gt.indexAdd(0, gr, ga, 0.3); ct.indexAdd(0, cr, ca, 0.3)
    assert_bits_equal(gt.toArray(), ct.toArray(), "indexAdd on a vector")


def test_deferred_index_check_reports_at_the_next_blocking_call(gc):
    """kth_set_index_check(0): an indexed move with an index outside its axis does not wait and returns OK; the next
    blocking call reports it, once; valid entries before the bad one are applied, the bad one is skipped."""
    lib = gc.lib
    x = gc.createRaw([2, 3], np.arange(6, dtype=np.float32))
    good = gc.createRaw([2], [0.0, 2.0]); bad = gc.createRaw([2], [1.0, 3.0])
    src = gc.createRaw([2, 2], np.ones(4, dtype=np.float32))
    abi.check(lib.kth_set_index_check(0))
    try:
        launches = gc.getMetrics()["launches"]
        x.indexAdd(1, bad, src)                      # no error here
        sel = x.indexSelect(1, good)                 # nor here: the flag is reported by a blocking call, not by the next op
        assert gc.getMetrics()["launches"] > launches
        with pytest.raises(ValueError, match="invalid index"):
            gc.sync()
        gc.sync()                                    # reported once
        np.testing.assert_array_equal(x.toArray(), np.array([[0, 2, 2], [3, 5, 5]], dtype=np.float32))
        np.testing.assert_array_equal(sel.toArray(), np.array([[0, 2], [3, 5]], dtype=np.float32))
        x.indexAdd(1, bad, src)
        with pytest.raises(ValueError, match="invalid index"):
            x.toArray()                              # a download reports it too
        x.indexAdd(1, bad, src)
        with pytest.raises(ValueError, match="invalid index"):
            x.containsNan()                          # and so does the NaN scan, which blocks as well
        assert x.containsNan() is False              # reported once
    finally:
        abi.check(lib.kth_set_index_check(1))
    with pytest.raises(ValueError):
        x.indexAdd(1, bad, src)                      # immediate again
