"""Layout movers on the device against the CPU checker, bit-exact: get / set / fill by
index and by ranges, narrow, concat, transpose, permute, maskedFill; float4 and scalar
forms, tile edges, error behaviour, and size-independent properties at large sizes."""
import ctypes
import itertools

import numpy as np
import pytest

from kten_amd import abi
from kten_amd.host_mirror.shape_functions import ALL
from oracle import jvm_oracle as jo
from parity import assert_bits_equal

pytestmark = pytest.mark.gpu


def both(gc, array):
    shape = list(array.shape)
    return gc.createRaw(shape, array), jo.JvmOracleOperations().createRaw(shape, array.reshape(-1))


def boxes(rng, shape, count):
    out = []
    for _ in range(count):
        k = int(rng.integers(1, len(shape) + 1))
        out.append([(f, int(rng.integers(f, shape[d]))) for d in range(k) for f in [int(rng.integers(0, shape[d]))]])
    return out


SHAPES = [[7], [4096], [5, 9], [64, 256], [33, 1024], [3, 4, 5], [6, 16, 64], [2, 3, 4, 5], [4, 8, 12, 16],
          [2, 3, 2, 3, 2, 3], [1, 1, 8], [300, 700]]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_range_get_set_fill_parity(shape, gc):
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    aligned = [[(0, shape[0] - 1)] + [(0, s - 1) if s % 4 else (4 * (s // 8), s - 1) for s in shape[1:]]]
    for box in boxes(rng, shape, 12) + aligned + [[ALL] * len(shape)]:
        g, c = both(gc, x)
        got, want = g.get(box), c.get(box)
        assert got.shape == want.shape
        assert_bits_equal(got.toArray(), want.toArray(), f"get {box}")
        v = rng.standard_normal(want.shape).astype(np.float32)
        gv, cv = both(gc, v)
        g.set(box, gv); c.set(box, cv)
        assert_bits_equal(g.toArray(), c.toArray(), f"set {box}")
        g.set(box, -3.5); c.set(box, -3.5)
        assert_bits_equal(g.toArray(), c.toArray(), f"fill {box}")


def test_int_index_get_set_parity(gc):
    x = np.arange(2 * 3 * 40, dtype=np.float32).reshape(2, 3, 40)
    for index in ([1], [-1, 2], [0, -1, 39], [1, 0]):
        g, c = both(gc, x)
        assert g.get(index).shape == c.get(index).shape
        assert_bits_equal(g.get(index).toArray(), c.get(index).toArray(), f"get {index}")
        v = np.full(c.get(index).shape, 0.5, dtype=np.float32)
        gv, cv = both(gc, v)
        g.set(index, gv); c.set(index, cv)
        assert_bits_equal(g.toArray(), c.toArray(), f"set {index}")
        g.set(index, 9.0); c.set(index, 9.0)
        assert_bits_equal(g.toArray(), c.toArray(), f"fill {index}")


def test_indexing_errors_match_the_reference(gc):
    x = gc.createRaw([3, 4], np.zeros(12, dtype=np.float32))
    for bad in ([(0, 4)], [(2, 1)], [(0, 0), (0, 0), (0, 0)], [(-5, 0)]):
        with pytest.raises(ValueError):
            x.get(bad)
        with pytest.raises(ValueError):
            x.set(bad, 1.0)
    with pytest.raises(ValueError):
        x.get([3])
    with pytest.raises(ValueError):
        x.set([(0, 1), (0, 1)], gc.createRaw([3], [1.0, 2.0, 3.0]))          # JVM:295-296 element count
    with pytest.raises(ValueError):
        x.set([1], gc.createRaw([3], [1.0, 2.0, 3.0]))                       # JVM:284-285
    x.set([(0, 1), (0, 1)], gc.createRaw([4], [1.0, 2.0, 3.0, 4.0]))         # only the count matters
    assert x.toArray()[:2, :2].reshape(-1).tolist() == [1.0, 2.0, 3.0, 4.0]
    with pytest.raises(ValueError):
        x.narrow(1, 3, 2)
    with pytest.raises(ValueError):
        x.transpose(1, -1)
    with pytest.raises(ValueError):
        x.permute([0, 0])
    with pytest.raises(ValueError):
        x.permute([0, 1, 2])
    with pytest.raises(ValueError):
        x.maskedFill(gc.createRaw([3], [1.0, 0.0, 1.0]), 0.0)
    with pytest.raises(ValueError):
        gc.concat(0, [x, gc.createRaw([3, 5], np.zeros(15, dtype=np.float32))])


TRANSPOSE_SHAPES = [[2, 3], [64, 64], [65, 63], [1, 7], [130, 257], [3, 5, 7], [2, 64, 128], [4, 3, 66, 70], [2, 3, 4, 5, 6],
                    [3, 1, 129], [1000, 3], [3, 1000]]


@pytest.mark.parametrize("shape", TRANSPOSE_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_transpose_every_axis_pair(shape, gc):
    x = np.random.default_rng(len(shape) + shape[-1]).standard_normal(shape).astype(np.float32)
    g, c = both(gc, x)
    for a1, a2 in itertools.permutations(range(len(shape)), 2):
        got = g.transpose(a1, a2)
        assert got.shape == list(np.swapaxes(x, a1, a2).shape)
        assert_bits_equal(got.toArray(), np.swapaxes(x, a1, a2), f"transpose({a1},{a2}) vs the axis swap")
        lo, hi = min(a1, a2), max(a1, a2)
        if all(s == 1 for s in shape[lo + 1:hi]):
            # where kten-jvm's slab copy is the axis swap, the device equals the restatement of kten-jvm
            assert_bits_equal(got.toArray(), c.transpose(a1, a2).toArray(), f"transpose({a1},{a2}) vs kten-jvm")
    assert_bits_equal(g.transpose(-1, 0).toArray(), np.swapaxes(x, -1, 0), "negative axis")


PERMUTE_SHAPES = [[2, 3, 2], [5, 6, 7], [8, 64, 68], [2, 3, 4, 5], [3, 4, 64, 65], [4, 16, 20, 24], [2, 2, 3, 3, 4, 4],
                  [128, 3], [6, 1, 5, 1],
                  # float4 / float2 elements kept innermost; batched small slabs; narrow tiles with ragged edges
                  [20, 33, 4], [17, 40, 2], [3, 18, 21, 4], [50, 6, 7], [1000, 16, 4], [70, 3, 100], [5, 9, 130, 3],
                  # a run of 5 ... 63 floats kept innermost: tiles of runs (float4 and scalar), ragged tile edges, exact tiles,
                  # a batch dim outside, a merged run ([.., 3, 4] -> 12), dims too short for a tile (the strided move instead)
                  [40, 50, 8], [33, 47, 12], [20, 35, 7], [18, 70, 33], [3, 17, 19, 5], [16, 16, 31], [19, 23, 3, 4], [100, 9, 6],
                  [9, 10, 63], [16, 48, 28], [40, 70, 3], [33, 35, 3], [2, 32, 32, 3],
                  # a short contiguous dim of the input (or of the output) whose neighbour there goes elsewhere: the two as one
                  # tile dim; both contiguous dims short with no neighbour to join: the element gather instead of mostly empty tiles
                  [300, 26, 3], [30, 8, 19, 8], [40, 7, 11, 23], [322, 14, 2, 5], [26, 17, 19, 4], [5, 5, 66, 23], [70, 3, 2, 90],
                  # three dims as one tile dim; joined dims in tiles of runs and of float2 / float4 elements
                  [155, 19, 3, 3], [3, 3, 19, 155], [470, 31, 3, 6], [3, 31, 470, 6], [60, 5, 7, 4], [90, 3, 3, 3, 2], [37, 3, 5, 2, 12],
                  [3, 2, 3, 200, 5]]


@pytest.mark.parametrize("shape", PERMUTE_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_permute_parity(shape, gc):
    x = np.random.default_rng(shape[0] * 31 + len(shape)).standard_normal(shape).astype(np.float32)
    g, c = both(gc, x)
    perms = list(itertools.permutations(range(len(shape))))
    if len(perms) > 40:
        perms = [perms[i] for i in np.random.default_rng(1).choice(len(perms), 40, replace=False)]
    for axes in perms:
        got, want = g.permute(list(axes)), c.permute(list(axes))
        assert got.shape == want.shape
        assert_bits_equal(got.toArray(), want.toArray(), f"permute{axes}")


def test_masked_fill_parity(gc):
    rng = np.random.default_rng(3)
    for shape, mshape in (([4, 5, 6], [5, 1]), ([4, 5, 6], [1]), ([4, 5, 8], [4, 5, 8]), ([32, 16, 8, 8], [16, 1, 1]),
                          ([1000, 7], [1000, 1]), ([128, 256], [256]), ([9], [9])):
        x = rng.standard_normal(shape).astype(np.float32)
        x.reshape(-1)[::7] = np.nan
        m = rng.choice(np.array([0.0, 1.0, 0.99999994, 2.0, np.nan, -1.0], dtype=np.float32), size=mshape)
        g, c = both(gc, x); gm, cm = both(gc, m)
        for value in (0.0, -2.5, float("inf")):
            assert_bits_equal(g.maskedFill(gm, value).toArray(), c.maskedFill(cm, value).toArray(), f"maskedFill {shape} {mshape}")
        assert_bits_equal(g.toArray(), x, "maskedFill must not touch its receiver")


CONCAT_CASES = [
    # shape (the axis entry is replaced), axis, lengths along the axis
    ([70001, 0], 1, [7, 3]),                      # rows of ten floats: most 16-byte units straddle both inputs
    ([300007, 0], 1, [1, 1]),                     # a unit holds two rows
    ([65536, 0], 1, [64, 64]),                    # aligned runs
    ([4099, 0], 1, [100, 28, 5]),                 # three inputs, the last unaligned
    ([0, 1021], 0, [300, 1, 212]),                # along the outermost axis: one row, runs at odd offsets
    ([33, 0, 517], 1, [2, 9, 1, 4, 3]),           # five inputs, a middle axis
    ([129, 0, 8], 1, [1, 2, 3, 4, 5, 6, 7, 8]),   # eight inputs: all the plan holds
    ([129, 0, 8], 1, [1, 2, 3, 4, 5, 6, 7, 8, 9]),# nine: a range set per input
    ([1, 0], 1, [3, 2]),                          # fewer than four floats in all ... and a ragged last unit below
    ([3, 0], 1, [1, 2]),
    ([2, 3, 0, 5, 7], 2, [6, 1]),
]


def test_concat_in_one_launch(gc):
    """concat writes every element of the result once, from whichever input holds it (TensorOperations.kt:41;
    the reference sets one range per input, AbstractJVMTensorOperations.kt:106-120): against numpy's concatenate."""
    rng = np.random.default_rng(40)
    for shape, axis, sizes in CONCAT_CASES:
        parts = []
        for length in sizes:
            sh = list(shape); sh[axis] = length
            parts.append(rng.standard_normal(sh).astype(np.float32))
        gc.profileBegin()
        got = gc.concat(axis, [gc.createRaw(list(p.shape), p) for p in parts])
        launched = " ".join(gc.profileEnd().keys())
        want = np.concatenate(parts, axis=axis)
        assert got.shape == list(want.shape)
        assert_bits_equal(got.toArray(), want, f"concat {shape} axis {axis} of {sizes}")
        if want.size:
            family = "move_kernel_set" if sum(1 for length in sizes if length) > 8 else "concat_kernel"
            assert family in launched, (shape, sizes, launched)
    # the result of an earlier operation that is still owed its fill, and a result tensor concatenated with itself
    z = gc.createRawFill([1000, 5], 2.5)
    x = gc.createRaw([1000, 3], np.arange(3000, dtype=np.float32))
    assert_bits_equal(gc.concat(1, [z, x, z]).toArray(),
                      np.concatenate([np.full((1000, 5), 2.5, np.float32), np.arange(3000, dtype=np.float32).reshape(1000, 3),
                                      np.full((1000, 5), 2.5, np.float32)], axis=1), "concat of an owed fill")
    with pytest.raises(ValueError):
        gc.concat(1, [x, gc.createRaw([999, 3], np.zeros(2997, np.float32))])
    # an empty input: an empty range to the reference's range sets, rejected there and, with the same words, here
    cpu = jo.JvmOracleOperations()
    empty = np.zeros((1000, 0), np.float32)
    with pytest.raises(ValueError) as on_checker:
        cpu.concat(1, [cpu.createRaw([1000, 3], np.zeros(3000, np.float32)), cpu.createRaw([1000, 0], empty.reshape(-1))])
    with pytest.raises(ValueError) as on_device:
        gc.concat(1, [x, gc.createRaw([1000, 0], empty)])
    assert str(on_device.value) == str(on_checker.value)
    # the entry point's own checks: lengths that do not add up, a result that is one of the inputs, a store too small
    L = gc.lib
    out = gc.createRaw([1000, 8])
    handles = (ctypes.c_uint64 * 2)(z.storeReference, x.storeReference)
    u64 = lambda *v: (ctypes.c_uint64 * len(v))(*v)
    i32 = lambda *v: (ctypes.c_int32 * len(v))(*v)
    assert L.kth_concat(handles, i32(5, 2), 2, abi.shape_array([1000, 8]), 2, 1, out.storeReference) == abi.KTH_E_SHAPE
    assert L.kth_concat(handles, i32(5, 3), 2, abi.shape_array([1000, 8]), 2, 2, out.storeReference) == abi.KTH_E_ARGUMENT
    assert L.kth_concat(u64(z.storeReference, out.storeReference), i32(5, 3), 2, abi.shape_array([1000, 8]), 2, 1,
                        out.storeReference) == abi.KTH_E_ARGUMENT
    assert "aliases" in abi.last_error()
    assert L.kth_concat(handles, i32(5, 3), 2, abi.shape_array([1001, 8]), 2, 1, out.storeReference) == abi.KTH_E_ARGUMENT
    assert L.kth_concat(u64(z.storeReference, 0xdeadbeef), i32(5, 3), 2, abi.shape_array([1000, 8]), 2, 1,
                        out.storeReference) == abi.KTH_E_HANDLE
    assert L.kth_concat(handles, i32(5, 3), 2, abi.shape_array([1000, 8]), 2, 1, out.storeReference) == abi.KTH_OK
    assert_bits_equal(out.toArray()[:, 5:], np.arange(3000, dtype=np.float32).reshape(1000, 3), "kth_concat")
    # ... and it takes inputs of length 0 itself
    out.inplaceFill(-1.0)
    nothing = gc.createRaw([1000, 0])
    assert L.kth_concat(u64(z.storeReference, nothing.storeReference, x.storeReference, nothing.storeReference), i32(5, 0, 3, 0), 4,
                        abi.shape_array([1000, 8]), 2, 1, out.storeReference) == abi.KTH_OK
    assert_bits_equal(out.toArray(), np.concatenate([np.full((1000, 5), 2.5, np.float32), np.arange(3000, dtype=np.float32).reshape(1000, 3)], axis=1),
                      "kth_concat with empty inputs")


def test_concat_and_narrow_parity(gc):
    rng = np.random.default_rng(4)
    cpu = jo.JvmOracleOperations()
    for shape, axis, sizes in (([3, 4], 0, [1, 2, 3]), ([3, 4], 1, [4, 1]), ([2, 3, 8], -2, [2, 5]), ([5], 0, [1, 1, 7]),
                               ([16, 8, 32], 1, [8, 24, 4]), ([4, 6, 10], 2, [3, 9])):
        parts = []
        for s in sizes:
            sh = list(shape); sh[axis] = s
            parts.append(rng.standard_normal(sh).astype(np.float32))
        got = gc.concat(axis, [gc.createRaw(list(p.shape), p) for p in parts])
        want = cpu.concat(axis, [cpu.createRaw(list(p.shape), p.reshape(-1)) for p in parts])
        assert got.shape == want.shape
        assert_bits_equal(got.toArray(), want.toArray(), f"concat {shape} axis {axis}")
        end = 0
        for p, s in zip(parts, sizes):
            assert_bits_equal(got.narrow(axis, end, s).toArray(), p, f"narrow {end}+{s}")
            end += s


def test_large_properties(gc):
    """At sizes the CPU checker would take long for: a transpose applied twice, a permute
    followed by its inverse and a narrow / concat round trip return the input bits, and a row
    of a transpose is a column of the input."""
    from kten_amd.host_mirror import inputs
    n = 4096
    x = inputs.SplitMix64(5).uniform([n, n], -1.0, 1.0)
    g = gc.createRaw([n, n], x)
    t = g.transpose(0, 1)
    assert_bits_equal(t.transpose(0, 1).toArray(), x, "transpose twice")
    assert_bits_equal(t.get([(17, 17), ALL]).toArray().reshape(-1), x[:, 17], "row of the transpose = column of the input")
    y = inputs.SplitMix64(6).uniform([16, 64, 56, 56], -1.0, 1.0)
    gy = gc.createRaw([16, 64, 56, 56], y)
    nhwc = gy.permute([0, 2, 3, 1])
    assert nhwc.shape == [16, 56, 56, 64]
    assert_bits_equal(nhwc.get([(3, 3), (5, 5), (7, 7), ALL]).toArray().reshape(-1), y[3, :, 5, 7], "NHWC pixel = NCHW channel column")
    assert_bits_equal(nhwc.permute([0, 3, 1, 2]).toArray(), y, "permute then its inverse")
    halves = [gy.narrow(1, 0, 24), gy.narrow(1, 24, 40)]
    assert_bits_equal(gc.concat(1, halves).toArray(), y, "narrow then concat")


@pytest.mark.parametrize("name,dims", [("transpose", {"rows": 300, "cols": 520}), ("permute", {"n": 6, "c": 16, "h": 12, "w": 20}),
                                       ("concat_mask", {"rows": 96, "left": 200, "right": 120})])
def test_layout_workloads_small_against_the_checker(name, dims, gc):
    from kten_amd.host_mirror.workloads import WORKLOADS
    wl = WORKLOADS[name]
    inputs = wl.make_inputs(dims)
    got = {k: v.toArray() for k, v in wl.run(gc, inputs).items()}
    want = {k: v.toArray() for k, v in wl.run(jo.JvmOracleOperations(), inputs).items()}
    for k in want:
        assert_bits_equal(got[k], want[k], f"{name}.{k}")


def test_layout_workloads_full_size(gc):
    """The benchmark shapes, against numpy's own movers (independent of both the device code
    and the checker)."""
    from kten_amd.host_mirror.workloads import WORKLOADS
    wl = WORKLOADS["transpose"]
    inp = wl.make_inputs(wl.full_dims)
    assert_bits_equal(wl.run(gc, inp)["xt"].toArray(), inp["x"].T, "transpose")
    wl = WORKLOADS["permute"]
    inp = wl.make_inputs(wl.full_dims)
    out = wl.run(gc, inp)
    assert_bits_equal(out["nhwc"].toArray(), np.transpose(inp["x"], (0, 2, 3, 1)), "NCHW -> NHWC")
    assert_bits_equal(out["back"].toArray(), inp["x"], "and back")
    wl = WORKLOADS["concat_mask"]
    inp = wl.make_inputs(wl.full_dims)
    out = wl.run(gc, inp)
    cat = np.concatenate([inp["a"], inp["b"]], axis=1)
    masked = np.where(inp["mask"] == 1.0, np.float32(0.0), cat)
    left = inp["a"].shape[1]
    assert_bits_equal(out["cat"].toArray(), cat, "concat")
    assert_bits_equal(out["right"].toArray(), masked[:, left:], "range get")
    masked[:, :left] = 1.0
    assert_bits_equal(out["masked"].toArray(), masked, "maskedFill then range fill")


@pytest.mark.parametrize("old,new", [([6], [2, 5]), ([2, 5], [3]), ([1000, 33], [1000, 40]), ([64, 64], [63, 65]), ([4099], [4099])])
def test_inplace_resize_parity(old, new, gc):
    x = np.random.default_rng(sum(old) + sum(new)).standard_normal(old).astype(np.float32)
    g, c = both(gc, x)
    shared = g.copy(shallow=True)
    g.inplaceResize(*new); c.inplaceResize(*new)
    assert g.shape == c.shape == new
    assert_bits_equal(g.toArray().reshape(-1), c.toArray().reshape(-1), f"inplaceResize {old} -> {new}")
    assert_bits_equal(shared.toArray().reshape(-1), x.reshape(-1), "the shallow copy keeps the old store")
    g.plusAssign(1.0); c.plusAssign(1.0)                      # the new store is an ordinary store
    assert_bits_equal(g.toArray().reshape(-1), c.toArray().reshape(-1), "arithmetic on the resized tensor")


def test_copy_between_any_offsets(hip):
    """kth_copy for every combination of source and destination offsets modulo 4 and lengths around
    the 16-byte units: the range arrives bit for bit and nothing next to it is touched."""
    import ctypes
    from kten_amd import abi
    lib = hip.lib
    size = 6000
    src_host = np.random.default_rng(9).standard_normal(size).astype(np.float32)
    hs, hd = ctypes.c_uint64(), ctypes.c_uint64()
    abi.check(lib.kth_alloc(size, ctypes.byref(hs))); abi.check(lib.kth_alloc(size, ctypes.byref(hd)))
    abi.check(lib.kth_upload(hs, 0, src_host.ctypes.data_as(ctypes.c_void_p), size))
    out = np.empty(size, np.float32)
    try:
        for n in (0, 1, 2, 3, 4, 5, 7, 8, 9, 255, 1023, 1024, 1025, 4099):
            for so in range(5):
                for do in range(5):
                    abi.check(lib.kth_fill(hd, 0, size, -7.0))
                    abi.check(lib.kth_copy(hd, 10 + do, hs, 20 + so, n))
                    abi.check(lib.kth_download(out.ctypes.data_as(ctypes.c_void_p), hd, 0, size))
                    want = np.full(size, -7.0, np.float32)
                    want[10 + do:10 + do + n] = src_host[20 + so:20 + so + n]
                    assert_bits_equal(out, want, f"copy of {n} floats from offset {20 + so} to offset {10 + do}")
        assert lib.kth_copy(hd, 0, hd, 2, 10) == abi.KTH_E_ARGUMENT          # overlapping ranges in one store
        assert lib.kth_copy(hd, size - 3, hs, 0, 4) == abi.KTH_E_ARGUMENT    # past the end of the destination
    finally:
        abi.check(lib.kth_release(hs)); abi.check(lib.kth_release(hd))
