"""Parity of the reduction kernels with the CPU checker, through the C ABI.
MAX / MIN / ARG_MAX / ARG_MIN: bit-exact. SUM / MEAN: the two-clause tolerance of
parity.py against the extended-precision sum, with the checker's own serial-float
error as the second clause."""
import numpy as np
import pytest

from oracle import jvm_oracle as jo
from parity import assert_bits_equal, assert_reduction_close

pytestmark = pytest.mark.gpu

# [shape, axis]: chosen to hit every kernel variant — rows with 1/4/16/64/256 lanes per
# row, aligned and unaligned; columns with float4 and scalar lanes, with and without
# axis segmentation; the strided kernel for small inner sizes.
GEOMETRIES = [
    ([7], 0), ([1000], 0), ([4099], 0), ([300000], 0), ([1 << 21], 0),
    ([5, 3], 1), ([100, 7], 1), ([64, 40], 1), ([50, 200], 1), ([9, 1000], 1), ([3, 5000], 1), ([2, 100001], 1),
    ([2, 70000], 1), ([3000, 16], 1), ([1000, 33], 1),
    ([8, 64], 0), ([100, 256], 0), ([5000, 128], 0), ([70000, 64], 0), ([333, 1000], 0), ([40000, 65], 0),
    ([4, 50, 64], 1), ([3, 2000, 68], 1), ([2, 3, 4], 0), ([2, 3, 4], 1), ([6, 30000, 5], 1), ([10, 56, 56], 1),
    ([128, 56, 56], 1), ([64, 16, 49], 0), ([3, 17, 1, 9], 1), ([2, 2, 2, 2, 2, 2, 2, 2, 2, 5], 4),
    # short rows staged through LDS (8 <= length < 256), every lanes-per-row variant, ragged last tile
    ([5000, 8], 1), ([1030, 9], 1), ([777, 31], 1), ([3001, 32], 1), ([515, 50], 1), ([130, 100], 1), ([67, 129], 1),
    ([33, 255], 1), ([1, 200], 1), ([300, 10], 1),
    # rows of 2 ... 7 floats through the same tiles; long rows that start off 16-byte boundaries (peeled to float4s)
    ([5000, 3], 1), ([70000, 2], 1), ([1030, 7], 1), ([333, 5], 1), ([300, 1250], 1), ([5, 100003], 1), ([40, 4097], 1),
    ([3, 7, 1001], 2), ([2, 300001], 1),
    # an axis of length 1 (elementwise pass) and unaligned rows of 256 ... 2048 floats through the row tiles
    ([1000, 1, 77], 1), ([5, 1], 1), ([1, 4099], 0), ([900, 261], 1), ([70, 555], 1), ([33, 2047], 1), ([9, 2049], 1),
    # an axis of 2 ... 7 over wide columns: four columns per thread, float4 and scalar, ragged last tile
    ([3, 2, 70001], 1), ([2, 3, 300000], 1), ([5, 7, 20000], 1), ([1, 5, 100003], 1), ([7, 66000], 0), ([2, 4, 40000, 2], 1),
    # short slabs, too few of them for the tiled kernel
    ([5000, 8, 8], 1), ([1000, 2, 2], 1), ([999, 3, 40], 1), ([257, 16, 16], 1), ([100, 4, 63], 1), ([70, 2, 3, 5], 2),    # slabs up to a whole tile for short axes: unaligned tiles, several lanes per output
    ([600, 8, 128], 1), ([300, 16, 64], 1), ([257, 3, 1024], 1), ([1100, 2, 300], 1), ([400, 4, 201], 1),
    # slabs of up to 2047 floats with any axis length, enough of them to take the tiled kernel
    ([8000, 17, 17], 1), ([7000, 40, 8], 1), ([8000, 100, 3], 1), ([3000, 500, 2], 1), ([1500, 24, 80], 1),
    ([1500, 19, 100], 1), ([1500, 128, 13], 1),
    # the smallest slabs (4 ... 10 floats) in numbers that take the tiled kernel: the odd LDS pitch adds a quarter to a slab of 4
    ([300000, 2, 2], 1), ([250000, 3, 2], 1), ([250000, 2, 3], 1), ([140000, 2, 4], 1), ([200000, 3, 3], 1), ([120000, 2, 5], 1),
    # a slab (or a segment of it) streamed by one workgroup: scalar and float4 columns, with and without segments
    ([300, 700, 3], 1), ([2, 50000, 12], 1), ([2000, 64, 33], 1), ([1500, 100, 40], 1), ([5, 2049, 1, 63], 1),
    ([3, 40000, 2], 1), ([1, 100000, 7], 1),
    # groups of four columns when the inner size is not a multiple of 4 (the last group overlaps its neighbour): streamed
    # slabs with inner 5 ... 511, the column kernel from 513 on, one and several outer indices, with and without segments
    ([3, 3000, 5], 1), ([2, 2500, 6], 1), ([4, 700, 7], 1), ([3, 900, 257], 1), ([1, 2000, 301], 1), ([2, 300, 479], 1), ([5000, 511], 0),
    ([2, 600, 513], 1), ([3000, 1001], 0), ([1, 4100, 515], 1), ([40000, 65], 0), ([9, 70, 130], 1),
    # scalar columns in tiles four waves wide, with and without segments
    ([300, 1001], 0), ([3, 500, 257], 1), ([2, 5000, 259], 1), ([7, 300], 0),
    # streamed slabs with wide columns: one group of threads per row, float4 columns up to 511
    ([40, 300, 129], 1), ([30, 64, 200], 1), ([3, 5000, 68], 1), ([20, 50, 300], 1), ([5, 2000, 255], 1), ([9, 40, 508], 1),
]
OPS = ["sum", "mean", "max", "min", "argMax", "argMin"]
CODE = {"sum": "sum", "mean": "mean", "max": "max", "min": "min", "argMax": "arg_max", "argMin": "arg_min"}


def raw(gc, a):
    return gc.createRaw(list(a.shape), a)


@pytest.mark.parametrize("shape,axis", GEOMETRIES, ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_axis_reductions(shape, axis, gc):
    rng = np.random.default_rng(len(shape) * 1000 + shape[0] + axis)
    x = rng.standard_normal(shape).astype(np.float32)
    # ties for the arg ops: quantise a slice
    flat = x.reshape(-1)
    flat[::3] = np.round(flat[::3] * 2) / 2
    t = raw(gc, x)
    ref64, _ = jo.axis_sum_f64(x, axis)
    for op in OPS:
        for keep in (False, True):
            res = getattr(t, op)(axis, keep)
            want_shape = list(shape); want_shape[axis] = 1
            if not keep and len(shape) > 1:
                del want_shape[axis]
            assert res.shape == want_shape
            got = res.toArray().reshape(-1)
            want = jo.aggregate(CODE[op], x, axis).reshape(-1)
            if op == "sum":
                assert_reduction_close(got, ref64, want, f"sum {shape} axis {axis}")
            elif op == "mean":
                assert_reduction_close(got, ref64 / shape[axis], want, f"mean {shape} axis {axis}")
            else:
                assert_bits_equal(got, want, f"{op} {shape} axis {axis}")


@pytest.mark.parametrize("shape,axis", [([64, 40], 1), ([9, 1000], 1), ([3, 5000], 1), ([333, 1000], 0), ([4, 50, 64], 1),
                                        ([6, 3000, 5], 1), ([2, 70000], 1), ([70000, 64], 0), ([600, 100], 1), ([300, 12, 9], 1),
                                        ([2, 50000, 12], 1), ([700, 300, 7], 1), ([300, 16, 64], 1),
                                        ([8000, 100, 3], 1), ([1500, 24, 80], 1), ([300, 1250], 1), ([5000, 3], 1), ([5, 100003], 1), ([600, 1, 33], 1), ([1, 5000], 0), ([2, 3, 70001], 1), ([5, 80000], 0)],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_special_values_in_reductions(shape, axis, gc):
    """NaN propagation in max/min, NaN skipping in arg ops, signed zeros, lanes of -inf / +inf, ties."""
    rng = np.random.default_rng(7)
    lanes = int(np.prod(shape)) // shape[axis]
    m = rng.integers(-2, 3, size=(shape[axis], lanes)).astype(np.float32)     # [axis, lane]: heavy ties, many zeros
    flat = m.reshape(-1)
    idx = rng.choice(flat.size, size=max(4, flat.size // 50), replace=False)
    flat[idx[0::4]] = np.nan
    flat[idx[1::4]] = -0.0
    flat[idx[2::4]] = np.inf
    flat[idx[3::4]] = -np.inf
    m[:, 0] = -np.inf                                                          # a lane with nothing > -inf
    m[:, -1] = np.where(np.arange(shape[axis]) % 2 == 0, 0.0, -0.0)            # a lane of signed zeros only
    m[:, lanes // 2] = np.nan                                                  # a lane of NaNs only
    rest = [d for i, d in enumerate(shape) if i != axis]
    x = np.ascontiguousarray(np.moveaxis(m.reshape([shape[axis]] + rest), 0, axis))
    t = raw(gc, x)
    for op in ("max", "min", "argMax", "argMin"):
        assert_bits_equal(getattr(t, op)(axis).toArray().reshape(-1), jo.aggregate(CODE[op], x, axis).reshape(-1),
                          f"{op} {shape} axis {axis}")


# Small tensors (up to 4 MiB) whose slabs a wave takes whole, and small tensors of short rows: inner sizes on and off
# multiples of 4 (the last column group overlaps its neighbour), 1 ... 32 row lanes per column group, slabs of one
# and of several batches of loads, outer counts that leave a workgroup's last waves without a slab.
SMALL_SLABS = [([128, 56, 56], 1), ([10, 56, 56], 1), ([1, 64, 200], 1), ([33, 120, 5], 1), ([17, 300, 7], 1), ([64, 9, 255], 1),
               ([200, 40, 31], 1), ([5, 1000, 4], 1), ([19, 128, 13], 1), ([70, 3, 256], 1), ([2, 2, 40, 129], 2), ([130, 600, 6], 1),
               ([128, 56, 56], 2), ([16, 2048, 4], 1)]
SMALL_ROWS = [([128, 56], 1), ([1, 128, 1, 56], 3), ([300, 10], 1), ([77, 255], 1), ([1000, 3], 1), ([40, 129], 1), ([2, 200], 1), ([500, 17], 1)]


@pytest.mark.parametrize("shape,axis", SMALL_SLABS + SMALL_ROWS, ids=lambda v: "x".join(map(str, v)) if isinstance(v, list) else str(v))
def test_small_inputs(shape, axis, gc):
    rng = np.random.default_rng(sum(shape) + axis)
    x = rng.standard_normal(shape).astype(np.float32)
    x.reshape(-1)[::3] = np.round(x.reshape(-1)[::3] * 2) / 2                 # ties for the arg reducers
    x.reshape(-1)[5::97] = np.nan
    x.reshape(-1)[11::89] = -np.inf
    t = raw(gc, x)
    gc.profileBegin()
    got = {op: getattr(t, op)(axis).toArray().reshape(-1) for op in OPS}
    kernels = gc.profileEnd()
    if (shape, axis) in SMALL_SLABS[:12]:
        assert any(k.startswith("reduce_wave_slabs_kernel") for k in kernels), f"expected a wave per slab, saw {sorted(kernels)}"
    if (shape, axis) in SMALL_ROWS:
        assert all(k.startswith("reduce_rows_kernel") for k in kernels), f"expected the row kernel, saw {sorted(kernels)}"
    for op in ("max", "min", "argMax", "argMin"):
        assert_bits_equal(got[op], jo.aggregate(CODE[op], x, axis).reshape(-1), f"{op} {shape} axis {axis}")
    y = np.nan_to_num(x, nan=0.5, neginf=-2.0)                                 # sums on finite values
    ty = raw(gc, y)
    ref64, _ = jo.axis_sum_f64(y, axis)
    assert_reduction_close(ty.sum(axis).toArray().reshape(-1), ref64, jo.aggregate("sum", y, axis).reshape(-1), f"sum {shape} axis {axis}")
    assert_reduction_close(ty.mean(axis).toArray().reshape(-1), ref64 / shape[axis], jo.aggregate("mean", y, axis).reshape(-1), f"mean {shape} axis {axis}")


@pytest.mark.parametrize("n", [1, 2, 5, 1000, 4099, 300001, 1 << 22])
def test_full_sum_and_mean(n, gc):
    x = (np.random.default_rng(n).standard_normal(n) * 10 + 0.5).astype(np.float32)
    t = raw(gc, x)
    ref = jo.sum_all_f64(x)
    s, m = t.sum(), t.mean()
    assert s.shape == [1] and m.shape == [1]
    assert_reduction_close(s.toArray(), [ref], [jo.sum_all(x)], f"sum() n={n}")
    assert_reduction_close(m.toArray(), [ref / n], [jo.mean_all(x)], f"mean() n={n}")
    # mean() accumulates in f64 on both sides: it should be the correctly rounded mean
    assert abs(float(m.toArray()[0]) - ref / n) <= abs(ref / n) * 2 ** -23


def test_sum_of_cancelling_terms_is_exact_in_f64(gc):
    # kten-jvm's serial float sum returns 0 here; the true sum is 1 and f64 accumulation finds it.
    x = np.array([1e8, 1.0, -1e8], np.float32)
    assert raw(gc, x).sum().toArray()[0] == 1.0
    y = np.array([16777216.0] + [1.0] * 64, np.float32)
    assert raw(gc, y).sum().toArray()[0] == np.float32(16777216.0 + 64.0)
    assert raw(gc, y).mean().toArray()[0] == jo.mean_all(y)


def test_reductions_are_deterministic(gc):
    x = np.random.default_rng(11).standard_normal((3000, 700)).astype(np.float32)
    t = raw(gc, x)
    for axis in (0, 1):
        a = t.sum(axis).toArray(); b = t.sum(axis).toArray()
        assert_bits_equal(a, b, f"sum axis {axis} twice")
    a = t.sum().toArray(); b = t.sum().toArray()
    assert_bits_equal(a, b, "sum() twice")


def test_reduce_to_shape_matches_numpy(gc):
    """mayUnexpand = numpy.sum over the broadcast axes with keepdims, reshaped to the operand."""
    from kten_amd.host_mirror.autograd import mayUnexpand
    rng = np.random.default_rng(13)
    for gshape, oshape, axes in [([6, 40, 7, 9], [1, 40, 1, 1], (0, 2, 3)), ([50, 30], [30], (0,)), ([50, 30], [1], (0, 1)),
                                 ([4, 5, 6], [5, 1], (0, 2)), ([3, 3], [3, 1], (1,))]:
        g = rng.standard_normal(gshape).astype(np.float32)
        res = mayUnexpand(raw(gc, g), oshape, gc)
        assert res.shape == oshape
        ref = g.astype(np.float64).sum(axes, keepdims=True).reshape(oshape)
        np.testing.assert_allclose(res.toArray(), ref, rtol=1e-5, atol=1e-5)


def test_sums_whose_float_running_sum_overflows_or_absorbs(gc):
    """Where kten-jvm's serial float accumulation (JVMRawTensor.kt:146-148,186-192) overflows or absorbs terms, this
    backend (f64 accumulation, one rounding) returns the correctly rounded sum instead: a divergence in kind, inside
    the reduction bar (its error is the smaller one), and not pinned by any test of the reference."""
    rows = np.array([[3e38, 3e38, -3e38, 1.0], [1e8, 1.0, -1e8, 0.0], [-3e38, -3e38, 3e38, 5.0], [16777216.0, 1.0, 1.0, 1.0]], dtype=np.float32)
    exact = rows.astype(np.float64).sum(1)
    for x, axis in ((rows, 1), (np.ascontiguousarray(rows.T), 0)):
        t = raw(gc, x)
        with np.errstate(all="ignore"):
            jvm_sum = jo.aggregate("sum", x, axis).reshape(-1)
            jvm_mean = jo.aggregate("mean", x, axis).reshape(-1)
        got_sum = t.sum(axis).toArray().reshape(-1)
        got_mean = t.mean(axis).toArray().reshape(-1)
        assert np.isposinf(jvm_sum[0]) and np.isneginf(jvm_sum[2]) and jvm_sum[1] == 0.0 and jvm_sum[3] == 16777216.0
        assert_bits_equal(got_sum, exact.astype(np.float32), "sum: the correctly rounded value")
        assert_bits_equal(got_mean, (exact / 4.0).astype(np.float32), "mean: the correctly rounded value")
        assert np.isinf(jvm_mean[0]) and np.isfinite(got_mean[0])
