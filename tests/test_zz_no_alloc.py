"""kth_reduce_axis_static, the axis reduction that allocates nothing (its partials live in a
fixed array in the library's device code), through the C ABI: the same bits as kth_reduce_axis
on two calls in a row, the second on a smaller input, which finds the array full of the first
call's partials. Both are also held against the CPU checker (SUM / MEAN by the two-clause
tolerance of parity.py, MAX / ARG_MAX bit-exact). The call must leave the pool untouched, and a
plan whose partials exceed the array must be refused before anything is launched.

Collected last (the file name sorts after every other test file): a failure here hides nothing.
"""
import ctypes

import numpy as np
import pytest

from kten_amd.abi import Op, check
from oracle import jvm_oracle as jo
from parity import assert_bits_equal, assert_reduction_close

pytestmark = pytest.mark.gpu

OPS = [("sum", Op.SUM), ("mean", Op.MEAN), ("max", Op.MAX), ("arg_max", Op.ARG_MAX)]


def reduce_both(gc, t, x, axis, two_pass):
    """{op: (static result, pooled result)} for tensor t (host copy x) over `axis`, plus the pool
    figures before and after the static calls."""
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    length = x.shape[axis]
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    res_shape = list(x.shape); res_shape[axis] = 1
    lib = gc.lib
    out = {}
    for name, code in OPS:
        a = gc.createRaw(res_shape); b = gc.createRaw(res_shape)
        a.inplaceFill(-7.0); b.inplaceFill(-7.0)
        before = gc.getMetrics()
        check(lib.kth_reduce_axis_static(code, t.storeReference, a.storeReference, outer, length, inner))
        after = gc.getMetrics()
        assert (before["liveBytes"], before["poolBytes"]) == (after["liveBytes"], after["poolBytes"]), \
            f"{name}: the static entry point moved pool memory"
        assert after["launches"] - before["launches"] == (2 if two_pass else 1), \
            f"{name} {list(x.shape)}: expected a {'two' if two_pass else 'single'}-pass plan"
        check(lib.kth_reduce_axis(code, t.storeReference, b.storeReference, outer, length, inner))
        out[name] = (a.toArray(), b.toArray())
    return out


def check_case(gc, shape, axis, seed, two_pass=True):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(shape).astype(np.float32)
    x.reshape(-1)[::5] = np.round(x.reshape(-1)[::5] * 2) / 2          # ties for arg_max
    t = gc.createRaw(list(shape), x)
    got = reduce_both(gc, t, x, axis, two_pass)
    ref64, _ = jo.axis_sum_f64(x, axis)
    for name, _ in OPS:
        static, pooled = got[name]
        assert_bits_equal(static, pooled, f"{name} {shape} axis {axis}: static against kth_reduce_axis")
        want = jo.aggregate(name, x, axis).reshape(-1)
        if name == "sum":
            assert_reduction_close(static.reshape(-1), ref64, want, f"sum {shape} axis {axis}")
        elif name == "mean":
            assert_reduction_close(static.reshape(-1), ref64 / shape[axis], want, f"mean {shape} axis {axis}")
        else:
            assert_bits_equal(static.reshape(-1), want, f"{name} {shape} axis {axis}: static against the checker")


def test_static_reduction_twice_then_smaller(gc):
    """Two-pass plans of every first-pass kernel (columns, rows, streamed slabs, strided), each
    followed by a smaller input of the same kind, then single-pass shapes."""
    # columns: [4096, 2048] over axis 0 leaves 8 column tiles -> 16 waves x many segments; then a ragged smaller one
    check_case(gc, [4096, 2048], 0, 1)
    check_case(gc, [3000, 1001], 0, 2)
    # rows: a full reduction in segments, then a shorter one
    check_case(gc, [1 << 21], 0, 3)
    check_case(gc, [300000], 0, 4)
    # a streamed slab in segments, then a smaller one
    check_case(gc, [2, 50000, 12], 1, 5)
    check_case(gc, [1, 20000, 7], 1, 6)
    # strided: small inner, few slabs
    check_case(gc, [3, 40000, 2], 1, 7)
    check_case(gc, [3, 9000, 2], 1, 8)
    # single pass: nothing goes through the array
    check_case(gc, [600, 8, 128], 1, 9, two_pass=False)
    check_case(gc, [515, 50], 1, 10, two_pass=False)


def test_static_reduction_refuses_what_does_not_fit(gc):
    size = ctypes.c_uint64()
    check(gc.lib.kth_reduce_scratch_bytes(ctypes.byref(size)))
    assert size.value == 4 << 20
    # [1024, 200000] over axis 0: 782 column tiles are cut into 3 axis segments -> 200000 * 3 * 8 bytes of partials
    shape = [1024, 200000]
    t = gc.createRawFill(shape, 1.0)
    out = gc.createRawFill([1, 200000], -7.0)
    assert t.getSingleValue([0, 0]) == 1.0                    # the input is in memory, not a fill still to be launched
    launches = gc.getMetrics()["launches"]
    rc = gc.lib.kth_reduce_axis_static(Op.SUM, t.storeReference, out.storeReference, 1, 1024, 200000)
    assert rc == -3, "a plan beyond the scratch array must return KTH_E_ARGUMENT"
    msg = gc.lib.kth_last_error().decode()
    assert "static scratch" in msg and "4800000" in msg, msg
    assert gc.getMetrics()["launches"] == launches, "nothing may be launched for a refused shape"
    assert_bits_equal(out.toArray(), np.full([1, 200000], -7.0, dtype=np.float32), "output of a refused call")
    # the same refusal while the input is still a noted constant: its fill is not launched either
    fresh = gc.createRawFill(shape, 2.0)
    launches = gc.getMetrics()["launches"]
    rc = gc.lib.kth_reduce_axis_static(Op.SUM, fresh.storeReference, out.storeReference, 1, 1024, 200000)
    assert rc == -3
    assert gc.getMetrics()["launches"] == launches, "a refused call must not launch the fill its input is owed"
    assert_bits_equal(out.toArray(), np.full([1, 200000], -7.0, dtype=np.float32), "output of the second refused call")
    check(gc.lib.kth_reduce_axis(Op.SUM, fresh.storeReference, out.storeReference, 1, 1024, 200000))
    assert_bits_equal(out.toArray(), np.full([1, 200000], 2048.0, dtype=np.float32), "the constant input after the refusal")
    # the pooled entry point takes the same shape
    check(gc.lib.kth_reduce_axis(Op.SUM, t.storeReference, out.storeReference, 1, 1024, 200000))
    assert_bits_equal(out.toArray(), np.full([1, 200000], 1024.0, dtype=np.float32), "kth_reduce_axis on the refused shape")
