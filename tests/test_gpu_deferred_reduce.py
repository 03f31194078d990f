"""A small axis SUM / MEAN whose result the next step of a reduce-to-shape chain could fold further is put off by the
library: the output is owed the reduction. If the chain's next step comes, one launch over the source does both steps
(and the intermediate is never computed unless somebody else asks for it); any other reader has the reduction launched
first. Every way into and out of that state must give the bits of the plain sequence, which the same library computes
here with the intermediate read in between; the launch counter and the profile show which form ran."""
import numpy as np
import pytest

from parity import assert_bits_equal

pytestmark = pytest.mark.gpu


def launches(gc):
    return gc.getMetrics()["launches"]


def data(shape, seed):
    return (np.random.default_rng(seed).standard_normal(shape) * 3 + 0.25).astype(np.float32)


# [outer, axis, inner]: the shapes of cfg4's chains, inner sizes of one to 63 16-byte units, axes of one and of several
# batches of loads, few and many outer indexes
CHAINS = [[128, 56, 56], [128, 4, 252], [16, 600, 4], [1000, 8, 64], [3, 64, 200], [40, 33, 100], [512, 16, 128], [17, 1000, 8]]


@pytest.mark.parametrize("first,second", [("sum", "sum"), ("mean", "mean"), ("sum", "mean"), ("mean", "sum")])
@pytest.mark.parametrize("shape", CHAINS, ids=lambda s: "x".join(map(str, s)))
def test_two_steps_of_a_chain_are_one_launch_with_the_bits_of_two(shape, first, second, gc):
    x = data(shape, sum(shape))
    t = gc.createRaw(shape, x)
    # the plain sequence: the intermediate is read (and so computed) before the second step
    mid = getattr(t, first)(1)
    mid_values = mid.toArray()
    want = getattr(mid, second)(1).toArray()
    # the chain: nothing runs at the first step, one launch does both at the second
    before = launches(gc)
    mid2 = getattr(t, first)(1)
    assert launches(gc) == before, "the first step is put off"
    gc.profileBegin()
    got = getattr(mid2, second)(1)
    kernels = gc.profileEnd()
    assert list(kernels) == [f"reduce_wave_slabs_rows_kernel<{'RedMean' if second == 'mean' else 'RedSum'}>"], sorted(kernels)
    assert_bits_equal(got.toArray(), want, f"{first} then {second} of {shape}")
    # the intermediate is still owed, and right when somebody asks for it after all
    assert_bits_equal(mid2.toArray(), mid_values, "intermediate read after the chain")
    ref64 = x.astype(np.float64).sum(1) if first == "sum" else x.astype(np.float64).mean(1)
    assert np.allclose(mid_values, ref64, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("shape", [[128, 2, 252], [8, 128, 300], [4, 3000, 64], [70000, 4, 4], [64, 128, 1]], ids=lambda s: "x".join(map(str, s)))
def test_shapes_outside_the_plan_run_at_once(shape, gc):
    x = data(shape, 5)
    t = gc.createRaw(shape, x)
    before = launches(gc)
    mid = t.sum(1)
    assert launches(gc) > before
    assert np.allclose(mid.sum(1).toArray(), x.astype(np.float64).sum(1).sum(1), rtol=1e-5, atol=1e-4)


def test_readers_of_a_sum_that_was_put_off(gc):
    shape = [128, 56, 56]
    x = data(shape, 1)
    t = gc.createRaw(shape, x)
    want = t.sum(1).toArray()                                   # computed at once: it is read here
    readers = {
        "download": lambda m: m.toArray(),
        "operand": lambda m: m._scalar("times", 1.0).toArray(),
        "binary": lambda m: m._binary("plus", gc.createRawFill([128, 56], 0.0)).toArray(),
        "copy": lambda m: m.copy().toArray(),
        "view": lambda m: m.view([128 * 56]).toArray().reshape(128, 56),
        "full sum": lambda m: m.sum().toArray(),
        "other axis": lambda m: m.sum(0).toArray(),
        "max": lambda m: m.max(1).toArray(),
        "transpose": lambda m: m._transpose(0, 1, [56, 128]).toArray().T,
    }
    expected = {"full sum": None, "other axis": None, "max": None}
    for name, read in readers.items():
        owed = t.sum(1)
        got = read(owed)
        if name in expected:
            plain = gc.createRaw([128, 56], want)
            ref = {"full sum": lambda m: m.sum(), "other axis": lambda m: m.sum(0), "max": lambda m: m.max(1)}[name](plain).toArray()
            assert_bits_equal(got, ref, name)
        else:
            assert_bits_equal(np.ascontiguousarray(got), want, name)


def test_the_source_of_a_sum_that_was_put_off(gc):
    shape = [64, 40, 100]
    x = data(shape, 2)
    want = gc.createRaw(shape, x).sum(1).toArray()
    # the source is written before anybody reads the sum: the sum is that of the old values
    t = gc.createRaw(shape, x)
    owed = t.sum(1)
    t._scalar_assign("times", 0.0)
    assert_bits_equal(owed.toArray(), want, "sum, then the source zeroed")
    assert not t.toArray().any()
    # the source is released first: its values outlive its handle until the sum is done or dropped
    t = gc.createRaw(shape, x)
    owed = t.sum(1)
    follow = None
    t.release()
    follow = owed.sum(1)
    assert_bits_equal(follow.toArray(), gc.createRaw([64, 100], want).sum(1).toArray(), "chain after the source was released")
    assert_bits_equal(owed.toArray(), want, "intermediate after the source was released")
    # dropped unread: nothing runs, nothing is left behind
    before = launches(gc)
    t = gc.createRaw(shape, x)
    after_upload = launches(gc)
    owed = t.sum(1)
    owed.release()
    t.release()
    assert launches(gc) == after_upload and after_upload - before <= 1
    # the output of a sum that is put off was holding something else: notes on it go, its old aliases keep their values
    old = gc.createRaw([64, 100], want * 0 + 7)
    keep = old.copy()
    t = gc.createRaw(shape, x)
    assert gc.lib.kth_reduce_axis(7, t.storeReference, old.storeReference, 64, 40, 100) == 0      # KTH_SUM into an existing store
    assert_bits_equal(keep.toArray(), np.full([64, 100], 7.0, np.float32), "copy of the output's old values")
    assert_bits_equal(old.toArray(), want, "sum into an existing store")


def test_cfg4_chains_take_three_launches_each(gc):
    """[64,128,56,56] summed over (0, 2, 3): the large step, then the two small ones as one launch."""
    x = data([8, 128, 56, 56], 3)
    t = gc.createRaw([8, 128, 56, 56], x)
    for op in ("sum", "mean"):
        gc.profileBegin()
        a = getattr(t, op)(0, True)
        b = getattr(a, op)(2, True)
        c = getattr(b, op)(3, True)
        got = c.toArray()
        kernels = gc.profileEnd()
        assert sum(v[0] for v in kernels.values()) == 2, sorted(kernels)
        x64 = x.astype(np.float64)
        ref = x64.sum((0, 2, 3)) if op == "sum" else x64.mean((0, 2, 3))
        assert np.allclose(got.reshape(-1), ref, rtol=1e-5)


def test_the_entry_point_that_allocates_nothing_puts_nothing_off(gc):
    """kth_reduce_axis_static launches at once, and an input that is still owed its sum has it launched first: the
    values are those of the plain entry point either way."""
    from kten_amd.abi import Op, check
    shape = [128, 56, 56]
    x = data(shape, 7)
    t = gc.createRaw(shape, x)
    mid = t.sum(1)
    mid_values = mid.toArray()
    want = mid.sum(1).toArray()
    # an owed input
    owed = t.sum(1)
    out = gc.createRaw([128])
    before = launches(gc)
    check(gc.lib.kth_reduce_axis_static(Op.SUM, owed.storeReference, out.storeReference, 128, 56, 1))
    assert launches(gc) == before + 2, "the owed sum, then this one"
    assert_bits_equal(out.toArray(), want, "static entry over an owed input")
    assert_bits_equal(owed.toArray(), mid_values, "the input afterwards")
    # a geometry that the plain entry point would put off
    out2 = gc.createRaw([128, 56])
    before = launches(gc)
    check(gc.lib.kth_reduce_axis_static(Op.SUM, t.storeReference, out2.storeReference, 128, 56, 56))
    assert launches(gc) == before + 1
    assert_bits_equal(out2.toArray(), mid_values, "static entry, first step")
