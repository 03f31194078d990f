"""A whole-store copy (`copy()`, kth_copy) and `pow` with the exponent 1 (what the backward pass of a square asks for)
are put off by the library: the new store reads the source's memory until one of the two is written, and only then is
the copy made; a source that is released first hands its buffer over. Every way into and out of that state must give
the values of the plain sequence (copy at once, then the op), which numpy computes here; the launch counter shows that
no copy kernel runs where none is needed."""
import numpy as np
import pytest

from parity import assert_bits_equal

pytestmark = pytest.mark.gpu


def launches(gc):
    return gc.getMetrics()["launches"]


def data(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("how", ["pow1", "copy"])
def test_a_copy_that_is_only_read_is_never_made(how, gc):
    x = data([300, 257], 1)
    a = gc.createRaw(list(x.shape), x)
    before = launches(gc)
    b = a._scalar("pow", 1.0) if how == "pow1" else a.copy()
    assert launches(gc) == before, "no kernel for the copy"
    assert_bits_equal(b.toArray(), x, "download of the copy")
    assert launches(gc) == before, "a download reads through"
    # binary ops, scalar ops, unary ops and reductions read through as well
    gc.profileBegin()
    c = b._binary("times", a)
    d = a._binary("plus", b)
    e = b._scalar("times", 3.0)
    f = b._unary("neg")
    s0 = b.sum(0)
    total = b.sum()
    kernels = gc.profileEnd()
    assert not any(k.startswith("copy_kernel") for k in kernels), f"no copy for readers: {sorted(kernels)}"
    assert_bits_equal(c.toArray(), x * x, "b * a")
    assert_bits_equal(d.toArray(), x + x, "a + b")
    assert_bits_equal(e.toArray(), x * np.float32(3), "b * 3")
    assert_bits_equal(f.toArray(), -x, "-b")
    assert np.allclose(s0.toArray(), x.astype(np.float64).sum(0), rtol=1e-5, atol=1e-5)
    assert np.allclose(total.toArray(), x.astype(np.float64).sum(), rtol=1e-5, atol=1e-4)
    # released unread: still no copy
    b.release()
    assert_bits_equal(a.toArray(), x, "the source after the copy was released")


def test_writing_the_source_makes_the_copy_first(gc):
    x = data([1000, 33], 2)
    for write in ("scalar_assign", "binary_assign", "fill", "upload", "scatter", "set_range", "as_output"):
        a = gc.createRaw(list(x.shape), x)
        b = a._scalar("pow", 1.0)
        c = a.copy()
        want_a = x.copy()
        if write == "scalar_assign":
            a._scalar_assign("plus", 1.0); want_a = x + np.float32(1)
        elif write == "binary_assign":
            a._binary_assign("times", gc.createRaw(list(x.shape), x)); want_a = x * x
        elif write == "fill":
            a.inplaceFill(4.0); want_a = np.full_like(x, 4.0)
        elif write == "upload":
            a._set_store_range(0, a.size, gc.createRaw([a.size], np.arange(a.size, dtype=np.float32)))
            want_a = np.arange(a.size, dtype=np.float32).reshape(x.shape)
        elif write == "scatter":
            idx = np.zeros([1000, 1], np.float32)
            a.inplaceScatter(1, gc.createRaw([1000, 1], idx), gc.createRaw([1000, 1], np.full([1000, 1], 9.0, np.float32)))
            want_a = x.copy(); want_a[:, 0] = 9.0
        elif write == "set_range":
            a._set_ranges([0, 0], [9, 32], 7.0); want_a = x.copy(); want_a[:10] = 7.0
        else:
            # the source as the output of an op that reads the copy: b must hold the old values while a is overwritten
            gc.lib.kth_unary(40, b.storeReference, a.storeReference, a.size)      # KTH_NEG: a = -b
            want_a = -x
        assert_bits_equal(b.toArray(), x, f"pow-1 copy after {write} of the source")
        assert_bits_equal(c.toArray(), x, f"copy() after {write} of the source")
        assert_bits_equal(a.toArray(), want_a, f"the source after {write}")


def test_writing_the_copy_leaves_the_source_alone(gc):
    x = data([64, 48, 40], 3)
    a = gc.createRaw(list(x.shape), x)
    b = a.copy()
    c = a._scalar("pow", 1.0)
    b._scalar_assign("times", 2.0)
    c._binary_assign("minus", a)
    assert_bits_equal(a.toArray(), x, "source")
    assert_bits_equal(b.toArray(), x * np.float32(2), "copy *= 2")
    assert_bits_equal(c.toArray(), x - x, "copy -= source")
    # a copy that is overwritten whole
    d = a.copy()
    d.inplaceFill(1.5)
    assert_bits_equal(d.toArray(), np.full_like(x, 1.5), "copy, then fill")
    assert_bits_equal(a.toArray(), x, "source after the copy was filled")


def test_a_source_released_first_hands_its_values_over(gc):
    x = data([70001], 4)
    # one copy: it takes the buffer over, no kernel
    a = gc.createRaw([70001], x)
    b = a._scalar("pow", 1.0)
    before = launches(gc)
    a.release()
    assert launches(gc) == before, "the buffer changes hands"
    assert_bits_equal(b.toArray(), x, "copy after the source was released")
    b._scalar_assign("plus", 1.0)
    assert_bits_equal(b.toArray(), x + np.float32(1), "and written")
    # several copies, and a copy of a copy (which aliases the first source)
    a = gc.createRaw([70001], x)
    b, c = a.copy(), a._scalar("pow", 1.0)
    d = c.copy()
    c.release()
    a.release()
    for t, name in ((b, "first copy"), (d, "copy of a copy")):
        assert_bits_equal(t.toArray(), x, f"{name} after source and middle copy were released")
    b._scalar_assign("times", 0.0)
    assert_bits_equal(d.toArray(), x, "copy of a copy after its sibling was written")
    # a copy into a smaller store than the source's (another size class): its values are copied at the release
    big = gc.createRaw([3, 70001], np.stack([x, x + 1, x + 2]))
    small = gc.createRaw([70001])
    gc.lib.kth_copy(small.storeReference, 0, big.storeReference, 0, 70001)
    big.release()
    assert_bits_equal(small.toArray(), x, "head of a larger store, released")


def test_views_and_shallow_copies_share_the_put_off_copy(gc):
    x = data([12, 17], 5)
    a = gc.createRaw([12, 17], x)
    b = a.copy()
    before = launches(gc)
    v = b.view([204])
    w = b.copy(shallow=True)
    assert launches(gc) == before
    a._scalar_assign("plus", 10.0)                  # the copy is made here, once, for b, v and w alike
    v._scalar_assign("times", 2.0)
    assert_bits_equal(b.toArray(), x * np.float32(2), "written through a view")
    assert_bits_equal(w.toArray(), x * np.float32(2), "shallow copy")
    assert_bits_equal(a.toArray(), x + np.float32(10), "source")


def test_a_constant_source_passes_its_note_on(gc):
    a = gc.createRawFill([500, 500], 3.0)
    before = launches(gc)
    b = a.copy()
    c = b._scalar("times", 2.0)
    assert launches(gc) == before, "constants fold, nothing runs"
    a.inplaceFill(1.0)
    assert_bits_equal(b.toArray(), np.full([500, 500], 3.0, np.float32), "copy of a constant")
    assert_bits_equal(c.toArray(), np.full([500, 500], 6.0, np.float32), "twice the copy")
    assert_bits_equal(a.toArray(), np.full([500, 500], 1.0, np.float32), "refilled source")


def test_the_backward_pass_of_a_square_copies_nothing(gc):
    """x.pow(2).sum().backward(): the gradient 2 * x'pow(1) * seed reads x through the put-off copy."""
    x = data([512, 384], 6)
    t = gc.create([512, 384], True, x)
    gc.profileBegin()
    loss = t.pow(2.0).sum()
    loss.backward()
    kernels = gc.profileEnd()
    assert not any(k.startswith("copy_kernel") or "OpIdentity" in k for k in kernels), sorted(kernels)
    assert_bits_equal(t.grad().toArray(), np.float32(2) * x, "gradient of a sum of squares")
