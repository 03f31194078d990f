"""Tensors at the top of the 32-bit element range (a Kotlin Int indexes the store, so
2^31 - 1 elements is the contract's limit): every kernel family once, checked through
values that are known in closed form, so that no host array of that size is needed.
x[i, j] = r[i] + c[j] is built on the device by a doubly broadcast add."""
import numpy as np
import pytest

from kten_amd.shape_functions import ALL

pytestmark = pytest.mark.gpu

ROWS, COLS = 32767, 65536                 # 2 147 418 112 elements, 8.6 GB per tensor
MAX = 2 ** 31 - 1


def sample_positions(rng, count):
    pos = [(0, 0), (ROWS - 1, COLS - 1), (ROWS - 1, 0), (0, COLS - 1), (16383, 32768), (32766, 65535)]
    pos += [(int(rng.integers(0, ROWS)), int(rng.integers(0, COLS))) for _ in range(count)]
    return pos


def test_two_dimensional_tensor_near_the_limit(gc):
    rng = np.random.default_rng(1)
    r = (rng.integers(-512, 512, ROWS) / 8.0).astype(np.float32)         # exactly representable sums below
    c = (rng.integers(-512, 512, COLS) / 8.0).astype(np.float32)
    gr, gcol = gc.createRaw([ROWS, 1], r), gc.createRaw([COLS], c)
    x = gr.plus(gcol)                                                    # both operands broadcast
    assert x.shape == [ROWS, COLS]
    pos = sample_positions(rng, 40)
    for i, j in pos:
        assert x.getSingleValue([i, j]) == r[i] + c[j]
    y = x.times(x)                                                       # same-shape binary
    z = y.plus(1.0)                                                      # scalar
    w = z.sqrt()                                                         # unary
    for i, j in pos:
        v = np.float32(r[i] + c[j])
        assert y.getSingleValue([i, j]) == v * v
        assert w.getSingleValue([i, j]) == np.sqrt(np.float32(v * v + np.float32(1.0)))
    gc.release(y, z, w)

    # reductions: column sums, row sums, full sum (sums of multiples of 1/8 are exact in f64)
    col_sum = x.sum(0).toArray().astype(np.float64)
    want = r.astype(np.float64).sum() + ROWS * c.astype(np.float64)
    assert np.abs(col_sum - want).max() <= 1e-6 * np.abs(want).max()
    row_sum = x.sum(1).toArray().astype(np.float64)
    want = COLS * r.astype(np.float64) + c.astype(np.float64).sum()
    assert np.abs(row_sum - want).max() <= 1e-6 * np.abs(want).max()
    total = float(x.sum().toArray()[0])
    want = COLS * r.astype(np.float64).sum() + ROWS * c.astype(np.float64).sum()
    assert abs(total - want) <= 1e-6 * max(abs(want), 1.0) + 64.0        # f32 rounding of a 2^31-term sum's result
    arg = x.argMax(1).toArray()
    assert np.all(c[arg.astype(np.int64)] == c.max())                    # the row's maximum sits where c is largest
    assert arg[0] == np.argmax(c) and arg[-1] == np.argmax(c)            # ties resolve to the lowest index

    # layout movers
    t = x.transpose(0, 1)
    assert t.shape == [COLS, ROWS]
    for i, j in pos:
        assert t.getSingleValue([j, i]) == r[i] + c[j]
    gc.release(t)
    tail = x.get([(ROWS - 2, ROWS - 1), (COLS - 8, COLS - 1)]).toArray()
    assert np.array_equal(tail, r[-2:, None] + c[None, -8:])
    x.set([(ROWS - 1, ROWS - 1), ALL], -1.0)
    assert x.getSingleValue([ROWS - 1, COLS - 1]) == -1.0 and x.getSingleValue([ROWS - 2, COLS - 1]) == r[-2] + c[-1]
    m = x.maskedFill(gc.createRaw([COLS], (np.arange(COLS) % 2).astype(np.float32)), 7.0)
    assert m.getSingleValue([ROWS - 2, COLS - 1]) == 7.0 and m.getSingleValue([ROWS - 2, COLS - 2]) == r[-2] + c[-2]


def test_flat_tensor_of_exactly_int_max_elements(gc):
    x = gc.createRawFill([MAX], 1.5)
    assert x.getSingleValue([MAX - 1]) == 1.5
    y = x.times(2.0)
    assert y.getSingleValue([MAX - 1]) == 3.0 and y.getSingleValue([0]) == 3.0 and y.getSingleValue([MAX - 2]) == 3.0
    y.plusAssign(x)
    assert y.getSingleValue([MAX - 1]) == 4.5
    assert float(x.sum().toArray()[0]) == float(np.float32(1.5 * MAX))
    assert float(x.mean().toArray()[0]) == 1.5
    e = x.exp()
    assert e.getSingleValue([MAX - 1]) == np.float32(np.exp(np.float64(1.5)))
    assert not x.containsNan()
    x.set([MAX - 1], float("nan"))
    assert x.containsNan()
    with pytest.raises((ValueError, MemoryError)):
        gc.createRaw([2, 2 ** 30])                                       # 2^31 elements: one past the limit
