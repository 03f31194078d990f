"""Tensors at the top of the 32-bit element range (a Kotlin Int indexes the store, so
2^31 - 1 elements is the contract's limit): every kernel family once, checked through
values that are known in closed form, so that no host array of that size is needed.
x[i, j] = r[i] + c[j] is built on the device by a doubly broadcast add."""
import numpy as np
import pytest

from kten_amd.host_mirror.shape_functions import ALL
from oracle import jvm_oracle as jo

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


def test_three_dimensional_tensor_near_the_limit(gc):
    """x[i, j, k] = r[i] + s[j] + c[k] on [2047, 1024, 1024] (2 146 435 072 elements): the kernels that the
    two-dimensional case does not reach -- reductions over a middle axis in their streamed, tiled and few-rows
    forms, a permute that keeps an innermost run, gather and scatter-add of rows inside LDS, indexSelect, the
    sorted indexAdd and the fused batch-norm -- with offsets at the top of the 32-bit range. Values are multiples
    of 1/8, so every expected value is exact in float32 or float64."""
    A, B, C = 2047, 1024, 1024
    rng = np.random.default_rng(2)
    gc.profileBegin()                             # the names of the kernels launched are checked at the end
    eighths = lambda n: (rng.integers(-256, 256, n) / 8.0).astype(np.float32)
    r, s, c = eighths(A), eighths(B), eighths(C)
    rs = gc.createRaw([A, 1, 1], r).plus(gc.createRaw([B, 1], s))
    x = rs.plus(gc.createRaw([C], c))
    assert x.shape == [A, B, C]
    gc.release(rs)
    pos = [(0, 0, 0), (A - 1, B - 1, C - 1), (A - 1, 0, C - 1), (1023, 512, 7)]
    pos += [(int(rng.integers(0, A)), int(rng.integers(0, B)), int(rng.integers(0, C))) for _ in range(30)]
    val = lambda i, j, k: np.float32(np.float32(r[i] + s[j]) + c[k])
    for i, j, k in pos:
        assert x.getSingleValue([i, j, k]) == val(i, j, k)
    r64, s64, c64 = r.astype(np.float64), s.astype(np.float64), c.astype(np.float64)

    # a middle axis streamed by a workgroup per slab segment: [A, B * 4, 256] over axis 1
    got = x.view([A, B * 4, 256]).sum(1).toArray().astype(np.float64)
    want = 4 * B * r64[:, None] + 4 * s64.sum() + B * c64.reshape(4, 256).sum(0)[None, :]
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()
    # small slabs through LDS tiles: [A * B, 64, 16] over axis 1
    got = x.view([A * B, 64, 16]).sum(1).toArray().astype(np.float64).reshape(A, B, 16)
    want = 64 * (r64[:, None, None] + s64[None, :, None]) + c64.reshape(64, 16).sum(0)[None, None, :]
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()
    # an axis of two over wide columns: [A * B / 8, 2, 4096]; the maximum of x[.., j, :] and x[.., j + 1, :] for even j,
    # seen as rows of four (i, j) pairs
    got = x.view([A * B // 8, 2, 4096]).max(1).toArray().reshape(A, B // 8, 4, C)
    for i, j, k in pos:
        g, q = divmod(j, 8)                       # q 0..3 pairs with q + 4
        if q < 4:
            assert got[i, g, q, k] == max(val(i, j, k), val(i, j + 4, k))
    del got

    # a permute that keeps the innermost run of 8 floats: [A, B, 128, 8] -> [A, 128, B, 8]
    p = x.view([A, B, 128, 8]).permute([0, 2, 1, 3])
    assert p.shape == [A, 128, B, 8]
    for i, j, k in pos:
        assert p.getSingleValue([i, k // 8, j, k % 8]) == val(i, j, k)
    gc.release(p)

    # gather and scatter-add along the innermost axis with rows of 128 indices (the row lives in LDS)
    cols = rng.integers(0, C, 128)
    zeros = gc.createRawFill([A, B, 1], 0.0)
    index = zeros.plus(gc.createRaw([128], cols.astype(np.float32)))
    assert index.shape == [A, B, 128]
    g = x.gather(2, index)
    for i, j, k in pos:
        m = k % 128
        assert g.getSingleValue([i, j, m]) == val(i, j, int(cols[m]))
    gc.release(g)
    ones = gc.createRawFill([A, B, 128], 1.0)
    x.inplaceScatterAdd(2, index, ones)
    hits = np.bincount(cols, minlength=C).astype(np.float32)
    for i, j, k in pos:
        assert x.getSingleValue([i, j, k]) == np.float32(val(i, j, k) + hits[k])      # small integers added to eighths: exact
    minus = gc.createRawFill([A, B, 128], -1.0)
    x.inplaceScatterAdd(2, index, minus)                                               # and taken off again
    for i, j, k in pos:
        assert x.getSingleValue([i, j, k]) == val(i, j, k)
    gc.release(index, ones, minus, zeros)

    # indexSelect and the sorted indexAdd along axis 0, the last rows of the tensor among them
    rows = np.concatenate([[A - 1, 0, A - 1], rng.integers(0, A, 61)]).astype(np.float32)
    sel = x.indexSelect(0, gc.createRaw([64], rows))
    assert sel.shape == [64, B, C]
    for m in (0, 1, 2, 40, 63):
        for _, j, k in pos[:8]:
            assert sel.getSingleValue([m, j, k]) == val(int(rows[m]), j, k)
    x.indexAdd(0, gc.createRaw([64], rows), sel, -1.0)          # x[row] -= x[row], once per occurrence of the row
    times = np.bincount(rows.astype(np.int64), minlength=A)
    for i, j, k in pos:
        v = val(i, j, k)
        want = v
        for _ in range(int(times[i])):
            want = np.float32(want + np.float32(v * np.float32(-1.0)))
        assert x.getSingleValue([i, j, k]) == want
    gc.release(sel)

    # the fused batch-norm over axis 1: statistics of 2 M elements per channel at offsets up to 2^31
    y = gc.createRaw([A, 1, 1], r).plus(gc.createRaw([B, 1], s)).plus(gc.createRaw([C], c))          # x again, untouched
    op = gc.batchNorm(1, 0.1, 1e-3, True)
    out, mean, std = op.calculateOutput(y, gc.createRawFill([B], 0.0), gc.createRawFill([B], 1.0), None, None)
    mean64 = s64 + r64.mean() + c64.mean()
    var64 = r64.var() + c64.var()                                  # r and c vary independently over a channel's elements
    assert np.abs(mean.toArray() - mean64).max() <= 1e-5 * np.abs(mean64).max() + 1e-6
    assert np.abs(std.toArray() - 1.0 / np.sqrt(var64 + 1e-3)).max() <= 1e-5 / np.sqrt(var64 + 1e-3)
    dm, ds = mean.toArray(), std.toArray()
    chan = np.array([j for _, j, _ in pos])
    want = jo.batch_norm_apply(np.array([val(i, j, k) for i, j, k in pos], np.float32), 0, dm[chan], ds[chan])
    for (i, j, k), w in zip(pos, want):
        assert out.getSingleValue([i, j, k]) == w

    # gather and scatter along axis 0 with 256 index rows (a million positions walk them side by side)
    perm = rng.permutation(A)[:256]
    perm[0], perm[1] = A - 1, 0
    q = eighths(256)
    plane = gc.createRawFill([B, C], 0.0)
    index0 = gc.createRaw([256, 1, 1], perm.astype(np.float32)).plus(plane)
    src0 = gc.createRaw([256, 1, 1], q).plus(plane)
    assert index0.shape == [256, B, C]
    g0 = y.gather(0, index0)
    for m in (0, 1, 2, 100, 255):
        for _, j, k in pos[:8]:
            assert g0.getSingleValue([m, j, k]) == val(int(perm[m]), j, k)
    gc.release(g0)
    y.inplaceScatter(0, index0, src0)
    row_of = {int(p): m for m, p in enumerate(perm)}
    for i, j, k in pos + [(A - 1, 5, 9), (0, B - 1, C - 1)]:
        want = q[row_of[i]] if i in row_of else val(i, j, k)
        assert y.getSingleValue([i, j, k]) == want

    launched = " ".join(gc.profileEnd().keys())
    for kernel in ("reduce_stream_kernel", "reduce_short_slabs_kernel", "reduce_few_kernel", "permute_runs_kernel",
                   "gather_rows_lds_kernel", "scatter_rows_lds_kernel<add>", "scatter_kernel<set>", "index_select_kernel",
                   "index_add_sorted_kernel", "bn_stats", "bn_apply"):
        assert kernel in launched, f"{kernel} was not reached: {launched}"


def test_scatter_along_a_long_axis_near_the_limit(gc):
    """inplaceScatter along axis 0 of [1 048 575, 2047] with an index of the same shape: target, index and source
    are permuted to axis-innermost layout (rows of a million elements, scattered in bands through LDS) and the
    target is permuted back; every copy holds 2 146 433 025 elements."""
    R, W = 1048575, 2047
    rng = np.random.default_rng(3)
    perm = rng.permutation(R)
    q = (rng.integers(-1024, 1024, R) / 8.0).astype(np.float32)
    zeros = gc.createRawFill([W], 0.0)
    index = gc.createRaw([R, 1], perm.astype(np.float32)).plus(zeros)
    src = gc.createRaw([R, 1], q).plus(gc.createRaw([W], np.arange(W, dtype=np.float32)))      # src[i, j] = q[i] + j, exact
    x = gc.createRawFill([R, W], -5.0)
    gc.profileBegin()
    x.inplaceScatter(0, index, src)
    launched = " ".join(gc.profileEnd().keys())
    assert "scatter_rows_lds_kernel<set>" in launched and "permute_tile_kernel" in launched, launched
    where = np.empty(R, np.int64); where[perm] = np.arange(R)          # x[perm[i], j] = src[i, j]
    rows = [0, R - 1, int(perm[0]), int(perm[-1])] + [int(v) for v in rng.integers(0, R, 30)]
    for row in rows:
        for j in (0, 1, W // 2, W - 1):
            assert x.getSingleValue([row, j]) == np.float32(q[where[row]] + np.float32(j))
    # the index survives the call untouched
    for i in (0, R - 1, 12345):
        assert index.getSingleValue([i, W - 1]) == float(perm[i])


def test_sorted_and_wave_scatter_near_the_limit(gc):
    """The scatter forms for one long index row and for many short ones, at offsets and keys at the top of the
    32-bit range. A flat target of 2^31 - 2 elements with one index row of 2^24 entries is sorted by element
    (keys up to 2^31 - 128, the last element a float32 index can name; the key for a bad entry is 2^31 - 2); a
    [1 048 575, 2047] target with index rows of 40 entries takes a wave per row. Sampled elements are checked against the entries that name them, in row order."""
    T, K = 2 ** 31 - 2, 2 ** 24
    TOP = 2 ** 31 - 128                                                  # the last element a float32 index can name
    rng = np.random.default_rng(6)
    idx_f = rng.integers(0, T, K).astype(np.float32)                     # the device sees the rounded values
    idx_f[idx_f > TOP] = TOP
    idx_f[0], idx_f[1], idx_f[-1], idx_f[-2] = TOP, 0, TOP, 0            # both ends, each named at least twice
    idx_f[1000:1400] = idx_f[500]                                        # a run of equal keys
    idx = idx_f.astype(np.int64)
    src = (rng.integers(-512, 512, K) / 8.0).astype(np.float32)
    order = np.argsort(idx, kind="stable")
    sorted_idx = idx[order]
    def entries_of(element):                                             # in the order of the index row
        lo, hi = np.searchsorted(sorted_idx, element, "left"), np.searchsorted(sorted_idx, element, "right")
        return order[lo:hi]
    sampled = [TOP, 0, int(idx[500])] + [int(v) for v in idx[rng.integers(0, K, 40)]]
    untouched = [int(v) for v in rng.integers(0, T, 20)] + [T - 1]
    untouched = [v for v in untouched if entries_of(v).size == 0]
    g_idx, g_src = gc.createRaw([K], idx_f), gc.createRaw([K], src)
    for mode in ("set", "add", "fill"):
        x = gc.createRawFill([T], -5.0)
        gc.profileBegin()
        if mode == "set": x.inplaceScatter(0, g_idx, g_src)
        elif mode == "add": x.inplaceScatterAdd(0, g_idx, g_src)
        else: x.inplaceScatter(0, g_idx, 3.5)
        launched = " ".join(gc.profileEnd().keys())
        assert "scatter_sort" in launched, launched
        for element in sampled:
            e = entries_of(element)
            assert e.size > 0
            if mode == "set": want = src[e[-1]]
            elif mode == "fill": want = np.float32(3.5)
            else:
                want = np.float32(-5.0)
                for i in e: want = np.float32(want + src[i])
            assert x.getSingleValue([element]) == want, (mode, element)
        for element in untouched:
            assert x.getSingleValue([element]) == -5.0
        gc.release(x)
    gc.release(g_idx, g_src)

    R, W, L = 1048575, 2047, 40
    pos = rng.integers(0, W, (R, L))
    pos[:, 7] = pos[:, 3]                                                # every row names one element twice
    val = (rng.integers(-512, 512, (R, L)) / 8.0).astype(np.float32)
    g_pos, g_val = gc.createRaw([R, L], pos.astype(np.float32)), gc.createRaw([R, L], val)
    rows = [0, R - 1, R - 2] + [int(v) for v in rng.integers(0, R, 40)]
    for mode in ("set", "add"):
        y = gc.createRawFill([R, W], 0.25)
        gc.profileBegin()
        if mode == "set": y.inplaceScatter(1, g_pos, g_val)
        else: y.inplaceScatterAdd(1, g_pos, g_val)
        launched = " ".join(gc.profileEnd().keys())
        assert "scatter_wave_kernel" in launched, launched
        for row in rows:
            want = np.full(W, 0.25, np.float32)
            for j in range(L):
                want[pos[row, j]] = val[row, j] if mode == "set" else np.float32(want[pos[row, j]] + val[row, j])
            got = y.get([(row, row), ALL]).toArray().reshape(-1)
            assert np.array_equal(got, want), (mode, row)
        gc.release(y)


def test_broadcast_with_a_large_repeating_operand_near_the_limit(gc):
    """x[i, j, k] = r[i] + y[j, k] on [64, 4095, 8188] (2 145 911 040 elements) with y of 134 MB repeating along the outermost
    dim: the vector kernel takes the output's tiles chunk by chunk across the 64 repeats; then z = x + y with one operand
    full-size. Values are multiples of 1/8: every sum is exact."""
    A, B, C = 64, 4095, 8188
    rng = np.random.default_rng(8)
    r = (rng.integers(-512, 512, A) / 8.0).astype(np.float32)
    y = (rng.integers(-512, 512, (B, C)) / 8.0).astype(np.float32)
    gr, gy = gc.createRaw([A, 1, 1], r), gc.createRaw([1, B, C], y)
    gc.profileBegin()
    x = gr.plus(gy)
    z = x.plus(gy)
    launched = " ".join(gc.profileEnd().keys())
    assert launched.count("_chunked") == 2, launched
    pos = [(0, 0, 0), (A - 1, B - 1, C - 1), (A - 1, 0, 0), (0, B - 1, C - 1), (A - 1, B - 1, 0), (31, 2047, 4093)]
    pos += [(int(rng.integers(0, A)), int(rng.integers(0, B)), int(rng.integers(0, C))) for _ in range(60)]
    for i, j, k in pos:
        assert x.getSingleValue([i, j, k]) == r[i] + y[j, k]
        assert z.getSingleValue([i, j, k]) == r[i] + y[j, k] + y[j, k]
    # the last rows of the last slice, whole: the tiles that end with the slice and with the tensor
    tail = z.get([(A - 1, A - 1), (B - 2, B - 1), ALL]).toArray().reshape(2, C)
    assert np.array_equal(tail, r[-1] + 2 * y[-2:, :])


def test_odd_shaped_tensor_near_the_limit(gc):
    """x[i, j] = r[i] + c[j] on [46339, 46337] (2 147 210 243 elements, rows that start off 16-byte boundaries):
    the forms the kernels take when nothing is a multiple of four -- element gathers in the broadcast, rows read
    from dword addresses in the reductions, scalar columns, ragged tile edges in the transpose, the mixed range
    moves, concat."""
    R, W = 46339, 46337
    rng = np.random.default_rng(4)
    r = (rng.integers(-512, 512, R) / 8.0).astype(np.float32)
    c = (rng.integers(-512, 512, W) / 8.0).astype(np.float32)
    gc.profileBegin()
    gcol = gc.createRaw([W], c)
    x = gc.createRaw([R, 1], r).plus(gcol)
    assert x.shape == [R, W]
    pos = [(0, 0), (R - 1, W - 1), (R - 1, 0), (0, W - 1), (R - 2, W - 3)]
    pos += [(int(rng.integers(0, R)), int(rng.integers(0, W))) for _ in range(30)]
    val = lambda i, j: np.float32(r[i] + c[j])
    for i, j in pos:
        assert x.getSingleValue([i, j]) == val(i, j)
    y = x.plus(gcol)                                                     # full-size operand and a row vector
    for i, j in pos:
        assert y.getSingleValue([i, j]) == np.float32(val(i, j) + c[j])
    gc.release(y)
    r64, c64 = r.astype(np.float64), c.astype(np.float64)
    got = x.sum(1).toArray().astype(np.float64)
    want = W * r64 + c64.sum()
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()
    got = x.sum(0).toArray().astype(np.float64)
    want = r64.sum() + R * c64
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()
    arg = x.argMax(1).toArray()
    assert arg[0] == np.argmax(c) and arg[-1] == np.argmax(c) and np.all(c[arg.astype(np.int64)] == c.max())
    arg = x.argMin(0).toArray()
    assert arg[0] == np.argmin(r) and arg[-1] == np.argmin(r)

    t = x.transpose(0, 1)
    for i, j in pos:
        assert t.getSingleValue([j, i]) == val(i, j)
    gc.release(t)
    box = x.get([(1, R - 2), (3, W - 2)])                                # rows of W - 4 floats cut out of rows of W
    assert box.shape == [R - 2, W - 4]
    for i, j in pos:
        if 1 <= i <= R - 2 and 3 <= j <= W - 2:
            assert box.getSingleValue([i - 1, j - 3]) == val(i, j)
    assert box.getSingleValue([R - 3, W - 5]) == val(R - 2, W - 2)
    gc.release(box)
    wide = gc.concat(1, [x, gc.createRaw([R, 3], np.tile(np.array([1.0, 2.0, 3.0], np.float32), (R, 1)))])
    assert wide.shape == [R, W + 3]
    for i, j in pos:
        assert wide.getSingleValue([i, j]) == val(i, j)
    assert wide.getSingleValue([R - 1, W + 2]) == 3.0 and wide.getSingleValue([0, W]) == 1.0
    gc.release(wide)
    x.set([(5, R - 1), (1, W - 1)], 9.0)
    for i, j in pos:
        assert x.getSingleValue([i, j]) == (9.0 if i >= 5 and j >= 1 else val(i, j))
    launched = " ".join(gc.profileEnd().keys())
    for kernel in ("binary_bcast_mixed_kernel", "reduce_rows_kernel", "reduce_cols_kernel", "permute_tile_kernel", "float4 dense side"):
        assert kernel in launched, f"{kernel} was not reached: {launched}"
