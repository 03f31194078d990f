"""Host-side logic that needs no GPU: the C-ABI library loads and exports every symbol
the header declares, entry points refuse to run before kth_init, the shape algebra and
error behaviour of the contract mirror, the seeded generator, the workloads' byte counts.
"""
import ctypes
import os
import re

import numpy as np
import pytest

from kten_amd import abi
from kten_amd.host_mirror import shape_functions as sf
from kten_amd.host_mirror.inputs import SplitMix64
from kten_amd.host_mirror.workloads import WORKLOADS

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols(name="kten_hip.h"):
    text = open(os.path.join(ROOT, "include", name)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kth_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = abi.load()
    names = header_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/kten_hip.h but not exported"
    assert sorted(abi.SIGNATURES) == names, "abi.SIGNATURES and include/kten_hip.h declare different entry points"


def test_library_exports_the_measurement_entry_points_of_their_own_header():
    lib = abi.load()
    names = header_symbols("kten_hip_bench.h")
    assert len(names) >= 9
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/kten_hip_bench.h but not exported"
    assert sorted(abi.BENCH_SIGNATURES) == names
    # The contract header holds none of them: a host that binds the contract does not meet them.
    assert not set(names) & set(header_symbols())
    assert not [n for n in header_symbols() if re.match(r"kth_(timer|profile|measure)_", n)]


def test_entry_points_refuse_to_run_before_init():
    import subprocess, sys
    # A fresh process, so that an initialised library elsewhere in this session cannot interfere.
    code = ("import ctypes, sys; sys.path.insert(0, %r); from kten_amd import abi; L = abi.load(); h = ctypes.c_uint64();"
            "rc = L.kth_alloc(16, ctypes.byref(h)); print(rc, abi.last_error())" % ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, check=True).stdout
    assert out.startswith(f"{abi.KTH_E_NOT_INIT} "), out
    assert "kth_init" in out


def test_status_codes_map_to_reference_exception_classes(monkeypatch):
    monkeypatch.setattr(abi, "last_error", lambda: "msg")
    with pytest.raises(ValueError):
        abi.check(abi.KTH_E_SHAPE)          # IllegalArgumentException
    with pytest.raises(ValueError):
        abi.check(abi.KTH_E_ARGUMENT)
    with pytest.raises(MemoryError):
        abi.check(abi.KTH_E_MEMORY)
    with pytest.raises(RuntimeError):
        abi.check(abi.KTH_E_DEVICE)
    abi.check(abi.KTH_OK)


# ---------------------------------------------------------------- shape algebra

def test_normalize_axis():
    assert sf.normalize_axis([2, 3, 4], -1) == 2 and sf.normalize_axis([2, 3, 4], 0) == 0
    for bad in (3, -4):
        with pytest.raises(ValueError):
            sf.normalize_axis([2, 3, 4], bad)


def test_aggregate_over_never_goes_0d():
    assert sf.aggregate_over([3, 4], 0, False) == [4]
    assert sf.aggregate_over([3, 4], 1, True) == [3, 1]
    assert sf.aggregate_over([5], 0, False) == [1]          # stays [1]


def test_broadcast_shape_inference():
    assert sf.infer_implicit_broadcast_shape([3, 1], [1, 3]) == [3, 3]
    assert sf.infer_implicit_broadcast_shape([4], [2, 3, 4]) == [2, 3, 4]
    assert sf.infer_explicit_broadcast_shape([1], [3, 3]) == [3, 3]
    with pytest.raises(ValueError):
        sf.infer_implicit_broadcast_shape([3], [4])
    with pytest.raises(ValueError):
        sf.infer_explicit_broadcast_shape([2, 3], [3])       # explicit broadcast never drops dims
    with pytest.raises(ValueError):
        sf.infer_explicit_broadcast_shape([3, 3], [3, 1])    # nor shrinks them


def test_reshape_squeeze_unsqueeze():
    assert sf.reshape([2, 3, 4], [-1, 4]) == [6, 4]
    with pytest.raises(ValueError):
        sf.reshape([2, 3], [4, -1, -1])
    with pytest.raises(ValueError):
        sf.reshape([2, 3], [4, 2])
    assert sf.squeeze([2, 1, 3], 1) == [2, 3]
    with pytest.raises(ValueError):
        sf.squeeze([2, 1, 3], 0)
    assert sf.unsqueeze([2, 3], 0) == [1, 2, 3]
    assert sf.unsqueeze([2, 3], 2) == [2, 3, 1]
    assert sf.unsqueeze([2, 3], -1) == [2, 3, 1]
    assert sf.unsqueeze([2, 3], -3) == [1, 2, 3]


def test_store_index_row_major_and_bounds():
    assert sf.store_index([2, 3, 4], [1, 2, 3]) == 23
    assert sf.store_index([2, 3, 4], [-1, 0, 0]) == 12
    with pytest.raises(ValueError):
        sf.store_index([2, 3], [0, 3])


def test_contract_error_behaviour_on_the_host(oracle_ops):
    # The same checks guard the HIP backend before any launch; exercised here on the CPU
    # implementation of the contract.
    a = oracle_ops.createRaw([2, 3], [1, 2, 3, 4, 5, 6])
    b = oracle_ops.createRaw([3, 2], [1, 2, 3, 4, 5, 6])
    with pytest.raises(ValueError):
        a.plusAssign(b)                                       # in-place needs equal shapes
    with pytest.raises(ValueError):
        a.plus(b)                                             # [2,3] and [3,2] do not broadcast
    with pytest.raises(ValueError):
        a.sum(2)
    assert a.sum(0).shape == [3] and a.sum(-1, True).shape == [2, 1]
    v = oracle_ops.createRaw([4], [1, 2, 3, 4])
    assert v.sum(0).shape == [1] and v.argMax(0).shape == [1]
    assert a.broadcastTo([2, 3]) is a                         # equal shape returns this
    assert a.calculateCommonShapeWith(oracle_ops.createRaw([4, 1, 3])) == [4, 2, 3]


def test_may_unexpand_axis_order(oracle_ops):
    from kten_amd.host_mirror.autograd import mayUnexpand
    calls = []
    g = oracle_ops.createRaw([2, 3, 4, 5], np.arange(120, dtype=np.float32))
    orig = type(g).sum
    def spy(self, axis=None, keepDimensions=False):
        calls.append((axis, keepDimensions, list(self.shape)))
        return orig(self, axis, keepDimensions)
    type(g).sum = spy
    try:
        res = mayUnexpand(g, [1, 3, 1, 1], oracle_ops)
        assert calls == [(0, True, [2, 3, 4, 5]), (2, True, [1, 3, 4, 5]), (3, True, [1, 3, 1, 5])]
        assert res.shape == [1, 3, 1, 1]
        np.testing.assert_array_equal(res.toArray(), np.arange(120, dtype=np.float32).reshape(2, 3, 4, 5).sum((0, 2, 3), keepdims=True))
        calls.clear()
        res = mayUnexpand(oracle_ops.createRaw([6, 4], np.ones(24, np.float32)), [1], oracle_ops)
        assert calls == [(0, False, [6, 4]), (0, True, [4])] and res.shape == [1] and res.toArray()[0] == 24
    finally:
        type(g).sum = orig


# ---------------------------------------------------------------- generator and workloads

def test_splitmix64_published_vectors():
    # First outputs of the reference SplitMix64 implementation for seed 1234567.
    assert SplitMix64(1234567).next_u64(5).tolist() == [6457827717110365317, 3203168211198807973, 9817491932198370423,
                                                         4593380528125082431, 16408922859458223821]
    g = SplitMix64(7)
    a = g.next_u64(3); b = g.next_u64(4)
    assert np.concatenate([a, b]).tolist() == SplitMix64(7).next_u64(7).tolist()      # one stream, any chunking


def test_generator_distributions_and_determinism():
    u = SplitMix64(0).uniform([100000], -1.0, 1.0)
    assert u.dtype == np.float32 and u.min() >= -1.0 and u.max() < 1.0 and abs(u.mean()) < 0.01
    assert u[:2].view(np.uint32).tolist() == [1061437776, 3188472592]
    n = SplitMix64(1).normal([100001])
    assert n.shape == (100001,) and abs(n.mean()) < 0.02 and abs(n.std() - 1) < 0.02
    assert np.array_equal(n[:1000], SplitMix64(1).normal([1000]))
    assert np.isfinite(n).all()


def test_algorithmic_bytes_match_the_published_plan():
    want = {"cfg1": 50335748, "cfg2": 4563402752, "cfg3": 1610809344, "cfg4": 623101952}
    for name, b in want.items():
        wl = WORKLOADS[name]
        assert wl.algorithmic_bytes(wl.full_dims) == b
    wl = WORKLOADS["cfg5"]
    m = 16384 * 4096
    got = wl.algorithmic_bytes(wl.full_dims)
    assert 22 * m * 4 <= got <= 22 * m * 4 + 200000


def test_workload_byte_formula_equals_the_ops_it_runs(oracle_ops):
    # Count bytes op by op on the CPU implementation of the contract (operands at their
    # true size + output; in-place: target twice + other) and compare with the formula.
    import contextlib
    from oracle.jvm_oracle import JvmOracleRawTensor as R
    counted = [0]
    saved = {}

    def wrap(name, cost):
        orig = getattr(R, name)
        saved[name] = orig
        def f(self, *a, **k):
            res = orig(self, *a, **k)
            counted[0] += cost(self, a + tuple(k.values()), res)
            return res
        setattr(R, name, f)

    size = lambda t: int(np.prod(t.shape))
    wrap("_binary", lambda s, a, r: size(s) + size(a[1]) + size(r))
    wrap("_binary_assign", lambda s, a, r: 2 * size(s) + size(a[1]))
    wrap("_scalar", lambda s, a, r: size(s) + size(r))
    wrap("_scalar_assign", lambda s, a, r: 2 * size(s))
    wrap("_unary", lambda s, a, r: size(s) + size(r))
    wrap("aggregateOverAxis", lambda s, a, r: size(s) + size(r))
    wrap("_sum_all", lambda s, a, r: size(s) + 1)
    wrap("broadcastTo", lambda s, a, r: 0 if r is s else size(s) + size(r))
    wrap("_mean_all", lambda s, a, r: size(s) + 1)
    wrap("clamp", lambda s, a, r: size(s) + size(r))
    wrap("gather", lambda s, a, r: 3 * size(r))
    wrap("_scatter", lambda s, a, r: size(a[1]) * (2 if isinstance(a[2], float) else 4 if a[3] else 3))
    wrap("inplaceFill", lambda s, a, r: size(s))
    wrap("copy", lambda s, a, r: 0 if (a and a[0]) else 2 * size(s))        # deep copies only
    box = lambda first, last: int(np.prod([l - f + 1 for f, l in zip(first, last)]))
    wrap("_get_ranges", lambda s, a, r: 2 * size(r))
    wrap("_set_ranges", lambda s, a, r: box(a[0], a[1]) * (1 if isinstance(a[2], float) else 2))
    wrap("_transpose", lambda s, a, r: 2 * size(s))
    wrap("_permute", lambda s, a, r: 2 * size(s))
    wrap("maskedFill", lambda s, a, r: 2 * size(s) + size(a[0]))
    orig_create = type(oracle_ops).createRaw
    def counting_create(self, shape, init=None):
        if callable(init):                      # the [1] seed gradient of backward(): one store
            counted[0] += int(np.prod(shape))
        return orig_create(self, shape, init)
    type(oracle_ops).createRaw = counting_create
    orig_fill = type(oracle_ops).createRawFill
    setting_up = [False]
    def counting_fill(self, shape, constant):     # zerosLike / createRawFill: one store per element
        if not setting_up[0]:
            counted[0] += int(np.prod(shape))
        return orig_fill(self, shape, constant)
    type(oracle_ops).createRawFill = counting_fill
    orig_tensor_create = type(oracle_ops).create
    def quiet_create(self, shape, requiresGrad=False, init=None):   # creating the leaves is set-up, not part of a step
        setting_up[0] = True
        try:
            return orig_tensor_create(self, shape, requiresGrad, init)
        finally:
            setting_up[0] = False
    type(oracle_ops).create = quiet_create
    try:
        small = {"cfg1": {"rows": 8, "cols": 12}, "cfg2": {"n": 100}, "cfg3": {"rows": 6, "cols": 10},
                 "cfg4": {"n": 2, "c": 3, "h": 4, "w": 5}, "cfg5": {"rows": 8, "cols": 12},
                 "max_backward": {"rows": 6, "cols": 10}, "softmax_ce": {"batch": 6, "classes": 10},
                 "transpose": {"rows": 6, "cols": 10}, "permute": {"n": 2, "c": 3, "h": 4, "w": 5},
                 "concat_mask": {"rows": 6, "left": 4, "right": 8}}
        assert WORKLOADS["batch_norm"].algorithmic_bytes({"n": 2, "c": 3, "h": 4, "w": 5}) == 4 * (8 * 120 + 14 * 3)
        for name, dims in small.items():
            wl = WORKLOADS[name]
            counted[0] = 0
            wl.run(oracle_ops, wl.make_inputs(dims))
            assert counted[0] * 4 == wl.algorithmic_bytes(dims), name
    finally:
        type(oracle_ops).createRaw = orig_create
        type(oracle_ops).createRawFill = orig_fill
        type(oracle_ops).create = orig_tensor_create
        for name, orig in saved.items():
            setattr(R, name, orig)


# ---------------------------------------------------------------- the shared host layer against numpy alone

# The checker and the HIP backend run the same host_mirror code, so a comparison of the two says nothing about it.
# These cases hold that layer (shape inference, keepDims and negative axes, reduce-to-shape, the shape rules of the
# indexed moves, autograd's gradients of broadcast operands) against numpy's own statement of the same rules, on
# random shapes, with values small enough that every float sum is exact.

def _random_shape(rng, dims, hi=5):
    return [int(rng.integers(1, hi + 1)) for _ in range(dims)]


def _ints(rng, shape, lo=-3, hi=4):
    return rng.integers(lo, hi, size=shape).astype(np.float32)


def test_reduce_to_shape_equals_numpy_sum_over_the_broadcast_axes(oracle_ops):
    from kten_amd.host_mirror.autograd import mayUnexpand
    rng = np.random.default_rng(101)
    for _ in range(300):
        gshape = _random_shape(rng, int(rng.integers(1, 6)))
        keep = int(rng.integers(1, len(gshape) + 1))                       # the operand's number of dims
        orig = [d if rng.random() < 0.5 else 1 for d in gshape[len(gshape) - keep:]]
        g = _ints(rng, gshape)
        res = mayUnexpand(oracle_ops.createRaw(gshape, g), orig, oracle_ops)
        lead = tuple(range(len(gshape) - keep))
        want = g.sum(axis=lead) if lead else g
        axes = tuple(i for i, (o, d) in enumerate(zip(orig, want.shape)) if o == 1 and d != 1)
        want = want.sum(axis=axes, keepdims=True) if axes else want
        assert res.shape == orig
        np.testing.assert_array_equal(res.toArray().reshape(orig), want.reshape(orig))


def test_axis_ops_keepdims_and_negative_axes_equal_numpy(oracle_ops):
    rng = np.random.default_rng(102)
    for _ in range(300):
        shape = _random_shape(rng, int(rng.integers(1, 5)))
        x = _ints(rng, shape)
        t = oracle_ops.createRaw(shape, x)
        axis = int(rng.integers(-len(shape), len(shape)))
        keep = bool(rng.integers(0, 2))
        for name, fn in (("sum", np.sum), ("max", np.max), ("min", np.min)):
            got = getattr(t, name)(axis, keep)
            want = fn(x, axis=axis, keepdims=keep)
            want_shape = list(want.shape) if want.ndim else [1]            # never 0-D (AbstractRawTensor.kt:101-105)
            assert got.shape == want_shape, (name, shape, axis, keep)
            np.testing.assert_array_equal(got.toArray().reshape(want_shape), np.asarray(want).reshape(want_shape))
        got = t.argMax(axis, keep)
        np.testing.assert_array_equal(got.toArray().reshape(-1), np.argmax(x, axis=axis).reshape(-1).astype(np.float32))
        with pytest.raises(ValueError):
            t.sum(len(shape))
        with pytest.raises(ValueError):
            t.sum(-len(shape) - 1)


def test_broadcast_binary_shapes_and_values_equal_numpy(oracle_ops):
    rng = np.random.default_rng(103)
    for _ in range(300):
        out = _random_shape(rng, int(rng.integers(1, 5)))
        a_shape = [d if rng.random() < 0.6 else 1 for d in out][int(rng.integers(0, len(out))):] or [1]
        b_shape = [d if rng.random() < 0.6 else 1 for d in out][int(rng.integers(0, len(out))):] or [1]
        a, b = _ints(rng, a_shape), _ints(rng, b_shape)
        want = a * b + a
        ta, tb = oracle_ops.createRaw(a_shape, a), oracle_ops.createRaw(b_shape, b)
        got = ta.times(tb).plus(ta)
        assert got.shape == list(want.shape)
        np.testing.assert_array_equal(got.toArray().reshape(want.shape), want)
    for a_shape, b_shape in (([3], [4]), ([2, 3], [3, 2]), ([2, 1, 3], [2, 2])):
        with pytest.raises(ValueError):
            oracle_ops.createRaw(a_shape, np.zeros(a_shape)).plus(oracle_ops.createRaw(b_shape, np.zeros(b_shape)))


def test_gradients_of_broadcast_operands_equal_the_closed_form(oracle_ops):
    """d/da and d/db of sum(a * b + b) for operands that broadcast against each other: the autograd mirror's
    backward formulas and its reduce-to-shape against the sums numpy takes over the broadcast axes."""
    rng = np.random.default_rng(104)
    for _ in range(100):
        out = _random_shape(rng, int(rng.integers(1, 5)), hi=4)
        a_shape = [d if rng.random() < 0.6 else 1 for d in out][int(rng.integers(0, len(out))):] or [1]
        b_shape = [d if rng.random() < 0.6 else 1 for d in out][int(rng.integers(0, len(out))):] or [1]
        a, b = _ints(rng, a_shape), _ints(rng, b_shape)
        ta = oracle_ops.create(a_shape, True, a)
        tb = oracle_ops.create(b_shape, True, b)
        (ta * tb + tb).sum().backward()
        full = np.broadcast_shapes(tuple(a_shape), tuple(b_shape))

        def reduce_to(g, shape):
            g = g.sum(axis=tuple(range(g.ndim - len(shape)))) if g.ndim > len(shape) else g
            axes = tuple(i for i, (o, d) in enumerate(zip(shape, g.shape)) if o == 1 and d != 1)
            return (g.sum(axis=axes, keepdims=True) if axes else g).reshape(shape)
        want_a = reduce_to(np.broadcast_to(b, full).astype(np.float32), a_shape)
        want_b = reduce_to(np.broadcast_to(a, full).astype(np.float32) + 1.0, b_shape)
        np.testing.assert_array_equal(ta.grad().toArray().reshape(a_shape), want_a)
        np.testing.assert_array_equal(tb.grad().toArray().reshape(b_shape), want_b)


def test_indexed_move_shape_rules_equal_numpy(oracle_ops):
    rng = np.random.default_rng(105)
    for _ in range(200):
        shape = _random_shape(rng, int(rng.integers(1, 4)))
        axis = int(rng.integers(-len(shape), len(shape)))
        ax = axis % len(shape)
        x = _ints(rng, shape)
        t = oracle_ops.createRaw(shape, x)
        k = int(rng.integers(1, 6))
        idx = rng.integers(0, shape[ax], size=k)
        sel = t.indexSelect(axis, oracle_ops.createRaw([k], idx.astype(np.float32)))
        want = np.take(x, idx, axis=ax)
        assert sel.shape == list(want.shape)
        np.testing.assert_array_equal(sel.toArray().reshape(want.shape), want)
        # gather with an index of the tensor's own shape equals numpy.take_along_axis
        gi = rng.integers(0, shape[ax], size=shape)
        got = t.gather(axis, oracle_ops.createRaw(shape, gi.astype(np.float32)))
        np.testing.assert_array_equal(got.toArray().reshape(shape), np.take_along_axis(x, gi, axis=ax))
        # indexAdd accumulates repeated rows in index order; the source must have the axis resized to k
        src_shape = list(shape); src_shape[ax] = k
        src = _ints(rng, src_shape)
        target = oracle_ops.createRaw(shape, x.copy())
        target.indexAdd(axis, oracle_ops.createRaw([k], idx.astype(np.float32)), oracle_ops.createRaw(src_shape, src), 2.0)
        want = x.copy()
        np.add.at(want, tuple(idx if d == ax else slice(None) for d in range(len(shape))), 2.0 * src)
        np.testing.assert_array_equal(target.toArray().reshape(shape), want)
        bad = list(src_shape); bad[ax] = k + 1
        with pytest.raises(ValueError):
            target.indexAdd(axis, oracle_ops.createRaw([k], idx.astype(np.float32)), oracle_ops.createRaw(bad, np.zeros(bad)), 1.0)
