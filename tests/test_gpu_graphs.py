"""Random autograd graphs on the device against the same graph on the CPU checker: values and
gradients of every leaf. Elementwise chains are bit-exact between the two; once a sum is
involved the summation order differs, so the comparison is relative (1e-4 of the largest
magnitude, far above float rounding of these small sums and far below any wrong-gradient
error). The graphs also exercise the lifetime rules (release of intermediates during
backward, garbage-collector scopes): a store released too early fails loudly on the device."""
import numpy as np
import pytest
from hypothesis import HealthCheck, given, settings, strategies as st

from kten_amd.host_mirror.autograd import concat
from kten_amd.host_mirror.shape_functions import ALL
from oracle import jvm_oracle as jo

pytestmark = pytest.mark.gpu

SETTINGS = dict(max_examples=200, deadline=None, derandomize=True,
                suppress_health_check=[HealthCheck.function_scoped_fixture, HealthCheck.too_slow])

UNARY = ["tanh", "sigmoid", "abs", "sin", "cos", "neg", "square", "exp_small", "softplus_like", "sqrt_abs"]
BINARY = ["plus", "minus", "times", "div_safe"]
SHAPED = ["sum_axis", "mean_axis", "max_axis", "min_axis", "transpose", "permute", "reshape", "get_range", "masked", "concat_self",
          "sum_keep", "expand_add"]


def apply_unary(name, t):
    if name == "neg": return -t
    if name == "square": return t ** 2.0
    if name == "exp_small": return (t * 0.1).exp()
    if name == "softplus_like": return ((t * 0.5).exp() + 1.0).log()
    if name == "sqrt_abs": return (t.abs() + 0.5).sqrt()
    return getattr(t, name)()


def apply_binary(name, a, b):
    if name == "plus": return a + b
    if name == "minus": return a - b
    if name == "times": return a * b
    return a / (b.abs() + 0.5)


def apply_shaped(name, t, ops, draw_int, mask_for):
    nd = len(t.shape)
    axis = draw_int(0, nd - 1)
    if name == "sum_axis": return t.sum(axis)
    if name == "sum_keep": return t.sum(axis, True)
    if name == "mean_axis": return t.mean(axis)
    if name == "max_axis": return t.max(axis)
    if name == "min_axis": return t.min(axis, True)
    if name == "transpose":
        if nd < 2: return t * 2.0
        # adjacent axes only: for other pairs kten-jvm's slab copy is not the axis swap the device computes
        other = axis + 1 if axis + 1 < nd else axis - 1
        return t.transpose(axis, other)
    if name == "permute":
        order = list(range(nd)); k = draw_int(0, nd - 1)
        order = order[k:] + order[:k]
        return t.permute(*order)
    if name == "reshape": return t.reshape(-1)
    if name == "get_range":
        first = draw_int(0, t.shape[0] - 1)
        return t[tuple([(first, t.shape[0] - 1)] + [ALL] * (nd - 1))]
    if name == "masked": return t.maskedFill(mask_for(t.shape[-1]), 0.25)
    if name == "concat_self": return concat(t, t * 0.5, axis=axis)
    if name == "expand_add":
        return t + t.sum(axis, True)
    raise AssertionError(name)


def build(ops, arrays, program, ints):
    """Runs `program` on backend `ops`; returns (loss value, [leaf gradients])."""
    it = iter(ints)
    draw_int = lambda lo, hi: lo + (next(it) % (hi - lo + 1)) if hi > lo else lo
    leaves = [ops.create(list(a.shape), True, a) for a in arrays]
    masks = {}
    def mask_for(n):
        if n not in masks:
            masks[n] = ops.create([n], False, (np.arange(n) % 3 == 0).astype(np.float32))
        return masks[n]
    t = leaves[0]
    for kind, name, operand in program:
        if kind == "u": t = apply_unary(name, t)
        elif kind == "b":
            other = leaves[operand % len(leaves)]
            try:
                t = apply_binary(name, t, other)
            except ValueError:                       # shapes that do not broadcast: use the leaf's total instead
                t = apply_binary(name, t, other.sum())
        else: t = apply_shaped(name, t, ops, draw_int, mask_for)
    loss = t.sum() if t.shape != [1] else t
    loss.backward()
    value = loss.toArray().astype(np.float64).reshape(-1)
    return value, [leaf.grad().toArray().astype(np.float64) for leaf in leaves]


@st.composite
def graph(draw):
    base = draw(st.lists(st.sampled_from([2, 3, 4, 5, 8, 16]), min_size=1, max_size=3))
    shapes = [base, base[-1:], [1]]
    if len(base) > 1:
        shapes.append([base[-2], 1])
    steps = []
    for _ in range(draw(st.integers(2, 7))):
        kind = draw(st.sampled_from("ubs"))
        name = draw(st.sampled_from(UNARY if kind == "u" else BINARY if kind == "b" else SHAPED))
        steps.append((kind, name, draw(st.integers(0, 7))))
    return shapes, steps, draw(st.lists(st.integers(0, 1000), min_size=40, max_size=40)), draw(st.integers(0, 2 ** 16))


@settings(**SETTINGS)
@given(g=graph())
def test_random_graph_matches_checker(g, hip):
    """Loss and every leaf gradient of a random program against the checker's, within 1e-4 of the result's scale plus
    what the checker's own result moves when every input moves by one ulp: the two backends differ by an ulp here and
    there by design (sums accumulate in f64, the transcendental maps are within 2 ulp), and a program such as
    sin((sum x)^4) turns one ulp of the sum into 2e-4 of the result."""
    shapes, program, ints, seed = g
    rng = np.random.default_rng(seed)
    arrays = [rng.uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
    with hip.garbageCollector():
        got_value, got_grads = build(hip, arrays, program, ints)
    checker = jo.JvmOracleOperations()
    want_value, want_grads = build(checker, arrays, program, ints)
    moved = [build(checker, [np.nextafter(a, np.float32(side)).astype(np.float32) for a in arrays], program, ints)
             for side in (-np.inf, np.inf)]

    def close(a, b, others, what):
        scale = max(np.abs(b).max(), 1.0)
        assert a.shape == b.shape, f"{what}: shape {a.shape} vs {b.shape}"
        with np.errstate(invalid="ignore"):
            sensitivity = max(float(np.nanmax(np.abs(o - b))) if o.shape == b.shape else 0.0 for o in others)
        if not np.isfinite(sensitivity):
            sensitivity = 0.0
        finite = np.isfinite(b)
        assert np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(a[~finite & ~np.isnan(b)], b[~finite & ~np.isnan(b)]), \
            f"{what}: infinities or NaNs in different places\n{program}"
        if not finite.any():
            return
        scale = max(np.abs(b[finite]).max(), 1.0)
        bound = 1e-4 * scale + 16.0 * sensitivity
        diff = np.abs(a[finite] - b[finite]).max()
        assert diff <= bound, f"{what}: max difference {diff:.3e} at scale {scale:.3e}, sensitivity {sensitivity:.3e}\n{program}"
    close(got_value, want_value, [m[0] for m in moved], "loss")
    for i, (a, b) in enumerate(zip(got_grads, want_grads)):
        close(a, b, [m[1][i] for m in moved], f"gradient of leaf {i} {shapes[i]}")


@settings(**SETTINGS)
@given(g=graph())
def test_random_graph_in_exact_mode_matches_checker(g, hip):
    """The same programs with the transcendental maps in exact mode: they then return the checker's floats, and what
    is left to differ are the sums."""
    shapes, program, ints, seed = g
    if any(name in ("square",) for _, name, _ in program) and any(name in ("sin", "cos") for _, name, _ in program):
        return                      # (a sum's ulp through squares into a sine: covered by the test above with its bound)
    rng = np.random.default_rng(seed)
    arrays = [rng.uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
    with hip.garbageCollector(), hip.mathMode("exact"):
        got_value, got_grads = build(hip, arrays, program, ints)
    want_value, want_grads = build(jo.JvmOracleOperations(), arrays, program, ints)

    def close(a, b, what):
        assert a.shape == b.shape, f"{what}: shape {a.shape} vs {b.shape}"
        finite = np.isfinite(b)
        assert np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(a[~finite & ~np.isnan(b)], b[~finite & ~np.isnan(b)]), \
            f"{what}: infinities or NaNs in different places\n{program}"
        if not finite.any():
            return
        scale = max(np.abs(b[finite]).max(), 1.0)
        diff = np.abs(a[finite] - b[finite]).max()
        assert diff <= 1e-4 * scale, f"{what}: max difference {diff:.3e} at scale {scale:.3e}\n{program}"
    close(got_value, want_value, "loss")
    for i, (a, b) in enumerate(zip(got_grads, want_grads)):
        close(a, b, f"gradient of leaf {i} {shapes[i]}")
