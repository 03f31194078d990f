"""Unary ops over the whole fp32 input space, against the CPU checker.

By default every 61st bit pattern of the 2^32 (70 M inputs per op, every exponent and
sign, all specials) is checked. With KTEN_ALL_FLOATS=1 all 2^32 patterns are checked,
64 Mi at a time (about a minute of CPU time per op for the checker): run by hand after a
change to one of these routines.
Bars: exact ops bit-exact; f64-libm-then-round ops at most 2 ulp (NaN matches NaN), in both math modes: "exact"
(f64 routines; no result of the default sample differs from the checker's) and "within_2_ulp" (fp32 routines)."""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

from oracle import jvm_oracle as jo
from parity import ulp_distance

pytestmark = pytest.mark.gpu

EXACT = ["neg", "reciprocal", "abs", "sign", "sqrt", "floor", "ceil", "round", "trunc", "rsqrt"]
LIBM = ["log", "exp", "sigmoid", "tanh", "sinh", "cosh", "sin", "cos", "tan", "asin", "acos", "atan"]
FULL = os.environ.get("KTEN_ALL_FLOATS") == "1"
CHUNK = 1 << 26


def chunks():
    if FULL:
        for start in range(0, 1 << 32, CHUNK):
            yield np.arange(start, start + CHUNK, dtype=np.uint64).astype(np.uint32)
    else:
        yield np.arange(0, 1 << 32, 61, dtype=np.uint64).astype(np.uint32)


def checker(op, x):
    """The single-threaded checker on 16 slices at once (ctypes releases the GIL)."""
    parts = np.array_split(x, 16)
    with ThreadPoolExecutor(16) as pool:
        return np.concatenate(list(pool.map(lambda p: jo.unary(op, p), parts)))


@pytest.mark.parametrize("op,mode", [(op, "exact") for op in EXACT + LIBM] + [(op, "within_2_ulp") for op in LIBM])
def test_unary_over_the_float_space(op, mode, hip):
    worst, differing, total = 0, 0, 0
    hist = np.zeros(4, dtype=np.int64)
    for bits in chunks():
        x = bits.view(np.float32)
        with hip.garbageCollector(), hip.mathMode(mode):
            got = hip.createRaw([x.size], x)._unary(op).toArray()
        want = checker(op, x)
        d = ulp_distance(got, want)
        if op in EXACT:
            # +0 and -0 are one "ulp step" apart in this metric and must not be confused
            bad = np.flatnonzero(d)
            assert bad.size == 0, f"{op}: {bad.size} mismatches, first x={x[bad[0]]!r} got {got[bad[0]]!r} want {want[bad[0]]!r}"
        worst = max(worst, int(d.max())); differing += int(np.count_nonzero(d)); total += x.size
        hist += np.bincount(np.minimum(d, 3).astype(np.int64), minlength=4)
    print(f"{op} [{mode}]: {total} inputs, {differing} differ from the checker, max distance {worst} ulp; "
          f"0 / 1 / 2 / more ulp: {hist[0]} / {hist[1]} / {hist[2]} / {hist[3]}")
    assert worst <= 2
    if mode == "exact" and not FULL and op != "log":
        assert differing == 0, f"{op}: the exact mode differs from the checker on {differing} of the sampled inputs"


def test_the_math_mode_is_a_switch_of_the_library(hip):
    """The default is within_2_ulp; exact can be chosen and chosen back; the modes give different kernels and, here and
    there, different last bits; ops outside the transcendental group do not depend on it."""
    assert hip.getMathMode() == "within_2_ulp"
    x = np.linspace(-3.0, 3.0, 1 << 16, dtype=np.float32)
    with hip.garbageCollector():
        t = hip.createRaw([x.size], x)
        hip.profileBegin()
        fast = t._unary("tanh").toArray()
        with hip.mathMode("exact"):
            assert hip.getMathMode() == "exact"
            exact = t._unary("tanh").toArray()
            sig_exact = t._unary("sigmoid").toArray(); sq_exact = t._unary("sqrt").toArray()
        kernels = hip.profileEnd()
        assert hip.getMathMode() == "within_2_ulp"
        sig_fast = t._unary("sigmoid").toArray(); sq_fast = t._unary("sqrt").toArray()
    assert "unary_kernel<OpTanhF>" in kernels and "unary_lds_kernel<OpTanh>" in kernels, sorted(kernels)
    assert int(ulp_distance(fast, exact).max()) <= 1
    np.testing.assert_array_equal(exact, jo.unary("tanh", x))
    np.testing.assert_array_equal(sig_exact.view(np.uint32), sig_fast.view(np.uint32))
    np.testing.assert_array_equal(sq_exact.view(np.uint32), sq_fast.view(np.uint32))
    with pytest.raises(ValueError):
        hip.setMathMode("fast")
    assert hip.lib.kth_set_math_mode(7) == -3


@pytest.mark.parametrize("mode", ["exact", "within_2_ulp"])
@pytest.mark.parametrize("c", [1.5, -0.7, 2.5, 0.33333334, 7.0, 33.3, -12.0, 1e-3])
def test_pow_over_the_float_space(c, mode, hip):
    """x pow c for every 61st bit pattern of x (all 2^32 with KTEN_ALL_FLOATS=1) and c pow x for the same patterns as
    exponents: at most 2 ulp from the checker's (float) pow((double) x, (double) c); the count of results that differ at all
    is printed (the long routine is good to 2e-14 before the rounding: a few dozen per 70 M inputs differ by 1 ulp)."""
    for reverse in (False, True):
        worst, differing, total = 0, 0, 0
        for bits in chunks():
            x = bits.view(np.float32)
            with hip.garbageCollector(), hip.mathMode(mode):
                t = hip.createRaw([x.size], x)
                got = (hip.pow(c, t) if reverse else t._scalar("pow", c)).toArray()
            parts = np.array_split(x, 16)
            with ThreadPoolExecutor(16) as pool:
                want = np.concatenate(list(pool.map(lambda p: jo.scalar("pow", p, c, reverse=reverse), parts)))
            d = ulp_distance(got, want)
            worst = max(worst, int(d.max())); differing += int(np.count_nonzero(d)); total += x.size
        print(f"{'c pow x' if reverse else 'x pow c'} [{mode}], c = {c}: {total} inputs, {differing} differ from the checker, max distance {worst} ulp")
        assert worst <= 2
