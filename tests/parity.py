"""Comparison helpers shared by the parity tests, with the bars written out:
  - integer / index / single-rounding IEEE results: bit-exact (NaN matches NaN);
  - transcendentals: at most 2 ulp from the checker's (float) f64-libm value;
  - reductions: |got - ref64| <= 1e-5 |ref64|  or  |got - ref64| <= |kten-jvm restatement - ref64|,
    per output element, where ref64 is the extended-precision sum of the same floats.
"""
import numpy as np

TRANSCENDENTAL_ULP = 2
REDUCTION_REL = 1e-5


def bits(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32)).view(np.uint32)


def ulp_distance(a, b):
    a = np.asarray(a, dtype=np.float32); b = np.asarray(b, dtype=np.float32)
    ia = a.view(np.int32).astype(np.int64); ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7fffffff), ia); ib = np.where(ib < 0, -(ib & 0x7fffffff), ib)
    return np.where(np.isnan(a) & np.isnan(b), 0, np.abs(ia - ib))


def assert_bits_equal(got, want, what=""):
    got = np.asarray(got, dtype=np.float32); want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    same = (bits(got) == bits(want)) | (np.isnan(got) & np.isnan(want))
    if not same.all():
        i = tuple(np.argwhere(~same)[0])
        raise AssertionError(f"{what}: {np.count_nonzero(~same)} of {same.size} differ; first at {i}: "
                             f"got {got[i]!r} ({bits(got)[i]:#x}) want {want[i]!r} ({bits(want)[i]:#x})")


def assert_ulp_close(got, want, max_ulp=TRANSCENDENTAL_ULP, what=""):
    d = ulp_distance(got, want)
    assert d.max() <= max_ulp, f"{what}: max ulp distance {d.max()} at {np.argmax(d)} (bar {max_ulp})"
    return int(d.max())


def assert_reduction_close(got, ref64, jvm, what=""):
    got = np.asarray(got, dtype=np.float64).reshape(-1); ref64 = np.asarray(ref64, dtype=np.float64).reshape(-1)
    jvm = np.asarray(jvm, dtype=np.float64).reshape(-1)
    assert got.shape == ref64.shape == jvm.shape, f"{what}: shapes {got.shape} {ref64.shape} {jvm.shape}"
    err = np.abs(got - ref64); jerr = np.abs(jvm - ref64)
    ok = (err <= REDUCTION_REL * np.abs(ref64)) | (err <= jerr)
    assert ok.all(), (f"{what}: {np.count_nonzero(~ok)} of {ok.size} outputs outside both clauses; worst |err| "
                      f"{err[~ok].max():.3e} vs kten-jvm's {jerr[~ok].max():.3e}")
    return float(err.max()), float(jerr.max())


def sample_floats(rng, n):
    a = rng.standard_normal(n).astype(np.float32)
    b = (rng.standard_normal(n) * np.exp(rng.uniform(-40, 40, n))).astype(np.float32)
    c = rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32)
    special = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.17549435e-38,
                        3.4028235e38, -3.4028235e38, 0.5, -0.5, 2.5, -2.5, 0.49999997, -0.49999997, 8388607.5,
                        8388608.0, 2147483520.0, 3e9, -3e9, 89.0, -104.0, 1e-40], dtype=np.float32)
    return np.concatenate([a, b, c, special])
