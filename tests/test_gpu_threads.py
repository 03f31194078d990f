"""Several host threads calling the C ABI at once. The library serialises calls with one
mutex and orders all work on one stream, so interleaved callers must each get the results
a lone caller gets: bit-exact elementwise results, max / arg_max bit-exact, and every
store handle released exactly once."""
import ctypes
import threading

import numpy as np
import pytest

from kten_amd import abi
from kten_amd.abi import Op

pytestmark = pytest.mark.gpu

THREADS = 6
ROUNDS = 40


def _shape(dims):
    return (ctypes.c_int32 * len(dims))(*dims)


def _worker(lib, seed, errors):
    """ctypes drops the interpreter lock for the duration of each call, so the threads
    really do contend for the library's mutex."""
    try:
        rng = np.random.default_rng(seed)
        for r in range(ROUNDS):
            rows, cols = int(rng.integers(1, 200)), int(rng.integers(1, 300))
            n = rows * cols
            x = rng.standard_normal((rows, cols)).astype(np.float32)
            b = rng.standard_normal(cols).astype(np.float32)
            hx, hb, hy, hm, ha = (ctypes.c_uint64() for _ in range(5))
            abi.check(lib.kth_alloc(n, ctypes.byref(hx)))
            abi.check(lib.kth_alloc(cols, ctypes.byref(hb)))
            abi.check(lib.kth_alloc(n, ctypes.byref(hy)))
            abi.check(lib.kth_alloc(rows, ctypes.byref(hm)))
            abi.check(lib.kth_alloc(rows, ctypes.byref(ha)))
            abi.check(lib.kth_upload(hx, 0, x.ctypes.data_as(ctypes.c_void_p), n))
            abi.check(lib.kth_upload(hb, 0, b.ctypes.data_as(ctypes.c_void_p), cols))
            abi.check(lib.kth_binary(Op.PLUS, hx, _shape([rows, cols]), 2, hb, _shape([cols]), 1, hy, _shape([rows, cols]), 2))
            abi.check(lib.kth_binary_inplace(Op.TIMES, hy, hx, n))
            abi.check(lib.kth_reduce_axis(Op.MAX, hy, hm, rows, cols, 1))
            abi.check(lib.kth_reduce_axis(Op.ARG_MAX, hy, ha, rows, cols, 1))
            y = np.empty(n, np.float32); m = np.empty(rows, np.float32); a = np.empty(rows, np.float32)
            abi.check(lib.kth_download(y.ctypes.data_as(ctypes.c_void_p), hy, 0, n))
            abi.check(lib.kth_download(m.ctypes.data_as(ctypes.c_void_p), hm, 0, rows))
            abi.check(lib.kth_download(a.ctypes.data_as(ctypes.c_void_p), ha, 0, rows))
            for h in (hx, hb, hy, hm, ha):
                abi.check(lib.kth_release(h))
            want = (x + b) * x                                   # float32 throughout, one rounding per op
            if not np.array_equal(y.view(np.uint32), want.reshape(-1).view(np.uint32)):
                raise AssertionError(f"thread {seed} round {r}: elementwise bits differ for {rows}x{cols}")
            if not np.array_equal(m.view(np.uint32), want.max(1).view(np.uint32)):
                raise AssertionError(f"thread {seed} round {r}: max differs for {rows}x{cols}")
            if not np.array_equal(a, want.argmax(1).astype(np.float32)):
                raise AssertionError(f"thread {seed} round {r}: arg_max differs for {rows}x{cols}")
            # a second release of a store this thread freed must be refused, whatever the others do
            if lib.kth_release(hx) != abi.KTH_E_HANDLE:
                raise AssertionError(f"thread {seed} round {r}: a released handle was accepted")
    except BaseException as e:                                    # noqa: BLE001 - reported by the main thread
        errors.append(e)


def test_concurrent_callers(hip):
    lib = hip.lib
    errors = []
    threads = [threading.Thread(target=_worker, args=(lib, 100 + i, errors)) for i in range(THREADS)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not any(t.is_alive() for t in threads), "a caller thread did not finish"
    if errors:
        raise errors[0]


def test_error_message_is_per_thread(hip):
    """kth_last_error returns the calling thread's message: a failure on one thread does not
    show up on another."""
    lib = hip.lib
    seen = {}

    def fail_here():
        assert lib.kth_release(0xdeadbeef) == abi.KTH_E_HANDLE
        seen["failing"] = lib.kth_last_error().decode()

    def clean_here():
        h = ctypes.c_uint64()
        abi.check(lib.kth_alloc(4, ctypes.byref(h)))
        abi.check(lib.kth_release(h))
        seen["clean"] = lib.kth_last_error().decode()

    a = threading.Thread(target=fail_here); a.start(); a.join(30)
    b = threading.Thread(target=clean_here); b.start(); b.join(30)
    assert "handle" in seen["failing"].lower() or seen["failing"] != ""
    assert seen["clean"] == ""
