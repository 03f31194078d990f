"""Library life cycle through the C ABI: the memory budget of memoryUsageScaleHint
(PlatformProvider.kt:23-29), the reuse pool, and shutdown followed by a new session."""
import ctypes
import os
import subprocess
import sys
import textwrap

import numpy as np
import pytest

from kten_amd import abi

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_memory_budget_is_enforced_and_pool_is_trimmed(hip):
    lib = hip.lib
    hip.sync()
    total = ctypes.c_uint64()
    abi.check(lib.kth_device_info(None, 0, ctypes.byref(total), None, None))
    before = hip.getMetrics()
    mib = 1 << 20
    # budget = what is live now + 1 GiB and a little: sixteen 64 MiB stores and some small ones
    budget = before["liveBytes"] + 1040 * mib
    try:
        abi.check(lib.kth_set_memory_scale_hint(budget / total.value))
        handles = []
        status = abi.KTH_OK
        for _ in range(64):                                       # 64 x 64 MiB = 4 GiB > budget
            h = ctypes.c_uint64()
            status = lib.kth_alloc(16 * mib, ctypes.byref(h))
            if status != abi.KTH_OK:
                break
            handles.append(h)
        assert status == abi.KTH_E_MEMORY, "allocations past the budget must be refused"
        assert len(handles) == 16
        assert b"cannot allocate" in lib.kth_last_error()
        with pytest.raises(MemoryError):
            abi.check(status)
        # the refused call left the library usable: a store that fits is still served
        small = ctypes.c_uint64()
        abi.check(lib.kth_alloc(1024, ctypes.byref(small)))
        abi.check(lib.kth_fill(small, 0, 1024, 2.5))
        out = np.empty(1024, np.float32)
        abi.check(lib.kth_download(out.ctypes.data_as(ctypes.c_void_p), small, 0, 1024))
        assert (out == 2.5).all()
        abi.check(lib.kth_release(small))
        # released stores wait in the pool; a request of another size class makes the pool give them up
        for h in handles:
            abi.check(lib.kth_release(h))
        parked = hip.getMetrics()
        assert parked["poolBytes"] >= len(handles) * 64 * mib
        big = ctypes.c_uint64()
        abi.check(lib.kth_alloc(200 * mib, ctypes.byref(big)))    # 800 MiB: fits only once the pool is trimmed
        after = hip.getMetrics()
        assert after["poolBytes"] < 64 * mib
        abi.check(lib.kth_release(big))
        assert lib.kth_set_memory_scale_hint(0.0) == abi.KTH_E_ARGUMENT
        assert lib.kth_set_memory_scale_hint(1.5) == abi.KTH_E_ARGUMENT
    finally:
        abi.check(lib.kth_set_memory_scale_hint(0.85))


SESSION = textwrap.dedent("""
    import ctypes, sys
    import numpy as np
    sys.path.insert(0, %r)
    from kten_amd import abi
    lib = abi.load()
    h = ctypes.c_uint64()
    assert lib.kth_alloc(4, ctypes.byref(h)) == abi.KTH_E_NOT_INIT          # nothing works before init
    abi.check(lib.kth_init(0))
    assert lib.kth_init(0) == abi.KTH_OK                                       # a second init of the same device is a no-op
    first = ctypes.c_uint64()
    abi.check(lib.kth_alloc(1000, ctypes.byref(first)))
    abi.check(lib.kth_fill(first, 0, 1000, 1.0))
    source, alias = ctypes.c_uint64(), ctypes.c_uint64()
    abi.check(lib.kth_alloc(5000, ctypes.byref(source)))
    abi.check(lib.kth_alloc(5000, ctypes.byref(alias)))
    abi.check(lib.kth_upload(source, 0, np.ones(5000, np.float32).ctypes.data_as(ctypes.c_void_p), 5000))
    abi.check(lib.kth_copy(alias, 0, source, 0, 5000))                         # a copy that is still put off ...
    big, owed, dropped = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
    abi.check(lib.kth_alloc(64 * 40 * 100, ctypes.byref(big)))
    abi.check(lib.kth_alloc(64 * 100, ctypes.byref(owed)))
    abi.check(lib.kth_alloc(64 * 100, ctypes.byref(dropped)))
    abi.check(lib.kth_fill(big, 0, 64 * 40 * 100, 0.5))
    abi.check(lib.kth_reduce_axis(abi.Op.SUM, big, owed, 64, 40, 100))          # ... a small sum that is still put off,
    abi.check(lib.kth_reduce_axis(abi.Op.SUM, big, dropped, 64, 40, 100))
    abi.check(lib.kth_release(dropped))                                        # one that nobody will ever read
    abi.check(lib.kth_release(big))                                            # and their source, kept for the first only
    assert lib.kth_release(big) == abi.KTH_E_HANDLE, "released is released, whatever the library still keeps of it"
    abi.check(lib.kth_shutdown())                                              # frees live stores too (each its own buffer, once)
    assert lib.kth_release(first) == abi.KTH_E_NOT_INIT
    abi.check(lib.kth_init(0))
    second = ctypes.c_uint64()
    abi.check(lib.kth_alloc(1000, ctypes.byref(second)))                       # takes the table slot `first` had
    assert lib.kth_release(first) == abi.KTH_E_HANDLE, "a handle of the previous session must not validate"
    x = np.arange(1000, dtype=np.float32)
    abi.check(lib.kth_upload(second, 0, x.ctypes.data_as(ctypes.c_void_p), 1000))
    abi.check(lib.kth_set_math_mode(abi.KTH_MATH_EXACT))                       # the f64 routines, which read the tables
    abi.check(lib.kth_unary(abi.Op.EXP, second, second, 1000))                 # the math tables were rebuilt
    y = np.empty(1000, np.float32)
    abi.check(lib.kth_download(y.ctypes.data_as(ctypes.c_void_p), second, 0, 1000))
    want = np.exp(x.astype(np.float64)).astype(np.float32)
    assert np.array_equal(y[:80], want[:80]) and np.isinf(y[100:]).all()
    abi.check(lib.kth_release(second))
    abi.check(lib.kth_shutdown())
    assert lib.kth_shutdown() == abi.KTH_OK                                    # idempotent
    print("session ok")
""") % ROOT


def test_shutdown_and_new_session_in_a_child_process():
    """Run in a child so the test session's own library instance stays up."""
    done = subprocess.run([sys.executable, "-c", SESSION], capture_output=True, text=True, timeout=150)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "session ok" in done.stdout
