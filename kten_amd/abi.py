"""ctypes binding of libkten_hip.so: the same entry points a Kotlin host would bind.

Every function of include/kten_hip.h and include/kten_hip_bench.h is declared here with its C signature; `check`
turns a negative status into the Python exception that corresponds to what the
reference throws for that class of error (IllegalArgumentException -> ValueError,
IllegalStateException / device failures -> RuntimeError).

There is no CPU fallback: if the shared library is missing this module raises.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_int32, c_size_t, c_uint64

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkten_hip.so")

KTH_MAX_DIMS = 10
KTH_MATH_EXACT, KTH_MATH_WITHIN_2_ULP = 0, 1
KTH_OK, KTH_E_NOT_INIT, KTH_E_HANDLE, KTH_E_ARGUMENT, KTH_E_SHAPE, KTH_E_MEMORY, KTH_E_DEVICE = 0, -1, -2, -3, -4, -5, -6


class Op:
    """Operation codes (OCLKernelConstant.kt:5-43 numbering, plus NEG)."""
    PLUS, MINUS, TIMES, DIV, POW, RECIPROCAL, LOG = 0, 1, 2, 3, 4, 5, 6
    SUM, MEAN, MAX, MIN, ARG_MAX, ARG_MIN = 7, 8, 9, 10, 11, 12
    LT, LTE, GT, GTE, EQ, NEQ = 13, 14, 15, 16, 17, 18
    EXP, TANH, SIGMOID, SINH, COSH, ABS, SIGN, SQRT = 19, 20, 21, 22, 23, 24, 25, 26
    SIN, COS, TAN, ASIN, ACOS, ATAN, FLOOR, CEIL, ROUND, TRUNC, RSQRT = 27, 28, 29, 30, 31, 32, 33, 34, 35, 36, 37
    NEG = 40


# name -> (restype, argtypes): exactly the declarations of include/kten_hip.h
SIGNATURES = {
    "kth_init": (c_int, [c_int]),
    "kth_shutdown": (c_int, []),
    "kth_last_error": (c_char_p, []),
    "kth_device_info": (c_int, [ctypes.c_char_p, c_size_t, POINTER(c_uint64), POINTER(c_int), POINTER(c_int)]),
    "kth_set_epsilon": (c_int, [c_float]),
    "kth_set_math_mode": (c_int, [c_int]),
    "kth_get_math_mode": (c_int, [POINTER(c_int)]),
    "kth_set_memory_scale_hint": (c_int, [c_double]),
    "kth_alloc": (c_int, [c_uint64, POINTER(c_uint64)]),
    "kth_retain": (c_int, [c_uint64]),
    "kth_release": (c_int, [c_uint64]),
    "kth_upload": (c_int, [c_uint64, c_uint64, ctypes.c_void_p, c_uint64]),
    "kth_download": (c_int, [ctypes.c_void_p, c_uint64, c_uint64, c_uint64]),
    "kth_read_scalar": (c_int, [c_uint64, c_uint64, POINTER(c_float)]),
    "kth_copy": (c_int, [c_uint64, c_uint64, c_uint64, c_uint64, c_uint64]),
    "kth_fill": (c_int, [c_uint64, c_uint64, c_uint64, c_float]),
    "kth_contains_nan": (c_int, [c_uint64, c_uint64, POINTER(c_int)]),
    "kth_binary": (c_int, [c_int, c_uint64, POINTER(c_int32), c_int, c_uint64, POINTER(c_int32), c_int,
                           c_uint64, POINTER(c_int32), c_int]),
    "kth_binary_inplace": (c_int, [c_int, c_uint64, c_uint64, c_uint64]),
    "kth_scalar": (c_int, [c_int, c_uint64, c_float, c_int, c_uint64, c_uint64]),
    "kth_unary": (c_int, [c_int, c_uint64, c_uint64, c_uint64]),
    "kth_clamp": (c_int, [c_uint64, c_uint64, c_uint64, c_float, c_float]),
    "kth_broadcast_to": (c_int, [c_uint64, POINTER(c_int32), c_int, c_uint64, POINTER(c_int32), c_int]),
    "kth_reduce_axis": (c_int, [c_int, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64]),
    "kth_reduce_all": (c_int, [c_int, c_uint64, c_uint64, c_uint64]),
    "kth_reduce_axis_static": (c_int, [c_int, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64]),
    "kth_reduce_scratch_bytes": (c_int, [POINTER(c_uint64)]),
    "kth_set_index_check": (c_int, [c_int]),
    "kth_gather": (c_int, [c_uint64, POINTER(c_int32), c_uint64, POINTER(c_int32), c_int, c_int, c_uint64]),
    "kth_scatter": (c_int, [c_int, c_uint64, POINTER(c_int32), c_uint64, POINTER(c_int32), c_uint64, POINTER(c_int32),
                            c_int, c_int]),
    "kth_scatter_fill": (c_int, [c_uint64, POINTER(c_int32), c_uint64, POINTER(c_int32), c_int, c_int, c_float]),
    "kth_index_select": (c_int, [c_uint64, POINTER(c_int32), c_int, c_int, c_uint64, c_uint64, c_uint64]),
    "kth_index_add": (c_int, [c_uint64, POINTER(c_int32), c_int, c_int, c_uint64, c_uint64, c_uint64, c_float]),
    "kth_get_range": (c_int, [c_uint64, POINTER(c_int32), c_int, POINTER(c_int32), POINTER(c_int32), c_uint64]),
    "kth_set_range": (c_int, [c_uint64, POINTER(c_int32), c_int, POINTER(c_int32), POINTER(c_int32), c_uint64, c_uint64]),
    "kth_concat": (c_int, [POINTER(c_uint64), POINTER(c_int32), c_int, POINTER(c_int32), c_int, c_int, c_uint64]),
    "kth_fill_range": (c_int, [c_uint64, POINTER(c_int32), c_int, POINTER(c_int32), POINTER(c_int32), c_float]),
    "kth_transpose": (c_int, [c_uint64, POINTER(c_int32), c_int, c_int, c_int, c_uint64]),
    "kth_permute": (c_int, [c_uint64, POINTER(c_int32), c_int, POINTER(c_int32), c_uint64]),
    "kth_masked_fill": (c_int, [c_uint64, POINTER(c_int32), c_int, c_uint64, POINTER(c_int32), c_int, c_float, c_uint64]),
    "kth_batch_norm_forward": (c_int, [c_uint64, POINTER(c_int32), c_int, c_int, c_int, c_float, c_float,
                                       c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64]),
    "kth_batch_norm_backward": (c_int, [c_uint64, POINTER(c_int32), c_int, c_int, c_int, c_float,
                                        c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64]),
    "kth_sync": (c_int, []),
    "kth_metrics": (c_int, [POINTER(c_uint64), POINTER(c_uint64), POINTER(c_uint64), POINTER(c_uint64)]),
}

# The measurement entry points of include/kten_hip_bench.h (same library; no counterpart in the contract).
BENCH_SIGNATURES = {
    "kth_timer_begin": (c_int, []),
    "kth_timer_end": (c_int, [POINTER(c_float)]),
    "kth_timer_lap": (c_int, []),
    "kth_timer_laps": (c_int, [POINTER(c_float), c_int, POINTER(c_int), POINTER(c_float)]),
    "kth_measure_copy": (c_int, [c_uint64, c_int, POINTER(c_float), POINTER(c_float)]),
    "kth_profile_begin": (c_int, []),
    "kth_profile_end": (c_int, []),
    "kth_profile_count": (c_int, [POINTER(c_int)]),
    "kth_profile_entry": (c_int, [c_int, ctypes.c_char_p, c_size_t, POINTER(c_uint64), POINTER(c_uint64), POINTER(c_double)]),
}

_lib = None


def load():
    """Loads libkten_hip.so (once) and declares every entry point. Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C kten_amd/csrc`. There is no CPU fallback for the HIP backend.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in list(SIGNATURES.items()) + list(BENCH_SIGNATURES.items()):
        fn = getattr(lib, name)          # AttributeError here means the .so is stale
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error():
    return load().kth_last_error().decode("utf-8", "replace")


def check(status):
    """Maps a status code to the exception class the reference would throw."""
    if status == KTH_OK:
        return
    msg = last_error()
    if status in (KTH_E_ARGUMENT, KTH_E_SHAPE):
        raise ValueError(msg)              # IllegalArgumentException
    if status == KTH_E_MEMORY:
        raise MemoryError(msg)
    raise RuntimeError(f"[kth status {status}] {msg}")   # IllegalStateException / device error


_SHAPE_ARRAYS = {}


def shape_array(shape):
    """The shape as an int32 array for the entry points, which only read it. Arrays are kept per shape: building one
    costs about a microsecond, a third of what a small launch takes to issue."""
    key = tuple(shape)
    arr = _SHAPE_ARRAYS.get(key)
    if arr is None:
        if len(_SHAPE_ARRAYS) >= 4096:
            _SHAPE_ARRAYS.clear()
        arr = _SHAPE_ARRAYS[key] = (c_int32 * max(len(key), 1))(*key)
    return arr
