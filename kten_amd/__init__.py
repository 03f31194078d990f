"""kten_amd — an MI355X (gfx950) backend for the kten tensor library's hot path:
broadcast elementwise ops, axis / full reductions and the autograd reduce-to-shape,
as hand-written HIP kernels behind a C ABI (libkten_hip.so, include/kten_hip.h).

`platform()` returns the process-wide `HipTensorOperations` (the role of
PlatformProvider.defaultOps() once a HIP PlatformInitializer has registered itself).
"""
from .abi import Op, LIB_PATH          # noqa: F401
from .host_mirror.raw_tensor import AbstractRawTensor, AggregatingOperation   # noqa: F401

_platform = None


def platform(device: int = 0):
    """The HIP operations object for `device`, created on first use. Raises if the
    shared library is missing or no GPU is visible: there is no CPU fallback."""
    global _platform
    if _platform is None:
        from .hip_raw_tensor import HipTensorOperations
        _platform = HipTensorOperations(device)
    return _platform
