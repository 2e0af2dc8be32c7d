"""The kernel library: HIP for gfx950, loaded through ctypes.  `load(device)` builds it at first use."""
from .ops import HipOps, KernelError   # noqa: F401

_loaded = {}


def load(device):
    key = str(device)
    if key not in _loaded:
        _loaded[key] = HipOps(device)
    return _loaded[key]
