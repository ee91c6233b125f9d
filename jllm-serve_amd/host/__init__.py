"""The native host library (csrc/host/): page pool and step layout, reached through ctypes.

It holds no GPU code, so it builds with the C++ compiler alone and loads on a machine without a GPU; it is built at
its first use when no current build is found (a second or two).
"""
from __future__ import annotations

import ctypes
import threading

from ..kernels import build as _build

ABI_VERSION = 1
_lock = threading.Lock()
_lib = None

i32p = ctypes.POINTER(ctypes.c_int32)


class StepSizes(ctypes.Structure):
    _fields_ = [("T", ctypes.c_int32), ("R", ctypes.c_int32), ("S", ctypes.c_int32), ("width", ctypes.c_int32),
                ("max_context", ctypes.c_int32)]


def _declare(lib) -> None:
    c_int, c_i64, vp = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p
    sig = {
        "jllm_host_abi_version": (c_int, []),
        "jllm_pool_new": (vp, [c_int]),
        "jllm_pool_delete": (None, [vp]),
        "jllm_pool_alloc": (c_int, [vp]),
        "jllm_pool_alloc_many": (c_int, [vp, c_int, vp]),
        "jllm_pool_retain": (c_int, [vp, c_int]),
        "jllm_pool_release": (c_int, [vp, c_int]),
        "jllm_pool_refs": (c_int, [vp, c_int]),
        "jllm_pool_free_pages": (c_int, [vp]),
        "jllm_pool_high_water": (c_int, [vp]),
        "jllm_pool_allocations": (c_i64, [vp]),
        "jllm_pool_free_list": (c_int, [vp, vp]),
        "jllm_pool_set_free_list": (c_int, [vp, vp, c_int]),
        "jllm_pool_check": (c_int, [vp, ctypes.POINTER(c_int)]),
        "jllm_step_layout": (c_i64, [c_int, vp, vp, vp, vp, vp, vp, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, c_i64,
                                     ctypes.POINTER(StepSizes)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args


def library():
    """The loaded library; built first when there is no current build. Raises when it cannot be built or loaded."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                lib = ctypes.CDLL(_build.ensure_host_built(verbose=False))
                _declare(lib)
                if lib.jllm_host_abi_version() != ABI_VERSION:
                    raise RuntimeError("the built host library is of another version than this package: build again")
                _lib = lib
    return _lib
