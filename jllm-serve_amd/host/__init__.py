"""The native host library (csrc/host/): page pool and step layout, reached through ctypes.

It holds no GPU code, so it builds with the C++ compiler alone and loads on a machine without a GPU; it is built at
its first use when no current build is found (a second or two).
"""
from __future__ import annotations

import ctypes
import threading

from ..kernels import build as _build

ABI_VERSION = 2
_lock = threading.Lock()
_lib = None

i32p = ctypes.POINTER(ctypes.c_int32)


class StepSizes(ctypes.Structure):
    _fields_ = [("T", ctypes.c_int32), ("R", ctypes.c_int32), ("S", ctypes.c_int32), ("width", ctypes.c_int32),
                ("max_context", ctypes.c_int32)]


class StepBatchArgs(ctypes.Structure):
    """JllmStepBatch of csrc/host/host_core.h."""
    _fields_ = [("n_entries", ctypes.c_int32), ("n_tokens", ctypes.c_void_p), ("pos0", ctypes.c_void_p),
                ("state_slots", ctypes.c_void_p), ("tokens", ctypes.c_void_p), ("tokens_len", ctypes.c_int64),
                ("want_counts", ctypes.c_void_p), ("wants", ctypes.c_void_p), ("wants_len", ctypes.c_int64),
                ("pad_rows", ctypes.c_int32), ("pad_state_slot", ctypes.c_int32), ("min_width", ctypes.c_int32),
                ("page_size", ctypes.c_int32), ("n_groups", ctypes.c_int32), ("arena_rows", ctypes.c_int32),
                ("arena", ctypes.c_void_p), ("arena_stride", ctypes.c_void_p), ("table_rows", ctypes.c_void_p),
                ("table_lens", ctypes.c_void_p)]


def step_layout(n_tokens, pos0, state_slots, tokens, want_counts, wants, pad_rows: int, pad_state_slot: int,
                min_width: int, page_size: int, arenas, table_rows, out, capacity=None):
    """Calls the native builder of a step's index arrays. The per-entry arguments and ``tokens`` / ``wants`` are int32
    numpy arrays; ``arenas`` are the groups' table arenas (``cache/tables.py``), ``table_rows`` each entry's row in
    them; ``out`` is the int32 array written. Returns (what the builder returned, the sizes it found)."""
    G = len(arenas)
    rows = min((a.data.shape[0] for a in arenas), default=0)
    ap = (ctypes.c_void_p * max(1, G))(*[a.data.ctypes.data for a in arenas])
    st = (ctypes.c_int64 * max(1, G))(*[a.data.shape[1] for a in arenas])
    lp = (ctypes.c_void_p * max(1, G))(*[a.lens.ctypes.data for a in arenas])
    args = StepBatchArgs(len(n_tokens), n_tokens.ctypes.data, pos0.ctypes.data, state_slots.ctypes.data,
                         tokens.ctypes.data, tokens.size, want_counts.ctypes.data, wants.ctypes.data, wants.size,
                         pad_rows, pad_state_slot, min_width, page_size, G, rows,
                         ctypes.cast(ap, ctypes.c_void_p), ctypes.cast(st, ctypes.c_void_p), table_rows.ctypes.data,
                         ctypes.cast(lp, ctypes.c_void_p))
    sizes = StepSizes()
    rc = library().jllm_step_layout(ctypes.byref(args), out.ctypes.data, out.size if capacity is None else capacity,
                                    ctypes.byref(sizes))
    return rc, sizes


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
        "jllm_step_layout": (c_i64, [ctypes.POINTER(StepBatchArgs), vp, c_i64, ctypes.POINTER(StepSizes)]),
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
