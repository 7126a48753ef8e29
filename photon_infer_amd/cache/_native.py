"""The host-side runtime library (``csrc/runtime``, plain C++): loaded once, built at first use."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int32, c_void_p
from typing import Optional

from ..errors import KernelLibraryMissing

_LIB: Optional[ctypes.CDLL] = None
_IP = POINTER(c_int)

_SIGNATURES = {
    # name: (restype, argtypes)
    "pi_pool_create": (c_void_p, [c_int]),
    "pi_pool_destroy": (None, [c_void_p]),
    "pi_pool_error": (c_char_p, [c_void_p]),
    "pi_pool_num_free": (c_int, [c_void_p]),
    "pi_pool_is_allocated": (c_int, [c_void_p, c_int]),
    "pi_pool_allocate": (c_int, [c_void_p, c_int, _IP]),
    "pi_pool_free": (c_int, [c_void_p, _IP, c_int]),
    "pi_pool_reset": (None, [c_void_p]),
    "pi_cache_create": (c_void_p, [c_int, _IP, c_int, _IP, c_int, c_int]),
    "pi_cache_destroy": (None, [c_void_p]),
    "pi_cache_error": (c_char_p, [c_void_p]),
    "pi_cache_max_blocks": (c_int, [c_void_p]),
    "pi_cache_table": (POINTER(c_int32), [c_void_p, c_int]),
    "pi_cache_next_block": (POINTER(c_int32), [c_void_p, c_int]),
    "pi_cache_first_block": (POINTER(c_int32), [c_void_p, c_int]),
    "pi_cache_lengths": (POINTER(c_int32), [c_void_p]),
    "pi_cache_free_slots": (c_int, [c_void_p]),
    "pi_cache_free_pages": (c_int, [c_void_p, c_int]),
    "pi_cache_page_allocated": (c_int, [c_void_p, c_int, c_int]),
    "pi_cache_admit": (c_int, [c_void_p]),
    "pi_cache_pages_needed": (c_int, [c_void_p, c_int, c_int, _IP]),
    "pi_cache_can_reserve": (c_int, [c_void_p, c_int, c_int, _IP]),
    "pi_cache_reserve": (c_int, [c_void_p, c_int, c_int]),
    "pi_cache_commit": (c_int, [c_void_p, c_int, c_int]),
    "pi_cache_release": (c_int, [c_void_p, c_int]),
    "pi_cache_pages_needed_many": (c_int, [c_void_p, _IP, _IP, c_int, _IP]),
    "pi_cache_reserve_many": (c_int, [c_void_p, _IP, _IP, c_int]),
    "pi_cache_commit_many": (c_int, [c_void_p, _IP, _IP, c_int]),
    "pi_cache_check": (c_int, [c_void_p]),
}

OK, OUT_OF_PAGES, MISUSE = 0, 1, 2


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        from ..ops import build
        path = build.build_module("runtime", quiet=True)
        try:
            loaded = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryMissing(f"cannot load the runtime library {path}: {e}") from e
        for name, (restype, argtypes) in _SIGNATURES.items():
            try:
                fn = getattr(loaded, name)
            except AttributeError:
                raise KernelLibraryMissing(f"runtime library {path} lacks entry point {name}") from None
            fn.restype = restype
            fn.argtypes = argtypes
        _LIB = loaded
    return _LIB


def int_array(values) -> ctypes.Array:
    values = list(values)
    return (c_int * max(1, len(values)))(*values)
