"""The compiled host library (page pools, block tables, step packing), loaded on first use.

It is plain C++ with no GPU code and is needed wherever the engine's bookkeeping runs, also on
machines without a GPU; it is compiled at its first use when no build is there.
"""
from __future__ import annotations

import ctypes

_lib = None


def lib():
    global _lib
    if _lib is None:
        from ..csrc.build import ensure_host_built
        path = ensure_host_built()
        try:
            l = ctypes.CDLL(path)
        except OSError as e:
            raise RuntimeError(f"cannot load the host library {path}: {e}") from e
        l.cc_last_error.restype = ctypes.c_char_p
        l.cc_create.restype = ctypes.c_void_p
        l.cc_waste_ratio.restype = ctypes.c_double
        for name in ("cc_destroy", "cc_add", "cc_release", "cc_num_tokens", "cc_pages_needed", "cc_reserve", "cc_commit",
                     "cc_truncate", "cc_table_len", "cc_table", "cc_slots", "cc_free_pages", "cc_num_live",
                     "cc_waste_ratio", "cc_check", "cc_fill_decode", "cc_fill_step", "hr_fill_normal"):
            getattr(l, name).argtypes = None
        _lib = l
    return _lib


def last_error() -> str:
    return lib().cc_last_error().decode()
