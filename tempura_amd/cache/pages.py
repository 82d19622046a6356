"""Page allocator: a free list of fixed-size pages with conservation checks.

The reference's CPU allocator is a LIFO free list whose invariant is
``available + in_use == total`` (/root/reference/engine/src/kv_cache.rs:762-795,
/root/reference/kernel-api/src/lib.rs:604-618).  A page id addresses the same
page in the key and value pool of every cache slot of its group.  The list itself
lives in the compiled host library (csrc/host/cache_core.cpp); this is its Python face.
"""
from __future__ import annotations

import ctypes

from . import native


class PagesExhausted(RuntimeError):
    """Not enough free pages (the reference's ``PoolExhausted{need_pages, free_pages}``,
    /root/reference/engine/src/cutile_kv_cache.rs:31-44)."""

    def __init__(self, need: int, free: int, group: int = 0):
        super().__init__(f"cache group {group}: need {need} pages, {free} free")
        self.need = need
        self.free = free
        self.group = group


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must be >= 0")
        self.num_pages = int(num_pages)
        self._lib = native.lib()
        self._h = ctypes.c_void_p(self._lib.pp_create(self.num_pages))

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.pp_destroy(self._h)
            self._h = None

    @property
    def num_free(self) -> int:
        return self._lib.pp_num_free(self._h)

    @property
    def num_held(self) -> int:
        return self.num_pages - self.num_free

    def alloc(self) -> int:
        p = self._lib.pp_alloc(self._h)
        if p < 0:
            raise PagesExhausted(1, 0)
        return p

    def free(self, page: int) -> None:
        if self._lib.pp_free(self._h, int(page)) != 0:
            raise ValueError(native.last_error())

    def is_held(self, page: int) -> bool:
        return bool(self._lib.pp_is_held(self._h, int(page)))

    def check(self) -> None:
        """Conservation: every page is either free or held, exactly once."""
        assert self._lib.pp_check(self._h) == 0, native.last_error()
