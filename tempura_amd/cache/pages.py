"""Page allocator: a free list of fixed-size pages with conservation checks.

The reference's CPU allocator is a LIFO free list whose invariant is
``available + in_use == total`` (/root/reference/engine/src/kv_cache.rs:762-795,
/root/reference/kernel-api/src/lib.rs:604-618).  A page id addresses the same
page in the key and value pool of every cache slot of its group.
"""
from __future__ import annotations

from typing import List


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
        self.num_pages = num_pages
        # LIFO: the most recently freed page is handed out first, so reuse is prompt.
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.num_pages - len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise PagesExhausted(1, 0)
        p = self._free.pop()
        assert not self._held[p], f"page {p} handed out twice"
        self._held[p] = True
        return p

    def free(self, page: int) -> None:
        if page < 0 or page >= self.num_pages:
            raise ValueError(f"page {page} out of range")
        if not self._held[page]:
            raise ValueError(f"page {page} freed twice (or never allocated)")
        self._held[page] = False
        self._free.append(page)

    def is_held(self, page: int) -> bool:
        return self._held[page]

    def check(self) -> None:
        """Conservation: every page is either free or held, exactly once."""
        assert len(set(self._free)) == len(self._free), "a page is on the free list twice"
        assert all(not self._held[p] for p in self._free), "a free page is marked held"
        assert sum(self._held) + len(self._free) == self.num_pages, "a page was lost"
