"""Cache manager: pages of keys and values with a block table per request, in
groups, and slots for fixed-size per-request state.

Layers whose mixers have the same ``CacheSpec`` form a group; each group has a
page pool of its own and every request has one block table per group (logical
page -> physical page), shared by all cache slots of the group.  A ``full``
group keeps every page until the request ends; a ``window`` group gives a page
back as soon as no later query can see any key in it.  Pages return to the free
list at once and are handed out again (most recently freed first).

This module is host bookkeeping only: it never touches device memory.  The
reference keeps one table per layer with ``u32::MAX`` for an empty entry and
grows by ``ceil(n / block) - have`` pages
(/root/reference/engine/src/kv_cache.rs:836-893,975-984); here a table is per
request and group, empty entries are -1, and growth reports need/free without
side effects when it cannot be met
(/root/reference/engine/src/cutile_kv_cache.rs:31-44).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np

from ..parts.base import CacheSpec
from .pages import PagePool, PagesExhausted


@dataclass
class _Request:
    rid: Hashable
    num_tokens: int = 0                      # tokens whose keys/values are in the cache
    tables: List[List[int]] = field(default_factory=list)   # per group: logical page -> physical, -1 = none
    first_live: List[int] = field(default_factory=list)     # per group: first logical page still held
    state_slot: int = -1


class CacheManager:
    def __init__(self, groups: Sequence[CacheSpec], page_size: int, num_pages, max_requests: int):
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.groups = list(groups)
        self.page_size = int(page_size)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(self.groups)
        if len(num_pages) != len(self.groups):
            raise ValueError("num_pages must give one count per cache group")
        self.pools = [PagePool(int(n)) for n in num_pages]
        self.max_requests = int(max_requests)
        self._free_state = list(range(self.max_requests - 1, -1, -1))
        self._requests: Dict[Hashable, _Request] = {}

    # ---- requests ------------------------------------------------------
    def has(self, rid) -> bool:
        return rid in self._requests

    def live_requests(self):
        return list(self._requests)

    def add(self, rid) -> int:
        """Start tracking ``rid``; returns its state slot."""
        if rid in self._requests:
            raise ValueError(f"request {rid!r} is already live")
        if not self._free_state:
            raise RuntimeError(f"no free state slot: {self.max_requests} requests are live")
        r = _Request(rid, 0, [[] for _ in self.groups], [0] * len(self.groups), self._free_state.pop())
        self._requests[rid] = r
        return r.state_slot

    def release(self, rid) -> None:
        """The request has ended: every page and its state slot go back."""
        r = self._requests.pop(rid, None)
        if r is None:
            raise ValueError(f"request {rid!r} is not live (released twice?)")
        for g, table in enumerate(r.tables):
            for p in table:
                if p >= 0:
                    self.pools[g].free(p)
        self._free_state.append(r.state_slot)

    def num_tokens(self, rid) -> int:
        return self._requests[rid].num_tokens

    def state_slot(self, rid) -> int:
        return self._requests[rid].state_slot

    # ---- pages ---------------------------------------------------------
    def _first_needed(self, g: int, start: int) -> int:
        """First logical page a query at position ``start`` can still see."""
        spec = self.groups[g]
        if spec.kind == "window" and spec.window is not None:
            return max(0, start - spec.window + 1) // self.page_size
        return 0

    def pages_needed(self, rid, n_new: int) -> List[int]:
        """Pages each group must allocate so that ``rid`` can take ``n_new`` more tokens."""
        r = self._requests[rid]
        end = r.num_tokens + n_new
        last_page = (end - 1) // self.page_size if end > 0 else -1
        need = []
        for g in range(len(self.groups)):
            lo = max(self._first_needed(g, r.num_tokens), r.first_live[g])
            # every entry from first_live up to the table's end holds a page (pages are given back
            # only below first_live), so what is missing is what lies beyond the table
            need.append(max(0, last_page + 1 - max(lo, len(r.tables[g]))))
        return need

    def can_reserve(self, rid, n_new: int) -> bool:
        return all(n <= pool.num_free for n, pool in zip(self.pages_needed(rid, n_new), self.pools))

    def reserve(self, rid, n_new: int) -> None:
        """Allocate the pages for ``n_new`` more tokens, or raise ``PagesExhausted``
        leaving everything as it was."""
        if n_new <= 0:
            raise ValueError("reserve needs at least one token")
        r = self._requests[rid]
        need = self.pages_needed(rid, n_new)
        for g, n in enumerate(need):
            if n > self.pools[g].num_free:
                raise PagesExhausted(n, self.pools[g].num_free, g)
        end = r.num_tokens + n_new
        last_page = (end - 1) // self.page_size
        for g in range(len(self.groups)):
            lo = max(self._first_needed(g, r.num_tokens), r.first_live[g])
            table = r.tables[g]
            have = len(table)
            while len(table) <= last_page:
                table.append(-1)
            # pages that a window has already passed (below lo) stay unallocated
            for lp in range(max(lo, have), last_page + 1):
                table[lp] = self.pools[g].alloc()
            if lo > have:
                r.first_live[g] = max(r.first_live[g], min(lo, len(table)))

    def commit(self, rid, n_new: int) -> None:
        """``n_new`` tokens were written; give back pages a window has passed."""
        r = self._requests[rid]
        r.num_tokens += n_new
        for g in range(len(self.groups)):
            keep_from = self._first_needed(g, r.num_tokens)
            table = r.tables[g]
            for lp in range(r.first_live[g], min(keep_from, len(table))):
                if table[lp] >= 0:
                    self.pools[g].free(table[lp])
                    table[lp] = -1
            r.first_live[g] = max(r.first_live[g], min(keep_from, len(table)))

    def truncate(self, rid, num_tokens: int) -> None:
        """Forget tokens past ``num_tokens`` and return whole pages beyond them."""
        r = self._requests[rid]
        if num_tokens > r.num_tokens or num_tokens < 0:
            raise ValueError("truncate beyond what is cached")
        keep_pages = (num_tokens + self.page_size - 1) // self.page_size
        for g, table in enumerate(r.tables):
            for lp in range(keep_pages, len(table)):
                if table[lp] >= 0:
                    self.pools[g].free(table[lp])
            del table[keep_pages:]
        r.num_tokens = num_tokens

    def table(self, rid, g: int) -> List[int]:
        return self._requests[rid].tables[g]

    def slot(self, rid, g: int, pos: int) -> int:
        """Physical cache row of one position (the single-token case of ``slots``)."""
        table = self._requests[rid].tables[g]
        lp = pos // self.page_size
        if pos < 0 or lp >= len(table) or table[lp] < 0:
            raise RuntimeError(f"request {rid!r}: position {pos} has no page reserved")
        return table[lp] * self.page_size + pos % self.page_size

    def slots(self, rid, g: int, start: int, n: int) -> np.ndarray:
        """Physical cache rows (page * page_size + offset) of positions start..start+n-1."""
        table = self._requests[rid].tables[g]
        pos = np.arange(start, start + n, dtype=np.int64)
        if start < 0 or (start + n - 1) // self.page_size >= len(table):
            raise RuntimeError(f"request {rid!r}: positions {start}..{start + n - 1} have no page reserved")
        pages = np.asarray(table, dtype=np.int64)[pos // self.page_size]
        if (pages < 0).any():
            raise RuntimeError(f"request {rid!r}: positions {start}..{start + n - 1} have no page reserved")
        return pages * self.page_size + pos % self.page_size

    # ---- statistics and invariants -------------------------------------
    def free_pages(self) -> List[int]:
        return [p.num_free for p in self.pools]

    def waste_ratio(self) -> float:
        """Share of held token places that hold no token
        (/root/reference/engine/src/kv_cache.rs:1066-1074)."""
        held = sum(p.num_held for p in self.pools) * self.page_size
        if held == 0:
            return 0.0
        used = 0
        for r in self._requests.values():
            for g in range(len(self.groups)):
                live_from = r.first_live[g] * self.page_size
                used += max(0, r.num_tokens - live_from)
        return max(0.0, 1.0 - used / held)

    def check(self) -> None:
        """No page lost, held twice or free while in a table; state slots likewise."""
        for g, pool in enumerate(self.pools):
            pool.check()
            seen = set()
            for r in self._requests.values():
                for p in r.tables[g]:
                    if p >= 0:
                        assert p not in seen, f"group {g}: page {p} is in two tables"
                        assert pool.is_held(p), f"group {g}: page {p} is in a table but free"
                        seen.add(p)
            assert len(seen) == pool.num_held, f"group {g}: {pool.num_held - len(seen)} pages held by no request"
        slots = [r.state_slot for r in self._requests.values()]
        assert len(set(slots)) == len(slots), "a state slot is held twice"
        assert len(slots) + len(self._free_state) == self.max_requests, "a state slot was lost"
        assert not (set(slots) & set(self._free_state)), "a held state slot is on the free list"
