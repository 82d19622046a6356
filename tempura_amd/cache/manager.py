"""Cache manager: pages of keys and values with a block table per request, in
groups, and slots for fixed-size per-request state.

Layers whose mixers have the same ``CacheSpec`` form a group; each group has a
page pool of its own and every request has one block table per group (logical
page -> physical page), shared by all cache slots of the group.  A ``full``
group keeps every page until the request ends; a group with another visibility
rule (``window``, ``chunk``; cache/rules.py) gives a page back as soon as no later
query can see any key in it.  Pages return to the free
list at once and are handed out again (most recently freed first).

This is host bookkeeping only: it never touches device memory.  The bookkeeping
itself is native code (csrc/host/cache_core.cpp, as the reference's is:
/root/reference/engine/src/kv_cache.rs:836-893,975-984); this class maps request
names to the core's request slots and turns its error codes into exceptions.  Empty
table entries are -1, and growth reports need/free without side effects when it
cannot be met (/root/reference/engine/src/cutile_kv_cache.rs:31-44).
"""
from __future__ import annotations

import ctypes
from typing import Dict, Hashable, List, Sequence

import numpy as np

from ..parts.base import CacheSpec
from . import native
from .rules import rule_args


class PagesExhausted(RuntimeError):
    """Not enough free pages (the reference's ``PoolExhausted{need_pages, free_pages}``,
    /root/reference/engine/src/cutile_kv_cache.rs:31-44)."""

    def __init__(self, need: int, free: int, group: int = 0):
        super().__init__(f"cache group {group}: need {need} pages, {free} free")
        self.need = need
        self.free = free
        self.group = group


class _PoolView:
    """Counts of one group's page pool."""

    def __init__(self, manager: "CacheManager", g: int, num_pages: int):
        self._m, self._g, self.num_pages = manager, g, num_pages

    @property
    def num_free(self) -> int:
        return self._m.free_pages()[self._g]

    @property
    def num_held(self) -> int:
        return self.num_pages - self.num_free


def _ints(values) -> ctypes.Array:
    return (ctypes.c_int * len(values))(*values)


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
        if any(int(n) < 0 for n in num_pages):
            raise ValueError("num_pages must be >= 0")
        self.max_requests = int(max_requests)
        self._lib = native.lib()
        # what each group's queries can still see: a rule of the core and its integers (cache/rules.py)
        args = [rule_args(s) for s in self.groups]
        self._h = ctypes.c_void_p(self._lib.cc_create(len(self.groups), _ints([a[0] for a in args]),
                                                      _ints([p for a in args for p in a[1]]), self.page_size,
                                                      _ints([int(n) for n in num_pages]), self.max_requests))
        if not self._h:
            raise ValueError(native.last_error())
        self.pools = [_PoolView(self, g, int(n)) for g, n in enumerate(num_pages)]
        self._slot_of: Dict[Hashable, int] = {}
        #: bumped by everything that changes what a request holds or where its next token goes (add, release,
        #: commit, truncate): whoever keeps values derived from the tables compares it before using them
        self.generation = 0
        self._g_buf = (ctypes.c_int * max(1, len(self.groups)))()

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.cc_destroy(self._h)
            self._h = None

    def _slot(self, rid) -> int:
        try:
            return self._slot_of[rid]
        except KeyError:
            raise KeyError(f"request {rid!r} is not live") from None

    # ---- requests ------------------------------------------------------
    def has(self, rid) -> bool:
        return rid in self._slot_of

    def live_requests(self):
        return list(self._slot_of)

    def add(self, rid) -> int:
        """Start tracking ``rid``; returns its state slot."""
        if rid in self._slot_of:
            raise ValueError(f"request {rid!r} is already live")
        s = self._lib.cc_add(self._h)
        if s < 0:
            raise RuntimeError(native.last_error())
        self._slot_of[rid] = s
        self.generation += 1
        return s

    def release(self, rid) -> None:
        """The request has ended: every page and its state slot go back."""
        s = self._slot_of.pop(rid, None)
        if s is None:
            raise ValueError(f"request {rid!r} is not live (released twice?)")
        self.generation += 1
        if self._lib.cc_release(self._h, s) != 0:
            raise RuntimeError(native.last_error())

    def num_tokens(self, rid) -> int:
        return self._lib.cc_num_tokens(self._h, self._slot(rid))

    def max_num_tokens(self, rids: Sequence) -> int:
        """The largest token count among ``rids``."""
        m = self._lib.cc_max_tokens(self._h, len(rids), _ints([self._slot(r) for r in rids]))
        if m < 0:
            raise RuntimeError(native.last_error())
        return m

    def state_slot(self, rid) -> int:
        return self._slot(rid)

    # ---- pages ---------------------------------------------------------
    def pages_needed(self, rid, n_new: int) -> List[int]:
        """Pages each group must allocate so that ``rid`` can take ``n_new`` more tokens."""
        self._lib.cc_pages_needed(self._h, self._slot(rid), int(n_new), self._g_buf)
        return list(self._g_buf[: len(self.groups)])

    def can_reserve(self, rid, n_new: int) -> bool:
        return all(n <= f for n, f in zip(self.pages_needed(rid, n_new), self.free_pages()))

    def reserve(self, rid, n_new: int) -> None:
        """Allocate the pages for ``n_new`` more tokens, or raise ``PagesExhausted``
        leaving everything as it was."""
        self.reserve_many([rid], [n_new])

    def reserve_many(self, rids: Sequence, n_new: Sequence[int]) -> None:
        """Pages for every request of a step, or ``PagesExhausted`` with nothing changed."""
        if any(int(n) <= 0 for n in n_new):
            raise ValueError("reserve needs at least one token")
        info = (ctypes.c_int * 3)()
        rc = self._lib.cc_reserve(self._h, len(rids), _ints([self._slot(r) for r in rids]), _ints([int(n) for n in n_new]),
                                  info)
        if rc == 1:
            raise PagesExhausted(info[0], info[1], info[2])
        if rc != 0:
            raise RuntimeError(native.last_error())

    def commit(self, rid, n_new: int) -> None:
        """``n_new`` tokens were written; give back pages a window has passed."""
        self.commit_many([rid], [n_new])

    def commit_many(self, rids: Sequence, n_new: Sequence[int]) -> None:
        self.generation += 1
        if self._lib.cc_commit(self._h, len(rids), _ints([self._slot(r) for r in rids]), _ints([int(n) for n in n_new])) != 0:
            raise RuntimeError(native.last_error())

    def truncate(self, rid, num_tokens: int) -> None:
        """Forget tokens past ``num_tokens`` and return whole pages beyond them."""
        self.generation += 1
        if self._lib.cc_truncate(self._h, self._slot(rid), int(num_tokens)) != 0:
            raise ValueError(native.last_error())

    def table(self, rid, g: int) -> List[int]:
        s = self._slot(rid)
        n = self._lib.cc_table_len(self._h, s, g)
        buf = (ctypes.c_int * max(1, n))()
        self._lib.cc_table(self._h, s, g, buf)
        return list(buf[:n])

    def slot(self, rid, g: int, pos: int) -> int:
        """Physical cache row of one position (the single-token case of ``slots``)."""
        return int(self.slots(rid, g, pos, 1)[0])

    def slots(self, rid, g: int, start: int, n: int) -> np.ndarray:
        """Physical cache rows (page * page_size + offset) of positions start..start+n-1."""
        out = np.empty(n, dtype=np.int32)
        if self._lib.cc_slots(self._h, self._slot(rid), g, int(start), int(n), out.ctypes.data_as(ctypes.c_void_p)) != 0:
            raise RuntimeError(f"request {rid!r}: {native.last_error()}")
        return out

    def fill_decode(self, rids: Sequence, tokens: Sequence[int], rows: int, width: int, scratch_pages: Sequence[int],
                    out: np.ndarray) -> None:
        """Pack the device inputs of a decode step (one new token per request, pages reserved) into ``out``
        (int32): tokens, positions, context lengths and state slots of ``rows`` rows, then per group the block
        tables [rows, width], then per group the cache rows of the new tokens.  Rows past ``len(rids)`` are
        padding that reads and writes the scratch page."""
        need = 4 * rows + len(self.groups) * rows * (width + 1)
        if out.dtype != np.int32 or out.size < need or not out.flags["C_CONTIGUOUS"]:
            raise ValueError("fill_decode: the buffer must be contiguous int32 of the packed size")
        rc = self._lib.cc_fill_decode(self._h, len(rids), _ints([self._slot(r) for r in rids]), _ints([int(t) for t in tokens]),
                                      int(rows), int(width), _ints([int(p) for p in scratch_pages]),
                                      out.ctypes.data_as(ctypes.c_void_p))
        if rc != 0:
            raise RuntimeError(native.last_error())

    def fill_step(self, slots: Sequence[int], n_new: np.ndarray, tokens: np.ndarray, n_want: np.ndarray, want: np.ndarray,
                  vocab: int, max_positions: int, scratch_pages: Sequence[int], out: np.ndarray):
        """Pack the device inputs of a step into ``out`` (int32): see ``cc_fill_step`` in the host library for the
        layout.  The step is checked (``ValueError``) and its pages are reserved (``PagesExhausted``) in the same call;
        a step that is refused changes nothing.  ``slots``: the state slots of the step's requests (``state_slot``).  Returns the meta list
        [N, M, total, largest count, largest context, single-token requests, widths per group], or None when
        ``out`` is too small (then ``self.last_fill_need`` says how many ints are needed)."""
        meta = (ctypes.c_int * (6 + max(1, len(self.groups))))()
        rc = self._lib.cc_fill_step(self._h, len(slots), _ints(slots), n_new.ctypes.data_as(ctypes.c_void_p),
                                    tokens.ctypes.data_as(ctypes.c_void_p), n_want.ctypes.data_as(ctypes.c_void_p),
                                    want.ctypes.data_as(ctypes.c_void_p), int(vocab), int(max_positions),
                                    _ints([int(p) for p in scratch_pages]), out.ctypes.data_as(ctypes.c_void_p),
                                    ctypes.c_long(out.size), meta)
        if rc == 1:
            raise PagesExhausted(meta[0], meta[1], meta[2])
        if rc == 2:
            self.last_fill_need = int(meta[2])
            return None
        if rc != 0:
            raise ValueError(native.last_error())
        return list(meta)

    # ---- statistics and invariants -------------------------------------
    def free_pages(self) -> List[int]:
        self._lib.cc_free_pages(self._h, self._g_buf)
        return list(self._g_buf[: len(self.groups)])

    def waste_ratio(self) -> float:
        """Share of held token places that hold no token
        (/root/reference/engine/src/kv_cache.rs:1066-1074)."""
        return float(self._lib.cc_waste_ratio(self._h))

    def check(self) -> None:
        """No page lost, held twice or free while in a table; state slots likewise."""
        assert self._lib.cc_check(self._h) == 0, native.last_error()
        assert self._lib.cc_num_live(self._h) == len(self._slot_of), "the core and the name table disagree"
