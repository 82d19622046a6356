"""The cache manager's bookkeeping (CPU): no page lost, held twice or freed twice, under random
orders of requests; windows give pages back; reservations fail without side effects."""
import random

import pytest

from tempura_amd.cache import CacheManager, PagesExhausted
from tempura_amd.parts import CacheSpec

FULL = CacheSpec("full", 2, 16)
WIN = CacheSpec("window", 2, 16, window=24)


def test_pages_are_conserved_and_used_again_most_recent_first():
    # invariant available + in_use == total (/root/reference/kernel-api/src/lib.rs:604-618)
    m = CacheManager([FULL], page_size=4, num_pages=4, max_requests=3)
    for rid in "ab":
        m.add(rid)
        m.reserve(rid, 4)
        m.commit(rid, 4)
    (pa,), (pb,) = m.table("a", 0), m.table("b", 0)
    assert pa != pb and m.free_pages() == [2]
    m.release("a")
    with pytest.raises(ValueError, match="not live"):
        m.release("a")                          # nothing is freed twice
    m.add("c")
    m.reserve("c", 12)
    assert m.table("c", 0)[0] == pa             # the most recently freed page is used again first
    m.add("a")
    with pytest.raises(PagesExhausted):
        m.reserve("a", 1)
    m.check()


def test_reserve_commit_release():
    m = CacheManager([FULL], page_size=8, num_pages=6, max_requests=2)
    m.add("a")
    assert m.pages_needed("a", 17) == [3]
    m.reserve("a", 17)
    m.commit("a", 17)
    assert m.num_tokens("a") == 17 and len(m.table("a", 0)) == 3 and m.free_pages() == [3]
    assert m.pages_needed("a", 7) == [0] and m.pages_needed("a", 8) == [1]
    slots = m.slots("a", 0, 15, 2)             # positions 15, 16: last row of page 1, first of page 2
    t = m.table("a", 0)
    assert list(slots) == [t[1] * 8 + 7, t[2] * 8 + 0]
    m.add("b")
    with pytest.raises(PagesExhausted) as ei:
        m.reserve("b", 8 * 4)
    assert ei.value.need == 4 and ei.value.free == 3
    assert m.table("b", 0) == [] and m.free_pages() == [3]        # nothing changed
    m.check()
    m.release("a")
    assert m.free_pages() == [6]
    with pytest.raises(ValueError, match="not live"):
        m.release("a")
    with pytest.raises(RuntimeError, match="no page reserved"):
        m.slots("b", 0, 0, 1)
    m.check()


def test_state_slots():
    m = CacheManager([FULL], 8, 4, max_requests=2)
    s0, s1 = m.add("a"), m.add("b")
    assert {s0, s1} == {0, 1}
    with pytest.raises(RuntimeError, match="no free state slot"):
        m.add("c")
    with pytest.raises(ValueError, match="already live"):
        m.add("a")
    m.release("a")
    assert m.add("c") == s0
    m.check()


def test_window_group_gives_pages_back():
    m = CacheManager([FULL, WIN], page_size=8, num_pages=[32, 12], max_requests=1)
    m.add("a")
    n = 0
    for chunk in [5, 20, 3, 1, 1, 40, 1, 1, 1, 17, 1]:
        m.reserve("a", chunk)
        m.commit("a", chunk)
        n += chunk
        t_full, t_win = m.table("a", 0), m.table("a", 1)
        assert all(p >= 0 for p in t_full) and len(t_full) == (n + 7) // 8
        first_visible = max(0, n - 24 + 1)       # the next query (position n) sees keys from here
        for lp, p in enumerate(t_win):
            if (lp + 1) * 8 <= first_visible:
                assert p == -1, f"page {lp} should be free after {n} tokens"
            else:
                assert p >= 0
        m.check()
    # between steps the window group holds the window and a page of slack, whatever the length
    assert m.pools[1].num_held <= 24 // 8 + 2
    m.release("a")
    assert m.free_pages() == [32, 12]


def test_window_pool_smaller_than_sequence():
    """A long request runs in a window pool far smaller than its length, because pages come back."""
    m = CacheManager([WIN], page_size=8, num_pages=6, max_requests=1)
    m.add("a")
    for _ in range(300):
        m.reserve("a", 1)
        m.commit("a", 1)
    assert m.num_tokens("a") == 300 and m.pools[0].num_held <= 4
    m.check()


def test_truncate():
    m = CacheManager([FULL], 8, 8, 1)
    m.add("a")
    m.reserve("a", 30)
    m.commit("a", 30)
    m.truncate("a", 9)
    assert m.num_tokens("a") == 9 and len(m.table("a", 0)) == 2 and m.free_pages() == [6]
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests(seed):
    """Requests arrive, grow by random portions, end in random order; the invariants hold throughout and
    every page comes back."""
    g = random.Random(seed)
    groups = [FULL, WIN] if seed % 2 else [FULL]
    m = CacheManager(groups, page_size=g.choice([4, 8, 16]), num_pages=40, max_requests=5)
    live = {}
    next_id = 0
    for _ in range(400):
        op = g.random()
        if op < 0.15 and len(live) < 5:
            m.add(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            rid = g.choice(list(live))
            n = g.choice([1, 1, 1, 2, 3, 7, 16, 33])
            before = (m.free_pages(), [m.table(rid, gi) for gi in range(len(groups))])
            try:
                m.reserve(rid, n)
            except PagesExhausted:
                assert (m.free_pages(), [m.table(rid, gi) for gi in range(len(groups))]) == before
                victim = g.choice(list(live))
                m.release(victim)
                del live[victim]
            else:
                m.commit(rid, n)
                live[rid] += n
                assert m.num_tokens(rid) == live[rid]
        elif live:
            rid = g.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.free_pages() == [40] * len(groups)


def test_fill_decode_packs_what_the_tables_say():
    """The packed inputs of a decode step: tokens, positions, lengths, state slots, block tables with
    given-back pages and padding pointed at the scratch page, and the cache row of every new token."""
    import numpy as np
    groups = [FULL, WIN]
    ps = 8
    m = CacheManager(groups, page_size=ps, num_pages=[20, 9], max_requests=4)
    lens = {"a": 45, "b": 3, "c": 16}
    for rid, n in lens.items():
        m.add(rid)
        m.reserve(rid, n)
        m.commit(rid, n)
    rids = ["c", "a", "b"]
    m.reserve_many(rids, [1, 1, 1])
    rows, width, scratch = 4, 8, [20, 9]
    out = np.full(4 * rows + 2 * rows * (width + 1), -7, dtype=np.int32)
    m.fill_decode(rids, [11, 12, 13], rows, width, scratch, out)
    tok, pos, ctxl, slot = (out[i * rows:(i + 1) * rows] for i in range(4))
    assert list(tok) == [11, 12, 13, 0] and list(pos) == [16, 45, 3, 0]
    assert list(ctxl) == [17, 46, 4, 1] and list(slot) == [m.state_slot(r) for r in rids] + [4]
    for g in range(2):
        bt = out[4 * rows + g * rows * width: 4 * rows + (g + 1) * rows * width].reshape(rows, width)
        sl = out[4 * rows + 2 * rows * width + g * rows: 4 * rows + 2 * rows * width + (g + 1) * rows]
        for r, rid in enumerate(rids):
            t = m.table(rid, g)
            want = [p if p >= 0 else scratch[g] for p in t] + [scratch[g]] * (width - len(t))
            assert list(bt[r]) == want
            assert sl[r] == m.slots(rid, g, lens[rid], 1)[0] == m.slot(rid, g, lens[rid])
        assert list(bt[3]) == [scratch[g]] * width and sl[3] == scratch[g] * ps
    assert any(p < 0 for p in m.table("a", 1)), "the window group gave pages of the long request back"
    assert m.max_num_tokens(rids) == 45
    m.commit_many(rids, [1, 1, 1])
    assert [m.num_tokens(r) for r in rids] == [17, 46, 4]
    m.check()
    with pytest.raises(RuntimeError):
        m.fill_decode(["a"], [1], rows, 3, scratch, out)          # a table of six pages does not fit three columns
    with pytest.raises(RuntimeError):
        m.fill_decode(["c", "a", "b", "c", "a"], [1] * 5, rows, width, scratch, out)   # more requests than rows


def test_visibility_rules_are_data():
    """A group's rule is a code of the host library and a few integers, named in cache/rules.py: ``chunk`` (a
    query sees the keys of its own aligned chunk) needs no line of the manager, and another kind that maps to one
    of the library's functions is registered from outside."""
    from tempura_amd.cache import VisibilityRule, register_rule
    chunk = CacheSpec("chunk", 2, 16, window=16)
    m = CacheManager([FULL, chunk], page_size=8, num_pages=[16, 4], max_requests=2)
    m.add("a")
    for n in (5, 20, 7, 1, 30):
        m.reserve("a", n)
        m.commit("a", n)
        m.check()
    # 63 tokens: the next query (position 63) lies in chunk 48..63, so pages below key 48 are back
    assert m.num_tokens("a") == 63 and [p >= 0 for p in m.table("a", 1)] == [False] * 6 + [True] * 2
    assert all(p >= 0 for p in m.table("a", 0)) and m.free_pages() == [8, 2]
    m.reserve("a", 1)
    m.commit("a", 1)                                 # position 64 opens a new chunk: nothing before it is seen again
    assert [p >= 0 for p in m.table("a", 1)] == [False] * 8
    m.release("a")
    # a kind of one's own over the library's "last n keys" rule, with twice the spec's number
    register_rule("window2x", VisibilityRule(1, lambda s: (2 * s.window,), lambda s, total, step: min(total, 2 * s.window + step)))
    m = CacheManager([CacheSpec("window2x", 1, 8, window=8)], page_size=8, num_pages=8, max_requests=1)
    m.add("b")
    m.reserve("b", 40)
    m.commit("b", 40)                                # the next query at 40 sees keys 25..40: pages 0..2 are back
    assert [p >= 0 for p in m.table("b", 0)] == [False] * 3 + [True] * 2
    with pytest.raises(ValueError, match="no visibility rule"):
        CacheManager([CacheSpec("sinks", 1, 8)], page_size=8, num_pages=8, max_requests=1)
