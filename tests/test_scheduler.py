"""The scheduler's decisions (CPU): admission, portions under a token budget, decoding first,
finishing and freeing, and what happens when pages run out."""
import random

import pytest

from tempura_amd.cache import CacheManager
from tempura_amd.engine.scheduler import Request, RequestState, Scheduler, SchedulerConfig
from tempura_amd.parts import CacheSpec
from tempura_amd.sampling import SamplingParams

FULL = CacheSpec("full", 2, 16)


def make(num_pages=64, page_size=8, **cfg):
    cache = CacheManager([FULL], page_size, num_pages, max_requests=cfg.get("max_num_seqs", 8))
    # (fill_budget off unless a test asks for it: the tests below pin the portions themselves)
    return Scheduler(SchedulerConfig(**{"max_num_seqs": 8, "max_num_batched_tokens": 32, "prefill_chunk_size": 16,
                                        "max_model_len": 512, "fill_budget": False, **cfg}), cache), cache


def req(rid, n_prompt, max_new=4, **kw):
    return Request(rid, list(range(1, n_prompt + 1)), SamplingParams(temperature=0, max_new_tokens=max_new, **kw))


def run(sched, cache, token_of=lambda r: 7, max_steps=10000, on_step=None):
    """Drive the scheduler as the engine does, with a stand-in for the model (reserve/commit only)."""
    steps = []
    while sched.has_unfinished():
        items = sched.schedule()
        assert items, "the scheduler made no progress"
        assert len({id(it.request) for it in items}) == len(items), "a request was scheduled twice in one step"
        for it in items:
            assert it.start == it.request.num_computed == cache.num_tokens(it.request.rid)
            cache.reserve(it.request.rid, it.count)
        for it in items:
            cache.commit(it.request.rid, it.count)
            sched.advance(it)
        for it in items:
            if it.samples:
                if sched.append_token(it.request, token_of(it.request)):
                    sched.finish(it.request)
        cache.check()
        steps.append([(it.request.rid, it.start, it.count, it.samples) for it in items])
        if on_step:
            on_step(items)
        assert len(steps) < max_steps
    return steps


def test_portions_under_budget_then_decode():
    sched, cache = make()
    sched.add_request(req("a", 40, max_new=3))
    steps = run(sched, cache)
    # 40 prompt tokens in portions of at most 16, the last portion samples; then one token per step
    assert steps[0] == [("a", 0, 16, False)] and steps[1] == [("a", 16, 16, False)] and steps[2] == [("a", 32, 8, True)]
    assert steps[3] == [("a", 40, 1, True)] and steps[4] == [("a", 41, 1, True)] and len(steps) == 5
    r = sched.finished[0]
    assert r.output == [7, 7, 7] and r.finish_reason == "length" and r.state == RequestState.FINISHED
    assert cache.free_pages() == [64] and not cache.live_requests()


def test_mixed_steps_decoding_first_and_budget():
    sched, cache = make(max_num_batched_tokens=20)
    sched.add_request(req("a", 5, max_new=30))
    sched.add_request(req("b", 50, max_new=2))
    sched.add_request(req("c", 9, max_new=2))
    seen_mixed = False

    def check(items):
        nonlocal seen_mixed
        assert sum(it.count for it in items) <= 20
        kinds = [it.request.is_decoding or it.count == 1 and it.samples for it in items]
        dec = [i for i, it in enumerate(items) if it.count == 1 and it.start >= len(it.request.prompt)]
        if dec and len(dec) < len(items):
            seen_mixed = True
            assert dec == list(range(len(dec))), "decoding requests come first in the batch"
    steps = run(sched, cache, on_step=check)
    assert seen_mixed, "prompt portions ran beside decoded tokens"
    assert sorted(r.rid for r in sched.finished) == ["a", "b", "c"]
    assert [len(r.output) for r in sorted(sched.finished, key=lambda r: r.rid)] == [30, 2, 2]
    # first step: a's whole prompt (5); b gets what is left of the budget of 20, cut at a multiple of 8 positions;
    # the 7 that remain reach no multiple of 8 of c's 9 tokens: c takes them all the same
    assert steps[0] == [("a", 0, 5, True), ("b", 0, 8, False), ("c", 0, 7, False)]


def test_portions_end_at_aligned_positions():
    """A portion that the budget or the chunk size cuts short of the prompt's end stops at a multiple of
    ``portion_align`` positions (when it has more than that many tokens), the last portion takes what is left;
    with an alignment of 1 the budget is used to the last token."""
    sched, cache = make(max_num_batched_tokens=21, prefill_chunk_size=13)
    sched.add_request(req("a", 50, max_new=1))
    steps = run(sched, cache)
    portions = [(start, count) for step in steps for _, start, count, _ in step if start < 50]
    assert portions == [(0, 8), (8, 8), (16, 8), (24, 8), (32, 8), (40, 10)]
    sched, cache = make(max_num_batched_tokens=21, prefill_chunk_size=13, portion_align=1)
    sched.add_request(req("a", 50, max_new=1))
    steps = run(sched, cache)
    assert [(start, count) for step in steps for _, start, count, _ in step if start < 50] == [(0, 13), (13, 13), (26, 13), (39, 11)]
    # a budget below the alignment is still used by a request that runs alone (and reaches a multiple when it can)
    sched, cache = make(max_num_batched_tokens=5, prefill_chunk_size=13)
    sched.add_request(req("a", 12, max_new=1))
    steps = run(sched, cache)
    assert [(start, count) for step in steps for _, start, count, _ in step if start < 12] == [(0, 5), (5, 3), (8, 4)]


def test_eos_stops_and_is_kept():
    sched, cache = make()
    r = req("a", 3, max_new=10)
    r.eos_token_ids = (99,)
    sched.add_request(r)
    toks = iter([5, 99, 6])
    run(sched, cache, token_of=lambda _r: next(toks))
    assert r.output == [5, 99] and r.finish_reason == "eos"      # the EOS token is kept (model.rs:9765)
    r2 = req("b", 3, max_new=3, ignore_eos=True)
    r2.eos_token_ids = (99,)
    sched.add_request(r2)
    run(sched, cache, token_of=lambda _r: 99)
    assert r2.output == [99, 99, 99] and r2.finish_reason == "length"


def test_max_num_seqs_and_fifo():
    sched, cache = make(max_num_seqs=2)
    for i in range(5):
        sched.add_request(req(i, 4, max_new=2))
    order = []
    run(sched, cache, on_step=lambda items: order.extend(it.request.rid for it in items if it.start == 0))
    assert order == [0, 1, 2, 3, 4]
    assert len(sched.finished) == 5


def test_request_that_can_never_fit_is_refused():
    sched, cache = make(num_pages=4, page_size=8)
    with pytest.raises(ValueError, match="pages"):
        sched.add_request(req("big", 30, max_new=10))
    with pytest.raises(ValueError, match="empty prompt"):
        sched.add_request(Request("e", [], SamplingParams()))
    with pytest.raises(ValueError, match="no room"):
        sched.add_request(req("long", 512, max_new=1))


def test_pages_run_out_preempt_newest_and_recompute():
    """Two requests outgrow the pool: the one admitted last is preempted (pages back, front of the queue,
    prompt + output recomputed) and both finish with every token they were promised."""
    sched, cache = make(num_pages=8, page_size=8, max_num_batched_tokens=64, prefill_chunk_size=64)
    a, b = req("a", 20, max_new=30), req("b", 20, max_new=30)     # each needs 50 tokens = 7 pages; the pool has 8
    sched.add_request(a)
    sched.add_request(b)
    counter = {"n": 0}

    def tok(r):
        counter["n"] += 1
        return len(r.output) + 100 * (1 if r.rid == "a" else 2)
    run(sched, cache, token_of=tok)
    assert sched.num_preemptions >= 1
    assert b.preemptions >= 1 and a.preemptions == 0, "the most recently admitted request is the victim"
    assert a.output == [100 + i for i in range(30)] and b.output == [200 + i for i in range(30)]
    assert cache.free_pages() == [8] and not cache.live_requests()


@pytest.mark.parametrize("seed", range(5))
def test_no_request_lost_under_a_tiny_pool(seed):
    # the reference's test_no_silent_drops (/root/reference/server/src/batch.rs:641-654)
    g = random.Random(seed)
    sched, cache = make(num_pages=12, page_size=4, max_num_seqs=4, max_num_batched_tokens=24, prefill_chunk_size=8,
                        max_model_len=64)
    want = {}
    for i in range(12):
        n, k = g.randint(1, 20), g.randint(1, 15)
        if n + k > 40:
            continue
        sched.add_request(req(i, n, max_new=k))
        want[i] = k
    steps = run(sched, cache)
    got = {r.rid: len(r.output) for r in sched.finished}
    assert got == want
    assert cache.free_pages() == [12]
    assert sched.pages_high_water[0] <= 12
    # and not by computing everything over and over: what preemptions threw away stays below what was kept
    useful = sum(len(r.prompt) + len(r.output) - 1 for r in sched.finished)
    assert sum(c for st in steps for _, _, c, _ in st) - useful <= useful // 2


def thrash_scenario(**cfg):
    sched, cache = make(page_size=8, max_num_batched_tokens=256, prefill_chunk_size=128, **cfg)
    rs = [req(i, 120, max_new=200) for i in range(4)]
    for r in rs:
        sched.add_request(r)
    steps = run(sched, cache, token_of=lambda r: 1000 * r.rid + len(r.output))
    return sched, rs, sum(c for st in steps for _, _, c, _ in st)


def test_admission_keeps_headroom_so_that_a_full_pool_is_not_admit_then_preempt():
    """Four requests of 120 + 200 tokens in a pool of 512 places: each alone needs 320, so they cannot all run to
    their ends at once.  Admitted whenever a first portion fits, the later ones were evicted a few steps after every
    admission (29 preemptions, two tokens recomputed for every useful one).  With the headroom
    (/root/reference/server/src/engine_task.rs:12-16,626-657) a request comes in only when all it has to compute
    fits beside a page of growth for everybody: same tokens as with room for all, at most four preemptions, and
    less thrown away than kept."""
    sched, rs, ran = thrash_scenario(num_pages=64)
    roomy, rs_roomy, ran_roomy = thrash_scenario(num_pages=256)
    assert roomy.num_preemptions == 0 and ran_roomy == 4 * (120 + 199)
    assert [r.output for r in rs] == [r.output for r in rs_roomy]
    assert all(len(r.output) == 200 for r in rs)
    assert sched.num_preemptions <= 4
    useful = 4 * (120 + 199)
    assert ran - useful <= useful, f"{ran - useful} tokens recomputed for {useful} useful ones"
    # the idle-pool exception: a pool that is smaller than prompt + headroom still admits when nothing runs
    sched, cache = make(num_pages=16, page_size=8, max_num_batched_tokens=256, prefill_chunk_size=128, admit_headroom=0.5)
    sched.add_request(req("a", 120, max_new=4))
    sched.add_request(req("b", 120, max_new=4))
    steps = run(sched, cache)
    assert sched.num_preemptions == 0 and sorted(r.rid for r in sched.finished) == ["a", "b"]
    assert all(len({rid for rid, *_ in st}) == 1 for st in steps), "b waits for a: 15 pages + headroom do not fit beside it"


def test_a_chunk_or_a_rest_of_the_budget_below_the_alignment_is_still_used():
    """Alignment buys speed, never a turn: with chunks of 4 tokens (below the alignment of 8) three prompts all
    advance in every step, and a prompt beside five decoding requests under a budget of 12 takes the 7 tokens left
    of it step by step instead of waiting until the decoders are done."""
    sched, cache = make(prefill_chunk_size=4, max_num_batched_tokens=32)
    for i in range(3):
        sched.add_request(req(i, 40, max_new=2))
    steps = run(sched, cache)
    assert steps[0] == [(0, 0, 4, False), (1, 0, 4, False), (2, 0, 4, False)]
    firsts = {}
    for n, st in enumerate(steps):
        for rid, _, _, samples in st:
            if samples:
                firsts.setdefault(rid, n)
    assert max(firsts.values()) - min(firsts.values()) <= 1, firsts
    sched, cache = make(max_num_batched_tokens=12, prefill_chunk_size=16)
    for i in range(5):
        sched.add_request(req(i, 2, max_new=400))
    for _ in range(2):                        # the five reach decoding (12 tokens of budget: 2+2+2+2+2)
        items = sched.schedule()
        for it in items:
            cache.reserve(it.request.rid, it.count); cache.commit(it.request.rid, it.count); sched.advance(it)
            if it.samples:
                sched.append_token(it.request, 7)
    sched.add_request(req("late", 30, max_new=1))
    seen = []
    for _ in range(6):
        items = sched.schedule()
        seen.append([(it.request.rid, it.start, it.count) for it in items if it.request.rid == "late"])
        for it in items:
            cache.reserve(it.request.rid, it.count); cache.commit(it.request.rid, it.count); sched.advance(it)
            if it.samples and sched.append_token(it.request, 7):
                sched.finish(it.request)
    assert seen[:5] == [[("late", 0, 7)], [("late", 7, 7)], [("late", 14, 7)], [("late", 21, 7)], [("late", 28, 2)]], seen


def test_abort_frees_at_once_wherever_the_request_stands():
    sched, cache = make(num_pages=16, max_num_seqs=2)
    a, b, c = req("a", 20, max_new=50), req("b", 20, max_new=50), req("c", 20, max_new=3)
    for r in (a, b, c):
        sched.add_request(r)
    seen = []

    def on_step(items):
        seen.append([it.request.rid for it in items])
        if len(seen) == 3:
            sched.abort(a, "client gone")        # running, holds pages
            sched.abort(c)                       # still waiting (two may run at once)
            sched.abort(c)                       # a second abort changes nothing
            assert not cache.has("a") and a.state == RequestState.FINISHED and a.finish_reason == "client gone"
            assert c.state == RequestState.FINISHED and c.finish_reason == "aborted" and c.num_computed == 0
            cache.check()

    run(sched, cache, on_step=on_step)
    assert b.finish_reason == "length" and len(b.output) == 50
    assert all("a" not in s and "c" not in s for s in seen[3:])
    assert sorted(r.rid for r in sched.finished) == ["a", "b", "c"]
    assert cache.pools[0].num_free == 16


def test_nothing_to_generate_finishes_on_arrival():
    sched, cache = make()
    r = req("z", 5, max_new=0)
    sched.add_request(r)
    assert r.state == RequestState.FINISHED and r.finish_reason == "length" and r.output == []
    assert not sched.has_unfinished() and cache.live_requests() == []
    sched.add_request(req("a", 5, max_new=2))
    steps = run(sched, cache)
    assert [s[0][0] for s in steps] == ["a", "a"]


def test_budget_nobody_else_can_use_lengthens_the_portions():
    """With ``fill_budget`` a chunk is a prompt's share while others wait for theirs: what is left of the budget
    when everybody has had a turn goes to the portions in the plan, in their order, still cut at aligned positions,
    never beyond the pages that are free; decoding requests keep their single tokens."""
    sched, cache = make(fill_budget=True)
    sched.add_request(req("a", 70, max_new=2))
    steps = run(sched, cache)
    assert steps[:3] == [[("a", 0, 32, False)], [("a", 32, 32, False)], [("a", 64, 6, True)]]
    # two prompts: each gets its chunk first, the first of them what is left
    sched, cache = make(fill_budget=True, max_num_batched_tokens=40)
    sched.add_request(req("a", 50, max_new=1))
    sched.add_request(req("b", 20, max_new=1))
    steps = run(sched, cache)
    assert steps[0] == [("a", 0, 24, False), ("b", 0, 16, False)]
    assert steps[1] == [("a", 24, 26, True), ("b", 16, 4, True)]
    # a decoding request beside a long prompt: one token for it, the rest of the budget for the prompt
    sched, cache = make(fill_budget=True)
    sched.add_request(req("d", 3, max_new=30))
    run_one = sched.schedule()
    for it in run_one:
        cache.reserve(it.request.rid, it.count); cache.commit(it.request.rid, it.count); sched.advance(it)
        sched.append_token(it.request, 7)
    sched.add_request(req("p", 100, max_new=1))
    items = sched.schedule()
    assert [(it.request.rid, it.start, it.count, it.samples) for it in items] == [("d", 3, 1, True), ("p", 0, 24, False)]
    # few pages: the portion grows only as far as the free pages allow (page size 8, 5 pages)
    sched, cache = make(num_pages=5, fill_budget=True, max_num_batched_tokens=64, prefill_chunk_size=16)
    sched.add_request(req("a", 39, max_new=1))
    sched.add_request(req("b", 30, max_new=1))
    items = sched.schedule()
    got = [(it.request.rid, it.start, it.count) for it in items]
    assert sum(-(-c // 8) for _, _, c in got) <= 5 and got[0][0] == "a" and got[0][2] >= 16
    # under random traffic nothing is lost and every request still finishes
    rng = random.Random(5)
    sched, cache = make(num_pages=24, fill_budget=True, max_num_batched_tokens=48)
    for i in range(12):
        sched.add_request(req(f"r{i}", rng.randint(1, 90), max_new=rng.randint(1, 6)))
    steps = run(sched, cache)
    assert all(sum(c for _, _, c, _ in st) <= 48 for st in steps)
    assert cache.free_pages() == [24]
