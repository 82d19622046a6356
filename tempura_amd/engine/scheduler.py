"""Continuous batching above the step function: admit, cut prompts into portions under
a token budget, decode, finish and free.

Every step is ONE mixed batch: first one token for every decoding request, then prompt
portions in admission order while the token budget lasts.  The reference instead runs one
512-token chunk per prefilling session per tick, each its own forward, and then one batched
decode (/root/reference/server/src/engine_task.rs:748-778; chunk size engine_task.rs:11,
queues and states /root/reference/server/src/batch.rs:13-56).

When pages run out the most recently admitted running request is preempted: its pages are
given back and it returns to the FRONT of the waiting queue with prompt + output so far as its
new prompt (recompute; the reference requeues preempted work first, batch.rs:137-142,214-229,
and otherwise swaps a victim out to host memory, engine_task.rs:261-289 — there is no host
tier here).  Its sampler draws are indexed by output length, so its continuation is unchanged.
A request that could never fit the pool alone is refused when it is added.

This module is host logic only; it needs a cache manager's bookkeeping, no GPU.
"""
from __future__ import annotations

import math
from collections import deque
from dataclasses import dataclass, field
from enum import Enum
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np

from ..cache import CacheManager
from ..cache.rules import rule_of
from ..sampling.params import SamplingParams


class RequestState(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass
class Request:
    rid: Hashable
    prompt: List[int]
    params: SamplingParams
    eos_token_ids: Tuple[int, ...] = ()
    output: List[int] = field(default_factory=list)
    state: RequestState = RequestState.WAITING
    num_computed: int = 0            # tokens of prompt + output whose keys/values are cached
    preemptions: int = 0
    finish_reason: Optional[str] = None
    arrival: int = 0
    logprobs_top_n: Optional[int] = None     # not None: keep a log-probability record per generated token
    logprobs: List[object] = field(default_factory=list)
    _array: Optional[object] = field(default=None, repr=False, compare=False)

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def num_tokens(self) -> int:
        return len(self.prompt) + len(self.output)

    def step_tokens(self, start: int, count: int):
        """Tokens start .. start + count - 1 of prompt + output, as a step entry takes them: the newest token alone
        as a list, a portion as a slice of an int32 array that is made once per prefill (not once per step)."""
        n = self.num_tokens
        if count == 1 and start == n - 1 and self.output:
            return self.output[-1:]
        arr = self._array
        if arr is None or arr.size != n:
            arr = self._array = np.asarray(self.prompt + self.output, dtype=np.int32)
        return arr[start: start + count]

    @property
    def is_decoding(self) -> bool:
        """Only the newest token is not yet cached."""
        return self.num_tokens - self.num_computed == 1 and len(self.output) > 0


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 64                  # the reference's --max-batch-size (server/src/lib.rs:45-110)
    max_num_batched_tokens: int = 2048      # token budget of one step
    prefill_chunk_size: int = 512           # largest prompt portion (engine_task.rs:11)
    max_model_len: int = 4096               # the reference's --max-seq-len
    portion_align: int = 8                  # a prompt portion that is not the last ends at a multiple of this (the engine asks the model's parts)
    fill_budget: bool = True                # budget that no other request can use lengthens the portions in the plan
    #: share of every page pool that an admission must leave free while other requests run (never less than one page
    #: for each of them and one for the newcomer): the reference stops admitting below a headroom of free tokens
    #: "to prevent admit/requeue spinning when the pool is full", with an exception for an idle pool
    #: (/root/reference/server/src/engine_task.rs:12-16,626-657)
    admit_headroom: Optional[float] = 0.02  # None: no headroom, a request comes in as soon as its first portion fits


@dataclass
class ScheduledItem:
    request: Request
    start: int          # first position run in this step
    count: int          # tokens run in this step
    samples: bool       # the step reaches the request's newest token: a token is sampled


class Scheduler:
    def __init__(self, config: SchedulerConfig, cache: CacheManager):
        if config.max_num_batched_tokens < 1 or config.prefill_chunk_size < 1 or config.max_num_seqs < 1:
            raise ValueError("scheduler limits must be positive")
        self.config = config
        self.cache = cache
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []      # in admission order
        self.finished: List[Request] = []
        self._arrivals = 0
        self.num_preemptions = 0
        self.pages_high_water = [0] * len(cache.pools)

    # ---- intake --------------------------------------------------------
    def add_request(self, req: Request) -> None:
        if not req.prompt:
            raise ValueError(f"request {req.rid!r}: empty prompt")
        if req.params.max_new_tokens == 0:
            # nothing to generate: finished as it arrives, without a step and without a sampled token
            req.arrival = self._arrivals
            self._arrivals += 1
            req.finish_reason = "length"
            req.state = RequestState.FINISHED
            self.finished.append(req)
            return
        total = len(req.prompt) + req.params.max_new_tokens
        limit = self.config.max_model_len
        if len(req.prompt) >= limit and req.params.max_new_tokens > 0:
            raise ValueError(f"request {req.rid!r}: prompt of {len(req.prompt)} tokens leaves no room under max length {limit}")
        # It must fit the pool when it is the only request, or it could never finish.
        need_tokens = min(total, limit)
        ps = self.cache.page_size
        step = min(self.config.prefill_chunk_size, self.config.max_num_batched_tokens)
        for g, pool in enumerate(self.cache.pools):
            spec = self.cache.groups[g]
            # (a group that gives pages back holds what its rule still shows plus the step in flight and a page of slack)
            tokens_held = rule_of(spec.kind).held_tokens(spec, need_tokens, step)
            if tokens_held < need_tokens:
                tokens_held = min(need_tokens, tokens_held + ps)
            if (tokens_held + ps - 1) // ps > pool.num_pages:
                raise ValueError(
                    f"request {req.rid!r}: needs {(tokens_held + ps - 1) // ps} pages of cache group {g}, the pool has {pool.num_pages}")
        req.arrival = self._arrivals
        self._arrivals += 1
        req.state = RequestState.WAITING
        self.waiting.append(req)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- one step's plan -------------------------------------------------
    def _portion(self, req: Request, budget: int) -> int:
        """Tokens of the request's prompt for this step: what is left, at most a chunk, at most the budget.  A
        portion that is cut short of the prompt's end is cut at a multiple of ``portion_align`` positions where it
        reaches one at the price of less than half its tokens, so that the next one starts there (cache rows are
        written in aligned groups of eight where they can be).  Otherwise (a chunk size or a rest of the budget
        about as small as the alignment) it takes the tokens all the same: the alignment buys speed, and a request
        that waited for an aligned cut beside busy decoders would wait for as long as they run."""
        rest = req.num_tokens - req.num_computed
        count = min(rest, self.config.prefill_chunk_size, budget)
        align = self.config.portion_align
        if count < rest and align > 1:
            over = (req.num_computed + count) % align
            if 2 * over <= count:
                count -= over
        return count

    def _fits(self, req: Request, count: int, planned: List[int]) -> bool:
        need = self.cache.pages_needed(req.rid, count)
        free = self.cache.free_pages()
        return all(n + p <= f for n, p, f in zip(need, planned, free))

    def _admissible(self, req: Request, count: int, planned: List[int]) -> bool:
        """May a waiting request join the step with a first portion of ``count`` tokens?  Into an idle engine: when
        that portion fits.  Beside running requests: when every pool can take ALL the tokens it has to compute (the
        whole prompt, and for a preempted request its output so far), not only the first portion, and still keeps
        the headroom free: the running requests go on growing by a page each every ``page_size`` steps, and a
        request admitted into the last free pages would be evicted again a few steps later, its work thrown away
        (admitted and preempted in turns, such a request cost two tokens computed for every useful one)."""
        if not self._fits(req, count, planned):
            return False
        if not self.running or self.config.admit_headroom is None:
            return True
        ps = self.cache.page_size
        rest = req.num_tokens - req.num_computed
        step = min(self.config.prefill_chunk_size, self.config.max_num_batched_tokens)
        free = self.cache.free_pages()
        for g, pool in enumerate(self.cache.pools):
            spec = self.cache.groups[g]
            held = rule_of(spec.kind).held_tokens(spec, rest, step)
            if held < rest:
                held = min(rest, held + ps)
            headroom = max(math.ceil(self.config.admit_headroom * pool.num_pages), len(self.running) + 1) * (1 + req.preemptions)
            if (held + ps - 1) // ps + headroom + planned[g] > free[g]:
                return False
        return True

    def _preempt(self, victim: Request) -> None:
        self.cache.release(victim.rid)
        victim.num_computed = 0
        victim.state = RequestState.WAITING
        victim.preemptions += 1
        self.num_preemptions += 1
        self.running.remove(victim)
        self.waiting.appendleft(victim)

    def schedule(self) -> List[ScheduledItem]:
        """Decide the next step.  Pages are only counted here; the step function reserves them."""
        budget = self.config.max_num_batched_tokens
        planned = [0] * len(self.cache.pools)          # pages promised to items already in the plan
        items: List[ScheduledItem] = []

        def take(req: Request, count: int) -> None:
            nonlocal budget
            need = self.cache.pages_needed(req.rid, count)
            for g, n in enumerate(need):
                planned[g] += n
            items.append(ScheduledItem(req, req.num_computed, count, req.num_computed + count == req.num_tokens))
            budget -= count

        # 1. running requests, decoding ones first, then prompt portions, each in admission order
        order = [r for r in self.running if r.is_decoding] + [r for r in self.running if not r.is_decoding]
        for req in order:
            if req not in self.running:          # preempted while serving an earlier one
                continue
            if budget <= 0:
                break
            count = 1 if req.is_decoding else self._portion(req, budget)
            if count == 0:
                continue
            while not self._fits(req, count, planned):
                # give back the pages of the most recently admitted request that is not in the plan yet
                victims = [r for r in reversed(self.running) if r is not req and all(it.request is not r for it in items)]
                if not victims:
                    break
                self._preempt(victims[0])
            else:
                take(req, count)
                continue
            # nothing left to preempt: skip this request in this step unless it is the only work
            if not items and len(self.running) == 1:
                raise RuntimeError(f"request {req.rid!r} cannot get pages although it runs alone")

        # 2. admit waiting requests (preempted ones are at the front)
        while self.waiting and budget > 0 and len(self.running) < self.config.max_num_seqs:
            req = self.waiting[0]
            if not self.cache.has(req.rid):
                if len(self.cache.live_requests()) >= self.cache.max_requests:
                    break
                self.cache.add(req.rid)
            count = self._portion(req, budget)
            if count == 0 or not self._admissible(req, count, planned):
                self.cache.release(req.rid)
                break
            self.waiting.popleft()
            req.state = RequestState.RUNNING
            self.running.append(req)
            take(req, count)

        # 3. budget that is left when everybody has had a turn goes to the prompt portions already in the plan, in
        # their order: a chunk is the share of a prompt while others wait for theirs, not a bound on a step that
        # has room (one request with a prompt of 2,048 tokens: one step instead of four of 512, which the kernels
        # run at three quarters of the speed)
        if self.config.fill_budget and budget > 0:
            align = self.config.portion_align
            free = self.cache.free_pages()
            for idx, it in enumerate(items):
                req = it.request
                rest = req.num_tokens - (it.start + it.count)
                if it.samples or rest <= 0:
                    continue
                extra = min(rest, budget)
                if extra < rest and align > 1:
                    extra -= (it.start + it.count + extra) % align
                if extra <= 0:
                    continue
                old = self.cache.pages_needed(req.rid, it.count)
                new = self.cache.pages_needed(req.rid, it.count + extra)
                if any(planned[g] + new[g] - old[g] > free[g] for g in range(len(planned))):
                    continue
                for g in range(len(planned)):
                    planned[g] += new[g] - old[g]
                items[idx] = ScheduledItem(req, it.start, it.count + extra, extra == rest)
                budget -= extra
                if budget <= 0:
                    break

        for g, pool in enumerate(self.cache.pools):
            self.pages_high_water[g] = max(self.pages_high_water[g], pool.num_held + planned[g])
        return items

    # ---- after the step ---------------------------------------------------
    def advance(self, item: ScheduledItem) -> None:
        """The step wrote ``item.count`` tokens of the request."""
        item.request.num_computed += item.count

    def append_token(self, req: Request, token: int) -> bool:
        """Record a sampled token; returns True when the request is finished
        (/root/reference/server/src/engine_task.rs:64-66: token budget or EOS; the EOS token is kept)."""
        req.output.append(int(token))
        if not req.params.ignore_eos and int(token) in req.eos_token_ids:
            req.finish_reason = "eos"
        elif len(req.output) >= req.params.max_new_tokens:
            req.finish_reason = "length"
        elif req.num_tokens >= self.config.max_model_len:
            req.finish_reason = "max_model_len"
        return req.finish_reason is not None

    def abort(self, req: Request, reason: str = "aborted") -> None:
        """End a request from outside, wherever it stands (the reference ends a sequence whose client is
        gone, /root/reference/server/src/engine_task.rs:64-66); what it holds is given back."""
        if req.state == RequestState.FINISHED:
            return
        if req in self.waiting:
            self.waiting.remove(req)
        req.finish_reason = reason
        self.finish(req)

    def finish(self, req: Request) -> None:
        """Give back the request's pages and state slot at once."""
        if req in self.running:
            self.running.remove(req)
        if self.cache.has(req.rid):
            self.cache.release(req.rid)
        req.state = RequestState.FINISHED
        self.finished.append(req)
