"""The Python entry point: a model folder (or a configuration with random weights) to tokens.

Shaped after the reference's ``InferenceModel`` (``forward``, ``generate``,
/root/reference/engine/src/model.rs:305-448) and its serving loop
(/root/reference/server/src/engine_task.rs:581-875), with option names taken from the
reference's ``ServeArgs`` where it has them (``max_batch_size``, ``max_seq_len``,
/root/reference/server/src/lib.rs:45-110).
"""
from __future__ import annotations

import itertools
import time
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Tuple, Union

import torch

from ..config import load_config
from ..kernels import ops
from ..sampling import Sampler, SamplingParams
from .loading import load_model, parse_dtype, random_model
from .model import CausalLM
from .runner import ModelRunner, StepEntry
from ..cache import PagesExhausted
from .scheduler import Request, RequestState, ScheduledItem, Scheduler, SchedulerConfig


class Engine:
    def __init__(self, model: Union[str, object], dtype: str = "bfloat16", random_weights: bool = False,
                 seed: int = 0, page_size: int = 16, kv_pages: Optional[int] = None,
                 gpu_memory_utilization: float = 0.9, max_batch_size: int = 64,
                 max_seq_len: Optional[int] = None, max_num_batched_tokens: int = 2048,
                 prefill_chunk_size: int = 512, device: str = "cuda:0", use_graph: bool = True,
                 chain_steps: bool = True, fill_budget: bool = True, admit_headroom: Optional[float] = 0.02):
        """``model``: a folder with config.json and safetensors, or (with ``random_weights``) a typed
        configuration such as ``LlamaConfig``/``PRESETS[name]``.
        ``kv_pages``: cache pages per group; by default as many as ``gpu_memory_utilization`` of the
        free memory holds, but no more than ``max_batch_size`` requests of ``max_seq_len`` need.
        ``prefill_chunk_size``: a prompt's share of a step while other prompts wait for theirs; with ``fill_budget``
        what is left of ``max_num_batched_tokens`` when everybody has had a turn lengthens the portions in the plan
        (a lone long prompt runs in steps of the whole budget).
        ``chain_steps``: while every running request is decoding and nobody waits, the next step is queued
        behind the sampling kernel (its tokens stay on the device) before the host has read this step's
        tokens, so the GPU does not wait for the host between steps; a request that ends on the token just
        read has then one row computed for nothing.  What the caller sees does not change.
        ``admit_headroom``: share of the cache pages that an admission leaves free beside running requests (None:
        a request comes in as soon as its first portion fits; see ``SchedulerConfig.admit_headroom``)."""
        self.device = torch.device(device)
        if isinstance(model, str):
            if random_weights:
                self.model = random_model(load_config(model), seed, dtype, device)
            else:
                self.model = load_model(model, dtype, device)
        elif isinstance(model, CausalLM):
            self.model = model
        else:
            if not random_weights:
                raise ValueError("a configuration without a folder needs random_weights=True")
            self.model = random_model(model, seed, dtype, device)
        spec = self.model.spec
        self.max_seq_len = min(int(max_seq_len or spec.max_positions), spec.max_positions)
        self.page_size = int(page_size)
        if kv_pages is None:
            kv_pages = self._pages_from_memory(gpu_memory_utilization, max_batch_size)
        # (one request slot more than the scheduler hands out: ``forward`` and ``dump`` run their fresh request in it
        # also while ``max_batch_size`` requests are live)
        self.runner = ModelRunner(self.model, self.page_size, int(kv_pages), max_requests=max_batch_size + 1,
                                  use_graph=use_graph)
        self.scheduler = Scheduler(
            SchedulerConfig(max_num_seqs=max_batch_size, max_num_batched_tokens=max_num_batched_tokens,
                            prefill_chunk_size=prefill_chunk_size, max_model_len=self.max_seq_len,
                            fill_budget=fill_budget, admit_headroom=admit_headroom,
                            portion_align=self.model.portion_align()),
            self.runner.cache)
        self.sampler = Sampler(spec.vocab_size, self.device, default_seed=seed)
        self._ids = itertools.count()            # request ids that add_request hands out: 0, 1, 2, ...
        self._own_ids = itertools.count()        # names of the engine's own short-lived requests (forward, profile)
        self._requests: Dict[Hashable, Request] = {}
        self.counters = {"steps": 0, "prompt_tokens": 0, "generated_tokens": 0, "batched_tokens": 0, "chained_steps": 0}
        self.chain_steps = bool(chain_steps) and self.runner.use_graph     # (a model with parts that cannot be captured runs eagerly)
        self._ahead = None      # (requests, logits) of a step that is already queued
        #: what the last call of ``step`` ran: single decoded tokens, prompt tokens in portions, requests, and
        #: whether the step had been queued ahead
        self.last_step = {"decode_tokens": 0, "prompt_tokens": 0, "requests": 0, "queued_ahead": False}

    def _pages_from_memory(self, utilization: float, max_batch_size: int) -> int:
        m = self.model
        elem = 2 if m.dtype == torch.bfloat16 else 4
        # (what a page costs is the cache spec's to say: every slot of every group holds one page of each plane)
        per_page = sum(n * g.page_bytes(self.page_size, elem) for g, n in zip(m.cache_groups, m.slots_per_group)) or 1
        pages_cap = max_batch_size * ((self.max_seq_len + self.page_size - 1) // self.page_size)
        if self.device.type != "cuda":
            return pages_cap
        free, _total = torch.cuda.mem_get_info(self.device)
        workspace = 2 << 30            # activations of the largest step, logits, sampler scratch
        # the fixed-size state of every request slot comes out of the same memory
        state_bytes = sum((max_batch_size + 2) * torch.Size(s.shape).numel() * torch.empty((), dtype=s.dtype).element_size()
                          for s in m.state_specs.values())
        budget = int(free * utilization) - workspace - state_bytes
        return max(1, min(pages_cap, budget // per_page))

    # ---- requests ------------------------------------------------------------
    def add_request(self, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    rid: Optional[Hashable] = None, logprobs_top_n: Optional[int] = None) -> Hashable:
        """Queue a request.  With ``logprobs_top_n`` (0..20) every generated token gets a ``TokenLogprob``
        record in ``request(rid).logprobs``."""
        params = params or SamplingParams()
        if rid is None:
            rid = next(self._ids)
        if rid in self._requests and self._requests[rid].state != RequestState.FINISHED:
            raise ValueError(f"request id {rid!r} is in use")
        vocab = self.model.spec.vocab_size
        for t in prompt_ids:
            if t < 0 or t >= vocab:
                raise ValueError(f"token id {t} outside the vocabulary of {vocab}")
        eos = params.eos_token_id if params.eos_token_id is not None else self.model.spec.eos_token_ids
        req = Request(rid, [int(t) for t in prompt_ids], params, tuple(int(e) for e in eos),
                      logprobs_top_n=logprobs_top_n)
        self.scheduler.add_request(req)
        self._requests[rid] = req
        self.counters["prompt_tokens"] += len(req.prompt)
        return rid

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished()

    def step(self) -> List[Tuple[Hashable, int, bool]]:
        """One scheduler decision, one model step, one sampling pass.
        Returns (request id, new token, finished) for every request that got a token."""
        ahead, self._ahead = self._ahead, None
        if ahead is not None:
            # This step was queued while the last one's tokens were read.  Rows of requests that ended on those
            # tokens (or were aborted since) are dropped; their pages are back already.
            reqs, logits = ahead
            live = [i for i, r in enumerate(reqs) if r.state != RequestState.FINISHED]
            if not live:
                return self.step() if self.has_unfinished() else []
            items = [ScheduledItem(reqs[i], reqs[i].num_tokens - 1, 1, True) for i in live]
            if len(live) < len(reqs):
                logits = ops.take_rows(logits, live)
            self.last_step = {"decode_tokens": len(items), "prompt_tokens": 0, "requests": len(items), "queued_ahead": True}
        else:
            items = self.scheduler.schedule()
            if not items:
                return []
            # Prompt portions go first in the batch, single tokens last: a portion that starts at a multiple of the
            # alignment the model's parts prefer (attention: eight positions) then also starts at that multiple of
            # rows, which is what lets the projection's epilogue store eight tokens' values as one piece of the
            # transposed value cache.
            # Among the single tokens the longest contexts go first: attention hands its blocks out in this order,
            # and a batch of short and long contexts ends sooner when the long ones start first (60 requests of
            # 128 to 2,304 keys: 77 -> 74 us a layer).
            # (and portions whose length is no such multiple, the ends of prompts, go behind the others: every
            # portion behind one of them starts at an odd row)
            align = self.scheduler.config.portion_align
            items.sort(key=lambda it: (it.count == 1, it.count % align != 0 if it.count > 1 else -it.start))
            entries = []
            for it in items:
                toks = it.request.step_tokens(it.start, it.count)
                entries.append(StepEntry(it.request.rid, toks, [it.count - 1] if it.samples else []))
            logits = self.runner.step(entries)
            self.counters["steps"] += 1
            self.counters["batched_tokens"] += sum(it.count for it in items)
            decoding = sum(1 for it in items if it.count == 1 and it.samples and it.request.output)
            self.last_step = {"decode_tokens": decoding, "prompt_tokens": sum(it.count for it in items) - decoding,
                              "requests": len(items), "queued_ahead": False}
        for it in items:
            self.scheduler.advance(it)
        sampling = [it.request for it in items if it.samples]
        out: List[Tuple[Hashable, int, bool]] = []
        if sampling:
            wanted = [r.logprobs_top_n for r in sampling if r.logprobs_top_n is not None]
            tokens = self.sampler.sample(
                logits, [r.params for r in sampling], [len(r.output) for r in sampling],
                [r.prompt for r in sampling], [r.output for r in sampling], top_n=max(wanted) if wanted else None,
                meanwhile=self._queue_next(items) if not wanted else None)
            if wanted:
                tokens, records = tokens
                for req, rec in zip(sampling, records):
                    if req.logprobs_top_n is not None:
                        rec.top_logprobs = rec.top_logprobs[: req.logprobs_top_n]
                        req.logprobs.append(rec)
            for req, tok in zip(sampling, tokens):
                done = self.scheduler.append_token(req, tok)
                self.counters["generated_tokens"] += 1
                if done:
                    self.scheduler.finish(req)
                out.append((req.rid, int(tok), done))
        return out

    def _queue_next(self, items) -> Optional[Callable]:
        """What to do between the launch of the sampling kernels and the wait for their tokens: when this was a
        step of single tokens and nobody waits, the next step will bring one token for the same requests, less
        those that reach their length now, so it is queued at once with the tokens still on the device (a
        request that ends on its token leaves a row computed for nothing).  None when that does not apply."""
        if not self.chain_steps or self.scheduler.waiting or not all(it.count == 1 and it.samples for it in items):
            return None
        if len(items) != len(self.scheduler.running):
            return None         # a running request was left out of this step: the scheduler must see it again
        limit = self.scheduler.config.max_model_len
        keep = [i for i, it in enumerate(items)
                if len(it.request.output) + 1 < it.request.params.max_new_tokens and it.request.num_tokens + 1 < limit]
        if not keep:
            return None
        reqs = [items[i].request for i in keep]

        def queue(chosen: torch.Tensor) -> None:
            rids = [r.rid for r in reqs]
            toks = chosen if len(keep) == len(items) else ops.take_rows(chosen, keep)
            try:
                logits = self.runner.step_chained(rids, toks)
            except PagesExhausted:
                return              # the scheduler decides who gives way, in the next call
            self.counters["steps"] += 1
            self.counters["chained_steps"] += 1
            self.counters["batched_tokens"] += len(rids)
            self._ahead = (reqs, logits)
            self.runner.prepare_decode(rids)
        return queue

    def generate(self, prompts: Sequence[Sequence[int]], params: Union[SamplingParams, Sequence[SamplingParams], None] = None
                 ) -> List[List[int]]:
        """Generate for every prompt (token ids in, token ids out); continuous batching inside."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt")
        rids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        while self.has_unfinished():
            self.step()
        return [list(self._requests[r].output) for r in rids]

    def generate_with_logprobs(self, prompts: Sequence[Sequence[int]],
                               params: Union[SamplingParams, Sequence[SamplingParams], None] = None, top_n: int = 0):
        """``generate`` that also returns, per prompt, one ``TokenLogprob`` per generated token: the token's
        log-probability under the distribution it was drawn from and the ``top_n`` (at most 20) most probable
        tokens of that distribution (/root/reference/engine/src/model.rs:9817-9887)."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt")
        rids = [self.add_request(p, sp, logprobs_top_n=top_n) for p, sp in zip(prompts, params)]
        while self.has_unfinished():
            self.step()
        return ([list(self._requests[r].output) for r in rids], [list(self._requests[r].logprobs) for r in rids])

    def generate_with_callback(self, prompts: Sequence[Sequence[int]],
                               params: Union[SamplingParams, Sequence[SamplingParams], None],
                               on_token: Callable[[int, int], bool]) -> List[List[int]]:
        """``generate`` that hands every new token to ``on_token(prompt index, token)`` as soon as it is drawn;
        a false return ends that prompt's generation there, the token kept
        (/root/reference/engine/src/model.rs:9889-9960)."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt")
        rids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        index = {r: i for i, r in enumerate(rids)}
        while self.has_unfinished():
            for rid, tok, done in self.step():
                if rid in index and not on_token(index[rid], tok) and not done:
                    self.abort(rid, "callback")
        return [list(self._requests[r].output) for r in rids]

    def abort(self, rid: Hashable, reason: str = "aborted") -> None:
        """End a request now, wherever it stands; its pages and state slot are free at once."""
        self.scheduler.abort(self._requests[rid], reason)

    def sample_from_logits(self, logits: torch.Tensor, params: Optional[SamplingParams] = None, draw_index: int = 0,
                           prompt_tokens: Sequence[int] = (), output_tokens: Sequence[int] = ()) -> int:
        """One token from one row of logits ([vocab], any float dtype, host or device) by the engine's sampler
        (/root/reference/engine/src/model.rs:363-368).  ``draw_index`` numbers the draw within its stream."""
        row = logits.detach().to(device=self.device, dtype=torch.float32).reshape(1, -1).contiguous()
        if row.shape[1] != self.model.spec.vocab_size:
            raise ValueError(f"logits of {row.shape[1]} entries for a vocabulary of {self.model.spec.vocab_size}")
        return int(self.sampler.sample(row, [params or SamplingParams()], [draw_index], [list(prompt_tokens)],
                                       [list(output_tokens)])[0])

    def forward(self, token_ids: Sequence[int]) -> torch.Tensor:
        """Logits [vocab] (float32, host) after a whole prompt of a fresh request
        (the reference's ``forward``, /root/reference/engine/src/model.rs:308)."""
        if self._ahead is not None:      # a queued step's logits live in a graph's output buffer: keep a copy
            self._ahead = (self._ahead[0], ops.take_rows(self._ahead[1]))
        rid = ("forward", next(self._own_ids))
        self.runner.add_request(rid)      # (the slot kept back from the scheduler: free whatever else is live)
        try:
            logits = self.runner.step([StepEntry(rid, list(token_ids), [len(token_ids) - 1])])
        except PagesExhausted as e:
            e.args = (f"forward: a prompt of {len(token_ids)} tokens needs {e.need} more cache pages of group {e.group} and "
                      f"the live requests leave {e.free} free; end some of them or give the engine more pages (kv_pages)",)
            raise
        finally:
            self.runner.end_request(rid)
        return logits[0].cpu()

    def profile(self, prompt_len: int = 128, batch: int = 1, decode_steps: int = 4, layer_stats: bool = False,
                seed: int = 0) -> Dict[str, object]:
        """Where a step's time goes: ``batch`` fresh requests with prompts of ``prompt_len`` seeded random tokens,
        one eager step for all prompts and ``decode_steps`` eager steps of one token each (after one untimed pass of
        the same shapes), every call into the kernel library between a pair of stream events (``ops.KernelTimer``;
        the reference times layers and prints per-tick times behind environment switches,
        /root/reference/engine/src/model.rs:1342-1345, /root/reference/server/src/engine_task.rs:530-553).  Returns ``{"prefill": rows, "decode": rows}`` with rows
        (entry point, calls, microseconds, share), the decode rows summed over the steps; with ``layer_stats`` also
        ``"layers"``: mean, variance and largest magnitude of the residual stream before every layer and after the
        last, for the prompts' step (the reference's summary trace, /root/reference/engine/src/pipeline.rs:149-187).
        The requests are ended afterwards; nothing of the engine's own queue is touched."""
        import random as _random
        if self._ahead is not None:
            self._ahead = (self._ahead[0], ops.take_rows(self._ahead[1]))
        g = _random.Random(seed)
        vocab = self.model.spec.vocab_size
        rids = [("profile", next(self._own_ids)) for _ in range(batch)]
        prompts = [[g.randrange(vocab) for _ in range(prompt_len)] for _ in rids]
        runner = self.runner
        keep_graph, runner.use_graph = runner.use_graph, False
        stats: List[tuple] = []

        def observe(i, h):
            hd = h.double()
            stats.append((i, float(hd.mean()), float(hd.var(unbiased=False)), float(hd.abs().max())))

        def rows_of(timer):
            table = timer.table()
            total = sum(r[3] for r in table) or 1.0
            return [(name, calls, round(us, 1), round(us / total, 4)) for name, _, calls, us in table]

        out: Dict[str, object] = {}
        # Once untimed: a pair of events also spans what the host does between them while the GPU waits, and the
        # first step of a new size allocates its buffers (the q/k/v projection of 2,048 rows showed as 117 us
        # cold, 39 us after).
        for rid in rids:
            runner.add_request(rid)
        try:
            logits = runner.step([StepEntry(rid, p, [prompt_len - 1]) for rid, p in zip(rids, prompts)])
            if decode_steps > 0:
                runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, ops.argmax(logits).tolist())])
        finally:
            for rid in rids:
                runner.end_request(rid)
        for rid in rids:
            runner.add_request(rid)
        try:
            self.model.observer = observe if layer_stats else None
            with ops.KernelTimer() as timer:
                logits = runner.step([StepEntry(rid, p, [prompt_len - 1]) for rid, p in zip(rids, prompts)])
            self.model.observer = None
            out["prefill"] = rows_of(timer)
            if layer_stats:
                out["layers"] = stats
            with ops.KernelTimer() as timer:
                for _ in range(decode_steps):
                    nxt = ops.argmax(logits).tolist()
                    logits = runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, nxt)])
            out["decode"] = rows_of(timer)
        finally:
            self.model.observer = None
            runner.use_graph = keep_graph
            for rid in rids:
                runner.end_request(rid)
        return out

    def request(self, rid) -> Request:
        return self._requests[rid]

    def stats(self) -> Dict[str, object]:
        s = dict(self.counters)
        s["preemptions"] = self.scheduler.num_preemptions
        s["pages_high_water"] = list(self.scheduler.pages_high_water)
        s["pages_total"] = [p.num_pages for p in self.runner.cache.pools]
        # share of the held token places that hold no token (/root/reference/engine/src/kv_cache.rs:1066-1074)
        s["waste_ratio"] = self.runner.cache.waste_ratio()
        s["cache_bytes"] = self.runner.pools.bytes()
        s["weight_bytes"] = self.model.weight_bytes()
        s["graph_steps"] = self.runner.graph_steps
        s["eager_steps"] = self.runner.host_steps["pack"]
        s["eager_step_pack_ms"] = 1e3 * self.runner.host_seconds["pack"] / max(1, self.runner.host_steps["pack"])
        return s
