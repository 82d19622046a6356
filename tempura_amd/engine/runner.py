"""The step function: one batch of (request, its next tokens) through the model.

A batch may hold portions of prompts beside single decoded tokens, cut anywhere.
Only the tokens given are run; everything earlier comes from the cache pages that
earlier steps wrote.  The reference has three disjoint calls instead (one
sequence of n tokens, or m sequences of exactly one token,
/root/reference/engine/src/model.rs:305-448) and never mixes them in a forward
(/root/reference/server/src/engine_task.rs:748-778).
"""
from __future__ import annotations

import itertools
import re
import time
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheManager, CachePools, LayerCache, PagesExhausted
from ..kernels import ops
from .model import CausalLM


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the places (indices into
    ``tokens``) whose logits are wanted."""

    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


class StepContext:
    """Everything a part may read about the batch.  Device tensors are int32.

    positions[n]      absolute position of each token in its request
    token_req[n]      index (row of this batch) of the request each token belongs to
    cu_seqlens[r+1]   where each request's tokens start in the flattened batch
    context_lens[r]   tokens of the request in the cache once this step is written
    block_tables[g]   [r, width] logical page -> physical page, per cache group
    slot_mapping[g]   [n] physical cache row (page * page_size + offset) of each new token
    state_slots[r]    row of the per-request state tensors
    logit_rows[m]     flattened token indices whose logits are returned
    Host copies (``q_starts``, ``q_lens``, ``ctx_lens``, ``state_slot_list``) serve parts
    that loop over requests on the host.
    ``shared``: what the parts of several layers compute once per step and keep under a key of
    their own (a rotation table, for instance); empty when the step begins.
    """

    def __init__(self):
        self.num_tokens = 0
        self.num_requests = 0
        self.positions = None
        self.token_req = None
        self.cu_seqlens = None
        self.context_lens = None
        self.block_tables: List[torch.Tensor] = []
        self.slot_mapping: List[torch.Tensor] = []
        self.state_slots = None
        self.logit_rows = None
        self.max_q_len = 0
        self.max_context_len = 0
        self.num_single = 0          # requests that bring exactly one token
        self.page_size = 0
        self.q_starts: List[int] = []
        self.q_lens: List[int] = []
        self.ctx_lens: List[int] = []
        self.state_slot_list: List[int] = []
        self.shared: dict = {}


class _DecodeGraph:
    """A captured decode step for a fixed number of rows and a bound on the context length.

    Every per-step value lives in ``packed`` (one int32 device buffer refreshed by one copy
    from pinned host memory); the kernels read lengths, tables and slots from there, so a
    replay runs the new step without any host-side launch work.  The reference's batch
    graphs are keyed by batch size with all per-step values device-read in the same way
    (/root/reference/engine/src/cutile_gpu_forward.rs:939-953)."""

    def __init__(self, runner: "ModelRunner", rows: int, ctx_bound: int):
        self.rows = rows
        self.ctx_bound = ctx_bound
        self.width = (ctx_bound + runner.page_size - 1) // runner.page_size
        n_groups = len(runner.cache.groups)
        # layout: tokens, positions, context_lens, state_slots | per group: table, slots
        self.sizes = [rows, rows, rows, rows] + [rows * self.width] * n_groups + [rows] * n_groups
        self.offs = np.cumsum([0] + self.sizes)
        total = int(self.offs[-1])
        # two pinned buffers taken in turn (the next step may be staged while the last copy is still queued),
        # and a small one for the tokens alone
        self.hosts = [torch.empty(total, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self.host_nps = [h.numpy() for h in self.hosts]
        self.copied = [torch.cuda.Event() for _ in range(2)]
        self.turn = 0
        self.tok_host = torch.empty(rows, dtype=torch.int32, pin_memory=True)
        self.tok_np = self.tok_host.numpy()
        self.tok_copied = torch.cuda.Event()
        self.packed = torch.zeros(total, dtype=torch.int32, device=runner.device)
        self.fixed = torch.arange(rows + 1, dtype=torch.int32, device=runner.device)
        self.graph = None
        self.logits = None

    def view(self, i: int) -> torch.Tensor:
        return self.packed[int(self.offs[i]): int(self.offs[i + 1])]

    def context(self, runner: "ModelRunner") -> "StepContext":
        n_groups = len(runner.cache.groups)
        ctx = StepContext()
        ctx.num_tokens = ctx.num_requests = self.rows
        ctx.positions = self.view(1)
        ctx.context_lens = self.view(2)
        ctx.state_slots = self.view(3)
        ctx.token_req = self.fixed[: self.rows]
        ctx.cu_seqlens = self.fixed
        ctx.logit_rows = None                     # every row
        ctx.block_tables = [self.view(4 + g).view(self.rows, self.width) for g in range(n_groups)]
        ctx.slot_mapping = [self.view(4 + n_groups + g) for g in range(n_groups)]
        ctx.max_q_len = 1
        ctx.num_single = self.rows
        ctx.max_context_len = self.width * runner.page_size
        ctx.page_size = runner.page_size
        return ctx


class _PackedStaging:
    """Host buffers for the packed inputs of eager steps on their way to the device.  On a GPU they are pinned
    and taken in turn from a small ring, so that the copy is queued behind the work in flight instead of making
    the host wait for it (a copy from pageable memory would); a buffer is used again once its copy has run."""
    RING = 4

    def __init__(self, device):
        self.device = device
        self.cuda = torch.device(device).type == "cuda"
        self.slots = [None] * self.RING          # (tensor, numpy view, event)
        self.turn = 0

    def take(self, need: int) -> np.ndarray:
        """A host buffer of at least ``need`` int32 (the next of the ring), free to be written.  The ring moves
        on when the buffer is sent; a buffer that is taken and not sent is simply taken again."""
        slot = self.slots[self.turn]
        if slot is None or slot[0].numel() < need:
            size = max(4096, 1 << int(need - 1).bit_length())
            t = torch.empty(size, dtype=torch.int32, pin_memory=self.cuda)
            slot = (t, t.numpy(), torch.cuda.Event() if self.cuda else None)
            self.slots[self.turn] = slot
        elif slot[2] is not None:
            slot[2].synchronize()                # the copy that last used this buffer has run
        return slot[1]

    def send(self, total: int) -> torch.Tensor:
        """The first ``total`` ints of the buffer taken last, as a device tensor."""
        t, arr, event = self.slots[self.turn]
        self.turn = (self.turn + 1) % self.RING
        if not self.cuda:
            return t[:total].clone()
        dev = torch.empty(total, dtype=torch.int32, device=self.device)
        dev.copy_(t[:total], non_blocking=True)
        event.record()
        return dev


class ModelRunner:
    def __init__(self, model: CausalLM, page_size: int, num_pages, max_requests: int,
                 cache_dtype: Optional[torch.dtype] = None, use_graph: bool = False):
        self.model = model
        self.device = model.device
        self.page_size = int(page_size)
        n_groups = len(model.cache_groups)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * n_groups
        self.cache = CacheManager(model.cache_groups, self.page_size, list(num_pages), max_requests)
        self.pools = CachePools(model.cache_groups, model.slots_per_group, self.page_size, list(num_pages),
                                cache_dtype or model.dtype, self.device, model.state_specs, max_requests)
        self.layer_caches: List[LayerCache] = []
        for i, call in enumerate(model.order):
            g, idx = model.slot_group[call.cache]
            planes = self.pools.slot(g, idx) if g >= 0 else {}
            self.layer_caches.append(LayerCache(g, planes, model.call_writes[i], self.page_size,
                                                self.pools.state.get(call.cache)))
        self.steps_run = 0
        self.tokens_run = 0
        self._staging = _PackedStaging(self.device)
        #: host time spent packing the inputs of eager steps, and how many such steps there were
        self.host_seconds = {"pack": 0.0}
        self.host_steps = {"pack": 0}
        # Decode-only steps replay a captured graph when every part of the model allows it (a part that keeps
        # per-request state says so like any other: it then finds its rows through ``ctx.state_slots`` on the device).
        self.use_graph = bool(use_graph) and self.device.type == "cuda" and \
            all(getattr(p, "graph_safe", False) for layer in model.layers for p in layer.parts())
        self.graph_steps = 0
        self._prepared = None          # (request ids, graph, cache generation) of a decode step staged ahead by prepare_decode
        self.staged_steps = 0          # decode steps that found their inputs staged
        self._graphs: Dict[tuple, _DecodeGraph] = {}
        self._graph_pool = None

    # ---- request lifetime ---------------------------------------------
    def has_request(self, rid) -> bool:
        return self.cache.has(rid)

    def add_request(self, rid) -> None:
        self._prepared = None
        self.cache.add(rid)

    def end_request(self, rid) -> None:
        self._prepared = None
        self.cache.release(rid)

    def num_cached(self, rid) -> int:
        return self.cache.num_tokens(rid)

    # ---- the step ------------------------------------------------------
    def _check_entries(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen = set()
        vocab = self.model.spec.vocab_size
        for e in entries:
            if e.rid in seen:
                raise ValueError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.rid!r}: a step entry needs at least one token")
            for t in e.tokens:
                if t < 0 or t >= vocab:
                    raise ValueError(f"request {e.rid!r}: token id {t} outside the vocabulary of {vocab}")
            for w in e.want:
                if w < 0 or w >= len(e.tokens):
                    raise ValueError(f"request {e.rid!r}: wanted place {w} outside its {len(e.tokens)} tokens")
            if not self.cache.has(e.rid):
                raise ValueError(f"request {e.rid!r} is not live; add_request first")
            end = self.cache.num_tokens(e.rid) + len(e.tokens)
            if end > self.model.spec.max_positions:
                raise ValueError(f"request {e.rid!r}: {end} tokens exceed max positions {self.model.spec.max_positions}")

    def reserve(self, entries: Sequence[StepEntry]) -> None:
        """Pages for every entry, or ``PagesExhausted`` with nothing changed."""
        self.cache.reserve_many([e.rid for e in entries], [len(e.tokens) for e in entries])

    def _pack_step(self, entries: Sequence[StepEntry]):
        """Host side of a step, one call into the host library: the step is checked, its pages are reserved (all or
        nothing, ``PagesExhausted``) and its device inputs are packed into one pinned buffer that goes to the
        device in one copy.  Returns (tokens on the device, context).  A refused step changes nothing."""
        t_start = time.perf_counter()
        R = len(entries)
        cache = self.cache
        try:
            slots = [cache._slot_of[e.rid] for e in entries]
        except KeyError:
            bad = next(e.rid for e in entries if not cache.has(e.rid))
            raise ValueError(f"request {bad!r} is not live; add_request first") from None
        try:
            n_new = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=R)
            pieces = [np.asarray(e.tokens, dtype=np.int32) for e in entries]
            tokens = pieces[0].reshape(-1) if R == 1 else np.concatenate(pieces, axis=None)
            n_want = np.fromiter((len(e.want) for e in entries), dtype=np.int32, count=R)
            want = np.fromiter(itertools.chain.from_iterable(e.want for e in entries), dtype=np.int32, count=int(n_want.sum()))
        except OverflowError:
            raise ValueError(f"a token id or wanted place outside the vocabulary of {self.model.spec.vocab_size}") from None
        tokens = np.ascontiguousarray(tokens)
        scratch = [self.pools.scratch_page(g) for g in range(len(cache.groups))]
        spec = self.model.spec
        guess = 4 * int(tokens.size) + 4 * R + int(want.size) + len(cache.groups) * (int(tokens.size) + R * 64) + 64
        while True:
            host = self._staging.take(guess)
            try:
                meta = cache.fill_step(slots, n_new, tokens, n_want, want, spec.vocab_size, spec.max_positions, scratch, host)
            except ValueError as e:
                msg = str(e)
                m = re.match(r"entry (\d+): (.*)", msg)
                if m:
                    msg = f"request {entries[int(m.group(1))].rid!r}: {m.group(2)}"
                raise ValueError(msg) from None
            if meta is not None:
                break
            guess = cache.last_fill_need
        N, M, total, max_q, max_ctx, singles = meta[:6]
        widths = meta[6: 6 + len(cache.groups)]
        n_groups = len(cache.groups)
        # what parts that loop over requests on the host may read (the pinned buffer is used again later)
        o = 3 * N
        cu = host[o: o + R + 1].copy()
        ctx_lens = host[o + R + 1: o + 2 * R + 1].copy()
        packed = self._staging.send(total)
        ctx = StepContext()
        ctx.num_tokens, ctx.num_requests = N, R
        tok_dev = packed[:N]
        ctx.positions = packed[N: 2 * N]
        ctx.token_req = packed[2 * N: 3 * N]
        ctx.cu_seqlens = packed[o: o + R + 1]
        ctx.context_lens = packed[o + R + 1: o + 2 * R + 1]
        ctx.state_slots = packed[o + 2 * R + 1: o + 3 * R + 1]
        o += 3 * R + 1
        ctx.logit_rows = packed[o: o + M]
        o += M
        ctx.block_tables = []
        for g in range(n_groups):
            ctx.block_tables.append(packed[o: o + R * widths[g]].view(R, widths[g]))
            o += R * widths[g]
        ctx.slot_mapping = [packed[o + g * N: o + (g + 1) * N] for g in range(n_groups)]
        ctx.max_q_len = max_q
        ctx.num_single = singles
        ctx.max_context_len = max_ctx
        ctx.page_size = self.page_size
        ctx.q_starts = cu[:-1].tolist()
        ctx.q_lens = n_new.tolist()
        ctx.ctx_lens = ctx_lens.tolist()
        ctx.state_slot_list = slots
        self.host_seconds["pack"] += time.perf_counter() - t_start
        self.host_steps["pack"] += 1
        return tok_dev, ctx

    # ---- decode steps as a graph -----------------------------------------
    def _graph_for(self, rows: int, ctx_len: int) -> Optional[_DecodeGraph]:
        # rows padded to a power of two, beyond 128 to a multiple of 128: the products see as many blocks of rows as
        # in the unpadded step and so choose the same tiles and parts of K (the same bits as an eager step)
        bucket = ops.decode_rows_padded(rows)
        bound = 256
        while bound < ctx_len:
            bound *= 2
        bound = min(bound, (self.model.spec.max_positions + self.page_size - 1) // self.page_size * self.page_size)
        key = (bucket, bound)
        g = self._graphs.get(key)
        if g is None:
            g = _DecodeGraph(self, bucket, bound)
            self._graphs[key] = g
        return g

    def _fill_graph_inputs(self, g: _DecodeGraph, rids: Sequence, tokens: Sequence[int]) -> None:
        i = g.turn
        g.turn ^= 1
        g.copied[i].synchronize()                  # the last copy out of this pinned buffer has finished
        self.cache.fill_decode(rids, tokens, g.rows, g.width,
                               [self.pools.scratch_page(gi) for gi in range(len(self.cache.groups))], g.host_nps[i])
        g.packed.copy_(g.hosts[i], non_blocking=True)
        g.copied[i].record()

    def prepare_decode(self, rids: Sequence) -> bool:
        """A hint that changes no result: the next step will most likely bring one token for each of these
        requests, in this order.  Pages are reserved and everything of that step but its tokens (positions,
        lengths, tables, cache rows) is staged and sent now, while the GPU is still busy with the step before;
        when the step comes and is what was announced, only its tokens follow.  Anything else in between
        (another step, a request added or ended) drops the staging.  False when nothing was staged."""
        self._prepared = None
        rids = list(rids)
        if not self.use_graph or not rids or len(set(rids)) != len(rids) or not all(self.cache.has(r) for r in rids):
            return False
        ctx_len = self.cache.max_num_tokens(rids) + 1
        if ctx_len > self.model.spec.max_positions:
            return False
        try:
            self.cache.reserve_many(rids, [1] * len(rids))
        except PagesExhausted:
            return False
        g = self._graph_for(len(rids), ctx_len)
        if g.graph is None:
            return False
        self._fill_graph_inputs(g, rids, [0] * len(rids))
        self._prepared = (tuple(rids), g, self.cache.generation)
        return True

    def _graph_step(self, rids: Sequence, tokens, want_rows: Optional[Sequence[int]] = None) -> torch.Tensor:
        """``tokens``: a list of ints, or an int32 device tensor [len(rids)] (tokens the host has not seen yet)."""
        on_device = torch.is_tensor(tokens)
        n = len(rids)
        prepared, self._prepared = self._prepared, None
        # (staged values are good only while nothing was added, ended, committed or truncated since: the scheduler
        # changes the cache manager directly, and a request that was preempted and readmitted, or a request
        # name used again, would otherwise find another request's positions and pages)
        if prepared is not None and prepared[0] == tuple(rids) and prepared[2] == self.cache.generation:
            g = prepared[1]                         # staged already: only the tokens are new
            self.staged_steps += 1
            if not on_device:
                g.tok_copied.synchronize()
                g.tok_np[:n] = tokens
                g.packed[:n].copy_(g.tok_host[:n], non_blocking=True)
                g.tok_copied.record()
        else:
            ctx_len = self.cache.max_num_tokens(rids) + 1
            g = self._graph_for(n, ctx_len)
            self._fill_graph_inputs(g, rids, [0] * n if on_device else tokens)
        if on_device:
            g.packed[:n].copy_(tokens)
        if self.pools.state:
            self._clear_state([self.cache.state_slot(r) for r in rids if self.cache.num_tokens(r) == 0])
        if g.graph is None:
            ctx = g.context(self)
            tok = g.view(0)
            # one eager run first: lazy initialisation must not happen under capture.  (What it writes into the
            # paged cache the replay writes again; per-request state it would advance twice, so that is put back.)
            kept = {slot: t.clone() for slot, t in self.pools.state.items()}
            self.model.forward(tok, ctx, self.layer_caches)
            for slot, t in kept.items():
                self.pools.state[slot].copy_(t)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                g.logits = self.model.forward(tok, ctx, self.layer_caches)
            if self._graph_pool is None:
                self._graph_pool = graph.pool()
            g.graph = graph
        g.graph.replay()
        self.graph_steps += 1
        if want_rows is None or len(want_rows) == n:
            return g.logits[:n]
        return ops.take_rows(g.logits, want_rows) if want_rows else g.logits[:0]

    def _clear_state(self, fresh: Sequence[int]) -> None:
        """A request that starts at position 0 gets a cleared state (also after a recompute)."""
        if fresh:
            for t in self.pools.state.values():
                ops.zero_rows(t, fresh)

    def step_chained(self, rids: Sequence, tokens: torch.Tensor) -> torch.Tensor:
        """A step of one token per request whose tokens are still on the device: ``tokens`` int32 [len(rids)],
        for instance what the sampling kernel chose after the step before, which the host has not read yet.
        The step is queued behind that kernel at once, so the GPU goes from one step to the next without
        waiting for the host.  The tokens must be valid ids (they are not checked here); every request must be
        live; needs the graph path.  Returns the logits of every row (a view of the graph's output buffer)."""
        rids = list(rids)
        if not self.use_graph:
            raise ValueError("step_chained needs use_graph")
        if not rids or len(set(rids)) != len(rids):
            raise ValueError("step_chained: one entry per request, at least one")
        if not (torch.is_tensor(tokens) and tokens.dtype == torch.int32 and tokens.dim() == 1 and tokens.numel() == len(rids)
                and tokens.device.type == torch.device(self.device).type):
            raise ValueError("step_chained: tokens must be an int32 device tensor with one id per request")
        for rid in rids:
            if not self.cache.has(rid):
                raise ValueError(f"request {rid!r} is not live; add_request first")
            if self.cache.num_tokens(rid) + 1 > self.model.spec.max_positions:
                raise ValueError(f"request {rid!r}: one more token exceeds max positions {self.model.spec.max_positions}")
        self.cache.reserve_many(rids, [1] * len(rids))
        logits = self._graph_step(rids, tokens)
        self.cache.commit_many(rids, [1] * len(rids))
        self.steps_run += 1
        self.tokens_run += len(rids)
        return logits

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run the batch; returns float32 logits [sum of wanted places, vocab] on the device,
        ordered by entry and then by ``want``.  After a decode-only step the result is a view of
        the graph's output buffer: use it before the next step."""
        entries = list(entries)
        if not entries:
            raise ValueError("a step needs at least one entry")
        if self.use_graph and all(len(e.tokens) == 1 for e in entries):
            self._check_entries(entries)
            self.reserve(entries)
            logits = self._graph_step([e.rid for e in entries], [e.tokens[0] for e in entries],
                                      [r for r, e in enumerate(entries) if len(e.want) > 0])
            self.cache.commit_many([e.rid for e in entries], [1] * len(entries))
            self.steps_run += 1
            self.tokens_run += len(entries)
            return logits
        self._prepared = None
        tok_dev, ctx = self._pack_step(entries)
        if self.pools.state:
            self._clear_state([s for s, n, c in zip(ctx.state_slot_list, ctx.q_lens, ctx.ctx_lens) if c == n])
        logits = self.model.forward(tok_dev, ctx, self.layer_caches)
        self.cache.commit_many([e.rid for e in entries], ctx.q_lens)
        self.steps_run += 1
        self.tokens_run += ctx.num_tokens
        return logits
