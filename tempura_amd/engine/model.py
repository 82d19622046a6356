"""The decoder built from a ``ModelSpec``: embedding, blocks in their run order,
final norm and output head.

The forward pass follows the reference's order
(/root/reference/engine/src/model.rs:643-1399): gather embeddings, run each
layer on the float32 residual stream, normalise and project.  Unlike the
reference, which projects the last row only (model.rs:1389-1396), logits are
produced at every requested row of the batch.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional, Tuple

import torch

from ..config.spec import ModelSpec
from ..kernels import ops
from ..parts.base import CacheSpec, StateSpec, WeightInfo, build_part, part_class
from ..parts.inventory import expected_weights


class CausalLM:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {dtype}")
        self.spec = spec
        self.dtype = dtype
        self.device = device
        h = spec.hidden_size
        self.embedding = part_class("embedding", spec.embedding.kind)(spec.embedding, h, dtype, device, spec.vocab_size)
        self.layers = [part_class("block", ls.block)(ls, h, dtype, device) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, h, dtype, device)
        self.lm_head = part_class("lm_head", spec.lm_head.kind)(spec.lm_head, h, dtype, device, spec.vocab_size)
        self.order = spec.resolved_order()
        #: None, or a callable (i, h) called before run-order entry i and once after the last with the residual
        #: stream as it stands (eager passes only; see ``Engine.profile``)
        self.observer = None
        self._plan_caches()

    # ---- caches --------------------------------------------------------
    def _cache_owner(self, layer: int):
        """The part of a layer whose cache and state needs its calls have (a block says which; by default its mixer)."""
        block = self.layers[layer]
        return block.cache_owner() if hasattr(block, "cache_owner") else block.mixer

    def _plan_caches(self) -> None:
        """Group cache slots by what their mixers need."""
        n_slots = 1 + max((c.cache for c in self.order), default=-1)
        owner: List[Optional[int]] = [None] * n_slots     # order index of the call that writes the slot
        self.call_writes: List[bool] = []
        for i, call in enumerate(self.order):
            if owner[call.cache] is None:
                owner[call.cache] = i
                self.call_writes.append(True)
            else:
                self.call_writes.append(False)
        self.cache_groups: List[CacheSpec] = []
        self.slot_group: List[Tuple[int, int]] = []        # slot -> (group, index within group)
        self.state_specs: Dict[int, StateSpec] = {}
        counts: List[int] = []
        for slot in range(n_slots):
            mixer = self._cache_owner(self.order[owner[slot]].layer)
            cs = mixer.cache_spec()
            if cs is None:
                self.slot_group.append((-1, 0))
            else:
                if cs not in self.cache_groups:
                    self.cache_groups.append(cs)
                    counts.append(0)
                g = self.cache_groups.index(cs)
                self.slot_group.append((g, counts[g]))
                counts[g] += 1
            ss = mixer.state_spec()
            if ss is not None:
                self.state_specs[slot] = ss
        self.slots_per_group = counts
        for i, call in enumerate(self.order):
            if not self.call_writes[i]:
                mine = self._cache_owner(call.layer).cache_spec()
                theirs = self._cache_owner(self.order[owner[call.cache]].layer).cache_spec()
                if mine != theirs:
                    raise ValueError(f"run order entry {i} reads cache slot {call.cache} whose layout differs from its own")

    def portion_align(self) -> int:
        """The multiple of positions at which the model's parts prefer prompt portions to be cut (the least common
        multiple of what the mixers say; 1 when none cares)."""
        import math
        align = 1
        for layer in self.layers:
            for part in layer.parts():
                align = math.lcm(align, int(getattr(part, "preferred_portion_align", 1)))
        return align

    # ---- weights -------------------------------------------------------
    def expected_weights(self) -> Dict[str, WeightInfo]:
        return expected_weights(self.spec)

    def load_weights(self, get: Callable) -> None:
        self.embedding.load_weights(get)
        for layer in self.layers:
            layer.load_weights(get)
        self.final_norm.load_weights(get)
        self.lm_head.load_weights(get, self.embedding)

    def weight_bytes(self, include_embedding: bool = True) -> int:
        seen, total = set(), 0

        def add(t):
            nonlocal total
            if isinstance(t, ops.TiledWeight):
                t = t.data
            if isinstance(t, torch.Tensor) and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        objs = [self.final_norm, self.lm_head]
        if include_embedding:
            objs.append(self.embedding)
        for layer in self.layers:
            objs.extend(layer.parts())
        for o in objs:
            for v in vars(o).values():
                add(v)
        return total

    # ---- forward -------------------------------------------------------
    def forward(self, tokens: torch.Tensor, ctx, caches) -> torch.Tensor:
        """``tokens`` int32 [n]; ``caches[i]`` is the ``LayerCache`` of run-order entry i.
        Returns float32 logits [len(ctx.logit_rows), vocab]."""
        if hasattr(ctx, "shared"):
            ctx.shared.clear()      # what layers share is computed anew in every pass (also in one that is captured)
        h = self.embedding.forward(tokens)
        m = h.shape[0]
        x = None      # rows handed from one block to the next (a norm carried by the products around it)
        observe = self.observer
        for i, call in enumerate(self.order):
            if observe is not None:
                observe(i, h)
            layer = self.layers[call.layer]
            if not hasattr(layer, "entry_norm"):
                layer.forward(h, ctx, caches[i])
                x = None
                continue
            after = self.layers[self.order[i + 1].layer] if i + 1 < len(self.order) else None
            next_norm = after.entry_norm(m) if hasattr(after, "entry_norm") else None
            x = layer.forward(h, ctx, caches[i], x, next_norm)
        if observe is not None:
            observe(len(self.order), h)
        x = self.final_norm.forward(h, ctx.logit_rows)
        return self.lm_head.forward(x)
