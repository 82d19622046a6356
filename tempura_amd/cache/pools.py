"""Device memory behind the cache manager: page pools and state slots.

What a page holds is the cache spec's business (``CacheSpec.planes``): a group has one allocation per plane,
``[slots, pages + 1, *plane shape]``, so that a physical page id addresses the same page of every plane for
every cache slot of the group and the pages of one plane of one slot lie one after the other.  For attention
that is keys ``[kv_heads, page_size, head_dim]`` per page (a head's keys of one page are one contiguous run)
and values transposed, ``[kv_heads, head_dim, page_size]``.  The extra last page is never handed out; padded
rows of a fixed-size decode batch write there.  State tensors are ``[max_requests + 1, *shape]`` per stateful
cache slot, the extra row likewise.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from ..parts.base import CacheSpec, StateSpec


@dataclass
class LayerCache:
    """What one entry of the run order sees of the caches."""

    group: int                       # index of the cache group (-1: the mixer has no paged cache)
    planes: Dict[str, torch.Tensor]  # the slot's tensors by the names of ``CacheSpec.planes``, each [pages + 1, *shape]
    writes: bool                     # False: this call only reads a slot another call writes
    page_size: int
    state: Optional[torch.Tensor]    # [max_requests + 1, *shape] or None

    @property
    def k(self) -> Optional[torch.Tensor]:
        """attention's keys, [pages + 1, kv_heads, page_size, head_dim]"""
        return self.planes.get("k")

    @property
    def v(self) -> Optional[torch.Tensor]:
        """attention's values, [pages + 1, kv_heads, head_dim, page_size]"""
        return self.planes.get("v")


class CachePools:
    def __init__(self, groups: Sequence[CacheSpec], slots_per_group: Sequence[int], page_size: int,
                 num_pages: Sequence[int], dtype: torch.dtype, device,
                 state_specs: Dict[int, StateSpec], max_requests: int):
        self.page_size = page_size
        self.num_pages = list(num_pages)
        #: per group: plane name -> [slots, pages + 1, *plane shape]
        self.kv: List[Dict[str, torch.Tensor]] = []
        for spec, n_slots, pages in zip(groups, slots_per_group, num_pages):
            self.kv.append({name: torch.zeros((n_slots, pages + 1, *shape), dtype=dtype, device=device)
                            for name, shape in spec.planes(page_size).items()})
        self.state: Dict[int, torch.Tensor] = {
            slot: torch.zeros((max_requests + 1, *s.shape), dtype=s.dtype, device=device)
            for slot, s in state_specs.items()
        }

    def scratch_page(self, g: int) -> int:
        return self.num_pages[g]

    def slot(self, g: int, idx: int) -> Dict[str, torch.Tensor]:
        """The tensors of cache slot ``idx`` of group ``g``, each [pages + 1, *plane shape]."""
        return {name: t[idx] for name, t in self.kv[g].items()}

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for planes in self.kv for t in planes.values()) + \
            sum(t.numel() * t.element_size() for t in self.state.values())
