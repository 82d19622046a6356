"""Device memory behind the cache manager: page pools and state slots.

One allocation per group, ``[slots, 2 (k, v), pages + 1, kv_heads, page_size *
head_dim]``: a physical page id addresses the same page for every cache slot of
the group, and within a page each kv head's rows lie together so that a head's
keys of one page are one contiguous run.  Keys are ``[page_size, head_dim]`` per
head and page; values are kept transposed, ``[head_dim, page_size]``, so that
the attention kernels fetch eight consecutive keys of one value element with one
16-byte load.  The extra last page is never handed
out; padded rows of a fixed-size decode batch write there.  State tensors are
``[max_requests + 1, *shape]`` per stateful cache slot, the extra row likewise.
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
    k: Optional[torch.Tensor]        # [pages + 1, kv_heads, page_size, head_dim]
    v: Optional[torch.Tensor]        # [pages + 1, kv_heads, head_dim, page_size]
    writes: bool                     # False: this call only reads a slot another call writes
    page_size: int
    state: Optional[torch.Tensor]    # [max_requests + 1, *shape] or None


class CachePools:
    def __init__(self, groups: Sequence[CacheSpec], slots_per_group: Sequence[int], page_size: int,
                 num_pages: Sequence[int], dtype: torch.dtype, device,
                 state_specs: Dict[int, StateSpec], max_requests: int):
        self.page_size = page_size
        self.num_pages = list(num_pages)
        self.kv: List[torch.Tensor] = []
        for spec, n_slots, pages in zip(groups, slots_per_group, num_pages):
            self.kv.append(torch.zeros((n_slots, 2, pages + 1, spec.num_kv_heads, page_size, spec.head_dim),
                                       dtype=dtype, device=device))
        self.state: Dict[int, torch.Tensor] = {
            slot: torch.zeros((max_requests + 1, *s.shape), dtype=s.dtype, device=device)
            for slot, s in state_specs.items()
        }

    def scratch_page(self, g: int) -> int:
        return self.num_pages[g]

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.kv) + \
            sum(t.numel() * t.element_size() for t in self.state.values())
