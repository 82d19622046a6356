"""Interfaces of the parts a layer is put together from, and their registry.

Five categories: ``mixer`` (attention here), ``ffn``, ``norm``, ``position`` and
``block`` (the arrangement of the other four), plus ``embedding`` and
``lm_head`` at the ends of the model.  A part is built from a ``PartSpec`` and
knows only its own sizes, constants and tensor names; it never sees the
architecture's config and never knows which model it is in.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

from ..config.spec import PartSpec


@dataclass(frozen=True)
class WeightInfo:
    """A tensor a part reads: its shape and how random-weight mode fills it."""

    shape: Tuple[int, ...]
    init: str = "normal"          # "normal" (N(0, std)) or "ones"
    optional: bool = False        # True: absence is legal (tied output head)
    kind: str = "float"           # "float": a weight (stored F32, BF16 or F16); "int": an integer table (kept as int32)


@dataclass(frozen=True)
class CacheSpec:
    """What a mixer needs of the paged cache.

    ``kind`` names the rule by which pages may be given back: ``"full"`` (every key is kept), ``"window"`` (only
    the last ``window`` keys are ever read), or any rule registered in cache/rules.py.
    Mixers whose specs are equal share one group of pages.

    The spec also says what a page HOLDS, so that the pools, the runner and the engine's sizing need not know:
    ``planes(page_size)`` names the tensors a cache slot consists of and the shape of one page of each.  The
    default is what grouped-query attention keeps: keys ``[kv_heads, page_size, head_dim]`` and values
    transposed, ``[kv_heads, head_dim, page_size]`` (the attention kernels fetch eight consecutive keys of one
    value element with one 16-byte load).  A mixer that keeps something else per token (one compressed vector,
    say) subclasses the spec and overrides ``planes``; its ``forward`` finds the tensors under the same names
    in ``LayerCache.planes``, each ``[pages + 1, *shape]`` with the page index first.
    """

    kind: str
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def planes(self, page_size: int) -> Dict[str, Tuple[int, ...]]:
        """name -> shape of one page of that tensor (in elements of the cache dtype)."""
        return {"k": (self.num_kv_heads, page_size, self.head_dim), "v": (self.num_kv_heads, self.head_dim, page_size)}

    def page_bytes(self, page_size: int, element_size: int) -> int:
        """Bytes of one page of one cache slot: what a token place costs, times ``page_size``."""
        total = 0
        for shape in self.planes(page_size).values():
            n = 1
            for d in shape:
                n *= int(d)
            total += n
        return total * element_size


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size (for instance a recurrent mixer's)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    """Base of every part.  ``spec`` carries sizes, constants and tensor names."""

    category = ""
    #: True when ``forward`` only launches kernels that read the step's data from device memory
    #: (no host-side values of the batch, no host loops): decode steps may then replay a captured graph.
    graph_safe = False

    def __init__(self, spec: PartSpec, hidden_size: int, dtype: torch.dtype, device):
        self.spec = spec
        self.hidden_size = hidden_size
        self.dtype = dtype            # compute dtype: torch.bfloat16 or torch.float32
        self.device = device

    @classmethod
    def expected_weights(cls, spec: PartSpec, hidden_size: int) -> Dict[str, WeightInfo]:
        """Checkpoint tensor name -> shape/init, for the loader and for random weights."""
        return {}

    def load_weights(self, get: Callable[[str], torch.Tensor]) -> None:
        """Fetch tensors by checkpoint name (``get`` returns them on the host as stored)."""

    def _to_device(self, t: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return t.to(device=self.device, dtype=dtype or self.dtype).contiguous()


class Mixer(Part):
    """Mixes information across positions of one request.

    ``forward(x, ctx, cache, residual)`` gets the normed activations ``x``
    [tokens, hidden] of the whole batch, the step's ``StepContext`` and the
    ``LayerCache`` of this call, and must ADD its output into ``residual``
    (float32 [tokens, hidden]) in place.
    """

    category = "mixer"

    #: a portion of a prompt is best cut at a multiple of this many positions (1: anywhere).  A hint for whoever
    #: cuts prompts, never a condition: every part takes every cut.
    preferred_portion_align = 1

    def cache_spec(self) -> Optional[CacheSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, x, ctx, cache, residual) -> None:
        raise NotImplementedError


class FeedForward(Part):
    """Position-wise transform.  ``forward(x, ctx, residual)`` adds into ``residual``."""

    category = "ffn"

    def forward(self, x, ctx, residual) -> None:
        raise NotImplementedError


class Norm(Part):
    """``forward(h, rows=None)`` returns the normed rows of the float32 stream ``h``
    in the compute dtype; ``rows`` (int32 indices) selects a subset."""

    category = "norm"

    def forward(self, h, rows=None):
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions enter a mixer.

    A rotary encoding returns its frequency table from ``rotary()`` and the mixer
    fuses the rotation into its key/value store kernel.  Any other encoding
    returns None there and implements ``apply(q, k, positions)``, which the mixer
    calls on the projected queries and keys before they are stored.
    """

    category = "position"

    def rotary(self):
        """(inv_freq float64 [rotary_dim/2] on device, rotary_dim, magnitude factor) or None."""
        return None

    def apply(self, q, k, positions):
        return q, k


class Block(Part):
    """Arranges a mixer, a feed-forward and their norms around the residual stream."""

    category = "block"

    def forward(self, h, ctx, cache) -> None:
        raise NotImplementedError


_REGISTRY: Dict[Tuple[str, str], Any] = {}


def register_part(category: str, kind: str, cls) -> None:
    """Make ``cls`` buildable from ``PartSpec(kind=...)`` in ``category``
    (``"mixer"``, ``"ffn"``, ``"norm"``, ``"position"``, ``"block"``, ``"embedding"``, ``"lm_head"``)."""
    _REGISTRY[(category, kind)] = cls


def part_class(category: str, kind: str):
    try:
        return _REGISTRY[(category, kind)]
    except KeyError:
        known = sorted(k for c, k in _REGISTRY if c == category)
        raise KeyError(f"no {category} part of kind {kind!r} is registered (known: {known})") from None


def build_part(category: str, spec: PartSpec, hidden_size: int, dtype, device):
    return part_class(category, spec.kind)(spec, hidden_size, dtype, device)
