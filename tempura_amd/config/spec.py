"""Architecture-neutral description of a decoder: what the engine builds from.

An architecture's typed configuration (for instance ``LlamaConfig``) is turned
into a ``ModelSpec``.  Everything below the configuration layer (parts, cache
manager, step function, weight loader) reads only the spec, never the
architecture's own config, so that another architecture is added by writing a
config class and a function that produces a spec.

A ``PartSpec`` names a registered part kind (``"attention"``, ``"swiglu"``,
``"rmsnorm"``, ``"rope"``, ...) and carries every size and constant that part
needs, plus the tensor names it reads its weights from.  Parts are chosen layer
by layer; the order in which layers run is a list of ``LayerCall`` entries that
may name a layer twice or let a call read the cache another call writes.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: a registered kind plus its parameters.

    ``params`` holds sizes and constants; ``weights`` maps the part's own role
    names (``"q"``, ``"gate"``, ``"weight"``) to tensor names in the checkpoint.
    """

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    weights: Dict[str, str] = field(default_factory=dict)

    def __hash__(self):  # dict fields: hash by identity of content
        return hash((self.kind, repr(sorted(self.params.items())), repr(sorted(self.weights.items()))))


@dataclass(frozen=True)
class LayerSpec:
    """A block: a registered arrangement and the parts it arranges, by the names the arrangement gives them.

    ``block`` names the arrangement (``"prenorm"``: x + mixer(norm(x)), then x + ffn(norm(x)), whose parts are
    ``mixer_norm``, ``mixer``, ``ffn_norm`` and ``ffn``).  Which names an arrangement reads, and which category of
    part (mixer, ffn, norm) each is, is the arrangement's business: one with other norms, or without a
    feed-forward, has other names and needs no change here.  ``spec.mixer`` reads ``spec.parts["mixer"]``.
    """

    block: str
    parts: Dict[str, PartSpec] = field(default_factory=dict)

    def __getattr__(self, name: str) -> PartSpec:
        parts = object.__getattribute__(self, "parts")
        try:
            return parts[name]
        except KeyError:
            raise AttributeError(f"block {self.block!r} has no part named {name!r} (it has {sorted(parts)})") from None

    def __hash__(self):
        return hash((self.block, tuple(sorted((k, hash(v)) for k, v in self.parts.items()))))


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer`` indexes ``ModelSpec.layers``.  ``cache`` names the cache slot the
    call uses; the first call that names a slot writes it, later calls naming the
    same slot only read it (they compute no keys or values of their own).  When
    ``cache`` is None the call owns a slot of its own.
    """

    layer: int
    cache: Optional[int] = None


@dataclass
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    layers: List[LayerSpec]
    order: List[LayerCall]
    final_norm: PartSpec
    embedding: PartSpec
    lm_head: PartSpec
    eos_token_ids: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None

    def resolved_order(self) -> List[LayerCall]:
        """The run order with every call's cache slot made explicit.

        Calls with ``cache=None`` get fresh slot numbers above every explicitly
        named one.  Returns calls whose ``cache`` is a dense slot index.
        """
        named = sorted({c.cache for c in self.order if c.cache is not None})
        dense = {n: i for i, n in enumerate(named)}
        nxt = len(named)
        out = []
        for c in self.order:
            if c.layer < 0 or c.layer >= len(self.layers):
                raise ValueError(f"run order names layer {c.layer}, model has {len(self.layers)}")
            if c.cache is None:
                out.append(LayerCall(c.layer, nxt))
                nxt += 1
            else:
                out.append(LayerCall(c.layer, dense[c.cache]))
        return out
