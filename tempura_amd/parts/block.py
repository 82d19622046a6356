"""Block arrangements.

``prenorm``: ``h += mixer(norm(h)); h += ffn(norm(h))`` — sequential, two
residual adds (/root/reference/engine/src/model.rs:952-1314; declared as
[PreNormAttention, PreNormFfn], /root/reference/engine/src/architecture.rs:56-65).
The residual stream ``h`` is float32 in every dtype.

A norm may be carried by the two products around it instead of running as a kernel of its own
(``Norm.deferred``, ``ops.Prenormed``): the part before it prepares the rows in the epilogue of its last
product, the part after it finishes them in its first.  The block arranges that for parts that declare
``split_norm``; any other part gets plain normed rows and returns nothing.
"""
from __future__ import annotations

from .base import build_part, part_class, register_part


class ArrangedBlock:
    """Base of the arrangements: builds the parts a ``LayerSpec`` names, by the categories the arrangement
    declares in ``ROLES`` (name -> ``"mixer"``, ``"ffn"`` or ``"norm"``), in that order, each as an attribute of
    its name.  A subclass writes ``forward(h, ctx, cache)`` and registers itself under ``"block"``; the model
    asks ``cache_owner()`` which part's cache and state needs a call of the layer has."""

    category = "block"
    ROLES: dict = {}

    def __init__(self, layer_spec, hidden_size, dtype, device):
        self.layer_spec = layer_spec
        missing = [name for name in self.ROLES if name not in layer_spec.parts]
        extra = [name for name in layer_spec.parts if name not in self.ROLES]
        if missing or extra:
            raise ValueError(f"block {layer_spec.block!r} arranges the parts {sorted(self.ROLES)}: "
                             f"missing {missing}, not its own {extra}")
        for name, cat in self.ROLES.items():
            setattr(self, name, build_part(cat, layer_spec.parts[name], hidden_size, dtype, device))

    def parts(self):
        return [getattr(self, name) for name in self.ROLES]

    def cache_owner(self):
        """The part whose ``cache_spec()`` / ``state_spec()`` this layer's cache slot serves."""
        return self.mixer

    @classmethod
    def expected_weights(cls, layer_spec, hidden_size):
        out = {}
        for name, cat in cls.ROLES.items():
            ps = layer_spec.parts[name]
            out.update(part_class(cat, ps.kind).expected_weights(ps, hidden_size))
        return out

    def load_weights(self, get):
        for p in self.parts():
            p.load_weights(get)


class PreNormBlock(ArrangedBlock):
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "ffn"}

    def entry_norm(self, m):
        """What the part before this block needs to prepare this block's first norm for ``m`` rows, or None."""
        if getattr(self.mixer, "split_norm", False) and hasattr(self.mixer_norm, "deferred"):
            return self.mixer_norm.deferred(m)
        return None

    def forward(self, h, ctx, cache, x=None, next_norm=None):
        """``x``: rows handed over by the block before (its last product prepared ``mixer_norm``);
        ``next_norm``: the ``entry_norm`` of the block after.  Returns the rows handed to that block, or None."""
        if x is None:
            x = self.mixer_norm.forward(h)
        x2 = None
        if getattr(self.mixer, "split_norm", False):
            mid = None
            if getattr(self.ffn, "split_norm", False) and hasattr(self.ffn_norm, "deferred"):
                mid = self.ffn_norm.deferred(h.shape[0])
            x2 = self.mixer.forward(x, ctx, cache, h, next_norm=mid)
        else:
            self.mixer.forward(x, ctx, cache, h)
        if x2 is None:
            x2 = self.ffn_norm.forward(h)
        if next_norm is not None and getattr(self.ffn, "split_norm", False):
            return self.ffn.forward(x2, ctx, h, next_norm=next_norm)
        self.ffn.forward(x2, ctx, h)
        return None


register_part("block", "prenorm", PreNormBlock)
