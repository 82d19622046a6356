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


class PreNormBlock:
    category = "block"

    def __init__(self, layer_spec, hidden_size, dtype, device):
        self.layer_spec = layer_spec
        self.mixer_norm = build_part("norm", layer_spec.mixer_norm, hidden_size, dtype, device)
        self.mixer = build_part("mixer", layer_spec.mixer, hidden_size, dtype, device)
        self.ffn_norm = build_part("norm", layer_spec.ffn_norm, hidden_size, dtype, device)
        self.ffn = build_part("ffn", layer_spec.ffn, hidden_size, dtype, device)

    def parts(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    @classmethod
    def expected_weights(cls, layer_spec, hidden_size):
        out = {}
        for cat, ps in (("norm", layer_spec.mixer_norm), ("mixer", layer_spec.mixer),
                        ("norm", layer_spec.ffn_norm), ("ffn", layer_spec.ffn)):
            out.update(part_class(cat, ps.kind).expected_weights(ps, hidden_size))
        return out

    def load_weights(self, get):
        for p in self.parts():
            p.load_weights(get)

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
