"""Block arrangements.

``prenorm``: ``h += mixer(norm(h)); h += ffn(norm(h))`` — sequential, two
residual adds (/root/reference/engine/src/model.rs:952-1314; declared as
[PreNormAttention, PreNormFfn], /root/reference/engine/src/architecture.rs:56-65).
The residual stream ``h`` is float32 in every dtype.
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

    def forward(self, h, ctx, cache):
        x = self.mixer_norm.forward(h)
        self.mixer.forward(x, ctx, cache, h)
        x = self.ffn_norm.forward(h)
        self.ffn.forward(x, ctx, h)


register_part("block", "prenorm", PreNormBlock)
