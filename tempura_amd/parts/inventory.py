"""Every checkpoint tensor a model reads, gathered from its parts (no device needed)."""
from __future__ import annotations

from typing import Dict

from ..config.spec import ModelSpec
from .base import WeightInfo, part_class


def expected_weights(spec: ModelSpec) -> Dict[str, WeightInfo]:
    """Every checkpoint tensor the model reads, by name (no device needed)."""
    out: Dict[str, WeightInfo] = {}
    out.update(part_class("embedding", spec.embedding.kind).expected_weights(
        spec.embedding, spec.hidden_size, spec.vocab_size))
    for ls in spec.layers:
        out.update(part_class("block", ls.block).expected_weights(ls, spec.hidden_size))
    out.update(part_class("norm", spec.final_norm.kind).expected_weights(spec.final_norm, spec.hidden_size))
    out.update(part_class("lm_head", spec.lm_head.kind).expected_weights(
        spec.lm_head, spec.hidden_size, spec.vocab_size))
    return out
