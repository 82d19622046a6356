from .base import (Part, Mixer, FeedForward, Norm, PositionEncoding, Block, CacheSpec, StateSpec,
                   WeightInfo, register_part, part_class, build_part)
from . import norm, rope, attention, ffn, block, embedding  # noqa: F401  (register the built-in parts)
from .inventory import expected_weights
from .block import ArrangedBlock

__all__ = ["Part", "Mixer", "FeedForward", "Norm", "PositionEncoding", "Block", "CacheSpec",
           "StateSpec", "WeightInfo", "register_part", "part_class", "build_part", "ArrangedBlock"]
