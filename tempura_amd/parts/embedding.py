"""Token embedding and output head.

``hidden[t] = embed[token[t]]`` with no scaling
(/root/reference/engine/src/model.rs:672-684); logits are
``norm(hidden)[rows] @ lm_head^T`` in float32, and when the checkpoint has no
output matrix the embedding matrix is used for it
(/root/reference/engine/src/weights.rs:156-166).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightInfo, register_part


class TokenEmbedding(Part):
    category = "embedding"

    def __init__(self, spec, hidden_size, dtype, device, vocab_size):
        super().__init__(spec, hidden_size, dtype, device)
        self.vocab_size = vocab_size
        self.weight = None

    @classmethod
    def expected_weights(cls, spec, hidden_size, vocab_size):
        return {spec.weights["weight"]: WeightInfo((vocab_size, hidden_size))}

    def load_weights(self, get):
        self.weight = self._to_device(get(self.spec.weights["weight"]))

    def forward(self, tokens):
        """int32 [tokens] -> float32 [tokens, hidden] (the residual stream)."""
        return ops.embed(tokens, self.weight)


class OutputHead(Part):
    category = "lm_head"

    def __init__(self, spec, hidden_size, dtype, device, vocab_size):
        super().__init__(spec, hidden_size, dtype, device)
        self.vocab_size = vocab_size
        self.weight = None
        self.tied = bool(spec.params.get("tied", False))

    @classmethod
    def expected_weights(cls, spec, hidden_size, vocab_size):
        # Tied: the tensor is neither required nor generated, and is ignored if present.
        init = "skip" if spec.params.get("tied", False) else "normal"
        return {spec.weights["weight"]: WeightInfo((vocab_size, hidden_size), init, optional=True)}

    def load_weights(self, get, embedding: TokenEmbedding = None):
        t = None if self.tied else get(self.spec.weights["weight"], optional=True)
        if t is None:
            if embedding is None or embedding.weight is None:
                raise ValueError("output head is tied but no embedding matrix is loaded")
            # The products read tiled weights at nearly twice the rate of row-major ones (the head of the 3B shape,
            # 128256 x 3072: 208 us row-major, 120 us tiled), and the lookup needs the rows as they are: the head
            # takes a tiled copy where the kernels have a tiled form (bfloat16 on the GPU; vocab x hidden x 2 bytes
            # more), else the same buffer.
            self.weight = ops.tile_weight(embedding.weight)
            self.tied = True
        else:
            self.weight = ops.tile_weight(self._to_device(t))

    def forward(self, x):
        """normed rows [m, hidden] -> float32 logits [m, vocab]."""
        return ops.linear(x, self.weight, torch.float32)


register_part("embedding", "embedding", TokenEmbedding)
register_part("lm_head", "lm_head", OutputHead)
