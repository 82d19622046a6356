"""RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w``.

The reference multiplies ``x * scale * w`` with eps inside the square root,
added to the mean (/root/reference/kernels/src/ggml/ops_llama.rs:201-216).
The sum of squares and the scale are computed in float32 in every dtype.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Norm, WeightInfo, register_part


class RMSNorm(Norm):
    graph_safe = True      # only kernels on device-resident step data: may be captured in a graph

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.eps = float(spec.params["eps"])
        self.weight = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        return {spec.weights["weight"]: WeightInfo((hidden_size,), "ones")}

    def load_weights(self, get):
        # Norm weights are tiny and multiply in float32: keep them in float32.
        self.weight = self._to_device(get(self.spec.weights["weight"]), torch.float32)

    def forward(self, h, rows=None):
        return ops.rmsnorm(h, self.weight, self.eps, self.dtype, rows)

    def deferred(self, m):
        """(weight, eps) when the two products around this norm can carry it for ``m`` rows (the one
        before prepares, the one after applies the scale), else None."""
        if ops.split_norm_ok(m, self.hidden_size, self.dtype):
            return self.weight, self.eps
        return None


register_part("norm", "rmsnorm", RMSNorm)
