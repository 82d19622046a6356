"""SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))``, no biases
(/root/reference/engine/src/model.rs:1203-1231,1301-1313;
``silu(x) = x / (1 + exp(-x))``, /root/reference/kernels/src/ggml/vec_llama.rs:808-810).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, WeightInfo, register_part


class SwiGLU(FeedForward):
    graph_safe = True      # only kernels on device-resident step data: may be captured in a graph
    split_norm = True      # takes rows whose norm its first product finishes; prepares the next norm in its last

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        self.intermediate_size = int(spec.params["intermediate_size"])
        self.w13 = None
        self.w2 = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        i, w = spec.params["intermediate_size"], spec.weights
        return {
            w["gate"]: WeightInfo((i, hidden_size)),
            w["up"]: WeightInfo((i, hidden_size)),
            w["down"]: WeightInfo((hidden_size, i)),
        }

    def load_weights(self, get):
        w = self.spec.weights
        gate, up = self._to_device(get(w["gate"])), self._to_device(get(w["up"]))
        # One matrix, one product instead of two.  In bfloat16 the rows alternate eight of gate and
        # eight of up, so that the product's epilogue applies silu(g) * u to its float32 sums.
        self.fused = self.dtype == torch.bfloat16 and ops.gated_layout_ok(self.intermediate_size, self.hidden_size)
        if self.fused:
            self.w13 = ops.tile_weight(ops.interleave_gate_up(gate, up))
        else:
            self.w13 = ops.tile_weight(torch.cat([gate, up], dim=0).contiguous())
        self.w2 = ops.tile_weight(self._to_device(get(w["down"])))

    def forward(self, x, ctx, residual, next_norm=None):
        if self.fused:
            # (a few rows go to the next product k-blocked: it reads them straight from global memory)
            a = ops.linear_swiglu(x, self.w13, blocked_out=True)
        else:
            gu = ops.linear(x, self.w13, torch.float32)
            a = ops.swiglu(gu, self.dtype)
        if next_norm is None:
            ops.linear(a, self.w2, torch.float32, residual=residual)
            return None
        return ops.linear(a, self.w2, torch.float32, residual=residual, next_norm=next_norm)[1]


register_part("ffn", "swiglu", SwiGLU)
