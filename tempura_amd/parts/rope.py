"""Rotary position encoding with optional llama3 frequency scaling.

Pairs are split-half: element ``d`` rotates with element ``d + D/2`` by the angle
``pos * inv_freq[d]`` (/root/reference/kernels/src/rope.rs:18-53, 900-921), with
``inv_freq[d] = theta^(-2d/D)``.  The llama3 rule rescales each frequency by its
wavelength (/root/reference/kernels/src/rope.rs:848-881).  The table is built in
float64 on the host; kernels form the angle from the integer position in 64-bit
and take sine and cosine of it, so no precision is lost at large positions.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import PositionEncoding, register_part


def rotary_inv_freq(head_dim: int, theta: float, scaling=None, rotary_dim=None) -> torch.Tensor:
    """float64 [rotary_dim/2] inverse frequencies."""
    rd = head_dim if rotary_dim is None else int(rotary_dim)
    if rd % 2 != 0 or rd > head_dim or rd < 0:
        raise ValueError(f"rotary_dim {rd} must be even and at most head_dim {head_dim}")
    half = rd // 2
    d = torch.arange(half, dtype=torch.float64)
    inv = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * d / rd) if half else d
    if scaling is None:
        return inv
    kind = scaling.get("rope_type", scaling.get("type"))
    if kind != "llama3":
        raise ValueError(f"rope scaling {kind!r} is not supported")
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    low_wl = orig / low
    high_wl = orig / high
    out = inv.clone()
    for i in range(half):
        f = float(inv[i])
        wl = 2.0 * math.pi / f
        if wl < high_wl:
            continue
        if wl > low_wl:
            out[i] = f / factor
        else:
            smooth = (orig / wl - low) / (high - low)
            out[i] = f / factor * (1.0 - smooth) + f * smooth
    return out


class RotaryPosition(PositionEncoding):
    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.head_dim = int(p["head_dim"])
        self.rotary_dim = int(p.get("rotary_dim") or self.head_dim)
        self.factor = float(p.get("attn_factor", 1.0))
        inv_freq = rotary_inv_freq(self.head_dim, float(p["theta"]), p.get("scaling"), self.rotary_dim)
        self.inv_freq = inv_freq.to(device)
        # layers whose rotations have the same frequencies share one table per step
        self._table_key = ("rope", self.rotary_dim, self.factor, hash(tuple(inv_freq.tolist())))

    #: steps with at least this many tokens compute cosines and sines once for all layers
    TABLE_FROM = 256

    def rotary(self):
        return self.inv_freq, self.rotary_dim, self.factor

    def table(self, ctx, always: bool = False):
        """This step's [tokens, rotary_dim / 2, 2] cosines and sines, shared by every layer whose rotation has
        the same frequencies; None for short steps (the rotation kernel then computes them itself) unless
        ``always`` (a product that rotates in its epilogue wants the table at any size)."""
        if self.rotary_dim == 0 or (ctx.num_tokens < self.TABLE_FROM and not always):
            return None
        if self._table_key not in ctx.shared:
            ctx.shared[self._table_key] = ops.rope_table(ctx.positions, self.inv_freq, self.rotary_dim, self.factor)
        return ctx.shared[self._table_key]


class NoPosition(PositionEncoding):
    """No positional signal inside the mixer."""


register_part("position", "rope", RotaryPosition)
register_part("position", "none", NoPosition)
