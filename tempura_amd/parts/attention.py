"""Grouped-query attention over the paged cache.

Per token: q, k, v projections (no bias), position encoding on q and k, k and v
stored into the cache pages, causal (optionally windowed) softmax attention
over the request's cached keys with ``kv_head = head // (heads / kv_heads)``,
output projection added into the residual stream
(/root/reference/engine/src/model.rs:1007-1152,
/root/reference/kernels/src/attention.rs:28-87).
A window of ``w`` lets query position p see keys p-w+1 .. p
(/root/reference/kernels/src/attention.rs:55-59).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import CacheSpec, Mixer, WeightInfo, build_part, part_class, register_part


class PagedAttention(Mixer):
    graph_safe = True      # only kernels on device-resident step data: may be captured in a graph
    #: the value cache is transposed, eight consecutive tokens of one element being one 16-byte piece: a portion that
    #: starts at a multiple of eight positions (and of eight rows of the batch) has its values stored piece by piece
    preferred_portion_align = 8
    split_norm = True      # takes rows whose norm its first product finishes; prepares the next norm in its last

    def __init__(self, spec, hidden_size, dtype, device):
        super().__init__(spec, hidden_size, dtype, device)
        p = spec.params
        self.num_heads = int(p["num_heads"])
        self.num_kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        if self.num_heads % self.num_kv_heads != 0:
            raise ValueError("attention: heads must be a multiple of kv heads")
        self.scale = float(p["scale"])
        self.window = p.get("window")
        self.q_dim = self.num_heads * self.head_dim
        self.kv_dim = self.num_kv_heads * self.head_dim
        self.position = build_part("position", p["position"], hidden_size, dtype, device)
        self.wqkv = None
        self.wo = None

    @classmethod
    def expected_weights(cls, spec, hidden_size):
        p, w = spec.params, spec.weights
        q_dim = p["num_heads"] * p["head_dim"]
        kv_dim = p["num_kv_heads"] * p["head_dim"]
        out = {
            w["q"]: WeightInfo((q_dim, hidden_size)),
            w["k"]: WeightInfo((kv_dim, hidden_size)),
            w["v"]: WeightInfo((kv_dim, hidden_size)),
            w["o"]: WeightInfo((hidden_size, q_dim)),
        }
        # a position encoding may have tensors of its own (a rotary one has none)
        out.update(part_class("position", p["position"].kind).expected_weights(p["position"], hidden_size))
        return out

    def _paired(self, t: torch.Tensor) -> torch.Tensor:
        """The rows of a q or k projection with every head's rotary elements in paired order: rows
        (2 d, 2 d + 1) of a head are rows (d, d + rotary_dim / 2) of the checkpoint's split-half order, so
        that the two elements that rotate together are neighbours (the rotation kernels expect that, and a
        product's epilogue can rotate what it holds).  q and k are permuted alike, which leaves every score
        as it was; the cache then holds keys in this order."""
        rot = self.position.rotary()
        if rot is None or rot[1] == 0:
            return t
        rd, half, d = rot[1], rot[1] // 2, self.head_dim
        order = torch.arange(d)
        order[0:rd:2] = torch.arange(half)
        order[1:rd:2] = torch.arange(half) + half
        heads = t.shape[0] // d
        return t.view(heads, d, -1)[:, order.to(t.device), :].reshape(t.shape)

    def load_weights(self, get):
        w = self.spec.weights
        # One [q_dim + 2 kv_dim, hidden] matrix: one product instead of three.
        parts = [self._paired(get(w["q"])), self._paired(get(w["k"])), get(w["v"])]
        # (stored tiled where the sizes allow: the products then read whole cache lines)
        self.wqkv = ops.tile_weight(torch.cat([self._to_device(t) for t in parts], dim=0).contiguous())
        self.wo = ops.tile_weight(self._to_device(get(w["o"])))
        self.position.load_weights(get)

    def cache_spec(self):
        kind = "window" if self.window is not None else "full"
        return CacheSpec(kind, self.num_kv_heads, self.head_dim, self.window)

    def forward(self, x, ctx, cache, residual, next_norm=None):
        rot = self.position.rotary()
        q = None
        if rot is not None and cache.writes:
            rows = x.x if isinstance(x, ops.Prenormed) else x
            if ops.linear_rope_ok(x.shape[0], self.wqkv.shape[0], x.shape[1], self.head_dim, rot[1], cache.k.shape[2],
                                  rows.dtype, cache.k.dtype, isinstance(x, ops.Prenormed)):
                # a few rows (decoding) or a long step: the projection rotates and stores its rows itself
                table = self.position.table(ctx, always=True) if hasattr(self.position, "table") else None
                q = ops.linear_rope_kv(x, self.wqkv, ctx.positions, ctx.slot_mapping[cache.group], rot[0], rot[1], rot[2],
                                       self.num_heads, self.num_kv_heads, self.head_dim, cache.k, cache.v, table)
        if q is None:
            q = self._project_and_rotate(x, ctx, cache, rot)
        a = ops.paged_attention(
            q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.cu_seqlens, ctx.context_lens,
            ctx.token_req, self.scale, int(self.window or 0), ctx.max_q_len, ctx.max_context_len,
            ctx.num_single)
        if next_norm is None:
            ops.linear(a, self.wo, torch.float32, residual=residual)
            return None
        return ops.linear(a, self.wo, torch.float32, residual=residual, next_norm=next_norm)[1]

    def _project_and_rotate(self, x, ctx, cache, rot):
        """q (rotated, [n, heads, head_dim]) of the projection; k and v go to the cache."""
        # (with a rotary position the next kernel may add the projection's partial sums itself)
        if cache.writes:
            qkv = ops.linear(x, self.wqkv, torch.float32, partial_ok=rot is not None)
        else:
            # A call that reads another call's cache needs queries only.
            qkv = ops.linear(x, ops.weight_rows(self.wqkv, 0, self.q_dim), torch.float32, partial_ok=rot is not None)
        if rot is None:
            q = qkv[:, : self.q_dim]
            k = qkv[:, self.q_dim: self.q_dim + self.kv_dim] if cache.writes else None
            q2, k2 = self.position.apply(q, k, ctx.positions)
            if cache.writes:
                qkv = torch.cat([q2, k2, qkv[:, self.q_dim + self.kv_dim:]], dim=1).contiguous()
            else:
                qkv = q2.contiguous()
            inv_freq, rotary_dim, factor, table = None, 0, 1.0, None
        else:
            inv_freq, rotary_dim, factor = rot
            table = self.position.table(ctx) if hasattr(self.position, "table") else None
        q = ops.rope_kv_write(
            qkv, ctx.positions, ctx.slot_mapping[cache.group] if cache.writes else None,
            inv_freq, rotary_dim, factor, self.num_heads, self.num_kv_heads, self.head_dim,
            cache.k if cache.writes else None, cache.v if cache.writes else None, self.dtype, table)
        return q


register_part("mixer", "attention", PagedAttention)
