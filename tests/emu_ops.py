"""Plain PyTorch versions of the kernel operations, one per kernel, with the same
signatures as ``tempura_amd.kernels.ops``.  They serve two purposes in tests only:
(1) the reference each HIP kernel is graded against on its own; (2) a host stand-in
installed with ``ops.set_backend`` so that the engine's bookkeeping (pages, batching,
cutting) can be tested without a GPU.  Everything is computed in float64 and rounded
to the requested dtype at the end.
"""
from __future__ import annotations

import torch


class EmuOps:
    def embed(self, tokens, table):
        return table[tokens.long()].to(torch.float32)

    def rmsnorm(self, h, weight, eps, out_dtype, rows=None):
        x = h.double()
        if rows is not None:
            x = x[rows.long()]
        y = x * (1.0 / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)) * weight.double()
        return y.to(out_dtype)

    def split_norm_ok(self, m, width, dtype):
        return dtype == torch.bfloat16 and 0 < m <= 128 and width % 32 == 0

    @staticmethod
    def _rows(x):
        """Plain rows, or handed-over rows (x = bfloat16(h * weight), ss = sums of squares per 16 columns)
        with the factor that finishes their norm."""
        from tempura_amd.kernels.ops import KBlocked, Prenormed
        if isinstance(x, KBlocked):
            return x.row_major().double(), 1.0
        if isinstance(x, Prenormed):
            rstd = torch.rsqrt(x.ss.double().sum(0)[: x.x.shape[0]] / x.x.shape[1] + x.eps)
            return x.x.double(), rstd[:, None]
        return x.double(), 1.0

    def linear(self, x, w, out_dtype, residual=None, next_norm=None):
        from tempura_amd.kernels.ops import Prenormed
        xd, scale = self._rows(x)
        y = (xd @ w.double().T) * scale
        if residual is not None:
            residual.copy_((residual.double() + y).to(torch.float32))
            if next_norm is None:
                return residual
            m, n = residual.shape
            if not (self.split_norm_ok(m, n, x.dtype if torch.is_tensor(x) else torch.bfloat16) and xd.shape[1] % 32 == 0):
                return residual, None
            weight, eps = next_norm
            if m > 16:       # the kernel that adds the product into the residual norms the rows as well
                return residual, self.rmsnorm(residual, weight, eps, torch.bfloat16)
            ss = torch.zeros(((n + 15) // 16, 16), dtype=torch.float32)
            sq = torch.nn.functional.pad(residual.double() ** 2, (0, ss.shape[0] * 16 - n))
            ss[:, :m] = sq.reshape(m, -1, 16).sum(2).T.to(torch.float32)
            return residual, Prenormed((residual * weight).to(torch.bfloat16), ss, eps)
        return y.to(out_dtype)

    def linear_swiglu(self, x, w, blocked_out=False):
        from tempura_amd.kernels.ops import KBlocked
        xd, scale = self._rows(x)
        x = xd
        y = ((x @ w.double().T) * scale).reshape(x.shape[0], -1, 2, 8)      # eight gate rows, eight up rows in turn
        g, u = y[:, :, 0].reshape(x.shape[0], -1), y[:, :, 1].reshape(x.shape[0], -1)
        out = (g / (1.0 + torch.exp(-g)) * u).to(torch.bfloat16)
        m, i = out.shape
        if blocked_out and 0 < m <= 16 and i % 32 == 0:
            return KBlocked(out.reshape(m, i // 8, 8).permute(1, 0, 2).contiguous(), m, i)
        return out

    def rope_kv_write(self, qkv, positions, slots, inv_freq, rotary_dim, factor, num_heads, num_kv_heads,
                      head_dim, k_cache, v_cache, q_dtype):
        n = qkv.shape[0]
        nrot = num_heads + (num_kv_heads if slots is not None else 0)
        x = qkv.double()[:, : nrot * head_dim].reshape(n, nrot, head_dim).clone()
        if rotary_dim:
            half = rotary_dim // 2
            ang = positions.double()[:, None] * inv_freq.double()[None, :]
            c = (torch.cos(ang) * factor)[:, None, :]
            s = (torch.sin(ang) * factor)[:, None, :]
            # paired order: elements (2 d, 2 d + 1) rotate together by the angle of pair d
            x0, x1 = x[..., 0:rotary_dim:2].clone(), x[..., 1:rotary_dim:2].clone()
            x[..., 0:rotary_dim:2] = x0 * c - x1 * s
            x[..., 1:rotary_dim:2] = x0 * s + x1 * c
        q = x[:, :num_heads].to(q_dtype).contiguous()
        if slots is not None:
            k = x[:, num_heads:]
            v = qkv.double()[:, nrot * head_dim:].reshape(n, num_kv_heads, head_dim)
            ps = k_cache.shape[2]
            page, off = slots.long() // ps, slots.long() % ps
            k_cache[page, :, off] = k.to(k_cache.dtype)
            v_cache[page, :, :, off] = v.to(v_cache.dtype)          # values are kept transposed
        return q

    def paged_attention(self, q, k_cache, v_cache, block_tables, cu_seqlens, context_lens, token_req, scale,
                        window, max_q_len, max_context_len, num_single=None):
        n, heads, d = q.shape
        kvh, ps = k_cache.shape[1], k_cache.shape[2]
        group = heads // kvh
        out = torch.zeros(n, heads, d, dtype=torch.float64)
        cu = cu_seqlens.tolist()
        for r in range(block_tables.shape[0]):
            qs, qe = cu[r], cu[r + 1]
            ctx = int(context_lens[r])
            pages = block_tables[r].long()
            j = torch.arange(ctx)
            rows_page, rows_off = pages[j // ps], j % ps
            K = k_cache[rows_page, :, rows_off].double()      # [ctx, kvh, d]
            V = v_cache[rows_page, :, :, rows_off].double()      # [ctx, kvh, d]
            for t in range(qs, qe):
                pos = ctx - (qe - qs) + (t - qs)
                lo = max(0, pos - window + 1) if window > 0 else 0
                for h in range(heads):
                    sc = (K[lo: pos + 1, h // group] @ q[t, h].double()) * scale
                    p = torch.softmax(sc, dim=0)
                    out[t, h] = p @ V[lo: pos + 1, h // group]
        return out.reshape(n, heads * d).to(q.dtype)

    def swiglu(self, gu, out_dtype):
        i = gu.shape[1] // 2
        g, u = gu.double()[:, :i], gu.double()[:, i:]
        return (g / (1.0 + torch.exp(-g)) * u).to(out_dtype)

    def argmax(self, logits):
        v = logits.shape[1]
        flipped = torch.flip(logits, dims=[1])
        return (v - 1 - torch.argmax(flipped, dim=1)).to(torch.int32)

    def take_rows(self, t, rows=None):
        return t.clone() if rows is None else t[torch.tensor(list(rows), dtype=torch.long)].clone()

    def zero_rows(self, t, rows):
        if len(rows):
            t[torch.tensor(list(rows), dtype=torch.long)] = 0
