"""Next-token choice on the GPU for a batch of rows with per-row options.

The reference samples on the CPU (/root/reference/kernels/src/sampling.rs:229-333);
here the logits never leave the device: penalties, temperature, min-p, typical-p, top-k, softmax,
top-p and the draw are kernels, and only the chosen token ids come back.

Random numbers: draw number n of a request with seed s is a 24-bit fraction of a
SplitMix64 hash of (s, n).  It depends on nothing else, so a request's tokens do not
change with batch composition, nor when it is preempted and recomputed.  (The reference
seeds Rust's StdRng per session, /root/reference/engine/src/session.rs:50; its stream is
not reproduced.)
"""
from __future__ import annotations

import ctypes
from collections import Counter
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingParams

_MASK = (1 << 64) - 1


def uniform_draw(seed: int, n: int) -> float:
    """The n-th uniform number in [0, 1) of the stream with this seed."""
    z = (seed * 0x9E3779B97F4A7C15 + (n + 1) * 0xD1B54A32D192ED03) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


@dataclass
class TokenLogprob:
    """A generated token with its log-probability and the most probable alternatives, most probable first
    (/root/reference/engine/src/model.rs:475-486)."""
    token_id: int
    logprob: float
    top_logprobs: List[Tuple[int, float]]


class Sampler:
    def __init__(self, vocab_size: int, device, default_seed: int = 0):
        self.vocab_size = vocab_size
        self.device = device
        self.default_seed = default_seed
        self._work = None

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], draw_index: Sequence[int],
               prompt_tokens: Sequence[Sequence[int]], output_tokens: Sequence[Sequence[int]],
               top_n: Optional[int] = None, meanwhile=None):
        """``logits`` float32 [m, vocab] on the device; one ``SamplingParams`` per row;
        ``draw_index[i]`` is how many tokens row i's request has drawn before; the token
        lists feed the penalties.  Returns the chosen token of each row.
        With ``top_n`` (0..20) it returns (tokens, records) instead, a record per row being
        ``TokenLogprob(token_id, logprob, top_logprobs)``: log-probabilities of the distribution the token was
        drawn from, after temperature and filters (/root/reference/engine/src/model.rs:497-526).
        ``meanwhile``: called with the chosen tokens (int32 on the device) once the kernels are launched and
        before the tokens are waited for: host work that can run while the GPU does, such as queueing the
        next step behind them."""
        m = logits.shape[0]
        if m == 0:
            return [] if top_n is None else ([], [])
        if top_n is None and all(p.is_greedy for p in params):
            chosen = ops.argmax(logits)
            if meanwhile is None:
                return chosen.tolist()
            coming = ops.HostCopy(chosen)          # (queued before whatever `meanwhile` queues)
            meanwhile(chosen)
            return coming.result()
        if any(p.has_penalties for p in params):
            logits = self._penalised(logits, params, prompt_tokens, output_tokens)
        temp = np.asarray([p.temperature for p in params], dtype=np.float32)
        top_k = np.asarray([p.top_k if 0 < p.top_k < self.vocab_size else 0 for p in params], dtype=np.int32)
        top_p = np.asarray([p.top_p for p in params], dtype=np.float32)
        min_p = np.asarray([p.min_p for p in params], dtype=np.float32)
        typical_p = np.asarray([p.typical_p for p in params], dtype=np.float32)
        rnd = np.asarray([uniform_draw(self.default_seed if p.seed is None else p.seed, n)
                          for p, n in zip(params, draw_index)], dtype=np.float32)
        if self._work is None or self._work.shape[0] < m:
            self._work = torch.empty((max(m, 8), self.vocab_size), dtype=torch.float32, device=self.device)
        if top_n is None:
            chosen = ops.sample(logits, self._work, temp, top_k, top_p, min_p, rnd, typical_p)
            if meanwhile is None:
                return chosen.tolist()
            coming = ops.HostCopy(chosen)
            meanwhile(chosen)
            return coming.result()
        top_n = max(0, min(int(top_n), 20, self.vocab_size))
        info = torch.empty((m, 4), dtype=torch.float32, device=logits.device)
        tokens = ops.sample(logits, self._work, temp, top_k, top_p, min_p, rnd, typical_p, info).tolist()
        ids, lps = ops.top_logprobs(self._work, info, self.vocab_size, top_n)
        ids, lps, chosen = ids.tolist(), lps.tolist(), info[:, 3].tolist()
        records = [TokenLogprob(tok, chosen[r], [(i, lp) for i, lp in zip(ids[r], lps[r]) if i >= 0])
                   for r, tok in enumerate(tokens)]
        return tokens, records

    def _penalised(self, logits, params, prompt_tokens, output_tokens):
        rows, toks, counts, inwin = [], [], [], []
        for r, p in enumerate(params):
            if not p.has_penalties:
                continue
            gen = Counter(output_tokens[r]) if (p.presence_penalty or p.frequency_penalty) else Counter()
            window = set()
            if p.repeat_penalty != 1.0 and p.penalty_last_n > 0:
                hist = list(prompt_tokens[r]) + list(output_tokens[r])
                window = set(hist[-p.penalty_last_n:])
            for tok in set(gen) | window:
                rows.append(r)
                toks.append(tok)
                counts.append(gen.get(tok, 0))
                inwin.append(1 if tok in window else 0)
        if not rows:
            return logits
        out = ops.take_rows(logits)          # (the caller's logits stay as they are)
        ops.apply_penalties(out, rows, toks, counts, inwin,
                            [p.presence_penalty for p in params], [p.frequency_penalty for p in params],
                            [p.repeat_penalty for p in params])
        return out
