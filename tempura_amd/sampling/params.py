"""Sampling options, with the reference's names, meanings and defaults
(/root/reference/kernel-api/src/lib.rs:247-290).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class SamplingParams:
    temperature: float = 1.0        # 0 => greedy (argmax, last maximum wins)
    top_k: int = 50                 # keep the k largest; 0 switches the filter off (the reference panics on 0)
    top_p: float = 1.0              # nucleus over the kept ones
    min_p: float = 0.0              # drop logits below max + ln(min_p)
    typical_p: float = 1.0          # keep the tokens nearest the entropy until their mass exceeds it; 1.0 = off
    repeat_penalty: float = 1.0     # over the last `penalty_last_n` tokens of prompt + output
    penalty_last_n: int = 64
    presence_penalty: float = 0.0   # over generated tokens
    frequency_penalty: float = 0.0
    seed: Optional[int] = None      # None: the engine's default seed
    max_new_tokens: int = 256       # the reference's HTTP default (/root/reference/server/src/api.rs:302-304)
    eos_token_id: Optional[List[int]] = None   # None: the model's; [] : never stop on a token
    ignore_eos: bool = False

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.top_k < 0:
            raise ValueError("top_k must be >= 0")
        if not (0 < self.top_p <= 1.0):
            raise ValueError("top_p must be in (0, 1]")
        if not (0 <= self.min_p <= 1.0):
            raise ValueError("min_p must be in [0, 1]")
        if not (0 <= self.typical_p <= 1.0):
            raise ValueError("typical_p must be in [0, 1]")
        if self.repeat_penalty <= 0:
            raise ValueError("repeat_penalty must be positive")
        if self.max_new_tokens < 0:
            raise ValueError("max_new_tokens must be >= 0")
        if isinstance(self.eos_token_id, int):
            self.eos_token_id = [self.eos_token_id]

    @property
    def is_greedy(self) -> bool:
        """Pure greedy: plain argmax of the untouched logits.  The reference's rule leaves the repetition
        penalty out (/root/reference/kernel-api/src/lib.rs:286-290) because its serving path hands that
        penalty no earlier tokens; here the penalty does see the request's history, so a temperature-0 row
        with any penalty takes the argmax of the penalised logits, whatever else is in the batch."""
        return self.temperature == 0.0 and not self.has_penalties

    @property
    def has_penalties(self) -> bool:
        return self.presence_penalty != 0.0 or self.frequency_penalty != 0.0 or self.repeat_penalty != 1.0
