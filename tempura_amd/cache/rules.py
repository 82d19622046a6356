"""Which keys a cache group's queries can still see, as data.

A ``CacheSpec.kind`` names a visibility rule: the first key that a query at position p can see, as a function
of p and a few integers.  Pages whose keys all lie before that key go back to the pool.  The rule functions
themselves live in the host library (``RULES`` in csrc/host/cache_core.cpp, indexed by ``code``); this table is
the one place that ties a kind's name to a code, to the integers it passes and to the page count a request can
hold under it.  A kind whose first visible key is one of the core's functions is added with ``register_rule``
and nothing else; a new function is one more entry of ``RULES`` there and one ``register_rule`` here.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Sequence

from ..parts.base import CacheSpec

#: integers a rule may take (``RULE_PARAMS`` of the core)
NUM_PARAMS = 4


@dataclass(frozen=True)
class VisibilityRule:
    code: int                                             # index into the core's RULES
    params: Callable[[CacheSpec], Sequence[int]]          # the rule's integers for a spec
    #: most tokens for which a request of ``total`` tokens holds pages at one time when a step brings at most
    #: ``step`` tokens (whole pages come on top); the scheduler refuses a request that could never fit
    held_tokens: Callable[[CacheSpec, int, int], int]


def _window_of(spec: CacheSpec) -> int:
    return int(spec.window) if spec.window is not None else 0


_RULES: Dict[str, VisibilityRule] = {
    # every key stays visible: pages are held until the request ends
    "full": VisibilityRule(0, lambda s: (), lambda s, total, step: total),
    # the last `window` keys (no window given: every key)
    "window": VisibilityRule(1, lambda s: (_window_of(s),),
                             lambda s, total, step: min(total, _window_of(s) + step) if _window_of(s) > 0 else total),
    # the keys of the query's own aligned chunk of `window` positions
    "chunk": VisibilityRule(2, lambda s: (_window_of(s),),
                            lambda s, total, step: min(total, _window_of(s) + step) if _window_of(s) > 0 else total),
}


def register_rule(kind: str, rule: VisibilityRule) -> None:
    """Make ``CacheSpec(kind=...)`` usable; ``rule.code`` must be a function the core has."""
    _RULES[kind] = rule


def rule_of(kind: str) -> VisibilityRule:
    try:
        return _RULES[kind]
    except KeyError:
        raise ValueError(f"no visibility rule is registered for cache kind {kind!r} (known: {sorted(_RULES)})") from None


def rule_args(spec: CacheSpec):
    """(code, NUM_PARAMS integers) of a spec's rule, as the core takes them."""
    rule = rule_of(spec.kind)
    params = [int(p) for p in rule.params(spec)]
    if len(params) > NUM_PARAMS:
        raise ValueError(f"cache kind {spec.kind!r}: {len(params)} integers, the core takes {NUM_PARAMS}")
    return rule.code, params + [0] * (NUM_PARAMS - len(params))
