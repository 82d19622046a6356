"""Shared pieces of the tests: tiny configurations, model folders, step schedules."""
from __future__ import annotations

import os
import random
from typing import Dict, List, Sequence, Tuple

import torch

import plain
from tempura_amd.config import LlamaConfig, RopeScaling
from tempura_amd.weights import write_random_model

# Two tiny configurations that differ in every size and option, plus a windowed one.
# A: groups of 2, head size 16, untied, plain rope.
# B: one kv head (MQA), head size 12 (no power of two, no multiple of 8), hidden 96, vocabulary
#    384, tied, llama3 scaling whose original length (64) is passed so all three branches are hit.
# C: head size 48, 6 heads in 3 groups, hidden 80 (!= heads * head size), a window of 24 on
#    alternating layers, vocabulary 300.
CONFIGS: Dict[str, LlamaConfig] = {
    "A": LlamaConfig(hidden_size=64, intermediate_size=192, num_hidden_layers=2, num_attention_heads=4,
                     num_key_value_heads=2, head_dim=16, vocab_size=256, max_position_embeddings=2048,
                     rms_norm_eps=1e-5, rope_theta=10000.0, rope_scaling=None, tie_word_embeddings=False),
    "B": LlamaConfig(hidden_size=96, intermediate_size=320, num_hidden_layers=3, num_attention_heads=8,
                     num_key_value_heads=1, head_dim=12, vocab_size=384, max_position_embeddings=1024,
                     rms_norm_eps=1e-6, rope_theta=500000.0,
                     rope_scaling=RopeScaling("llama3", 8.0, 1.0, 4.0, 64), tie_word_embeddings=True),
    "C": LlamaConfig(hidden_size=80, intermediate_size=136, num_hidden_layers=4, num_attention_heads=6,
                     num_key_value_heads=3, head_dim=48, vocab_size=300, max_position_embeddings=512,
                     rms_norm_eps=3e-6, rope_theta=25000.0,
                     rope_scaling=RopeScaling("llama3", 4.0, 1.0, 2.0, 32), tie_word_embeddings=False,
                     sliding_window=24,
                     layer_types=["sliding_attention", "full_attention", "sliding_attention", "full_attention"]),
    # D: sizes the matrix-core kernels take (head size 64, widths that are multiples of 32, gate/up rows
    #    in eights): in bfloat16 every fast path runs end to end (skinny, mid and tiled products, fused
    #    SwiGLU, MFMA attention for portions and for single tokens with a split context)
    "D": LlamaConfig(hidden_size=128, intermediate_size=320, num_hidden_layers=2, num_attention_heads=4,
                     num_key_value_heads=2, head_dim=64, vocab_size=512, max_position_embeddings=2048,
                     rms_norm_eps=1e-5, rope_theta=500000.0,
                     rope_scaling=RopeScaling("llama3", 8.0, 1.0, 4.0, 128), tie_word_embeddings=False),
    # E: head size 80 (a multiple of 16, no power of two), groups of 3, an odd vocabulary, pages of 64, and a
    #    feed-forward width (136) that the gated product takes but the k-blocked hand-over between the two
    #    feed-forward products does not (it steps by 32)
    "E": LlamaConfig(hidden_size=160, intermediate_size=136, num_hidden_layers=2, num_attention_heads=6,
                     num_key_value_heads=2, head_dim=80, vocab_size=1001, max_position_embeddings=4096,
                     rms_norm_eps=1e-4, rope_theta=1000000.0, rope_scaling=None, tie_word_embeddings=True),
}
#: weights are N(0, STD): large enough that attention is peaked and faults show
STD = 0.15
STD_OF = {"E": 0.1}
SEED_OF = {"A": 11, "B": 23, "C": 37, "D": 41, "E": 53}


class TinyModels:
    def __init__(self, root):
        self.root = str(root)
        self._made = {}

    def path(self, name: str, dtype: str = "float32") -> str:
        key = (name, dtype)
        if key not in self._made:
            d = os.path.join(self.root, f"{name}_{dtype}")
            cfg = LlamaConfig.from_dict(CONFIGS[name].to_dict())
            write_random_model(cfg, d, seed=SEED_OF[name], std=STD_OF.get(name, STD), norm_jitter=0.2, dtype=dtype)
            self._made[key] = d
        return self._made[key]

    def plain_model(self, name: str, dtype: str = "float32"):
        return plain.read_model_dir(self.path(name, dtype))


def random_tokens(vocab: int, n: int, seed: int) -> List[int]:
    g = random.Random(seed)
    return [g.randrange(vocab) for _ in range(n)]


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Largest difference relative to the largest reference logit."""
    return float((got.double() - ref.double()).abs().max() / ref.double().abs().max().clamp_min(1e-30))


#: bounds on rel_err against the plain float64 implementation.  The float32 engine is held to a constant.  The
#: bfloat16 engine is held to the noise that its storage type explains: ``BF16_FACTOR`` times the distance between
#: the plain implementation with every stored value rounded to bfloat16 (``plain.forward(stored=plain.as_bfloat16)``)
#: and the exact one, request by request (``noise_bound``).  Peaked attention under large weights makes that noise
#: large and flat attention makes it small; a constant would be too loose for the one and too tight for the other.
#: ``TOL["bfloat16"]`` remains for single parts and kernels, whose operands are rounded once.
TOL = {"float32": 2e-5, "bfloat16": 3e-2}
BF16_FACTOR = 2.0


def float32_bound(cfg: dict) -> float:
    """The float32 engine's bound for a model of these widths.  A float32 sum of K terms carries a rounding error
    that grows like sqrt(K); ``TOL["float32"]`` was set on models whose longest sum has a few hundred terms, and a
    model whose products run over thousands gets the constant times sqrt(K / 512) (the Llama-3.1-8B widths, K up to
    14,336: 1.06e-4; every tiny configuration: the constant itself).  A wrong key, page or position costs 1e-2 and
    more at any width."""
    H = cfg["hidden_size"]
    nH = cfg["num_attention_heads"]
    K = max(H, cfg["intermediate_size"], nH * (cfg.get("head_dim") or H // nH))
    return TOL["float32"] * max(1.0, (K / 512.0) ** 0.5)


def plain_reference(cfg, W, tokens, dtype: str):
    """(exact logits [T, vocab] of the plain implementation, bound on rel_err for an engine of ``dtype``): the
    constant in float32 (``float32_bound``: scaled up for wide models); in bfloat16 ``BF16_FACTOR`` times the rounding noise of bfloat16 storage on this request."""
    exact = plain.forward(cfg, W, tokens)
    if dtype == "float32":
        return exact, float32_bound(cfg)
    rounded = plain.forward(cfg, W, tokens, stored=plain.as_bfloat16)
    return exact, BF16_FACTOR * rel_err(rounded, exact)


# ---- step schedules ---------------------------------------------------------------------------
# A schedule is a list of steps; a step is (entries, end) with entries = [(rid, start, count)].
def roundup(n: int, m: int) -> int:
    return (n + m - 1) // m * m


def schedule_whole(lengths: Dict[str, int]):
    return [([(rid, 0, n)], [rid]) for rid, n in lengths.items()]


def schedule_bulk_tail(lengths: Dict[str, int], tail: int = 32):
    steps = []
    for rid, n in lengths.items():
        t = min(tail, n - 1) if n > 1 else 0
        if n - t > 0:
            steps.append(([(rid, 0, n - t)], []))
        for i in range(n - t, n):
            steps.append(([(rid, i, 1)], []))
        steps[-1] = (steps[-1][0], [rid])
    return steps


def schedule_portions(lengths: Dict[str, int], sizes=(7, 2, 16, 3, 2, 31, 5, 2, 64, 9, 2, 17)):
    steps = []
    k = 0
    for rid, n in lengths.items():
        i = 0
        while i < n:
            c = min(sizes[k % len(sizes)], n - i)
            k += 1
            steps.append(([(rid, i, c)], []))
            i += c
        steps[-1] = (steps[-1][0], [rid])
    return steps


def schedule_mixed(lengths: Dict[str, int], max_tokens: int, seed: int, max_live: int = 4):
    """Up to ``max_live`` requests at a time, portions of some beside single tokens of others;
    a request is admitted only while the live ones (each rounded up to 64) fit ``max_tokens``."""
    g = random.Random(seed)
    waiting = list(lengths.items())
    live: Dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, n = waiting[0]
            held = sum(roundup(lengths[r], 64) for r in live)
            if held + roundup(n, 64) > max_tokens:
                break
            live[rid] = 0
            waiting.pop(0)
        assert live, "max_tokens too small for the next request"
        entries, end = [], []
        for rid in list(live):
            done, n = live[rid], lengths[rid]
            if len(live) > 1 and g.random() < 0.2:
                continue                      # left out of this step, goes on later
            rest = n - done
            if rest > 32:
                c = min(g.choice([2, 3, 5, 8, 13, 16, 17, 31, 40]), rest - 32)
            else:
                c = 1                         # the tail is decoded token by token
            entries.append((rid, done, c))
            live[rid] = done + c
            if live[rid] == n:
                end.append(rid)
                del live[rid]
        if entries:
            steps.append((entries, end))
    return steps


def schedule_random(lengths: Dict[str, int], seed: int):
    """A schedule drawn from ``seed``: how many requests are live at a time (one to four) and so how small the pool
    is, in which order the requests come and in which order the entries of a step stand, how long the portions
    are (1 to 70 tokens, so that they end before, at and behind pages' edges), from where on a request goes token
    by token, and how often a request sits a step out.  Returns (steps, max_tokens)."""
    g = random.Random(seed)
    max_live = g.choice([1, 2, 3, 4, 4])
    order = list(lengths.items())
    g.shuffle(order)
    biggest = sorted(roundup(n, 64) for n in lengths.values())
    max_tokens = sum(biggest[-max(1, max_live - 1):]) + (64 if max_live > 1 else 0)
    tail = {rid: g.choice([0, 1, 2, 7, 32, 40]) for rid in lengths}
    skip = g.choice([0.0, 0.1, 0.3])
    waiting = list(order)
    live: Dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, n = waiting[0]
            held = sum(roundup(lengths[r], 64) for r in live)
            if held + roundup(n, 64) > max_tokens:
                break
            live[rid] = 0
            waiting.pop(0)
        assert live, "max_tokens too small for the next request"
        entries, end = [], []
        rids = list(live)
        g.shuffle(rids)
        for rid in rids:
            done, n = live[rid], lengths[rid]
            if len(live) > 1 and g.random() < skip:
                continue
            rest = n - done
            c = min(g.randint(1, 70), rest - tail[rid]) if rest > tail[rid] else 1
            entries.append((rid, done, c))
            live[rid] = done + c
            if live[rid] == n:
                end.append(rid)
                del live[rid]
        if entries:
            steps.append((entries, end))
    return steps, max_tokens


# ---- replaying a schedule through a runner -----------------------------------------------------
LENGTHS = {"A": {"a0": 5, "a1": 17, "a2": 33, "a3": 150, "a4": 97, "a5": 64},
           "B": {"b0": 1, "b1": 9, "b2": 40, "b3": 63, "b4": 120, "b5": 201},
           "C": {"c0": 3, "c1": 49, "c2": 130, "c3": 75, "c4": 25, "c5": 88},
           "D": {"d0": 7, "d1": 300, "d2": 41, "d3": 170, "d4": 96, "d5": 33},
           "E": {"e0": 2, "e1": 129, "e2": 64, "e3": 260, "e4": 31, "e5": 65}}
PAGE_SIZE = {"A": 16, "B": 8, "C": 32, "D": 16, "E": 64}


def requests_for(name: str) -> Dict[str, List[int]]:
    vocab = CONFIGS[name].vocab_size
    return {rid: random_tokens(vocab, n, seed=1000 + i) for i, (rid, n) in enumerate(LENGTHS[name].items())}


def schedule_for(name: str, mode: str):
    """(steps, max_tokens) of a replay mode for a configuration's requests."""
    lengths = LENGTHS[name]
    if mode == "mixed":
        # room for about three of the requests: pages of finished ones must be used again
        max_tokens = sum(sorted(roundup(n, 64) for n in lengths.values())[-2:]) + 64
        return schedule_mixed(lengths, max_tokens, seed=5), max_tokens
    max_tokens = max(roundup(n, 64) for n in lengths.values())
    fn = {"whole": schedule_whole, "bulk_tail": schedule_bulk_tail, "portions": schedule_portions}[mode]
    return fn(lengths), max_tokens


def run_schedule(runner, requests, steps):
    """Run a schedule asking for logits everywhere; returns {rid: [len, vocab] float32 on the host}."""
    from tempura_amd.engine.runner import StepEntry
    got = {rid: [None] * len(t) for rid, t in requests.items()}
    for entries, end in steps:
        batch = []
        for rid, start, count in entries:
            if not runner.has_request(rid):
                runner.add_request(rid)
            assert runner.num_cached(rid) == start
            batch.append(StepEntry(rid, requests[rid][start:start + count], list(range(count))))
        logits = runner.step(batch).cpu()
        row = 0
        for rid, start, count in entries:
            for i in range(count):
                got[rid][start + i] = logits[row].clone()
                row += 1
        for rid in end:
            runner.end_request(rid)
        runner.cache.check()
    return {rid: torch.stack(rows) for rid, rows in got.items()}


def first_difference(got: torch.Tensor, ref: torch.Tensor, tol: float):
    """Index of the first position whose logits differ by more than tol (relative to the largest logit), or None."""
    scale = float(ref.double().abs().max())
    err = (got.double() - ref.double()).abs().amax(dim=-1) / scale
    bad = torch.nonzero(err > tol)
    return None if bad.numel() == 0 else int(bad[0])


# ---- a far key that decides ---------------------------------------------------------------------
def plant_pointer(cfg: dict, W: Dict[str, torch.Tensor], needles: Sequence[int], probe: int, strength: float = 80.0,
                  layer: int = 0) -> Dict[str, torch.Tensor]:
    """Weights (a new dict; float64 values, to be stored in the model's type) in which every head of ``layer``'s
    attention, at a query that is the token ``probe``, scores about ``strength`` (after the scale) against the key
    of any token of ``needles``, however far back it lies; every other score stays what the random weights make it
    (a few units).  The softmax of a probe is then all but one-hot on the needle of its sequence, and a kernel
    that misses that one key (a page's edge, a split's edge, a page handed to another request) changes the
    layer's output from the needle's value row to a mixture of the others: the logits move by a large part of
    their range instead of by rounding.

    How: the rotary pair with the lowest frequency turns by a negligible angle over a few thousand positions
    (plain.rope_inv_freq), so a product of q and k components in that pair does not depend on the distance.  With
    x_t the normed embedding of token t (layer 0 sees exactly that), the k rows of that pair's first element get
    a * g added, g the shortest vector with g . x_n = 1 for every needle n, and the q rows get a * x_p / |x_p|^2,
    a^2 * scale = strength."""
    assert layer == 0, "the planted direction is made from normed embeddings, which only layer 0 sees"
    H = cfg["hidden_size"]
    nH = cfg["num_attention_heads"]
    nKV = cfg.get("num_key_value_heads", nH)
    D = cfg.get("head_dim") or H // nH
    eps = cfg.get("rms_norm_eps", 1e-5)
    out = {k: v for k, v in W.items()}
    emb = W["model.embed_tokens.weight"].double()
    wn = W["model.layers.0.input_layernorm.weight"].double()
    xs = plain.rmsnorm(emb[torch.tensor(list(needles) + [probe])], wn, eps)
    xn, xp = xs[:-1], xs[-1]
    g = xn.T @ torch.linalg.solve(xn @ xn.T, torch.ones(len(needles), dtype=torch.float64))
    gp = xp / (xp @ xp)
    a = (strength * (D ** 0.5)) ** 0.5
    d = D // 2 - 1                               # the slowest pair's first element, in the checkpoint's split-half order
    wq = W["model.layers.0.self_attn.q_proj.weight"].double().clone()
    wk = W["model.layers.0.self_attn.k_proj.weight"].double().clone()
    for h in range(nH):
        wq[h * D + d] += a * gp
    for h in range(nKV):
        wk[h * D + d] += a * g
    out["model.layers.0.self_attn.q_proj.weight"] = wq
    out["model.layers.0.self_attn.k_proj.weight"] = wk
    return out


def pointer_sequence(vocab: int, n: int, needle: int, needle_at: int, probe: int, probes_at: Sequence[int], special: Sequence[int],
                     seed: int) -> List[int]:
    """``n`` random tokens that avoid the ``special`` ids, the needle at one place and the probe at others."""
    g = random.Random(seed)
    free = [t for t in range(vocab) if t not in set(special)]
    toks = [g.choice(free) for _ in range(n)]
    toks[needle_at] = needle
    for p in probes_at:
        assert needle_at < p < n
        toks[p] = probe
    return toks


def random_arrivals(eng, cfg, W, g, seed: int, n_requests: int = 12) -> None:
    """Requests of drawn lengths (prompts of 1 to 80 tokens, 1 to 40 new ones) are added to ``eng`` between its
    steps, none to three at a time, until all are done; asserts that every request got the plain implementation's
    greedy tokens, that ``finished`` came with the last one, and that no page or request is left in the cache."""
    from tempura_amd.sampling import SamplingParams
    todo = [(random_tokens(cfg["vocab_size"], g.randint(1, 80), seed=900 + 20 * seed + i), g.randint(1, 40)) for i in range(n_requests)]
    got, asked = {}, {}
    steps = 0
    while todo or eng.has_unfinished():
        for _ in range(g.choice([0, 0, 1, 2, 3]) if eng.has_unfinished() else 1):
            if todo:
                prompt, n = todo.pop()
                rid = eng.add_request(prompt, SamplingParams(temperature=0.0, max_new_tokens=n, ignore_eos=True))
                asked[rid] = (prompt, n)
                got[rid] = []
        for rid, tok, finished in eng.step():
            got[rid].append(tok)
            assert finished == (len(got[rid]) == asked[rid][1])
        steps += 1
        assert steps < 3000, "the engine does not come to an end"
    cache = eng.runner.cache
    assert cache.free_pages() == [p.num_pages for p in cache.pools] and not cache.live_requests()
    for rid, (prompt, n) in asked.items():
        assert got[rid] == plain.greedy_generate(cfg, W, prompt, n), f"request {rid} (prompt of {len(prompt)}, {n} new tokens)"
