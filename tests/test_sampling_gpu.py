"""The sampling kernels against the reference's rules written out plainly in Python."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def plain_typical(x, typical_p):
    """Keep the tokens whose information -ln p is nearest the entropy, nearest first (ties by index), until
    their mass exceeds typical_p; the others become -inf (/root/reference/kernels/src/sampler_chain.rs:87-141)."""
    p = torch.softmax(x, 0)
    pos = p > 0
    ent = -(p[pos] * p[pos].log()).sum()
    score = torch.full_like(p, math.inf)
    score[pos] = (-p[pos].log() - ent).abs()
    order = torch.argsort(score, stable=True)
    out = torch.full_like(x, -math.inf)
    cum = 0.0
    for i in order.tolist():
        if not pos[i]:
            break
        cum += float(p[i])
        out[i] = x[i]
        if cum > typical_p:
            break
    return out


def plain_sample(logits, temperature, top_k, top_p, min_p, r, typical_p=1.0):
    """temperature scale, min-p, typical-p, top-k, softmax over the kept, top-p prefix, renormalise, walk the
    probabilities in INDEX order and return the first index whose cumulative sum exceeds r
    (/root/reference/kernels/src/sampling.rs:192-333, min-p /root/reference/kernels/src/sampler_chain.rs:54-80)."""
    x = logits.double().clone()
    if temperature == 0:
        mx = x.max()
        return int(torch.nonzero(x == mx).max())
    if temperature != 1.0:
        x = x / temperature
    if min_p > 0:
        x[x < x.max() + math.log(min_p)] = -math.inf
    if typical_p < 1.0:
        x = plain_typical(x, typical_p)
    V = x.numel()
    order = torch.argsort(x, descending=True, stable=True)
    k = V if top_k <= 0 else min(top_k, V)
    keep = order[:k]
    p = torch.zeros(V, dtype=torch.float64)
    p[keep] = torch.exp(x[keep] - x.max())
    p /= p.sum()
    if top_p < 1.0:
        o2 = torch.argsort(p, descending=True, stable=True)
        cs = torch.cumsum(p[o2], 0)
        cut = int(torch.nonzero(cs >= top_p)[0]) + 1
        mask = torch.zeros(V, dtype=torch.bool)
        mask[o2[:cut]] = True
        p[~mask] = 0
        p /= p.sum()
    cs = torch.cumsum(p, 0)
    hit = torch.nonzero(cs > r)
    return int(hit[0]) if hit.numel() else V - 1


def _sample(logits, temperature, top_k, top_p, min_p, r, typical_p=1.0, settled=None):
    from tempura_amd.kernels import ops
    ops.set_backend(None)
    m, v = logits.shape
    work = torch.empty(m, v, device=DEV)
    full = lambda a: [a] * m if not isinstance(a, (list, tuple)) else list(a)
    return ops.sample(logits.to(DEV), work, full(temperature), full(top_k), full(top_p), full(min_p), full(r), full(typical_p),
                      settled=settled).tolist()


@pytest.mark.parametrize("vocab", [16, 301, 4099, 50021])    # (the largest: whole rounds of sixteen loads and their rests)
@pytest.mark.parametrize("temperature,top_k,top_p,min_p", [(1.0, 0, 1.0, 0.0), (0.8, 0, 1.0, 0.0), (1.0, 5, 1.0, 0.0), (0.7, 50, 0.9, 0.0),
                                                            (1.3, 0, 0.5, 0.0), (1.0, 0, 1.0, 0.1), (0.9, 40, 0.95, 0.05), (0.0, 50, 0.9, 0.0)])
def test_sample_matches_plain_rules(vocab, temperature, top_k, top_p, min_p):
    g = torch.Generator().manual_seed(vocab + int(top_k))
    logits = torch.randn(24, vocab, generator=g) * 2.5
    rs = [(i + 0.37) / 24 for i in range(24)]
    got = _sample(logits, temperature, top_k, top_p, min_p, rs)
    want = [plain_sample(logits[i], temperature, top_k, top_p, min_p, rs[i]) for i in range(24)]
    assert got == want


@pytest.mark.parametrize("vocab", [16, 301, 4099])
@pytest.mark.parametrize("temperature,top_k,top_p,min_p,typical_p", [(1.0, 0, 1.0, 0.0, 0.9), (0.8, 0, 1.0, 0.0, 0.5), (1.2, 20, 0.9, 0.0, 0.7),
                                                                      (1.0, 0, 1.0, 0.05, 0.3), (1.0, 0, 1.0, 0.0, 0.0)])
def test_typical_p_matches_plain_rules(vocab, temperature, top_k, top_p, min_p, typical_p):
    g = torch.Generator().manual_seed(7 * vocab + int(typical_p * 10))
    logits = torch.randn(24, vocab, generator=g) * 2.5
    rs = [(i + 0.61) / 24 for i in range(24)]
    got = _sample(logits, temperature, top_k, top_p, min_p, rs, typical_p)
    want = [plain_sample(logits[i], temperature, top_k, top_p, min_p, rs[i], typical_p) for i in range(24)]
    assert got == want


def test_typical_p_and_tie_cuts_on_a_long_row():
    """The cuts that go through a row in index order (typical_p's last ties, surplus ties of top_k and top_p) on rows
    long enough for every wave to read several rounds of sixteen groups, with many equal values."""
    vocab = 50021
    g = torch.Generator().manual_seed(50021)
    spread = torch.randn(6, vocab, generator=g) * 2.5
    levels = (torch.randn(6, vocab, generator=g) * 2.0).round() * 0.5       # ties everywhere
    rs = [(i + 0.61) / 6 for i in range(6)]
    for logits in (spread, levels):
        for t, k, p, ty in [(1.0, 0, 1.0, 0.9), (0.8, 0, 0.9, 0.5), (1.0, 300, 0.9, 1.0), (1.0, 300, 1.0, 1.0), (1.0, 0, 0.7, 1.0)]:
            got = _sample(logits, t, k, p, 0.0, rs, ty)
            want = [plain_sample(logits[i], t, k, p, 0.0, rs[i], ty) for i in range(6)]
            assert got == want, (t, k, p, ty)


def test_typical_p_drops_a_likely_but_untypical_token():
    # token 0 holds 30 % of the mass, 700 others share the rest: the entropy is near the information of a tail
    # token, so token 0 is the LEAST typical and leaves first, although every other filter would keep it
    V = 701
    lg = torch.full((1, V), math.log(0.7 / 700))
    lg[0, 0] = math.log(0.3)
    rows = lg.repeat(64, 1)
    rs = [(i + 0.5) / 64 for i in range(64)]
    assert 0 in _sample(rows, 1.0, 0, 1.0, 0.0, rs)                      # without the filter a draw below 0.3 takes it
    got = _sample(rows, 1.0, 0, 1.0, 0.0, rs, 0.5005)
    assert 0 not in got
    # equal scores are admitted in index order: a mass above 0.5005 needs 501 of the 700 tail tokens
    assert got == [plain_sample(lg[0], 1.0, 0, 1.0, 0.0, r, 0.5005) for r in rs]
    assert 490 <= max(got) <= 501 and min(got) >= 1
    # all logits equal: every token is equally typical, the first ones in index order whose mass exceeds 0.255 stay
    flat = torch.zeros(32, 100)
    got = _sample(flat, 1.0, 0, 1.0, 0.0, [(i + 0.5) / 32 for i in range(32)], 0.255)
    assert max(got) == 25 and min(got) == 0


def test_logprobs_of_the_filtered_distribution():
    """Per row: the chosen token's log-probability and the most probable survivors, from the distribution after
    temperature and filters (/root/reference/engine/src/model.rs:497-526)."""
    from tempura_amd.sampling import Sampler, SamplingParams
    g = torch.Generator().manual_seed(11)
    V = 4099
    lg = (torch.randn(5, V, generator=g) * 3).to(DEV)
    ps = [SamplingParams(temperature=0.0), SamplingParams(temperature=0.7, top_k=40, top_p=0.9, seed=5),
          SamplingParams(temperature=1.0, top_k=0, seed=6), SamplingParams(temperature=1.3, top_k=3, seed=7),
          SamplingParams(temperature=1.0, top_k=0, min_p=0.2, typical_p=0.6, seed=8)]
    s = Sampler(V, DEV, default_seed=0)
    toks, recs = s.sample(lg, ps, [0, 1, 2, 3, 4], [[]] * 5, [[]] * 5, top_n=5)
    assert toks == s.sample(lg, ps, [0, 1, 2, 3, 4], [[]] * 5, [[]] * 5)
    for r, (p, tok, rec) in enumerate(zip(ps, toks, recs)):
        x = lg[r].double().cpu()
        if p.temperature not in (0.0, 1.0):
            x = x / p.temperature
        if p.min_p > 0:
            x[x < x.max() + math.log(p.min_p)] = -math.inf
        if p.typical_p < 1:
            x = plain_typical(x, p.typical_p)
        if p.top_k > 0:
            x[x < torch.topk(x, p.top_k).values[-1]] = -math.inf
        pr = torch.softmax(x, 0)
        if p.top_p < 1:
            o = torch.argsort(pr, descending=True, stable=True)
            cut = int(torch.nonzero(torch.cumsum(pr[o], 0) >= p.top_p)[0]) + 1
            keep = torch.zeros(V, dtype=torch.bool)
            keep[o[:cut]] = True
            pr[~keep] = 0
            pr /= pr.sum()
        assert rec.token_id == tok and abs(rec.logprob - math.log(float(pr[tok]))) < 1e-4
        n = min(5, int((pr > 0).sum()))
        want = torch.topk(pr, n)
        assert [i for i, _ in rec.top_logprobs] == want.indices.tolist()
        assert all(abs(got - math.log(float(w))) < 1e-4 for (_, got), w in zip(rec.top_logprobs, want.values))
    assert len(recs[3].top_logprobs) == 3, "three survivors of top_k = 3, although five were asked for"


def test_greedy_ties_and_fallthrough():
    lg = torch.zeros(3, 100)
    lg[0, 5] = lg[0, 70] = 3.0                       # tie: the later index wins (model.rs:459-473)
    lg[1] = -math.inf                                 # nothing to choose from: the last index (sampling.rs:496-520)
    lg[2, 9] = 1.0
    assert _sample(lg, [0.0, 1.0, 0.0], 0, 1.0, 0.0, 0.5) == [70, 99, 9]


def test_temperature_to_zero_converges_to_argmax():
    g = torch.Generator().manual_seed(1)
    lg = torch.randn(16, 500, generator=g)
    got = _sample(lg, 1e-4, 0, 1.0, 0.0, [i / 16 + 0.01 for i in range(16)])
    assert got == lg.argmax(dim=1).tolist()


def test_top_k_keeps_at_most_k_even_with_ties():
    lg = torch.zeros(1, 64)                           # all equal: ties at the cut are admitted in index order
    seen = set()
    for i in range(200):
        seen.update(_sample(lg, 1.0, 5, 1.0, 0.0, (i + 0.5) / 200))
    assert seen == {0, 1, 2, 3, 4}
    lg[0, 40:] = 1.0
    seen = set()
    for i in range(200):
        seen.update(_sample(lg, 1.0, 30, 1.0, 0.0, (i + 0.5) / 200))
    assert seen == set(range(40, 64)) | set(range(6))


def _sample_one_block(logits, temperature, top_k, top_p, min_p, r):
    """The same rows through the path of one block per row (a report of probabilities asks for it)."""
    from tempura_amd.kernels import ops
    ops.set_backend(None)
    m, v = logits.shape
    work = torch.empty(m, v, device=DEV)
    info = torch.empty(m, 4, device=DEV)
    full = lambda a: [a] * m if not isinstance(a, (list, tuple)) else list(a)
    return ops.sample(logits.to(DEV), work, full(temperature), full(top_k), full(top_p), full(min_p), full(r), full(1.0), info).tolist()


@pytest.mark.parametrize("vocab", [4099, 50021, 128256])
def test_small_top_k_and_top_p_from_the_candidates_of_the_pieces(vocab):
    """A row cut by a small top_k, or by top_p alone when the prefix it keeps is short, is settled from the candidates
    that the 32 pieces of the row hand over; the answer is that of the one-block path in every case, and that of the
    plain rules.  Rows that cannot be settled so (nearly equal logits) are left to the one block per row."""
    g = torch.Generator().manual_seed(vocab)
    m = 16
    rs = [(i + 0.41) / m for i in range(m)]
    rows = {
        "random": torch.randn(m, vocab, generator=g) * 3.0,
        "few levels": (torch.randn(m, vocab, generator=g) * 2.0).round(),          # many ties, also at the cut
        "flat": torch.zeros(m, vocab),                                             # every piece has too many candidates
        "one piece holds them all": torch.randn(m, vocab, generator=g) * 0.1,
        "mostly -inf": torch.full((m, vocab), -math.inf),
        "nan": torch.randn(m, vocab, generator=g) * 3.0,
    }
    per = -(-vocab // 32)
    rows["one piece holds them all"][:, 3 * per:3 * per + 100] += 10.0            # the k largest lie in one piece
    rows["one piece holds them all"][:, 3 * per + 7] = rows["one piece holds them all"][:, 3 * per + 9]
    rows["mostly -inf"][:, [5, vocab // 2, vocab - 1]] = torch.tensor([0.3, 1.0, 0.3])
    rows["mostly -inf"][m - 1] = -math.inf                                          # nothing at all: the last index
    rows["nan"][:, ::7] = math.nan
    for name, lg in rows.items():
        for t, k, p, mp in [(1.0, 1, 1.0, 0.0), (0.8, 5, 1.0, 0.0), (0.7, 50, 0.9, 0.0), (1.0, 128, 0.95, 0.0), (0.9, 40, 0.95, 0.3),
                            (1.0, 128, 1.0, 0.0), (1.0, 129, 0.9, 0.0), (0.8, 0, 0.9, 0.0), (1.0, 0, 0.5, 0.0), (1.0, 0, 0.95, 0.1),
                            (1.2, 0, 0.999, 0.0), (0.6, 0, 0.01, 0.0)]:
            if k >= vocab:
                continue
            settled = []
            got = _sample(lg, t, k, p, mp, rs, settled=settled)
            assert got == _sample_one_block(lg, t, k, p, mp, rs), (name, t, k, p, mp)
            if name == "random" and (0 < k <= 128 or (k == 0 and p <= 0.9)):
                assert settled == [1] * m, (name, t, k, p, mp)
            if name == "flat" or k > 128:
                assert settled == [0] * m, (name, t, k, p, mp)
            if name != "nan":
                want = [plain_sample(lg[i], t, k, p, mp, rs[i]) for i in range(0, m - 1, 5)]
                assert got[:m - 1:5] == want, (name, t, k, p, mp)
            if name == "mostly -inf":
                assert got[m - 1] == vocab - 1
    # rows of both kinds in one call
    lg = rows["few levels"]
    ks = [(3, 200, 0, 64)[i % 4] for i in range(m)]
    ts = [(1.0, 0.0, 0.9)[i % 3] for i in range(m)]
    ps = [(0.9, 1.0, 0.7, 0.9, 0.5)[i % 5] for i in range(m)]
    assert _sample(lg, ts, ks, ps, 0.0, rs) == _sample_one_block(lg, ts, ks, ps, 0.0, rs)


def test_frequencies_follow_softmax():
    """Chi-square of 20,000 draws against softmax(logits / T) on a vocabulary of 16."""
    from tempura_amd.sampling import uniform_draw
    g = torch.Generator().manual_seed(2)
    lg = torch.randn(1, 16, generator=g) * 1.5
    p = torch.softmax(lg[0].double() / 0.8, 0)
    n = 20000
    rows = lg.expand(2000, 16).contiguous()
    counts = torch.zeros(16)
    for b in range(n // 2000):
        rs = [uniform_draw(123, b * 2000 + i) for i in range(2000)]
        counts += torch.bincount(torch.tensor(_sample(rows, 0.8, 0, 1.0, 0.0, rs)), minlength=16)
    chi2 = float(((counts - n * p) ** 2 / (n * p)).sum())
    assert chi2 < 45.0, f"chi-square {chi2:.1f} with 15 degrees of freedom"        # p ~ 1e-4


def test_penalties():
    from tempura_amd.kernels import ops
    ops.set_backend(None)
    lg = torch.tensor([[1.0, -2.0, 3.0, 0.5, -1.0], [1.0, -2.0, 3.0, 0.5, -1.0]])
    d = lg.clone().to(DEV)
    # row 0: token 2 generated twice, token 1 once; tokens 0 and 1 in the repetition window
    ops.apply_penalties(d, [0, 0, 0], [2, 1, 0], [2, 1, 0], [0, 1, 1], [0.5, 0.0], [0.25, 0.0], [2.0, 1.0])
    want = lg.clone()
    want[0, 2] -= 0.25 * 2 + 0.5           # frequency * count + presence (kernel-api/src/lib.rs:292-308)
    want[0, 1] = (want[0, 1] - (0.25 + 0.5)) * 2.0      # non-positive logits are multiplied (sampler_chain.rs:239-243)
    want[0, 0] = want[0, 0] / 2.0                        # positive ones divided
    assert torch.allclose(d.cpu(), want)


def test_sampler_class_rows_with_different_options():
    from tempura_amd.sampling import Sampler, SamplingParams
    g = torch.Generator().manual_seed(3)
    lg = torch.randn(3, 300, generator=g).to(DEV)
    s = Sampler(300, torch.device(DEV), default_seed=9)
    ps = [SamplingParams(temperature=0.0), SamplingParams(temperature=0.9, top_k=10, seed=4),
          SamplingParams(temperature=1.0, top_k=0, presence_penalty=100.0)]
    out = s.sample(lg, ps, [0, 3, 1], [[], [], []], [[], [], [int(lg[2].argmax())]])
    assert out[0] == int(lg[0].argmax())
    assert out[1] in lg[1].topk(10).indices.tolist()
    assert out[2] != int(lg[2].argmax()), "a huge presence penalty bans the generated token"
    assert s.sample(lg, ps, [0, 3, 1], [[], [], []], [[], [], [int(lg[2].argmax())]]) == out


def test_temperature_zero_with_repetition_penalty_does_not_depend_on_the_batch():
    """A temperature-0 row with a repetition penalty takes the argmax of the penalised logits whether it is alone,
    beside a sampled row, or asked for log-probabilities."""
    from tempura_amd.sampling import Sampler, SamplingParams
    V = 300
    lg = torch.zeros(2, V)
    lg[0, 17], lg[0, 40] = 5.0, 4.0             # the penalty (5.0 / 1.3 < 4.0) moves the maximum from 17 to 40
    lg[1] = torch.randn(V, generator=torch.Generator().manual_seed(4))
    lg = lg.to(DEV)
    s = Sampler(V, torch.device(DEV), default_seed=1)
    greedy = SamplingParams(temperature=0.0, repeat_penalty=1.3)
    assert not greedy.is_greedy and SamplingParams(temperature=0.0).is_greedy
    hist = [3, 17, 9]
    alone = s.sample(lg[:1], [greedy], [0], [hist], [[]])
    beside = s.sample(lg, [greedy, SamplingParams(temperature=0.9, seed=3)], [0, 0], [hist, []], [[], []])
    with_lp, recs = s.sample(lg[:1], [greedy], [0], [hist], [[]], top_n=2)
    assert alone == [40] and beside[0] == 40 and with_lp == [40] and recs[0].token_id == 40
    assert s.sample(lg[:1], [SamplingParams(temperature=0.0)], [0], [hist], [[]]) == [17]
    assert float(lg[0, 17]) == 5.0, "the caller's logits are left as they were"
