"""Generation through the entry point on the GPU: greedy tokens against the plain implementation,
temperature sampling, preemption under a tiny pool, the command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

import helpers
import plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _engine(tiny_dirs, name, dtype="float32", **kw):
    from tempura_amd.engine import Engine
    from tempura_amd.kernels import ops
    ops.set_backend(None)
    args = dict(page_size=helpers.PAGE_SIZE[name], kv_pages=64, max_batch_size=4, max_num_batched_tokens=48,
                prefill_chunk_size=16)
    args.update(kw)
    return Engine(tiny_dirs.path(name, dtype), dtype=dtype, **args)


@pytest.mark.parametrize("name,prompt_lens,n_new", [("A", [5, 17, 33], 16), ("B", [1, 9, 40, 63, 120], 24)])
def test_greedy_generation_matches_plain(tiny_dirs, name, prompt_lens, n_new):
    from tempura_amd.sampling import SamplingParams
    cfg, W = tiny_dirs.plain_model(name)
    prompts = [helpers.random_tokens(cfg["vocab_size"], n, seed=200 + i) for i, n in enumerate(prompt_lens)]
    eng = _engine(tiny_dirs, name)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=n_new))
    for p, o in zip(prompts, outs):
        assert o == plain.greedy_generate(cfg, W, p, n_new)
    st = eng.stats()
    assert st["generated_tokens"] == n_new * len(prompts) and st["graph_steps"] > 0
    assert eng.runner.cache.free_pages() == [64] * len(eng.runner.cache.pools)
    # forward(): the last position's logits of a fresh request
    lg = eng.forward(prompts[1])
    assert helpers.rel_err(lg, plain.forward(cfg, W, prompts[1])[-1]) <= helpers.TOL["float32"]


def test_bfloat16_greedy_generation_runs_and_is_repeatable(tiny_dirs):
    from tempura_amd.sampling import SamplingParams
    prompts = [helpers.random_tokens(300, n, seed=300 + n) for n in (3, 50, 21)]
    a = _engine(tiny_dirs, "C", "bfloat16").generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=20))
    b = _engine(tiny_dirs, "C", "bfloat16", use_graph=False).generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=20))
    assert a == b and all(len(o) == 20 for o in a)


def test_bfloat16_greedy_generation_against_plain(tiny_dirs):
    """The bfloat16 engine generates greedily; at every step the plain implementation (float64, on the same
    bfloat16 weights, fed the engine's own tokens so far) must rank the engine's token first, or within the
    rounding noise of bfloat16 storage of its own first: the token's plain logit may lie below the plain maximum
    by no more than twice that noise (``helpers.plain_reference``'s bound, in logit units)."""
    from tempura_amd.sampling import SamplingParams
    for name in ("C", "D"):
        cfg, W = tiny_dirs.plain_model(name, "bfloat16")
        prompts = [helpers.random_tokens(cfg["vocab_size"], n, seed=300 + n) for n in (3, 50, 21)]
        outs = _engine(tiny_dirs, name, "bfloat16").generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=20))
        agree = total = 0
        for p, o in zip(prompts, outs):
            assert len(o) == 20
            exact, bound = helpers.plain_reference(cfg, W, p + o, "bfloat16")
            slack = bound * float(exact.abs().max())
            for i, tok in enumerate(o):
                row = exact[len(p) + i - 1]
                assert float(row.max() - row[tok]) <= slack, \
                    f"{name}: token {i} of the bfloat16 engine is {float(row.max() - row[tok]):.3e} below the plain maximum (slack {slack:.3e})"
                agree += int(tok == int(torch.nonzero(row == row.max()).max()))
                total += 1
        assert agree >= 0.9 * total, f"{name}: only {agree} of {total} tokens are the plain implementation's first choice"


def test_baseline_tiny_workloads(tmp_path):
    """The two tiny workloads as they are specified: configuration A with a position limit of 128 (prompts of 5, 17
    and 33 ids, 16 greedy steps, pages of 16) and B with a limit of 256 (prompts of 1, 9, 40, 63 and 120 ids, 24
    steps at temperature 0.8 from seed 2, pages of 8), float32, weights N(0, 0.02) from seeds 0 and 1 with norm
    weights 1.  Greedy tokens equal the plain implementation's; sampled tokens are the same alone and in the
    batch and each is the token that the plain sampling rules give on the plain implementation's logits with the
    same uniform number; and a request that reaches the position limit ends there with the reason max_model_len."""
    from tempura_amd.config import LlamaConfig
    from tempura_amd.engine import Engine
    from tempura_amd.kernels import ops
    from tempura_amd.sampling import SamplingParams
    from tempura_amd.weights import write_random_model
    ops.set_backend(None)
    a = LlamaConfig.from_dict({**helpers.CONFIGS["A"].to_dict(), "max_position_embeddings": 128})
    b = LlamaConfig.from_dict({**helpers.CONFIGS["B"].to_dict(), "max_position_embeddings": 256})
    da = write_random_model(a, str(tmp_path / "a"), seed=0, std=0.02, dtype="float32")
    db = write_random_model(b, str(tmp_path / "b"), seed=1, std=0.02, dtype="float32")
    ca, Wa = plain.read_model_dir(da)
    prompts = [helpers.random_tokens(256, n, seed=i) for i, n in enumerate((5, 17, 33))]
    eng = Engine(da, dtype="float32", page_size=16, kv_pages=24, max_batch_size=3)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=16))
    assert outs == [plain.greedy_generate(ca, Wa, p, 16) for p in prompts]
    # 120 prompt ids and room for 8 more: the request ends at the limit of 128 positions
    rid = eng.add_request(helpers.random_tokens(256, 120, seed=9), SamplingParams(temperature=0.0, max_new_tokens=50, ignore_eos=True))
    while eng.has_unfinished():
        eng.step()
    assert eng.request(rid).finish_reason == "max_model_len" and len(eng.request(rid).output) == 8
    with pytest.raises(ValueError, match="no room"):
        eng.add_request(helpers.random_tokens(256, 128, seed=9), SamplingParams(max_new_tokens=1))
    cb, Wb = plain.read_model_dir(db)
    prompts = [helpers.random_tokens(384, n, seed=10 + i) for i, n in enumerate((1, 9, 40, 63, 120))]
    params = SamplingParams(temperature=0.8, seed=2, max_new_tokens=24)
    eng = Engine(db, dtype="float32", page_size=8, kv_pages=96, max_batch_size=5)
    outs = eng.generate(prompts, params)
    assert all(len(o) == 24 for o in outs)
    assert outs[3] == Engine(db, dtype="float32", page_size=8, kv_pages=32, max_batch_size=1).generate([prompts[3]], params)[0]
    # every sampled token is the one that the plain rules give on the plain implementation's logits with the same
    # uniform number (draw i of the stream with seed 2; /root/reference/kernels/src/sampling.rs:229-333): top-k 50
    # (the default), temperature 0.8, index-order walk.  The engine's logits are float32, so a draw that lands within
    # 1e-5 of a step of the cumulative sum may fall on either side; anything else must agree exactly.
    import numpy as np
    from tempura_amd.sampling import uniform_draw
    from test_sampling_gpu import plain_sample
    checked = 0
    for p, o in zip(prompts, outs):
        logits = plain.forward(cb, Wb, p + o)
        for i, tok in enumerate(o):
            row = logits[len(p) + i - 1]
            r = float(np.float32(uniform_draw(2, i)))
            want = plain_sample(row, 0.8, 50, 1.0, 0.0, r)
            if tok != want:
                near = {plain_sample(row, 0.8, 50, 1.0, 0.0, min(max(r + d, 0.0), 1.0 - 1e-9)) for d in (-1e-5, 1e-5)}
                assert tok in near, f"prompt of {len(p)}: token {i} is {tok}, the plain rules give {want}"
            checked += 1
    assert checked == 5 * 24


def test_preemption_by_recompute_keeps_tokens(tiny_dirs):
    """So few pages that running requests are preempted: every request still gets exactly the tokens it gets
    with plenty of pages, in greedy and in seeded temperature sampling."""
    from tempura_amd.sampling import SamplingParams
    prompts = [helpers.random_tokens(256, n, seed=400 + n) for n in (30, 45, 38, 20)]
    for params in (SamplingParams(temperature=0.0, max_new_tokens=40),
                   SamplingParams(temperature=0.8, top_k=0, seed=2, max_new_tokens=40)):
        roomy = _engine(tiny_dirs, "A", kv_pages=64)
        want = roomy.generate(prompts, params)
        assert roomy.stats()["preemptions"] == 0
        tight = _engine(tiny_dirs, "A", kv_pages=11)        # 176 tokens of cache for 333 tokens of work
        got = tight.generate(prompts, params)
        assert tight.stats()["preemptions"] > 0
        assert got == want
        assert tight.runner.cache.free_pages() == [11]


@pytest.mark.parametrize("name,seed", [("A", 0), ("A", 1), ("A", 2), ("C", 3), ("D", 4), ("E", 5)])
def test_requests_arriving_at_random_times_get_the_plain_tokens(tiny_dirs, name, seed):
    """Twelve requests of drawn lengths (prompts of 1 to 80 tokens, 1 to 40 new ones) arrive while others run, into an
    engine whose pool holds a third of them: prompts in portions beside decoding requests, steps queued ahead of
    the host, requests finishing at different times, admission with headroom and, where it comes to that,
    preemption; also with a window whose pages go back while a request runs (C) and with pages of 64 (E).  Every
    request gets the plain implementation's greedy tokens, and in the end no page is held."""
    import random
    cfg, W = tiny_dirs.plain_model(name)
    g = random.Random(seed)
    tokens = g.choice([224, 320, 448])
    eng = _engine(tiny_dirs, name, kv_pages=tokens // helpers.PAGE_SIZE[name], max_num_batched_tokens=g.choice([24, 48, 96]),
                  prefill_chunk_size=g.choice([8, 16, 40]))
    helpers.random_arrivals(eng, cfg, W, g, seed)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("D", "bfloat16"), ("C", "bfloat16")])
def test_four_hundred_requests_with_aborts_leave_nothing_behind(tiny_dirs, name, dtype):
    """A long run of the whole engine on a pool that holds a handful of requests: 400 requests of drawn lengths and
    sampling options (greedy, temperature, top-k, top-p, min-p, repetition penalty) arrive in bursts, one in twenty
    steps aborts a running or waiting request, requests are preempted and recomputed.  No comparison of tokens here
    (the other tests have it): every token is a token of the vocabulary, the cache manager's invariants hold
    throughout, every request ends, and in the end no page and no request slot is held."""
    import random
    from tempura_amd.sampling import SamplingParams
    vocab = helpers.CONFIGS[name].vocab_size
    g = random.Random(7)
    ps = helpers.PAGE_SIZE[name]
    eng = _engine(tiny_dirs, name, dtype=dtype, kv_pages=640 // ps, max_batch_size=6, max_num_batched_tokens=64, prefill_chunk_size=24)
    live, finished, aborted, added, steps = set(), 0, 0, 0, 0
    while added < 400 or eng.has_unfinished():
        for _ in range(g.choice([0, 0, 1, 1, 2, 4])):
            if added < 400:
                params = SamplingParams(temperature=g.choice([0.0, 0.7, 1.0]), top_k=g.choice([0, 5, 50]), top_p=g.choice([1.0, 0.9]),
                                        min_p=g.choice([0.0, 0.05]), repeat_penalty=g.choice([1.0, 1.1]), seed=g.randint(0, 99),
                                        max_new_tokens=g.randint(1, 60), ignore_eos=True)
                live.add(eng.add_request(helpers.random_tokens(vocab, g.randint(1, 150), seed=added), params))
                added += 1
        if live and g.random() < 0.05:
            rid = g.choice(sorted(live))
            eng.abort(rid)
            live.discard(rid)
            aborted += 1
        for rid, tok, fin in eng.step():
            assert 0 <= tok < vocab and rid in live
            if fin:
                live.discard(rid)
                finished += 1
        steps += 1
        if steps % 50 == 0:
            eng.runner.cache.check()
        assert steps < 20000, "the engine does not come to an end"
    cache = eng.runner.cache
    assert not live and finished + aborted == 400 and aborted > 20
    assert cache.free_pages() == [p.num_pages for p in cache.pools] and not cache.live_requests()
    assert eng.stats()["preemptions"] > 0 and eng.runner.graph_steps > 500


def test_temperature_sampling_seeded(tiny_dirs):
    from tempura_amd.sampling import SamplingParams
    prompts = [helpers.random_tokens(384, n, seed=500 + n) for n in (1, 9, 40)]
    eng = _engine(tiny_dirs, "B")
    p = SamplingParams(temperature=0.8, top_k=0, seed=2, max_new_tokens=24)
    a = eng.generate(prompts, p)
    b = _engine(tiny_dirs, "B").generate(prompts, p)
    c = _engine(tiny_dirs, "B").generate(prompts, SamplingParams(temperature=0.8, top_k=0, seed=3, max_new_tokens=24))
    assert a == b, "same seed, same tokens"
    assert a != c, "another seed, other tokens"
    # alone or in a batch: the same tokens (draws depend on the seed and the draw's number only)
    alone = _engine(tiny_dirs, "B").generate([prompts[2]], p)
    assert alone[0] == a[2]


def test_generate_with_logprobs(tiny_dirs):
    """Greedy: the tokens of ``generate``, and records that agree with a softmax of the plain implementation's
    logits over the top_k kept tokens (the reference reports the filtered distribution,
    /root/reference/engine/src/model.rs:497-526)."""
    from tempura_amd.sampling import SamplingParams
    cfg, W = tiny_dirs.plain_model("A")
    prompts = [helpers.random_tokens(256, n, seed=700 + n) for n in (5, 17)]
    p = SamplingParams(temperature=0.0, top_k=8, max_new_tokens=6)
    tokens, records = _engine(tiny_dirs, "A").generate_with_logprobs(prompts, p, top_n=3)
    assert tokens == _engine(tiny_dirs, "A").generate(prompts, p)
    for prompt, toks, recs in zip(prompts, tokens, records):
        assert [r.token_id for r in recs] == toks
        seq = list(prompt)
        for tok, rec in zip(toks, recs):
            lg = plain.forward(cfg, W, seq)[-1].double()
            kept = torch.topk(lg, 8)
            lp = torch.log_softmax(kept.values, 0)
            assert rec.top_logprobs[0][0] == tok == int(kept.indices[0])
            assert [i for i, _ in rec.top_logprobs] == kept.indices[:3].tolist()
            assert abs(rec.logprob - float(lp[0])) < 1e-4
            for (_, got), want in zip(rec.top_logprobs, lp[:3].tolist()):
                assert abs(got - want) < 1e-4
            seq.append(tok)
    # requests with and without records in one batch
    eng = _engine(tiny_dirs, "A")
    r0 = eng.add_request(prompts[0], p, logprobs_top_n=0)
    r1 = eng.add_request(prompts[1], p)
    while eng.has_unfinished():
        eng.step()
    assert eng.request(r0).output == tokens[0] and eng.request(r1).output == tokens[1]
    assert len(eng.request(r0).logprobs) == 6 and eng.request(r1).logprobs == []
    assert all(r.top_logprobs == [] for r in eng.request(r0).logprobs)


def test_generate_with_callback_and_abort(tiny_dirs):
    from tempura_amd.sampling import SamplingParams
    prompts = [helpers.random_tokens(256, n, seed=710 + n) for n in (5, 17, 30)]
    p = SamplingParams(temperature=0.0, max_new_tokens=12)
    full = _engine(tiny_dirs, "A").generate(prompts, p)
    seen = {0: [], 1: [], 2: []}

    def on_token(i, tok):
        seen[i].append(tok)
        return not (i == 1 and len(seen[1]) == 4)        # the second prompt stops after four tokens

    eng = _engine(tiny_dirs, "A")
    out = eng.generate_with_callback(prompts, p, on_token)
    assert out == [full[0], full[1][:4], full[2]] and [seen[i] for i in range(3)] == out
    assert all(pool.num_free == pool.num_pages for pool in eng.runner.cache.pools)
    # one token from given logits, by the same sampler
    lg = torch.randn(256)
    assert eng.sample_from_logits(lg, SamplingParams(temperature=0.0)) == int(lg.argmax())
    t = eng.sample_from_logits(lg, SamplingParams(temperature=0.9, top_k=5, seed=1), draw_index=3)
    assert t in torch.topk(lg, 5).indices.tolist()
    assert t == eng.sample_from_logits(lg, SamplingParams(temperature=0.9, top_k=5, seed=1), draw_index=3)


def test_eos_and_length_limits(tiny_dirs):
    from tempura_amd.sampling import SamplingParams
    cfg, W = tiny_dirs.plain_model("A")
    prompt = helpers.random_tokens(256, 12, seed=600)
    ref = plain.greedy_generate(cfg, W, prompt, 10)
    eng = _engine(tiny_dirs, "A")
    out = eng.generate([prompt], SamplingParams(temperature=0.0, max_new_tokens=10, eos_token_id=[ref[3]]))[0]
    stop = ref.index(ref[3])
    assert out == ref[:stop + 1], "generation stops after the first EOS token, which is kept"
    out = eng.generate([prompt], SamplingParams(temperature=0.0, max_new_tokens=10, eos_token_id=[ref[3]], ignore_eos=True))[0]
    assert out == ref


def test_steps_queued_ahead_change_nothing(tiny_dirs):
    """While all requests decode, the engine queues the next step before it has read this step's tokens.  The
    tokens and the final state are those of an engine that does not: with requests
    of different lengths, one that ends on an EOS token (its row in the step already queued is dropped), seeded
    temperature sampling with penalties, a request added and one aborted on the way."""
    from tempura_amd.sampling import SamplingParams
    cfg, W = tiny_dirs.plain_model("A")
    prompts = [helpers.random_tokens(256, n, seed=700 + n) for n in (9, 30, 4, 17)]
    ref = [plain.greedy_generate(cfg, W, p, 24) for p in prompts]
    eos = ref[1][9]                                           # request 1 stops early
    params = [SamplingParams(temperature=0.0, max_new_tokens=24),
              SamplingParams(temperature=0.0, max_new_tokens=24, eos_token_id=[eos]),
              SamplingParams(temperature=0.0, max_new_tokens=7),
              SamplingParams(temperature=0.9, top_k=20, seed=5, repeat_penalty=1.2, presence_penalty=0.3, max_new_tokens=24)]

    def run(chain):
        eng = _engine(tiny_dirs, "A", chain_steps=chain)
        rids = [eng.add_request(p, sp) for p, sp in zip(prompts, params)]
        events, calls = [], 0
        while eng.has_unfinished():
            events.append(eng.step())
            calls += 1
            if calls == 12:
                rids.append(eng.add_request(prompts[0][:5], SamplingParams(temperature=0.0, max_new_tokens=6)))
            if calls == 20:
                eng.abort(rids[0])
        outs = [list(eng.request(r).output) for r in rids]
        assert eng.runner.cache.free_pages() == [64]
        return outs, events, eng.stats()

    outs0, events0, st0 = run(False)
    outs1, events1, st1 = run(True)
    assert st0["chained_steps"] == 0 and st1["chained_steps"] > 10
    assert outs1 == outs0
    for outs, events in ((outs0, events0), (outs1, events1)):      # every token was reported once, in order
        seen = {}
        for call in events:
            for rid, tok, _done in call:
                seen.setdefault(rid, []).append(tok)
        assert [seen.get(i, []) for i in range(len(outs))] == outs
    assert outs1[1] == ref[1][: ref[1].index(eos) + 1] and outs1[2] == ref[2][:7]
    assert st1["generated_tokens"] == st0["generated_tokens"]


def test_command_line(tiny_dirs, tmp_path):
    cfg, W = tiny_dirs.plain_model("A")
    model = tiny_dirs.path("A", "float32")
    tempura = os.path.join(ROOT, "bin", "tempura")
    p = subprocess.run([sys.executable, tempura, "inspect", model, "--json"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr
    info = json.loads(p.stdout)
    assert info["hidden_size"] == 64 and info["kv_heads"] == 2 and info["architecture"] == "LlamaForCausalLM"
    prompt = helpers.random_tokens(256, 7, seed=601)
    p = subprocess.run([sys.executable, tempura, "run", "--model", model, "--dtype", "float32", "--prompt-ids",
                        ",".join(map(str, prompt)), "--max-new-tokens", "6", "--temperature", "0", "--kv-blocks", "16",
                        "--max-batch-size", "2", "--stats"], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    rec = json.loads(p.stdout.strip().splitlines()[-1])
    assert rec["output_ids"] == plain.greedy_generate(cfg, W, prompt, 6) and rec["finish_reason"] == "length"
    assert '"stats"' in p.stderr
    # --dump-logits: the logits after the last token of every prompt, float32 little-endian, against the plain implementation
    prompts = [prompt, helpers.random_tokens(256, 21, seed=602)]
    ids = tmp_path / "ids.txt"
    ids.write_text("\n".join(" ".join(map(str, q)) for q in prompts) + "\n")
    out = tmp_path / "logits.f32"
    # (the model folder as the positional argument, as in `tempura inspect`)
    p = subprocess.run([sys.executable, tempura, "run", model, "--dtype", "float32", "--prompt-file", str(ids),
                        "--max-new-tokens", "2", "--temperature", "0", "--kv-blocks", "16", "--max-batch-size", "2",
                        "--dump-logits", str(out)], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    import numpy as np
    got = torch.from_numpy(np.fromfile(out, dtype="<f4").reshape(2, 256).copy()).double()
    for row, q in zip(got, prompts):
        want = plain.forward(cfg, W, q)
        assert float((row - want[-1]).abs().max() / want.abs().max()) <= helpers.float32_bound(cfg)
    p = subprocess.run([sys.executable, tempura, "profile", "--model", model, "--dtype", "float32", "--prompt-len", "12",
                        "--batch", "2", "--decode-steps", "2", "--kv-blocks", "16", "--max-batch-size", "2", "--json"],
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    rep = json.loads(p.stdout.strip().splitlines()[-1])
    assert rep["prefill"] and rep["decode"] and any(r[0] == "tp_paged_attention" for r in rep["decode"])


def test_profile_times_every_call_and_reports_the_residual_stream(tiny_dirs):
    """``Engine.profile``: the step of the prompts makes the calls the model's layers make (one attention call a
    layer), the statistics of the residual stream before every layer are the plain implementation's, and the
    engine generates afterwards as if nothing had happened."""
    import math
    from tempura_amd.engine import Engine
    from tempura_amd.sampling import SamplingParams
    cfg, W = tiny_dirs.plain_model("A")
    eng = Engine(tiny_dirs.path("A", "float32"), dtype="float32", page_size=16, kv_pages=24, max_batch_size=3)
    prompt = helpers.random_tokens(cfg["vocab_size"], 9, seed=77)
    params = SamplingParams(temperature=0.0, max_new_tokens=5)
    before = eng.generate([prompt], params)
    rep = eng.profile(prompt_len=21, batch=2, decode_steps=3, layer_stats=True, seed=5)
    L = cfg["num_hidden_layers"]
    calls = {name: n for name, n, _, _ in rep["prefill"]}
    assert calls["tp_paged_attention"] == L and sum(n for name, n in calls.items() if name.startswith("tp_linear")) >= 4 * L and all(us > 0 for _, _, us, _ in rep["prefill"])
    assert abs(sum(share for *_, share in rep["prefill"]) - 1.0) < 1e-2
    assert {name: n for name, n, _, _ in rep["decode"]}["tp_paged_attention"] == 3 * L
    # the residual stream of both prompts, from the plain implementation's formulas
    import random
    g = random.Random(5)
    prompts = [[g.randrange(cfg["vocab_size"]) for _ in range(21)] for _ in range(2)]
    get = lambda name: W[name].double()
    inv = plain.rope_inv_freq(cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"],
                              cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))
    hs = [get("model.embed_tokens.weight")[torch.tensor(p)] for p in prompts]
    assert len(rep["layers"]) == L + 1
    for l in range(L + 1):
        h = torch.cat(hs)
        i, mean, var, top = rep["layers"][l]
        assert i == l
        assert math.isclose(mean, float(h.mean()), rel_tol=1e-3, abs_tol=1e-6)
        assert math.isclose(var, float(h.var(unbiased=False)), rel_tol=1e-3)
        assert math.isclose(top, float(h.abs().max()), rel_tol=1e-3)
        if l < L:
            hs = [plain.decoder_layer(cfg, get, l, h1, torch.arange(21), inv) for h1 in hs]
    assert eng.generate([prompt], params) == before
    assert eng.runner.cache.free_pages() == [p.num_pages for p in eng.runner.cache.pools]


def test_model_width_layer_against_plain(tmp_path):
    """One layer with the widths of Llama-3.1-8B (hidden 4096, 32 heads of 128 in 8 groups, intermediate 14336;
    a vocabulary of 8,192 keeps the folder at half a gigabyte) against the plain float64 implementation, which
    shares nothing with the kernels: a prompt of 600 tokens whole, in uneven portions, and with its last 32
    tokens one by one through the graph, in float32 and in bfloat16 (weights N(0, 0.02), stored as bfloat16)."""
    from tempura_amd.config import LlamaConfig, RopeScaling
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    from tempura_amd.kernels import ops
    from tempura_amd.weights import write_random_model
    ops.set_backend(None)
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=1, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, vocab_size=8192, max_position_embeddings=131072,
                      rms_norm_eps=1e-5, rope_theta=500000.0, rope_scaling=RopeScaling("llama3", 8.0, 1.0, 4.0, 8192),
                      tie_word_embeddings=False)
    folder = str(tmp_path / "wide")
    write_random_model(cfg, folder, seed=3, std=0.02, dtype="bfloat16")
    pc, W = plain.read_model_dir(folder)
    toks = helpers.random_tokens(8192, 600, seed=1)
    ref = plain.forward(pc, W, toks)
    cuts = {"whole": [(0, 600)], "portions": [(0, 300), (300, 17), (317, 2), (319, 160), (479, 121)],
            "tail": [(0, 568)] + [(i, 1) for i in range(568, 600)]}
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 2e-2)):
        model = load_model(folder, dtype, "cuda:0")
        for mode, steps in cuts.items():
            runner = ModelRunner(model, 16, 48, max_requests=2, use_graph=(mode == "tail"))
            runner.add_request("x")
            got = torch.cat([runner.step([StepEntry("x", toks[s: s + n], list(range(n)))]).cpu().clone() for s, n in steps])
            err = helpers.rel_err(got, ref)
            assert err <= tol, f"{dtype}/{mode}: {err:.3e} from the plain implementation, first at {helpers.first_difference(got, ref, tol)}"
        del model
        torch.cuda.empty_cache()


def _wide_config(layers, vocab):
    from tempura_amd.config import LlamaConfig, RopeScaling
    return LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=layers, num_attention_heads=32,
                       num_key_value_heads=8, head_dim=128, vocab_size=vocab, max_position_embeddings=131072,
                       rms_norm_eps=1e-5, rope_theta=500000.0, rope_scaling=RopeScaling("llama3", 8.0, 1.0, 4.0, 8192),
                       tie_word_embeddings=False)


def test_model_width_mixed_schedule_against_plain(tmp_path):
    """Two layers with the widths of Llama-3.1-8B under the mixed schedule: up to four live requests, portions of
    some beside single decoded tokens of others, the last 32 tokens of each one by one (decode-only steps replay
    the graph), and so few pages that finished requests' pages are used again; float32 and bfloat16 against the
    plain float64 implementation.  The q and k projections are doubled (scores four times those of N(0, 0.02)
    weights: a standard deviation of about 6.5 over a few hundred keys), so that attention is sharply peaked.
    And every request holds one key that decides (``helpers.plant_pointer``): at its probe positions all of the
    first layer's attention sits on one far key, at a page's edge, the first key or anywhere, so that a kernel
    that loses this one key moves those logits by most of their range, far above what bfloat16 explains; the
    test works out both numbers and compares the probes against the tighter one."""
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.kernels import ops
    from tempura_amd.weights import random_weights, write_safetensors
    ops.set_backend(None)
    cfg = _wide_config(2, 8192)
    W = random_weights(cfg, seed=4, std=0.02, dtype="bfloat16")
    for name in W:
        if name.endswith("q_proj.weight") or name.endswith("k_proj.weight"):
            W[name] = (W[name].float() * 2.0).to(torch.bfloat16)
    needles, probe = [8000, 8001, 8002], 8003
    planted = helpers.plant_pointer(json.loads(cfg.to_json()), W, needles, probe, strength=100.0)
    for name in ("model.layers.0.self_attn.q_proj.weight", "model.layers.0.self_attn.k_proj.weight"):
        W[name] = planted[name].to(torch.bfloat16)
    del planted
    folder = tmp_path / "wide2"
    folder.mkdir()
    (folder / "config.json").write_text(cfg.to_json())
    write_safetensors(str(folder / "model.safetensors"), W.items())
    del W
    pc, PW = plain.read_model_dir(str(folder))
    # request: (length, needle, its place, probes: in portions and among the last 32 tokens, decoded one by one)
    layout = {"w0": (150, 8000, 15, [16, 60, 130, 149]), "w1": (97, 8001, 0, [1, 50, 96]), "w2": (210, 8002, 16, [17, 100, 190, 209]),
              "w3": (64, 8000, 31, [32, 63]), "w4": (131, 8001, 64, [65, 100, 130]), "w5": (40, 8002, 7, [8, 39])}
    lengths = {rid: n for rid, (n, *_rest) in layout.items()}
    requests = {rid: helpers.pointer_sequence(8192, n, needle, at, probe, probes, needles + [probe], seed=300 + i)
                for i, (rid, (n, needle, at, probes)) in enumerate(layout.items())}
    max_tokens = 256 + 192 + 64                 # room for about three requests: pages must come back and be used again
    steps = helpers.schedule_mixed(lengths, max_tokens, seed=9)
    assert max(len(e) for e, _ in steps) >= 3 and any(len(e) > 1 and all(c == 1 for _, _, c in e) for e, _ in steps)
    missed = {}
    for rid, (n, needle, at, probes) in layout.items():
        lost = list(requests[rid])
        lost[at] = 11
        missed[rid] = plain.forward(pc, PW, lost)[torch.tensor(probes)]
    for dtype in ("float32", "bfloat16"):
        variants = (None,) if dtype == "float32" else (None, plain.as_bfloat16)
        outs = plain.forward_many(pc, PW, [requests[rid] for rid in layout], variants)
        model = load_model(str(folder), dtype, "cuda:0")
        runner = ModelRunner(model, 16, max_tokens // 16, max_requests=4, use_graph=True)
        got = helpers.run_schedule(runner, requests, steps)
        assert runner.graph_steps > 0 and not runner.cache.live_requests()
        for (rid, (n, needle, at, probes)), res in zip(layout.items(), outs):
            exact = res[0]
            scale = float(exact.abs().max())
            rows = torch.tensor(probes)
            if dtype == "float32":
                bound = probe_bound = helpers.float32_bound(pc)
            else:
                bound = helpers.BF16_FACTOR * helpers.rel_err(res[1], exact)
                probe_bound = helpers.BF16_FACTOR * float((res[1][rows] - exact[rows]).abs().max()) / scale
            err = helpers.rel_err(got[rid], exact)
            assert err <= bound, f"{dtype}: request {rid} differs from the plain implementation by {err:.3e} (bound {bound:.3e}), " \
                                 f"first at {helpers.first_difference(got[rid], exact, bound)}"
            cost = float((missed[rid] - exact[rows]).abs().amax(dim=-1).min()) / scale
            assert cost >= 10 * probe_bound, f"{rid}: losing the needle moves a probe's logits by {cost:.2e}, the bound is {probe_bound:.2e}"
            perr = float((got[rid][rows].double() - exact[rows]).abs().max()) / scale
            assert perr <= probe_bound, f"{dtype}: request {rid}: probes off by {perr:.2e} (bound {probe_bound:.2e}; a lost needle costs {cost:.2e})"
        del model, runner
        torch.cuda.empty_cache()


def test_full_depth_model_against_plain_streamed():
    """All 32 layers of the Llama-3.1-8B preset (vocabulary 128,256), weights made in device memory, under a mixed
    schedule of three requests (portions, single tokens, pages used again): the float32 engine and the bfloat16
    engine against the plain float64 implementation, which gets every tensor from the same generator, one at a
    time (``fill_normal`` has the bits of its numpy twin, tests/plain_random.py), so that no layer's weights are
    ever held twice."""
    from tempura_amd.config import PRESETS, LlamaConfig
    from tempura_amd.engine.loading import random_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.kernels import ops
    import plain_random
    ops.set_backend(None)
    cfg = LlamaConfig.from_dict(PRESETS["llama-3.1-8b"].to_dict())
    cfg.validate()
    seed, std = 6, 0.02
    pc = json.loads(cfg.to_json())
    expected = None

    def get(name):
        """The tensor as the device generator makes it (bfloat16 values), widened on the host."""
        info = expected[name]
        if info.init == "ones":
            return torch.ones(info.shape, dtype=torch.float64)
        t = ops.fill_normal(torch.empty(info.shape, dtype=torch.bfloat16, device="cuda:0"), plain_random.tensor_key(seed, name), 0.0, std)
        return t.cpu().double()

    lengths = {"f0": 96, "f1": 40, "f2": 70}
    requests = {rid: helpers.random_tokens(cfg.vocab_size, n, seed=400 + i) for i, (rid, n) in enumerate(lengths.items())}
    max_tokens = 128 + 64
    steps = helpers.schedule_mixed(lengths, max_tokens, seed=3)
    refs = None
    for dtype in ("float32", "bfloat16"):
        model = random_model(cfg, seed=seed, dtype=dtype, device="cuda:0", std=std, values_as="bfloat16")
        if refs is None:
            expected = model.expected_weights()
            both = plain.forward_many(pc, get, list(requests.values()), [None, plain.as_bfloat16])      # one pass over the weights
            exact = {rid: both[i][0] for i, rid in enumerate(requests)}
            noisy = {rid: both[i][1] for i, rid in enumerate(requests)}
            refs = {"float32": {rid: (exact[rid], helpers.float32_bound(pc)) for rid in requests},
                    "bfloat16": {rid: (exact[rid], helpers.BF16_FACTOR * helpers.rel_err(noisy[rid], exact[rid])) for rid in requests}}
        runner = ModelRunner(model, 16, max_tokens // 16, max_requests=4, use_graph=True)
        got = helpers.run_schedule(runner, requests, steps)
        for rid, (ex, bound) in refs[dtype].items():
            err = helpers.rel_err(got[rid], ex)
            assert err <= bound, f"{dtype}: request {rid} differs from the plain implementation by {err:.3e} (bound {bound:.3e}), " \
                                 f"first at {helpers.first_difference(got[rid], ex, bound)}"
        del model, runner
        torch.cuda.empty_cache()


def test_model_sized_layers_bfloat16_against_float32():
    """Two layers with the sizes of Llama-3.1-8B (hidden 4096, 32 heads of 128 in 8 groups, intermediate 14336,
    vocabulary 128256) and the same weights in both precisions: the bfloat16 engine (pipelined products of
    2,200 rows in one step: 256 x 256 and 256 x 128 tiles side by side, the long-step rotation kernels; the
    decode products with the norm carried by them, k-blocked rows, LDS attention, graphs) against the float32 engine's plain-FMA kernels, portion by
    portion and token by token.  The weights have the scale of trained checkpoints (N(0, 0.02)); the rounding of
    bfloat16 operands then costs about 1e-2 of the largest logit at this width, with the matrix-core kernels
    and with the general ones alike (at N(0, 0.05) both reach 3.5e-2: the scores get ten times sharper)."""
    from tempura_amd.config import PRESETS, LlamaConfig
    from tempura_amd.engine.loading import random_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    from tempura_amd.kernels import ops
    ops.set_backend(None)
    cfg = LlamaConfig.from_dict(PRESETS["llama-3.1-8b"].to_dict())
    cfg.num_hidden_layers = 2
    cfg.validate()
    prompts = {r: helpers.random_tokens(cfg.vocab_size, n, seed=500 + n) for r, n in (("a", 2100), ("b", 70), ("c", 23), ("d", 5))}
    tails = {r: helpers.random_tokens(cfg.vocab_size, 6, seed=600 + i) for i, r in enumerate(prompts)}
    logits = {}
    for dtype in ("float32", "bfloat16"):
        model = random_model(cfg, seed=3, dtype=dtype, device="cuda:0", std=0.02, values_as="bfloat16")
        runner = ModelRunner(model, 16, 160, max_requests=4, use_graph=(dtype == "bfloat16"))
        got = {r: [] for r in prompts}
        for r, toks in prompts.items():
            runner.add_request(r)
        # portions of different sizes in one step, then every request decoding together
        lg = runner.step([StepEntry(r, toks, [len(toks) - 1]) for r, toks in prompts.items()])
        for i, r in enumerate(prompts):
            got[r].append(lg[i].float().cpu())
        for t in range(6):
            lg = runner.step([StepEntry(r, [tails[r][t]], [0]) for r in prompts])
            for i, r in enumerate(prompts):
                got[r].append(lg[i].float().cpu())
        if dtype == "bfloat16":
            assert runner.graph_steps == 6
        logits[dtype] = {r: torch.stack(v) for r, v in got.items()}
        del runner, model
        torch.cuda.empty_cache()
    for r in prompts:
        err = helpers.rel_err(logits["bfloat16"][r], logits["float32"][r].double())
        assert err <= helpers.TOL["bfloat16"], f"request {r}: bfloat16 differs from float32 by {err:.3e}"


def test_a_captured_step_padded_to_more_rows_gives_the_bits_of_the_eager_step():
    """Decode steps replay graphs captured for a power of two of rows; 75 requests run as 128 rows there and as 75
    rows without graphs.  The products choose their tiles and the parts of K by the rows counted in whole blocks, so
    that both give the same bits (two layers of the width of Llama-3.2-3B: with random weights the logits lie close
    together, and a different order of additions moves tokens at once)."""
    import random
    from tempura_amd.config import PRESETS, LlamaConfig
    from tempura_amd.engine import Engine
    from tempura_amd.kernels import ops
    from tempura_amd.sampling import SamplingParams
    ops.set_backend(None)
    cfg = LlamaConfig.from_dict(PRESETS["llama-3.2-3b"].to_dict())
    cfg.num_hidden_layers = 2
    cfg.vocab_size = 8192
    cfg.validate()
    g = random.Random(3)
    prompts = [[g.randrange(cfg.vocab_size) for _ in range(g.choice([40, 64, 90]))] for _ in range(75)]
    outs = {}
    for graph in (True, False):
        eng = Engine(cfg, random_weights=True, seed=11, max_batch_size=128, max_seq_len=256, kv_pages=800, use_graph=graph)
        outs[graph] = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=8, ignore_eos=True))
        assert (eng.stats()["graph_steps"] > 0) == graph
        del eng
        torch.cuda.empty_cache()
    assert outs[True] == outs[False]
