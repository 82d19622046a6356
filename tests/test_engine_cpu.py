"""The engine's bookkeeping on the host (CPU): with the kernel operations replaced by their plain PyTorch
stand-ins (tests/emu_ops.py), every way of cutting and batching must reproduce the plain implementation.
A difference here is a fault of the cache or the batch, not of a kernel."""
import pytest
import torch

import helpers
import plain
from emu_ops import EmuOps


@pytest.fixture(autouse=True)
def host_ops():
    from tempura_amd.kernels import ops
    ops.set_backend(EmuOps())
    yield
    ops.set_backend(None)


def _runner(tiny_dirs, name, max_tokens):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    ps = helpers.PAGE_SIZE[name]
    model = load_model(tiny_dirs.path(name, "float32"), "float32", "cpu")
    return ModelRunner(model, ps, (max_tokens + ps - 1) // ps, max_requests=4)


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_every_cutting_matches_plain(tiny_dirs, name, mode):
    cfg, W = tiny_dirs.plain_model(name)
    requests = helpers.requests_for(name)
    steps, max_tokens = helpers.schedule_for(name, mode)
    runner = _runner(tiny_dirs, name, max_tokens)
    got = helpers.run_schedule(runner, requests, steps)
    for rid, toks in requests.items():
        ref = plain.forward(cfg, W, toks)
        bad = helpers.first_difference(got[rid], ref, 1e-6)
        assert bad is None, f"{name}/{mode}: request {rid} first differs at position {bad}"
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]


def test_mixed_schedule_really_reuses_pages(tiny_dirs):
    steps, max_tokens = helpers.schedule_for("A", "mixed")
    runner = _runner(tiny_dirs, "A", max_tokens)
    seen, reused = {}, 0
    requests = helpers.requests_for("A")
    from tempura_amd.engine.runner import StepEntry
    for entries, end in steps:
        batch = []
        for rid, s, c in entries:
            if not runner.has_request(rid):
                runner.add_request(rid)
            batch.append(StepEntry(rid, requests[rid][s:s + c], []))
        runner.step(batch)
        for rid, _, _ in entries:
            for p in runner.cache.table(rid, 0):
                if p in seen and seen[p] != rid:
                    reused += 1
                seen[p] = rid
        assert max(len(e) for e, _ in steps) >= 3
        for rid in end:
            runner.end_request(rid)
    assert reused > 0, "the pool is so small that pages pass from finished requests to later ones"
    assert max(len(entries) for entries, _ in steps) == 4


def test_layer_order_is_data(tiny_dirs):
    """A run order that names a layer twice (its second call has a cache slot of its own) and lets a call read
    the cache another call wrote, against the same thing written out with the plain parts."""
    import math
    from tempura_amd.config import LayerCall, LlamaConfig
    from tempura_amd.engine.model import CausalLM
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    from tempura_amd.weights import random_weights
    cfg = LlamaConfig.from_dict(helpers.CONFIGS["A"].to_dict())
    spec = cfg.build_spec()
    spec.order = [LayerCall(0, cache=0), LayerCall(1, cache=1), LayerCall(0, cache=2), LayerCall(1, cache=1)]
    model = CausalLM(spec, torch.float32, torch.device("cpu"))
    assert model.call_writes == [True, True, True, False] and model.slots_per_group == [3]
    W = {k: v.double() for k, v in random_weights(cfg, seed=5, std=helpers.STD, norm_jitter=0.2, dtype="float32").items()}
    model.load_weights(lambda n, optional=False: W[n].float())
    runner = ModelRunner(model, 16, 8, 2)
    toks = helpers.random_tokens(cfg.vocab_size, 37, seed=9)
    runner.add_request("x")
    got = torch.cat([runner.step([StepEntry("x", toks[:20], list(range(20)))]),
                     runner.step([StepEntry("x", toks[20:], list(range(17)))])])

    T, D, nH, nKV = 37, 16, 4, 2
    inv = plain.rope_inv_freq(D, 10000.0, None)
    pos = torch.arange(T)
    h = W["model.embed_tokens.weight"][torch.tensor(toks)]
    kv_of_slot = {}
    for layer, slot, writes in [(0, 0, True), (1, 1, True), (0, 2, True), (1, 1, False)]:
        p = f"model.layers.{layer}."
        x = plain.rmsnorm(h, W[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        q = plain.rope((x @ W[p + "self_attn.q_proj.weight"].T).reshape(T, nH, D), pos, inv)
        if writes:
            k = plain.rope((x @ W[p + "self_attn.k_proj.weight"].T).reshape(T, nKV, D), pos, inv)
            v = (x @ W[p + "self_attn.v_proj.weight"].T).reshape(T, nKV, D)
            kv_of_slot[slot] = (k, v)
        k, v = kv_of_slot[slot]
        h = h + plain.attention(q, k, v, 1 / math.sqrt(D)) @ W[p + "self_attn.o_proj.weight"].T
        x = plain.rmsnorm(h, W[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        h = h + plain.swiglu_ffn(x, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])
    ref = plain.rmsnorm(h, W["model.norm.weight"], cfg.rms_norm_eps) @ W["lm_head.weight"].T
    assert helpers.rel_err(got, ref) < 1e-6


def test_step_rejects_bad_batches(tiny_dirs):
    from tempura_amd.cache import PagesExhausted
    from tempura_amd.engine.runner import StepEntry
    runner = _runner(tiny_dirs, "A", 64)
    runner.add_request("a")
    with pytest.raises(ValueError, match="not live"):
        runner.step([StepEntry("nobody", [1], [0])])
    with pytest.raises(ValueError, match="twice"):
        runner.step([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(ValueError, match="vocabulary"):
        runner.step([StepEntry("a", [256], [])])
    with pytest.raises(ValueError, match="wanted place"):
        runner.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(ValueError, match="at least one token"):
        runner.step([StepEntry("a", [], [])])
    with pytest.raises(PagesExhausted):
        runner.step([StepEntry("a", [1] * 65, [])])
    assert runner.num_cached("a") == 0 and runner.cache.free_pages() == [4]      # nothing happened
    runner.cache.check()


@pytest.mark.parametrize("fill_budget", [True, False])
def test_generate_and_preemption_on_host(tiny_dirs, fill_budget):
    """(with and without prompt portions that take up the budget nobody else uses)"""
    from tempura_amd.engine import Engine
    from tempura_amd.sampling import SamplingParams
    cfg, W = tiny_dirs.plain_model("A")
    prompts = [helpers.random_tokens(256, n, seed=700 + n) for n in (5, 17, 33, 26)]
    params = SamplingParams(temperature=0.0, max_new_tokens=12)
    kw = dict(dtype="float32", device="cpu", page_size=16, max_batch_size=4, max_num_batched_tokens=24, prefill_chunk_size=16,
              fill_budget=fill_budget)
    want = [plain.greedy_generate(cfg, W, p, 12) for p in prompts]
    roomy = Engine(tiny_dirs.path("A"), kv_pages=32, **kw)
    assert roomy.generate(prompts, params) == want
    # (the longest request alone needs all three pages; without the admission headroom, so that requests are evicted)
    tight = Engine(tiny_dirs.path("A"), kv_pages=3, admit_headroom=None, **kw)
    assert tight.generate(prompts, params) == want
    assert tight.stats()["preemptions"] > 0 and tight.runner.cache.free_pages() == [3]


def test_requests_arriving_at_random_times_get_the_plain_tokens(tiny_dirs):
    """Scheduler, cache manager and step function under requests that arrive while others run, into a pool that holds
    a third of them (the kernel operations replaced by the stand-ins): the plain implementation's greedy tokens."""
    import random
    from tempura_amd.engine import Engine
    cfg, W = tiny_dirs.plain_model("A")
    eng = Engine(tiny_dirs.path("A"), dtype="float32", device="cpu", page_size=16, kv_pages=14, max_batch_size=4,
                 max_num_batched_tokens=24, prefill_chunk_size=8)
    helpers.random_arrivals(eng, cfg, W, random.Random(3), seed=3, n_requests=8)


def test_zero_new_tokens_and_a_request_left_out_of_a_step(tiny_dirs):
    from tempura_amd.engine import Engine
    from tempura_amd.sampling import SamplingParams
    cfg, W = tiny_dirs.plain_model("A")
    prompts = [helpers.random_tokens(256, n, seed=900 + n) for n in (4, 6, 9)]
    kw = dict(dtype="float32", device="cpu", page_size=16, max_batch_size=4, kv_pages=32)
    eng = Engine(tiny_dirs.path("A"), **kw)
    outs = eng.generate(prompts, [SamplingParams(temperature=0.0, max_new_tokens=n) for n in (0, 3, 0)])
    assert outs == [[], plain.greedy_generate(cfg, W, prompts[1], 3), []]
    assert eng.stats()["generated_tokens"] == 3
    # A token budget below the number of decoding requests leaves one out of the step.  Such a step must not be
    # followed by a step queued ahead for the same requests (the one left out would wait until the others end).
    eng = Engine(tiny_dirs.path("A"), max_num_batched_tokens=32, **kw)
    eng.chain_steps = True                       # (what a GPU engine has; the decision is host logic)
    for p in prompts:
        eng.add_request(p, SamplingParams(temperature=0.0, max_new_tokens=6))
    eng.step()
    assert all(r.is_decoding for r in eng.scheduler.running) and len(eng.scheduler.running) == 3
    items = eng.scheduler.schedule()
    assert len(items) == 3 and eng._queue_next(items) is not None, "every running request decodes: the next step may be queued"
    eng.scheduler.config.max_num_batched_tokens = 2
    items = eng.scheduler.schedule()
    assert len(items) == 2 and all(it.count == 1 and it.samples for it in items)
    assert eng._queue_next(items) is None


@pytest.mark.parametrize("on_device", [False, True])
def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path, on_device):
    """A mixer defined in the tests, with per-request state and no paged cache, in an architecture of its own
    (``on_device``: the variant that finds its rows of the state through the step's device-side slots)."""
    import toy_parts
    from tempura_amd.config import load_config
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToyConfig(state_on_device=on_device)
    d = write_random_model(cfg, str(tmp_path / "toy"), seed=4, std=0.2, norm_jitter=0.1, dtype="float32")
    assert type(load_config(d)) is toy_parts.ToyConfig and load_config(d).state_on_device == on_device
    model = load_model(d, "float32", "cpu")
    assert sorted(model.state_specs) == [0, 2] and model.slots_per_group == [1]     # two state layers, one attention layer
    _, W = plain.read_model_dir(d)
    runner = ModelRunner(model, 8, 12, max_requests=3)
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=i) for i, (r, n) in enumerate({"p": 21, "q": 9, "r": 30}.items())}
    ref = {r: toy_parts.plain_toy_forward(cfg, W, t) for r, t in reqs.items()}
    steps = [([("p", 0, 6)], []), ([("p", 6, 3), ("q", 0, 8)], []), ([("p", 9, 1), ("q", 8, 1)], ["q"]),
             ([("p", 10, 1), ("r", 0, 1)], []), ([("p", 11, 1), ("r", 1, 1)], []), ([("p", 12, 9), ("r", 2, 28)], ["p", "r"])]
    got = helpers.run_schedule(runner, reqs, steps)
    for r in reqs:
        assert helpers.first_difference(got[r], ref[r], 1e-6) is None, r
    # a state slot used again starts from zero
    runner.add_request("again")
    lg = runner.step([StepEntry("again", reqs["q"], list(range(9)))])
    assert helpers.rel_err(lg, ref["q"]) < 1e-6


def test_toy_routed_ffn_and_learned_position_register_build_and_step(tmp_path):
    """A feed-forward with routing and a position encoding that is not rotary (with a tensor of its own),
    defined in the tests, in layers beside the library's rotary attention (windowed: a second cache group)
    and SwiGLU."""
    import toy_parts
    from tempura_amd.config import load_config
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToyRoutedConfig()
    d = write_random_model(cfg, str(tmp_path / "routed"), seed=6, std=0.25, norm_jitter=0.1, dtype="float32")
    assert type(load_config(d)) is toy_parts.ToyRoutedConfig
    model = load_model(d, "float32", "cpu")
    assert sorted(g.kind for g in model.cache_groups) == ["full", "window"] and not model.state_specs
    _, W = plain.read_model_dir(d)
    assert {"r.0.pos", "r.2.pos", "r.0.router", "r.1.gate"} <= set(W)
    runner = ModelRunner(model, 8, [12, 8], max_requests=3)
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=10 + i) for i, (r, n) in enumerate({"p": 21, "q": 9, "r": 30}.items())}
    ref = {r: toy_parts.plain_routed_forward(cfg, W, t) for r, t in reqs.items()}
    steps = [([("p", 0, 6)], []), ([("p", 6, 3), ("q", 0, 8)], []), ([("p", 9, 1), ("q", 8, 1), ("r", 0, 17)], ["q"]),
             ([("p", 10, 11), ("r", 17, 13)], ["p", "r"])]
    got = helpers.run_schedule(runner, reqs, steps)
    for r in reqs:
        assert helpers.first_difference(got[r], ref[r], 1e-6) is None, r
    assert runner.cache.free_pages() == [12, 8]


def test_toy_mixer_with_pages_of_its_own_layout_registers_builds_and_steps(tmp_path):
    """A mixer whose pages hold one compressed vector per token instead of keys and values of heads: its cache spec
    (a subclass defined in the tests) says what a page holds, and pools, runner and engine take it from there.  Its
    layers form a cache group of their own beside the attention layer's; pages come back and are used again."""
    import toy_parts
    from tempura_amd import Engine
    from tempura_amd.config import load_config
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToyLatentConfig()
    d = write_random_model(cfg, str(tmp_path / "latent"), seed=9, std=0.25, norm_jitter=0.1, dtype="float32")
    assert type(load_config(d)) is toy_parts.ToyLatentConfig
    model = load_model(d, "float32", "cpu")
    assert [type(g).__name__ for g in model.cache_groups] == ["LatentCacheSpec", "CacheSpec"] and model.slots_per_group == [2, 1]
    assert model.cache_groups[0].page_bytes(8, 4) == 8 * 20 * 4 and model.cache_groups[1].page_bytes(8, 4) == 2 * 2 * 8 * 16 * 4
    _, W = plain.read_model_dir(d)
    runner = ModelRunner(model, 8, [9, 9], max_requests=3)
    assert {n: tuple(t.shape) for n, t in runner.pools.kv[0].items()} == {"c": (2, 10, 8, 20)}
    assert sorted(runner.layer_caches[0].planes) == ["c"] and runner.layer_caches[0].k is None
    assert sorted(runner.layer_caches[1].planes) == ["k", "v"]
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=30 + i) for i, (r, n) in enumerate({"p": 21, "q": 9, "r": 30, "s": 12}.items())}
    ref = {r: toy_parts.plain_latent_forward(cfg, W, t) for r, t in reqs.items()}
    steps = [([("p", 0, 6)], []), ([("p", 6, 3), ("q", 0, 8)], []), ([("p", 9, 1), ("q", 8, 1), ("r", 0, 17)], ["q"]),
             ([("p", 10, 11), ("r", 17, 13)], ["p"]), ([("s", 0, 2)], ["r"]), ([("s", 2, 10)], ["s"])]     # (s takes pages that q and p gave back)
    got = helpers.run_schedule(runner, reqs, steps)
    for r in reqs:      # (the toy mixer works in float32: a few 1e-6 of rounding; a vector from a wrong page costs 1e-2 and more)
        assert helpers.first_difference(got[r], ref[r], helpers.TOL["float32"]) is None, r
    assert runner.cache.free_pages() == [9, 9]
    # the engine sizes the pools by what the specs say a page costs, and generates through them
    eng = Engine(d, dtype="float32", device="cpu", page_size=8, kv_pages=12, max_batch_size=2)
    assert eng.stats()["cache_bytes"] == 13 * (2 * 8 * 20 + 2 * 2 * 8 * 16) * 4
    # where prompts are best cut is the parts' to say: the attention layer prefers multiples of eight, the toy mixer does not care
    assert eng.scheduler.config.portion_align == 8 == model.portion_align()
    assert {type(p).__name__: p.preferred_portion_align for l in model.layers for p in l.parts() if p.category == "mixer"} == \
        {"LatentMixer": 1, "PagedAttention": 8}
    from tempura_amd import SamplingParams
    out = eng.generate([reqs["q"]], SamplingParams(temperature=0.0, max_new_tokens=3))[0]
    seq = list(reqs["q"])
    for tok in out:
        assert tok == int(torch.argmax(toy_parts.plain_latent_forward(cfg, W, seq)[-1]))
        seq.append(tok)


def test_toy_block_arrangements_with_other_parts_register_build_and_step(tmp_path):
    """Two block arrangements defined in the tests: one with norms before and after the mixer and the feed-forward
    (six named parts), one with a mixer and no feed-forward.  ``LayerSpec`` carries the parts by the names the
    arrangement gives them, so neither needs a change to the framework's files."""
    import toy_parts
    from tempura_amd.config import load_config
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToySandwichConfig()
    spec = cfg.build_spec()
    assert sorted(spec.layers[0].parts) == ["ffn", "mixer", "post_ffn_norm", "post_mixer_norm", "pre_ffn_norm", "pre_mixer_norm"]
    assert sorted(spec.layers[1].parts) == ["mixer", "norm"] and spec.layers[1].mixer.kind == "attention"
    with pytest.raises(AttributeError, match="no part named"):
        spec.layers[1].ffn
    d = write_random_model(cfg, str(tmp_path / "sandwich"), seed=8, std=0.2, norm_jitter=0.1, dtype="float32")
    assert type(load_config(d)) is toy_parts.ToySandwichConfig
    model = load_model(d, "float32", "cpu")
    # (embedding, head and the last norm's two tensors; q, k, v, o of three layers; a sandwich layer's two plain and
    # two centred norms (two tensors each) and its feed-forward; the norm of the layer without a feed-forward)
    assert model.slots_per_group == [3] and len(model.expected_weights()) == 4 + 4 * 3 + (2 + 2 * 2 + 3) * 2 + 1
    _, W = plain.read_model_dir(d)
    runner = ModelRunner(model, 8, 12, max_requests=3)
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=20 + i) for i, (r, n) in enumerate({"p": 21, "q": 9, "r": 30}.items())}
    ref = {r: toy_parts.plain_sandwich_forward(cfg, W, t) for r, t in reqs.items()}
    steps = [([("p", 0, 6)], []), ([("p", 6, 3), ("q", 0, 8)], []), ([("p", 9, 1), ("q", 8, 1), ("r", 0, 17)], ["q"]),
             ([("p", 10, 11), ("r", 17, 13)], ["p", "r"])]
    got = helpers.run_schedule(runner, reqs, steps)
    for r in reqs:
        assert helpers.first_difference(got[r], ref[r], 1e-6) is None, r
    # a spec that names parts the arrangement does not have is refused when the block is built
    from tempura_amd.config import LayerSpec
    from tempura_amd.parts import part_class
    with pytest.raises(ValueError, match="missing"):
        part_class("block", "prenorm")(LayerSpec("prenorm", {"mixer": spec.layers[1].mixer}), cfg.hidden_size, torch.float32, "cpu")


def test_forward_while_every_request_slot_is_live_and_the_waste_ratio(tiny_dirs):
    """``Engine.forward`` runs a fresh request of its own; the engine keeps one request slot back for it, so it
    works while ``max_batch_size`` requests are running, and refuses with a message that names the pages when
    the live requests leave too few.  ``stats()`` reports the share of held cache places that hold no token
    (/root/reference/engine/src/kv_cache.rs:1066-1074)."""
    from tempura_amd import Engine, SamplingParams
    from tempura_amd.cache import PagesExhausted
    cfg, W = tiny_dirs.plain_model("A")
    eng = Engine(tiny_dirs.path("A", "float32"), dtype="float32", device="cpu", page_size=16, kv_pages=8, max_batch_size=2)
    prompts = [helpers.random_tokens(256, n, seed=40 + n) for n in (5, 20)]
    for p in prompts:
        eng.add_request(p, SamplingParams(temperature=0.0, max_new_tokens=8))
    eng.step(); eng.step()
    assert len(eng.scheduler.running) == 2
    st = eng.stats()
    held = 1 * 16 + 2 * 16                       # 5 + 1 cached tokens hold one page, 20 + 1 hold two
    assert abs(st["waste_ratio"] - (1 - (6 + 21) / held)) < 1e-6
    probe = helpers.random_tokens(256, 30, seed=99)
    got = eng.forward(probe)
    ref = plain.forward(cfg, W, probe)
    assert float((got.double() - ref[-1]).abs().max() / ref.abs().max()) < 1e-6
    with pytest.raises(PagesExhausted, match="forward: a prompt of 100 tokens"):
        eng.forward(helpers.random_tokens(256, 100, seed=98))          # 7 pages, 5 are free
    while eng.has_unfinished():
        eng.step()
    assert [eng.request(i).output for i in range(2)] == [plain.greedy_generate(cfg, W, p, 8) for p in prompts]
    assert eng.runner.cache.free_pages() == [8] and eng.stats()["waste_ratio"] == 0.0


@pytest.mark.skipif(torch.cuda.is_available(), reason="needs a machine without a GPU")
def test_no_gpu_is_one_clear_error(tiny_dirs, capsys):
    """Without a GPU the engine says so in one line (it has no CPU path): from the loader, from the entry point
    and, with exit status 2, from the command line."""
    from tempura_amd import Engine
    from tempura_amd.cli import main
    from tempura_amd.engine.loading import NoDeviceError, load_model
    d = tiny_dirs.path("A", "float32")
    with pytest.raises(NoDeviceError, match="no GPU is visible"):
        load_model(d, "float32", "cuda:0")
    with pytest.raises(NoDeviceError, match="no CPU path"):
        Engine(d, dtype="float32")
    assert main(["run", "--model", d, "--prompt-ids", "1,2,3", "--max-new-tokens", "2"]) == 2
    assert "no GPU is visible" in capsys.readouterr().err
