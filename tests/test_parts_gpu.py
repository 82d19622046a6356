"""Each part of a layer alone on the GPU against the plain formulas, at sizes other than the models',
and a toy mixer with state of its own, defined in the tests, registered, built and stepped."""
import math

import pytest
import torch

import helpers
import plain

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture(autouse=True)
def real_kernels():
    from tempura_amd.kernels import ops
    ops.set_backend(None)


def _ctx(q_lens, ctx_lens, page_size, tables, slots):
    """A hand-made step context for one cache group."""
    from tempura_amd.engine.runner import StepContext
    c = StepContext()
    R = len(q_lens)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    c.num_tokens, c.num_requests = cu[-1], R
    c.positions = i32([p for n, cl in zip(q_lens, ctx_lens) for p in range(cl - n, cl)])
    c.token_req = i32([r for r, n in enumerate(q_lens) for _ in range(n)])
    c.cu_seqlens, c.context_lens = i32(cu), i32(ctx_lens)
    c.block_tables, c.slot_mapping = [i32(tables)], [i32(slots)]
    c.state_slots = i32(list(range(R)))
    c.max_q_len, c.max_context_len, c.num_single = max(q_lens), max(ctx_lens), sum(1 for n in q_lens if n == 1)
    c.page_size = page_size
    c.q_starts, c.q_lens, c.ctx_lens, c.state_slot_list = cu[:-1], list(q_lens), list(ctx_lens), list(range(R))
    return c


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from tempura_amd.config import PartSpec
    from tempura_amd.parts import build_part
    g = torch.Generator().manual_seed(0)
    part = build_part("norm", PartSpec("rmsnorm", {"eps": 2e-3}, {"weight": "w"}), 72, dtype, DEV)
    w = 1 + 0.5 * torch.randn(72, generator=g)
    part.load_weights(lambda n, optional=False: w)
    h = torch.randn(5, 72, generator=g) * 0.05
    got = part.forward(h.to(DEV))
    assert got.dtype == dtype
    ref = plain.rmsnorm(h.double(), w.double(), 2e-3)
    assert helpers.rel_err(got.cpu(), ref) < (1e-6 if dtype == torch.float32 else 5e-3)


def test_rotary_part_table():
    from tempura_amd.config import PartSpec
    from tempura_amd.parts import build_part
    sc = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 64}
    part = build_part("position", PartSpec("rope", {"head_dim": 48, "theta": 25000.0, "scaling": sc}), 80, torch.float32, DEV)
    inv, rot, fac = part.rotary()
    assert rot == 48 and fac == 1.0 and inv.dtype == torch.float64
    assert torch.allclose(inv.cpu(), plain.rope_inv_freq(48, 25000.0, sc), rtol=1e-14)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,d,hidden,window", [(4, 2, 16, 64, None), (6, 3, 32, 80, 20), (5, 1, 24, 56, None)])
def test_attention_part(dtype, heads, kv, d, hidden, window):
    """The mixer alone: two requests (one with a cached prefix written by an earlier call), shuffled pages."""
    from tempura_amd.cache import LayerCache
    from tempura_amd.config import PartSpec
    from tempura_amd.parts import build_part
    g = torch.Generator().manual_seed(1)
    ps, pages = 8, 12
    spec = PartSpec("attention", {"num_heads": heads, "num_kv_heads": kv, "head_dim": d, "scale": 1 / math.sqrt(d),
                                  "window": window, "position": PartSpec("rope", {"head_dim": d, "theta": 1e4, "scaling": None})},
                    {"q": "q", "k": "k", "v": "v", "o": "o"})
    part = build_part("mixer", spec, hidden, dtype, DEV)
    W = {"q": torch.randn(heads * d, hidden, generator=g) * 0.2, "k": torch.randn(kv * d, hidden, generator=g) * 0.2,
         "v": torch.randn(kv * d, hidden, generator=g) * 0.2, "o": torch.randn(hidden, heads * d, generator=g) * 0.2}
    W = {k: v.to(dtype).float() for k, v in W.items()}
    part.load_weights(lambda n, optional=False: W[n])
    assert part.cache_spec().kind == ("window" if window else "full")
    kc = torch.zeros(pages + 1, kv, ps, d, dtype=dtype, device=DEV)
    vc = torch.zeros(pages + 1, kv, d, ps, dtype=dtype, device=DEV)
    cache = LayerCache(0, {"k": kc, "v": vc}, True, ps, None)
    xa = (torch.randn(30, hidden, generator=g)).to(dtype)      # request a: 19 tokens cached first, then 11
    xb = (torch.randn(7, hidden, generator=g)).to(dtype)
    ta, tb = [5, 2, 9, 0], [7, 11]                              # shuffled pages
    slots = lambda table, lo, hi: [table[p // ps] * ps + p % ps for p in range(lo, hi)]
    res = torch.zeros(19, hidden, device=DEV)
    part.forward(xa[:19].to(DEV), _ctx([19], [19], ps, [ta], slots(ta, 0, 19)), cache, res)
    res = torch.ones(18, hidden, device=DEV)                   # the mixer ADDS into the residual stream
    bt = [ta, tb + [pages, pages]]
    part.forward(torch.cat([xa[19:], xb]).to(DEV), _ctx([11, 7], [30, 7], ps, bt, slots(ta, 19, 30) + slots(tb, 0, 7)), cache, res)

    def ref(x):
        T = x.shape[0]
        xd = x.double()
        inv = plain.rope_inv_freq(d, 1e4, None)
        q = plain.rope((xd @ W["q"].double().T).reshape(T, heads, d), torch.arange(T), inv)
        k = plain.rope((xd @ W["k"].double().T).reshape(T, kv, d), torch.arange(T), inv)
        v = (xd @ W["v"].double().T).reshape(T, kv, d)
        return plain.attention(q, k, v, 1 / math.sqrt(d), window) @ W["o"].double().T
    want = torch.cat([ref(xa)[19:], ref(xb)]) + 1.0
    assert helpers.rel_err(res.cpu(), want) < (2e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ffn_part(dtype):
    from tempura_amd.config import PartSpec
    from tempura_amd.parts import build_part
    g = torch.Generator().manual_seed(2)
    part = build_part("ffn", PartSpec("swiglu", {"intermediate_size": 136}, {"gate": "g", "up": "u", "down": "d"}), 80, dtype, DEV)
    W = {"g": torch.randn(136, 80, generator=g) * 0.2, "u": torch.randn(136, 80, generator=g) * 0.2, "d": torch.randn(80, 136, generator=g) * 0.2}
    W = {k: v.to(dtype).float() for k, v in W.items()}
    part.load_weights(lambda n, optional=False: W[n])
    x = torch.randn(9, 80, generator=g).to(dtype)
    res = torch.full((9, 80), 2.0, device=DEV)
    part.forward(x.to(DEV), None, res)
    want = plain.swiglu_ffn(x.double(), W["g"].double(), W["u"].double(), W["d"].double()) + 2.0
    assert helpers.rel_err(res.cpu(), want) < (1e-5 if dtype == torch.float32 else 2e-2)


def test_embedding_and_head_parts():
    from tempura_amd.config import PartSpec
    from tempura_amd.parts import part_class
    g = torch.Generator().manual_seed(3)
    E = torch.randn(301, 40, generator=g)
    emb = part_class("embedding", "embedding")(PartSpec("embedding", {}, {"weight": "e"}), 40, torch.float32, DEV, 301)
    emb.load_weights(lambda n, optional=False: E)
    tok = torch.tensor([300, 0, 17], dtype=torch.int32, device=DEV)
    assert torch.equal(emb.forward(tok).cpu(), E[[300, 0, 17]])
    head = part_class("lm_head", "lm_head")(PartSpec("lm_head", {"tied": True}, {"weight": "h"}), 40, torch.float32, DEV, 301)
    head.load_weights(lambda n, optional=False: None, emb)
    assert head.weight.data_ptr() == emb.weight.data_ptr()
    x = torch.randn(2, 40, generator=g)
    assert helpers.rel_err(head.forward(x.to(DEV)).cpu(), x.double() @ E.double().T) < 1e-5


def test_block_part(tiny_dirs):
    """The pre-norm arrangement alone: h += mixer(norm(h)); h += ffn(norm(h)) — one layer of config C."""
    from tempura_amd.cache import LayerCache
    from tempura_amd.config import LlamaConfig
    from tempura_amd.parts import part_class
    cfg = LlamaConfig.from_dict(helpers.CONFIGS["C"].to_dict())
    _, W = tiny_dirs.plain_model("C")
    ls = cfg.build_spec().layers[1]                       # a full-attention layer
    block = part_class("block", ls.block)(ls, cfg.hidden_size, torch.float32, DEV)
    block.load_weights(lambda n, optional=False: W[n].float())
    g = torch.Generator().manual_seed(4)
    T, ps = 21, 8
    h = torch.randn(T, cfg.hidden_size, generator=g)
    kc = torch.zeros(5, 3, ps, 48, device=DEV)
    vc = torch.zeros(5, 3, 48, ps, device=DEV)
    hd = h.clone().to(DEV)
    table = [3, 1, 0]
    block.forward(hd, _ctx([T], [T], ps, [table], [table[p // ps] * ps + p % ps for p in range(T)]), LayerCache(0, {"k": kc, "v": vc}, True, ps, None))
    p = "model.layers.1."
    x = plain.rmsnorm(h.double(), W[p + "input_layernorm.weight"], cfg.rms_norm_eps)
    inv = plain.rope_inv_freq(48, cfg.rope_theta, cfg.to_dict()["rope_scaling"])
    q = plain.rope((x @ W[p + "self_attn.q_proj.weight"].T).reshape(T, 6, 48), torch.arange(T), inv)
    k = plain.rope((x @ W[p + "self_attn.k_proj.weight"].T).reshape(T, 3, 48), torch.arange(T), inv)
    v = (x @ W[p + "self_attn.v_proj.weight"].T).reshape(T, 3, 48)
    ref = h.double() + plain.attention(q, k, v, 48 ** -0.5) @ W[p + "self_attn.o_proj.weight"].T
    x = plain.rmsnorm(ref, W[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
    ref = ref + plain.swiglu_ffn(x, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])
    assert helpers.rel_err(hd.cpu(), ref) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_with_state_on_the_gpu(tmp_path, dtype):
    """Registered, built and stepped without a change to the framework: a stateful mixer from the tests beside
    attention layers that use the HIP kernels, portions and single tokens of three requests mixed."""
    import toy_parts
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToyConfig()
    d = write_random_model(cfg, str(tmp_path / "toy"), seed=4, std=0.2, norm_jitter=0.1, dtype=dtype)
    model = load_model(d, dtype, "cuda:0")
    _, W = plain.read_model_dir(d)
    runner = ModelRunner(model, 8, 12, max_requests=3, use_graph=True)
    assert not runner.use_graph, "a part that loops on the host keeps decode steps out of the graph"
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=i) for i, (r, n) in enumerate({"p": 21, "q": 9, "r": 30}.items())}
    steps = [([("p", 0, 6)], []), ([("p", 6, 3), ("q", 0, 8)], []), ([("p", 9, 1), ("q", 8, 1), ("r", 0, 17)], ["q"]),
             ([("p", 10, 11), ("r", 17, 13)], ["p", "r"])]
    got = helpers.run_schedule(runner, reqs, steps)
    for r, t in reqs.items():
        ref = toy_parts.plain_toy_forward(cfg, W, t)
        assert helpers.rel_err(got[r], ref) < helpers.TOL[dtype], r
    if dtype == "float32":
        # and through the entry point (which then neither replays graphs nor queues steps ahead)
        from tempura_amd.engine import Engine
        from tempura_amd.sampling import SamplingParams
        eng = Engine(model, dtype=dtype, page_size=8, kv_pages=24, max_batch_size=3)
        assert not eng.chain_steps
        outs = eng.generate([reqs["q"], reqs["p"][:5]], SamplingParams(temperature=0.0, max_new_tokens=6))
        for prompt, out in zip([reqs["q"], reqs["p"][:5]], outs):
            seq = list(prompt)
            for tok in out:         # greedy by the plain implementation, token by token
                assert tok == int(torch.argmax(toy_parts.plain_toy_forward(cfg, W, seq)[-1]))
                seq.append(tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_with_state_in_captured_steps(tmp_path, dtype):
    """Per-request state and captured decode steps together: the stateful toy mixer that finds its rows through the
    step's device-side slots declares itself safe to capture, and a model with it decodes through replayed graphs.
    The schedule holds what could go wrong there: a request whose first token comes in a captured step (its state
    row must be cleared first, also when another request left it dirty), the step that captures a graph (run once
    eagerly before the capture: the state must not advance twice), steps of three requests in a graph of four rows
    (the spare row's state belongs to nobody), a request that sits out steps, and a request that ends and whose
    row the next one takes.  Compared with the plain implementation and, bit for bit, with eager steps."""
    import toy_parts
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToyConfig(state_on_device=True)
    d = write_random_model(cfg, str(tmp_path / "toy"), seed=4, std=0.2, norm_jitter=0.1, dtype=dtype)
    model = load_model(d, dtype, "cuda:0")
    _, W = plain.read_model_dir(d)
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=i) for i, (r, n) in enumerate({"p": 24, "q": 14, "r": 12, "s": 9}.items())}
    steps = [([("p", 0, 9)], []), ([("p", 9, 2), ("q", 0, 6)], [])]
    steps += [([("p", 11 + i, 1), ("q", 6 + i, 1)], []) for i in range(3)]                       # two rows: first graph
    steps += [([("p", 14, 1), ("q", 9, 1), ("r", 0, 1)], [])]                                    # r starts inside a captured step
    steps += [([("p", 15 + i, 1), ("q", 10 + i, 1), ("r", 1 + i, 1)], []) for i in range(3)]     # three rows in a graph of four
    steps += [([("p", 18, 1), ("r", 4, 1)], []), ([("q", 13, 1), ("r", 5, 1)], ["q"])]           # q sits out, then ends
    steps += [([("p", 19, 1), ("r", 6, 1), ("s", 0, 1)], [])]                                    # s takes q's row
    steps += [([("p", 20 + i, 1), ("r", 7 + i, 1), ("s", 1 + i, 1)], []) for i in range(4)]
    steps += [([("r", 11, 1), ("s", 5, 4)], ["p", "r", "s"])]
    eager = helpers.run_schedule(ModelRunner(model, 8, 12, max_requests=3), reqs, steps)
    runner = ModelRunner(model, 8, 12, max_requests=3, use_graph=True)
    assert runner.use_graph, "every part of this model may be captured"
    got = helpers.run_schedule(runner, reqs, steps)
    assert runner.graph_steps == 14
    for r, t in reqs.items():
        ref = toy_parts.plain_toy_forward(cfg, W, t)
        assert helpers.rel_err(got[r], ref) < helpers.TOL[dtype], f"{r}: first at {helpers.first_difference(got[r], ref, helpers.TOL[dtype])}"
        assert torch.equal(got[r], eager[r]), f"{r}: a captured step differs from the eager step (first at {helpers.first_difference(got[r], eager[r], 0.0)})"
    # through the entry point: graphs, and steps queued behind the sampler of the step before
    from tempura_amd.engine import Engine
    from tempura_amd.sampling import SamplingParams
    eng = Engine(model, dtype=dtype, page_size=8, kv_pages=24, max_batch_size=3)
    assert eng.chain_steps and eng.runner.use_graph
    if dtype == "float32":
        prompts = [reqs["q"], reqs["p"][:5], reqs["s"][:1]]
        outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=8))
        assert eng.runner.graph_steps > 0
        for prompt, out in zip(prompts, outs):
            seq = list(prompt)
            for tok in out:         # greedy by the plain implementation, token by token
                assert tok == int(torch.argmax(toy_parts.plain_toy_forward(cfg, W, seq)[-1]))
                seq.append(tok)


def test_toy_block_arrangements_and_norm_on_the_gpu(tmp_path):
    """Registered, built and stepped without a change to the framework: block arrangements of the tests (norms
    before and after mixer and feed-forward; a layer without a feed-forward) and a norm of the tests (centred,
    with a shift; also the model's last norm, which then picks the wanted rows itself), around the library's
    attention and SwiGLU kernels; and greedy generation through the entry point, decode steps as replayed graphs."""
    import toy_parts
    from tempura_amd.engine import Engine
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.sampling import SamplingParams
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToySandwichConfig()
    d = write_random_model(cfg, str(tmp_path / "sandwich"), seed=8, std=0.2, norm_jitter=0.1, dtype="float32")
    model = load_model(d, "float32", "cuda:0")
    _, W = plain.read_model_dir(d)
    runner = ModelRunner(model, 8, 12, max_requests=3)
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=20 + i) for i, (r, n) in enumerate({"p": 21, "q": 9, "r": 30}.items())}
    steps = [([("p", 0, 6)], []), ([("p", 6, 3), ("q", 0, 8)], []), ([("p", 9, 1), ("q", 8, 1), ("r", 0, 17)], ["q"]),
             ([("p", 10, 11), ("r", 17, 13)], ["p", "r"])]
    got = helpers.run_schedule(runner, reqs, steps)
    for r, t in reqs.items():
        assert helpers.rel_err(got[r], toy_parts.plain_sandwich_forward(cfg, W, t)) < helpers.TOL["float32"], r
    eng = Engine(model, dtype="float32", page_size=8, kv_pages=24, max_batch_size=3)
    prompts = [reqs["q"], reqs["p"][:5]]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=6))
    for prompt, out in zip(prompts, outs):
        seq = list(prompt)
        for tok in out:         # greedy by the plain implementation, token by token
            assert tok == int(torch.argmax(toy_parts.plain_sandwich_forward(cfg, W, seq)[-1]))
            seq.append(tok)


def test_toy_routed_ffn_and_learned_position_on_the_gpu(tmp_path):
    """Registered, built and stepped without a change to the framework: a feed-forward with routing and a
    learned position encoding from the tests, beside the library's kernels (rotary windowed attention, SwiGLU),
    portions and single tokens of three requests mixed.  In float32 only: rounding to bfloat16 may send a token
    whose two best experts score alike to the other one, which no tolerance covers."""
    dtype = "float32"
    import toy_parts
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToyRoutedConfig()
    d = write_random_model(cfg, str(tmp_path / "routed"), seed=6, std=0.25, norm_jitter=0.1, dtype=dtype)
    model = load_model(d, dtype, "cuda:0")
    _, W = plain.read_model_dir(d)
    runner = ModelRunner(model, 8, [12, 8], max_requests=3)
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=10 + i) for i, (r, n) in enumerate({"p": 21, "q": 9, "r": 30}.items())}
    steps = [([("p", 0, 6)], []), ([("p", 6, 3), ("q", 0, 8)], []), ([("p", 9, 1), ("q", 8, 1), ("r", 0, 17)], ["q"]),
             ([("p", 10, 11), ("r", 17, 13)], ["p", "r"])]
    got = helpers.run_schedule(runner, reqs, steps)
    for r, t in reqs.items():
        ref = toy_parts.plain_routed_forward(cfg, W, t)
        assert helpers.rel_err(got[r], ref) < helpers.TOL[dtype], r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_with_pages_of_its_own_layout_on_the_gpu(tmp_path, dtype):
    """Registered, built and stepped without a change to the framework: a mixer from the tests whose pages hold one
    compressed vector per token (its cache spec says so), in a cache group of its own beside an attention layer
    that uses the HIP kernels; portions and single tokens of four requests, pages given back and used again."""
    import toy_parts
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.weights import write_random_model
    cfg = toy_parts.ToyLatentConfig()
    d = write_random_model(cfg, str(tmp_path / "latent"), seed=9, std=0.25, norm_jitter=0.1, dtype=dtype)
    model = load_model(d, dtype, "cuda:0")
    _, W = plain.read_model_dir(d)
    runner = ModelRunner(model, 8, [9, 9], max_requests=3)
    assert {n: tuple(t.shape) for n, t in runner.pools.kv[0].items()} == {"c": (2, 10, 8, 20)}
    reqs = {r: helpers.random_tokens(cfg.vocab_size, n, seed=30 + i) for i, (r, n) in enumerate({"p": 21, "q": 9, "r": 30, "s": 12}.items())}
    steps = [([("p", 0, 6)], []), ([("p", 6, 3), ("q", 0, 8)], []), ([("p", 9, 1), ("q", 8, 1), ("r", 0, 17)], ["q"]),
             ([("p", 10, 11), ("r", 17, 13)], ["p"]), ([("s", 0, 2)], ["r"]), ([("s", 2, 10)], ["s"])]
    got = helpers.run_schedule(runner, reqs, steps)
    for r, t in reqs.items():
        ref = toy_parts.plain_latent_forward(cfg, W, t)
        # (bfloat16: twice what rounding the stored values to bfloat16 does to this request in the plain
        # implementation, 1.3e-2 to 7e-2 here; a constant would be too tight for one request and too loose for the next)
        bound = helpers.TOL[dtype] if dtype == "float32" else \
            helpers.BF16_FACTOR * helpers.rel_err(toy_parts.plain_latent_forward(cfg, W, t, stored=plain.as_bfloat16), ref)
        assert helpers.rel_err(got[r], ref) < bound, f"{r}: {helpers.rel_err(got[r], ref):.3e} against {bound:.3e}"
    assert runner.cache.free_pages() == [9, 9]
