"""Replay on the GPU: the same requests whole, with the last 32 tokens decoded one by one, in
portions of changing size, and mixed with other requests under so few pages that they are used
again — in float32 and in bfloat16 — all compared with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain

pytestmark = pytest.mark.gpu



def _runner(tiny_dirs, name, dtype, max_tokens, page_size=16, use_graph=False):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    from tempura_amd.kernels import ops
    ops.set_backend(None)
    model = load_model(tiny_dirs.path(name, dtype), dtype, "cuda:0")
    return ModelRunner(model, page_size, (max_tokens + page_size - 1) // page_size, max_requests=4, use_graph=use_graph)


_REF = {}


def _reference(tiny_dirs, name, dtype):
    """{request: (exact logits, bound)} of a configuration's requests (``helpers.plain_reference``)."""
    key = (name, dtype)
    if key not in _REF:
        cfg, W = tiny_dirs.plain_model(name, dtype)
        _REF[key] = {rid: helpers.plain_reference(cfg, W, toks, dtype) for rid, toks in helpers.requests_for(name).items()}
    return _REF[key]


def _compare(got, ref, dtype, what):
    for rid, (exact, bound) in ref.items():
        err = helpers.rel_err(got[rid], exact)
        bad = helpers.first_difference(got[rid], exact, bound)
        assert err <= bound, \
            f"{what}: request {rid} differs from the plain implementation by {err:.3e} (bound {bound:.3e}), first at position {bad}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_replay_modes(tiny_dirs, name, dtype, mode):
    requests = helpers.requests_for(name)
    steps, max_tokens = helpers.schedule_for(name, mode)
    runner = _runner(tiny_dirs, name, dtype, max_tokens, helpers.PAGE_SIZE[name])
    got = helpers.run_schedule(runner, requests, steps)
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]
    _compare(got, _reference(tiny_dirs, name, dtype), dtype, f"{name}/{dtype}/{mode}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_replay_random_schedules(tiny_dirs, name, dtype):
    """Twelve schedules drawn from seeds (``helpers.schedule_random``: pool size, order of requests and of a step's
    entries, portion lengths, where single tokens begin, requests sitting out), decode-only steps as replayed
    graphs: every position of every request against the plain implementation, no page left behind."""
    requests = helpers.requests_for(name)
    ref = _reference(tiny_dirs, name, dtype)
    for seed in range(12):
        steps, max_tokens = helpers.schedule_random(helpers.LENGTHS[name], seed=100 * seed + ord(name))
        runner = _runner(tiny_dirs, name, dtype, max_tokens, helpers.PAGE_SIZE[name], use_graph=True)
        got = helpers.run_schedule(runner, requests, steps)
        assert not runner.cache.live_requests()
        assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]
        _compare(got, ref, dtype, f"{name}/{dtype}/random schedule of seed {seed}")


def test_cutting_modes_against_each_other(tiny_dirs, capsys):
    """The four ways of cutting compared with each other, not only with the plain implementation (float32,
    config A).  Every kernel computes a row in an order that does not involve other rows; the one thing that
    changes with a step's size is which product kernel runs: steps of at most eight rows take the kernel that
    splits K over a block's threads, longer steps the tiled one, and the two add in different orders.  A position
    reads the keys and values of the positions before it, so its logits are bit-equal between two modes whenever
    both ran it AND everything before it in steps of the same class, and differ by float32 rounding otherwise;
    the measured differences are printed."""
    name, dtype = "A", "float32"
    requests = helpers.requests_for(name)
    results, classes = {}, {}
    for mode in ("whole", "bulk_tail", "portions", "mixed"):
        steps, max_tokens = helpers.schedule_for(name, mode)
        runner = _runner(tiny_dirs, name, dtype, max_tokens, helpers.PAGE_SIZE[name])
        results[mode] = helpers.run_schedule(runner, requests, steps)
        cls = {rid: [None] * len(t) for rid, t in requests.items()}
        for entries, _ in steps:
            rows = sum(c for _, _, c in entries)
            for rid, start, count in entries:
                for i in range(start, start + count):
                    cls[rid][i] = rows <= 8
        classes[mode] = cls
    report = []
    for mode in ("bulk_tail", "portions", "mixed"):
        same = other = 0
        worst = 0.0
        for rid in requests:
            a, b = results["whole"][rid], results[mode][rid]
            scale = float(a.abs().max())
            alike = True
            for i in range(a.shape[0]):
                alike = alike and classes["whole"][rid][i] == classes[mode][rid][i]
                if alike:
                    assert torch.equal(a[i], b[i]), f"{mode}: request {rid} position {i} ran the same kernels and differs"
                    same += 1
                else:
                    worst = max(worst, float((a[i] - b[i]).abs().max()) / scale)
                    other += 1
        assert worst <= 2e-6, f"{mode}: {worst:.3e} between two orders of float32 addition"
        report.append(f"{mode} vs whole: {same} positions bit-equal, {other} under the other product kernel, largest difference {worst:.2e}")
    assert any("0 under" not in r for r in report), "no position was run by the other kernel: the comparison is empty"
    with capsys.disabled():
        print("\n  " + "\n  ".join(report))


def test_cutting_modes_against_each_other_bfloat16(tiny_dirs, capsys):
    """The same comparison in bfloat16 on config D, where every fast path runs (products chosen by the step's rows,
    rotation in the projection's epilogue, matrix-core attention for portions and for single tokens with a split
    context).  Two things are asked.  (1) Where the tokens lie in the cache is no input at all: the mixed schedule
    on a pool so small that pages are used again, and on a larger pool whose free list was stirred first and that
    another live request shares, gives the same BITS at every position, captured steps included.  (2) Between two
    ways of cutting, the kernels differ (another product for another number of rows; single tokens split their
    context, portions do not; a probability is rounded to bfloat16 against another running maximum), so the bits
    differ, and what remains is the noise of the storage type: every mode stays within the request's bound of the
    whole-prompt run, which is the bound both keep against the plain implementation.  The share of bit-equal
    positions and the largest difference are printed."""
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    name, dtype = "D", "bfloat16"
    requests = helpers.requests_for(name)
    ref = _reference(tiny_dirs, name, dtype)
    # (1) placement
    steps, max_tokens = helpers.schedule_for(name, "mixed")
    tight = _runner(tiny_dirs, name, dtype, max_tokens, helpers.PAGE_SIZE[name], use_graph=True)
    a = helpers.run_schedule(tight, requests, steps)
    model = load_model(tiny_dirs.path(name, dtype), dtype, "cuda:0")
    roomy = ModelRunner(model, helpers.PAGE_SIZE[name], 3 * max_tokens // helpers.PAGE_SIZE[name], max_requests=5, use_graph=True)
    filler = helpers.random_tokens(helpers.CONFIGS[name].vocab_size, 200, seed=5)
    for rid, n in (("x", 50), ("y", 90), ("z", 23)):
        roomy.add_request(rid)
        roomy.step([StepEntry(rid, filler[:n], [])])
    roomy.end_request("x")
    roomy.end_request("z")                       # pages 0..3 and 10, 11 are free again, in that order of return; "y" stays live
    b = helpers.run_schedule(roomy, requests, steps)
    assert tight.graph_steps > 0 and roomy.graph_steps == tight.graph_steps
    for rid in requests:
        assert torch.equal(a[rid], b[rid]), f"request {rid}: other pages, other bits (first at {helpers.first_difference(a[rid], b[rid], 0.0)})"
    roomy.end_request("y")
    # (2) cutting
    results = {"mixed": a}
    for mode in ("whole", "bulk_tail", "portions"):
        steps, max_tokens = helpers.schedule_for(name, mode)
        results[mode] = helpers.run_schedule(_runner(tiny_dirs, name, dtype, max_tokens, helpers.PAGE_SIZE[name]), requests, steps)
    report = []
    for mode in ("bulk_tail", "portions", "mixed"):
        same = total = 0
        worst = 0.0
        for rid in requests:
            x, y = results["whole"][rid], results[mode][rid]
            exact, bound = ref[rid]
            diff = float((x.double() - y.double()).abs().max() / exact.abs().max())
            worst = max(worst, diff / bound)
            # (both keep `bound` against the plain implementation; against each other they were measured at a quarter of it)
            assert diff <= bound / 2, f"{mode} vs whole, request {rid}: {diff:.3e} apart, the storage noise bound is {bound:.3e}"
            same += int((x == y).all(dim=-1).sum())
            total += x.shape[0]
        report.append(f"{mode} vs whole: {same} of {total} positions bit-equal, largest difference {worst:.2f} of the bound")
    with capsys.disabled():
        print("\n  " + "\n  ".join(report))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_graph_replays_match_eager(tiny_dirs, name, dtype):
    """Decode steps replayed as a captured graph give the eager steps' logits, replay after replay, with
    eager steps (prompt portions of other requests) and synchronisations between the replays."""
    requests = helpers.requests_for(name)
    steps, max_tokens = helpers.schedule_for(name, "mixed")
    eager = helpers.run_schedule(_runner(tiny_dirs, name, dtype, max_tokens, helpers.PAGE_SIZE[name]), requests, steps)
    runner = _runner(tiny_dirs, name, dtype, max_tokens, helpers.PAGE_SIZE[name], use_graph=True)
    assert runner.use_graph
    graphed = helpers.run_schedule(runner, requests, steps)
    assert runner.graph_steps >= 32, "decode-only steps went through the graph"
    for rid in eager:
        # (single tokens split their context by its length rounded up as a captured step's bound is: the same cut)
        assert torch.equal(graphed[rid], eager[rid]), f"request {rid}: graph replay differs from the eager step"
    _compare(graphed, _reference(tiny_dirs, name, dtype), dtype, f"{name}/{dtype}/graph")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_staged_ahead_change_nothing(tiny_dirs, dtype):
    """``prepare_decode`` is a hint: steps that find their inputs staged give the bits of steps that do not, and a
    hint that does not come true (other requests, another order, a request ended in between) is dropped.
    ``step_chained`` (tokens from device memory) gives the same bits again, staged or not."""
    from tempura_amd.engine.runner import StepEntry
    name = "D"
    reqs = {rid: toks for rid, toks in list(helpers.requests_for(name).items())[1:4]}

    def run(hints, on_device=False):
        runner = _runner(tiny_dirs, name, dtype, 1024, helpers.PAGE_SIZE[name], use_graph=True)
        for rid, toks in reqs.items():
            runner.add_request(rid)
            runner.step([StepEntry(rid, toks[:5], [])])
        live, out = list(reqs), []
        for i in range(5, 30):
            if i == 20:                                    # a request ends between a hint and its step
                runner.end_request(live.pop(1))
            if on_device:                                  # the tokens come from device memory
                toks = torch.tensor([reqs[rid][i] for rid in live], dtype=torch.int32, device="cuda:0")
                out.append(runner.step_chained(live, toks).clone())
            else:
                out.append(runner.step([StepEntry(rid, [reqs[rid][i]], [0]) for rid in live]).clone())
            hint = hints(i, live)
            if hint is not None:
                runner.prepare_decode(hint)
        return out, runner

    plain_out, r0 = run(lambda i, live: None)
    staged_out, r1 = run(lambda i, live: list(live))
    wrong_out, r2 = run(lambda i, live: list(reversed(live)) if i % 2 else live[:1])
    chained_out, r3 = run(lambda i, live: list(live), on_device=True)
    chained_cold, r4 = run(lambda i, live: None, on_device=True)
    assert r0.staged_steps == 0 and r1.staged_steps >= 22 and r2.staged_steps == 0 and r3.staged_steps >= 22
    for a, b, c, d, e in zip(plain_out, staged_out, wrong_out, chained_out, chained_cold):
        assert torch.equal(a, b) and torch.equal(a, c) and torch.equal(a, d) and torch.equal(a, e)
    for r in (r0, r1, r2, r3, r4):
        r.cache.check()


def test_staged_inputs_are_dropped_when_the_cache_changed_behind_the_runner(tiny_dirs):
    """The scheduler ends and readmits requests on the cache manager itself.  A decode step that was staged for
    the same request names before such a change must not replay the old positions and pages."""
    from tempura_amd.engine.runner import StepEntry
    name, dtype = "D", "float32"
    reqs = {rid: toks for rid, toks in list(helpers.requests_for(name).items())[1:3]}
    rids = list(reqs)
    ref = _reference(tiny_dirs, name, dtype)
    runner = _runner(tiny_dirs, name, dtype, 1024, helpers.PAGE_SIZE[name], use_graph=True)
    for rid in rids:
        runner.add_request(rid)
        runner.step([StepEntry(rid, reqs[rid][:9], [])])
    runner.step([StepEntry(rid, [reqs[rid][9]], [0]) for rid in rids])            # captures the graph
    assert runner.prepare_decode(rids)
    # preempted and readmitted behind the runner's back, as the scheduler does it: another length, other pages
    runner.cache.release(rids[0])
    runner.cache.add(rids[0])
    runner.step([StepEntry(rids[0], reqs[rids[0]][:4], [])])
    assert runner.prepare_decode(rids)
    runner.cache.release(rids[0])
    runner.cache.add(rids[0])
    runner.step([StepEntry(rids[0], reqs[rids[0]][:6], [])])
    before = runner.staged_steps
    got = runner.step([StepEntry(rids[0], [reqs[rids[0]][6]], [0]), StepEntry(rids[1], [reqs[rids[1]][10]], [0])]).cpu()
    assert runner.staged_steps == before, "the stale staging was used"
    assert helpers.rel_err(got[0], ref[rids[0]][0][6]) <= helpers.TOL[dtype]
    assert helpers.rel_err(got[1], ref[rids[1]][0][10]) <= helpers.TOL[dtype]
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tiny_dirs, dtype):
    """700 tokens decoded one by one after a short prompt (config A, 44 pages of 16)."""
    cfg, W = tiny_dirs.plain_model("A", dtype)
    toks = helpers.random_tokens(cfg["vocab_size"], 700, seed=77)
    ref = helpers.plain_reference(cfg, W, toks, dtype)
    runner = _runner(tiny_dirs, "A", dtype, 704, 16, use_graph=True)
    steps = [([("x", 0, 9)], [])] + [([("x", i, 1)], []) for i in range(9, 700)]
    got = helpers.run_schedule(runner, {"x": toks}, steps)
    _compare(got, {"x": ref}, dtype, f"long decode {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_first_tokens(tiny_dirs, name, dtype):
    """The first tokens of a sequence, one by one from position 0 (one key, then two, ...)."""
    cfg, W = tiny_dirs.plain_model(name, dtype)
    toks = helpers.random_tokens(cfg["vocab_size"], 6, seed=78)
    ref = helpers.plain_reference(cfg, W, toks, dtype)
    runner = _runner(tiny_dirs, name, dtype, 64, helpers.PAGE_SIZE[name])
    got = helpers.run_schedule(runner, {"x": toks}, [([("x", i, 1)], []) for i in range(6)])
    _compare(got, {"x": ref}, dtype, f"first tokens {name} {dtype}")


def test_window_layers_give_pages_back(tiny_dirs):
    """Config C has a window of 24 on two of its four layers: portions and single tokens cross the window's
    edge at every offset, logits match the plain implementation, and the windowed group holds one page where
    the full group holds three."""
    cfg, W = tiny_dirs.plain_model("C", "float32")
    toks = helpers.random_tokens(cfg["vocab_size"], 90, seed=79)
    ref = helpers.plain_reference(cfg, W, toks, "float32")
    runner = _runner(tiny_dirs, "C", "float32", 128, 32)
    steps = [([("x", 0, 38)], []), ([("x", 38, 5)], [])] + [([("x", i, 1)], []) for i in range(43, 90)]
    got = helpers.run_schedule(runner, {"x": toks}, steps)
    _compare(got, {"x": ref}, "float32", "window edge")
    kinds = [g.kind for g in runner.cache.groups]
    held = {k: p.num_held for k, p in zip(kinds, runner.cache.pools)}
    assert held == {"window": 1, "full": 3}
    runner.end_request("x")


def test_trace_run_says_what_is_wrong_with_a_step(tiny_dirs, tmp_path):
    """A step that cannot be run (a token outside the vocabulary, a wanted place outside the entry, more tokens than
    the pool holds, a line that is no JSON) ends the replay with status 2 and one line that names the step and the
    fault; the steps before it are done and written."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    good = json.dumps({"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []})
    bad = {"token id 999": json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [7, 999], "want": [1]}], "end": []}),
           "wanted place 4": json.dumps({"step": 1, "entries": [{"id": "a", "tokens": [7, 9], "want": [4]}], "end": []}),
           "PagesExhausted": json.dumps({"step": 1, "entries": [{"id": "b", "tokens": [1] * 100, "want": []}], "end": []}),
           "JSONDecodeError": "step one"}
    for marker, line in bad.items():
        out_dir = tmp_path / marker.replace(" ", "_")
        p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", tiny_dirs.path("A", "float32"),
                            "--dtype", "float32", "--out", str(out_dir), "--max-tokens", "64"],
                           input=good + "\n" + line + "\n", capture_output=True, text=True, timeout=600)
        assert p.returncode == 2, (marker, p.returncode, p.stderr[-500:])
        said = [l for l in p.stderr.splitlines() if l.startswith("trace_run:")]
        assert len(said) == 1 and marker in said[0] and "Traceback" not in p.stderr, (marker, p.stderr[-500:])
        assert ("step 1" in said[0]) == (marker != "JSONDecodeError")
        assert p.stdout.splitlines() == ["done 0"] and (out_dir / "0.f32").stat().st_size == 2 * 256 * 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tiny_dirs, tmp_path, dtype):
    """bin/trace_run as a user runs it: JSON steps on standard input, logits files out."""
    name = "B"
    requests = helpers.requests_for(name)
    steps, max_tokens = helpers.schedule_for(name, "mixed")
    out_dir = tmp_path / "out"
    lines = []
    for i, (entries, end) in enumerate(steps):
        want_all = i % 3 != 1
        lines.append(json.dumps({"step": i, "end": end, "entries": [
            {"id": rid, "tokens": requests[rid][s:s + c], "want": list(range(c)) if want_all else []}
            for rid, s, c in entries]}))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", tiny_dirs.path(name, dtype),
                        "--dtype", dtype, "--out", str(out_dir), "--max-tokens", str(max_tokens)],
                       input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    ref = _reference(tiny_dirs, name, dtype)
    vocab = helpers.CONFIGS[name].vocab_size
    checked = 0
    for i, (entries, end) in enumerate(steps):
        path = out_dir / f"{i}.f32"
        if i % 3 == 1:
            assert not path.exists(), "a step in which nothing is wanted writes no file"
            continue
        arr = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(-1, vocab))
        row = 0
        for rid, s, c in entries:
            # the same measure as everywhere: the difference relative to the request's largest logit
            exact, bound = ref[rid]
            err = float((arr[row:row + c].double() - exact[s:s + c]).abs().max() / exact.abs().max())
            assert err <= bound, f"step {i} request {rid}: {err:.3e} (bound {bound:.3e})"
            row += c
            checked += c
        assert row == arr.shape[0]
    assert checked > 200


def test_long_context_decoding_bfloat16_fast_paths(tiny_dirs):
    """Config D in bfloat16: 1,500 tokens in three portions (the tiled product and the MFMA prefill attention,
    with and without a cached prefix), then 40 tokens one by one over a context long enough that the decode
    attention splits it (graph replays)."""
    cfg, W = tiny_dirs.plain_model("D", "bfloat16")
    toks = helpers.random_tokens(cfg["vocab_size"], 1540, seed=81)
    ref = helpers.plain_reference(cfg, W, toks, "bfloat16")
    runner = _runner(tiny_dirs, "D", "bfloat16", 1600, 16, use_graph=True)
    steps = [([("x", 0, 700)], []), ([("x", 700, 90)], []), ([("x", 790, 710)], [])] + [([("x", i, 1)], []) for i in range(1500, 1540)]
    got = helpers.run_schedule(runner, {"x": toks}, steps)
    assert runner.graph_steps == 40
    _compare(got, {"x": ref}, "bfloat16", "long context D")
