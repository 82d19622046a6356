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

LENGTHS = {"A": {"a0": 5, "a1": 17, "a2": 33, "a3": 150, "a4": 97, "a5": 64},
           "B": {"b0": 1, "b1": 9, "b2": 40, "b3": 63, "b4": 120, "b5": 201},
           "C": {"c0": 3, "c1": 49, "c2": 130, "c3": 75, "c4": 25, "c5": 88}}


def _requests(name):
    vocab = helpers.CONFIGS[name].vocab_size
    return {rid: helpers.random_tokens(vocab, n, seed=1000 + i)
            for i, (rid, n) in enumerate(LENGTHS[name].items())}


def _runner(tiny_dirs, name, dtype, max_tokens, page_size=16):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    model = load_model(tiny_dirs.path(name, dtype), dtype, "cuda:0")
    return ModelRunner(model, page_size, (max_tokens + page_size - 1) // page_size, max_requests=4)


def _run(runner, requests, steps):
    """Run a schedule asking for logits everywhere; returns {rid: [len, vocab] float32}."""
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
                got[rid][start + i] = logits[row]
                row += 1
        for rid in end:
            runner.end_request(rid)
        runner.cache.check()
    return {rid: torch.stack(rows) for rid, rows in got.items()}


_REF = {}


def _reference(tiny_dirs, name, dtype):
    key = (name, dtype)
    if key not in _REF:
        cfg, W = tiny_dirs.plain_model(name, dtype)
        _REF[key] = {rid: plain.forward(cfg, W, toks) for rid, toks in _requests(name).items()}
    return _REF[key]


def _compare(got, ref, dtype, what):
    for rid in ref:
        err = helpers.rel_err(got[rid], ref[rid])
        assert err <= helpers.TOL[dtype], f"{what}: request {rid} differs from the plain implementation by {err:.3e}"
        # the first wrong token, if any, for the report
    return True


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_replay_modes(tiny_dirs, name, dtype, mode):
    requests = _requests(name)
    lengths = LENGTHS[name]
    if mode == "mixed":
        # room for about three of the requests: pages of finished ones must be used again
        max_tokens = sum(sorted(helpers.roundup(n, 64) for n in lengths.values())[-2:]) + 64
        steps = helpers.schedule_mixed(lengths, max_tokens, seed=5)
    else:
        max_tokens = max(helpers.roundup(n, 64) for n in lengths.values())
        steps = {"whole": helpers.schedule_whole, "bulk_tail": helpers.schedule_bulk_tail,
                 "portions": helpers.schedule_portions}[mode](lengths)
    page_size = {"A": 16, "B": 8, "C": 32}[name]
    runner = _runner(tiny_dirs, name, dtype, max_tokens, page_size)
    got = _run(runner, requests, steps)
    assert not runner.cache.live_requests()
    assert runner.cache.free_pages() == [p.num_pages for p in runner.cache.pools]
    _compare(got, _reference(tiny_dirs, name, dtype), dtype, f"{name}/{dtype}/{mode}")
