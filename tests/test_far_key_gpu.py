"""A far key that decides, at model level: in every request one key among hundreds carries all the attention of
certain later queries (``helpers.plant_pointer``), so that a kernel or a cache that loses that one key (a page's
edge, a split's edge, a page that went to another request, a value row in the wrong place) moves the logits by most
of their range, fifty and more times what bfloat16 storage explains.  With random weights alone the bfloat16 bound is
as large as what one wrong key among hundreds costs; here it is not.

The reference's own tests of this kind: exact equality of chunked and whole logits
(/root/reference/engine/src/model.rs:11687-11707) and paged against contiguous attention under shuffled block
tables (/root/reference/kernels/src/attention.rs:2515-2591)."""
import json
import os

import pytest
import torch

import helpers
import plain

pytestmark = pytest.mark.gpu

NEEDLES, PROBE = [500, 501, 502, 503], 504
# request: (length, needle token, its place, probes): places at a page's last and first slot, the first key of all,
# the two sides of 128 (where the decode kernel's splits meet), one in the middle of nowhere; probes in prompt
# portions, at portion starts, and among the last 32 tokens, which are decoded one by one
LAYOUT = {
    "p0": (70, 500, 15, [16, 40, 69]),
    "p1": (1100, 501, 16, [17, 500, 1067, 1068, 1085, 1099]),
    "p2": (333, 502, 0, [1, 2, 150, 301, 320, 332]),
    "p3": (520, 503, 127, [128, 129, 400, 488, 500, 519]),
    "p4": (96, 500, 31, [32, 63, 64, 80, 95]),
    "p5": (200, 501, 128, [129, 167, 168, 180, 199]),
}


def _folder(tiny_dirs, tmp_path_factory, dtype):
    """Config D's folder of this dtype with the pointer planted in layer 0 (weights stored in the folder's type)."""
    from tempura_amd.weights import write_safetensors
    cfg, W = tiny_dirs.plain_model("D", dtype)
    W2 = helpers.plant_pointer(cfg, W, NEEDLES, PROBE, strength=80.0)
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    d = tmp_path_factory.mktemp(f"pointer_{dtype}")
    with open(os.path.join(tiny_dirs.path("D", dtype), "config.json")) as f:
        (d / "config.json").write_text(f.read())
    write_safetensors(str(d / "model.safetensors"), [(k, v.to(store)) for k, v in W2.items()])
    return str(d)


_CACHE = {}


def _setup(tiny_dirs, tmp_path_factory, dtype):
    if dtype in _CACHE:
        return _CACHE[dtype]
    folder = _folder(tiny_dirs, tmp_path_factory, dtype)
    cfg, W = plain.read_model_dir(folder)
    requests, refs = {}, {}
    for i, (rid, (n, needle, at, probes)) in enumerate(LAYOUT.items()):
        toks = helpers.pointer_sequence(cfg["vocab_size"], n, needle, at, PROBE, probes, NEEDLES + [PROBE], seed=50 + i)
        requests[rid] = toks
        exact = plain.forward(cfg, W, toks)
        scale = float(exact.abs().max())
        rows = torch.tensor(probes)
        if dtype == "float32":
            bound = helpers.float32_bound(cfg)
        else:
            noisy = plain.forward(cfg, W, toks, stored=plain.as_bfloat16)
            bound = helpers.BF16_FACTOR * float((noisy[rows] - exact[rows]).abs().max()) / scale
        lost = list(toks)
        lost[at] = 7                                   # the same sequence without its needle: what a miss computes
        missed = plain.forward(cfg, W, lost)
        cost = float((missed[rows] - exact[rows]).abs().amax(dim=-1).min()) / scale
        assert cost >= 25 * bound, f"{rid}: losing the needle moves a probe's logits by {cost:.2e}, the bound is {bound:.2e}"
        refs[rid] = (exact, scale, rows, bound, cost)
    _CACHE[dtype] = (folder, requests, refs)
    return _CACHE[dtype]


def _runner(folder, dtype, max_tokens, use_graph):
    from tempura_amd.engine.loading import load_model
    from tempura_amd.engine.runner import ModelRunner
    model = load_model(folder, dtype, "cuda:0")
    return ModelRunner(model, 16, (max_tokens + 15) // 16, max_requests=4, use_graph=use_graph)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_a_far_key_decides(tiny_dirs, tmp_path_factory, dtype, mode, capsys):
    folder, requests, refs = _setup(tiny_dirs, tmp_path_factory, dtype)
    lengths = {rid: len(t) for rid, t in requests.items()}
    if mode == "mixed":
        max_tokens = sum(sorted(helpers.roundup(n, 64) for n in lengths.values())[-2:]) + 64     # pages are used again
        steps = helpers.schedule_mixed(lengths, max_tokens, seed=6)
    else:
        max_tokens = max(helpers.roundup(n, 64) for n in lengths.values())
        steps = {"whole": helpers.schedule_whole, "bulk_tail": helpers.schedule_bulk_tail,
                 "portions": helpers.schedule_portions}[mode](lengths)
    runner = _runner(folder, dtype, max_tokens, use_graph=True)
    got = helpers.run_schedule(runner, requests, steps)
    assert not runner.cache.live_requests()
    if mode in ("bulk_tail", "mixed"):
        assert runner.graph_steps > 0, "the decoded tails went through captured steps"
    report = []
    for rid, (exact, scale, rows, bound, cost) in refs.items():
        err = float((got[rid][rows].double() - exact[rows]).abs().max()) / scale
        report.append(f"{rid}: probes off by {err:.2e}, bound {bound:.2e}, a lost needle costs {cost:.2e}")
        assert err <= bound, f"{dtype}/{mode}: {report[-1]}"
    with capsys.disabled():
        print(f"\n  {dtype}/{mode}: " + "; ".join(report[:2]))
