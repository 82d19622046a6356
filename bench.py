#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Llama-3.1-8B shape, bfloat16,
random weights, synthetic token ids.

    python bench.py --gpus 1 --steps K --warmup W

A "step" is one decode step of the whole batch (default 8 requests).  The timed steps are centred on a cache
length of 3,072 tokens, the middle of the named sweep from 2,048 to 4,096: the default 2,000 steps cover the
sweep itself (prompts of 2,048 tokens), a short run (`--steps 20`) starts from prompts of about 3,050 tokens and
times the steps around 3,072, so that a step reads what a step of the sweep reads on average; `metric` names
the range that was timed.  The headline runs through the engine's own entry point: `Engine.add_request` and
`Engine.step`, with its scheduler, step function and sampler (greedy), as `tempura run` does.  Prints ONE
JSON line: decoded tokens per second (`value`), the step's share of the HBM roofline, the 2,048-token
prefill, and under `points`: batch 1 and 64 through the engine, the same three batches through the bare
step function (`runner_b*`: no scheduler, no sampler object), longer prefills, decoding at a 32 k context,
and the mixed serving workload (64 requests, prompts of 128..2,048 tokens in portions of 512 beside running
decodes, 256 output tokens each, Llama-3.2-3B shape) whose details are under `mixed`.
The reference measures prefill and single-token forwards its own way, with percentiles and a fingerprint of
the logits for run-to-run determinism (/root/reference/tools/bench-gpu/src/bench_real_model.rs:160-278);
its serving loop is /root/reference/server/src/engine_task.rs:581-875.
"""
from __future__ import annotations

import argparse
import json
import random
import sys
import time

HBM_PEAK_GBS = 8000.0                                   # MI355X HBM3E, published
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense, published


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000, help="timed decode steps")
    ap.add_argument("--warmup", type=int, default=16, help="untimed decode steps")
    ap.add_argument("--model-config", default="llama-3.1-8b")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-chain", action="store_true", help="wait for each step's tokens on the host before queueing the next step")
    ap.add_argument("--no-points", action="store_true", help="only the headline: no other batches, no bare step function")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-long", action="store_true", help="skip the long prefills and the 32 k decode point")
    ap.add_argument("--no-large-batches", action="store_true", help="skip decoding at batch 128 and 256")
    ap.add_argument("--no-mixed", action="store_true", help="skip the mixed serving workload")
    ap.add_argument("--no-fingerprint", action="store_true", help="skip the run-to-run determinism check")
    ap.add_argument("--point-steps", type=int, default=500, help="timed steps of the other points")
    ap.add_argument("--mixed-config", default="llama-3.2-3b")
    ap.add_argument("--mixed-requests", type=int, default=64)
    ap.add_argument("--mixed-output", type=int, default=256)
    ap.add_argument("--mixed-chunk", type=int, default=512)
    ap.add_argument("--mixed-temperature", type=float, default=0.0, help="0: greedy; above: seeded sampling with top-k 50")
    ap.add_argument("--decode-target-blocks", type=int, default=None, help="tuning: blocks the split decode attention aims at")
    return ap.parse_args()


def percentile(xs, p):
    ys = sorted(xs)
    if not ys:
        return 0.0
    k = (len(ys) - 1) * p / 100.0
    lo = int(k)
    hi = min(lo + 1, len(ys) - 1)
    return ys[lo] + (ys[hi] - ys[lo]) * (k - lo)


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (this engine has no multi-GPU path); --gpus {args.gpus} is not supported")
        return 2

    import torch
    from tempura_amd.config import PRESETS, LlamaConfig
    from tempura_amd.engine import Engine
    from tempura_amd.engine.loading import random_model
    from tempura_amd.engine.runner import StepEntry
    from tempura_amd.kernels import ops
    from tempura_amd.sampling import SamplingParams

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 3
    if args.decode_target_blocks:
        ops.decode_target_blocks = args.decode_target_blocks
    elem = 2 if args.dtype == "bfloat16" else 4
    dshort = "bf16" if args.dtype == "bfloat16" else "fp32"
    rng = random.Random(0)

    def say(msg):
        print(f"[bench] {msg}", file=sys.stderr, flush=True)

    def make_engine(name, layers, max_batch, tokens_per_request, chunk):
        """An engine with random weights made on the device and room for max_batch requests of that length."""
        full = PRESETS[name]
        cfg = LlamaConfig.from_dict(full.to_dict())
        if layers is not None:
            cfg.num_hidden_layers = layers
        cfg.validate()
        t0 = time.time()
        model = random_model(cfg, seed=0, dtype=args.dtype, device="cuda:0")
        torch.cuda.synchronize()
        say(f"{name} model built in {time.time() - t0:.1f} s")
        pages = max_batch * ((tokens_per_request + args.page_size - 1) // args.page_size) + 8
        eng = Engine(model, dtype=args.dtype, page_size=args.page_size, kv_pages=pages, max_batch_size=max_batch,
                     max_num_batched_tokens=2048, prefill_chunk_size=chunk, use_graph=not args.no_graph,
                     chain_steps=not args.no_chain)
        weight_bytes = model.weight_bytes(include_embedding=False)
        if model.lm_head.tied:
            weight_bytes += model.embedding.weight.numel() * model.embedding.weight.element_size()
        return eng, cfg, full, weight_bytes

    def prompt(vocab, n):
        return [rng.randrange(vocab) for _ in range(n)]

    greedy = dict(temperature=0.0, ignore_eos=True)

    # ---- through the engine: add_request / step with scheduler, step function and sampler ---------------------
    def engine_decode(eng, cfg, weight_bytes, batch, prompt_len, n_warm, n_steps):
        """`batch` requests with prompts of prompt_len tokens decode n_warm + n_steps tokens; the steps after the
        warm-up are timed between synchronisations.  Returns tokens a second, the mean, median and 95th
        percentile of the step time in ms (from the arrival of each step's tokens on the host), the bytes a
        step has to read, and the range of cache lengths that was timed."""
        # (early requests decode while late ones still bring their prompts, a portion a step)
        margin = batch * (-(-prompt_len // 2048) + 1) + 8
        params = SamplingParams(max_new_tokens=n_warm + n_steps + margin, **greedy)
        rids = [eng.add_request(prompt(cfg.vocab_size, prompt_len), params) for _ in range(batch)]
        reqs = [eng.request(r) for r in rids]
        while not all(r.output for r in reqs):               # prompts in portions, until every request decodes
            eng.step()
        for _ in range(n_warm):
            eng.step()
        torch.cuda.synchronize()
        kv0 = sum(r.num_computed for r in reqs) / batch
        stamps = [time.perf_counter()]
        for _ in range(n_steps):
            out = eng.step()
            assert len(out) == batch
            stamps.append(time.perf_counter())
        torch.cuda.synchronize()
        dt = time.perf_counter() - stamps[0]
        kv1 = sum(r.num_computed for r in reqs) / batch
        for r in rids:
            eng.abort(r)
        while eng.has_unfinished():
            eng.step()
        per = [1e3 * (b - a) for a, b in zip(stamps, stamps[1:])]
        mean_ctx = (kv0 + kv1 + 1) / 2.0
        bytes_step = weight_bytes + batch * mean_ctx * cfg.kv_bytes_per_token(elem)
        return {"tps": batch * n_steps / dt, "ms": 1e3 * dt / n_steps, "p50": percentile(per, 50), "p95": percentile(per, 95),
                "bytes": bytes_step, "kv": (int(round(kv0)), int(round(kv1)))}

    # ---- the bare step function: tokens stay on the device, no scheduler, no sampler object -------------------
    def runner_decode(eng, cfg, batch, prompt_len, n_warm, n_steps):
        runner = eng.runner
        rids = [("d", batch, i) for i in range(batch)]
        for rid in rids:
            runner.add_request(rid)
            runner.step([StepEntry(rid, prompt(cfg.vocab_size, prompt_len), [])])
        lg = runner.step([StepEntry(rid, [rng.randrange(cfg.vocab_size)], [0]) for rid in rids])
        chosen = ops.argmax(lg)
        coming = ops.HostCopy(chosen)

        def one():
            nonlocal chosen, coming
            if not runner.use_graph or args.no_chain:
                lg = runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, coming.result())])
                chosen = ops.argmax(lg)
                coming = ops.HostCopy(chosen)
                return
            lg = runner.step_chained(rids, chosen)
            nxt = ops.argmax(lg)
            nxt_coming = ops.HostCopy(nxt)
            runner.prepare_decode(rids)
            coming.result()
            chosen, coming = nxt, nxt_coming

        for _ in range(n_warm):
            one()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(n_steps):
            one()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        for rid in rids:
            runner.end_request(rid)
        return batch * n_steps / dt, 1e3 * dt / n_steps

    def prefill_point(eng, cfg, T, runs, warm=3):
        """One prompt of T tokens from an empty cache as one step; mean of `runs` after `warm` warm-ups, a fresh
        request (no cached keys) each time (/root/reference/tools/bench-gpu/src/bench_real_model.rs:160-278: warm-ups,
        then timed forwards on fresh sessions, tokens a second from the mean time)."""
        runner = eng.runner
        times = []
        for i in range(warm + runs):
            rid = ("p", T, i)
            runner.add_request(rid)
            toks = prompt(cfg.vocab_size, T)
            torch.cuda.synchronize()
            t = time.perf_counter()
            runner.step([StepEntry(rid, toks, [T - 1])])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            runner.end_request(rid)
            if i >= warm:
                times.append(dt)
        ms = 1e3 * sum(times) / len(times)
        L, H, I, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
        qd, kvd = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
        linear = L * (H * (qd + 2 * kvd) + qd * H + 3 * H * I)
        flops = 2.0 * T * linear + 2.0 * V * H + L * 4.0 * cfg.num_attention_heads * cfg.head_dim * T * (T + 1) / 2
        peak = MFMA_PEAK[dshort]
        return {"value": round(T / (ms / 1e3), 1), "tokens": T, "ms": round(ms, 3), "frac": round(flops / (ms / 1e3) / peak, 4)}

    def fingerprint(eng, cfg, batch, prompt_len, n_steps):
        """Two fresh runs of the same requests (greedy): the sum of the bit patterns of the last step's logits and
        the tokens must agree (/root/reference/tools/bench-gpu/src/bench_real_model.rs:193-224)."""
        runner = eng.runner
        g = random.Random(1234)
        prompts = [[g.randrange(cfg.vocab_size) for _ in range(prompt_len)] for _ in range(batch)]
        sums, toks = [], []
        for run in range(2):
            rids = [("f", run, i) for i in range(batch)]
            for rid, p in zip(rids, prompts):
                runner.add_request(rid)
                lg = runner.step([StepEntry(rid, p, [prompt_len - 1])])
            cur = [0] * batch
            seen = []
            lg = runner.step([StepEntry(rid, [p[-1]], [0]) for rid, p in zip(rids, prompts)])
            for _ in range(n_steps):
                cur = ops.argmax(lg).tolist()
                seen.append(cur)
                lg = runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, cur)])
            bits = lg.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
            sums.append(int(bits.sum().item()))
            nan = int(torch.isnan(lg).sum().item())
            toks.append(seen)
            for rid in rids:
                runner.end_request(rid)
        return {"bits_sum": sums[0], "runs": 2, "nan": nan, "equal": sums[0] == sums[1] and toks[0] == toks[1] and nan == 0}

    # ---- the mixed serving workload ---------------------------------------------------------------------------
    def mixed_workload(eng, cfg, weight_bytes):
        g = random.Random(7)
        n_req = args.mixed_requests
        lens = [g.randint(128, 2048) for _ in range(n_req)]
        prompts = [[g.randrange(cfg.vocab_size) for _ in range(n)] for n in lens]
        if args.mixed_temperature > 0:
            mk = lambda i: SamplingParams(temperature=args.mixed_temperature, top_k=50, seed=100 + i,
                                          max_new_tokens=args.mixed_output, ignore_eos=True)
        else:
            mk = lambda i: SamplingParams(max_new_tokens=args.mixed_output, **greedy)
        # (warm the graphs and the allocator with a short run of the same shape, untimed)
        warm = [eng.add_request(p[:160], SamplingParams(max_new_tokens=4, **greedy)) for p in prompts[: min(n_req, 64)]]
        while eng.has_unfinished():
            eng.step()
        before = eng.stats()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        rids = [eng.add_request(p, mk(i)) for i, p in enumerate(prompts)]
        first = {}
        kinds = {"decode_only": 0, "mixed": 0, "prefill_only": 0}
        tokens_by_kind = {"decode_only": 0, "mixed": 0, "prefill_only": 0}
        host_by_kind = {"decode_only": 0.0, "mixed": 0.0, "prefill_only": 0.0}
        step_ms = []
        n_out = 0
        while eng.has_unfinished():
            ts = time.perf_counter()
            out = eng.step()
            te = time.perf_counter()
            ls = eng.last_step
            kind = "decode_only" if ls["prompt_tokens"] == 0 else ("prefill_only" if ls["decode_tokens"] == 0 else "mixed")
            kinds[kind] += 1
            tokens_by_kind[kind] += ls["prompt_tokens"] + ls["decode_tokens"]
            step_ms.append(1e3 * (te - ts))
            for rid, tok, done in out:
                n_out += 1
                if rid not in first:
                    first[rid] = te - t0
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        after = eng.stats()
        ttft = [1e3 * first[r] for r in rids]
        steps = sum(kinds.values())
        eager = after["eager_steps"] - before["eager_steps"]
        pack_ms = (after["eager_step_pack_ms"] * after["eager_steps"] - before["eager_step_pack_ms"] * before["eager_steps"]) / max(1, eager)
        return {
            "model": args.mixed_config, "requests": n_req, "prompt_tokens": sum(lens), "output_tokens": n_out,
            "chunk": args.mixed_chunk, "sampling": "greedy" if args.mixed_temperature <= 0 else f"T={args.mixed_temperature} top_k=50",
            "seconds": round(dt, 3), "output_tok_s": round(n_out / dt, 1), "total_tok_s": round((n_out + sum(lens)) / dt, 1),
            "ttft_ms": {"mean": round(sum(ttft) / len(ttft), 1), "p50": round(percentile(ttft, 50), 1), "p95": round(percentile(ttft, 95), 1)},
            "steps": steps, "steps_by_kind": kinds,
            "tokens_per_step": {k: round(tokens_by_kind[k] / kinds[k], 1) if kinds[k] else 0 for k in kinds},
            "step_ms": {"mean": round(sum(step_ms) / len(step_ms), 3), "p50": round(percentile(step_ms, 50), 3), "p95": round(percentile(step_ms, 95), 3)},
            "preemptions": after["preemptions"] - before["preemptions"],
            "eager_steps": eager, "host_pack_ms_per_eager_step": round(pack_ms, 4),
        }

    # =============================================================================================================
    large = [] if (args.no_points or args.no_large_batches) else [128, 256]
    max_batch = args.batch if args.no_points else max([args.batch, 64] + large)
    long_tokens = 0 if (args.no_long or args.no_points) else 8 * 33536       # eight requests at a 32 k context
    per_request = max(args.context, -(-long_tokens // max_batch))
    eng, cfg, full, weight_bytes = make_engine(args.model_config, args.layers, max_batch, per_request, 2048)
    steps, warmup = args.steps, args.warmup
    if args.prompt_len + warmup + steps + 2 > args.context:
        steps = max(1, args.context - args.prompt_len - warmup - 2)
    points = {}

    def centred(n_warm, n_steps):
        """The prompt length from which n_warm untimed and n_steps timed steps are centred on the middle of the
        sweep from --prompt-len to --context (never below --prompt-len)."""
        mid = (args.prompt_len + args.context) // 2
        return max(args.prompt_len, mid - n_warm - n_steps // 2)

    prefill = None
    if not args.no_prefill:
        prefill = prefill_point(eng, cfg, args.prompt_len, 10)
        say(f"prefill {prefill}")

    head = engine_decode(eng, cfg, weight_bytes, args.batch, centred(warmup, steps), warmup, steps)
    say(f"engine decode b{args.batch}: {head['tps']:.1f} tok/s, {head['ms']:.3f} ms/step (p50 {head['p50']:.3f}, p95 {head['p95']:.3f}), KV {head['kv']}")
    achieved = head["bytes"] / (head["ms"] / 1e3) / 1e9

    determinism = None
    if not args.no_fingerprint:
        determinism = fingerprint(eng, cfg, min(args.batch, 8), 256, 16)
        say(f"determinism {determinism}")

    if not args.no_points:
        ps = max(1, min(args.point_steps, steps))
        for b in (1, 64):
            r = engine_decode(eng, cfg, weight_bytes, b, centred(8, ps), 8, ps)
            points[f"decode_b{b}"] = round(r["tps"], 1)
            points[f"decode_b{b}_hbm_frac"] = round(r["bytes"] / (r["ms"] / 1e3) / 1e9 / HBM_PEAK_GBS, 4)
            say(f"engine decode b{b}: {r['tps']:.1f} tok/s, {r['ms']:.3f} ms/step")
        for b in large:
            # (their prompts alone are b x 3,000 tokens of prefill: fewer timed steps, around the same cache length)
            r = engine_decode(eng, cfg, weight_bytes, b, centred(4, 100), 4, 100)
            points[f"decode_b{b}"] = round(r["tps"], 1)
            points[f"decode_b{b}_hbm_frac"] = round(r["bytes"] / (r["ms"] / 1e3) / 1e9 / HBM_PEAK_GBS, 4)
            say(f"engine decode b{b}: {r['tps']:.1f} tok/s, {r['ms']:.3f} ms/step, KV {r['kv']}")
        for b in sorted({1, args.batch, 64}):
            # (the same number of steps, so the same range of context lengths, as the engine's figure it stands beside)
            nw, ns = (warmup, steps) if b == args.batch else (8, ps)
            tps, ms = runner_decode(eng, cfg, b, centred(nw, ns), nw, ns)
            points[f"runner_b{b}"] = round(tps, 1)
            say(f"step function alone b{b}: {tps:.1f} tok/s, {ms:.3f} ms/step")
        if not args.no_long:
            for T in (8192, 32768):
                p = prefill_point(eng, cfg, T, 3 if T <= 8192 else 2, warm=2)
                points[f"prefill_{T}"] = p["value"]
                points[f"prefill_{T}_frac"] = p["frac"]
                say(f"prefill {p}")
            r = engine_decode(eng, cfg, weight_bytes, 8, 32768, 4, min(ps, 200))
            points["decode_b8_kv32k"] = round(r["tps"], 1)
            points["decode_b8_kv32k_hbm_frac"] = round(r["bytes"] / (r["ms"] / 1e3) / 1e9 / HBM_PEAK_GBS, 4)
            say(f"engine decode b8 at KV {r['kv']}: {r['tps']:.1f} tok/s, {r['ms']:.3f} ms/step")

    mixed = None
    if not args.no_mixed:
        del eng
        torch.cuda.empty_cache()
        eng3, cfg3, _, wb3 = make_engine(args.mixed_config, None, args.mixed_requests, 2048 + args.mixed_output + 64, args.mixed_chunk)
        # the named workload: portions of exactly the chunk; then the engine's default, which lengthens portions
        # with budget that no other request can use
        eng3.scheduler.config.fill_budget = False
        mixed = mixed_workload(eng3, cfg3, wb3)
        points["mixed_output_tok_s"] = mixed["output_tok_s"]
        points["mixed_ttft_p50_ms"] = mixed["ttft_ms"]["p50"]
        points["mixed_ttft_p95_ms"] = mixed["ttft_ms"]["p95"]
        say(f"mixed {mixed}")
        eng3.scheduler.config.fill_budget = True
        filled = mixed_workload(eng3, cfg3, wb3)
        points["mixed_fill_budget_output_tok_s"] = filled["output_tok_s"]
        points["mixed_fill_budget_ttft_p50_ms"] = filled["ttft_ms"]["p50"]
        say(f"mixed, portions lengthened into spare budget {filled}")

    out = {
        "metric": f"decode tok/s at batch {args.batch} through the engine, {args.model_config} shape {dshort}, "
                  f"KV {head['kv'][0]}->{head['kv'][1]}",
        "value": round(head["tps"], 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(head["ms"], 4),
        "ms_per_step_p50": round(head["p50"], 4),
        "ms_per_step_p95": round(head["p95"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dshort,
        "data": "synthetic",
        "config": {
            "model": args.model_config, "layers": cfg.num_hidden_layers, "layers_full": full.num_hidden_layers,
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "prompt_len": args.prompt_len,
            "decode_from_kv": head["kv"][0],
            "page_size": args.page_size, "weights": "random N(0,0.02)", "parallelism": "single GPU",
            "graph": not args.no_graph, "steps_queued_ahead": not args.no_chain, "sampling": "greedy",
            "path": "Engine.add_request/step",
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
        "determinism": determinism,
        "mixed": mixed,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
