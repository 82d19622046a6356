#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Llama-3.1-8B shape, bfloat16,
random weights, synthetic token ids.

    python bench.py --gpus 1 --steps K --warmup W

A "step" is one decode step of the whole batch (default 8 requests whose caches hold 2,048
tokens each when timing starts; context limit 4,096).  Prints ONE JSON line: decoded tokens per
second (`value`), the 2,048-token prefill, the decode step's share of the HBM roofline, and the
batch-1 and batch-64 points.  The reference measures the same two things its own way (prefill of a
synthetic prompt, then timed single-token forwards, /root/reference/tools/bench-gpu/src/bench_real_model.rs:160-278).
"""
from __future__ import annotations

import argparse
import copy
import json
import os
import random
import sys
import time

HBM_PEAK_GBS = 8000.0                                   # MI355X HBM3E, published
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense, published


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000, help="timed decode steps (KV grows from 2,048 towards 4,096)")
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
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 points")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--point-steps", type=int, default=1000, help="timed steps of the batch-1 and batch-64 points")
    ap.add_argument("--decode-target-blocks", type=int, default=None, help="tuning: blocks the split decode attention aims at")
    return ap.parse_args()


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (this engine has no multi-GPU path); --gpus {args.gpus} is not supported")
        return 2

    import torch
    from tempura_amd.config import PRESETS, LlamaConfig
    from tempura_amd.engine.loading import random_model
    from tempura_amd.engine.runner import ModelRunner, StepEntry
    from tempura_amd.kernels import ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    if args.decode_target_blocks:
        ops.decode_target_blocks = args.decode_target_blocks
    full = PRESETS[args.model_config]
    cfg = LlamaConfig.from_dict(full.to_dict())
    if args.layers is not None:
        cfg.num_hidden_layers = args.layers
    cfg.validate()
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    steps, warmup = args.steps, args.warmup
    if args.prompt_len + warmup + steps > args.context:
        steps = max(1, args.context - args.prompt_len - warmup)

    t0 = time.time()
    model = random_model(cfg, seed=0, dtype=args.dtype, device="cuda:0")
    torch.cuda.synchronize()
    print(f"[bench] model built in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    pages = max_batch * ((args.context + args.page_size - 1) // args.page_size) + 8
    runner = ModelRunner(model, args.page_size, pages, max_requests=max_batch, use_graph=not args.no_graph)
    if not runner.use_graph:
        args.no_chain = True          # (a step can only be queued ahead of its tokens where steps replay a graph)
    rng = random.Random(0)
    V = cfg.vocab_size
    elem = 2 if args.dtype == "bfloat16" else 4
    kv_per_token = cfg.kv_bytes_per_token(elem)
    weight_bytes = model.weight_bytes(include_embedding=False)
    if model.lm_head.tied:
        weight_bytes += model.embedding.weight.numel() * model.embedding.weight.element_size()

    def prompt(n):
        return [rng.randrange(V) for _ in range(n)]

    # ---- prefill of one 2,048-token prompt -------------------------------------------------
    prefill = None
    if not args.no_prefill:
        T = args.prompt_len
        times = []
        for i in range(2 + 5):
            rid = ("p", i)
            runner.add_request(rid)
            toks = prompt(T)
            torch.cuda.synchronize()
            t = time.perf_counter()
            lg = runner.step([StepEntry(rid, toks, [T - 1])])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            runner.end_request(rid)
            if i >= 2:
                times.append(dt)
        ms = 1e3 * sum(times) / len(times)
        L, H, I = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size
        qd, kvd = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
        linear = L * (H * (qd + 2 * kvd) + qd * H + 3 * H * I)
        flops = 2.0 * T * linear + 2.0 * V * H + L * 4.0 * cfg.num_attention_heads * cfg.head_dim * T * (T + 1) / 2
        peak = MFMA_PEAK["bf16" if args.dtype == "bfloat16" else "fp32"]
        prefill = {"value": round(T / (ms / 1e3), 1), "tokens": T, "ms": round(ms, 3),
                   "frac": round(flops / (ms / 1e3) / peak, 4)}
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- decode -----------------------------------------------------------------------------
    def decode_run(batch, n_warm, n_steps):
        rids = [("d", batch, i) for i in range(batch)]
        for rid in rids:
            runner.add_request(rid)
            runner.step([StepEntry(rid, prompt(args.prompt_len), [])])
        # The first step takes its tokens from the host; from then on a step takes the tokens the argmax kernel
        # chose (still on the device) and is queued behind it at once, while the tokens of the step before
        # travel to the host, where serving needs them one step later (the engine's loop does the same).
        lg = runner.step([StepEntry(rid, [rng.randrange(V)], [0]) for rid in rids])
        chosen = ops.argmax(lg)
        coming = ops.HostCopy(chosen)
        seen = []

        def one():
            nonlocal chosen, coming
            if args.no_chain:                       # (for comparison: wait for the tokens, then queue the step)
                lg = runner.step([StepEntry(rid, [t], [0]) for rid, t in zip(rids, coming.result())])
                chosen = ops.argmax(lg)
                coming = ops.HostCopy(chosen)
                return
            lg = runner.step_chained(rids, chosen)
            nxt = ops.argmax(lg)
            nxt_coming = ops.HostCopy(nxt)
            runner.prepare_decode(rids)             # stage the step after this one while the GPU works
            seen.append(coming.result()[0])         # the tokens of the step before, on the host
            chosen, coming = nxt, nxt_coming

        for _ in range(n_warm):
            one()
        torch.cuda.synchronize()
        ctx0 = runner.num_cached(rids[0])
        t = time.perf_counter()
        for _ in range(n_steps):
            one()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        for rid in rids:
            runner.end_request(rid)
        mean_ctx = ctx0 + (n_steps + 1) / 2.0
        bytes_step = weight_bytes + batch * mean_ctx * kv_per_token
        return batch * n_steps / dt, 1e3 * dt / n_steps, bytes_step

    tps, ms_step, bytes_step = decode_run(args.batch, warmup, steps)
    print(f"[bench] decode b{args.batch}: {tps:.1f} tok/s, {ms_step:.3f} ms/step", file=sys.stderr, flush=True)
    achieved = bytes_step / (ms_step / 1e3) / 1e9
    points = {}
    if not args.no_points:
        for b in (1, 64):
            ps = min(args.point_steps, steps, args.context - args.prompt_len - 8)
            p_tps, p_ms, _ = decode_run(b, 8, ps)
            points[f"decode_b{b}"] = round(p_tps, 1)
            print(f"[bench] decode b{b}: {p_tps:.1f} tok/s, {p_ms:.3f} ms/step", file=sys.stderr, flush=True)

    out = {
        "metric": f"decode tok/s at batch {args.batch}, {args.model_config} shape {'bf16' if args.dtype == 'bfloat16' else 'fp32'}, "
                  f"KV {args.prompt_len}->{args.context}",
        "value": round(tps, 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic",
        "config": {
            "model": args.model_config, "layers": cfg.num_hidden_layers, "layers_full": full.num_hidden_layers,
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "prompt_len": args.prompt_len,
            "page_size": args.page_size, "weights": "random N(0,0.02)", "parallelism": "single GPU",
            "graph": not args.no_graph, "steps_queued_ahead": not args.no_chain,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
