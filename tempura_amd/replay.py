"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives
the same model, step function, cache manager and kernels that generation uses.
The reference's nearest pieces are its deterministic replay
(/root/reference/server/src/replay.rs:38-68) and its logits probes
(/root/reference/tests-ggml/llama_logitprobe.cpp:20-30); neither records how a
batch was composed, so the step-level format is this engine's own:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

one JSON object a line on standard input.  All entries of a step are one batch.
For a step in which something is wanted, ``<out>/<step>.f32`` holds the logits at
the wanted places in entry order, little-endian float32 [wanted, vocab].  After
every step a line ``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page (divides 64)")
    ap.add_argument("--max-requests", type=int, default=8)
    args = ap.parse_args(argv)
    if args.max_tokens <= 0:
        ap.error("--max-tokens must be positive")
    if args.page_size <= 0 or 64 % args.page_size != 0:
        ap.error("--page-size must divide 64")

    import torch
    from .cache import PagesExhausted
    from .engine.loading import load_model
    from .engine.runner import ModelRunner, StepEntry
    from .kernels import ops

    if not torch.cuda.is_available():
        print("trace_run: no GPU visible; there is no CPU path", file=sys.stderr)
        return 3
    ops.library()           # compile (first call) and load the kernels before touching the model
    os.makedirs(args.out, exist_ok=True)
    model = load_model(args.model, args.dtype, "cuda:0")
    num_pages = (args.max_tokens + args.page_size - 1) // args.page_size
    runner = ModelRunner(model, args.page_size, num_pages, args.max_requests)

    while True:
        line = sys.stdin.readline()
        if not line:
            break
        line = line.strip()
        if not line:
            continue
        # (a line that cannot be run ends the replay with one line on standard error and status 2; the steps
        # before it have been written)
        rec = None
        try:
            rec = json.loads(line)
            step = rec["step"]
            entries = []
            for e in rec.get("entries", []):
                rid = e["id"]
                if not runner.has_request(rid):
                    runner.add_request(rid)
                entries.append(StepEntry(rid, [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
            logits = runner.step(entries) if entries else None
        except (ValueError, KeyError, TypeError, PagesExhausted) as err:
            what = f"step {rec['step']}" if isinstance(rec, dict) and "step" in rec else f"line {line[:60]!r}"
            print(f"trace_run: {what}: {type(err).__name__}: {err}", file=sys.stderr)
            return 2
        if entries:
            if logits.shape[0] > 0:
                arr = logits.detach().to("cpu", torch.float32).numpy().astype("<f4", copy=False)
                tmp = os.path.join(args.out, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
            else:
                torch.cuda.synchronize()
        for rid in rec.get("end", []):
            if runner.has_request(rid):
                runner.end_request(rid)
        sys.stdout.write(f"done {step}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
