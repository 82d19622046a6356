"""The ``tempura`` command line.

The reference has ``serve | pull | list | inspect`` (/root/reference/cli/src/main.rs:18-34); serving
and downloading are out of this engine's scope, so the subcommands here are ``inspect`` (same
meaning), ``run`` (generate from token ids, the in-process core of ``serve``), ``random-model``
(write a random-weights folder) and ``replay`` (trace replay).  Option names follow the
reference's ``serve`` flags where it has them: ``--model``, ``--model-config``, ``--max-batch-size``,
``--max-seq-len`` (/root/reference/server/src/lib.rs:45-110); sampling options carry the names of
its ``SamplingParams`` (/root/reference/kernel-api/src/lib.rs:247-274).
"""
from __future__ import annotations

import argparse
import json
import random
import sys
import time


def _add_engine_args(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("model_dir", nargs="?", help="model folder (the same as --model)")
    ap.add_argument("--model", help="model folder (config.json + *.safetensors)")
    ap.add_argument("--model-config", "--preset", dest="model_config",
                    help="named size for --random-weights (see `tempura random-model --list`)")
    ap.add_argument("--random-weights", action="store_true", help="seeded N(0, 0.02) weights instead of a checkpoint")
    ap.add_argument("--seed", type=int, default=0, help="seed of random weights and default sampling seed")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "fp32"])
    ap.add_argument("--max-batch-size", type=int, default=32, help="requests running at once")
    ap.add_argument("--max-seq-len", type=int, default=4096, help="longest prompt + output")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--kv-blocks", type=int, default=None, help="cache pages (default: from free memory)")
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048, help="token budget of one step")
    ap.add_argument("--prefill-chunk-size", type=int, default=512,
                    help="a prompt's portion of one step while other prompts wait for theirs")
    ap.add_argument("--strict-chunks", action="store_true",
                    help="never lengthen a prompt portion with budget that nobody else can use")
    ap.add_argument("--no-graph", action="store_true", help="do not replay decode steps as a HIP graph")
    ap.add_argument("--no-chain-steps", action="store_true",
                    help="wait for a step's tokens on the host before queueing the next decode step")


def _engine_from_args(args):
    from .config import PRESETS
    from .engine import Engine
    if getattr(args, "model_dir", None):
        if args.model and args.model != args.model_dir:
            raise SystemExit(f"two model folders given: {args.model_dir!r} and --model {args.model!r}")
        args.model = args.model_dir
    if args.random_weights:
        if args.model_config:
            if args.model_config not in PRESETS:
                raise SystemExit(f"unknown --model-config {args.model_config!r}; known: {', '.join(sorted(PRESETS))}")
            model = PRESETS[args.model_config]
        elif args.model:
            model = args.model
        else:
            raise SystemExit("--random-weights needs --model-config NAME or --model DIR (for its config.json)")
    else:
        if not args.model:
            raise SystemExit("--model DIR is required (or --random-weights --model-config NAME)")
        model = args.model
    return Engine(model, dtype=args.dtype, random_weights=args.random_weights, seed=args.seed,
                  page_size=args.block_size, kv_pages=args.kv_blocks,
                  gpu_memory_utilization=args.gpu_memory_utilization, max_batch_size=args.max_batch_size,
                  max_seq_len=args.max_seq_len, max_num_batched_tokens=args.max_num_batched_tokens,
                  prefill_chunk_size=args.prefill_chunk_size, fill_budget=not args.strict_chunks, use_graph=not args.no_graph,
                  chain_steps=not args.no_chain_steps)


def _prompts_from_args(args, vocab: int):
    if args.prompt_ids:
        return [[int(t) for t in args.prompt_ids.replace(" ", "").split(",") if t]]
    if args.prompt_file:
        out = []
        with open(args.prompt_file) as f:
            for line in f:
                line = line.strip()
                if line:
                    out.append([int(t) for t in line.replace(",", " ").split()])
        return out
    if args.random_prompts:
        g = random.Random(args.seed)
        return [[g.randrange(vocab) for _ in range(args.prompt_len)] for _ in range(args.random_prompts)]
    raise SystemExit("give --prompt-ids, --prompt-file or --random-prompts N")


def cmd_run(args) -> int:
    from .sampling import SamplingParams
    eng = _engine_from_args(args)
    prompts = _prompts_from_args(args, eng.model.spec.vocab_size)
    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, min_p=args.min_p, typical_p=args.typical_p,
                            repeat_penalty=args.repeat_penalty, penalty_last_n=args.penalty_last_n,
                            presence_penalty=args.presence_penalty, frequency_penalty=args.frequency_penalty,
                            seed=args.sampling_seed, max_new_tokens=args.max_new_tokens,
                            eos_token_id=args.eos_token, ignore_eos=args.ignore_eos)
    if args.dump_logits:
        # The logits after each prompt's last token, from a fresh request that runs the whole prompt
        # (the reference's logits probe: /root/reference/server/src/api.rs:1154-1183; float32 little-endian
        # rows as /root/reference/tests-ggml/llama_logitprobe.cpp:20-30 writes them), [prompts, vocab].
        import numpy as np
        with open(args.dump_logits, "wb") as f:
            for p in prompts:
                f.write(np.ascontiguousarray(eng.forward(p).numpy(), dtype="<f4").tobytes())
    t0 = time.time()
    outs = eng.generate(prompts, params)
    dt = time.time() - t0
    for i, o in enumerate(outs):
        print(json.dumps({"request": i, "prompt_tokens": len(prompts[i]), "output_ids": o,
                          "finish_reason": eng.request(i).finish_reason}))
    if args.stats:
        s = eng.stats()
        s["seconds"] = round(dt, 4)
        s["output_tokens_per_second"] = round(s["generated_tokens"] / dt, 2) if dt > 0 else None
        print(json.dumps({"stats": s}), file=sys.stderr)
    return 0


def cmd_profile(args) -> int:
    """Per-entry-point times of one step of prompts and of a few decode steps, run eagerly with events around every
    call into the kernel library; with --layer-stats the residual stream's mean, variance and largest magnitude
    before every layer."""
    eng = _engine_from_args(args)
    rep = eng.profile(prompt_len=args.prompt_len, batch=args.batch, decode_steps=args.decode_steps,
                      layer_stats=args.layer_stats, seed=args.seed)
    if args.json:
        print(json.dumps(rep))
        return 0
    for phase, what in (("prefill", f"{args.batch} prompts of {args.prompt_len} tokens, one step"),
                        ("decode", f"{args.decode_steps} steps of {args.batch} tokens")):
        total = sum(r[2] for r in rep[phase])
        print(f"{phase} ({what}): {total / 1e3:.3f} ms in the kernel library")
        for name, calls, us, share in rep[phase]:
            print(f"  {name:40s} {calls:6d} calls {us:12.1f} us {100 * share:5.1f} %")
    if args.layer_stats:
        print("residual stream before each layer (and after the last): mean, variance, largest magnitude")
        for i, mean, var, top in rep["layers"]:
            print(f"  {i:4d} {mean: .4e} {var:.4e} {top:.4e}")
    return 0


def cmd_inspect(args) -> int:
    from .inspect import format_report, inspect
    info = inspect(args.path)
    print(json.dumps(info, indent=2) if args.json else format_report(info))
    return 0


def cmd_random_model(args) -> int:
    from .config import PRESETS, LlamaConfig
    from .weights import write_random_model
    if args.list:
        for name, cfg in sorted(PRESETS.items()):
            print(f"{name}: {cfg.num_hidden_layers} layers, hidden {cfg.hidden_size}, {cfg.num_parameters() / 1e6:.1f} M parameters")
        return 0
    if args.config_json:
        with open(args.config_json) as f:
            cfg = LlamaConfig.from_json(f.read())
    elif args.model_config in PRESETS:
        cfg = LlamaConfig.from_dict(PRESETS[args.model_config].to_dict())
    else:
        raise SystemExit(f"unknown --model-config {args.model_config!r}; known: {', '.join(sorted(PRESETS))}")
    if not args.out:
        raise SystemExit("--out DIR is required")
    write_random_model(cfg, args.out, seed=args.seed, std=args.std, dtype=args.dtype)
    print(args.out)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="tempura", description="Llama 3 inference on one MI355X")
    sub = ap.add_subparsers(dest="cmd", required=True)

    p = sub.add_parser("inspect", help="print what a model folder holds")
    p.add_argument("path")
    p.add_argument("--json", action="store_true")
    p.set_defaults(fn=cmd_inspect)

    p = sub.add_parser("run", help="generate from token ids")
    _add_engine_args(p)
    p.add_argument("--prompt-ids", help='one prompt: "1,2,3"')
    p.add_argument("--prompt-file", help="one prompt per line, ids separated by blanks or commas")
    p.add_argument("--random-prompts", type=int, default=0, help="N prompts of uniform random ids")
    p.add_argument("--prompt-len", type=int, default=128)
    p.add_argument("--max-new-tokens", type=int, default=256)
    p.add_argument("--temperature", type=float, default=1.0)
    p.add_argument("--top-k", type=int, default=50)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--min-p", type=float, default=0.0)
    p.add_argument("--typical-p", type=float, default=1.0)
    p.add_argument("--repeat-penalty", type=float, default=1.0)
    p.add_argument("--penalty-last-n", type=int, default=64)
    p.add_argument("--presence-penalty", type=float, default=0.0)
    p.add_argument("--frequency-penalty", type=float, default=0.0)
    p.add_argument("--sampling-seed", type=int, default=None)
    p.add_argument("--eos-token", type=int, action="append", default=None, help="stop token id (repeatable)")
    p.add_argument("--ignore-eos", action="store_true")
    p.add_argument("--stats", action="store_true", help="print counters to standard error")
    p.add_argument("--dump-logits", metavar="PATH",
                   help="write the logits after every prompt's last token to PATH (float32 little-endian, [prompts, vocab])")
    p.set_defaults(fn=cmd_run)

    p = sub.add_parser("random-model", help="write a folder with config.json and seeded random weights")
    p.add_argument("--model-config", default="tiny-a")
    p.add_argument("--config-json", help="a config.json to take the sizes from instead of a named size")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--std", type=float, default=0.02)
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "float16"])
    p.add_argument("--out")
    p.add_argument("--list", action="store_true")
    p.set_defaults(fn=cmd_random_model)

    p = sub.add_parser("profile", help="time every kernel-library call of a prompt step and of decode steps (eager)")
    _add_engine_args(p)
    p.add_argument("--prompt-len", type=int, default=128)
    p.add_argument("--batch", type=int, default=1, help="requests, all in one step")
    p.add_argument("--decode-steps", type=int, default=4)
    p.add_argument("--layer-stats", action="store_true", help="also the residual stream's statistics per layer")
    p.add_argument("--json", action="store_true")
    p.set_defaults(fn=cmd_profile)

    p = sub.add_parser("replay", help="trace replay (same as bin/trace_run)", add_help=False)
    p.set_defaults(fn=None)
    p = sub.add_parser("bench", help="decode and prefill throughput of a named size (bench.py of the checkout)", add_help=False)
    p.set_defaults(fn=None)

    if argv is None:
        argv = sys.argv[1:]
    if argv and argv[0] == "replay":
        from .replay import main as replay_main
        return replay_main(argv[1:])
    if argv and argv[0] == "bench":
        # bench.py lies beside the package in a checkout (the measuring harness calls it by that path)
        import os
        import runpy
        script = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py")
        if not os.path.isfile(script):
            raise SystemExit(f"tempura bench: {script} not found (it ships with the source checkout)")
        rest = list(argv[1:])
        if rest and not rest[0].startswith("-"):
            rest = ["--model-config", rest[0]] + rest[1:]       # `tempura bench llama-3.2-3b`
        sys.argv = [script] + rest
        try:
            runpy.run_path(script, run_name="__main__")
        except SystemExit as e:
            return int(e.code or 0)
        return 0
    args = ap.parse_args(argv)
    # what is wrong with a folder, a configuration, a checkpoint or the machine is one line and status 2
    # (TEMPURA_TRACEBACK=1 shows where it was raised)
    import os
    from .cache import PagesExhausted
    from .config import ConfigError
    from .engine.loading import NoDeviceError
    from .weights import SafetensorsError, WeightsError
    try:
        return args.fn(args)
    except NoDeviceError as e:
        print(f"tempura: {e}", file=sys.stderr)
        return 2
    except (ConfigError, WeightsError, SafetensorsError, PagesExhausted) as e:
        if os.environ.get("TEMPURA_TRACEBACK"):
            raise
        print(f"tempura: {type(e).__name__}: {e}", file=sys.stderr)
        return 2


if __name__ == "__main__":
    sys.exit(main())
