"""Command line.

    python -m atoma_infer_amd generate --config-path engine.toml --requests requests.jsonl
    python -m atoma_infer_amd generate --model DIR --dtype bf16 --prompt-ids 1,2,3 --max-new-tokens 16
    python -m atoma_infer_amd random-weights --config config.json --out DIR --seed 0
    python -m atoma_infer_amd replay --model DIR --dtype float32 --out DIR --max-tokens 4096 [--page-size P] [--max-live L] < trace.jsonl

``--config-path`` is the reference's one flag (server/src/main.rs:22-27): a TOML file with the sections
[inference], [cache], [scheduler] and [validation].  A line of ``--requests`` is the reference's
``GenerateRequest`` (backends/vllm/src/types.rs:17-27): ``{"request_id", "inputs", "parameters": {...}}``, where
``inputs`` is a string (needs tokenizer.json) or a list of token ids.  Each finished request is printed as one
JSON line shaped like the reference's ``GenerateRequestOutput``.
"""
from __future__ import annotations

import argparse
import dataclasses
import json
import sys


def _engine(args):
    from .config.engine import CacheConfig, EngineConfig, SchedulerConfig
    from .engine.engine import LlmEngine
    if args.config_path:
        cfg = EngineConfig.from_toml(args.config_path)
        if args.model:
            cfg.inference.model_name = args.model
        return LlmEngine.from_config(cfg)
    if not args.model:
        raise SystemExit("give --config-path or --model")
    cache = CacheConfig(block_size=args.block_size, gpu_memory_utilization=args.gpu_memory_utilization,
                        num_gpu_blocks_override=args.num_gpu_blocks_override)
    sched = SchedulerConfig(max_num_batched_tokens=args.max_num_batched_tokens,
                            max_num_sequences=args.max_num_sequences, max_model_len=args.max_model_len)
    eng = LlmEngine(args.model, args.dtype, cache=cache, scheduler=sched)
    eng.load_tokenizer(args.model)
    return eng


def _cmd_generate(args) -> int:
    from .sampling.params import GenerateParameters
    eng = _engine(args)
    fields = {f.name for f in dataclasses.fields(GenerateParameters)}
    jobs = []
    if args.requests:
        with (sys.stdin if args.requests == "-" else open(args.requests)) as f:
            for line in f:
                if line.strip():
                    o = json.loads(line)
                    p = {k: v for k, v in (o.get("parameters") or {}).items() if k in fields}
                    jobs.append((o.get("request_id"), o["inputs"], GenerateParameters(**p)))
    base = GenerateParameters(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                              do_sample=not args.greedy, max_new_tokens=args.max_new_tokens,
                              random_seed=args.random_seed, repetition_penalty=args.repetition_penalty,
                              repeat_last_n=args.repeat_last_n, ignore_eos_token=args.ignore_eos_token)
    for ids in args.prompt_ids or []:
        jobs.append((None, [int(t) for t in ids.replace(",", " ").split()], base))
    for text in args.prompt or []:
        jobs.append((None, text, base))
    if not jobs:
        raise SystemExit("nothing to generate: give --requests, --prompt-ids or --prompt")
    for rid, inputs, p in jobs:
        eng.add_request(inputs, p, rid)
    while eng.has_unfinished():
        for out in eng.step():
            print(json.dumps(dataclasses.asdict(out)), flush=True)
    print(json.dumps({"stats": eng.stats}), file=sys.stderr)
    return 0


def _cmd_random(args) -> int:
    from .weights import write_random_model
    with open(args.config) as f:
        cfg = json.load(f)
    write_random_model(args.out, cfg, seed=args.seed, dtype=args.store_dtype, norm_jitter=args.norm_jitter)
    print(args.out)
    return 0


def _cmd_replay(args) -> int:
    from .engine.replay import main as replay_main
    argv = ["--model", args.model, "--dtype", args.dtype, "--out", args.out, "--max-tokens", str(args.max_tokens)]
    if args.page_size is not None:
        argv += ["--page-size", str(args.page_size)]
    if args.max_live is not None:
        argv += ["--max-live", str(args.max_live)]
    return replay_main(argv)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="atoma_infer_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)

    g = sub.add_parser("generate", help="run requests to their end")
    g.add_argument("--config-path", help="engine TOML: [inference] [cache] [scheduler] [validation]")
    g.add_argument("--model", help="model folder (overrides [inference] model_name)")
    g.add_argument("--dtype", default="bf16", help="bf16 or f32")
    g.add_argument("--block-size", type=int, default=16)
    g.add_argument("--gpu-memory-utilization", type=float, default=0.5)
    g.add_argument("--num-gpu-blocks-override", type=int, default=None)
    g.add_argument("--max-num-batched-tokens", type=int, default=2048)
    g.add_argument("--max-num-sequences", type=int, default=64)
    g.add_argument("--max-model-len", type=int, default=8192)
    g.add_argument("--requests", help="JSON lines of GenerateRequest objects ('-': standard input)")
    g.add_argument("--prompt-ids", action="append", help="token ids, comma or space separated (repeatable)")
    g.add_argument("--prompt", action="append", help="text (needs tokenizer.json; repeatable)")
    g.add_argument("--temperature", type=float, default=None)
    g.add_argument("--top-k", type=int, default=None)
    g.add_argument("--top-p", type=float, default=None)
    g.add_argument("--greedy", action="store_true", help="do_sample = false")
    g.add_argument("--max-new-tokens", type=int, default=100)
    g.add_argument("--random-seed", type=int, default=None)
    g.add_argument("--repetition-penalty", type=float, default=None)
    g.add_argument("--repeat-last-n", type=int, default=None)
    g.add_argument("--ignore-eos-token", action="store_true")
    g.set_defaults(fn=_cmd_generate)

    r = sub.add_parser("random-weights", help="write config.json and model.safetensors with random weights")
    r.add_argument("--config", required=True, help="a config.json")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--store-dtype", default="bfloat16", choices=["bfloat16", "float32"])
    r.add_argument("--norm-jitter", type=float, default=0.0)
    r.set_defaults(fn=_cmd_random)

    t = sub.add_parser("replay", help="trace replay (same as bin/trace_run)")
    t.add_argument("--model", required=True)
    t.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    t.add_argument("--out", required=True)
    t.add_argument("--max-tokens", type=int, required=True)
    t.add_argument("--page-size", type=int, default=None, help="tokens a page of the cache (bin/trace_run's default)")
    t.add_argument("--max-live", type=int, default=None, help="most requests live at a time (bin/trace_run's default)")
    t.set_defaults(fn=_cmd_replay)

    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
