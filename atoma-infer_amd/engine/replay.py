"""Trace replay: feed given token ids through the model step by step and write logits.  Nothing is sampled.

It drives the same model, step function, cache and kernels as generation does.  Steps are read one JSON object a
line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step that wants logits, ``<out>/<step>.f32`` receives them as little-endian float32 [wanted, vocab], in the
order of the entries and of ``want``.  After every step a line ``done <step>`` is printed and flushed.
The reference has nothing comparable; its nearest relatives are the hand-built metadata loops of its model tests
(models/src/llama.rs:597-691).
"""
from __future__ import annotations

import json
import os
import sys
from typing import Dict, IO

import torch

from ..cache.manager import OutOfPages
from ..cache.pool import CachePool, pages_for_tokens, plan_cache
from ..models.model import load_model
from .step import ModelRunner, StepEntry

REPLAY_PAGE_SIZE = 16       # the engine's default block size ([cache] block_size)
REPLAY_MAX_LIVE = 16


def make_runner(model_dir: str, dtype: str, max_tokens: int, page_size: int = REPLAY_PAGE_SIZE,
                max_live: int = REPLAY_MAX_LIVE, device: str = "cuda:0") -> ModelRunner:
    model = load_model(model_dir, dtype, device)
    plan = plan_cache(model.spec)
    pages = pages_for_tokens(plan, page_size, max_tokens, max_live)
    pool = CachePool(plan, page_size, pages, max_live, model.act_dtype, model.device)
    return ModelRunner(model, pool)


def replay(runner: ModelRunner, lines: IO[str], out_dir: str, report: IO[str] = sys.stdout) -> int:
    os.makedirs(out_dir, exist_ok=True)
    ids: Dict[str, int] = {}
    next_id = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        obj = json.loads(line)
        step = obj["step"]
        entries = []
        for e in obj.get("entries", []):
            name = str(e["id"])
            if name not in ids:
                try:
                    runner.add_request(next_id)
                except OutOfPages:
                    raise SystemExit(f"trace_run: step {step} brings request '{name}' while {len(ids)} others are "
                                     f"live, which is all that --max-live allows") from None
                ids[name] = next_id
                next_id += 1
            rid = ids[name]
            entries.append(StepEntry(rid, [int(t) for t in e["tokens"]], runner.computed_len(rid),
                                     [int(w) for w in e.get("want", [])]))
        if entries:
            logits = runner.step(entries)
            if logits is not None:
                arr = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f"{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
            else:
                torch.cuda.synchronize()
        for name in obj.get("end", []):
            name = str(name)
            if name in ids:
                runner.free_request(ids.pop(name))
        print(f"done {step}", file=report, flush=True)
    return 0


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time, each request's count rounded up to a "
                         "multiple of 64 by the caller; the cache pool is made for this many")
    ap.add_argument("--page-size", type=int, default=REPLAY_PAGE_SIZE,
                    help=f"tokens a page of the cache (default {REPLAY_PAGE_SIZE}, the engine's [cache] block_size)")
    ap.add_argument("--max-live", type=int, default=REPLAY_MAX_LIVE,
                    help=f"most requests live at a time (default {REPLAY_MAX_LIVE})")
    args = ap.parse_args(argv)
    if args.page_size <= 0 or args.max_live <= 0 or args.max_tokens <= 0:
        ap.error("--max-tokens, --page-size and --max-live must be positive")
    print(f"[trace_run] loading {args.model} ({args.dtype})", file=sys.stderr, flush=True)
    runner = make_runner(args.model, args.dtype, args.max_tokens, args.page_size, args.max_live)
    return replay(runner, sys.stdin, args.out)
