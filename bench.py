#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Llama-3.2-1B sizes with random weights, on one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--sizes 1b|3b|8b] [--layers N]
    python bench.py --workload serve3b|long8b [--layers N] [--requests R]

A "step" is one decode step of the whole engine (scheduler, step function, sampler).  The default run has the
layer sizes of Llama-3.2-1B (16 layers, width 2048, 32 heads over 8 KV heads of 64, feed-forward 8192, vocabulary
128256, llama3 rope scaling, tied head), bfloat16, random weights N(0, 0.02), 2048-token prompts of uniform random
token ids, a batch of 8, and a maximum context of 8192.  It prints ONE JSON line: decoded tokens a second as
``value``, plus the 2048-token prefill, the decode step's roofline fraction (bytes it has to read / time / 8 TB/s)
and decode throughput at batch 1 and 64; the read and copy bandwidth and the MFMA rate that this GPU delivers,
measured by small probes, stand beside the published peaks (which stay the yardstick of every fraction).

``--workload`` runs one of the other two workloads instead and prints ONE line of its own:
``serve3b``: Llama-3.2-3B sizes, 64 requests with prompt lengths uniform in [128, 4096] (seeded), 256 generated tokens
each, continuous batching with chunked prefill under 2,048 tokens a step; ``long8b``: Llama-3.1-8B sizes, 16 requests
of 32,768 tokens of context (32,512 of prompt, 256 generated), prompts in 2,048-token portions beside decoding
requests.  ``value`` is generated tokens a second over the whole run, prompts included.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

LLAMA_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 2048, "intermediate_size": 8192, "vocab_size": 128256, "num_hidden_layers": 16,
    "num_attention_heads": 32, "num_key_value_heads": 8, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192, "rope_type": "llama3"},
    "max_position_embeddings": 131072, "tie_word_embeddings": True,
}
# other members of the family, for measurements beside the default (``--sizes``): what differs from LLAMA_1B
OTHER_SIZES = {
    "3b": dict(hidden_size=3072, num_attention_heads=24, num_key_value_heads=8, intermediate_size=8192,
               num_hidden_layers=28),
    "8b": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, intermediate_size=14336,
               num_hidden_layers=32, tie_word_embeddings=False,
               rope_scaling=dict(LLAMA_1B["rope_scaling"], factor=8.0)),
}


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def make_engine(model, batch, context, page=16):
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig, ValidationConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    pages = batch * (-(-context // page)) + 8
    return LlmEngine(model, cache=CacheConfig(block_size=page, num_gpu_blocks_override=pages),
                     scheduler=SchedulerConfig(max_num_batched_tokens=max(2048, batch), max_num_sequences=max(batch, 1),
                                               max_model_len=context, enable_chunked_prefill=True),
                     validation=ValidationConfig(max_input_length=context - 1, max_total_tokens=context))


def decode_run(model, batch, prompt_len, steps, warmup, context, seed=0, sampling=None):
    """Prefill ``batch`` prompts (untimed), then time ``steps`` decode steps.  Returns (seconds, mean context)."""
    import torch
    from atoma_infer_amd.sampling import GenerateParameters
    eng = make_engine(model, batch, context)
    g = torch.Generator().manual_seed(seed)
    vocab = model.vocab_size
    # requests that finish their prompt early decode while the others are still in theirs
    # (the decoded tokens share the step's budget with the prompts, hence the factor of two)
    prompt_steps = 2 * batch * (-(-prompt_len // max(2048, batch)))
    params = GenerateParameters(do_sample=False, max_new_tokens=steps + warmup + prompt_steps + 8,
                                ignore_eos_token=True)
    if sampling:        # (temperature, top_k, top_p): draw instead of the default argmax
        params = GenerateParameters(do_sample=True, temperature=sampling[0], top_k=sampling[1] or None,
                                    top_p=sampling[2] if sampling[2] < 1.0 else None,
                                    random_seed=seed, max_new_tokens=params.max_new_tokens, ignore_eos_token=True)
    for _ in range(batch):
        eng.add_request(torch.randint(0, vocab, (prompt_len,), generator=g).tolist(), params)
    while any(r.in_prefill for r in eng.scheduler.running) or eng.scheduler.waiting:
        eng.step()
    for _ in range(warmup):
        eng.step()
    eng.drain()
    ctx0 = sum(r.length for r in eng.scheduler.running)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.step()
    eng.drain()             # the engine runs one step ahead of the sampled tokens: read the last ones too
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(r.length for r in eng.scheduler.running)
    assert len(eng.scheduler.running) == batch, "a request ended or was preempted during the timed steps"
    mean_ctx = (ctx0 + ctx1) / 2.0 / batch
    del eng
    torch.cuda.empty_cache()
    return dt, mean_ctx


def prefill_run(model, n_tokens, reps, context):
    import torch
    from atoma_infer_amd.cache import CachePool, plan_cache
    from atoma_infer_amd.engine import ModelRunner, StepEntry
    plan = plan_cache(model.spec)
    pool = CachePool(plan, 16, [(-(-n_tokens // 16)) + 4] * len(plan.groups), 4, model.act_dtype, model.device)
    runner = ModelRunner(model, pool)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, model.vocab_size, (n_tokens,), generator=g).tolist()
    times = []
    for i in range(reps + 1):
        runner.add_request(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry(i, toks, 0, [n_tokens - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.free_request(i)
    del runner, pool
    torch.cuda.empty_cache()
    return min(times[1:])


WORKLOADS = {
    # name: (sizes, requests, shortest prompt, longest prompt, generated tokens, tokens a step)
    "serve3b": ("3b", 64, 128, 4096, 256, 2048),
    "long8b": ("8b", 16, 32768 - 256, 32768 - 256, 256, 2048),
}


def serve_run(model, n_req, lo, hi, out_tokens, budget, seed=3):
    """All requests arrive at once; the engine runs them to their end.  Returns what was measured."""
    import random

    import torch
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig, ValidationConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling import GenerateParameters
    rnd = random.Random(seed)
    lens = [rnd.randint(lo, hi) for _ in range(n_req)]
    ctx = hi + out_tokens + 16
    pages = sum(-(-(n + out_tokens) // 16) + 1 for n in lens) + 64
    eng = LlmEngine(model, cache=CacheConfig(block_size=16, num_gpu_blocks_override=pages),
                    scheduler=SchedulerConfig(max_num_batched_tokens=budget, max_num_sequences=n_req,
                                              max_model_len=ctx, enable_chunked_prefill=True),
                    validation=ValidationConfig(max_input_length=ctx - 1, max_total_tokens=ctx))
    g = torch.Generator().manual_seed(1)
    params = GenerateParameters(do_sample=False, max_new_tokens=out_tokens, ignore_eos_token=True)
    for n in lens:
        eng.add_request(torch.randint(0, model.vocab_size, (n,), generator=g).tolist(), params)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps, done, times, last = 0, 0, [], t0
    while eng.has_unfinished():
        done += len(eng.step())
        now = time.perf_counter()
        times.append(now - last)
        last = now
        steps += 1
        if steps % 200 == 0:
            log(f"  step {steps}: {done} of {n_req} requests done, {now - t0:.1f} s")
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    times.sort()
    assert done == n_req
    return {"seconds": dt, "prompt_tokens": sum(lens), "generated": n_req * out_tokens, "steps": steps,
            "preemptions": eng.stats["preemptions"], "step_median_ms": times[len(times) // 2] * 1e3,
            "step_p99_ms": times[int(len(times) * 0.99)] * 1e3}


def workload_main(args) -> int:
    import atoma_infer_amd  # noqa: F401
    from atoma_infer_amd.models import random_model
    sizes, n_req, lo, hi, out_tokens, budget = WORKLOADS[args.workload]
    n_req = args.requests or n_req
    base = dict(LLAMA_1B, **OTHER_SIZES[sizes])
    full_layers = base["num_hidden_layers"]
    layers = args.layers or full_layers
    name = {"3b": "Llama-3.2-3B", "8b": "Llama-3.1-8B"}[sizes]
    log(f"{args.workload}: building {name} sizes ({layers} of {full_layers} layers, random weights) ...")
    model = random_model(dict(base, num_hidden_layers=layers), seed=0, dtype="bfloat16", stored="bfloat16")
    log(f"{n_req} requests, prompts of {lo} to {hi} tokens, {out_tokens} generated each, {budget} tokens a step ...")
    r = serve_run(model, n_req, lo, hi, out_tokens, budget)
    c = model.config
    line = {
        "metric": f"generated tok/s, workload {args.workload} ({name} sizes, {n_req} requests, continuous batching "
                  f"with chunked prefill)",
        "value": round(r["generated"] / r["seconds"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": r["steps"],
        "warmup": 0, "ms_per_step": round(r["seconds"] / r["steps"] * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (uniform random token ids, random weights N(0, 0.02))",
        "config": {"model": name + " sizes", "layers": layers, "layers_full": full_layers, "hidden": c.hidden_size,
                   "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads, "head_dim": c.head_size,
                   "intermediate": c.intermediate_size, "vocab": c.vocab_size, "requests": n_req,
                   "prompt_min": lo, "prompt_max": hi, "generated_each": out_tokens, "tokens_a_step": budget,
                   "kv_block": 16, "sampling": "argmax", "parallelism": "single GPU"},
        "total_tokens_per_s": round((r["prompt_tokens"] + r["generated"]) / r["seconds"], 1),
        "prompt_tokens": r["prompt_tokens"], "generated_tokens": r["generated"], "seconds": round(r["seconds"], 3),
        "preemptions": r["preemptions"], "step_median_ms": round(r["step_median_ms"], 3),
        "step_p99_ms": round(r["step_p99_ms"], 3),
    }
    print(json.dumps(line), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--sizes", choices=["1b", "3b", "8b"], default="1b",
                    help="layer sizes of Llama-3.2-1B (the default run), Llama-3.2-3B or Llama-3.1-8B")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (default: all)")
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 runs")
    ap.add_argument("--temperature", type=float, default=0.0,
                    help="sample with this temperature (and --top-k, --top-p) instead of the default argmax")
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--workload", choices=["decode", *WORKLOADS], default="decode",
                    help="decode: the default run; serve3b, long8b: the other two workloads, one line of their own")
    ap.add_argument("--requests", type=int, default=0, help="requests of a --workload run (default: the workload's)")
    ap.add_argument("--no-peaks", action="store_true", help="skip the probes of what the GPU delivers")
    ap.add_argument("--chain-floors", action="store_true",
                    help="only measure what a chain of dependent kernels costs beyond its bytes (an empty kernel, read "
                         "streams of 8 to 64 MB, a grid-wide barrier), print one JSON line and stop")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2
    if int(os.environ.get("WORLD_SIZE", "1")) > 1:
        print("bench.py: started with WORLD_SIZE > 1; this engine runs on one GPU", flush=True)
        return 2
    if args.chain_floors:
        import atoma_infer_amd  # noqa: F401
        from atoma_infer_amd.kernels.ops import measure_chain_floors
        print(json.dumps({"chain_floors": measure_chain_floors(), "unit": "us a kernel"}), flush=True)
        return 0
    if args.workload != "decode":
        return workload_main(args)
    if args.prompt_len + args.steps + args.warmup + 2 * args.batch * (-(-args.prompt_len // 2048)) + 8 > args.context:
        print("bench.py: prompt + steps exceed the context", file=sys.stderr)
        return 1

    import torch
    import atoma_infer_amd  # noqa: F401
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.models import random_model

    base = dict(LLAMA_1B, **OTHER_SIZES.get(args.sizes, {}))
    full_layers = base["num_hidden_layers"]
    args.layers = args.layers or full_layers
    cfg = dict(base, num_hidden_layers=args.layers)
    name = {"1b": "Llama-3.2-1B", "3b": "Llama-3.2-3B", "8b": "Llama-3.1-8B"}[args.sizes]
    log(f"building the model ({args.layers} layers, random weights) ...")
    t0 = time.time()
    model = random_model(cfg, seed=0, dtype="bfloat16", stored="bfloat16")
    log(f"model ready in {time.time() - t0:.1f} s; weights read per step: {model.weight_bytes() / 1e6:.1f} MB")
    kv_bytes_per_token = plan_cache(model.spec).bytes_per_token(2)

    log(f"prefill of {args.prefill_tokens} tokens ...")
    pre_s = prefill_run(model, args.prefill_tokens, 8, args.context)
    c = model.config
    hd = c.head_size
    layer_params = (c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * hd
                    + c.num_attention_heads * hd * c.hidden_size + 3 * c.hidden_size * c.intermediate_size)
    t = args.prefill_tokens
    pre_flops = (2.0 * t * layer_params * c.num_hidden_layers
                 + 4.0 * (t * (t + 1) / 2.0) * hd * c.num_attention_heads * c.num_hidden_layers
                 + 2.0 * c.hidden_size * c.vocab_size)
    prefill = {"value": round(t / pre_s, 1), "tokens": t, "ms": round(pre_s * 1e3, 3),
               "frac": round(pre_flops / pre_s / PEAK_FLOPS["bf16"], 4)}

    log(f"decode at batch {args.batch}: {args.warmup} warm-up + {args.steps} timed steps ...")
    sampling = (args.temperature, args.top_k, args.top_p) if args.temperature > 0 else None
    dt, mean_ctx = decode_run(model, args.batch, args.prompt_len, args.steps, args.warmup, args.context,
                              sampling=sampling)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = model.weight_bytes() + kv_bytes_per_token * mean_ctx * args.batch
    achieved = step_bytes / (dt / args.steps) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4)}

    points = {}
    if not args.no_points:
        for b, st in ((1, min(args.steps, 128)), (64, min(args.steps, 64))):
            log(f"decode at batch {b} ...")
            d, ctx_b = decode_run(model, b, args.prompt_len, st, min(args.warmup, 4), args.context, sampling=sampling)
            points[f"decode_b{b}"] = round(b * st / d, 1)
            # the same roofline fraction as the headline's, with this batch's own mean context
            bytes_b = model.weight_bytes() + kv_bytes_per_token * ctx_b * b
            points[f"decode_b{b}_frac"] = round(bytes_b / (d / st) / 1e9 / HBM_PEAK_GBS, 4)

    # the probes of what the GPU delivers run last: minutes of full load before the timed steps would only warm the
    # chip against them
    peaks = {}
    if not args.no_peaks:
        from atoma_infer_amd.kernels.ops import measure_device_peaks
        log("probing what the GPU delivers (read stream, copy, MFMA loop) ...")
        peaks = measure_device_peaks(model.device)
        log(f"  {peaks}")
    if peaks:
        # what the probes reached on this GPU, beside the published peaks that the fractions above are of
        roofline["measured_peak"] = peaks["hbm_read_gbs"]
        roofline["measured_how"] = peaks.get("hbm_read_how", "")
        roofline["measured_copy"] = peaks["hbm_copy_gbs"]
        roofline["frac_of_measured"] = round(achieved / peaks["hbm_read_gbs"], 4)
        prefill["measured_peak_tflops"] = peaks["mfma_bf16_tflops"]
        prefill["frac_of_measured"] = round(pre_flops / pre_s / (peaks["mfma_bf16_tflops"] * 1e12), 4)

    line = {
        "metric": f"decode tok/s at batch {args.batch} ({name} sizes, {args.prompt_len}-token prompts); "
                  "points: batch 1 and 64; prefill tok/s at 2048 tokens",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (uniform random token ids, random weights N(0, 0.02))",
        "config": {"model": name + " sizes",
                   "layers": args.layers, "layers_full": full_layers,
                   "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "head_dim": hd, "intermediate": c.intermediate_size, "vocab": c.vocab_size,
                   "global_batch": args.batch, "seq_len": args.prompt_len, "context": args.context,
                   "mean_decode_context": round(mean_ctx, 1), "kv_block": 16, "sampling": ("argmax" if not sampling else f"T={sampling[0]} top_k={sampling[1]} top_p={sampling[2]}"),
                   "tied_embeddings": bool(base["tie_word_embeddings"]),
                   "parallelism": "single GPU"},
        "prefill": prefill, "roofline": roofline, "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
