"""Generation through the entry points: greedy tokens against the plain implementation, sampling kernels against
the plain sampling functions, the scheduler under page pressure on the GPU, and bin/trace_run as a program."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama
from util import (NORM_JITTER, TINY, TOL_BF16, TOL_F32, check_greedy_tokens, frob_err, make_model_dir, plain_config,
                  plain_weights, random_tokens, rel_err)

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    return {name: make_model_dir(str(tmp_path_factory.mktemp(f"gen_{name}")), cfg, seed=21, dtype="bfloat16",
                                 norm_jitter=NORM_JITTER[name]) for name, cfg in TINY.items()}


def engine(model_dir, dtype, page, pages, **sched):
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    sched.setdefault("max_num_batched_tokens", 64)
    sched.setdefault("max_num_sequences", 4)
    sched.setdefault("max_model_len", 128)
    return LlmEngine(model_dir, dtype, cache=CacheConfig(block_size=page, num_gpu_blocks_override=pages),
                     scheduler=SchedulerConfig(**sched))


def test_greedy_generation_tiny_a_workload(model_dirs):
    """The tiny workload A: 2 prompts of 8 and 5 ids, 8 greedy steps each, float32, block size 4."""
    from atoma_infer_amd.sampling import GenerateParameters
    d = model_dirs["A"]
    w, cfg = plain_weights(d), plain_config(d)
    prompts = [random_tokens(8, 512, 1), random_tokens(5, 512, 2)]
    want = [plain_llama.greedy_generate(p, 8, w, cfg) for p in prompts]
    eng = engine(d, "float32", 4, 16)
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=8, ignore_eos_token=True))
    assert [o.inference_outputs[0].token_ids for o in outs] == want
    assert all(o.is_finished and o.inference_outputs[0].finish_reason == "length_capped" for o in outs)
    assert eng.runner.manager.num_free_pages() == 16 and eng.runner.manager.num_requests() == 0
    # the function-style entry point gives the same
    from atoma_infer_amd import generate
    from atoma_infer_amd.config import CacheConfig
    outs2 = generate(d, prompts, GenerateParameters(do_sample=False, max_new_tokens=8, ignore_eos_token=True),
                     dtype="float32", cache=CacheConfig(block_size=4, num_gpu_blocks_override=16))
    assert [o.inference_outputs[0].token_ids for o in outs2] == want


def test_engine_with_every_option_at_its_default(model_dirs):
    """No option given: the pool is sized from the memory that is free, capped at what the scheduler's limits can
    ever use, and generation is that of the plain model."""
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling import GenerateParameters
    d = model_dirs["C"]
    w, cfg = plain_weights(d), plain_config(d)
    prompts = [random_tokens(40, TINY["C"]["vocab_size"], 5), random_tokens(3, TINY["C"]["vocab_size"], 6)]
    want = [plain_llama.greedy_generate(p, 6, w, cfg) for p in prompts]
    eng = LlmEngine(d, "float32")
    sched, mgr = eng.scheduler_config, eng.runner.manager
    assert sched.max_model_len == TINY["C"]["max_position_embeddings"]        # the model's own limit caps the default
    assert mgr.num_pages() == sched.max_num_sequences * -(-sched.max_model_len // eng.cache_config.block_size)
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=6, ignore_eos_token=True))
    assert [o.inference_outputs[0].token_ids for o in outs] == want
    assert mgr.num_free_pages() == mgr.num_pages()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cache_option_sliding_window(model_dirs, dtype):
    """``[cache] sliding_window``: every layer attends the last N keys only, and pages that the window has passed
    go back while the request runs, so a pool far smaller than the sequences serves them."""
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling import GenerateParameters
    d, window = model_dirs["C"], 40
    w, cfg = plain_weights(d), dict(plain_config(d), sliding_window=window)
    vocab = TINY["C"]["vocab_size"]
    prompts = [random_tokens(200, vocab, 11), random_tokens(90, vocab, 12)]
    eng = LlmEngine(d, dtype, cache=CacheConfig(block_size=16, num_gpu_blocks_override=12, sliding_window=window),
                    scheduler=SchedulerConfig(max_num_batched_tokens=32, max_num_sequences=2, max_model_len=400))
    assert eng.model.config.sliding_window == window
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=30, ignore_eos_token=True))
    assert eng.stats["preemptions"] == 0          # 230 and 120 tokens would need 23 pages without the window
    assert eng.runner.manager.num_free_pages() == 12
    for p, o in zip(prompts, outs):
        got = o.inference_outputs[0].token_ids
        if dtype == "float32":
            assert got == plain_llama.greedy_generate(p, 30, w, cfg)
        else:
            # bfloat16 may turn a near tie: every token and its logit against the plain windowed model on the same past
            check_greedy_tokens(p, got, o.inference_outputs[0].logprobs, w, cfg, TOL_BF16)
    # all keys again without the option: the plain model without a window, and other tokens and logits than with it
    # (the window does change what is computed, in either dtype)
    full = LlmEngine(d, dtype, cache=CacheConfig(block_size=16, num_gpu_blocks_override=40),
                     scheduler=SchedulerConfig(max_num_batched_tokens=32, max_num_sequences=2, max_model_len=400))
    outs_full = full.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=30, ignore_eos_token=True))
    for p, o, ow in zip(prompts, outs_full, outs):
        check_greedy_tokens(p, o.inference_outputs[0].token_ids, o.inference_outputs[0].logprobs, w, plain_config(d),
                            TOL_F32 * 10 if dtype == "float32" else TOL_BF16)
        first_full, first_win = o.inference_outputs[0].logprobs[0], ow.inference_outputs[0].logprobs[0]
        assert o.inference_outputs[0].token_ids != ow.inference_outputs[0].token_ids or \
            abs(first_full - first_win) > 1e-3 * abs(first_full), "the window changed nothing"
    if dtype == "float32":
        assert [o.inference_outputs[0].token_ids for o in outs_full] == \
            [plain_llama.greedy_generate(p, 30, w, plain_config(d)) for p in prompts]


def test_tiny_b_workload_portions_beside_decodes_with_temperature(model_dirs):
    """The tiny workload B: prompts of 37, 1 and 20 ids in 16-token portions alongside decodes, temperature
    0.7 with a fixed seed.  The sampled tokens must be what the plain model and plain sampler give for the same
    uniform numbers, and must not depend on how requests were batched."""
    from atoma_infer_amd.sampling import GenerateParameters, uniform
    d = model_dirs["B"]
    w, cfg = plain_weights(d), plain_config(d)
    prompts = [random_tokens(37, 1000, 3), random_tokens(1, 1000, 4), random_tokens(20, 1000, 5)]
    params = GenerateParameters(temperature=0.7, random_seed=99, max_new_tokens=6, ignore_eos_token=True)
    eng = engine(d, "float32", 16, 12, max_num_batched_tokens=16, max_prefill_chunk=16)
    outs = eng.generate(prompts, params)
    got = [o.inference_outputs[0].token_ids for o in outs]
    for p, toks in zip(prompts, got):
        seq = list(p)
        for step, tok in enumerate(toks):
            logits = plain_llama.forward(seq, w, cfg)[-1]
            dist = plain_llama.sampling_distribution(logits, 0.7)
            u = uniform(99, step)
            want = plain_llama.draw(dist, u)
            if tok != want:
                # allowed only when u lands on the boundary between the two tokens within float32 rounding
                c = torch.cumsum(dist.double(), 0) / dist.double().sum()
                lo, hi = sorted((tok, want))
                assert abs(float(c[lo:hi].max()) - u) < 1e-5 or abs(float(c[lo]) - u) < 1e-5, (step, tok, want)
            seq.append(tok)
    # alone, each request samples the same tokens
    for p, toks in zip(prompts, got):
        eng1 = engine(d, "float32", 16, 12)
        alone = eng1.generate([p], params)[0].inference_outputs[0].token_ids
        assert alone == toks
    assert eng.stats["steps"] > 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_preemption_under_page_pressure_keeps_results(model_dirs, dtype):
    """So few pages that running requests are preempted and recomputed: the tokens stay what they are alone."""
    from atoma_infer_amd.sampling import GenerateParameters
    d = model_dirs["C"]
    prompts = [random_tokens(n, 331, 40 + i) for i, n in enumerate([30, 45, 20, 33, 12])]
    params = GenerateParameters(do_sample=False, max_new_tokens=40, ignore_eos_token=True)
    roomy = engine(d, dtype, 16, 64, max_model_len=256)
    want = [o.inference_outputs[0].token_ids for o in roomy.generate(prompts, params)]
    tight = engine(d, dtype, 16, 12, max_model_len=256)
    outs = tight.generate(prompts, params)
    got = [o.inference_outputs[0].token_ids for o in outs]
    assert tight.stats["preemptions"] > 0
    assert tight.runner.manager.num_free_pages() == 12
    if dtype == "float32":
        assert got == want
    else:
        # bfloat16 logits may differ in the last bits between batch shapes, and a flipped argmax changes what
        # follows: every token is checked, with its logit, against the plain model run on what was generated
        w, cfg = plain_weights(d), plain_config(d)
        for p, o in zip(prompts, outs):
            check_greedy_tokens(p, o.inference_outputs[0].token_ids, o.inference_outputs[0].logprobs, w, cfg, TOL_BF16)


def test_eos_stops_and_too_long_is_ignored(model_dirs):
    from atoma_infer_amd.sampling import GenerateParameters
    d = model_dirs["A"]
    w, cfg = plain_weights(d), plain_config(d)
    prompt = random_tokens(6, 512, 9)
    free_run = plain_llama.greedy_generate(prompt, 10, w, cfg)
    eng = engine(d, "float32", 4, 32, max_model_len=64)
    eng.eos_ids = {free_run[3]}
    out = eng.generate([prompt], GenerateParameters(do_sample=False, max_new_tokens=10))[0].inference_outputs[0]
    stop_at = free_run.index(free_run[3])
    assert out.token_ids == free_run[:stop_at + 1] and out.finish_reason == "stopped" and out.stop_reason == free_run[3]
    outs = eng.generate([random_tokens(70, 512, 1)], GenerateParameters(do_sample=False, max_new_tokens=2))
    assert outs[0].inference_outputs[0].finish_reason == "ignored" and outs[0].inference_outputs[0].token_ids == []
    from atoma_infer_amd.sampling import ValidationError
    with pytest.raises(ValidationError):
        eng.add_request([1, 2, 9999])
    with pytest.raises(ValidationError):
        eng.add_request("text without a tokenizer")


# ----------------------------------------------------------------------------------------------------------
# the sampling kernel against the plain sampling functions


SPLIT = [False, True]       # a block a row in one launch, or every row shared by several blocks over six launches


@pytest.mark.parametrize("split", SPLIT)
@pytest.mark.parametrize("vocab", [331, 1000, 5000, 50001, 128256])
def test_sample_kernel(vocab, split):
    """Rows of a batch against the plain distribution and draw; 50001 leaves all rows but the first unaligned, 128256
    is a real vocabulary (every wave of the kernel has several slices of several pieces)."""
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(vocab)
    rows = [(0.0, 0, 1.0), (0.7, 0, 1.0), (1.3, 5, 1.0), (0.7, 0, 0.6), (0.9, 20, 0.8), (0.5, 1, 1.0), (2.0, 0, 0.999)]
    logits = torch.randn(len(rows), vocab, generator=g) * 2.0
    logits[2, 10] = logits[2, 20] = logits[2].max() + 1.0        # ties at the top
    dists = [None if t == 0.0 else plain_llama.sampling_distribution(logits[i], t, k, p)
             for i, (t, k, p) in enumerate(rows)]
    cdfs = [None if d is None else torch.cumsum(d.double(), 0) / d.double().sum() for d in dists]
    dev = lambda x, dt: torch.tensor(x, dtype=dt, device="cuda:0")
    for u in (0.0, 0.013, 0.25, 0.5, 0.77, 0.999):
        tok, lg = ops.sample(logits.cuda(), dev([r[0] for r in rows], torch.float32),
                             dev([r[1] for r in rows], torch.int32), dev([r[2] for r in rows], torch.float32),
                             dev([u] * len(rows), torch.float32), split=split)
        tok, lg = tok.cpu().tolist(), lg.cpu()
        for i, (t, k, p) in enumerate(rows):
            if t == 0.0:
                assert tok[i] == int(torch.argmax(logits[i]))
                continue
            want = plain_llama.draw(dists[i], u)
            assert dists[i][tok[i]] > 0, f"row {i}: token {tok[i]} is outside the kept set"
            if tok[i] != want:
                lo, hi = sorted((tok[i], want))
                assert abs(float(cdfs[i][lo]) - u) < 1e-5 or abs(float(cdfs[i][hi - 1]) - u) < 1e-5, (i, u, tok[i], want)
            assert float(lg[i]) == float(logits[i, tok[i]])


@pytest.mark.parametrize("split", SPLIT)
def test_sample_kernel_many_ties_in_a_large_vocabulary(split):
    """Ties at the threshold that are only partly kept, spread over the stretches of several waves (and over the
    parts of a row that several blocks share): the kept ones are those of lowest index, and every kept token can be
    drawn."""
    from atoma_infer_amd.kernels import ops
    vocab = 40000
    logits = torch.full((2, vocab), -3.0)
    tied = list(range(5, vocab, 997))                   # 41 tied tokens across the vocabulary
    logits[0, tied] = 2.0
    logits[1, tied] = 2.0
    logits[1, 123] = 4.0                                # one token above the ties
    dev = lambda x, dt: torch.tensor(x, dtype=dt, device="cuda:0")
    seen = [set(), set()]
    n = 400
    for i in range(n):
        u = (i + 0.5) / n
        tok, _ = ops.sample(logits.cuda(), dev([1.0, 1.0], torch.float32), dev([7, 12], torch.int32),
                            dev([1.0, 1.0], torch.float32), dev([u, u], torch.float32), split=split)
        for r, t in enumerate(tok.cpu().tolist()):
            seen[r].add(t)
    assert seen[0] == set(tied[:7])
    assert seen[1] == {123} | set(tied[:11])


@pytest.mark.parametrize("split", SPLIT)
def test_sample_kernel_kept_sets_and_ties(split):
    from atoma_infer_amd.kernels import ops
    vocab = 700
    logits = torch.zeros(3, vocab)
    logits[0, [5, 100, 300, 650]] = 3.0                # four tied tokens, top_k = 2 keeps ids 5 and 100
    logits[1, 7] = 20.0                                # nearly all mass on one token, top_p = 0.5 keeps only it
    logits[2] = torch.linspace(0, 5, vocab)
    seen = [set(), set(), set()]
    for i in range(64):
        u = (i + 0.5) / 64
        dev = lambda x, dt: torch.tensor(x, dtype=dt, device="cuda:0")
        tok, _ = ops.sample(logits.cuda(), dev([1.0, 1.0, 1.0], torch.float32), dev([2, 0, 3], torch.int32),
                            dev([1.0, 0.5, 1.0], torch.float32), dev([u] * 3, torch.float32), split=split)
        for r, t in enumerate(tok.cpu().tolist()):
            seen[r].add(t)
    assert seen[0] == {5, 100} and seen[1] == {7} and seen[2] == {vocab - 3, vocab - 2, vocab - 1}


@pytest.mark.parametrize("rows,vocab", [(1, 128256), (8, 128256), (3, 200003), (70, 50001), (300, 40000), (2, 262144)])
def test_rows_shared_by_several_blocks_draw_the_same_tokens(rows, vocab):
    """The six launches that share every row among several blocks against the one launch of a block a row: the same
    tokens and logits bit for bit, for rows of every mode (greedy ones among them), flat and peaked logits, NaN rows,
    vocabularies that leave rows unaligned and parts of unequal length."""
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(rows * 7 + vocab)
    logits = torch.randn(rows, vocab, generator=g) * torch.where(torch.arange(rows) % 2 == 0, 0.3, 3.0)[:, None]
    modes = [(0.0, 0, 1.0), (0.8, 0, 1.0), (0.8, 50, 1.0), (0.8, 0, 0.9), (0.8, 50, 0.9), (1.5, 3, 0.5), (0.3, 1000, 0.99)]
    pick = [modes[i % len(modes)] for i in range(rows)]
    if rows >= 8:
        logits[5] = float("nan")
        logits[6, 100:5000] = 1.25                       # thousands of ties, partly kept
        pick[6] = (1.0, 700, 0.9)
    dev = lambda x, dt: torch.tensor(x, dtype=dt, device="cuda:0")
    lg = logits.cuda()
    t, k, p = (dev([m[i] for m in pick], dt) for i, dt in ((0, torch.float32), (1, torch.int32), (2, torch.float32)))
    for u in (0.0, 0.31, 0.5, 0.93, 0.999999):
        uu = dev([(u + 0.37 * i) % 1.0 for i in range(rows)], torch.float32)
        one = ops.sample_packed(lg, t, k, p, uu)
        six = ops.sample_packed(lg, t, k, p, uu, split=True)
        assert torch.equal(one[0].view(torch.int32), six[0].view(torch.int32)), (u, one[0].view(torch.int32), six[0].view(torch.int32))
        assert torch.equal(one[1].isnan(), six[1].isnan()) and torch.equal(one[1].nan_to_num(), six[1].nan_to_num())
    # a caller that knows of no cut leaves the search out: the rows are then drawn from all of their weights
    no_k, no_p = torch.zeros_like(k), torch.ones_like(p)
    uu = dev([(0.77 + 0.37 * i) % 1.0 for i in range(rows)], torch.float32)
    one = ops.sample_packed(lg, t, no_k, no_p, uu)
    four = ops.sample_packed(lg, t, k, p, uu, split=True, cuts=False)
    assert torch.equal(one[0].view(torch.int32), four[0].view(torch.int32))


def test_the_sampler_shares_the_rows_of_a_large_vocabulary():
    """Through the engine's sampler: a step whose rows draw from 128k logits goes to the launches that share every
    row among several blocks, with the search left out when no row has a cut; the tokens are those of a block a row
    with the same uniform numbers, and those of the plain distribution."""
    from atoma_infer_amd.kernels import ops
    from atoma_infer_amd.sampling import Sampler, validate, GenerateParameters
    from atoma_infer_amd.sampling.sampler import uniform
    vocab = 128256
    logits = (torch.randn(5, vocab, generator=torch.Generator().manual_seed(3)) * 2.5).cuda()
    make = lambda **kw: validate(GenerateParameters(ignore_eos_token=True, **kw), 3, 100, 200)
    with_cuts = [make(temperature=0.8, top_k=50, top_p=0.9, random_seed=5), make(do_sample=False),
                 make(temperature=1.3, random_seed=6), make(temperature=0.6, top_p=0.5, random_seed=7),
                 make(temperature=0.9, top_k=3, random_seed=8)]
    without = [make(temperature=0.8, random_seed=5), make(do_sample=False), make(temperature=1.3, random_seed=6),
               make(temperature=0.6, random_seed=7), make(temperature=2.0, random_seed=8)]
    sampler = Sampler(torch.device("cuda:0"))
    dev = lambda x, dt: torch.tensor(x, dtype=dt, device="cuda:0")
    calls = []
    real = ops.sample_packed
    try:
        # (the sampler names its options; the comparison below goes through ops.sample, which does not)
        ops.sample_packed = lambda *a, **kw: (calls.append(kw) if kw else None, real(*a, **kw))[1]
        for plans in (with_cuts, without):
            for step in (0, 1, 17):
                got, got_lg = sampler.sample(logits.clone(), plans, [step] * 5, [()] * 5)
                uu = [0.0 if pl.greedy else uniform(pl.random_seed, step) for pl in plans]
                t = [0.0 if pl.greedy else pl.temperature for pl in plans]
                want, want_lg = ops.sample(logits, dev(t, torch.float32), dev([pl.top_k for pl in plans], torch.int32),
                                           dev([pl.top_p for pl in plans], torch.float32), dev(uu, torch.float32))
                assert got == want.cpu().tolist() and got_lg == want_lg.cpu().tolist()
                for i, pl in enumerate(plans):
                    if pl.greedy:
                        assert got[i] == int(logits[i].argmax())
                    else:
                        d = plain_llama.sampling_distribution(logits[i].cpu(), pl.temperature, pl.top_k, pl.top_p)
                        assert d[got[i]] > 0
    finally:
        ops.sample_packed = real
    assert all(kw.get("split") for kw in calls)
    assert [kw.get("cuts") for kw in calls] == [True] * 3 + [False] * 3


def test_repeat_penalty_kernel_and_temperature_limit():
    from atoma_infer_amd.kernels import ops
    from atoma_infer_amd.sampling import Sampler, validate, GenerateParameters
    logits = torch.tensor([[1.0, -1.0, 2.0, 0.5], [3.0, 1.0, -2.0, 0.0]], device="cuda:0")
    want0 = plain_llama.repeat_penalty(logits[0].cpu(), 2.0, [0, 1, 1])
    ops.repeat_penalty(logits, torch.tensor([0, 0], dtype=torch.int32, device="cuda:0"),
                       torch.tensor([0, 1], dtype=torch.int32, device="cuda:0"),
                       torch.tensor([2.0, 1.0], device="cuda:0"))
    assert torch.equal(logits[0].cpu(), want0) and logits[1].cpu().tolist() == [3.0, 1.0, -2.0, 0.0]
    # through the sampler: the penalty turns the argmax away from a repeated token
    s = Sampler(torch.device("cuda:0"))
    lg = torch.tensor([[2.0, 1.9, 0.0]], device="cuda:0")
    p1 = validate(GenerateParameters(do_sample=False), 3, 100, 200)
    p2 = validate(GenerateParameters(do_sample=False, repetition_penalty=1.5, repeat_last_n=4), 3, 100, 200)
    assert s.sample(lg.clone(), [p1], [0], [[0, 0, 0]])[0] == [0]
    assert s.sample(lg.clone(), [p2], [0], [[0, 0, 0]])[0] == [1]
    # a very low temperature is greedy in effect
    p3 = validate(GenerateParameters(temperature=1e-3, random_seed=5), 3, 100, 200)
    big = torch.randn(1, 2000, generator=torch.Generator().manual_seed(0)).cuda()
    assert s.sample(big.clone(), [p3], [0], [()])[0] == [int(big.argmax())]


# ----------------------------------------------------------------------------------------------------------
# bin/trace_run as a program


def run_trace(model_dir, dtype, steps, out_dir, max_tokens, extra=(), ok=True, program="bin/trace_run"):
    """``program``: bin/trace_run, or the package's own ``replay`` command (the two are one function)."""
    env = dict(os.environ)
    if program == "bin/trace_run":
        head = [sys.executable, os.path.join(ROOT, "bin", "trace_run")]
    else:
        head = [sys.executable, "-m", "atoma_infer_amd", "replay"]
        env["PYTHONPATH"] = ROOT + os.pathsep + env.get("PYTHONPATH", "")
    proc = subprocess.run([*head, "--model", model_dir, "--dtype", dtype, "--out", out_dir, "--max-tokens",
                           str(max_tokens), *extra],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
                          env=env, timeout=300)
    if not ok:
        return proc
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    return proc


@pytest.mark.parametrize("dtype,program", [("float32", "bin/trace_run"), ("bfloat16", "python -m atoma_infer_amd replay")])
def test_trace_run_with_pages_of_four_tokens(model_dirs, tmp_path, dtype, program):
    """Tiny A with its own block size of 4 through the program's --page-size, three requests with two live at a time
    in a pool of 128 tokens; then a third live request beyond --max-live ends the program with a clear message.
    Once through bin/trace_run and once through the package's ``replay`` command, which takes the same options."""
    d = model_dirs["A"]
    vocab = TINY["A"]["vocab_size"]
    a, b, c = random_tokens(50, vocab, 1), random_tokens(9, vocab, 2), random_tokens(30, vocab, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:21], "want": [20]}, {"id": "b", "tokens": b[:5], "want": [4]}],
         "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[5:], "want": [3]}, {"id": "a", "tokens": a[21:], "want": [0, 28]}],
         "end": ["b"]},
        {"step": 2, "entries": [{"id": "c", "tokens": c[:2], "want": [1]}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "c", "tokens": c[2:], "want": [27]}], "end": ["c"]},
    ]
    out = str(tmp_path / "out")
    run_trace(d, dtype, steps, out, 128, extra=("--page-size", "4", "--max-live", "2"), program=program)
    w, cfg = plain_weights(d), plain_config(d)
    pa, pb, pc = (plain_llama.forward(t, w, cfg) for t in (a, b, c))
    want = {0: torch.stack([pa[20], pb[4]]), 1: torch.stack([pb[8], pa[21], pa[49]]), 2: pc[1][None], 3: pc[29][None]}
    for step, ref in want.items():
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, vocab))
        assert got.shape == ref.shape
        assert (rel_err(got, ref) < TOL_F32) if dtype == "float32" else (frob_err(got, ref) < TOL_BF16)
    if dtype == "float32":
        crowd = [{"step": 0, "entries": [{"id": n, "tokens": a[:3], "want": []} for n in ("x", "y", "z")], "end": []}]
        proc = run_trace(d, dtype, crowd, str(tmp_path / "out2"), 128, extra=("--page-size", "4", "--max-live", "2"),
                         ok=False)
        assert proc.returncode != 0 and "--max-live" in proc.stderr and "Traceback" not in proc.stderr


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, tmp_path, dtype):
    d = model_dirs["B"]
    vocab = TINY["B"]["vocab_size"]
    a, b, c = random_tokens(70, vocab, 1), random_tokens(40, vocab, 2), random_tokens(64, vocab, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}, {"id": "a", "tokens": a[33:35], "want": [1]}],
         "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[35:], "want": [34]}, {"id": "b", "tokens": b[2:], "want": [0, 37]}],
         "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "c", "tokens": c[:63], "want": []}], "end": []},
        {"step": 4, "entries": [{"id": "c", "tokens": c[63:], "want": [0]}], "end": ["c"]},
    ]
    out = str(tmp_path / "out")
    # a and b round up to 128 + 64 tokens; c reuses their pages
    run_trace(d, dtype, steps, out, 192)
    assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "2.f32", "4.f32"]
    w, cfg = plain_weights(d), plain_config(d)
    pa, pb, pc = (plain_llama.forward(t, w, cfg) for t in (a, b, c))
    want = {0: torch.stack([pa[0], pa[32]]), 1: pa[34][None], 2: torch.stack([pa[69], pb[2], pb[39]]), 4: pc[63][None]}
    for step, ref in want.items():
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, vocab))
        assert got.shape == ref.shape
        if dtype == "float32":
            assert rel_err(got, ref) < TOL_F32
        else:
            assert frob_err(got, ref) < TOL_BF16


# ----------------------------------------------------------------------------------------------------------
# the engine runs one step ahead of the sampled tokens


def test_running_ahead_changes_no_token(model_dirs):
    """EOS is seen one step late and the token sampled meanwhile is dropped; a repeat penalty makes the engine
    read tokens at once.  Either way the tokens are those of the plain model."""
    from atoma_infer_amd.sampling import GenerateParameters
    d = model_dirs["B"]
    w, cfg = plain_weights(d), plain_config(d)
    prompts = [random_tokens(9, 1000, 11), random_tokens(4, 1000, 12), random_tokens(15, 1000, 13)]
    free = [plain_llama.greedy_generate(p, 12, w, cfg) for p in prompts]
    eng = engine(d, "float32", 16, 16)
    eng.eos_ids = {free[0][5], free[2][2]}
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=12))
    for o, f in zip(outs, free):
        cut = next((i for i, t in enumerate(f) if t in eng.eos_ids), None)
        want = f if cut is None else f[:cut + 1]
        assert o.inference_outputs[0].token_ids == want
        assert o.inference_outputs[0].finish_reason == ("length_capped" if cut is None else "stopped")
    assert eng.runner.manager.num_requests() == 0 and eng.runner.manager.num_free_pages() == 16
    assert not eng.has_unfinished()
    # with a repeat penalty: greedy over penalised logits, token by token, as the plain functions give it
    eng2 = engine(d, "float32", 16, 16)
    params = GenerateParameters(do_sample=False, max_new_tokens=8, repetition_penalty=1.3, repeat_last_n=6,
                                ignore_eos_token=True)
    got = eng2.generate(prompts[:2], params)
    for p, o in zip(prompts, got):
        seq = list(p)
        for tok in o.inference_outputs[0].token_ids:
            logits = plain_llama.repeat_penalty(plain_llama.forward(seq, w, cfg)[-1], 1.3, seq[-6:])
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) > 1e-4:       # a near tie may fall either way in float32
                assert tok == int(torch.argmax(logits))
            seq.append(tok)
    # step by step from outside: outputs arrive when requests finish, and drain() leaves nothing in flight
    eng3 = engine(d, "float32", 16, 16)
    rid = eng3.add_request(prompts[1], GenerateParameters(do_sample=False, max_new_tokens=3, ignore_eos_token=True))
    seen = []
    for _ in range(10):
        seen += eng3.step()
        if not eng3.has_unfinished():
            break
    assert [o.request_id for o in seen] == [rid] and seen[0].inference_outputs[0].token_ids == free[1][:3]
    assert eng3.drain() == []


def test_command_line_generates(model_dirs, tmp_path):
    d = model_dirs["A"]
    w, cfg = plain_weights(d), plain_config(d)
    prompt = random_tokens(7, 512, 5)
    want = plain_llama.greedy_generate(prompt, 5, w, cfg)
    toml = tmp_path / "engine.toml"
    toml.write_text(f'''
[inference]
model_name = "{d}"
dtype = "f32"
device_ids = [0]
[cache]
block_size = 4
num_gpu_blocks_override = 16
[scheduler]
max_num_batched_tokens = 32
max_num_sequences = 4
max_model_len = 64
enable_chunked_prefill = true
[validation]
max_input_length = 32
max_total_tokens = 64
''')
    reqs = tmp_path / "requests.jsonl"
    reqs.write_text(json.dumps({"request_id": "one", "inputs": prompt,
                                "parameters": {"do_sample": False, "max_new_tokens": 5, "ignore_eos_token": True}}) + "\n")
    env = dict(os.environ, PYTHONPATH=ROOT)
    proc = subprocess.run([sys.executable, "-m", "atoma_infer_amd", "generate", "--config-path", str(toml),
                           "--requests", str(reqs)], capture_output=True, text=True, env=env, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads(proc.stdout.strip().splitlines()[-1])
    assert out["request_id"] == "one" and out["is_finished"]
    assert out["inference_outputs"][0]["token_ids"] == want
    assert out["inference_outputs"][0]["finish_reason"] == "length_capped"
    # the same through flags instead of files
    proc = subprocess.run([sys.executable, "-m", "atoma_infer_amd", "generate", "--model", d, "--dtype", "f32",
                           "--block-size", "4", "--num-gpu-blocks-override", "16", "--max-model-len", "64",
                           "--max-num-batched-tokens", "64", "--max-num-sequences", "4", "--greedy",
                           "--max-new-tokens", "5", "--ignore-eos-token", "--prompt-ids",
                           ",".join(str(t) for t in prompt)], capture_output=True, text=True, env=env, timeout=300,
                          cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert json.loads(proc.stdout.strip().splitlines()[-1])["inference_outputs"][0]["token_ids"] == want


def test_abort_loses_no_other_request(model_dirs):
    """Aborting reads the step in flight; what that step finished must still be handed out."""
    from atoma_infer_amd.sampling import GenerateParameters
    d = model_dirs["A"]
    w, cfg = plain_weights(d), plain_config(d)
    prompts = [random_tokens(5, 512, 21), random_tokens(7, 512, 22), random_tokens(6, 512, 23)]
    for steps_before in (1, 2, 3, 4):
        eng = engine(d, "float32", 4, 32)
        short = GenerateParameters(do_sample=False, max_new_tokens=3, ignore_eos_token=True)
        ids = [eng.add_request(prompts[0], short), eng.add_request(prompts[1], short),
               eng.add_request(prompts[2], GenerateParameters(do_sample=False, max_new_tokens=30, ignore_eos_token=True))]
        seen = []
        for _ in range(steps_before):
            seen += eng.step()
        gone = eng.abort(ids[2])
        assert gone is not None and gone.request_id == ids[2]
        assert gone.inference_outputs[0].token_ids == plain_llama.greedy_generate(
            prompts[2], 30, w, cfg)[:len(gone.inference_outputs[0].token_ids)]
        while eng.has_unfinished():
            seen += eng.step()
        assert sorted(o.request_id for o in seen) == sorted(ids[:2])
        for o in seen:
            want = plain_llama.greedy_generate(prompts[ids.index(o.request_id)], 3, w, cfg)
            assert o.inference_outputs[0].token_ids == want
        assert eng.runner.manager.num_requests() == 0 and eng.runner.manager.num_free_pages() == 32


def test_text_in_and_out_with_a_tokenizer(model_dirs, tmp_path):
    """With tokenizer.json in the model folder prompts may be text, outputs carry text, ``stop`` strings end a
    request at the piece that equals one of them, ``truncate`` keeps the end of the prompt's text and
    ``return_full_text`` puts the prompt before the output."""
    import shutil
    from tokenizers import Tokenizer, models, pre_tokenizers
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling import GenerateParameters
    d = str(tmp_path / "model")
    shutil.copytree(model_dirs["A"], d)
    vocab = {f"w{i}": i for i in range(512)}
    tok = Tokenizer(models.WordLevel(vocab, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.save(os.path.join(d, "tokenizer.json"))
    w, cfg = plain_weights(d), plain_config(d)
    eng = LlmEngine(d, "float32", cache=CacheConfig(block_size=4, num_gpu_blocks_override=32),
                    scheduler=SchedulerConfig(max_num_batched_tokens=64, max_num_sequences=4, max_model_len=128))
    assert eng.load_tokenizer(d)
    eng.eos_ids = set()
    ids = [5, 17, 3, 250]
    text = " ".join(f"w{i}" for i in ids)
    free = plain_llama.greedy_generate(ids, 8, w, cfg)
    out = eng.generate([text], GenerateParameters(do_sample=False, max_new_tokens=8, ignore_eos_token=True))[0]
    assert out.prompt == text and out.prompt_token_ids == ids
    assert out.inference_outputs[0].token_ids == free
    assert out.inference_outputs[0].output_text == tok.decode(free)
    # a stop string: the piece of the third new token (if it did not occur before)
    piece = tok.decode([free[2]])
    cut = next(i for i, t in enumerate(free) if tok.decode([t]) == piece)
    out = eng.generate([text], GenerateParameters(do_sample=False, max_new_tokens=8, stop=[piece]))[0].inference_outputs[0]
    assert out.token_ids == free[:cut + 1] and out.finish_reason == "stopped" and out.stop_reason == piece
    # the prompt before the output
    out = eng.generate([text], GenerateParameters(do_sample=False, max_new_tokens=3, return_full_text=True,
                                                  ignore_eos_token=True))[0].inference_outputs[0]
    assert out.output_text == text + tok.decode(free[:3])
    # truncate keeps the last characters of the text (the reference cuts text, not tokens: tokenizer.rs:185-206)
    keep = len("w3 w250")
    out = eng.generate([text], GenerateParameters(do_sample=False, max_new_tokens=2, truncate=keep, ignore_eos_token=True))[0]
    assert out.prompt_token_ids == [3, 250]
    assert out.inference_outputs[0].token_ids == plain_llama.greedy_generate([3, 250], 2, w, cfg)


def random_trace(rng, requests, max_live=4):
    """Steps in the replay program's format for the given requests: up to four live, portions of random sizes down
    to two tokens beside single tokens, requests that sit out steps, random wanted places (also none).  Returns
    (steps, the most tokens live at a time with every request rounded up to 64)."""
    waiting, live, done, steps, peak = list(requests), [], {k: 0 for k in requests}, [], 0
    while waiting or live:
        while waiting and len(live) < max_live and (rng.random() < 0.6 or not live):
            live.append(waiting.pop(0))
        entries, end = [], []
        for k in live:
            left = len(requests[k]) - done[k]
            if rng.random() < 0.2 and len(live) > 1:
                continue
            mode = rng.random()
            if left <= rng.randint(1, 10) or mode < 0.3:
                n = 1
            elif mode < 0.5:
                n = min(2, left)
            else:
                n = min(rng.choice([2, 3, 7, 16, 17, 31, 64, 100]), left)
            want = sorted(rng.sample(range(n), rng.randint(0, min(n, 3))))
            entries.append({"id": k, "tokens": requests[k][done[k]:done[k] + n], "want": want})
            done[k] += n
            if done[k] == len(requests[k]):
                end.append(k)
        if not entries:
            continue
        rng.shuffle(entries)
        peak = max(peak, sum(-(-done[k] // 64) * 64 for k in live))
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [k for k in live if k not in end]
    return steps, peak


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,seed", [("A", 0), ("B", 1), ("C", 2), ("D", 3), ("D", 4), ("E", 5)])
def test_random_traces_replay_like_the_plain_model(model_dirs, tmp_path, name, seed, dtype):
    import io
    import random
    from atoma_infer_amd.engine.replay import make_runner, replay
    rng = random.Random(seed)
    cfg = TINY[name]
    vocab = cfg["vocab_size"]
    longest = 400 if name in ("D", "E") else min(cfg["max_position_embeddings"], 120)
    requests = {f"q{i}": random_tokens(rng.randint(1, longest), vocab, 900 * seed + i) for i in range(rng.randint(3, 7))}
    steps, peak = random_trace(rng, requests)
    runner = make_runner(model_dirs[name], dtype, peak)
    report = io.StringIO()
    assert replay(runner, io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n"), str(tmp_path), report) == 0
    assert report.getvalue().split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    w, c = plain_weights(model_dirs[name]), plain_config(model_dirs[name])
    want = {k: plain_llama.forward(v, w, c) for k, v in requests.items()}
    pos = {k: 0 for k in requests}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        path = tmp_path / f"{s['step']}.f32"
        assert path.exists() == (n_want > 0)
        if n_want:
            got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n_want, vocab))
            row = 0
            for e in s["entries"]:
                for i in e["want"]:
                    ref = want[e["id"]][pos[e["id"]] + i]
                    if dtype == "float32":
                        assert rel_err(got[row], ref) < TOL_F32, (s["step"], e["id"], i)
                    else:
                        assert frob_err(got[row], ref) < 2.5 * TOL_BF16, (s["step"], e["id"], i)
                    row += 1
        for e in s["entries"]:
            pos[e["id"]] += len(e["tokens"])
    assert runner.manager.num_requests() == 0
