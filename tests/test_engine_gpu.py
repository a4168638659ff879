"""The engine against the plain implementation: whole prompts, decoding, portions, mixed batches with few pages.

Every schedule must give, for every (request, position), the logits of the plain float32 model run on the whole
sequence: float32 within accumulation-order noise, bfloat16 within its rounding.
"""
import random

import pytest
import torch

import plain_llama
from util import (NORM_JITTER, TINY, TOL_BF16, TOL_F32, force_chunked_decode, frob_err, make_model_dir, plain_config,
                  plain_weights, random_tokens, rel_err)

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
# how the bfloat16 attention plans decoded tokens: as its planner decides (at the contexts of these tests: whole key
# ranges walked by eight waves, where the head size allows them), or in chunks merged by a second kernel, as it does
# at long contexts with few requests (merged by the attention kernel itself, or by a second kernel); the float32
# attention has one way only
DTYPE_TASKS = [(d, "planned") for d in DTYPES] + [("bfloat16", "chunks"), ("bfloat16", "chunks, second kernel")]
PAGE = {"A": 4, "B": 16, "C": 16, "D": 16, "E": 16, "F": 16}


@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    out = {}
    for name, cfg in TINY.items():
        # bfloat16 storage: both dtypes then compute from exactly the same numbers
        out[name] = make_model_dir(str(tmp_path_factory.mktemp(f"tiny_{name}")), cfg, seed=11 + len(name),
                                   dtype="bfloat16", norm_jitter=NORM_JITTER[name])
    return out


_plain_cache = {}


def plain_logits(model_dir, tokens):
    key = (model_dir, tuple(tokens))
    if key not in _plain_cache:
        _plain_cache[key] = plain_llama.forward(list(tokens), plain_weights(model_dir), plain_config(model_dir))
    return _plain_cache[key]


def make_runner(model_dir, dtype, page_size, num_pages, slots=8):
    from atoma_infer_amd.cache import CachePool, plan_cache
    from atoma_infer_amd.engine import ModelRunner
    from atoma_infer_amd.models import load_model
    model = load_model(model_dir, dtype)
    plan = plan_cache(model.spec)
    pool = CachePool(plan, page_size, [num_pages] * len(plan.groups), slots, model.act_dtype, model.device)
    return ModelRunner(model, pool)


def run_schedule(runner, requests, steps):
    """``steps``: list of (entries, end); entries are (name, n_tokens).  Returns {(name, position): logits row}."""
    from atoma_infer_amd.engine import StepEntry
    ids, out = {}, {}
    for entries, end in steps:
        batch, places = [], []
        for name, n in entries:
            if name not in ids:
                ids[name] = len(ids)
                runner.add_request(ids[name])
            start = runner.computed_len(ids[name])
            toks = requests[name][start:start + n]
            assert len(toks) == n, (name, start, n)
            batch.append(StepEntry(ids[name], toks, start, list(range(n))))
            places += [(name, start + i) for i in range(n)]
        logits = runner.step(batch).cpu()
        assert logits.shape[0] == len(places)
        for row, key in enumerate(places):
            out[key] = logits[row]
        for name in end:
            runner.free_request(ids[name])
        runner.manager.check()
    return out


def check_against_plain(model_dir, requests, got, dtype):
    worst = 0.0
    for name, toks in requests.items():
        rows = [p for (n, p) in got if n == name]
        if not rows:
            continue
        want = plain_logits(model_dir, toks)
        mine = torch.stack([got[(name, p)] for p in sorted(rows)])
        ref = want[sorted(rows)]
        if dtype == "float32":
            err = rel_err(mine, ref)
            assert err < TOL_F32, f"request {name}: float32 logits differ by {err:.3e} of the largest"
        else:
            err = frob_err(mine, ref)
            assert err < TOL_BF16, f"request {name}: bfloat16 logits differ by {err:.3e} of the norm"
            # row by row too, so that one bad position cannot hide among many good ones
            for i, p in enumerate(sorted(rows)):
                e = frob_err(mine[i], ref[i])
                assert e < 2.5 * TOL_BF16, f"request {name} position {p}: {e:.3e}"
        worst = max(worst, err)
    return worst


def lengths(name):
    return {"A": [100, 37, 64, 5], "B": [200, 1, 77, 130], "C": [150, 48, 97, 16], "D": [900, 300, 150, 40],
            "E": [600, 290, 33, 129], "F": [180, 61, 16, 99]}[name]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TINY))
def test_whole_prompts(model_dirs, name, dtype):
    vocab = TINY[name]["vocab_size"]
    requests = {f"r{i}": random_tokens(n, vocab, 100 + i) for i, n in enumerate(lengths(name))}
    runner = make_runner(model_dirs[name], dtype, PAGE[name], 64)
    steps = [([(r, len(t))], [r]) for r, t in requests.items()]
    got = run_schedule(runner, requests, steps)
    check_against_plain(model_dirs[name], requests, got, dtype)
    assert runner.manager.num_free_pages(0) == 64


@pytest.mark.parametrize("dtype,tasks", DTYPE_TASKS)
@pytest.mark.parametrize("name", list(TINY))
def test_last_32_one_by_one(model_dirs, name, dtype, tasks, monkeypatch):
    if tasks.startswith("chunks"):
        force_chunked_decode(monkeypatch, second_kernel=tasks.endswith("second kernel"))
    vocab = TINY[name]["vocab_size"]
    n = lengths(name)[0]
    requests = {"r": random_tokens(n, vocab, 7)}
    runner = make_runner(model_dirs[name], dtype, PAGE[name], 64)
    steps = [([("r", n - 32)], [])] + [([("r", 1)], []) for _ in range(32)]
    got = run_schedule(runner, requests, steps)
    assert len(got) == n
    check_against_plain(model_dirs[name], requests, got, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TINY))
def test_portions_of_changing_size(model_dirs, name, dtype):
    vocab = TINY[name]["vocab_size"]
    n = lengths(name)[0]
    requests = {"r": random_tokens(n, vocab, 8)}
    runner = make_runner(model_dirs[name], dtype, PAGE[name], 64)
    sizes, left, cycle = [], n, [17, 2, 31, 3, 16, 2, 5, 33, 1, 4]
    i = 0
    while left:
        s = min(cycle[i % len(cycle)], left)
        sizes.append(s)
        left -= s
        i += 1
    got = run_schedule(runner, requests, [([("r", s)], []) for s in sizes])
    check_against_plain(model_dirs[name], requests, got, dtype)


@pytest.mark.parametrize("dtype,tasks", DTYPE_TASKS)
@pytest.mark.parametrize("name", list(TINY))
def test_mixed_batches_with_few_pages(model_dirs, name, dtype, tasks, monkeypatch):
    """Up to four live requests, portions of some beside decoded tokens of others; the pool is so small that
    pages freed by finished requests are used again at once."""
    if tasks.startswith("chunks"):
        force_chunked_decode(monkeypatch, second_kernel=tasks.endswith("second kernel"))
    vocab = TINY[name]["vocab_size"]
    lens = {"A": [60, 33, 47, 21, 58, 40, 9, 52], "B": [120, 1, 77, 90, 45, 130, 18, 66],
            "C": [90, 48, 97, 16, 70, 33, 80, 25], "D": [700, 48, 97, 530, 70, 33, 80, 25],
            "E": [300, 48, 97, 610, 70, 33, 80, 25], "F": [110, 48, 97, 16, 70, 33, 80, 25]}[name]
    requests = {f"r{i}": random_tokens(n, vocab, 300 + i) for i, n in enumerate(lens)}
    page = PAGE[name]
    rng = random.Random(5)
    # pool: what the four longest need at once, nothing more
    need = sum(sorted(-(-n // page) for n in lens)[-4:])
    runner = make_runner(model_dirs[name], dtype, page, need, slots=4)
    waiting = list(requests)
    live, done_tokens, steps = [], {r: 0 for r in requests}, []
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            left = len(requests[r]) - done_tokens[r]
            # the last 8 tokens of every request are "decoded" one at a time; before that portions of 2..24
            if left <= 8:
                n = 1
            else:
                n = min(rng.choice([2, 3, 5, 8, 13, 24]), left - 8)
            if rng.random() < 0.15 and len(live) > 1:
                continue  # a request may sit out a step
            entries.append((r, n))
            done_tokens[r] += n
            if done_tokens[r] == len(requests[r]):
                end.append(r)
        if not entries:
            continue
        rng.shuffle(entries)
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    got = run_schedule(runner, requests, steps)
    assert len(got) == sum(lens)
    check_against_plain(model_dirs[name], requests, got, dtype)
    assert runner.manager.num_free_pages(0) == need and runner.manager.num_requests() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_place_wanted_twice_beside_an_entry_that_wants_nothing(model_dirs, dtype):
    """Two decoded tokens, the first entry wanting its place twice, the second nothing: as many wanted rows as
    tokens, but not "every row once" (the bfloat16 path that lets the last product begin the final norm on all rows
    must not take it)."""
    from atoma_infer_amd.engine import StepEntry
    name = "D"
    vocab = TINY[name]["vocab_size"]
    a, b = random_tokens(40, vocab, 41), random_tokens(23, vocab, 42)
    runner = make_runner(model_dirs[name], dtype, PAGE[name], 16)
    runner.add_request(0)
    runner.add_request(1)
    assert runner.step([StepEntry(0, a[:39], 0, []), StepEntry(1, b[:22], 0, [])]) is None
    logits = runner.step([StepEntry(0, a[39:], 39, [0, 0]), StepEntry(1, b[22:], 22, [])]).cpu()
    assert logits.shape == (2, vocab)
    assert torch.equal(logits[0], logits[1])
    check_against_plain(model_dirs[name], {"a": a}, {("a", 39): logits[0]}, dtype)
    # ... and the other way round: the second entry's row, not the first's
    runner.free_request(0)
    runner.free_request(1)
    runner.add_request(0)
    runner.add_request(1)
    runner.step([StepEntry(0, a[:39], 0, []), StepEntry(1, b[:22], 0, [])])
    logits = runner.step([StepEntry(0, a[39:], 39, []), StepEntry(1, b[22:], 22, [0, 0])]).cpu()
    assert torch.equal(logits[0], logits[1])
    check_against_plain(model_dirs[name], {"b": b}, {("b", 22): logits[0]}, dtype)


@pytest.mark.parametrize("page", [32, 64])
@pytest.mark.parametrize("name", ["B", "D", "E"])
def test_larger_pages_run_on_the_matrix_cores(model_dirs, name, page, monkeypatch):
    """bfloat16 with pages of 32 and 64 tokens (the reference takes every multiple of 16: csrc/src/lib.rs:778-785):
    portions of changing size, the last tokens one by one, then requests mixed in a pool so small that pages are used
    again; the general attention kernel must not be called."""
    from atoma_infer_amd.kernels import ops

    def refuse(*a, **k):
        raise AssertionError("the general attention kernel ran")

    monkeypatch.setattr(ops, "paged_attention_generic", refuse)
    force_chunked_decode(monkeypatch)
    vocab = TINY[name]["vocab_size"]
    lens = {"B": [120, 1, 77, 90, 45, 130], "D": [700, 48, 97, 530, 70, 33], "E": [300, 48, 97, 610, 70, 33]}[name]
    requests = {f"r{i}": random_tokens(n, vocab, 500 + i) for i, n in enumerate(lens)}
    need = sum(sorted(-(-n // page) for n in lens)[-3:])
    runner = make_runner(model_dirs[name], "bfloat16", page, need, slots=3)
    rng = random.Random(page + len(name))
    waiting, live, done, steps = list(requests), [], {r: 0 for r in requests}, []
    while waiting or live:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            left = len(requests[r]) - done[r]
            n = 1 if left <= 12 else min(rng.choice([2, 5, 16, 31, 33, 70]), left - 12)
            entries.append((r, n))
            done[r] += n
            if done[r] == len(requests[r]):
                end.append(r)
        rng.shuffle(entries)
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    got = run_schedule(runner, requests, steps)
    assert len(got) == sum(lens)
    check_against_plain(model_dirs[name], requests, got, "bfloat16")
    assert runner.manager.num_free_pages(0) == need


def test_pages_the_matrix_core_attention_refuses_are_announced(model_dirs):
    """bfloat16 with pages of 4 tokens is right (the tests above run it) but takes the general attention kernel:
    building the runner says so once."""
    with pytest.warns(UserWarning, match="general kernel"):
        make_runner(model_dirs["A"], "bfloat16", 4, 8)


@pytest.mark.parametrize("dtype,tasks", DTYPE_TASKS)
def test_first_tokens_and_long_decoding(model_dirs, dtype, tasks, monkeypatch):
    """A one-token prompt, then everything decoded token by token up to the model's last position."""
    if tasks.startswith("chunks"):
        force_chunked_decode(monkeypatch, second_kernel=tasks.endswith("second kernel"))
    name = "A"
    vocab, n = TINY[name]["vocab_size"], TINY[name]["max_position_embeddings"]
    requests = {"r": random_tokens(n, vocab, 9)}
    runner = make_runner(model_dirs[name], dtype, PAGE[name], 40)
    got = run_schedule(runner, requests, [([("r", 1)], []) for _ in range(n)])
    check_against_plain(model_dirs[name], requests, got, dtype)
    from atoma_infer_amd.engine import StepEntry, StepError
    with pytest.raises(StepError):
        runner.step([StepEntry(0, [1], n, [0])])  # beyond max_position_embeddings


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_decode_graphs_replay_like_eager_steps(model_dirs, name, dtype):
    """Decode steps are captured into HIP graphs.  Every replay is compared with the same step run eagerly, with
    eager work (prompt portions of another request, frees, new requests) and synchronisations between replays."""
    from atoma_infer_amd.engine import StepEntry
    vocab = TINY[name]["vocab_size"]
    toks = {r: random_tokens(n, vocab, 70 + i) for i, (r, n) in enumerate([("a", 90), ("b", 60), ("c", 50)])}
    graphed = make_runner(model_dirs[name], dtype, PAGE[name], 32)
    eager = make_runner(model_dirs[name], dtype, PAGE[name], 32)
    eager.use_graphs = False
    for rn in (graphed, eager):
        for i in range(3):
            rn.add_request(i)
    ids = {"a": 0, "b": 1, "c": 2}

    def both(entries):
        outs = []
        for rn in (graphed, eager):
            batch = [StepEntry(ids[r], toks[r][rn.computed_len(ids[r]):rn.computed_len(ids[r]) + n],
                               rn.computed_len(ids[r]), [n - 1]) for r, n in entries]
            outs.append(rn.step(batch).cpu())
        return outs

    g, e = both([("a", 40), ("b", 20)])
    assert torch.equal(g, e)
    replays = 0
    for step in range(25):
        g, e = both([("a", 1), ("b", 1)])          # the same shape again and again: captured, then replayed
        assert torch.equal(g, e), f"decode step {step}"
        replays += 1
        if step % 6 == 2:                          # eager work between replays
            g, e = both([("c", 7)])
            assert torch.equal(g, e)
        if step == 12:
            torch.cuda.synchronize()
    assert (2, 1) in graphed._graphs and graphed._graphs[(2, 1)].graph is not None
    assert not eager._graphs
    # three decoding requests: another graph; then back to two
    for step in range(4):
        g, e = both([("a", 1), ("b", 1), ("c", 1)])
        assert torch.equal(g, e)
    g, e = both([("b", 1), ("a", 1)])
    assert torch.equal(g, e)
    # and all of it equals the plain model
    got = {("a", graphed.computed_len(0) - 1): g[1], ("b", graphed.computed_len(1) - 1): g[0]}
    check_against_plain(model_dirs[name], {k: v for k, v in toks.items() if k != "c"}, got, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["E", "LLAMA_1B"])
def test_prompt_graphs_replay_like_eager_steps(model_dirs, tmp_path, name, dtype):
    """A prompt (or a portion of one) alone in its step is recorded as a graph the third time its first position and
    length are seen.  Every replay, with other tokens each time, is compared with the same step run eagerly, with
    eager work and synchronisations between the replays (the library's products are part of such a graph: what they
    record must replay right every time)."""
    from atoma_infer_amd.engine import StepEntry
    if name == "LLAMA_1B":
        if dtype != "bfloat16":
            pytest.skip("the serving sizes run in bfloat16")
        model_dir = make_model_dir(str(tmp_path / "m"), LLAMA_1B_LAYERS, seed=4, dtype="bfloat16", norm_jitter=0.1)
        vocab, page, first, second = LLAMA_1B_LAYERS["vocab_size"], 16, 2048, 700
    else:
        model_dir, vocab, page, first, second = model_dirs[name], TINY[name]["vocab_size"], PAGE[name], 300, 270
    pages = -(-(first + second) // page) + 2
    graphed = make_runner(model_dir, dtype, page, pages)
    eager = make_runner(model_dir, dtype, page, pages)
    eager.use_graphs = False
    for rep in range(7):
        toks = random_tokens(first + second, vocab, 900 + rep)
        outs = []
        for rn in (graphed, eager):
            rn.add_request(rep)
            a = rn.step([StepEntry(rep, toks[:first], 0, [first - 1])]).cpu()
            if rep == 4:
                torch.cuda.synchronize()
            b = rn.step([StepEntry(rep, toks[first:first + second], first, [])])          # a portion that wants nothing
            assert b is None
            outs.append(a)
            rn.free_request(rep)
        assert torch.equal(outs[0], outs[1]), f"prompt {rep}"
    keys = [k for k in graphed._graphs if k[0] == "prompt"]
    assert ("prompt", 0, first, 1) in keys and ("prompt", first, second, 0) in keys
    assert all(graphed._graphs[k].graph is not None for k in keys) and not eager._graphs
    # what the second portion left in the cache is what an eager step leaves: decode on top of both
    toks = random_tokens(first + second + 1, vocab, 77)
    outs = []
    for rn in (graphed, eager):
        rn.add_request(99)
        rn.step([StepEntry(99, toks[:first], 0, [first - 1])])
        rn.step([StepEntry(99, toks[first:first + second], first, [])])
        outs.append(rn.step([StepEntry(99, toks[first + second:], first + second, [0])]).cpu())
        rn.free_request(99)
    assert torch.equal(outs[0], outs[1])
    if name == "E":
        check_against_plain(model_dir, {"r": toks}, {("r", first + second): outs[0][0]}, dtype)


def test_decoding_with_whole_key_ranges(model_dirs, monkeypatch):
    """Many decoding requests make every (request, KV head) pair one attention task for eight waves.  Here the
    threshold is lowered so that three requests do it: decoded through graphs, against the plain model."""
    from atoma_infer_amd.kernels import attention_bf16
    monkeypatch.setattr(attention_bf16, "WHOLE_MIN_PAIRS", 2)
    name, dtype = "D", "bfloat16"
    vocab = TINY[name]["vocab_size"]
    requests = {"a": random_tokens(700, vocab, 31), "b": random_tokens(90, vocab, 32), "c": random_tokens(300, vocab, 33)}
    runner = make_runner(model_dirs[name], dtype, PAGE[name], 80)
    steps = [([("a", 660), ("b", 50), ("c", 260)], [])] + [([("a", 1), ("b", 1), ("c", 1)], []) for _ in range(40)]
    got = run_schedule(runner, requests, steps)
    check_against_plain(model_dirs[name], requests, got, dtype)
    g = runner._graphs.get((3, 3))
    assert g is not None and g.graph is not None, "the decode steps were meant to replay as a graph"
    assert attention_bf16.chunk_for(3, 700, 2, whole_ok=True) == (0, 8)


def test_decoding_at_contexts_of_thousands_of_tokens(tmp_path):
    """Beyond a few thousand keys a decoded token's chunks grow with the step's tasks, four waves share each and the
    attention kernel merges a row piece's parts itself, twenty of them here.  Three requests of 5,000, 2,290 and 40
    tokens decode together through graphs; the second crosses the length at which the plans change."""
    from atoma_infer_amd.kernels import attention_bf16
    cfg = dict(TINY["D"], max_position_embeddings=8192)
    path = make_model_dir(str(tmp_path / "long"), cfg, seed=21, dtype="bfloat16", norm_jitter=0.1)
    vocab = cfg["vocab_size"]
    requests = {"a": random_tokens(5000, vocab, 41), "b": random_tokens(2330, vocab, 42), "c": random_tokens(82, vocab, 43)}
    runner = make_runner(path, "bfloat16", 16, 480)
    steps = [([("a", 2048)], []), ([("a", 2048)], []), ([("a", 862), ("b", 1100)], []), ([("b", 1188), ("c", 40)], [])]
    steps += [([("a", 1), ("b", 1), ("c", 1)], []) for _ in range(42)]
    got = run_schedule(runner, requests, steps)
    check_against_plain(path, requests, got, "bfloat16")
    graphs = [k for k, g in runner._graphs.items() if g.graph is not None]
    assert any(k[0] == 3 for k in graphs), "the decode steps were meant to replay as graphs"
    assert attention_bf16.chunk_for(3, 5120, 2, whole_ok=True) == (256, 4)
    assert attention_bf16.merges_in_kernel(5120, 4)


LLAMA_1B_LAYERS = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 2048, "intermediate_size": 8192,
    "vocab_size": 128256, "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 8,
    "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192, "rope_type": "llama3"},
    "max_position_embeddings": 131072, "tie_word_embeddings": True,
}


# the widths of Llama 3.1 8B (heads of 128, where the bfloat16 attention has one wave per task only) with one layer,
# an untied head and a smaller vocabulary that is no multiple of anything
LLAMA_8B_LAYER = dict(LLAMA_1B_LAYERS, hidden_size=4096, intermediate_size=14336, vocab_size=32003,
                      num_hidden_layers=1, tie_word_embeddings=False)


@pytest.mark.parametrize("cfg", [LLAMA_1B_LAYERS, LLAMA_8B_LAYER], ids=["1b", "8b"])
def test_layers_of_serving_size_in_mixed_steps(tmp_path, cfg, monkeypatch):
    """Layers with the sizes of Llama 3.2 1B (and its whole vocabulary) and of Llama 3.1 8B: at these widths the
    products take other plans (wider waves, K split over the grid, the library from 65 rows on) than any tiny
    configuration reaches."""
    model_dir = make_model_dir(str(tmp_path / "m"), cfg, seed=3, dtype="bfloat16", norm_jitter=0.1)
    vocab = cfg["vocab_size"]
    requests = {"a": random_tokens(300, vocab, 1), "b": random_tokens(90, vocab, 2), "c": random_tokens(33, vocab, 3)}
    steps = [([("a", 200)], []), ([("a", 37), ("b", 50)], []), ([("a", 2), ("b", 1), ("c", 30)], [])]
    steps += [([("a", 1), ("b", 1), ("c", 1)], [])] * 3
    steps += [([("a", 58), ("b", 36)], ["a", "b", "c"])]
    from atoma_infer_amd.kernels import gemm_bf16
    for dtype in DTYPES:
        runner = make_runner(model_dir, dtype, 16, 40)
        got = run_schedule(runner, requests, steps)
        assert len(got) == 300 + 90 + 33
        check_against_plain(model_dir, requests, got, dtype)
        assert runner.manager.num_free_pages() == 40
        if dtype == "bfloat16":
            # steps of few rows read copies of the weights in the order their kernels read them; without the copies
            # the same steps give the same bits
            block = runner.model.spec.layers[0][1]
            copies = [block.mixer.w_qkv_tiled, block.mixer.w_o_tiled, block.feed_forward.w_gate_up_tiled,
                      block.feed_forward.w_down_tiled]
            if vocab % 32 == 0:             # (a vocabulary that does not divide into the kernel's tiles has no copy)
                copies.append(runner.model.spec.head[1].tiled)
            assert all(c is not None for c in copies), copies
            del runner, block, copies
            torch.cuda.empty_cache()
            monkeypatch.setattr(gemm_bf16, "TILED_COPIES", False)
            runner = make_runner(model_dir, dtype, 16, 40)
            block = runner.model.spec.layers[0][1]
            assert block.mixer.w_o_tiled is None and block.feed_forward.w_gate_up_tiled is None
            plain_layout = run_schedule(runner, requests, steps)
            monkeypatch.undo()
            assert got.keys() == plain_layout.keys() and all(torch.equal(got[k], plain_layout[k]) for k in got)
            del block
        del runner
        torch.cuda.empty_cache()
    _plain_cache.clear()


def _four_schedules(requests, rng):
    """For requests r0..: each alone and whole; most of r0 in one step and its last 32 tokens one by one; r0 in portions
    of changing size down to two tokens; all mixed, up to four live, portions beside decoded tokens."""
    names = list(requests)
    whole = [([(r, len(requests[r]))], [r]) for r in names]
    n0 = len(requests[names[0]])
    last32 = [([(names[0], n0 - 32)], [])] + [([(names[0], 1)], [])] * 31 + [([(names[0], 1)], [names[0]])]
    sizes, left, cycle, i = [], n0, [17, 2, 31, 3, 16, 2, 5, 33, 1, 4], 0
    while left:
        sizes.append(min(cycle[i % len(cycle)], left))
        left -= sizes[-1]
        i += 1
    portions = [([(names[0], k)], [names[0]] if j == len(sizes) - 1 else []) for j, k in enumerate(sizes)]
    mixed, waiting, live, done = [], list(names), [], {r: 0 for r in names}
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            left = len(requests[r]) - done[r]
            n = 1 if left <= 6 else min(rng.choice([2, 3, 5, 8, 13, 24]), left - 6)
            if rng.random() < 0.15 and len(live) > 1:
                continue
            entries.append((r, n))
            done[r] += n
            if done[r] == len(requests[r]):
                end.append(r)
        if entries:
            rng.shuffle(entries)
            mixed.append((entries, end))
            live = [r for r in live if r not in end]
    return {"whole": whole, "last 32 one by one": last32, "portions": portions, "mixed": mixed}


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_checkpoint_stored_in_float32(tmp_path, dtype):
    """Tensors stored in 32 bits stay float32 on the device whatever the activation dtype is: the four schedules at
    Tiny B from such a file, against the plain model on the same float32 numbers."""
    name = "B"
    model_dir = make_model_dir(str(tmp_path / "m"), TINY[name], seed=17, dtype="float32", norm_jitter=NORM_JITTER[name])
    vocab = TINY[name]["vocab_size"]
    lens = [120, 1, 77, 90, 45, 18]
    requests = {f"r{i}": random_tokens(n, vocab, 500 + i) for i, n in enumerate(lens)}
    need = sum(sorted(-(-n // 16) for n in lens)[-4:])
    for kind, steps in _four_schedules(requests, random.Random(2)).items():
        runner = make_runner(model_dir, dtype, 16, need, slots=4)
        stored = {w.dtype for _, blk in runner.model.spec.layers for w in (blk.mixer.w_qkv, blk.mixer.w_o)}
        assert stored == {torch.float32}, stored
        got = run_schedule(runner, requests, steps)
        check_against_plain(model_dir, requests, got, dtype)
        assert runner.manager.num_free_pages(0) == need, kind
    _plain_cache.clear()


def test_all_sixteen_layers_of_llama_1b_size(tmp_path):
    """The whole Llama 3.2 1B shape (16 layers, the full vocabulary, tied head, llama3 scaling with its own
    constants) against the plain model (models/src/llama.rs:456-478): a prompt in uneven portions, three live
    requests, a fourth that takes over the pages of the first, float32 and bfloat16."""
    cfg = dict(LLAMA_1B_LAYERS, num_hidden_layers=16)
    model_dir = make_model_dir(str(tmp_path / "m"), cfg, seed=9, dtype="bfloat16", norm_jitter=0.1)
    vocab = cfg["vocab_size"]
    requests = {"a": random_tokens(150, vocab, 1), "b": random_tokens(72, vocab, 2), "c": random_tokens(33, vocab, 3),
                "d": random_tokens(90, vocab, 4)}
    steps = [([("a", 93)], []), ([("a", 37), ("b", 50)], []), ([("a", 2), ("b", 1), ("c", 30)], [])]
    steps += [([("a", 1), ("b", 1), ("c", 1)], [])] * 3
    steps += [([("a", 15), ("b", 16)], ["a", "c"])]
    steps += [([("d", 67), ("b", 1)], []), ([("d", 2)], []), ([("d", 21), ("b", 1)], ["b", "d"])]
    pages = 10 + 5 + 3 + 1             # a, b, c and one to spare: d (6 pages) must take what a gave back
    for dtype in DTYPES:
        runner = make_runner(model_dir, dtype, 16, pages, slots=3)
        got = run_schedule(runner, requests, steps)
        assert len(got) == sum(len(v) for v in requests.values())
        worst = check_against_plain(model_dir, requests, got, dtype)
        print(f"16 layers, {dtype}: worst error {worst:.3e}", flush=True)
        assert runner.manager.num_free_pages() == pages
        del runner
        torch.cuda.empty_cache()
    _plain_cache.clear()


def test_decode_graphs_with_library_products_inside(tmp_path):
    """With more than 64 decoding requests the linears of a step are the library's, inside the recorded graph.
    Every replay is compared with the same step run eagerly, with eager work and a synchronisation between
    replays: a library call that clears memory through a node of its own would show here after the first replay."""
    from atoma_infer_amd.engine import StepEntry
    model_dir = make_model_dir(str(tmp_path / "m"), LLAMA_1B_LAYERS, seed=5, dtype="bfloat16", norm_jitter=0.1)
    vocab, n_req = LLAMA_1B_LAYERS["vocab_size"], 70
    toks = [random_tokens(22 + (i % 9) + 14, vocab, 200 + i) for i in range(n_req + 1)]
    graphed = make_runner(model_dir, "bfloat16", 16, 4 * (n_req + 1), slots=n_req + 1)
    eager = make_runner(model_dir, "bfloat16", 16, 4 * (n_req + 1), slots=n_req + 1)
    eager.use_graphs = False
    for rn in (graphed, eager):
        for i in range(n_req + 1):
            rn.add_request(i)

    def both(entries):
        outs = []
        for rn in (graphed, eager):
            batch = [StepEntry(r, toks[r][rn.computed_len(r):rn.computed_len(r) + n], rn.computed_len(r), [n - 1])
                     for r, n in entries]
            outs.append(rn.step(batch).clone())
        return outs

    g, e = both([(r, len(toks[r]) - 14) for r in range(n_req)])          # the prompts, one step
    assert torch.equal(g, e)
    for step in range(12):
        g, e = both([(r, 1) for r in range(n_req)])
        assert torch.equal(g, e), f"decode step {step}"
        assert bool(torch.isfinite(g).all())
        if step in (3, 7):
            g, e = both([(n_req, 9)])                                      # eager work between replays
            assert torch.equal(g, e)
        if step == 5:
            torch.cuda.synchronize()
    key = (n_req, 1)
    assert key in graphed._graphs and graphed._graphs[key].graph is not None and not eager._graphs
    # and the last replay against the plain model, for a few of the requests
    last = {r: graphed.computed_len(r) - 1 for r in (0, 33, 69)}
    got = {(f"r{r}", p): g[r].cpu() for r, p in last.items()}
    check_against_plain(model_dir, {f"r{r}": toks[r] for r in last}, got, "bfloat16")
    _plain_cache.clear()


def test_decode_graphs_are_dropped_and_recorded_again(model_dirs, monkeypatch):
    """Only so many graphs are kept; the one unused longest goes.  With room for two, steps of one to four requests
    take turns, so that graphs are dropped while the step before may still run, and recorded anew."""
    from atoma_infer_amd.engine import StepEntry, step as step_module
    monkeypatch.setattr(step_module, "MAX_GRAPHS", 2)
    name, dtype = "B", "bfloat16"
    vocab = TINY[name]["vocab_size"]
    toks = [random_tokens(120, vocab, 300 + i) for i in range(4)]
    graphed = make_runner(model_dirs[name], dtype, PAGE[name], 40)
    eager = make_runner(model_dirs[name], dtype, PAGE[name], 40)
    eager.use_graphs = False
    for rn in (graphed, eager):
        for i in range(4):
            rn.add_request(i)

    def both(entries):
        outs = []
        for rn in (graphed, eager):
            batch = [StepEntry(r, toks[r][rn.computed_len(r):rn.computed_len(r) + n], rn.computed_len(r), [n - 1])
                     for r, n in entries]
            outs.append(rn.step(batch).clone())
        return outs

    g, e = both([(r, 20 + r) for r in range(4)])
    assert torch.equal(g, e)
    recorded = set()
    for step in range(48):
        n = [1, 2, 3, 4, 2, 1, 4, 3][step % 8] if step % 3 else 2
        g, e = both([(r, 1) for r in range(n)])
        assert torch.equal(g, e), f"step {step} with {n} requests"
        assert len(graphed._graphs) <= 2
        recorded |= {k for k, v in graphed._graphs.items() if v.graph is not None}
    assert len(recorded) >= 2          # graphs were recorded, dropped and recorded again along the way
    got = {("r0", graphed.computed_len(0) - 1): g[0].cpu()}
    check_against_plain(model_dirs[name], {"r0": toks[0]}, got, dtype)


def _random_configuration(rng):
    """Every size drawn: head size in steps of 16, any number of heads and groups, widths and a vocabulary that
    are no powers of two (the feed-forward width sometimes no multiple of 8), one to three layers."""
    hd = rng.choice(list(range(16, 257, 16)))
    nkv = rng.choice([1, 2, 3, 5])
    nh = nkv * rng.choice([1, 2, 3, 4, 7])
    while nh * hd > 1536:
        nh = max(nh // 2, 1)
    if nh % nkv:
        nkv = 1
    cfg = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": nh * hd,
           "intermediate_size": rng.choice([rng.randint(8, 700), 8 * rng.randint(2, 90), 32 * rng.randint(1, 24)]),
           "vocab_size": rng.randint(50, 3000), "num_hidden_layers": rng.randint(1, 3),
           "num_attention_heads": nh, "num_key_value_heads": nkv, "rms_norm_eps": rng.choice([1e-5, 1e-6, 3e-6]),
           "rope_theta": rng.choice([10000.0, 500000.0]), "max_position_embeddings": 1024,
           "tie_word_embeddings": rng.random() < 0.5}
    if rng.random() < 0.5:
        cfg["rope_scaling"] = {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                               "original_max_position_embeddings": 64, "rope_type": "llama3"}
    return cfg


@pytest.mark.parametrize("seed", range(16))
def test_random_configurations_step_like_the_plain_model(tmp_path, seed):
    rng = random.Random(7000 + seed)
    _step_a_random_schedule(tmp_path, _random_configuration(rng), rng, seed)


@pytest.mark.parametrize("hd", [8, 24, 40, 72, 88, 104, 120, 136, 200, 248])
def test_head_sizes_that_are_odd_multiples_of_eight(tmp_path, hd):
    """The reference's attention takes every head size that is a multiple of 8 up to 256 (csrc/src/lib.rs:136-143,
    790); here those that are no multiple of 16 run the general attention kernel, in both dtypes."""
    rng = random.Random(9000 + hd)
    cfg = _random_configuration(rng)
    nkv = rng.choice([1, 2, 3])
    nh = nkv * rng.choice([1, 2, 4])
    while nh * hd > 1024 and nh > nkv:
        nh //= 2
    cfg.update(hidden_size=nh * hd, num_attention_heads=nh, num_key_value_heads=nkv)
    _step_a_random_schedule(tmp_path, cfg, rng, hd)


def _step_a_random_schedule(tmp_path, cfg, rng, seed):
    model_dir = make_model_dir(str(tmp_path / "m"), cfg, seed=seed, dtype="bfloat16", norm_jitter=0.1)
    vocab = cfg["vocab_size"]
    la, lb, lc = rng.randint(150, 400), rng.randint(20, 200), rng.randint(2, 70)
    requests = {"a": random_tokens(la, vocab, 1), "b": random_tokens(lb, vocab, 2), "c": random_tokens(lc, vocab, 3)}
    first = rng.randint(1, la - 40)
    steps, left = [([("a", first)], [])], {"a": la - first, "b": lb, "c": lc}
    while any(left.values()):
        entries = []
        for k in ("a", "b", "c"):
            if left[k] and rng.random() < 0.8:
                n = min(left[k], rng.choice([1, 1, 1, 2, 3, 17, 40, 70, 130]))
                entries.append((k, n))
                left[k] -= n
        if entries:
            rng.shuffle(entries)
            steps.append((entries, []))
    pages = sum(-(-len(v) // 16) for v in requests.values()) + 2
    for dtype in DTYPES:
        runner = make_runner(model_dir, dtype, 16, pages)
        got = run_schedule(runner, requests, steps)
        check_against_plain(model_dir, requests, got, dtype)
        del runner
    _plain_cache.clear()
