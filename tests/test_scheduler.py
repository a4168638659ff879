"""The scheduler's decisions, on the CPU, against the real cache manager and a model that only appends tokens
(the reference tests its scheduler the same way: backends/vllm/src/scheduler.rs:2286-2353)."""
import itertools
import random


from atoma_infer_amd.cache import CacheManager, GroupGeometry
from atoma_infer_amd.config import SchedulerConfig
from atoma_infer_amd.engine.request import Request, RequestMetrics, Status
from atoma_infer_amd.engine.scheduler import Scheduler
from atoma_infer_amd.sampling.params import GenerateParameters, validate

_clock = itertools.count()


def make_request(uid, prompt_len, max_new=8):
    plan = validate(GenerateParameters(do_sample=False, max_new_tokens=max_new), prompt_len, 10_000, 20_000)
    return Request(uid, f"r{uid}", list(range(1, prompt_len + 1)), plan, RequestMetrics(arrival_time=next(_clock)))


def make_scheduler(pages=64, page=4, slots=8, **cfg):
    cfg.setdefault("max_num_batched_tokens", 32)
    cfg.setdefault("max_num_sequences", 8)
    cfg.setdefault("max_model_len", 256)
    cache = CacheManager([GroupGeometry(page, pages)], slots)
    return Scheduler(SchedulerConfig(**cfg), cache), cache


def run_step(s, out, finish_at=None):
    """What the engine does after a step: count computed tokens, append a token where one was sampled."""
    done = []
    for e in out.entries:
        r = e.request
        assert e.start == r.num_computed
        r.num_computed += e.num_tokens
        if e.do_sample:
            r.output_ids.append(1000 + len(r.output_ids))
            if len(r.output_ids) >= r.plan.max_new_tokens or (finish_at and len(r.output_ids) >= finish_at):
                s.finish(r, Status.FINISHED_LENGTH_CAPPED)
                done.append(r)
    return done


def test_prompts_are_cut_under_the_token_budget_and_decodes_come_first():
    s, cache = make_scheduler(max_num_batched_tokens=16)
    a, b = make_request(0, 40), make_request(1, 5)
    s.add(a)
    s.add(b)
    out = s.schedule()
    assert [(e.request.uid, e.num_tokens, e.start, e.do_sample) for e in out.entries] == [(0, 16, 0, False)]
    run_step(s, out)
    out = s.schedule()      # a continues (it is running), b waits for budget
    assert [(e.request.uid, e.num_tokens, e.start) for e in out.entries] == [(0, 16, 16)]
    run_step(s, out)
    out = s.schedule()      # a's last 8 tokens, then b fits whole
    assert [(e.request.uid, e.num_tokens, e.do_sample) for e in out.entries] == [(0, 8, True), (1, 5, True)]
    run_step(s, out)
    out = s.schedule()      # both decode
    assert [(e.request.uid, e.num_tokens, e.start) for e in out.entries] == [(0, 1, 40), (1, 1, 5)]
    assert out.num_tokens <= 16
    run_step(s, out)
    # a new prompt arrives: decodes first, then the new portion with what is left of the budget
    c = make_request(2, 30)
    s.add(c)
    out = s.schedule()
    assert [(e.request.uid, e.num_tokens) for e in out.entries] == [(0, 1), (1, 1), (2, 14)]
    cache.check()


def test_budgets_are_never_exceeded_and_everything_finishes():
    rng = random.Random(3)
    s, cache = make_scheduler(pages=40, max_num_batched_tokens=24, max_num_sequences=4)
    reqs = [make_request(i, rng.randint(1, 50), max_new=rng.randint(1, 12)) for i in range(20)]
    for r in reqs:
        s.add(r)
    finished, steps = [], 0
    while s.has_unfinished():
        out = s.schedule()
        assert not out.empty or out.ignored or out.capped
        assert out.num_tokens <= 24 and len(out.entries) <= 4
        assert len({e.request.uid for e in out.entries}) == len(out.entries)
        finished += run_step(s, out)
        cache.check()
        steps += 1
        assert steps < 2000
    assert len(finished) == 20 and cache.num_free_pages() == 40 and cache.num_requests() == 0
    for r in reqs:
        assert r.num_computed == r.length - 1 and len(r.output_ids) == r.plan.max_new_tokens


def test_first_come_first_served_and_head_of_line_blocking():
    s, cache = make_scheduler(pages=12, page=4, max_num_batched_tokens=64)
    a, b, c = make_request(0, 40), make_request(1, 30), make_request(2, 4)
    for r in (a, b, c):
        s.add(r)
    out = s.schedule()
    # a takes 10 pages; b (8 pages) does not fit and blocks c behind it although c would fit
    assert [e.request.uid for e in out.entries] == [0]
    assert [r.uid for r in s.waiting] == [1, 2]


def test_too_long_prompts_are_ignored():
    s, cache = make_scheduler(pages=8, page=4, max_model_len=64)
    long_for_model, long_for_pool, fine = make_request(0, 100), make_request(1, 40), make_request(2, 8)
    for r in (long_for_model, long_for_pool, fine):
        s.add(r)
    out = s.schedule()
    assert [r.uid for r in out.ignored] == [0, 1]
    assert long_for_model.status is Status.FINISHED_IGNORED and long_for_pool.status is Status.FINISHED_IGNORED
    assert [e.request.uid for e in out.entries] == [2]


def test_when_pages_run_out_the_latest_arrival_is_preempted_and_recomputed():
    """backends/vllm/src/scheduler.rs:650-690, 1778-1896: the victim is the back of the arrival-ordered running
    queue; it returns to the front of the waiting queue and later prefills prompt and generated tokens again."""
    s, cache = make_scheduler(pages=4, page=4, max_num_batched_tokens=64)
    a, b = make_request(0, 7, max_new=6), make_request(1, 7, max_new=6)
    s.add(a)
    s.add(b)
    out = s.schedule()
    assert [e.request.uid for e in out.entries] == [0, 1]
    run_step(s, out)                       # both now hold 8 tokens = 2 pages each: the pool is full
    out = s.schedule()
    assert [e.request.uid for e in out.entries] == [0, 1]
    run_step(s, out)                       # lengths 9: each needs a 3rd page at the next step
    out = s.schedule()
    assert [r.uid for r in out.preempted] == [1]
    assert [e.request.uid for e in out.entries] == [0]
    assert b.status is Status.WAITING and b.num_computed == 0 and list(s.waiting)[0] is b
    assert len(b.output_ids) == 2          # what it generated is kept
    assert b.metrics.num_preemptions == 1 and s.num_preemptions == 1
    cache.check()
    run_step(s, out)
    # a alone runs on; b cannot come back while a holds 3 of 4 pages and b needs 3
    out = s.schedule()
    assert [e.request.uid for e in out.entries] == [0] and [r.uid for r in s.waiting] == [1]
    finished = run_step(s, out)
    for _ in range(200):
        if not s.has_unfinished():
            break
        out = s.schedule()
        finished += run_step(s, out)
        cache.check()
    assert {r.uid for r in finished} == {0, 1} and cache.num_free_pages() == 4
    # b's recomputation prefilled its prompt and its generated tokens in one portion
    assert b.num_computed == b.length - 1


def test_a_request_that_outgrows_the_pool_alone_is_capped():
    s, cache = make_scheduler(pages=2, page=4, max_num_batched_tokens=64)
    a = make_request(0, 7, max_new=50)
    s.add(a)
    capped = []
    for _ in range(10):
        out = s.schedule()
        capped += out.capped
        run_step(s, out)
        if capped:
            break
    assert capped == [a] and a.status is Status.FINISHED_LENGTH_CAPPED
    assert cache.num_free_pages() == 2 and not s.has_unfinished()


def test_abort_frees_and_unchunked_prompts_wait_for_room():
    s, cache = make_scheduler(pages=128, page=4, max_num_batched_tokens=256, max_model_len=256,
                              enable_chunked_prefill=False)
    a, b = make_request(0, 100), make_request(1, 200)
    s.add(a)
    s.add(b)
    out = s.schedule()
    assert [(e.request.uid, e.num_tokens) for e in out.entries] == [(0, 100)]   # b is not cut to fit the rest
    run_step(s, out)
    assert s.abort("r0") is a and a.status is Status.FINISHED_ABORTED
    assert cache.num_free_pages() == 128
    assert s.abort("r1") is b and not s.has_unfinished()
    assert s.abort("nobody") is None


def test_max_prefill_chunk_caps_portions():
    s, cache = make_scheduler(max_num_batched_tokens=32, max_prefill_chunk=16)
    a = make_request(0, 37)
    s.add(a)
    sizes = []
    for _ in range(3):
        out = s.schedule()
        sizes.append(out.entries[0].num_tokens)
        run_step(s, out)
    assert sizes == [16, 16, 5]
