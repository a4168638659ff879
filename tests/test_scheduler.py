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


def test_a_request_alone_takes_shorter_portions_before_it_gives_up():
    cache2 = CacheManager([GroupGeometry(4, 5)], 8)
    s2 = Scheduler(SchedulerConfig(max_num_batched_tokens=64, max_num_sequences=8, max_model_len=256), cache2)
    blocker, c = make_request(5, 4, max_new=30), make_request(6, 16)
    s2.add(blocker)
    run_step(s2, s2.schedule())                 # blocker holds 1 page (4 tokens) and will need a 2nd
    s2.add(c)
    out = s2.schedule()                         # blocker decodes (page 2), c's 16 tokens need 4 pages, 3 are free
    assert [(e.request.uid, e.num_tokens) for e in out.entries] == [(5, 1)]      # the head of the queue waits
    s2.finish(blocker, Status.FINISHED_STOPPED)
    out = s2.schedule()
    assert [(e.request.uid, e.num_tokens) for e in out.entries] == [(6, 16)]
    run_step(s2, out)
    # alone with 4 of 5 pages: decoding goes on until the pool is full, then it is capped, not preempted
    for _ in range(8):
        out = s2.schedule()
        if out.capped:
            break
        assert [(e.request.uid, e.num_tokens) for e in out.entries] == [(6, 1)]
        run_step(s2, out)
    assert [r.uid for r in out.capped] == [6] and c.num_computed == 20
    # a running request whose next portion does not fit while it is alone takes half of it, and half again
    cache3 = CacheManager([GroupGeometry(4, 6)], 8)
    s3 = Scheduler(SchedulerConfig(max_num_batched_tokens=8, max_num_sequences=8, max_model_len=256,
                                   max_prefill_chunk=0), cache3)
    d = make_request(7, 23)                     # 6 pages in all: fits at all
    s3.add(d)
    for want in (8, 8):
        out = s3.schedule()
        assert [(e.request.uid, e.num_tokens) for e in out.entries] == [(7, want)]
        run_step(s3, out)
    hog = cache3._lib.cm_add_request(cache3.handle, 99)       # someone else takes the last two pages but one
    assert hog >= 0
    cache3.reserve(99, 4)
    out = s3.schedule()                         # 7 tokens left need 2 pages, 1 is free: 7 // 2 = 3 fit
    assert [(e.request.uid, e.num_tokens, e.do_sample) for e in out.entries] == [(7, 3, False)]
    cache3.check()


def test_a_window_of_keys_lets_long_requests_into_a_small_pool():
    """A group that keeps a window gives pages back as a request moves on (cache_manager.cpp): the pool must hold
    the window and one page more, not the whole request."""
    cache = CacheManager([GroupGeometry(4, 5, window=10)], 4)
    assert cache.fits_at_all(1000) and not CacheManager([GroupGeometry(4, 3, window=10)], 4).fits_at_all(1000)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=8, max_num_sequences=4, max_model_len=2000), cache)
    a = make_request(0, 100, max_new=4)
    s.add(a)
    steps = 0
    while s.has_unfinished():
        out = s.schedule()
        assert not out.ignored and not out.capped and out.entries
        for e in out.entries:
            cache.release_behind(e.request.uid, e.request.num_computed + e.num_tokens)    # as the runner does
        run_step(s, out)
        cache.check()
        steps += 1
        assert steps < 200
    assert len(a.output_ids) == 4 and cache.num_free_pages() == 5


def _run_windowed(cache, s, reqs, limit=400):
    steps = preempted = 0
    while s.has_unfinished():
        out = s.schedule()
        assert out.entries or out.ignored or out.capped or out.preempted, "an empty plan: nothing would ever change"
        preempted += len(out.preempted)
        for e in out.entries:
            cache.release_behind(e.request.uid, e.request.num_computed + e.num_tokens)    # as the runner does
        run_step(s, out)
        cache.check()
        steps += 1
        assert steps < limit
    return steps, preempted


def test_a_first_portion_longer_than_the_pool_is_shortened_not_waited_for():
    """A prompt of 100 tokens, a token budget of 64, a pool of 20 tokens that keeps a window of 10: the first
    portion must shrink to what the idle pool holds (waiting frees nothing), and the request runs to its end."""
    cache = CacheManager([GroupGeometry(4, 5, window=10)], 4)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=64, max_num_sequences=4, max_model_len=2000), cache)
    a = make_request(0, 100, max_new=4)
    s.add(a)
    out = s.schedule()
    assert [(e.request.uid, e.num_tokens) for e in out.entries] == [(0, 16)]      # 64 -> 32 -> 16 tokens = 4 pages
    for e in out.entries:
        cache.release_behind(e.request.uid, e.num_tokens)
    run_step(s, out)
    _run_windowed(cache, s, [a])
    assert len(a.output_ids) == 4 and cache.num_free_pages() == 5 and a.status.finished


def test_an_uncut_prompt_longer_than_a_windowed_pool_is_ignored():
    cache = CacheManager([GroupGeometry(4, 5, window=10)], 4)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=2000, max_num_sequences=4, max_model_len=2000,
                                  enable_chunked_prefill=False), cache)
    a, b = make_request(0, 100), make_request(1, 12, max_new=3)
    s.add(a)
    s.add(b)
    out = s.schedule()
    assert [r.uid for r in out.ignored] == [0] and [e.request.uid for e in out.entries] == [1]


def test_admission_into_a_windowed_pool_leaves_room_for_those_already_there():
    """Two long requests and a pool that holds the window (and one page) of two requests but not of three: the
    third waits until one of the others is done instead of being admitted and preempted over and over."""
    cache = CacheManager([GroupGeometry(4, 9, window=10)], 4)         # steady need: 3 + 1 pages a request
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=8, max_num_sequences=4, max_model_len=2000), cache)
    reqs = [make_request(i, 40, max_new=30) for i in range(3)]
    for r in reqs:
        s.add(r)
    out = s.schedule()
    assert [e.request.uid for e in out.entries] == [0]                 # 8 tokens of budget: one portion
    steps, preempted = _run_windowed(cache, s, reqs)
    assert preempted == 0 and all(len(r.output_ids) == 30 for r in reqs) and cache.num_free_pages() == 9


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


def test_portions_end_where_the_model_allows():
    """``ModelSpec.chunk_alignment``: a portion that does not end the request's tokens ends at a multiple of it,
    under a token budget shared with decoding requests, and the last portion is free."""
    cache = CacheManager([GroupGeometry(4, 64)], 8)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=21, max_num_sequences=8, max_model_len=256), cache,
                  chunk_alignment=8)
    a, b = make_request(0, 45, max_new=3), make_request(1, 30, max_new=3)
    s.add(a)
    s.add(b)
    seen = []
    while s.has_unfinished():
        out = s.schedule()
        assert out.num_tokens <= 21
        for e in out.entries:
            end = e.start + e.num_tokens
            assert e.num_tokens == 1 or e.start % 8 == 0
            assert end % 8 == 0 or end == e.request.length, (e.request.uid, e.start, e.num_tokens)
        seen.append([(e.request.uid, e.num_tokens) for e in out.entries])
        run_step(s, out)
    assert seen[0] == [(0, 16)] and seen[1] == [(0, 16)]          # 21 tokens of budget: 16 is what ends aligned
    assert seen[2] == [(0, 13), (1, 8)]                             # the rest of a (unaligned, its last), 8 of b
    import pytest
    from atoma_infer_amd.engine.scheduler import SchedulerError
    with pytest.raises(SchedulerError):                              # no aligned portion fits such a budget
        Scheduler(SchedulerConfig(max_num_batched_tokens=6, max_num_sequences=4, max_model_len=256), cache,
                  chunk_alignment=8)
    # ... nor one that an aligned portion fits only while nothing decodes: the prompt would stand still meanwhile
    with pytest.raises(SchedulerError, match="alignment"):
        Scheduler(SchedulerConfig(max_num_batched_tokens=8, max_num_sequences=2, max_model_len=256), cache,
                  chunk_alignment=8)


def test_an_aligned_portion_fits_beside_every_decoding_request():
    """The smallest budget the scheduler takes with aligned portions (alignment + requests - 1): one request decodes,
    another is in its prompt, and the prompt moves on by an aligned portion in every step."""
    cache = CacheManager([GroupGeometry(4, 64)], 4)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=9, max_num_sequences=2, max_model_len=256), cache,
                  chunk_alignment=8)
    a, b = make_request(0, 5, max_new=12), make_request(1, 40, max_new=2)
    s.add(a)
    run_step(s, s.schedule())                                        # a's prompt; a decodes from here on
    s.add(b)
    starts = []
    for _ in range(5):
        out = s.schedule()
        plan = {e.request.uid: (e.start, e.num_tokens) for e in out.entries}
        assert plan[0][1] == 1 and plan[1][1] == 8, plan           # a decodes, b takes 8 of its 40
        starts.append(plan[1][0])
        run_step(s, out)
    assert starts == [0, 8, 16, 24, 32]


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


def test_delay_factor_holds_admissions_back_while_something_runs():
    """backends/vllm/src/scheduler.rs:2077-2097: after a step with a prompt, a waiting request is admitted only
    once it has waited longer than delay_factor times that step's duration, or when nothing runs."""
    now = [0.0]
    cache = CacheManager([GroupGeometry(4, 64)], 8)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=64, max_num_sequences=8, max_model_len=256,
                                  delay_factor=2.0), cache, clock=lambda: now[0])
    a = make_request(0, 10)
    a.metrics.arrival_time = 0.0
    s.add(a)
    out = s.schedule()                       # nothing runs: admitted at once
    assert [e.request.uid for e in out.entries] == [0]
    run_step(s, out)
    now[0] = 1.0                             # the prompt step took 1.0
    b = make_request(1, 10)
    b.metrics.arrival_time = 1.0
    s.add(b)
    out = s.schedule()
    assert s.last_prompt_latency == 1.0
    assert [e.request.uid for e in out.entries] == [0]          # b has waited 0 < 2 * 1.0
    run_step(s, out)
    now[0] = 2.5
    out = s.schedule()
    assert [e.request.uid for e in out.entries] == [0]          # 1.5 < 2.0
    run_step(s, out)
    now[0] = 3.5
    out = s.schedule()
    assert [e.request.uid for e in out.entries] == [0, 1]       # 2.5 > 2.0


class _Limits:
    def __init__(self, **kw):
        self.__dict__.update(kw)


def _random_world(seed):
    """The same random traffic through the native scheduler and the plain one; every plan must be the same.

    The engine's pipelining is played too: a sampled token is pending for one step, a request whose last token is
    pending is frozen, and a request may end (or be aborted) while it waits after a preemption."""
    from plain_scheduler import PlainPages, PlainRequest, PlainScheduler
    rng = random.Random(seed)
    page, pages, slots = rng.choice([1, 3, 4, 16]), rng.randint(3, 40), rng.randint(1, 6)
    lim = _Limits(max_tokens=rng.randint(4, 48), max_requests=rng.randint(1, 6), max_model_len=rng.randint(30, 120),
                  cut=rng.random() < 0.8, max_portion=rng.choice([0, 0, 5, 16]),
                  delay_factor=rng.choice([0.0, 0.0, 0.5, 3.0]))
    lim.align = rng.choice([1, 1, 1, 4, 8])
    if not lim.cut:
        lim.max_tokens = max(lim.max_tokens, lim.max_model_len)      # the configuration demands it
    lim.max_tokens = max(lim.max_tokens, lim.max_requests, lim.align)
    if lim.cut and lim.align > 1:
        lim.max_tokens = max(lim.max_tokens, lim.align + lim.max_requests - 1)   # room for an aligned portion
    if lim.max_portion:
        lim.max_portion = max(lim.max_portion, lim.align)
    now = [0.0]
    window = rng.choice([0, 0, 5, 12, 33])
    cache = CacheManager([GroupGeometry(page, pages, window=window or None)], slots)
    native = Scheduler(SchedulerConfig(max_num_batched_tokens=lim.max_tokens, max_num_sequences=lim.max_requests,
                                       max_model_len=lim.max_model_len, enable_chunked_prefill=lim.cut,
                                       max_prefill_chunk=lim.max_portion, delay_factor=lim.delay_factor),
                       cache, clock=lambda: now[0], chunk_alignment=lim.align)
    plain_pages = PlainPages(page, pages, slots, window)
    plain = PlainScheduler(lim, plain_pages)
    mine, theirs, uid = {}, {}, 0
    pending_mine, pending_theirs = [], []
    plans = preemptions = 0
    for step in range(rng.randint(40, 160)):
        now[0] += rng.choice([0.1, 0.5, 2.0])
        for _ in range(rng.choice([0, 0, 1, 1, 2, 4])):
            n, max_new = rng.choice([1, 2, 7, 20, 45, 130]), rng.choice([1, 2, 5, 30])
            a = make_request(uid, n, max_new=max_new)
            a.metrics.arrival_time = now[0]
            b = PlainRequest(uid, n, now[0], max_new)
            native.add(a)
            plain.add(b)
            mine[uid], theirs[uid] = a, b
            uid += 1
        if mine and rng.random() < 0.05:
            u = rng.choice(sorted(mine))
            assert native.abort(f"r{u}") is mine.pop(u)
            plain.take_out(theirs.pop(u), "aborted")
        out_a, out_b = native.schedule(), plain.schedule(now[0])
        plans += 1
        preemptions += len(out_b.preempted)
        assert [(e.request.uid, e.num_tokens, e.start, e.do_sample) for e in out_a.entries] == \
            [(r.uid, n, st, sm) for r, n, st, sm in out_b.entries], (seed, step)
        for name in ("preempted", "ignored", "capped"):
            assert [r.uid for r in getattr(out_a, name)] == [r.uid for r in getattr(out_b, name)], (seed, step, name)
        assert [r.uid for r in native.waiting] == [r.uid for r in plain.waiting], (seed, step)
        assert sorted(r.uid for r in native.running) == sorted(r.uid for r in plain.running), (seed, step)
        assert cache.num_free_pages() == plain_pages.free_pages() and \
            cache.num_free_slots() == plain_pages.num_free_slots(), (seed, step)
        assert out_a.num_tokens <= lim.max_tokens and len(out_a.entries) <= lim.max_requests
        cache.check()
        for r in out_a.ignored + out_a.capped:
            mine.pop(r.uid), theirs.pop(r.uid)
        for r in out_a.preempted:
            assert r.num_computed == 0 and r.status is Status.WAITING
        # the tokens of the step before reach the host: requests may end on them, also while they wait
        for a in pending_mine:
            a.pending -= 1
            if a.uid in mine:
                a.output_ids.append(7)
                if len(a.output_ids) >= a.plan.max_new_tokens or a.length > lim.max_model_len:
                    native.finish(mine.pop(a.uid), Status.FINISHED_LENGTH_CAPPED)
        for b in pending_theirs:
            b.pending -= 1
            if b.uid in theirs:
                b.outputs += 1
                if b.outputs >= b.max_new or b.length > lim.max_model_len:
                    plain.take_out(theirs.pop(b.uid), "capped")
        # this step runs: tokens are computed, sampled tokens are pending until the next step
        pending_mine, pending_theirs = [], []
        for e in out_a.entries:
            a = e.request
            a.num_computed += e.num_tokens
            cache.release_behind(a.uid, a.num_computed)          # as the runner does after a step
            if e.do_sample:
                a.pending += 1
                a.frozen = a.num_sampled >= a.plan.max_new_tokens or a.length > lim.max_model_len
                pending_mine.append(a)
        for b, n, _, sample in out_b.entries:
            b.num_computed += n
            plain_pages.release_behind(b.uid, b.num_computed)
            if sample:
                b.pending += 1
                b.frozen = b.num_sampled >= b.max_new or b.length > lim.max_model_len
                pending_theirs.append(b)
    assert native.num_preemptions == plain.num_preemptions
    return plans, preemptions


def test_native_scheduler_decides_like_the_plain_one_under_random_traffic():
    plans = preemptions = 0
    for seed in range(60):
        p, q = _random_world(seed)
        plans, preemptions = plans + p, preemptions + q
    assert plans > 3000 and preemptions > 50      # the traffic did drive pages out


def test_the_native_scheduler_refuses_what_does_not_fit_its_books():
    import pytest
    from atoma_infer_amd.engine.scheduler import SchedulerError
    s, cache = make_scheduler()
    a = make_request(0, 5)
    s.add(a)
    with pytest.raises(SchedulerError):
        s.add(make_request(0, 9))                      # the number is taken
    stranger = make_request(77, 5)
    with pytest.raises(SchedulerError):
        s.finish(stranger, Status.FINISHED_STOPPED)    # never queued
    out = s.schedule()
    assert [e.request.uid for e in out.entries] == [0] and s.num_unfinished() == 1
    # the runner's books are told of every request the scheduler registers or releases by itself
    calls = []

    class Books:
        def __init__(self, mgr):
            self._mgr = mgr

        def adopted(self, uid):
            calls.append(("adopted", uid, self._mgr.state_slot(uid)))

        def forgot(self, uid):
            calls.append(("forgot", uid, self._mgr.has(uid)))

        def __getattr__(self, name):
            return getattr(self._mgr, name)

    mgr = CacheManager([GroupGeometry(4, 4)], 4)
    s = Scheduler(SchedulerConfig(max_num_batched_tokens=64, max_num_sequences=4, max_model_len=64), Books(mgr))
    a, b = make_request(0, 7, max_new=6), make_request(1, 7, max_new=6)
    s.add(a)
    s.add(b)
    run_step(s, s.schedule())
    run_step(s, s.schedule())
    out = s.schedule()                                 # b is preempted: the pool is full
    assert [r.uid for r in out.preempted] == [1]
    s.abort("r0")
    assert calls == [("adopted", 0, 0), ("adopted", 1, 1), ("forgot", 1, False), ("forgot", 0, False)]
    mgr.check()
