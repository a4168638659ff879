"""Continuous batching with chunked prefill.

Each call of ``schedule`` plans one step under a token budget (``max_num_batched_tokens``) and a request budget
(``max_num_sequences``), as the reference's chunked policy does (backends/vllm/src/scheduler.rs:1257-1379, budget
:40-149):

1. running requests that decode (one token each), in order of arrival;
2. running requests still in their prompt: the next portion, as large as the remaining budget allows
   (scheduler.rs:1588-1623);
3. waiting requests, first come first served, while budget and pages last; the head of the queue blocks those
   behind it (scheduler.rs:897-1016).  A prompt longer than ``max_model_len``, or one that the whole pool could
   not hold, is ignored (finish reason "ignored").

Pages are reserved for what a step adds, not for the whole prompt up front.  **When pages run out** for a running
request, the running request that arrived last is preempted by recomputation: its pages are given back, it
returns to the *front* of the waiting queue and later prefills its prompt and the tokens it had generated
(scheduler.rs:650-690, 1778-1896).  If the request that cannot grow is the only one running, it is finished as
"length_capped": nothing could be given back for it.

Differences from the reference, on purpose: portions of a prompt stay in the running queue until the prompt is
done (the reference drops them, scheduler.rs:1313-1338), pages are given back when a request finishes (the
reference frees only on abort and preemption), and there is no swap space.
"""
from __future__ import annotations

import dataclasses
import time
from collections import deque
from typing import Deque, List, Optional

from ..cache.manager import CacheManager
from ..config.engine import SchedulerConfig
from .request import Request, Status


@dataclasses.dataclass
class ScheduledEntry:
    request: Request
    num_tokens: int
    start: int
    do_sample: bool      # false for a portion that does not reach the end of what the request holds


@dataclasses.dataclass
class ScheduleOutput:
    entries: List[ScheduledEntry]
    preempted: List[Request]
    ignored: List[Request]
    capped: List[Request]

    @property
    def num_tokens(self) -> int:
        return sum(e.num_tokens for e in self.entries)

    @property
    def empty(self) -> bool:
        return not self.entries


class Scheduler:
    def __init__(self, config: SchedulerConfig, cache: CacheManager, clock=time.monotonic):
        config.validate()
        self.config, self.cache, self.clock = config, cache, clock
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.num_preemptions = 0
        self.last_prompt_latency = 0.0
        self._prev_prompt = False
        self._prev_time = 0.0

    # -- queue operations --------------------------------------------------------------------------------
    def add(self, request: Request) -> None:
        request.status = Status.WAITING
        self.waiting.append(request)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    def num_unfinished(self) -> int:
        return len(self.waiting) + len(self.running)

    def abort(self, request_id: str) -> Optional[Request]:
        """Remove a request wherever it is; its pages go back (scheduler.rs:390-443)."""
        for r in list(self.waiting):
            if r.request_id == request_id:
                self.waiting.remove(r)
                r.status = Status.FINISHED_ABORTED
                return r
        for r in self.running:
            if r.request_id == request_id:
                self.running.remove(r)
                self._release(r)
                r.status = Status.FINISHED_ABORTED
                return r
        return None

    def finish(self, request: Request, status: Status) -> None:
        """A request has produced its last token: give back what it holds.  It is usually running; it waits if it
        was preempted while that token was still on its way."""
        assert status.finished
        if request.status is Status.RUNNING:
            self.running.remove(request)
        else:
            self.waiting.remove(request)
        self._release(request)
        request.status = status

    def _release(self, r: Request) -> None:
        if self.cache.has(r.uid):
            self.cache.free(r.uid)

    # -- one step's plan -----------------------------------------------------------------------------------
    def _chunk(self, r: Request, budget: int) -> int:
        n = min(r.num_uncomputed, budget)
        if self.config.max_prefill_chunk > 0 and r.num_uncomputed > 1:
            n = min(n, self.config.max_prefill_chunk)
        if not self.config.enable_chunked_prefill and n < r.num_uncomputed:
            return 0  # prompts are not cut: wait for a step with room for all of it
        return n

    def _preempt(self, victim: Request, out: ScheduleOutput) -> None:
        self.running.remove(victim)
        self._release(victim)
        victim.num_computed = 0
        victim.status = Status.WAITING
        victim.metrics.num_preemptions += 1
        self.waiting.appendleft(victim)
        self.num_preemptions += 1
        out.preempted.append(victim)
        # a victim already planned into this step gives its place back
        out.entries[:] = [e for e in out.entries if e.request is not victim]

    def _passed_delay(self, now: float) -> bool:
        """The reference's optional batching delay (scheduler.rs:2077-2097)."""
        if self._prev_prompt:
            self.last_prompt_latency = now - self._prev_time
        self._prev_time, self._prev_prompt = now, False
        if self.config.delay_factor > 0 and self.waiting:
            earliest = min(r.metrics.arrival_time for r in self.waiting)
            return (now - earliest) > self.config.delay_factor * self.last_prompt_latency or not self.running
        return True

    def schedule(self) -> ScheduleOutput:
        out = ScheduleOutput([], [], [], [])
        cfg = self.config
        now = self.clock()
        self.running.sort(key=lambda r: r.metrics.arrival_time)  # first come first served (policy.rs:56-61)

        def used_tokens():
            return sum(e.num_tokens for e in out.entries)

        # 1 and 2: running requests, decodes before portions of prompts
        live = [r for r in self.running if not r.frozen]
        order = [r for r in live if not r.in_prefill] + [r for r in live if r.in_prefill]
        if len(order) <= cfg.max_num_sequences and len(order) <= cfg.max_num_batched_tokens and \
                all(r.num_uncomputed == 1 for r in order):
            # the common step: everything running decodes one token and fits both budgets; pages are taken
            # request by request, and the general path below takes over at the first that finds none
            done = 0
            for r in order:
                if not self.cache.can_reserve(r.uid, r.num_computed + 1):
                    break
                self.cache.reserve(r.uid, r.num_computed + 1)
                out.entries.append(ScheduledEntry(r, 1, r.num_computed, True))
                done += 1
            order = order[done:]
        for r in order:
            if r.status is not Status.RUNNING:
                continue  # preempted while serving an earlier request
            if len(out.entries) >= cfg.max_num_sequences:
                break
            n = self._chunk(r, cfg.max_num_batched_tokens - used_tokens())
            if n <= 0:
                continue
            while not self.cache.can_reserve(r.uid, r.num_computed + n):
                # the latest arrival that is not just waiting for its last token (that one frees its pages soon)
                victim = next((v for v in reversed(self.running) if not v.frozen), r)
                if victim is r and len(self.running) == 1:
                    # nothing else to give back: the pool cannot hold this request any longer
                    self.running.remove(r)
                    self._release(r)
                    r.status = Status.FINISHED_LENGTH_CAPPED
                    out.capped.append(r)
                    break
                self._preempt(victim, out)
                if victim is r:
                    break
            if r.status is not Status.RUNNING:
                continue
            self.cache.reserve(r.uid, r.num_computed + n)
            out.entries.append(ScheduledEntry(r, n, r.num_computed, r.num_computed + n == r.length))

        # 3: admissions, unless something was preempted in this step (its pages are meant for the running ones)
        if not out.preempted and self._passed_delay(now):
            while self.waiting:
                r = self.waiting[0]
                if r.length > cfg.max_model_len or not self.cache.fits_at_all(r.length):
                    self.waiting.popleft()
                    r.status = Status.FINISHED_IGNORED
                    out.ignored.append(r)
                    continue
                if len(out.entries) >= cfg.max_num_sequences or len(self.running) >= cfg.max_num_sequences:
                    break
                n = self._chunk(r, cfg.max_num_batched_tokens - used_tokens())
                if n <= 0:
                    break
                if self.cache.num_free_slots() == 0 or not self.cache.can_reserve(-1, n):
                    break  # later: the head of the queue blocks those behind it
                self.waiting.popleft()
                self.cache.add(r.uid)
                self.cache.reserve(r.uid, n)
                r.status = Status.RUNNING
                if r.metrics.first_scheduled_time is None:
                    r.metrics.first_scheduled_time = now
                self.running.append(r)
                out.entries.append(ScheduledEntry(r, n, 0, n == r.length))
                self._prev_prompt = True
        return out
