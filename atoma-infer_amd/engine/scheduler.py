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
(scheduler.rs:650-690, 1778-1896).  If the request that cannot grow is the only one running, it takes portions half
as long (with a window of keys, pages come back as it moves on); when not even one token finds a page it is
finished as "length_capped": nothing could be given back for it.

The decisions are made in the host library (csrc/host/scheduler.cpp), next to the cache manager it draws pages
from; this module keeps the ``Request`` objects, reports their counters before each plan and applies the plan's
outcome to them.

Differences from the reference, on purpose: portions of a prompt stay in the running queue until the prompt is
done (the reference drops them, scheduler.rs:1313-1338), pages are given back when a request finishes (the
reference frees only on abort and preemption), and there is no swap space.
"""
from __future__ import annotations

import ctypes
import dataclasses
import time
from typing import Dict, List, Optional

import numpy as np

from ..cache.manager import CacheManager
from ..config.engine import SchedulerConfig
from ..kernels.library import load_host_library
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


class SchedulerError(RuntimeError):
    pass


_PREEMPTED, _IGNORED, _CAPPED, _ADMITTED, _WAITING, _RUNNING = range(6)
_lib = None


def _native():
    global _lib
    if _lib is None:
        lib = load_host_library()
        p, i, i64, f64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_double
        lib.sc_create.restype = p
        lib.sc_create.argtypes = [p, i, i, i, i, i, f64, i]
        lib.sc_destroy.restype = None
        lib.sc_destroy.argtypes = [p]
        lib.sc_add.argtypes = [p, i64, f64, ctypes.c_int32]
        lib.sc_remove.argtypes = [p, i64]
        lib.sc_sync.argtypes = [p, i, p]
        lib.sc_schedule.argtypes = [p, f64]
        lib.sc_entries.argtypes = [p, p, i]
        lib.sc_list.argtypes = [p, i, p, i]
        for name in ("sc_num_waiting", "sc_num_running", "sc_num_preemptions", "sc_last_prompt_latency"):
            getattr(lib, name).argtypes = [p]
        lib.sc_num_preemptions.restype = i64
        lib.sc_last_prompt_latency.restype = f64
        _lib = lib
    return _lib


class Scheduler:
    """``cache`` is a ``CacheManager`` or anything that forwards to one (``handle`` is what the native scheduler
    draws pages from).  If it has ``adopted(request)`` and ``forgot(request)``, they are called for every request
    that a plan registered with the manager or released from it, so that books kept beside the manager follow."""

    def __init__(self, config: SchedulerConfig, cache: CacheManager, clock=time.monotonic, chunk_alignment: int = 1):
        """``chunk_alignment``: a portion that does not end a request's tokens ends at a multiple of it (what the
        model asks for, ``ModelSpec.chunk_alignment``)."""
        config.validate()
        self.config, self.cache, self.clock = config, cache, clock
        self._lib = _native()
        self._h = self._lib.sc_create(cache.handle, config.max_num_batched_tokens, config.max_num_sequences,
                                      config.max_model_len, int(config.enable_chunked_prefill),
                                      config.max_prefill_chunk, float(config.delay_factor), int(chunk_alignment))
        if not self._h:
            raise SchedulerError(f"the native scheduler refused {config} with portions aligned to {chunk_alignment} "
                                 f"(a cut prompt needs max_num_batched_tokens >= alignment + max_num_sequences - 1, so "
                                 f"that an aligned portion fits beside the decoding requests, and max_prefill_chunk, "
                                 f"if set, >= alignment)")
        self._requests: Dict[int, Request] = {}
        self._running: Dict[int, Request] = {}
        self._adopted = getattr(cache, "adopted", None)
        self._forgot = getattr(cache, "forgot", None)
        self._ids = np.zeros(max(64, 4 * config.max_num_sequences), dtype=np.int64)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.sc_destroy(h)

    # -- queue operations --------------------------------------------------------------------------------
    def add(self, request: Request) -> None:
        if self._lib.sc_add(self._h, request.uid, float(request.metrics.arrival_time), request.length) != 0:
            raise SchedulerError(f"request number {request.uid} is already queued")
        request.status = Status.WAITING
        self._requests[request.uid] = request

    def has_unfinished(self) -> bool:
        return bool(self._requests)

    def num_unfinished(self) -> int:
        return len(self._requests)

    def _take_out(self, r: Request, status: Status) -> None:
        held = self._lib.sc_remove(self._h, r.uid)
        if held < 0:
            raise SchedulerError(f"request {r.request_id} is not queued")
        del self._requests[r.uid]
        self._running.pop(r.uid, None)
        if held and self._forgot is not None:
            self._forgot(r.uid)
        r.status = status

    def abort(self, request_id: str) -> Optional[Request]:
        """Remove a request wherever it is; its pages go back (scheduler.rs:390-443)."""
        for r in self._requests.values():
            if r.request_id == request_id:
                self._take_out(r, Status.FINISHED_ABORTED)
                return r
        return None

    def finish(self, request: Request, status: Status) -> None:
        """A request has produced its last token: give back what it holds.  It is usually running; it waits if it
        was preempted while that token was still on its way."""
        assert status.finished
        self._take_out(request, status)

    # -- inspection --------------------------------------------------------------------------------------
    def _list(self, kind: int) -> List[Request]:
        n = self._lib.sc_list(self._h, kind, self._ids.ctypes.data, self._ids.size)
        if n > self._ids.size:
            self._ids = np.zeros(2 * n, dtype=np.int64)
            n = self._lib.sc_list(self._h, kind, self._ids.ctypes.data, self._ids.size)
        return [self._requests[u] for u in self._ids[:n].tolist()]

    @property
    def waiting(self) -> List[Request]:
        """The waiting queue from its head."""
        return self._list(_WAITING)

    @property
    def running(self) -> List[Request]:
        return self._list(_RUNNING)

    @property
    def num_preemptions(self) -> int:
        return self._lib.sc_num_preemptions(self._h)

    @property
    def last_prompt_latency(self) -> float:
        return self._lib.sc_last_prompt_latency(self._h)

    # -- one step's plan -----------------------------------------------------------------------------------
    def schedule(self) -> ScheduleOutput:
        now = self.clock()
        lib, h = self._lib, self._h
        if self._running:
            rows = np.array([x for r in self._running.values()
                             for x in (r.uid, r.length, r.num_computed, r.num_sampled, r.frozen)], dtype=np.int64)
            if lib.sc_sync(h, len(self._running), rows.ctypes.data) != 0:
                raise SchedulerError("a running request is unknown to the native scheduler")
        n = lib.sc_schedule(h, float(now))
        if n < 0:
            raise SchedulerError("the cache manager refused pages it had just promised")
        out = ScheduleOutput([], [], [], [])
        # releases first: a request's number leaves the books beside the manager before anything else happens
        for r in self._list(_PREEMPTED):
            del self._running[r.uid]
            r.num_computed = 0
            r.status = Status.WAITING
            r.metrics.num_preemptions += 1
            out.preempted.append(r)
            if self._forgot is not None:
                self._forgot(r.uid)
        for r in self._list(_CAPPED):
            del self._running[r.uid]
            del self._requests[r.uid]
            r.status = Status.FINISHED_LENGTH_CAPPED
            out.capped.append(r)
            if self._forgot is not None:
                self._forgot(r.uid)
        for r in self._list(_IGNORED):
            del self._requests[r.uid]
            r.status = Status.FINISHED_IGNORED
            out.ignored.append(r)
        for r in self._list(_ADMITTED):
            self._running[r.uid] = r
            r.status = Status.RUNNING
            if r.metrics.first_scheduled_time is None:
                r.metrics.first_scheduled_time = now
            if self._adopted is not None:
                self._adopted(r.uid)
        if n:
            rows = np.empty((n, 4), dtype=np.int64)
            lib.sc_entries(h, rows.ctypes.data, n)
            reqs = self._requests
            out.entries = [ScheduledEntry(reqs[u], k, s, bool(d)) for u, k, s, d in rows.tolist()]
        return out
