"""The scheduler's policy written out plainly, to compare the native scheduler's decisions with.

It shares nothing with the product: requests are ``PlainRequest`` objects, statuses are strings, and pages are
counted by ``PlainPages`` (one group of pages, with or without a window of keys).  The policy is the reference's chunked one
(backends/vllm/src/scheduler.rs:1257-1379 with the budget of :40-149, admissions :897-1016, recompute-preemption
:650-690 and :1778-1896, the optional delay :2077-2097, first come first served policy.rs:56-61):

1. running requests that decode (one token each), in order of arrival;
2. running requests still in their prompt: the next portion, as large as the remaining budget allows;
3. waiting requests in order, while budget, pages and slots last; the head of the queue blocks those behind it.

When pages run out for a running request, the running request that arrived last (and is not frozen) is preempted:
its pages go back, it returns to the front of the waiting queue with nothing computed.  A request that runs alone
tries portions half as long, and is capped when not even one token finds a page.  A waiting request longer than
the model length or the pool is ignored.  With a window of keys portions are shortened before anything is
preempted, a first portion that finds the pool idle is shortened until it fits, and a newcomer must leave room for
the window (and one page) of everyone already there.
"""
from collections import deque


class PlainRequest:
    def __init__(self, uid, prompt_len, arrival, max_new):
        self.uid, self.prompt_len, self.arrival, self.max_new = uid, prompt_len, arrival, max_new
        self.outputs = 0          # tokens the host has read
        self.pending = 0          # tokens sampled that the host has not read yet
        self.num_computed = 0
        self.frozen = False
        self.status = "waiting"
        self.num_preemptions = 0

    @property
    def length(self):
        return self.prompt_len + self.outputs + self.pending

    @property
    def num_sampled(self):
        return self.outputs + self.pending

    @property
    def num_uncomputed(self):
        return self.length - self.num_computed

    @property
    def in_prefill(self):
        return self.num_uncomputed > 1 or self.num_sampled == 0


class PlainPages:
    """How many pages each request holds; pages are not told apart.  With ``window`` W a request needs the pages
    that hold its last W tokens only: ``release_behind`` gives back those wholly below ``computed - W + 1``."""

    def __init__(self, page_size, num_pages, slots, window=0):
        self.page_size, self.num_pages, self.slots, self.window = page_size, num_pages, slots, window
        self.held = {}          # uid -> pages ever taken (the length of its table)
        self.released = {}      # uid -> how many of them went back behind the window

    def _pages(self, length):
        return -(-length // self.page_size)

    def _live(self, uid):
        return self.held[uid] - self.released[uid]

    def free_pages(self):
        return self.num_pages - sum(self._live(u) for u in self.held)

    def has(self, uid):
        return uid in self.held

    def num_free_slots(self):
        return self.slots - len(self.held)

    def idle(self):
        return not self.held

    def fits_at_all(self, length):
        need = self._pages(length)
        if self.window:
            need = min(need, self._pages(self.window) + 1)
        return need <= self.num_pages

    def can_reserve(self, uid, length):
        if uid not in self.held and self.num_free_slots() == 0:
            return False
        return max(0, self._pages(length) - self.held.get(uid, 0)) <= self.free_pages()

    def can_admit(self, total, first):
        """A newcomer's first portion, and with a window also what it and everyone already there will need once
        they have moved on: the window and one page each."""
        if self.num_free_slots() == 0:
            return False
        need = self._pages(first)
        if self.window:
            steady = self._pages(self.window) + 1
            need = max(need, min(self._pages(total), steady))
            need += sum(max(0, steady - self._live(u)) for u in self.held)
        return need <= self.free_pages()

    def add(self, uid):
        assert uid not in self.held and self.num_free_slots() > 0
        self.held[uid] = 0
        self.released[uid] = 0

    def reserve(self, uid, length):
        assert self.can_reserve(uid, length)
        self.held[uid] = max(self.held[uid], self._pages(length))

    def release_behind(self, uid, computed):
        if self.window and computed - self.window + 1 > 0:
            dead = min((computed - self.window + 1) // self.page_size, self.held[uid])
            self.released[uid] = max(self.released[uid], dead)

    def free(self, uid):
        del self.held[uid]
        del self.released[uid]


class PlainOutput:
    def __init__(self):
        self.entries, self.preempted, self.ignored, self.capped = [], [], [], []   # entries: (request, n, start, sample)


class PlainScheduler:
    """``limits``: max_tokens, max_requests, max_model_len, cut (prompts may be cut), max_portion (0: none) and
    delay_factor, as attributes of any object."""

    def __init__(self, limits, pages):
        self.limits, self.pages = limits, pages
        self.waiting, self.running = deque(), []
        self.num_preemptions = 0
        self.last_prompt_latency, self._prev_prompt, self._prev_time = 0.0, False, 0.0

    def add(self, r):
        r.status = "waiting"
        self.waiting.append(r)

    def take_out(self, r, status):
        """Aborted, or the request has its last token: wherever it is, it leaves and gives back what it holds."""
        if r.status == "running":
            self.running.remove(r)
        else:
            self.waiting.remove(r)
        self._release(r)
        r.status = status

    def _release(self, r):
        if self.pages.has(r.uid):
            self.pages.free(r.uid)

    def _aligned(self, r, n):
        """A portion that does not end the request's tokens ends at a multiple of ``limits.align``; 0 if none fits."""
        a = getattr(self.limits, "align", 1)
        if a <= 1 or n >= r.num_uncomputed:
            return n
        end = (r.num_computed + n) // a * a
        return max(end - r.num_computed, 0)

    def _portion(self, r, budget):
        n = min(r.num_uncomputed, budget)
        if self.limits.max_portion > 0 and r.num_uncomputed > 1:
            n = min(n, self.limits.max_portion)
        if not self.limits.cut and n < r.num_uncomputed:
            return 0
        return self._aligned(r, n)

    def _preempt(self, victim, out):
        self.running.remove(victim)
        self._release(victim)
        victim.num_computed = 0
        victim.status = "waiting"
        victim.num_preemptions += 1
        self.waiting.appendleft(victim)
        self.num_preemptions += 1
        out.preempted.append(victim)
        out.entries[:] = [e for e in out.entries if e[0] is not victim]

    def _passed_delay(self, now):
        if self._prev_prompt:
            self.last_prompt_latency = now - self._prev_time
        self._prev_time, self._prev_prompt = now, False
        if self.limits.delay_factor > 0 and self.waiting:
            earliest = min(r.arrival for r in self.waiting)
            return (now - earliest) > self.limits.delay_factor * self.last_prompt_latency or not self.running
        return True

    def schedule(self, now):
        out, lim = PlainOutput(), self.limits
        self.running.sort(key=lambda r: r.arrival)

        def used():
            return sum(e[1] for e in out.entries)

        live = [r for r in self.running if not r.frozen]
        for r in [r for r in live if not r.in_prefill] + [r for r in live if r.in_prefill]:
            if r.status != "running":
                continue      # preempted for an earlier request of this step
            if len(out.entries) >= lim.max_requests:
                break
            n = whole = self._portion(r, lim.max_tokens - used())
            if n <= 0:
                continue
            while not self.pages.can_reserve(r.uid, r.num_computed + n):
                victim = next((v for v in reversed(self.running) if not v.frozen), r)
                alone = victim is r and len(self.running) == 1
                shorter = self._aligned(r, n // 2) if n > 1 else 0
                if shorter > 0 and lim.cut and (alone or self.pages.window):
                    n = shorter       # a shorter portion may still find its pages
                    continue
                if alone:
                    self.running.remove(r)
                    self._release(r)
                    r.status = "capped"
                    out.capped.append(r)
                    break
                self._preempt(victim, out)
                if victim is r:
                    break
                n = whole
            if r.status != "running":
                continue
            self.pages.reserve(r.uid, r.num_computed + n)
            out.entries.append((r, n, r.num_computed, r.num_computed + n == r.length))

        if not out.preempted and self._passed_delay(now):
            while self.waiting:
                r = self.waiting[0]
                if r.length > lim.max_model_len or not self.pages.fits_at_all(r.length):
                    self.waiting.popleft()
                    r.status = "ignored"
                    out.ignored.append(r)
                    continue
                if len(out.entries) >= lim.max_requests or len(self.running) >= lim.max_requests:
                    break
                n = self._portion(r, lim.max_tokens - used())
                if n <= 0 or self.pages.num_free_slots() == 0:
                    break
                idle = self.pages.idle()
                while n > 1 and lim.cut and idle and not self.pages.can_admit(r.length, n):
                    n = self._aligned(r, n // 2)       # nothing holds pages: only a shorter first portion helps
                if n <= 0 or not self.pages.can_admit(r.length, n):
                    if not idle:
                        break
                    self.waiting.popleft()
                    r.status = "ignored"
                    out.ignored.append(r)
                    continue
                self.waiting.popleft()
                self.pages.add(r.uid)
                self.pages.reserve(r.uid, n)
                r.status = "running"
                self.running.append(r)
                out.entries.append((r, n, 0, n == r.length))
                self._prev_prompt = True
        return out
