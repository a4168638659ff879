"""The step function: run one batch of (request, its next tokens) from the cache and return logits.

A step's entries may be portions of prompts beside single decoded tokens, in any order and cut anywhere.  The
step runs only the tokens it is given, as one batch; keys and values of those tokens are written to the cache
first, then every token at position p attends keys 0..p of its own request through the block table.  Logits
come back only for the places asked for, in float32.

The reference's counterpart is ``ModelWorker::execute_model`` with ``prepare_input_tensors``
(backends/vllm/src/worker.rs:111-191, 224-460); unlike it, a later portion of a prompt sees the earlier ones.
All integer metadata of a step (including what mixers plan for their kernels, such as attention task lists)
travels to the device in one pinned buffer and one copy.

Steps that only decode (one token per entry, its logits wanted) are launch-bound, so their kernel sequence is
captured once per (number of entries, context bucket of 256 tokens) into a HIP graph and replayed; between
replays only the metadata buffer changes.  A shape is run eagerly the first time it is seen and captured the
second time.
"""
from __future__ import annotations

import dataclasses
import itertools
from collections import OrderedDict
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.pool import CachePool, LayerCache

DECODE_BUCKET = 256      # tokens; a decode graph serves contexts up to a multiple of this
MAX_GRAPHS = 48
MAX_SEEN = 1024          # shapes of steps whose sightings are counted before they are recorded
# A step that is one prompt, or one portion of a prompt, of at least this many tokens is recorded as a graph too, the
# third time its (first position, length) is seen: its 150 launches then cost the GPU about 0.2 ms less
PROMPT_GRAPH_MIN_TOKENS = 256
PROMPT_GRAPH_SIGHTINGS = 3


class StepError(ValueError):
    pass


@dataclasses.dataclass
class StepEntry:
    """The next tokens of one request.

    ``start`` is the position of ``tokens[0]``: the number of tokens of this request already in the cache.
    ``want`` lists the indices into ``tokens`` whose logits are asked for.
    """
    request: int
    tokens: Sequence[int]
    start: int
    want: Sequence[int] = ()
    #: for an entry of one token that the host does not know yet: the row of the previous step's sampled tokens
    #: (a device tensor given to ``step``) to take it from; ``tokens`` then holds any valid id as a stand-in
    feed: int = -1


@dataclasses.dataclass
class StepContext:
    """Device-side description of one step, as the parts see it."""
    n_tokens: int
    n_entries: int
    n_want: int
    tokens: torch.Tensor            # [T] int32
    positions: torch.Tensor         # [T] int32 absolute positions
    token_seq: torch.Tensor         # [T] int32: the entry (row of the block tables) of each token
    q_start: torch.Tensor           # [S+1] int32: first token of each entry
    seq_lens: torch.Tensor          # [S] int32: tokens of each request after this step
    state_slots: torch.Tensor       # [S] int32
    want_rows: Optional[torch.Tensor]   # [n_want] int32 rows of the step
    # host copies, for launch decisions
    h_starts: np.ndarray            # [S] position of each entry's first token
    h_counts: np.ndarray            # [S] tokens of each entry
    h_state_slots: np.ndarray
    max_count: int
    max_seq_len: int
    slot_mappings: List[torch.Tensor] = dataclasses.field(default_factory=list)   # per group [T]
    block_tables: List[torch.Tensor] = dataclasses.field(default_factory=list)    # per group [S, blocks]
    pool: Optional[CachePool] = None
    #: what mixers planned for this step: key -> (int32 device tensor, meta)
    plans: Dict[object, Tuple[torch.Tensor, tuple]] = dataclasses.field(default_factory=dict)
    #: per-step notes and workspaces of kernels
    scratch: Dict[object, object] = dataclasses.field(default_factory=dict)
    #: not None inside a decode graph: the number of 256-token buckets the graph serves
    decode_bucket: Optional[int] = None
    #: the logits of every token are wanted, in the order of the tokens (``want_rows`` counts 0, 1, 2, ...)
    wants_all_rows: bool = False

    def layer_cache(self, pos: int) -> LayerCache:
        return self.pool.layer_cache(pos, self.slot_mappings, self.block_tables)


class _Staging:
    """Two pinned host buffers, taken in turn, and their one device twin, grown on demand.

    A buffer may be written again when the copy out of it has been read, which an event behind that copy says.  The
    event is the staging's own, or (``upload(record=False)``) one that the caller records later on the same stream
    and names with ``mark``: with two buffers a caller that waits for a step's results before it builds the step
    after the next never waits here, and a step needs no event beside the one its results have anyway.
    """

    def __init__(self, device: torch.device):
        self.device = device
        self.hosts: List[Optional[torch.Tensor]] = [None, None]
        self.events: List[Optional[torch.cuda.Event]] = [None, None]
        self.unmarked = [False, False]        # a copy out of the buffer is on its way and no event marks its end
        self.turn = 0
        self.dev: Optional[torch.Tensor] = None

    def _wait(self, i: int) -> None:
        if self.events[i] is not None:
            self.events[i].synchronize()
            self.events[i] = None
        elif self.unmarked[i]:
            torch.cuda.current_stream(self.device).synchronize()
        self.unmarked[i] = False

    def begin(self, n: int) -> np.ndarray:
        """The next host buffer, at least ``n`` words long and free to be written."""
        self.turn ^= 1
        i = self.turn
        self._wait(i)
        if self.hosts[i] is None or self.hosts[i].numel() < n:
            self.hosts[i] = torch.empty(max(1024, 1 << (n - 1).bit_length()), dtype=torch.int32, pin_memory=True)
        if self.dev is None or self.dev.numel() < n:
            self.dev = torch.empty(max(1024, 1 << (n - 1).bit_length()), dtype=torch.int32, device=self.device)
        return self.hosts[i].numpy()

    def wait(self) -> None:
        """Wait until every copy out of the host buffers has been read."""
        self._wait(0)
        self._wait(1)

    def upload(self, n: int, record: bool = True) -> None:
        """Copy the first ``n`` words of the buffer that ``begin`` gave to the device.  ``record``: mark the copy's end
        with an event of its own; else the caller names one with ``mark`` (an event is a packet of its own in the
        GPU's queue, 4 us on the path of every step, and a step that samples records one anyway)."""
        i = self.turn
        self.dev[:n].copy_(self.hosts[i][:n], non_blocking=True)
        self.events[i], self.unmarked[i] = None, not record
        if record:
            self.events[i] = torch.cuda.Event()
            self.events[i].record()

    def mark(self, event: torch.cuda.Event) -> None:
        """``event`` was recorded on the copies' stream behind the last ``upload(record=False)``."""
        if self.unmarked[self.turn]:
            self.events[self.turn] = event


@dataclasses.dataclass
class _Graph:
    stage: _Staging
    graph: Optional[torch.cuda.CUDAGraph] = None
    logits: Optional[torch.Tensor] = None
    ctx: Optional[StepContext] = None


class RunnerCache:
    """The cache manager as the scheduler sees it, with the runner's own books kept in step.

    Everything is forwarded to the ``CacheManager``; ``adopted`` and ``forgot`` are what the scheduler calls after
    it has registered a request with the manager, or released one from it, by itself.
    """

    def __init__(self, runner: "ModelRunner"):
        self._runner, self._mgr = runner, runner.manager

    def adopted(self, request: int) -> None:
        self._runner.adopt_request(request)

    def forgot(self, request: int) -> None:
        self._runner.forget_request(request)

    def __getattr__(self, name):
        return getattr(self._mgr, name)


class ModelRunner:
    """Owns the model and the cache pool of one GPU and steps batches through them."""

    def __init__(self, model, pool: CachePool, use_graphs: bool = True):
        self.model, self.pool = model, pool
        self.manager = pool.manager
        # decode steps are recorded into graphs only if every part of the model can be replayed
        self.use_graphs = use_graphs and model.spec.graph_safe()
        self._stage = _Staging(model.device)
        self._last_stage: Optional[_Staging] = None
        self._prompt_pool = None
        #: True: the caller records an event behind every step's work and hands it to ``fence``; the steps then record
        #: none of their own (a step whose event never comes waits for the whole stream before its buffer is reused)
        self.external_fence = False
        self._computed: Dict[int, int] = {}       # request -> tokens in the cache
        self._graphs: "OrderedDict[Tuple[int, int], _Graph]" = OrderedDict()
        self._seen: "OrderedDict[tuple, int]" = OrderedDict()
        # planners of the mixers, one per distinct key
        self._planners: Dict[object, Callable] = {}
        for _, block in model.spec.layers:
            plan = getattr(block.mixer, "step_planner", None)
            got = plan(pool.page_size, pool.dtype) if plan is not None else None
            if got is not None:
                self._planners.setdefault(got[0], got[1])

    # -- requests ------------------------------------------------------------------------------------
    def add_request(self, request: int) -> int:
        slot = self.manager.add(request)
        self.adopt_request(request)
        return slot

    def adopt_request(self, request: int) -> None:
        """Open the books for a request that the manager already knows: nothing computed, state cleared."""
        slot = self.manager.state_slot(request)
        self._computed[request] = 0
        for st in self.pool.states.values():
            st[slot].zero_()

    def has_request(self, request: int) -> bool:
        return request in self._computed

    def computed_len(self, request: int) -> int:
        return self._computed[request]

    def free_request(self, request: int) -> None:
        self.manager.free(request)
        self.forget_request(request)

    def forget_request(self, request: int) -> None:
        """Close the books of a request that the manager has already released."""
        del self._computed[request]

    def reset_request(self, request: int) -> None:
        """Drop what a request holds but keep it registered (recompute-preemption)."""
        self.free_request(request)
        self.add_request(request)

    # -- the step ------------------------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        vocab, max_pos = self.model.vocab_size, self.model.spec.max_positions
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request} appears twice in one step")
            seen.add(e.request)
            if e.request not in self._computed:
                raise StepError(f"request {e.request} is not registered")
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.request}: an entry needs at least one token")
            if e.start != self._computed[e.request]:
                raise StepError(f"request {e.request}: tokens start at position {e.start}, but the cache holds "
                                f"{self._computed[e.request]} tokens")
            if e.start + n > max_pos:
                raise StepError(f"request {e.request}: position {e.start + n - 1} exceeds max_position_embeddings "
                                f"{max_pos}")
            lo, hi = min(e.tokens), max(e.tokens)
            if lo < 0 or hi >= vocab:
                raise StepError(f"request {e.request}: token id {lo if lo < 0 else hi} outside the vocabulary "
                                f"of {vocab}")
            for w in e.want:
                if not 0 <= w < n:
                    raise StepError(f"request {e.request}: wanted place {w} outside its {n} tokens")
            if e.feed >= 0 and n != 1:
                raise StepError(f"request {e.request}: only an entry of one token can be fed from the device")

    @staticmethod
    def _arrays(entries: Sequence[StepEntry]) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
        """(request ids, first positions, token counts) of the entries."""
        s = len(entries)
        return (np.fromiter((e.request for e in entries), dtype=np.int64, count=s),
                np.fromiter((e.start for e in entries), dtype=np.int32, count=s),
                np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=s))

    def _build(self, entries: Sequence[StepEntry], stage: _Staging, bucket: Optional[int],
               feed_src: Optional[torch.Tensor] = None, arrays=None) -> StepContext:
        """Fill ``stage`` with the step's metadata, start its copy to the device and describe it.

        With ``bucket`` (decode graphs) every size is a function of (entries, bucket) alone, so the layout, and
        with it every device address a captured kernel reads, is the same at every replay.
        """
        mgr = self.manager
        s = len(entries)
        ids, starts, counts = arrays if arrays is not None else self._arrays(entries)
        t = int(counts.sum())
        n_want = sum(len(e.want) for e in entries)
        n_groups = len(self.pool.plan.groups)
        max_seq = int((starts + counts).max())
        page = self.pool.page_size
        max_blocks = -(-max_seq // page) if bucket is None else -(-bucket * DECODE_BUCKET // page)
        # a step that only decodes is planned the same way whether it is captured or run eagerly
        plan_bucket = bucket
        if plan_bucket is None and int(counts.max()) == 1:
            plan_bucket = -(-max_seq // DECODE_BUCKET)
        # (planners are told the context length that the bucket serves, in tokens)
        bucket_tokens = None if plan_bucket is None else plan_bucket * DECODE_BUCKET
        extras = [(key, *fn(starts, counts, bucket_tokens)) for key, fn in self._planners.items()]
        # layout of the one staging buffer
        o_tok, o_pos, o_seq = 0, t, 2 * t
        o_qs, o_len, o_slot = 3 * t, 3 * t + s + 1, 3 * t + 2 * s + 1
        o_want = 3 * t + 3 * s + 1
        o_sm = o_want + n_want
        o_bt = o_sm + n_groups * t
        o_feed = o_bt + n_groups * s * max_blocks          # pairs (token row, row of the fed tokens), 2 per entry
        total = o_feed + 2 * s
        ex_off = []
        for _, arr, _ in extras:
            total += (-total) % 4                  # every extra starts on a 16-byte boundary
            ex_off.append(total)
            total += arr.size
        buf = stage.begin(total)
        # the arrays that depend on the entries alone are written by the host library in one call
        if t == s:
            tokens = np.fromiter((e.tokens[0] for e in entries), dtype=np.int32, count=s)
        else:
            tokens = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries), dtype=np.int32, count=t)
        feeds = np.fromiter((e.feed for e in entries), dtype=np.int32, count=s)
        want_counts = np.fromiter((len(e.want) for e in entries), dtype=np.int32, count=s)
        wants = np.fromiter(itertools.chain.from_iterable(e.want for e in entries), dtype=np.int32, count=n_want)
        offsets = np.asarray((o_tok, o_pos, o_seq, o_qs, o_len, o_slot, o_want, o_sm, o_bt, o_feed), dtype=np.int64)
        n_feed = mgr.pack_step(ids, starts, counts, tokens, feeds, want_counts, wants, buf, offsets, max_blocks)
        slots = buf[o_slot: o_slot + s].copy()
        for off, (_, arr, _) in zip(ex_off, extras):
            buf[off: off + arr.size] = arr.reshape(-1)
        stage.upload(total, record=not self.external_fence)
        self._last_stage = stage
        dev = stage.dev
        if n_feed:
            from ..kernels import ops
            ops.feed_tokens(dev[o_tok: o_tok + t], feed_src, dev[o_feed: o_feed + 2 * n_feed].view(n_feed, 2))
        ctx = StepContext(
            n_tokens=t, n_entries=s, n_want=n_want,
            tokens=dev[o_tok: o_tok + t], positions=dev[o_pos: o_pos + t], token_seq=dev[o_seq: o_seq + t],
            q_start=dev[o_qs: o_qs + s + 1], seq_lens=dev[o_len: o_len + s], state_slots=dev[o_slot: o_slot + s],
            want_rows=dev[o_want: o_want + n_want] if n_want else None,
            h_starts=starts, h_counts=counts, h_state_slots=slots, max_count=int(counts.max()), max_seq_len=max_seq,
            slot_mappings=[dev[o_sm + g * t: o_sm + (g + 1) * t] for g in range(n_groups)],
            block_tables=[dev[o_bt + g * s * max_blocks: o_bt + (g + 1) * s * max_blocks].view(s, max_blocks)
                          for g in range(n_groups)],
            pool=self.pool, decode_bucket=bucket,
            # (one token an entry: every entry must want its one place, once; two wanting [0, 0] and [] do not)
            wants_all_rows=n_want == t and (bool((want_counts == 1).all()) if t == s else
                                            all(len(e.want) == len(e.tokens) and
                                                          all(w == j for j, w in enumerate(e.want))
                                                          for e in entries)))
        for off, (key, arr, meta) in zip(ex_off, extras):
            ctx.plans[key] = (dev[off: off + arr.size].view(arr.shape), meta)
        return ctx

    def prepare(self, entries: Sequence[StepEntry]) -> StepContext:
        """Check the entries, reserve their pages and build the step's metadata on the device."""
        self._validate(entries)
        arrays = self._arrays(entries)
        self.manager.reserve_all(*arrays)
        return self._build(entries, self._stage, None, arrays=arrays)

    def _finish(self, entries: Sequence[StepEntry], arrays) -> None:
        ids, starts, counts = arrays
        done = starts + counts
        for e, d in zip(entries, done.tolist()):
            self._computed[e.request] = d
        self.manager.release_behind_all(ids, done)

    def step(self, entries: Sequence[StepEntry], feed_src: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run one batch; returns float32 logits [wanted places, vocab] (order: entries, then ``want``) or None.

        ``feed_src`` (int32 device tensor) supplies the token of every entry with ``feed >= 0``.

        The tensor returned by a step that ran as a graph (decode steps, lone prompts) belongs to that graph and is
        overwritten by a later step: use it (sample, copy) before stepping again.
        """
        self._validate(entries)
        arrays = self._arrays(entries)
        self.manager.reserve_all(*arrays)
        ran, logits = False, None
        if self.use_graphs:
            if int(arrays[2].max()) == 1 and all(len(e.want) == 1 for e in entries):
                max_seq = int(arrays[1].max()) + 1
                bucket = -(-max_seq // DECODE_BUCKET)
                ran, logits = self._with_graph((len(entries), bucket), bucket, 2, entries, feed_src, arrays)
            elif (len(entries) == 1 and int(arrays[2][0]) >= PROMPT_GRAPH_MIN_TOKENS and entries[0].feed < 0
                  and list(entries[0].want) in ([], [int(arrays[2][0]) - 1])):
                # a prompt, or a portion of one, alone in its step: every launch of the step is a function of where
                # the portion begins and how long it is
                key = ("prompt", int(arrays[1][0]), int(arrays[2][0]), len(entries[0].want))
                ran, logits = self._with_graph(key, None, PROMPT_GRAPH_SIGHTINGS, entries, feed_src, arrays)
        if not ran:
            ctx = self._build(entries, self._stage, None, feed_src, arrays)
            logits = self.model.forward(ctx)
        self._finish(entries, arrays)
        return logits

    def _with_graph(self, key, bucket: Optional[int], sightings: int, entries: Sequence[StepEntry], feed_src, arrays):
        """(True, logits) if the step ran as the graph of its ``key``: recorded at the ``sightings``-th step with that
        key (the earlier ones run eagerly, which also loads every kernel the step needs), replayed from then on."""
        g = self._graphs.get(key)
        if g is None:
            # (shapes that have not been seen often enough are counted apart: they must not push recorded graphs out)
            seen = self._seen.pop(key, 0) + 1
            if seen < sightings:
                self._seen[key] = seen
                while len(self._seen) > MAX_SEEN:
                    self._seen.popitem(last=False)
                return False, None
            g = self._graphs[key] = _Graph(_Staging(self.model.device))
            while len(self._graphs) > MAX_GRAPHS:
                self._graphs.popitem(last=False)
        self._graphs.move_to_end(key)
        ctx = self._build(entries, g.stage, bucket, feed_src, arrays)
        if g.graph is None:
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            # the graphs of prompt steps hold a prompt's activations: they share one pool (no two run at a time, and a
            # step's logits are the caller's only until the next step)
            pool = None
            if bucket is None:
                if self._prompt_pool is None:
                    self._prompt_pool = torch.cuda.graph_pool_handle()
                pool = self._prompt_pool
            with torch.cuda.graph(graph, pool=pool):
                out = self.model.forward(ctx)
            g.graph, g.logits, g.ctx = graph, out, ctx
        g.graph.replay()
        return True, g.logits

    def fence(self, event: torch.cuda.Event) -> None:
        """With ``external_fence``: ``event`` was recorded on the step's stream behind the last step's work."""
        if self._last_stage is not None:
            self._last_stage.mark(event)

    def wait_staging(self):
        self._stage.wait()
