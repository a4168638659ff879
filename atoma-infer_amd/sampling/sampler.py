"""The sampler: from float32 logits on the device to one token per row.

Greedy rows take the argmax (lowest index on ties).  Sampled rows draw from softmax(logits / T), cut by top-k
and/or top-p, with the inverse-CDF method from one uniform number per (request seed, step): a counter-based
generator, so a request's tokens do not depend on which other requests share its batches, and portions of
prompts that sample nothing consume nothing (the reference advances each request's generator even for discarded
samples: backends/vllm/src/model_executor.rs:231-235, llm_engine.rs:379).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingPlan

_MASK = (1 << 64) - 1
# vocabularies from which on the rows of a step that draws are cut into parts (a block walks fewer values quickly enough)
SPLIT_MIN_VOCAB = 32768


def uniform(seed: int, counter: int) -> float:
    """A number in [0, 1) with 24 random bits, a pure function of (seed, counter) (splitmix64 finaliser)."""
    z = (seed * 0x9E3779B97F4A7C15 + (counter + 1) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


class Pending:
    """A sampling launched on the device whose tokens the host has not read yet."""

    def __init__(self, tokens: torch.Tensor, logits: torch.Tensor, host: torch.Tensor, event: torch.cuda.Event,
                 pool: Optional[list] = None):
        self.tokens, self.logits, self._host, self.event, self._pool = tokens, logits, host, event, pool
        self._meta, self._meta_pool = None, None

    def result(self) -> Tuple[List[int], List[float]]:
        """Wait for the copy and return (tokens, logits of the chosen tokens)."""
        self.event.synchronize()
        n = self.tokens.numel()
        got = self._host[0, :n].view(torch.int32).tolist(), self._host[1, :n].tolist()
        if self._pool is not None:            # the pinned buffer serves a later step
            self._pool.append(self._host)
            self._pool = None
        if self._meta_pool is not None:       # (so does the one that brought the parameters: its copy is over too)
            self._meta_pool.append(self._meta)
            self._meta_pool = None
        return got


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device
        self._greedy_meta = {}        # rows -> the device copy of the parameters of that many greedy rows
        # rows -> pinned buffers [2, rows] that have been read (a pinned tensor made and dropped every step costs an
        # event in the GPU's queue when torch takes it back: 4 us a step)
        self._host_pool = {}
        self._meta_pool = {}          # rows -> pinned buffers [5, rows] for the rows' parameters, likewise

    def _host_buffer(self, s: int):
        pool = self._host_pool.setdefault(s, [])
        host = pool.pop() if pool else torch.empty((2, s), dtype=torch.float32, pin_memory=True)
        return host, pool

    def launch(self, logits: torch.Tensor, plans: Sequence[SamplingPlan], steps: Sequence[int],
               contexts: Sequence[Sequence[int]]) -> Pending:
        """Start sampling one token per row of ``logits`` [S, V]; nothing waits for the GPU.

        ``steps[i]`` is how many tokens request i has sampled before (the generator's counter); ``contexts[i]``
        the token ids (prompt and output) the repeat penalty looks back over.  The sampled tokens stay on the
        device (``Pending.tokens``, int32 [S]) for the next step to read, and travel to the host in the background.
        """
        s = logits.shape[0]
        assert len(plans) == s and len(steps) == s
        pen_rows, pen_toks = [], []
        for i, pl in enumerate(plans):
            if pl.repetition_penalty != 1.0 and pl.repeat_last_n > 0:
                uniq = set(contexts[i][-pl.repeat_last_n:])
                pen_rows += [i] * len(uniq)
                pen_toks += list(uniq)
        # rows that all take the largest logit need no parameters of their own: one upload per batch size, ever
        all_greedy = not pen_rows and all(pl.greedy for pl in plans)
        if all_greedy and s in self._greedy_meta:
            m = self._greedy_meta[s]
            out = ops.sample_packed(logits, m[0], m[4].view(torch.int32), m[1], m[2])
            host, pool = self._host_buffer(s)
            host.copy_(out, non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            return Pending(out[0].view(torch.int32), out[1], host, ev, pool)
        # one packed upload: temperature, top_p, uniform, penalty (float32) and top_k (int32 bits)
        meta_pool = self._meta_pool.setdefault(s, [])
        meta = meta_pool.pop() if meta_pool else torch.empty((5, s), dtype=torch.float32, pin_memory=True)
        mn = meta.numpy()
        top_k = mn[4].view(np.int32)
        for i, pl in enumerate(plans):
            mn[0, i] = 0.0 if pl.greedy else pl.temperature
            mn[1, i] = pl.top_p
            mn[2, i] = uniform(pl.random_seed, steps[i]) if not pl.greedy else 0.0
            mn[3, i] = pl.repetition_penalty
            top_k[i] = pl.top_k
        m = meta.to(self.device, non_blocking=True)
        if all_greedy:
            # (top_p, penalty and top_k of a greedy row are never read; the copy kept is this batch's)
            self._greedy_meta[s] = m
        if pen_rows:
            pen = torch.tensor([pen_rows, pen_toks], dtype=torch.int32).to(self.device)
            ops.repeat_penalty(logits, pen[0], pen[1], m[3])
        # (rows that draw are shared by several blocks each: a block walks a row of a large vocabulary too slowly)
        cuts = any(not pl.greedy and (pl.top_k > 0 or pl.top_p < 1.0) for pl in plans)
        out = ops.sample_packed(logits, m[0], m[4].view(torch.int32), m[1], m[2],
                                split=not all_greedy and logits.shape[1] >= SPLIT_MIN_VOCAB, cuts=cuts)
        tok, lg = out[0].view(torch.int32), out[1]
        host, pool = self._host_buffer(s)
        host.copy_(out, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        pending = Pending(tok, lg, host, ev, pool)
        # (pinned memory must outlive the copy that reads it; a greedy batch's copy is kept, and its buffer with it)
        pending._meta, pending._meta_pool = meta, (None if all_greedy else meta_pool)
        return pending

    def sample(self, logits: torch.Tensor, plans: Sequence[SamplingPlan], steps: Sequence[int],
               contexts: Sequence[Sequence[int]]) -> Tuple[List[int], List[float]]:
        """``launch`` and wait: the tokens and the (penalised) logits of the chosen tokens."""
        return self.launch(logits, plans, steps, contexts).result()
