"""The sampler: from float32 logits on the device to one token per row.

Greedy rows take the argmax (lowest index on ties).  Sampled rows draw from softmax(logits / T), cut by top-k
and/or top-p, with the inverse-CDF method from one uniform number per (request seed, step): a counter-based
generator, so a request's tokens do not depend on which other requests share its batches, and portions of
prompts that sample nothing consume nothing (the reference advances each request's generator even for discarded
samples: backends/vllm/src/model_executor.rs:231-235, llm_engine.rs:379).
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingPlan

_MASK = (1 << 64) - 1


def uniform(seed: int, counter: int) -> float:
    """A number in [0, 1) with 24 random bits, a pure function of (seed, counter) (splitmix64 finaliser)."""
    z = (seed * 0x9E3779B97F4A7C15 + (counter + 1) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device

    def sample(self, logits: torch.Tensor, plans: Sequence[SamplingPlan], steps: Sequence[int],
               contexts: Sequence[Sequence[int]]) -> Tuple[List[int], List[float]]:
        """One token per row of ``logits`` [S, V].

        ``steps[i]`` is how many tokens request i has sampled before (the generator's counter); ``contexts[i]``
        the token ids (prompt and output) the repeat penalty looks back over.
        Returns the tokens and the (penalised) logits of the chosen tokens.
        """
        s = logits.shape[0]
        assert len(plans) == s and len(steps) == s
        pen_rows, pen_toks = [], []
        for i, pl in enumerate(plans):
            if pl.repetition_penalty != 1.0 and pl.repeat_last_n > 0:
                uniq = set(contexts[i][-pl.repeat_last_n:])
                pen_rows += [i] * len(uniq)
                pen_toks += list(uniq)
        # one packed upload: temperature, top_p, uniform, penalty (float32) and top_k (int32 bits)
        meta = np.zeros((5, s), dtype=np.float32)
        top_k = meta[4].view(np.int32)
        for i, pl in enumerate(plans):
            meta[0, i] = 0.0 if pl.greedy else pl.temperature
            meta[1, i] = pl.top_p
            meta[2, i] = uniform(pl.random_seed, steps[i]) if not pl.greedy else 0.0
            meta[3, i] = pl.repetition_penalty
            top_k[i] = pl.top_k
        m = torch.from_numpy(meta).to(self.device)
        if pen_rows:
            pen = torch.tensor([pen_rows, pen_toks], dtype=torch.int32, device=self.device)
            ops.repeat_penalty(logits, pen[0], pen[1], m[3])
        tok, lg = ops.sample(logits, m[0], m[4].view(torch.int32), m[1], m[2])
        both = torch.stack([tok.view(torch.float32), lg]).cpu()      # one download
        return both[0].view(torch.int32).tolist(), both[1].tolist()
