"""A request's state between admission and its last token, and what the caller gets back.

Mirrors what the reference keeps in ``SequenceData`` / ``Sequence`` / ``SequenceGroup``
(backends/vllm/src/sequence.rs:166-465, 467-995, 1045-1943) for the one-sequence-per-request case, and its
``GenerateRequestOutput`` (backends/vllm/src/llm_engine.rs:526-618) with the finish reasons of
backends/vllm/src/sequence.rs:118-128.
"""
from __future__ import annotations

import dataclasses
import enum
from typing import List, Optional

from ..sampling.params import SamplingPlan


class Status(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED_STOPPED = "stopped"
    FINISHED_LENGTH_CAPPED = "length_capped"
    FINISHED_ABORTED = "aborted"
    FINISHED_IGNORED = "ignored"

    @property
    def finished(self) -> bool:
        return self in (Status.FINISHED_STOPPED, Status.FINISHED_LENGTH_CAPPED, Status.FINISHED_ABORTED,
                        Status.FINISHED_IGNORED)


@dataclasses.dataclass
class RequestMetrics:
    arrival_time: float
    first_scheduled_time: Optional[float] = None
    first_token_time: Optional[float] = None
    last_token_time: Optional[float] = None
    finished_time: Optional[float] = None
    num_preemptions: int = 0


@dataclasses.dataclass(eq=False)
class Request:
    uid: int                      # engine-wide unique number, the cache manager's key
    request_id: str               # the caller's name
    prompt_ids: List[int]
    plan: SamplingPlan
    metrics: RequestMetrics
    prompt_text: Optional[str] = None
    output_ids: List[int] = dataclasses.field(default_factory=list)
    output_logits: List[float] = dataclasses.field(default_factory=list)
    num_computed: int = 0         # tokens whose keys and values are in the cache
    status: Status = Status.WAITING
    stop_reason: Optional[object] = None
    #: tokens sampled on the device that the host has not read yet (the engine runs one step ahead of them)
    pending: int = 0
    #: the token that ends this request by count is on its way: nothing more is scheduled for it
    frozen: bool = False

    @property
    def length(self) -> int:
        return len(self.prompt_ids) + len(self.output_ids) + self.pending

    @property
    def num_sampled(self) -> int:
        return len(self.output_ids) + self.pending

    @property
    def num_uncomputed(self) -> int:
        """Tokens still to run; includes generated tokens after a recompute-preemption
        (backends/vllm/src/sequence.rs:347-352)."""
        return self.length - self.num_computed

    @property
    def in_prefill(self) -> bool:
        return self.num_uncomputed > 1 or self.num_sampled == 0

    def all_ids(self) -> List[int]:
        return self.prompt_ids + self.output_ids

    def next_tokens(self, n: int) -> List[int]:
        """The next ``n`` tokens to run.  A token still pending on the device is given as 0; the caller feeds it."""
        known = len(self.prompt_ids) + len(self.output_ids)
        if self.num_computed + n > known:
            assert n == 1 and self.num_computed == known and self.pending > 0
            return [0]
        lo = self.num_computed
        p = len(self.prompt_ids)
        if lo + n <= p:
            return self.prompt_ids[lo:lo + n]
        if lo >= p:
            return self.output_ids[lo - p:lo - p + n]
        return self.prompt_ids[lo:] + self.output_ids[:lo + n - p]


@dataclasses.dataclass
class InferenceOutput:
    index: int
    output_text: Optional[str]
    token_ids: List[int]
    cumulative_logprob: float
    logprobs: List[float]
    finish_reason: Optional[str]
    stop_reason: Optional[object]


@dataclasses.dataclass
class GenerateRequestOutput:
    request_id: str
    prompt: Optional[str]
    inference_outputs: List[InferenceOutput]
    prompt_token_ids: List[int]
    is_finished: bool
    metrics: RequestMetrics

    @classmethod
    def from_request(cls, r: Request, text: Optional[str] = None) -> "GenerateRequestOutput":
        out = InferenceOutput(index=0, output_text=text, token_ids=list(r.output_ids),
                              cumulative_logprob=float(sum(r.output_logits)), logprobs=list(r.output_logits),
                              finish_reason=r.status.value if r.status.finished else None,
                              stop_reason=r.stop_reason)
        return cls(r.request_id, r.prompt_text, [out], list(r.prompt_ids), r.status.finished, r.metrics)
