"""The engine: requests in, tokens out.

``LlmEngine`` plays the parts of the reference's ``LlmService`` (start-up order, request validation, sampling mode:
backends/vllm/src/llm_service.rs:102-260, 267-391) and ``LlmEngine`` (step = schedule + execute + sample, then
``update_sequence`` with its stop checks: backends/vllm/src/llm_engine.rs:216-245, 264-342, 367-521), in one
thread and one process.  The cache pool is sized after the weights are on the device, from free memory times
``gpu_memory_utilization`` unless ``num_gpu_blocks_override`` fixes it (backends/vllm/src/config.rs:195-208).
"""
from __future__ import annotations

import dataclasses
import os
import time
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..cache.pool import CachePool, pages_for_memory, plan_cache
from ..config.engine import CacheConfig, EngineConfig, SchedulerConfig, ValidationConfig, parse_dtype
from ..models.model import Model, load_model
from ..sampling.params import GenerateParameters, ValidationError, validate
from ..sampling.sampler import Pending, Sampler
from .request import GenerateRequestOutput, Request, RequestMetrics, Status
from .scheduler import ScheduleOutput, Scheduler
from .step import ModelRunner, RunnerCache, StepEntry

Inputs = Union[str, Sequence[int]]


@dataclasses.dataclass
class _InFlight:
    """A launched step whose sampled tokens the host has not read yet."""
    sampled: List[Request]
    pending: Optional[Pending]
    rows: Dict[int, int]          # request uid -> row of the sampled tokens
    sync: bool                    # the tokens are needed before the next step can be planned


class LlmEngine:
    def __init__(self, model: Union[str, Model], dtype: str = "bfloat16", *, cache: Optional[CacheConfig] = None,
                 scheduler: Optional[SchedulerConfig] = None, validation: Optional[ValidationConfig] = None,
                 device: str = "cuda:0"):
        self.cache_config = cache or CacheConfig()
        window = self.cache_config.sliding_window
        if isinstance(model, str):
            self.model = load_model(model, parse_dtype(dtype), device, sliding_window=window)
        else:
            self.model = model
            if window is not None and getattr(model.config, "sliding_window", None) != window:
                raise ValueError("[cache] sliding_window differs from that of the model given; load the model with it")
        self.scheduler_config = scheduler or SchedulerConfig()
        self.validation = validation or ValidationConfig()
        self.cache_config.validate()
        self.scheduler_config.validate()
        spec = self.model.spec
        if self.scheduler_config.max_model_len > spec.max_positions:
            self.scheduler_config.max_model_len = spec.max_positions
        plan = plan_cache(spec)
        cache_dtype = self.model.act_dtype
        if self.cache_config.cache_dtype != "auto":
            want = parse_dtype(self.cache_config.cache_dtype)
            if want != {torch.bfloat16: "bfloat16", torch.float32: "float32"}[cache_dtype]:
                raise ValueError("[cache] cache_dtype must agree with the model dtype (or be 'auto')")
        page = self.cache_config.block_size
        elem = torch.empty((), dtype=cache_dtype).element_size()
        if self.cache_config.num_gpu_blocks_override is not None:
            pages = [self.cache_config.num_gpu_blocks_override] * len(plan.groups)
        else:
            free, _ = torch.cuda.mem_get_info(self.model.device)
            pages = pages_for_memory(plan, page, elem, int(free * self.cache_config.gpu_memory_utilization))
            # no request can use more than max_model_len tokens, and no step holds more than max_num_sequences
            cap = self.scheduler_config.max_num_sequences * (-(-self.scheduler_config.max_model_len // page))
            pages = [min(p, cap) for p in pages]
        pool = CachePool(plan, page, pages, self.scheduler_config.max_num_sequences, cache_dtype, self.model.device)
        self.runner = ModelRunner(self.model, pool)
        self.runner.external_fence = True       # the event behind a step's sampled tokens serves its staging buffer too
        self.scheduler = Scheduler(self.scheduler_config, RunnerCache(self.runner),
                                   chunk_alignment=spec.chunk_alignment)
        self.sampler = Sampler(self.model.device)
        self.eos_ids = set(spec.eos_token_ids)
        self._next_uid = 0
        self._requests: Dict[str, Request] = {}
        self.tokenizer = None
        self._in_flight: Optional[_InFlight] = None
        self._undelivered: List[GenerateRequestOutput] = []     # finished while aborting another request
        self.stats = {"steps": 0, "tokens": 0, "sampled": 0, "preemptions": 0}

    # -- construction from the reference's TOML ----------------------------------------------------------
    @classmethod
    def from_config(cls, config: EngineConfig) -> "LlmEngine":
        if not config.inference.model_name:
            raise ValueError("[inference] model_name must name a folder with config.json and model.safetensors")
        eng = cls(config.inference.model_name, config.inference.dtype, cache=config.cache,
                  scheduler=config.scheduler, validation=config.validation,
                  device=f"cuda:{config.inference.device_ids[0]}")
        eng.load_tokenizer(config.inference.model_name)
        return eng

    @classmethod
    def from_toml(cls, path: str) -> "LlmEngine":
        return cls.from_config(EngineConfig.from_toml(path))

    def load_tokenizer(self, model_dir: str) -> bool:
        """Text in and out need ``tokenizer.json`` in the model folder; token ids work without it."""
        path = os.path.join(model_dir, "tokenizer.json")
        if not os.path.isfile(path):
            return False
        from tokenizers import Tokenizer
        self.tokenizer = Tokenizer.from_file(path)
        return True

    # -- requests ------------------------------------------------------------------------------------------
    def add_request(self, inputs: Inputs, parameters: Optional[GenerateParameters] = None,
                    request_id: Optional[str] = None) -> str:
        params = parameters or GenerateParameters()
        text = None
        if isinstance(inputs, str):
            if self.tokenizer is None:
                raise ValidationError("text input needs tokenizer.json in the model folder; pass token ids instead")
            text = inputs
            if params.truncate is not None:
                text = text[-params.truncate:] if len(text) > params.truncate else text  # tokenizer.rs:185-206
            ids = self.tokenizer.encode(text, add_special_tokens=True).ids
        else:
            ids = [int(t) for t in inputs]
        vocab = self.model.vocab_size
        if any(t < 0 or t >= vocab for t in ids):
            raise ValidationError(f"a token id lies outside the vocabulary of {vocab}")
        if params.stop and self.tokenizer is None:
            raise ValidationError("`stop` strings need tokenizer.json in the model folder")
        v = self.validation
        plan = validate(params, len(ids), v.max_input_length, v.max_total_tokens, v.max_stop_sequences,
                        v.max_top_n_tokens)
        uid = self._next_uid
        self._next_uid += 1
        rid = request_id if request_id is not None else f"request-{uid}"
        if rid in self._requests:
            raise ValidationError(f"request id '{rid}' is in use")
        req = Request(uid, rid, ids, plan, RequestMetrics(arrival_time=time.monotonic()), prompt_text=text)
        self._requests[rid] = req
        self.scheduler.add(req)
        return rid

    def abort(self, request_id: str) -> Optional[GenerateRequestOutput]:
        """Stop a request wherever it is.  The step in flight is read first; requests that it finished are handed
        out by the next ``step`` (or ``drain``), the aborted one (if it had not just finished) here."""
        self._undelivered = self.drain()
        r = self.scheduler.abort(request_id)
        if r is None:
            return None
        return self._output(r)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished() or self._in_flight is not None or bool(self._undelivered)

    # -- one step ------------------------------------------------------------------------------------------
    def step(self) -> List[GenerateRequestOutput]:
        """Plan and launch one step, then read the tokens of the step before it; returns the requests that finished.

        The engine runs one step ahead of the host's knowledge of the sampled tokens: the tokens a step samples
        stay on the device, where the next step reads them, and reach the host while that next step runs.  So the
        GPU does not wait for scheduling and bookkeeping.  A request that ends on a token (EOS, a stop string) is
        seen one step late; the token it sampled meanwhile is dropped.  Requests whose sampling needs the host to
        know every earlier token (a repeat penalty, stop strings) are read at once instead.
        """
        plan: ScheduleOutput = self.scheduler.schedule()
        finished: List[Request] = list(plan.ignored) + list(plan.capped)
        self.stats["preemptions"] += len(plan.preempted)
        launched = None
        if not plan.empty:
            launched = self._launch(plan)
        elif self._in_flight is None and not (finished or plan.preempted) and self.scheduler.has_unfinished():
            # nothing runs, nothing is on its way, nothing left the queue: the next plan would be the same
            raise RuntimeError(f"the scheduler plans nothing although {self.scheduler.num_unfinished()} request(s) "
                               f"wait: its limits admit none of them")
        if self._in_flight is not None:
            finished += self._resolve(self._in_flight)
        self._in_flight = launched
        if launched is not None and launched.sync:
            finished += self._resolve(launched)
            self._in_flight = None
        outs, self._undelivered = self._undelivered, []
        for r in finished:
            r.metrics.finished_time = time.monotonic()
            outs.append(self._output(r))
        return outs

    def _launch(self, plan: ScheduleOutput) -> "_InFlight":
        prev = self._in_flight
        entries, sampled = [], []
        for e in plan.entries:
            r = e.request
            feed = -1
            if e.num_tokens == 1 and r.num_computed == len(r.prompt_ids) + len(r.output_ids):
                # its last token is still on the device: row of the previous step's sampled tokens
                feed = prev.rows[r.uid]
            entries.append(StepEntry(r.uid, r.next_tokens(e.num_tokens), e.start,
                                     [e.num_tokens - 1] if e.do_sample else [], feed))
            if e.do_sample:
                sampled.append(r)
        logits = self.runner.step(entries, prev.pending.tokens if prev is not None and prev.pending else None)
        for e in plan.entries:
            e.request.num_computed += e.num_tokens
        self.stats["steps"] += 1
        self.stats["tokens"] += plan.num_tokens
        flight = _InFlight(sampled, None, {r.uid: i for i, r in enumerate(sampled)}, False)
        if not sampled:
            fence = torch.cuda.Event()
            fence.record()
            self.runner.fence(fence)
        if sampled:
            flight.pending = self.sampler.launch(
                logits, [r.plan for r in sampled], [r.num_sampled for r in sampled],
                [r.all_ids() if r.plan.repetition_penalty != 1.0 else () for r in sampled])
            self.runner.fence(flight.pending.event)       # (the step's staging buffer is free when the tokens are here)
            self.stats["sampled"] += len(sampled)
            limit = self.scheduler_config.max_model_len
            for r in sampled:
                r.pending += 1
                # by count alone this may be the request's last token: then nothing more is scheduled for it
                if r.num_sampled >= r.plan.max_new_tokens or r.length > limit:
                    r.frozen = True
                if r.plan.repetition_penalty != 1.0 or r.plan.stop:
                    flight.sync = True
        return flight

    def _resolve(self, flight: "_InFlight") -> List[Request]:
        """Read the tokens of a launched step and apply them; returns the requests that ended."""
        done: List[Request] = []
        if flight.pending is None:
            return done
        toks, lgs = flight.pending.result()
        now = time.monotonic()
        for r, tok, lg in zip(flight.sampled, toks, lgs):
            r.pending -= 1
            if r.status.finished:
                continue      # it ended on an earlier token; this one was sampled in vain
            status = self._append(r, tok, lg, now)
            if status is not None:
                self.scheduler.finish(r, status)
                done.append(r)
        return done

    def drain(self) -> List[GenerateRequestOutput]:
        """Read what is still in flight (call before reading clocks or state from outside)."""
        outs, self._undelivered = self._undelivered, []
        if self._in_flight is not None:
            for r in self._resolve(self._in_flight):
                r.metrics.finished_time = time.monotonic()
                outs.append(self._output(r))
            self._in_flight = None
        return outs

    def _append(self, r: Request, tok: int, logit: float, now: float) -> Optional[Status]:
        """Take a sampled token and apply the stop checks in the reference's order (llm_engine.rs:438-501)."""
        r.output_ids.append(tok)
        r.output_logits.append(logit)
        if r.metrics.first_token_time is None:
            r.metrics.first_token_time = now
        r.metrics.last_token_time = now
        if r.plan.stop and self.tokenizer is not None:
            piece = self.tokenizer.decode([tok])
            if piece in r.plan.stop:
                r.stop_reason = piece
                return Status.FINISHED_STOPPED
        if tok in self.eos_ids and not r.plan.ignore_eos_token:
            r.stop_reason = tok
            return Status.FINISHED_STOPPED
        if len(r.prompt_ids) + len(r.output_ids) > self.scheduler_config.max_model_len:
            return Status.FINISHED_LENGTH_CAPPED
        if len(r.output_ids) >= r.plan.max_new_tokens:
            return Status.FINISHED_LENGTH_CAPPED
        return None

    def _output(self, r: Request) -> GenerateRequestOutput:
        self._requests.pop(r.request_id, None)
        text = None
        if self.tokenizer is not None:
            text = self.tokenizer.decode(r.output_ids)
            if r.plan.return_full_text and r.prompt_text is not None:
                text = r.prompt_text + text  # sequence.rs:520-524
        return GenerateRequestOutput.from_request(r, text)

    # -- the Python entry point ---------------------------------------------------------------------------
    def generate(self, inputs: Sequence[Inputs], parameters: Union[GenerateParameters, Sequence[GenerateParameters],
                                                                    None] = None) -> List[GenerateRequestOutput]:
        """Run the given prompts (token-id lists, or strings with a tokenizer) to their end; outputs in input order."""
        if parameters is None or isinstance(parameters, GenerateParameters):
            parameters = [parameters or GenerateParameters()] * len(inputs)
        if len(parameters) != len(inputs):
            raise ValueError("one GenerateParameters per input, or one for all")
        rids = [self.add_request(x, p) for x, p in zip(inputs, parameters)]
        done: Dict[str, GenerateRequestOutput] = {}
        while self.has_unfinished():
            for o in self.step():
                done[o.request_id] = o
        return [done[r] for r in rids]


def generate(model_dir: str, inputs: Sequence[Inputs], parameters=None, dtype: str = "bfloat16",
             **engine_options) -> List[GenerateRequestOutput]:
    """One call from a model folder to finished outputs."""
    return LlmEngine(model_dir, dtype, **engine_options).generate(inputs, parameters)
