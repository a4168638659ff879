"""Generation parameters under the reference's names, defaults and checks.

``GenerateParameters`` mirrors backends/vllm/src/types.rs:24-95 and its validation
backends/vllm/src/validation.rs:187-380.  The sampling mode follows backends/vllm/src/llm_service.rs:346-372:
greedy (argmax) when ``do_sample`` is false **or the temperature equals 1.0**; otherwise temperature sampling over
all tokens, the top k, the top p, or top k then top p.  ``frequency_penalty``, ``typical_p``, ``best_of``, ``n``,
``top_n_tokens``, ``decoder_input_details`` and ``truncate`` are checked and carried but, as in the reference,
change nothing in sampling.  ``ignore_eos_token`` is an addition (the reference fixes it to false,
validation.rs:358) that benchmarks need.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional

DEFAULT_RANDOM_SEED = 1_283_768_955  # backends/vllm/src/validation.rs:11


class ValidationError(ValueError):
    pass


@dataclasses.dataclass
class GenerateParameters:
    best_of: Optional[int] = None
    temperature: Optional[float] = None
    repetition_penalty: Optional[float] = None
    frequency_penalty: Optional[float] = None
    repeat_last_n: Optional[int] = None
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    typical_p: Optional[float] = None
    do_sample: bool = True
    max_new_tokens: Optional[int] = 100
    return_full_text: Optional[bool] = None
    stop: List[str] = dataclasses.field(default_factory=list)
    truncate: Optional[int] = None
    decoder_input_details: bool = False
    random_seed: Optional[int] = None
    top_n_tokens: Optional[int] = None
    n: int = 1
    ignore_eos_token: bool = False


@dataclasses.dataclass(frozen=True)
class SamplingPlan:
    """What the sampler needs for one request, after validation."""
    greedy: bool
    temperature: float
    top_k: int            # 0: off
    top_p: float          # 1.0: off
    repetition_penalty: float
    repeat_last_n: int
    random_seed: int
    max_new_tokens: int
    stop: tuple
    ignore_eos_token: bool
    return_full_text: bool

    @property
    def mode(self) -> str:
        """The reference's name of the mode (llm_service.rs:346-372)."""
        if self.greedy:
            return "ArgMax"
        if self.top_k == 0 and self.top_p == 1.0:
            return "All"
        if self.top_k == 0:
            return "TopP"
        if self.top_p == 1.0:
            return "TopK"
        return "TopKThenTopP"


def validate(params: GenerateParameters, input_len: int, max_input_length: int, max_total_tokens: int,
             max_stop_sequences: int = 1, max_top_n_tokens: int = 1) -> SamplingPlan:
    p = params
    best_of = 1 if p.best_of is None else p.best_of
    sampling = p.do_sample or any(v is not None for v in (p.temperature, p.top_k, p.top_p, p.typical_p))
    if best_of > 1 and not sampling:
        raise ValidationError("`best_of` > 1 is only supported with sampling")
    if best_of != 1 or p.n != 1:
        raise ValidationError("only one sequence per request is generated (best_of = n = 1)")
    temperature = 1.0 if p.temperature is None else float(p.temperature)
    if temperature <= 0.0:
        raise ValidationError("`temperature` must be strictly positive")
    rep = 1.0 if p.repetition_penalty is None else float(p.repetition_penalty)
    if rep <= 0.0:
        raise ValidationError("`repetition_penalty` must be strictly positive")
    freq = 0.0 if p.frequency_penalty is None else float(p.frequency_penalty)
    if not -2.0 <= freq <= 2.0:
        raise ValidationError("`frequency_penalty` must be between -2.0 and 2.0")
    top_p = 1.0
    if p.top_p is not None:
        if not 0.0 < p.top_p < 1.0:
            raise ValidationError("`top_p` must be > 0.0 and < 1.0")
        top_p = float(p.top_p)
    if p.typical_p is not None and not 0.0 < p.typical_p < 1.0:
        raise ValidationError("`typical_p` must be > 0.0 and < 1.0")
    top_k = 0
    if p.top_k is not None:
        if p.top_k <= 0:
            raise ValidationError("`top_k` must be strictly positive")
        top_k = int(p.top_k)
    if p.max_new_tokens is not None and p.max_new_tokens <= 0:
        raise ValidationError("`max_new_tokens` must be strictly positive")
    if len(p.stop) > max_stop_sequences:
        raise ValidationError(f"`stop` supports up to {max_stop_sequences} stop sequences, {len(p.stop)} given")
    if p.top_n_tokens is not None and p.top_n_tokens > max_top_n_tokens:
        raise ValidationError(f"`top_n_tokens` must be <= {max_top_n_tokens}")
    if p.truncate is not None and not 0 < p.truncate <= max_input_length:
        raise ValidationError(f"`truncate` must be strictly positive and at most {max_input_length}")
    if input_len == 0:
        raise ValidationError("empty input")
    if input_len > max_input_length:
        raise ValidationError(f"`inputs` must have at most {max_input_length} tokens, {input_len} given")
    # validation.rs:133-137: without a limit the request may use all of max_total_tokens
    max_new = p.max_new_tokens if p.max_new_tokens is not None else max_total_tokens - input_len
    if max_new <= 0 or input_len + max_new > max_total_tokens:
        raise ValidationError(f"`inputs` tokens + `max_new_tokens` must be <= {max_total_tokens}, "
                              f"given {input_len} + {max_new}")
    rep_n = 0 if p.repeat_last_n is None else int(p.repeat_last_n)
    if rep != 1.0 and rep_n <= 0:
        raise ValidationError("`repeat_last_n` must be positive when `repetition_penalty` is not 1.0")
    seed = DEFAULT_RANDOM_SEED if p.random_seed is None else int(p.random_seed)
    greedy = (not p.do_sample) or temperature == 1.0
    return SamplingPlan(greedy=greedy, temperature=temperature, top_k=top_k, top_p=top_p, repetition_penalty=rep,
                        repeat_last_n=rep_n, random_seed=seed, max_new_tokens=int(max_new), stop=tuple(p.stop),
                        ignore_eos_token=bool(p.ignore_eos_token), return_full_text=bool(p.return_full_text))
