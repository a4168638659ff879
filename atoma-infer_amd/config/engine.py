"""Engine options: the reference's TOML file with its four sections.

``[inference]``, ``[cache]``, ``[scheduler]`` and ``[validation]`` keep the
reference's key names and meanings (backends/vllm/src/config.rs:17-43, 137-159,
349-365, 462-473; an example is backends/vllm/src/tests/test_config.toml).
Keys that only make sense for what this engine leaves out (hub download,
tokenizer workers, swap space, several devices) are accepted and ignored.
``model_name`` is a local folder holding config.json and model.safetensors.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional

from .base import ConfigError, as_bool, as_float, as_int, as_positive_int, key, parse_fields

_DTYPES = {"bf16": "bfloat16", "bfloat16": "bfloat16", "f32": "float32", "fp32": "float32", "float32": "float32"}


def parse_dtype(name: str) -> str:
    """'bf16' / 'f32' as the reference spells them (backends/vllm/src/llm_service.rs:132), or the long names."""
    n = str(name).lower()
    if n not in _DTYPES:
        raise ConfigError(f"dtype '{name}' is not supported (bf16/bfloat16 or f32/float32)")
    return _DTYPES[n]


@dataclasses.dataclass
class InferenceConfig:
    model_name: str = key(default="", convert=str)
    dtype: str = key(default="bfloat16", convert=parse_dtype)
    device_ids: tuple = key(default=(0,), convert=lambda v: tuple(as_int(x) for x in v))
    seed: int = key(default=0, convert=as_int)


@dataclasses.dataclass
class CacheConfig:
    """``[cache]``: page size in tokens and how many pages the pool has.

    ``num_gpu_blocks_override`` fixes the pool; otherwise it is sized after the
    weights are resident as floor(free memory x gpu_memory_utilization / bytes
    per page) (backends/vllm/src/config.rs:195-208, 590-643).
    """
    block_size: int = key(default=16, convert=as_positive_int)
    cache_dtype: str = key(default="auto", convert=str)
    gpu_memory_utilization: float = key(default=0.5, convert=as_float)
    num_gpu_blocks_override: Optional[int] = key(default=None, convert=as_positive_int)
    sliding_window: Optional[int] = key(default=None, convert=as_positive_int)

    def validate(self):
        if not 0 < self.gpu_memory_utilization <= 1:
            raise ConfigError("[cache] gpu_memory_utilization must be in (0, 1]")
        if self.cache_dtype not in ("auto",) and parse_dtype(self.cache_dtype) is None:
            raise ConfigError("[cache] cache_dtype")


@dataclasses.dataclass
class SchedulerConfig:
    """``[scheduler]`` (backends/vllm/src/config.rs:349-406)."""
    max_num_batched_tokens: int = key(default=2048, convert=as_positive_int)
    max_num_sequences: int = key(default=64, convert=as_positive_int)
    max_model_len: int = key(default=8192, convert=as_positive_int)
    delay_factor: float = key(default=0.0, convert=as_float)
    enable_chunked_prefill: bool = key(default=True, convert=as_bool)
    #: largest portion of one prompt in a step, besides the token budget (0: the budget alone decides)
    max_prefill_chunk: int = key(default=0, convert=as_int)

    def validate(self):
        if self.max_num_batched_tokens < self.max_model_len and not self.enable_chunked_prefill:
            raise ConfigError(
                f"[scheduler] max_num_batched_tokens ({self.max_num_batched_tokens}) is smaller than max_model_len "
                f"({self.max_model_len}) and chunked prefill is off: longer prompts could never be scheduled")
        if self.max_num_batched_tokens < self.max_num_sequences:
            raise ConfigError(
                f"[scheduler] max_num_batched_tokens ({self.max_num_batched_tokens}) must be at least "
                f"max_num_sequences ({self.max_num_sequences})")
        if self.delay_factor < 0:
            raise ConfigError("[scheduler] delay_factor must not be negative")


@dataclasses.dataclass
class ValidationConfig:
    """``[validation]`` (backends/vllm/src/config.rs:462-473)."""
    best_of: int = key(default=1, convert=as_positive_int)
    max_stop_sequences: int = key(default=1, convert=as_int)
    max_top_n_tokens: int = key(default=1, convert=as_int)
    max_input_length: int = key(default=4096, convert=as_positive_int)
    max_total_tokens: int = key(default=8192, convert=as_positive_int)

    def validate(self):
        if self.max_input_length >= self.max_total_tokens:
            raise ConfigError("[validation] max_input_length must be smaller than max_total_tokens")


@dataclasses.dataclass
class EngineConfig:
    inference: InferenceConfig = dataclasses.field(default_factory=InferenceConfig)
    cache: CacheConfig = dataclasses.field(default_factory=CacheConfig)
    scheduler: SchedulerConfig = dataclasses.field(default_factory=SchedulerConfig)
    validation: ValidationConfig = dataclasses.field(default_factory=ValidationConfig)

    @classmethod
    def from_dict(cls, obj: Dict[str, Any], where: str = "engine config") -> "EngineConfig":
        out = cls()
        for name, sub in (("inference", InferenceConfig), ("cache", CacheConfig), ("scheduler", SchedulerConfig),
                          ("validation", ValidationConfig)):
            sec = obj.get(name, {})
            setattr(out, name, sub(**parse_fields(sub, sec, f"{where} [{name}]")))
        out.validate()
        return out

    @classmethod
    def from_toml(cls, path: str) -> "EngineConfig":
        import tomli
        try:
            with open(path, "rb") as f:
                obj = tomli.load(f)
        except OSError as e:
            raise ConfigError(f"cannot read {path}: {e}") from None
        except tomli.TOMLDecodeError as e:
            raise ConfigError(f"{path}: not valid TOML: {e}") from None
        return cls.from_dict(obj, path)

    def validate(self):
        self.cache.validate()
        self.scheduler.validate()
        self.validation.validate()
