"""Typed configuration of the dense Llama decoder.

Keys and defaults follow the reference's ``LlamaConfig`` and its
``into_config`` (models/src/llama.rs:36-82): ``num_key_value_heads`` defaults to
the number of attention heads, ``rope_theta`` to 10000, ``tie_word_embeddings``
to false; ``rope_scaling`` is optional and, when present, holds all five of its
keys (models/src/llama.rs:21-28).  The head size is hidden_size divided by the
number of heads (models/src/llama.rs:326); there is no ``head_dim`` key.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional, Tuple

from .base import (ConfigError, ModelConfig, as_bool, as_float, as_int, as_positive_int, key,
                   parse_fields)


@dataclasses.dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` object (models/src/llama.rs:12-28)."""
    factor: float = key(convert=as_float)
    low_freq_factor: float = key(convert=as_float)
    high_freq_factor: float = key(convert=as_float)
    original_max_position_embeddings: int = key(convert=as_positive_int)
    rope_type: str = key(convert=str)

    @classmethod
    def from_json(cls, obj: Any) -> "RopeScaling":
        if isinstance(obj, dict) and "rope_type" not in obj and "type" in obj:
            obj = dict(obj, rope_type=obj["type"])  # older spelling of the same key
        rs = cls(**parse_fields(cls, obj, "rope_scaling"))
        if rs.rope_type not in ("llama3", "default"):
            raise ConfigError(f"rope_scaling.rope_type: '{rs.rope_type}' is not supported (known: llama3, default)")
        if rs.rope_type == "llama3":
            if rs.factor <= 0:
                raise ConfigError("rope_scaling.factor must be positive")
            if rs.high_freq_factor == rs.low_freq_factor:
                raise ConfigError("rope_scaling: high_freq_factor equals low_freq_factor (division by zero)")
            if rs.low_freq_factor <= 0 or rs.high_freq_factor <= 0:
                raise ConfigError("rope_scaling: low_freq_factor and high_freq_factor must be positive")
        return rs

    def to_dict(self) -> Dict[str, Any]:
        return dataclasses.asdict(self)


def _eos(v: Any) -> Tuple[int, ...]:
    """``eos_token_id``: one integer or a list of them (models/src/llama.rs:29-34)."""
    if isinstance(v, list):
        return tuple(as_int(x) for x in v)
    return (as_int(v),)


@dataclasses.dataclass(frozen=True)
class LlamaConfig(ModelConfig):
    architectures = ("LlamaForCausalLM", "llama")

    hidden_size: int = key(convert=as_positive_int)
    intermediate_size: int = key(convert=as_positive_int)
    vocab_size: int = key(convert=as_positive_int)
    num_hidden_layers: int = key(convert=as_positive_int)
    num_attention_heads: int = key(convert=as_positive_int)
    rms_norm_eps: float = key(convert=as_float)
    max_position_embeddings: int = key(convert=as_positive_int)
    num_key_value_heads: Optional[int] = key(default=None, convert=as_positive_int)
    rope_theta: float = key(default=10000.0, convert=as_float)
    bos_token_id: Optional[int] = key(default=None, convert=as_int)
    eos_token_id: Tuple[int, ...] = key(default=(), convert=_eos)
    rope_scaling: Optional[RopeScaling] = key(default=None, convert=RopeScaling.from_json)
    tie_word_embeddings: bool = key(default=False, convert=as_bool)
    # attention over the last N keys only (none: all keys).  The reference's models report it to the engine through
    # ``sliding_window()`` (backends/vllm/src/model_executor.rs:116-140; none for Llama) and its ``[cache]``
    # section has the same option (backends/vllm/src/config.rs:137-159), which the engine writes in here.
    sliding_window: Optional[int] = key(default=None, convert=as_positive_int)
    # Keys the reference does not read.  They are accepted only with the value
    # that the reference's code fixes, so that a checkpoint which needs another
    # value is refused instead of being run wrongly.
    head_dim: Optional[int] = key(default=None, convert=as_positive_int)
    hidden_act: str = key(default="silu", convert=str)
    attention_bias: bool = key(default=False, convert=as_bool)
    mlp_bias: bool = key(default=False, convert=as_bool)

    def __post_init__(self):
        if self.num_key_value_heads is None:
            object.__setattr__(self, "num_key_value_heads", self.num_attention_heads)

    def validate(self, where: str) -> None:
        p = []
        if self.hidden_size % self.num_attention_heads:
            p.append(f"hidden_size {self.hidden_size} is not a multiple of num_attention_heads "
                     f"{self.num_attention_heads}")
        elif self.head_dim is not None and self.head_dim != self.hidden_size // self.num_attention_heads:
            p.append(f"head_dim {self.head_dim} differs from hidden_size/num_attention_heads "
                     f"{self.hidden_size // self.num_attention_heads}; this architecture fixes it to the quotient")
        elif (self.hidden_size // self.num_attention_heads) % 2:
            p.append("the head size must be even for rotary position encoding")
        if self.num_attention_heads % self.num_key_value_heads:
            p.append(f"num_attention_heads {self.num_attention_heads} is not a multiple of num_key_value_heads "
                     f"{self.num_key_value_heads}")
        if not self.rms_norm_eps > 0:
            p.append("rms_norm_eps must be positive")
        if not self.rope_theta > 0:
            p.append("rope_theta must be positive")
        if self.hidden_act != "silu":
            p.append(f"hidden_act '{self.hidden_act}' is not supported (the feed-forward is SwiGLU: silu)")
        if self.attention_bias or self.mlp_bias:
            p.append("attention_bias / mlp_bias are not supported (all projections are bias-free)")
        for t in self.eos_token_id:
            if not 0 <= t < self.vocab_size:
                p.append(f"eos_token_id {t} outside the vocabulary")
        if p:
            raise ConfigError(f"{where}: " + "; ".join(p))

    @property
    def head_size(self) -> int:
        return self.hidden_size // self.num_attention_heads

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": ["LlamaForCausalLM"],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
        }
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id:
            d["eos_token_id"] = self.eos_token_id[0] if len(self.eos_token_id) == 1 else list(self.eos_token_id)
        if self.rope_scaling is not None:
            d["rope_scaling"] = self.rope_scaling.to_dict()
        if self.sliding_window is not None:
            d["sliding_window"] = self.sliding_window
        return d
