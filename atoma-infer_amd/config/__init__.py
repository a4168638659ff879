"""Typed configurations and the architecture registry."""
from .base import ConfigError, ModelConfig, key, read_json
from .engine import (CacheConfig, EngineConfig, InferenceConfig, SchedulerConfig, ValidationConfig, parse_dtype)
from .llama import LlamaConfig, RopeScaling
from .registry import (Architecture, known_architectures, load_model_config, register_architecture,
                       resolve_architecture, unregister_architecture)

__all__ = [
    "ConfigError", "ModelConfig", "key", "read_json", "CacheConfig", "EngineConfig", "InferenceConfig",
    "SchedulerConfig", "ValidationConfig", "parse_dtype", "LlamaConfig", "RopeScaling", "Architecture",
    "known_architectures", "load_model_config", "register_architecture", "resolve_architecture",
    "unregister_architecture",
]
