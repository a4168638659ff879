"""The one registry from an architecture's name to its configuration class and model builder.

The reference picks the model type at compile time
(``LlmService::start::<LlamaModel,_>``, server/src/main.rs:45); here the name in
config.json's ``architectures`` (or, failing that, ``model_type``) picks it at run
time.  A builder is a function ``build(config) -> ModelSpec`` (see
``atoma_infer_amd.models.spec``); registering one is all that a new
architecture needs.
"""
from __future__ import annotations

import dataclasses
import os
from typing import Any, Callable, Dict, Tuple, Type

from .base import ConfigError, ModelConfig, read_json


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Type[ModelConfig]
    build: Callable[[ModelConfig], Any]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig], build: Callable[[ModelConfig], Any],
                          *, replace: bool = False) -> Architecture:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    arch = Architecture(name, config_cls, build)
    _ARCHITECTURES[name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures() -> Tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def resolve_architecture(obj: Dict[str, Any], where: str = "config.json") -> Architecture:
    names = []
    archs = obj.get("architectures")
    if isinstance(archs, list):
        names += [a for a in archs if isinstance(a, str)]
    elif isinstance(archs, str):
        names.append(archs)
    if isinstance(obj.get("model_type"), str):
        names.append(obj["model_type"])
    if not names:
        raise ConfigError(f"{where}: neither 'architectures' nor 'model_type' names the model; "
                          f"known architectures: {', '.join(known_architectures())}")
    for n in names:
        if n in _ARCHITECTURES:
            return _ARCHITECTURES[n]
    raise ConfigError(f"{where}: architecture {names} is not registered; known: {', '.join(known_architectures())}")


def load_model_config(model_dir: str) -> Tuple[Architecture, ModelConfig]:
    """Read ``model_dir/config.json`` and return its architecture entry and typed configuration."""
    path = os.path.join(model_dir, "config.json")
    obj = read_json(path)
    arch = resolve_architecture(obj, path)
    return arch, arch.config_cls.from_dict(obj, path)
